"""Writes tests/golden/gilbert_golden.json: the curve order the reference's vendored gilbert3d yields for a few
boxes (full order for small boxes, SHA-256 of the order for the model-sized ones).  The exact curve is not fixed
by any property test (many Hamiltonian paths exist), hence these vectors.  Needs the reference checkout; only the
data is committed.

    python tests/golden/make_gilbert_golden.py [/root/reference]
"""
import hashlib
import importlib.util
import json
import os
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
spec = importlib.util.spec_from_file_location("ref_gilbert3d", os.path.join(REF, "src/psa_triton/utils/gilbert3d.py"))
mod = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mod)

out = {"full": {}, "sha256": {}}
for box in [(1, 1, 1), (2, 2, 2), (5, 4, 3), (3, 7, 2), (2, 3, 9), (8, 6, 2), (7, 7, 7), (6, 1, 4), (1, 5, 1)]:
    out["full"]["x".join(map(str, box))] = [x + box[0] * (y + box[1] * z) for x, y, z in mod.gilbert3d(*box)]
for box in [(52, 30, 21), (45, 30, 13), (80, 45, 21), (40, 22, 31), (85, 48, 11)]:
    order = [x + box[0] * (y + box[1] * z) for x, y, z in mod.gilbert3d(*box)]
    out["sha256"]["x".join(map(str, box))] = hashlib.sha256(",".join(map(str, order)).encode()).hexdigest()
dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gilbert_golden.json")
json.dump(out, open(dst, "w"))
print("wrote", dst, os.path.getsize(dst))
