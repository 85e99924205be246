"""Builds psa_hip/libpsa_hip.so (the C-ABI library of hand-written gfx950 kernels) with hipcc.

    python build_ext.py            # compile every csrc/*.hip and link
"""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "psa_hip", "libpsa_hip.so")
OBJ = os.path.join(HERE, "build")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wno-unused-command-line-argument",
    # the tile-copy helpers write M0 in inline assembly and say so in their clobber lists (the compiler must not assume
    # that a value it left in M0 survives them); M0 being a reserved register, every such list draws a warning
    "-Wno-inline-asm",
    # no packed fp32 arithmetic in device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# Per-file additions.  These kernels never produce a NaN on purpose (empty rows are handled by explicit
# -inf tests), and without NaN semantics their maximum chains compile to v_max3_f32 without a
# canonicalising pass over the MFMA results.
FILE_FLAGS = {
    "psa_fwd.hip": ["-fno-honor-nans"],
    "psa_estimate.hip": ["-fno-honor-nans"],
}


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    raise RuntimeError("hipcc not found")


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=True, extra_flags=(), out=OUT):
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def one(pair):
        s, o = pair
        out = _run([hipcc, *FLAGS, *FILE_FLAGS.get(os.path.basename(s), []), *extra_flags, "-c", s, "-o", o])
        if verbose and out.strip():
            print(out)
        return o

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(one, zip(srcs, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out, *objs])
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build(extra_flags=tuple(os.environ.get("PSA_EXTRA_HIPCC_FLAGS", "").split()))
    sys.exit(0)
