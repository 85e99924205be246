"""Writes tests/golden/level_map_golden.npz.

Runs the reference's pure-torch `transfer_attn_to_mask` (loaded by file path, CPU only,
no Triton import involved) on small seeded, tie-free fp32 score matrices and stores
inputs + outputs.  The level-map algorithm is ad-hoc integer logic that neither
mathematics nor any fixture of the reference pins, hence these vectors.  Only data is
committed; this script needs the reference checkout and is not run by the tests.

    python tests/golden/make_level_map_golden.py [/root/reference]
"""

import importlib.util
import json
import os
import sys

import numpy as np
import torch

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SRC = os.path.join(REF, "src/psa_triton/utils/transfer_attn_to_mask.py")

CASES = [
    # name, (B,H,Mq,Nk), mask_ratios (ordered list of [level, lo, hi]), mode, text_length, blocksize, compute_tile, sharpness
    ("wan14b_thr", (1, 2, 6, 40), [[1, 0.0, 0.4], [2, 0.4, 0.5], [4, 0.5, 0.6], [8, 0.6, 0.8], [0, 0.8, 1.0]], "thresholdbound", 0, 128, 32, 3.0),
    ("wan13b_thr", (1, 2, 6, 37), [[1, 0.0, 0.5], [2, 0.5, 0.6], [4, 0.6, 0.7], [8, 0.7, 0.8], [0, 0.8, 1.0]], "thresholdbound", 0, 128, 32, 5.0),
    ("thr_bn32", (1, 2, 5, 50), [[1, 0.0, 0.5], [2, 0.5, 0.6], [4, 0.6, 0.6], [8, 0.6, 0.8], [0, 0.8, 1.0]], "thresholdbound", 0, 32, 32, 4.0),
    ("thr_text", (2, 1, 4, 23), [[1, 0.0, 0.3], [2, 0.3, 0.5], [4, 0.5, 0.7], [8, 0.7, 0.9], [0, 0.9, 1.0]], "thresholdbound", 226, 128, 32, 2.0),
    ("thr_flat", (1, 1, 4, 16), [[1, 0.0, 0.4], [2, 0.4, 0.5], [4, 0.5, 0.6], [8, 0.6, 0.8], [0, 0.8, 1.0]], "thresholdbound", 0, 128, 32, 0.2),
    ("thr_bn64", (1, 2, 4, 33), [[1, 0.0, 0.2], [2, 0.2, 0.4], [4, 0.4, 0.6], [8, 0.6, 0.95], [0, 0.95, 1.0]], "thresholdbound", 0, 64, 32, 3.0),
    ("topk_default", (1, 2, 4, 40), [[1, 0.0, 0.1], [2, 0.1, 0.15], [4, 0.15, 0.15], [8, 0.15, 0.35], [0, 0.35, 1.0]], "topk", 0, 64, 32, 3.0),
    ("topk_cog", (2, 2, 3, 31), [[1, 0.0, 0.05], [2, 0.05, 0.15], [4, 0.15, 0.25], [8, 0.25, 0.5], [0, 0.5, 1.0]], "topk", 226, 128, 32, 3.0),
    ("topk_bn32", (1, 1, 4, 64), [[1, 0.0, 0.05], [2, 0.05, 0.1], [4, 0.1, 0.15], [8, 0.15, 0.25], [0, 0.25, 1.0]], "topk", 0, 32, 32, 3.0),
    ("topk_full8", (1, 1, 3, 21), [[1, 0.0, 0.1], [2, 0.1, 0.3], [4, 0.3, 0.5], [8, 0.5, 1.0], [0, 1.0, 1.0]], "topk", 0, 128, 32, 3.0),
    ("thr_new", (1, 2, 5, 40), [[1, 0.0, 0.4], [2, 0.4, 0.5], [4, 0.5, 0.6], [8, 0.6, 0.8], [0, 0.8, 1.0]], "thresholdbound_newtype", 0, 128, 32, 3.0),
    ("thr_new_bn32", (1, 1, 5, 48), [[1, 0.0, 0.5], [2, 0.5, 0.6], [4, 0.6, 0.6], [8, 0.6, 0.8], [0, 0.8, 1.0]], "thresholdbound_newtype", 0, 32, 32, 4.0),
    ("topk_new", (1, 2, 4, 40), [[1, 0.0, 0.1], [2, 0.1, 0.15], [4, 0.15, 0.15], [8, 0.15, 0.35], [0, 0.35, 1.0]], "topk_newtype", 0, 64, 32, 3.0),
    ("topk_new_bn32", (1, 1, 3, 64), [[1, 0.0, 0.05], [2, 0.05, 0.1], [4, 0.1, 0.15], [8, 0.15, 0.25], [0, 0.25, 1.0]], "topk_newtype", 0, 32, 32, 3.0),
]


def main():
    spec = importlib.util.spec_from_file_location("ref_transfer_attn_to_mask", SRC)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    meta = []
    g = torch.Generator().manual_seed(20261125)
    for name, shape, ratios, mode, text, bs, tile, sharp in CASES:
        logits = torch.randn(shape, generator=g) * sharp
        scores = torch.softmax(logits, -1).float()
        # tie-free by construction (continuous values); assert it
        s = scores.sort(-1).values
        assert (s[..., 1:] != s[..., :-1]).all()
        mr = {int(lv): (float(lo), float(hi)) for lv, lo, hi in ratios}
        m = mod.transfer_attn_to_mask(scores.clone(), mr, text_length=text, mode=mode, blocksize=bs, compute_tile=tile)
        out[name + "__scores"] = scores.numpy()
        out[name + "__mask"] = m.numpy().astype(np.int32)
        meta.append(dict(name=name, ratios=ratios, mode=mode, text_length=text, blocksize=bs, compute_tile=tile))
    out["meta_json"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "level_map_golden.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes,", len(CASES), "cases")


if __name__ == "__main__":
    main()
