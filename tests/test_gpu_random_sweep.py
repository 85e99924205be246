"""Seeded random sweeps over shapes, GQA ratios, block sizes, map styles and causality: the forward, the backward and
the antidiagonal estimator against the oracle, through the C ABI.  Tolerances as in the per-operator tests."""
import numpy as np
import pytest
import torch

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, dev

pytestmark = pytest.mark.gpu
LEVELS = np.array([0, 1, 2, 4, 8], np.int32)
STYLES = ([0.35, 0.2, 0.15, 0.15, 0.15], [0.85, 0.05, 0.04, 0.03, 0.03], [0.05, 0.8, 0.05, 0.05, 0.05], [0.6, 0.0, 0.0, 0.2, 0.2])


def _rand(g, *shape, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def test_forward_sweep():
    from psa_hip import ops

    rng = np.random.default_rng(2024)
    for case in range(40):
        B, Hkv, rep = int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.choice([1, 1, 2, 4]))
        Hq, L, D = Hkv * rep, int(rng.integers(1, 2600)), int(rng.choice([64, 128, 128]))
        bm, bn = int(rng.choice([64, 128, 128])), int(rng.choice([32, 64, 128]))
        causal = bool(rng.integers(0, 2)) and bn == bm
        Mq, Nk = -(-L // bm), -(-L // bn)
        lm = rng.choice(LEVELS, size=(B, Hq, Mq, Nk), p=STYLES[int(rng.integers(0, 4))])
        if rng.integers(0, 3) == 0 and Mq > 1:
            lm[:, :, rng.integers(0, Mq)] = 0  # a q-block that keeps nothing
        g = torch.Generator().manual_seed(int(rng.integers(0, 1 << 30)))
        q, k, v = _rand(g, B, Hq, L, D), _rand(g, B, Hkv, L, D), _rand(g, B, Hkv, L, D)
        info = dict(case=case, B=B, Hq=Hq, Hkv=Hkv, L=L, D=D, bm=bm, bn=bn, causal=causal)
        out, lse, _ = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), torch.from_numpy(lm).to(dev()), bm, bn, causal=causal,
                                              return_lse=True, balance=bool(rng.integers(0, 2)))
        ref, ref_lse = O.psa_attention_dense(q, k, v, lm, bm, bn, causal=causal)
        err = (out.float().cpu() - ref.float()).abs()
        assert float(err.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (info, float(err.max()), float(err.mean()))
        fin = torch.isfinite(ref_lse)
        assert torch.equal(torch.isfinite(lse.cpu()), fin), info
        if fin.any():
            assert float((lse.cpu().double()[fin] - ref_lse[fin]).abs().max()) <= 2e-2, info


def test_backward_sweep():
    from psa_hip import ops

    def rel_l2(a, b):
        a, b = a.double().cpu(), b.double().cpu()
        return float((a - b).norm() / b.norm().clamp_min(1e-30))

    rng = np.random.default_rng(7)
    for case in range(24):
        B, Hkv, rep = int(rng.integers(1, 3)), int(rng.integers(1, 3)), int(rng.choice([1, 1, 2, 3]))
        Hq, L, D = Hkv * rep, int(rng.integers(40, 1100)), int(rng.choice([64, 128]))
        bm, bn = int(rng.choice([64, 128])), int(rng.choice([32, 64, 128]))
        causal = bool(rng.integers(0, 2)) and bn == bm
        Mq, Nk = -(-L // bm), -(-L // bn)
        lm = rng.choice(LEVELS, size=(B, Hq, Mq, Nk), p=[0.3, 0.25, 0.15, 0.15, 0.15])
        if causal:
            lm[..., np.arange(Mq), np.arange(Mq)] = 1
        lm[..., 0] = np.maximum(lm[..., 0], 1)
        g = torch.Generator().manual_seed(int(rng.integers(0, 1 << 30)))
        q, k, v, do = _rand(g, B, Hq, L, D), _rand(g, B, Hkv, L, D), _rand(g, B, Hkv, L, D), _rand(g, B, Hq, L, D, scale=0.5)
        md = torch.from_numpy(lm).to(dev())
        out, lse, pools = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), md, bm, bn, causal=causal, return_lse=True)
        dq, dk, dv = ops.sparse_attention_bwd(q.to(dev()), k.to(dev()), v.to(dev()), md, out, do.to(dev()), lse, bm, bn, causal=causal, pools=pools)
        rq, rk, rv = O.psa_backward_dense(q, k, v, lm, do, bm, bn, causal=causal)
        errs = rel_l2(dq, rq), rel_l2(dk, rk), rel_l2(dv, rv)
        assert max(errs) <= 5e-2, (dict(case=case, B=B, Hq=Hq, Hkv=Hkv, L=L, D=D, bm=bm, bn=bn, causal=causal), errs)


def test_xattn_sweep():
    from psa_hip import ops

    rng = np.random.default_rng(11)
    for case in range(20):
        B, Hkv, rep = int(rng.integers(1, 3)), int(rng.integers(1, 3)), int(rng.choice([1, 2, 4]))
        Hq, D, stride = Hkv * rep, int(rng.choice([64, 128])), int(rng.choice([4, 8, 16]))
        block = int(rng.choice([8, 16, 32])) * stride
        chunk = 128 * stride * int(rng.integers(1, 4))
        L, causal = int(rng.integers(block, 5000)), bool(rng.integers(0, 2))
        g = torch.Generator().manual_seed(int(rng.integers(0, 1 << 30)))
        q, k = _rand(g, B, Hq, L, D), _rand(g, B, Hkv, L, D)
        got = ops.estimate_xattn(q.to(dev()), k.to(dev()), block_size=block, stride=stride, causal=causal, chunk_size=chunk).cpu()
        ref = O.estimate_xattn(q.float(), k.float(), block_size=block, stride=stride, causal=causal, chunk_size=chunk)
        np.testing.assert_allclose(got.numpy(), ref.numpy(), rtol=2e-3, atol=2e-6,
                                   err_msg=str(dict(case=case, B=B, Hq=Hq, Hkv=Hkv, L=L, D=D, block=block, stride=stride, chunk=chunk, causal=causal)))
