"""GPU parity of the backward (dQ, dK, dV) against autograd through the oracle, through the C ABI.
Tolerance: relative L2 error <= 5e-2 per gradient tensor."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O
from gpu_util import dev, random_map, rnd

pytestmark = pytest.mark.gpu
REL_L2 = 5e-2


def rel_l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def run_bwd(B, Hq, Hkv, L, D, bm, bn, causal, seed, lmap=None, dtype=torch.bfloat16):
    from psa_hip import ops

    q, k, v = rnd(B, Hq, L, D, seed=seed, dtype=dtype), rnd(B, Hkv, L, D, seed=seed + 1, dtype=dtype), rnd(B, Hkv, L, D, seed=seed + 2, dtype=dtype)
    do = rnd(B, Hq, L, D, seed=seed + 3, scale=0.5, dtype=dtype)
    Mq, Nk = -(-L // bm), -(-L // bn)
    if lmap is None:
        lmap = random_map(B, Hq, Mq, Nk, seed)
        if causal:
            lmap[..., np.arange(Mq), np.arange(Mq)] = 1  # the reference's callers force the diagonal to level 1
    md = torch.from_numpy(lmap).to(dev())
    qd, kd, vd, dod = q.to(dev()), k.to(dev()), v.to(dev()), do.to(dev())
    out, lse, pools = ops.sparse_attention_fwd(qd, kd, vd, md, bm, bn, causal=causal, return_lse=True)
    dq, dk, dv = ops.sparse_attention_bwd(qd, kd, vd, md, out, dod, lse, bm, bn, causal=causal, pools=pools)
    torch.cuda.synchronize()
    rq, rk, rv = O.psa_backward_dense(q, k, v, lmap, do, bm, bn, causal=causal)
    errs = rel_l2(dq, rq), rel_l2(dk, rk), rel_l2(dv, rv)
    assert max(errs) <= REL_L2, errs
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    assert dq.dtype == dtype and dk.dtype == dtype and dv.dtype == dtype
    return dq, dk, dv, lmap, errs


@pytest.mark.parametrize(
    "B,Hq,Hkv,L,D,bm,bn",
    [
        (1, 2, 2, 512, 128, 128, 128),
        (1, 2, 2, 600, 128, 128, 128),    # ragged tail: pad gradient folds into the last token
        (2, 2, 2, 500, 64, 128, 128),
        (1, 4, 2, 384, 128, 128, 128),    # GQA: dK/dV accumulate over the head group
        (1, 2, 2, 320, 64, 64, 64),
        (1, 1, 1, 400, 128, 128, 32),
        (1, 1, 1, 300, 64, 128, 64),
        (1, 2, 2, 330, 128, 64, 64),      # head dim 128 with 64-row q-blocks
        (1, 1, 1, 67, 128, 128, 128),     # a single, partly filled block
        (1, 3, 1, 200, 128, 128, 64),     # GQA with three query heads per kv head
    ],
)
@pytest.mark.parametrize("causal", [False, True])
def test_bwd_random_maps(B, Hq, Hkv, L, D, bm, bn, causal):
    if causal and bm != bn:
        pytest.skip("causal maps are square in the reference")
    run_bwd(B, Hq, Hkv, L, D, bm, bn, causal, seed=L + D)


def test_bwd_each_level_alone_and_unused_blocks():
    for lv in (1, 2, 4, 8):
        run_bwd(1, 1, 1, 300, 128, 128, 128, False, seed=lv, lmap=np.full((1, 1, 3, 3), lv, np.int32))
    m = np.zeros((1, 2, 4, 4), np.int32)
    m[0, 0, 1, 2] = 8
    m[0, 1, 3, 3] = 1
    m[0, 1, 0, 0] = 2
    dq, dk, dv, _, _ = run_bwd(1, 2, 2, 500, 128, 128, 128, False, seed=9, lmap=m)
    assert torch.all(dq[0, 0, :128] == 0)            # rows without keys
    assert torch.all(dk[0, 0, :256] == 0) and torch.all(dv[0, 0, :256] == 0)  # kv-blocks nobody retains


@pytest.mark.parametrize("causal", [False, True])
def test_bwd_more_than_256_rows_ordered_walks(causal):
    """272 rows of the map (B 2, 4 query heads on 2 kv heads, 34 q-blocks of 128, ragged last block): the dQ walk runs in
    its longest-first issue order (chunk sort, -1 padding, early return of the padded entries), the level-0 dK/dV walk
    writes bf16 directly.  Random map with skipped blocks and rows that retain nothing, against the oracle."""
    B, Hq, Hkv, L = 2, 4, 2, 128 * 33 + 40
    Mq = 34
    lmap = random_map(B, Hq, Mq, Mq, 91, p=(0.55, 0.15, 0.1, 0.1, 0.1), ensure_row=False)
    if causal:
        lmap[..., np.arange(Mq), np.arange(Mq)] = 1
    else:
        lmap[0, 1, 5] = 0   # rows without keys
        lmap[1, 3, 33] = 0  # ... incl. the ragged last q-block
        lmap[1, 0, :, 7] = 0  # a kv-block nobody retains
    assert B * Hq * Mq > 256
    dq, dk, dv, _, _ = run_bwd(B, Hq, Hkv, L, 128, 128, 128, causal, seed=92, lmap=lmap)
    if not causal:
        assert torch.all(dq[0, 1, 5 * 128:6 * 128] == 0) and torch.all(dq[1, 3, 33 * 128:] == 0)


def test_bwd_all_ones_matches_sdpa_autograd():
    from psa_hip import ops

    B, H, L, D = 1, 2, 384, 128
    q, k, v, do = (rnd(B, H, L, D, seed=s) for s in (1, 2, 3, 4))
    qq, kk, vv = (t.double().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(qq, kk, vv).backward(do.double())
    qd, kd, vd, dod = (t.to(dev()) for t in (q, k, v, do))
    out, lse, _ = ops.sparse_attention_fwd(qd, kd, vd, None, 128, 128, return_lse=True)
    dq, dk, dv = ops.sparse_attention_bwd(qd, kd, vd, None, out, dod, lse, 128, 128)
    assert max(rel_l2(dq, qq.grad), rel_l2(dk, kk.grad), rel_l2(dv, vv.grad)) <= REL_L2


def test_bwd_strided_bf16_head_dim_128():
    """q, k, v, dO in [B,L,H,D] memory layout (views), gradients returned densely."""
    from psa_hip import ops

    B, H, L, D = 1, 2, 390, 128
    q, k, v, do = (rnd(B, L, H, D, seed=s) for s in (21, 22, 23, 24))
    lmap = random_map(B, H, 4, 4, 5)
    qd, kd, vd, dod = (t.to(dev()).transpose(1, 2) for t in (q, k, v, do))
    md = torch.from_numpy(lmap).to(dev())
    out, lse, pools = ops.sparse_attention_fwd(qd, kd, vd, md, 128, 128, return_lse=True)
    dq, dk, dv = ops.sparse_attention_bwd(qd, kd, vd, md, out, dod, lse, 128, 128, pools=pools)
    rq, rk, rv = O.psa_backward_dense(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), lmap, do.transpose(1, 2), 128, 128)
    assert max(rel_l2(dq, rq), rel_l2(dk, rk), rel_l2(dv, rv)) <= REL_L2


def test_legacy_factory_autograd():
    """sparse_attention_factory(128, 32, 128)(q, k, v, mask) is differentiable like the reference's."""
    from psa_hip.kernels.psa_kernel_legacy import sparse_attention_factory

    B, H, L, D = 1, 2, 300, 64
    q, k, v, do = (rnd(B, H, L, D, seed=s) for s in (5, 6, 7, 8))
    lmap = random_map(B, H, 3, 3, 3)
    fn = sparse_attention_factory(128, 32, 128)
    qd, kd, vd = (t.to(dev()).requires_grad_(True) for t in (q, k, v))
    out = fn(qd, kd, vd, torch.from_numpy(lmap).to(dev()))
    out.backward(do.to(dev()))
    rq, rk, rv = O.psa_backward_dense(q, k, v, lmap, do, 128, 128)
    assert max(rel_l2(qd.grad, rq), rel_l2(kd.grad, rk), rel_l2(vd.grad, rv)) <= REL_L2
    with pytest.raises(ValueError):
        sparse_attention_factory(64, 32, 128)
    with pytest.raises(ValueError):
        sparse_attention_factory(128, 64, 128)
    with pytest.raises(ValueError):
        sparse_attention_factory(128, 32, 64)


@pytest.mark.parametrize(
    "B,Hq,Hkv,L,D,bm,bn,causal",
    [
        (1, 2, 2, 600, 128, 128, 128, False),
        (1, 4, 2, 384, 128, 128, 128, True),
        (2, 2, 2, 500, 64, 128, 128, False),
        (1, 2, 2, 320, 64, 64, 64, True),
        (1, 1, 1, 400, 128, 128, 32, False),
    ],
)
def test_bwd_fp16(B, Hq, Hkv, L, D, bm, bn, causal):
    """fp16 tensors are differentiated in fp16 (fp16 MFMA operands, fp32 accumulation, gradients returned in fp16):
    against the oracle's autograd on the fp16 values themselves, at the bound of the bf16 path - and, fp16 carrying three
    more mantissa bits, closer to it than the bf16 run of the same case."""
    *_, e16 = run_bwd(B, Hq, Hkv, L, D, bm, bn, causal, seed=L + D, dtype=torch.float16)
    *_, eb = run_bwd(B, Hq, Hkv, L, D, bm, bn, causal, seed=L + D, dtype=torch.bfloat16)
    assert max(e16) <= 0.5 * max(eb), (e16, eb)
