"""GPU parity of the sparse attention forward against the oracle, through the C ABI.
Tolerance (bf16 outputs): max-abs <= 2e-2 and mean-abs <= 2e-3."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, attn_errors, dev, random_map, rnd

pytestmark = pytest.mark.gpu


def run_case(B, Hq, Hkv, L, D, bm, bn, causal, seed, lmap=None, p=(0.35, 0.2, 0.15, 0.15, 0.15)):
    from psa_hip import ops

    q, k, v = rnd(B, Hq, L, D, seed=seed), rnd(B, Hkv, L, D, seed=seed + 1), rnd(B, Hkv, L, D, seed=seed + 2)
    Mq, Nk = -(-L // bm), -(-L // bn)
    if lmap is None:
        lmap = random_map(B, Hq, Mq, Nk, seed, p=p)
    out, lse, _ = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), torch.from_numpy(lmap).to(dev()), bm, bn,
                                          causal=causal, return_lse=True)
    torch.cuda.synchronize()
    ref, ref_lse = O.psa_attention_dense(q, k, v, lmap, bm, bn, causal=causal)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    lse_c, ref_l = lse.cpu().double(), ref_lse
    fin = torch.isfinite(ref_l)
    assert torch.equal(torch.isfinite(lse_c), fin)
    assert float((lse_c[fin] - ref_l[fin]).abs().max()) <= 2e-2
    return out, lmap


@pytest.mark.parametrize(
    "B,Hq,Hkv,L,D,bm,bn",
    [
        (1, 2, 2, 512, 128, 128, 128),
        (1, 2, 2, 1000, 128, 128, 128),   # ragged tail
        (2, 2, 2, 777, 64, 128, 128),
        (1, 2, 2, 640, 64, 64, 64),       # c1-like blocks
        (1, 2, 2, 1000, 128, 128, 32),    # Wan2.2 / CogVideoX1.5 presets
        (1, 2, 2, 600, 128, 128, 64),
        (1, 4, 2, 512, 128, 128, 128),    # GQA
        (1, 1, 1, 100, 64, 64, 32),
        (1, 2, 2, 700, 128, 64, 64),      # head dim 128 with 64-row q-blocks (2 waves per workgroup)
        (1, 2, 1, 333, 128, 64, 32),
        (1, 2, 2, 130, 128, 64, 128),
        (1, 1, 1, 3, 128, 128, 128),      # shorter than one run of 4 tile rows
        (1, 1, 1, 65, 128, 128, 128),
    ],
)
@pytest.mark.parametrize("causal", [False, True])
def test_fwd_random_maps(B, Hq, Hkv, L, D, bm, bn, causal):
    if causal and bm != bn:
        pytest.skip("causal maps are square in the reference")
    run_case(B, Hq, Hkv, L, D, bm, bn, causal, seed=L + D)


def test_fwd_each_level_alone_and_empty_rows():
    for lv in (1, 2, 4, 8):
        m = np.full((1, 1, 3, 3), lv, np.int32)
        run_case(1, 1, 1, 300, 128, 128, 128, False, seed=lv, lmap=m)
    m = np.zeros((1, 2, 4, 4), np.int32)
    m[0, 0, 1, 2] = 8
    m[0, 1, 3, 3] = 1
    out, _ = run_case(1, 2, 2, 500, 128, 128, 128, False, seed=9, lmap=m)
    assert torch.all(out[0, 0, :128] == 0) and torch.all(out[0, 1, :384] == 0)  # rows without keys give 0


def test_fwd_odd_counts_of_small_blocks():
    # level 4 / 8 blocks are packed 2 / 4 per tile: exercise partly filled tiles
    for n8 in (1, 2, 3, 5):
        L = 1024 - 37
        mm = np.zeros((1, 1, 8, 8), np.int32)
        mm[..., :n8] = 8
        mm[..., 7] = 4
        run_case(1, 1, 1, L, 64, 128, 128, False, seed=n8, lmap=mm)


def test_fwd_two_row_workgroups_uneven_rows():
    # head dim 128 with 128-row q-blocks runs two map rows per workgroup: pair rows of very different length
    # (many tiles / one partly filled tile / none), an odd number of rows, partly filled level-4/8 tiles
    L = 1024 - 37
    for causal in (False, True):
        mm = np.zeros((1, 3, 8, 8), np.int32)
        mm[0, 0, 0, :] = 1            # 16 tiles next to ...
        mm[0, 0, 1, 0] = 8            # ... a quarter of a tile
        mm[0, 0, 3, :3] = 8           # empty row 2 next to 3/4 of a tile
        mm[0, 0, 4, :] = 2
        mm[0, 0, 5, 1:4] = 4
        mm[0, 0, 7, :] = [1, 2, 4, 8, 8, 4, 2, 1]
        mm[0, 1] = 1
        mm[0, 2, 5:, :] = 4           # head 2: rows 0-4 empty
        if causal:
            mm = np.where(np.arange(8)[None, None, None, :] > np.arange(8)[None, None, :, None], 0, mm)
        for balance in (True, False):
            from psa_hip import ops

            q, k, v = rnd(1, 3, L, 128, seed=5), rnd(1, 3, L, 128, seed=6), rnd(1, 3, L, 128, seed=7)
            out, lse, _ = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), torch.from_numpy(mm).to(dev()), 128, 128,
                                                  causal=causal, return_lse=True, balance=balance)
            ref, ref_lse = O.psa_attention_dense(q, k, v, mm, 128, 128, causal=causal)
            mx, mean = attn_errors(out, ref)
            assert mx <= MAX_ABS and mean <= MEAN_ABS, (causal, balance, mx, mean)
            fin = torch.isfinite(ref_lse)
            assert torch.equal(torch.isfinite(lse.cpu()), fin)
            assert float((lse.cpu().double()[fin] - ref_lse[fin]).abs().max()) <= 2e-2


def test_fwd_dense_equals_sdpa_and_all_ones_map():
    from psa_hip import ops

    B, H, L, D = 1, 2, 900, 128
    q, k, v = rnd(B, H, L, D, seed=1), rnd(B, H, L, D, seed=2), rnd(B, H, L, D, seed=3)
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float())
    o1 = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), None, 128, 128)
    ones = torch.ones(B, H, 8, 8, dtype=torch.int8, device=dev())
    o2 = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), ones, 128, 128)
    for o in (o1, o2):
        mx, mean = attn_errors(o, ref)
        assert mx <= MAX_ABS and mean <= MEAN_ABS
    assert torch.equal(o1, o2)
    refc = F.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    oc = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), None, 128, 128, causal=True)
    mx, mean = attn_errors(oc, refc)
    assert mx <= MAX_ABS and mean <= MEAN_ABS


def test_fwd_long_sequence_takes_the_one_row_kernel():
    # with 128-key blocks the schedules of two rows stop fitting into LDS above ~85k tokens: the launch falls back
    # to one row per workgroup.  Dense attention on 88k tokens against torch SDPA on the GPU (bf16), plus a sparse
    # map through the size-independent property that rows whose blocks are all level 1 equal the dense rows.
    from psa_hip import ops

    B, H, L, D = 1, 1, 88000, 128
    g = torch.Generator(device="cpu").manual_seed(11)
    q, k, v = (torch.randn(B, H, L, D, generator=g).to(torch.bfloat16).to(dev()) for _ in range(3))
    ref = F.scaled_dot_product_attention(q, k, v).float()
    o = ops.sparse_attention_fwd(q, k, v, None, 128, 128)
    assert float((o.float() - ref).abs().max()) <= MAX_ABS and float((o.float() - ref).abs().mean()) <= MEAN_ABS
    Nk = -(-L // 128)
    mp = torch.zeros(B, H, Nk, Nk, dtype=torch.int8, device=dev())
    mp[..., ::7, :] = 1          # every 7th q-block keeps everything at level 1
    mp[..., 1::7, ::3] = 4       # some other rows: a third of the blocks, pooled 4x
    o2 = ops.sparse_attention_fwd(q, k, v, mp, 128, 128)
    rows = torch.arange(L, device=dev()) // 128 % 7 == 0
    assert float((o2[..., rows, :].float() - ref[..., rows, :]).abs().max()) <= MAX_ABS
    assert torch.isfinite(o2.float()).all()


def test_fwd_lossless_pooling_invariant_full_size_heads():
    """K and V constant inside aligned groups of 8 tokens: every map without skips must give plain
    attention - checked at the Wan2.1-1.3B sequence length on one head against SDPA on the GPU."""
    from psa_hip import ops

    L, D = 32760, 128
    g = torch.Generator().manual_seed(0)
    bk = torch.randn(1, 1, L // 8, D, generator=g).bfloat16()
    bv = torch.randn(1, 1, L // 8, D, generator=g).bfloat16()
    k, v = bk.repeat_interleave(8, 2).to(dev()), bv.repeat_interleave(8, 2).to(dev())
    q = (torch.randn(1, 1, L, D, generator=g) * 0.5).bfloat16().to(dev())
    lm = torch.from_numpy(np.random.default_rng(0).choice([1, 2, 4, 8], size=(1, 1, 256, 256)).astype(np.int8)).to(dev())
    out = ops.sparse_attention_fwd(q, k, v, lm, 128, 128)
    ref = F.scaled_dot_product_attention(q, k, v)
    d = (out.float() - ref.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS


def test_fwd_strided_and_fp32_inputs():
    from psa_hip import ops

    B, H, L, D = 1, 2, 300, 64
    q, k, v = rnd(B, L, H, D, seed=4, dtype=torch.float32), rnd(B, L, H, D, seed=5, dtype=torch.float32), rnd(B, L, H, D, seed=6, dtype=torch.float32)
    lm = random_map(B, H, 3, 3, 1)
    qt, kt, vt = (t.transpose(1, 2) for t in (q, k, v))
    out = ops.sparse_attention_fwd(qt.to(dev()), kt.to(dev()), vt.to(dev()), torch.from_numpy(lm).to(dev()), 128, 128)
    assert out.dtype == torch.float32 and out.shape == (B, H, L, D)
    ref, _ = O.psa_attention_dense(qt, kt, vt, lm, 128, 128)  # on the fp32 values themselves: nothing is rounded
    mx, mean = attn_errors(out, ref)
    assert mx <= 2e-5 and mean <= 2e-6, (mx, mean)


def test_fwd_strided_bf16_head_dim_128():
    """[B,L,H,D] memory layout passed as a [B,H,L,D] view: rows of a head are H*D elements apart."""
    from psa_hip import ops

    B, H, L, D = 1, 3, 700, 128
    q, k, v = rnd(B, L, H, D, seed=14), rnd(B, L, H, D, seed=15), rnd(B, L, H, D, seed=16)
    lm = random_map(B, H, 6, 6, 2)
    qt, kt, vt = (t.to(dev()).transpose(1, 2) for t in (q, k, v))
    assert not kt.is_contiguous()
    for causal in (False, True):
        out = ops.sparse_attention_fwd(qt, kt, vt, torch.from_numpy(lm).to(dev()), 128, 128, causal=causal)
        ref, _ = O.psa_attention_dense(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), lm, 128, 128, causal=causal)
        mx, mean = attn_errors(out, ref)
        assert mx <= MAX_ABS and mean <= MEAN_ABS


def test_fwd_errors():
    from psa_hip import ops

    q = rnd(1, 1, 128, 96).to(dev())
    with pytest.raises(ValueError):
        ops.sparse_attention_fwd(q, q, q, None, 128, 128)  # head dim 96
    q = rnd(1, 1, 128, 64).to(dev())
    with pytest.raises(ValueError):
        ops.sparse_attention_fwd(q, q, q, torch.ones(1, 1, 2, 1, dtype=torch.int8, device=dev()), 128, 128)  # map shape
    with pytest.raises(ValueError):
        ops.sparse_attention_fwd(q, q, q, None, 100, 128)


@pytest.mark.parametrize("causal", [False, True])
def test_longest_first_order_is_a_pure_reordering(causal):
    """With the workspace the rows are issued longest first; every row must still be computed exactly
    once and bit-identically (the unordered launch is the one checked against the oracle above)."""
    from psa_hip import ops

    B, H, L, D, bm, bn = 1, 5, 128 * 67 + 40, 128, 128, 128
    Mq, Nk = -(-L // bm), -(-L // bn)
    rng = np.random.default_rng(5)
    lmap = random_map(B, H, Mq, Nk, 11)
    # strongly uneven rows: some empty, some full
    keep = rng.random((B, H, Mq, 1)) ** 2
    lmap = np.where(rng.random(lmap.shape) < keep, lmap, 0).astype(lmap.dtype)
    lmap[:, :, 3] = 0
    lmap[:, :, 7] = 1
    q, k, v = (rnd(B, H, L, D, seed=s).to(dev()) for s in (1, 2, 3))
    m = torch.from_numpy(lmap).to(dev())
    outs = []
    for balance in (False, True):
        o = torch.full((B, H, L, D), float("nan"), dtype=torch.bfloat16, device=dev())
        res, lse, _ = ops.sparse_attention_fwd(q, k, v, m, bm, bn, causal=causal, return_lse=True, out=o, balance=balance)
        assert res.data_ptr() == o.data_ptr()
        outs.append((res.clone(), lse.clone()))
    torch.cuda.synchronize()
    assert not torch.isnan(outs[1][0]).any()
    assert torch.equal(outs[0][0], outs[1][0])
    assert torch.equal(outs[0][1], outs[1][1])
