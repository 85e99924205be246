"""GPU parity of the operators in fp16 and fp32 (every stage computes in the element type of its inputs: bf16 and fp16
on the matrix cores with fp32 accumulation, fp32 on the vector units).  The oracle is always run on the caller's own
values, never on copies rounded to another type; tolerances: pooling bit-exact in the element type, estimator scores
rtol 2e-4, attention outputs max-abs 2e-2 / mean-abs 2e-3 (16-bit types) and 2e-5 / 2e-6 (fp32)."""
import numpy as np
import pytest
import torch

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, attn_errors, dev, random_map, rnd

pytestmark = pytest.mark.gpu

TOL = {torch.float16: (MAX_ABS, MEAN_ABS), torch.bfloat16: (MAX_ABS, MEAN_ABS), torch.float32: (2e-5, 2e-6)}
BITS = {torch.float16: torch.int16, torch.bfloat16: torch.int16, torch.float32: torch.int32}


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("B,H,L,D,bn", [(1, 2, 256, 128, 128), (2, 3, 1000, 64, 128), (1, 1, 77, 128, 32), (1, 2, 4097, 64, 64)])
def test_pool_bit_exact_in_the_input_type(dtype, B, H, L, D, bn):
    """Level 2 / 4 / 8 means, each rounded once to the element type (the chained torch.mean of the reference)."""
    from psa_hip import ops

    k, v = rnd(B, H, L, D, seed=1, dtype=dtype), rnd(B, H, L, D, seed=2, dtype=dtype)
    kp, vp = ops.pool_kv(k.to(dev()), v.to(dev()), bn)
    torch.cuda.synchronize()
    assert kp.dtype == dtype and vp.dtype == dtype
    for src, pool in ((k, kp), (v, vp)):
        lv = ops.pool_levels(pool, B, H, L, D, bn)
        ref = O.pool_kv(src, bn)
        for l in (2, 4, 8):
            assert torch.equal(lv[l].cpu().view(BITS[dtype]), ref[l].view(BITS[dtype])), (l,)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_pool_indexed_in_the_input_type(dtype):
    from psa_hip import ops

    B, H, L, D, bn = 1, 2, 700, 128, 128
    k, v = rnd(B, H, L, D, seed=3, dtype=dtype), rnd(B, H, L, D, seed=4, dtype=dtype)
    g = torch.Generator().manual_seed(5)
    idx = torch.randperm(L, generator=g).to(torch.int32)
    kp, vp, ko, vo = ops.pool_kv_indexed(k.to(dev()), v.to(dev()), idx.to(dev()), bn)
    assert torch.equal(ko.cpu(), k[:, :, idx.long()]) and torch.equal(vo.cpu(), v[:, :, idx.long()])
    lv = ops.pool_levels(kp, B, H, L, D, bn)
    ref = O.pool_kv(k[:, :, idx.long()], bn)
    for l in (2, 4, 8):
        assert torch.equal(lv[l].cpu().view(BITS[dtype]), ref[l].view(BITS[dtype])), (l,)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("B,Hq,Hkv,L,D,bm,bn", [(1, 2, 2, 4096, 64, 64, 64), (1, 4, 2, 3000, 128, 128, 128), (2, 2, 1, 1111, 128, 128, 64)])
def test_estimator_in_the_input_type(dtype, B, Hq, Hkv, L, D, bm, bn):
    from psa_hip import ops
    from psa_hip.utils.synthetic import sample_offsets

    q, k = rnd(B, Hq, L, D, seed=11, dtype=dtype, scale=0.7), rnd(B, Hkv, L, D, seed=12, dtype=dtype, scale=0.7)
    oq, ok = sample_offsets(B, Hq, bm, bm // 4, 21), sample_offsets(B, Hkv, bn, bn // 4, 22)
    got = ops.estimate_sampled(q.to(dev()), k.to(dev()), oq.to(dev()), ok.to(dev()), bm, bn, bm // 4, bn // 4)
    okq = ok.repeat_interleave(Hq // Hkv, dim=1)
    ref = O.estimate_sampled(q, k.repeat_interleave(Hq // Hkv, dim=1), bm, bn, oq, okq)
    assert got.shape == ref.shape and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), ref.numpy(), rtol=2e-4, atol=1e-9)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize(
    "B,Hq,Hkv,L,D,bm,bn,causal",
    [
        (1, 2, 2, 128 * 9 + 40, 128, 128, 128, False),   # fp16: the two-group kernel on a prebuilt schedule, ragged end
        (1, 4, 2, 128 * 6, 128, 128, 128, True),          # causal, grouped heads
        (2, 2, 1, 700, 64, 128, 128, False),              # head dim 64: the one-row kernel
        (1, 2, 2, 1000, 64, 64, 64, True),                # blocks of 64
        (1, 1, 1, 900, 128, 64, 128, False),              # block_m != block_n
    ],
)
def test_forward_and_lse_in_the_input_type(dtype, B, Hq, Hkv, L, D, bm, bn, causal):
    from psa_hip import ops

    Mq, Nk = -(-L // bm), -(-L // bn)
    lm = random_map(B, Hq, Mq, Nk, 31)
    if causal:
        lm = np.where(np.arange(Nk)[None, :] * bn < (np.arange(Mq)[:, None] + 1) * bm, lm, 0)
        lm[..., np.arange(min(Mq, Nk)), np.arange(min(Mq, Nk))] = 1
    q, k, v = (rnd(B, h, L, D, seed=s, dtype=dtype, scale=0.8) for h, s in ((Hq, 41), (Hkv, 42), (Hkv, 43)))
    m = torch.from_numpy(lm.astype(np.int8)).to(dev())
    out, lse, _ = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), m, bm, bn, causal=causal, return_lse=True)
    torch.cuda.synchronize()
    assert out.dtype == dtype and lse.dtype == torch.float32
    rep = Hq // Hkv
    ref, ref_lse = O.psa_attention_dense(q, k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1), lm, bm, bn, causal=causal)
    mx, mean = attn_errors(out, ref)
    assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], (mx, mean)
    live = torch.isfinite(ref_lse)
    dl = (lse.cpu().double() - ref_lse.double())[live].abs().max()
    assert float(dl) <= (2e-5 if dtype == torch.float32 else 5e-3), float(dl)
    if dtype != torch.float32 and D == 128 and bm == 128 and bn == 128:
        # the walk over the map itself gives the bits of the scheduled walk
        out2, lse2, _ = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), m, bm, bn, causal=causal, return_lse=True, schedule=False)
        assert torch.equal(out, out2) and torch.equal(lse, lse2)


def test_fp16_values_outside_the_bf16_grid_are_used_as_they_are():
    """Inputs with 10 significant mantissa bits, so that rounding them to bf16 (8 bits) anywhere on the way would be
    visible: against the oracle on the fp16 values the error stays at the accumulation level, an order of magnitude
    under the error that the same oracle shows for bf16-rounded copies of the inputs."""
    from psa_hip import ops

    B, H, L, D = 1, 2, 1024, 128
    q, k, v = (rnd(B, H, L, D, seed=s, dtype=torch.float16, scale=1.5) for s in (51, 52, 53))
    lm = random_map(B, H, 8, 8, 54)
    out = ops.sparse_attention_fwd(q.to(dev()), k.to(dev()), v.to(dev()), torch.from_numpy(lm.astype(np.int8)).to(dev()), 128, 128)
    ref, _ = O.psa_attention_dense(q, k, v, lm, 128, 128)
    rounded, _ = O.psa_attention_dense(q.bfloat16(), k.bfloat16(), v.bfloat16(), lm, 128, 128)
    mean = attn_errors(out, ref)[1]
    mean_rounded = float((rounded.float() - ref.float()).abs().mean())
    assert mean <= 0.25 * mean_rounded, (mean, mean_rounded)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_forward_with_token_index_in_the_input_type(dtype):
    """The re-ordered walk: queries gathered through a permutation inside the kernel, outputs scattered back."""
    from psa_hip import ops

    B, H, L, D, bm, bn = 1, 2, 128 * 5 + 17, 128, 128, 128
    Mq = -(-L // bm)
    lm = random_map(B, H, Mq, Mq, 61)
    q, k, v = (rnd(B, H, L, D, seed=s, dtype=dtype, scale=0.8) for s in (62, 63, 64))
    idx = torch.randperm(L, generator=torch.Generator().manual_seed(65)).to(torch.int32)
    m = torch.from_numpy(lm.astype(np.int8)).to(dev())
    il = idx.long()
    # keys and values are handed over in the re-ordered token order, queries are read (and outputs written) through the index
    out = ops.sparse_attention_fwd(q.to(dev()), k[:, :, il].to(dev()), v[:, :, il].to(dev()), m, bm, bn, q_index=idx.to(dev()))
    ref_perm, _ = O.psa_attention_dense(q[:, :, il], k[:, :, il], v[:, :, il], lm, bm, bn)
    ref = torch.empty_like(ref_perm)
    ref[:, :, il] = ref_perm
    mx, mean = attn_errors(out, ref)
    assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], (mx, mean)


def test_key_similarity_fp16():
    from psa_hip import ops

    B, H, L, D, bn = 1, 3, 1500, 128, 128
    g = torch.Generator().manual_seed(71)
    base = torch.randn(B, H, -(-L // 8), D, generator=g).repeat_interleave(8, dim=2)[:, :, :L]
    k = (base + 0.6 * torch.randn(B, H, L, D, generator=g) * torch.rand(B, H, L, 1, generator=g)).to(torch.float16)

    def pick(s):  # a threshold in the widest gap between observed scores: no score is within rounding of it
        vals = np.sort(s.numpy().ravel())
        i = int(np.argmax(np.diff(vals)))
        return float((vals[i] + vals[i + 1]) / 2)

    t2, t4, t8 = (pick(s) for s in O.k_similarity_scores(k, bn))
    got = ops.k_similarity(k.to(dev()), bn, t2, t4, t8)
    ref = O.k_similarity(k, bn, t2, t4, t8)
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), ref)
    assert len(set(ref.view(-1).tolist())) >= 2


def test_layer_operator_fp16_pools_are_not_fed_to_the_bf16_backward():
    """A backward call given the pools of an fp16 forward recomputes bf16 pools instead of reading fp16 bits as bf16."""
    from psa_hip import ops

    B, H, L, D = 1, 2, 512, 128
    q, k, v, do = (rnd(B, H, L, D, seed=s, scale=0.7) for s in (81, 82, 83, 84))
    lm = torch.from_numpy(random_map(B, H, 4, 4, 85).astype(np.int8)).to(dev())
    qd, kd, vd, dod = (t.to(dev()) for t in (q, k, v, do))
    out, lse, pools = ops.sparse_attention_fwd(qd, kd, vd, lm, 128, 128, return_lse=True)
    want = ops.sparse_attention_bwd(qd, kd, vd, lm, out, dod, lse, 128, 128, pools=pools)
    pools16 = ops.pool_kv(kd.half(), vd.half(), 128)
    got = ops.sparse_attention_bwd(qd, kd, vd, lm, out, dod, lse, 128, 128, pools=pools16)
    for a, b in zip(got, want):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_layer_operator_in_the_input_type_head_dim_128(dtype):
    """The whole layer operator (estimate + map, pooling, tile schedule for the 16-bit types, forward) on fp16 / fp32
    tensors with head dim 128 and 128-token blocks: scores, map and output against the oracle on the same values."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn = 1, 2, 128, 128, 128, 32
    q, k, v = make_qkv(B, H, H, (3, 20, 26), D, seed=5, dtype=dtype)  # 1560 tokens, ragged last block
    oq, ok = sample_offsets(B, H, bm, 32, 6), sample_offsets(B, H, bn, 32, 7)
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.45), 4: (0.45, 0.6), 8: (0.6, 0.8), 0: (0.8, 1.0)}
    qd, kd, vd, oqd, okd = (t.to(dev()) for t in (q, k, v, oq, ok))
    out, mp = ops.psa_layer_fwd(qd, kd, vd, oqd, okd, ratios, "thresholdbound", bm, bn, tn, return_map=True)
    scores = ops.estimate_sampled(qd, kd, oqd, okd, bm, bn, 32, 32)
    torch.cuda.synchronize()
    assert out.dtype == dtype
    np.testing.assert_allclose(scores.cpu().numpy(), O.estimate_sampled(q, k, bm, bn, oq, ok).numpy(), rtol=2e-4, atol=1e-9)
    ref_map = O.level_map(scores.cpu().numpy(), ratios, 0, "thresholdbound", blocksize=bn, compute_tile=tn)
    assert np.array_equal(mp.cpu().numpy(), ref_map)
    ref, _ = O.psa_attention_blockwalk(q, k, v, ref_map, bm, bn)
    mx, mean = attn_errors(out, ref)
    assert mx <= TOL[dtype][0] and mean <= TOL[dtype][1], (mx, mean)
