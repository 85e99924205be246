"""GPU tests that run the five named workloads (small fp32-sized layer, Wan2.1 layer, CogVideoX joint attention,
training step, causal GQA prefill) as workloads through the C ABI:

  * at sizes the CPU oracle finishes in seconds: the whole layer against the oracle (scores within 2e-4, level map
    bit-exact from the GPU's fp32 scores, output within max-abs 2e-2 / mean-abs 2e-3);
  * at the full sequence lengths: through a size-independent property.  If K and V are constant inside aligned
    groups of 8 tokens, mean-pooling by 2/4/8 loses nothing and the +log(level) bias makes a pooled key count as
    `level` keys, so ANY level map without skips must reproduce plain attention - forward and backward - and causal
    attention when the diagonal blocks are at level 1.  The comparison partner is torch's
    scaled_dot_product_attention (and its autograd) on the GPU.
Gradient tolerance: relative L2 <= 5e-2 per tensor."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, attn_errors, dev

pytestmark = pytest.mark.gpu
REL_L2 = 5e-2
WAN13 = {1: (0.0, 0.5), 2: (0.5, 0.6), 4: (0.6, 0.7), 8: (0.7, 0.8), 0: (0.8, 1.0)}
COG_4STEPS = {1: (0.0, 0.05), 2: (0.05, 0.15), 4: (0.15, 0.25), 8: (0.25, 0.5), 0: (0.5, 1.0)}


def rel_l2(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def scaled(tau):
    return {lv: (lo * tau if lv else 0.8 * tau, hi * tau if lv else 1.0) for lv, (lo, hi) in WAN13.items()}


def calibrate(ops, scores, target_sparsity, bn, tn, text=0):
    lo, hi = 0.05, 1.25
    for _ in range(16):
        tau = 0.5 * (lo + hi)
        m = ops.level_map(scores, scaled(tau), text, "thresholdbound", blocksize=bn, compute_tile=tn, map_dtype=torch.int8)
        if 1 - float(ops.density(m)[-1]) > target_sparsity:
            lo = tau
        else:
            hi = tau
    return scaled(tau)


def group_constant_kv(Hkv, L, D, seed, q_scale=0.5, Hq=None):
    """q random; k, v constant inside aligned groups of 8 tokens (the last group may be cut by L)."""
    g = torch.Generator().manual_seed(seed)
    n8 = -(-L // 8)
    bk = torch.randn(1, Hkv, n8, D, generator=g).bfloat16()
    bv = torch.randn(1, Hkv, n8, D, generator=g).bfloat16()
    k = bk.repeat_interleave(8, 2)[:, :, :L].contiguous()
    v = bv.repeat_interleave(8, 2)[:, :, :L].contiguous()
    q = (torch.randn(1, Hq or Hkv, L, D, generator=g) * q_scale).bfloat16()
    return q, k, v


def no_skip_map(H, Mq, Nk, seed, causal=False):
    m = np.random.default_rng(seed).choice([1, 2, 4, 8], size=(1, H, Mq, Nk)).astype(np.int8)
    m[..., -1] = 1  # the last kv-block holds the replicate-padded tail: pooled keys there would add copies of the last token
    if causal:
        d = np.arange(min(Mq, Nk))
        m[..., d, d] = 1  # what the causal callers of the reference force
    return m


# ------------------------------------------------------------------------------------------------ c1
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_c1_small_layer_full_size_vs_oracle(in_dtype):
    """B1 H2 N4096 (4x32x32 grid) D64, blocks of 64, tile_n 16, thresholdbound at ~80 % sparsity: the whole layer.
    Every stage computes in the dtype of its inputs (bf16 and fp16 on the matrix cores with fp32 accumulation, fp32
    on the vector units): the oracle is run on the inputs as they are, never on rounded copies, and the output must
    meet the same bound for each of the three dtypes."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn = 1, 2, 64, 64, 64, 16
    q32, k32, v32 = make_qkv(B, H, H, (4, 32, 32), D, seed=1234, dtype=torch.float32)
    qi, ki, vi = (t.to(in_dtype) for t in (q32, k32, v32))
    oq, ok = sample_offsets(B, H, bm, bm // 4, 1244), sample_offsets(B, H, bn, bn // 4, 1245)
    qd, kd, vd, oqd, okd = (t.to(dev()) for t in (qi, ki, vi, oq, ok))
    scores = ops.estimate_sampled(qd, kd, oqd, okd, bm, bn, bm // 4, bn // 4)
    ratios = calibrate(ops, scores, 0.80, bn, tn)
    out, mp = ops.psa_layer_fwd(qd, kd, vd, oqd, okd, ratios, "thresholdbound", bm, bn, tn, return_map=True)
    torch.cuda.synchronize()
    assert out.dtype == in_dtype and out.shape == qi.shape
    sparsity = 1 - float(ops.density(mp)[-1])
    assert 0.74 <= sparsity <= 0.86, sparsity
    # estimator, level map, attention against the oracle on the very values the caller passed
    ref_scores = O.estimate_sampled(qi, ki, bm, bn, oq, ok)
    np.testing.assert_allclose(scores.cpu().numpy(), ref_scores.numpy(), rtol=2e-4, atol=1e-9)
    ref_map = O.level_map(scores.cpu().numpy(), ratios, 0, "thresholdbound", blocksize=bn, compute_tile=tn)
    assert np.array_equal(mp.cpu().numpy(), ref_map)
    ref, _ = O.psa_attention_blockwalk(qi, ki, vi, ref_map, bm, bn)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    if in_dtype == torch.float32:
        # nothing is rounded on the fp32 path but the order of the sums: three orders of magnitude below the bound
        assert mx <= 2e-5, mx


# ------------------------------------------------------------------------------------------------ c2 (reduced; the full size is the benchmark's workload)
def test_c2_wan_layer_reduced_vs_oracle():
    """The Wan2.1 layer configuration (D 128, blocks of 128, thresholdbound at ~90 % sparsity) on a 6x20x26 grid
    (3120 tokens, ragged last block), 3 heads, end to end against the oracle."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn = 1, 3, 128, 128, 128, 32
    q, k, v = make_qkv(B, H, H, (6, 20, 26), D, seed=1234)
    oq, ok = sample_offsets(B, H, bm, 32, 1244), sample_offsets(B, H, bn, 32, 1245)
    qd, kd, vd, oqd, okd = (t.to(dev()) for t in (q, k, v, oq, ok))
    scores = ops.estimate_sampled(qd, kd, oqd, okd, bm, bn, 32, 32)
    ratios = calibrate(ops, scores, 0.90, bn, tn)
    out, mp = ops.psa_layer_fwd(qd, kd, vd, oqd, okd, ratios, "thresholdbound", bm, bn, tn, return_map=True)
    np.testing.assert_allclose(scores.cpu().numpy(), O.estimate_sampled(q, k, bm, bn, oq, ok).numpy(), rtol=2e-4, atol=1e-9)
    ref_map = O.level_map(scores.cpu().numpy(), ratios, 0, "thresholdbound", blocksize=bn, compute_tile=tn)
    assert np.array_equal(mp.cpu().numpy(), ref_map)
    ref, _ = O.psa_attention_blockwalk(q, k, v, ref_map, bm, bn)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)


def test_c2_wan_layer_full_size_vs_oracle():
    """The headline workload at its own size: B 1, H 12, N 32760 (21x30x52 grid), D 128, blocks of 128, thresholdbound
    calibrated to ~90 % sparsity, rows issued longest first through the tile schedule - the whole layer operator.
    Scores of all 12 heads against the oracle (rtol 2e-4), the level map of all heads bit for bit from the GPU's
    scores, and the output of two heads - every q-block, so every phase of the row dealing and both ends of the
    longest-first order - against the oracle's block walk on the host (max-abs 2e-2, mean-abs 2e-3)."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn = 1, 12, 128, 128, 128, 32
    q, k, v = make_qkv(B, H, H, (21, 30, 52), D, seed=1234)
    L = q.shape[2]
    assert L == 32760
    oq, ok = sample_offsets(B, H, bm, 32, 1244), sample_offsets(B, H, bn, 32, 1245)
    qd, kd, vd, oqd, okd = (t.to(dev()) for t in (q, k, v, oq, ok))
    scores = ops.estimate_sampled(qd, kd, oqd, okd, bm, bn, 32, 32)
    ratios = calibrate(ops, scores, 0.90, bn, tn)
    out, mp = ops.psa_layer_fwd(qd, kd, vd, oqd, okd, ratios, "thresholdbound", bm, bn, tn, return_map=True)
    torch.cuda.synchronize()
    assert abs(float(ops.density(mp)[-1]) - 0.10) < 0.01
    torch.set_num_threads(min(torch.get_num_threads(), 16))
    heads = [1, 10]  # (one head per half of the phases of the row dealing)
    np.testing.assert_allclose(scores.cpu().numpy(), O.estimate_sampled(q, k, bm, bn, oq, ok).numpy(), rtol=2e-4, atol=1e-9)
    ref_map = O.level_map(scores.cpu().numpy(), ratios, 0, "thresholdbound", blocksize=bn, compute_tile=tn)
    assert np.array_equal(mp.cpu().numpy(), ref_map)
    ref, _ = O.psa_attention_blockwalk(q[:, heads], k[:, heads], v[:, heads], ref_map[:, heads], bm, bn)
    mx, mean = attn_errors(out[:, heads], ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)


# ------------------------------------------------------------------------------------------------ c3
def test_c3_cogvideox_reduced_end_to_end_vs_oracle():
    """B 2 (CFG), D 64, blocks of 128, 226 text tokens after a 5x12x20 video grid, top-k with the ratios of the
    4-step CogVideoX-5B preset, dense ("old type") map so that the text rule applies: the last ceil(226/128) = 2
    kv-block columns are at level 1 for every q-block."""
    from psa_hip import PSAAttention, PSAConfig, ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn, text = 2, 4, 64, 128, 128, 32, 226
    q, k, v = make_qkv(B, H, H, (5, 12, 20), D, seed=77, text_tokens=text)
    L = q.shape[2]
    assert L == 1200 + 226
    oq, ok = sample_offsets(B, H, bm, 32, 5), sample_offsets(B, H, bn, 32, 6)
    qd, kd, vd, oqd, okd = (t.to(dev()) for t in (q, k, v, oq, ok))
    out, mp = ops.psa_layer_fwd(qd, kd, vd, oqd, okd, COG_4STEPS, "topk", bm, bn, tn, return_map=True, text_length=text)
    scores = ops.estimate_sampled(qd, kd, oqd, okd, bm, bn, 32, 32)
    np.testing.assert_allclose(scores.cpu().numpy(), O.estimate_sampled(q, k, bm, bn, oq, ok).numpy(), rtol=2e-4, atol=1e-9)
    ref_map = O.level_map(scores.cpu().numpy(), COG_4STEPS, text, "topk", blocksize=bn, compute_tile=tn)
    got_map = mp.cpu().numpy()
    assert np.array_equal(got_map, ref_map)
    assert (got_map[..., -2:] == 1).all()
    ref, _ = O.psa_attention_blockwalk(q, k, v, ref_map, bm, bn)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    # the module surface with the preset's fields gives the same map and output
    cfg = PSAConfig(block_m=bm, block_n=bn, tile_n=tn, mask_ratios=COG_4STEPS, mask_mode="topk", attn_impl="old_mask_type")
    psa = PSAAttention(cfg)
    psa.sample_offsets = (oqd, okd)
    mask = psa.build_mask(qd, kd, vd)
    # (PSAAttention applies no text rule - that is the diffusers module's, which passes text_length - so its map is
    # the same ranking without the forced columns)
    assert np.array_equal(mask.cpu().numpy(), O.level_map(scores.cpu().numpy(), COG_4STEPS, 0, "topk", blocksize=bn, compute_tile=tn))


def test_c3_cogvideox_full_size_vs_oracle():
    """The CogVideoX-5B configuration at its own size: B 2, H 48, N 17776 (13x30x45 video grid + 226 text tokens), D 64,
    blocks of 128, top-k with the preset's ratios, the layer operator (head dim 64: the one-row kernel).  Scores of four
    (batch, head) pairs against the oracle (rtol 2e-4), their map rows bit for bit from the GPU's scores (text columns at
    level 1), and their outputs - all q-blocks - against the oracle's block walk (max-abs 2e-2, mean-abs 2e-3)."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn, text = 2, 48, 64, 128, 128, 32, 226
    q, k, v = make_qkv(B, H, H, (13, 30, 45), D, seed=1234, text_tokens=text)
    L = q.shape[2]
    assert L == 17776
    oq, ok = sample_offsets(B, H, bm, 32, 1244), sample_offsets(B, H, bn, 32, 1245)
    qd, kd, vd, oqd, okd = (t.to(dev()) for t in (q, k, v, oq, ok))
    out, mp = ops.psa_layer_fwd(qd, kd, vd, oqd, okd, COG_4STEPS, "topk", bm, bn, tn, return_map=True, text_length=text)
    scores = ops.estimate_sampled(qd, kd, oqd, okd, bm, bn, 32, 32)
    torch.cuda.synchronize()
    torch.set_num_threads(min(torch.get_num_threads(), 16))
    heads = [0, 47]
    ref_scores = O.estimate_sampled(q[:, heads], k[:, heads], bm, bn, oq[:, heads], ok[:, heads])
    np.testing.assert_allclose(scores[:, heads].cpu().numpy(), ref_scores.numpy(), rtol=2e-4, atol=1e-9)
    ref_map = O.level_map(scores[:, heads].cpu().numpy(), COG_4STEPS, text, "topk", blocksize=bn, compute_tile=tn)
    got_map = mp[:, heads].cpu().numpy()
    assert np.array_equal(got_map, ref_map)
    assert (got_map[..., -2:] == 1).all()
    ref, _ = O.psa_attention_blockwalk(q[:, heads], k[:, heads], v[:, heads], ref_map, bm, bn)
    mx, mean = attn_errors(out[:, heads], ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)


def test_c3_kernel_at_full_length_lossless_property():
    """The kernel c3 runs (head dim 64, 128-row q-blocks: the one-row kernel) at c3's sequence length N = 17776
    (139 blocks, last one 112 tokens), one head, random map without skips on group-constant K/V vs SDPA."""
    from psa_hip import ops

    L, D = 17776, 64
    q, k, v = group_constant_kv(1, L, D, 3)
    lm = torch.from_numpy(no_skip_map(1, 139, 139, 4)).to(dev())
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    out = ops.sparse_attention_fwd(qd, kd, vd, lm, 128, 128)
    ref = F.scaled_dot_product_attention(qd, kd, vd)
    d = (out.float() - ref.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS, (float(d.max()), float(d.mean()))


# ------------------------------------------------------------------------------------------------ c4
def _sdpa_grads(q, k, v, do, causal, n_rep=1):
    q, k, v = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    kk, vv = (k.repeat_interleave(n_rep, 1), v.repeat_interleave(n_rep, 1)) if n_rep > 1 else (k, v)
    o = F.scaled_dot_product_attention(q, kk, vv, is_causal=causal)
    o.backward(do)
    return o.detach(), q.grad, k.grad, v.grad


def test_c4_training_step_at_full_length_lossless_property():
    """Forward with LSE + backward at N = 32760, D 128, one head: 256 q-blocks per key-block column (the column
    sort, the long q-block lists of the dK/dV walk, the large row offsets) - dQ, dK, dV against SDPA autograd."""
    from psa_hip import ops

    L, D = 32760, 128
    q, k, v = group_constant_kv(1, L, D, 5)
    g = torch.Generator().manual_seed(9)
    do = (torch.randn(1, 1, L, D, generator=g) * 0.02).bfloat16()
    lm = torch.from_numpy(no_skip_map(1, 256, 256, 6)).to(dev())
    qd, kd, vd, dod = (t.to(dev()) for t in (q, k, v, do))
    out, lse, pools = ops.sparse_attention_fwd(qd, kd, vd, lm, 128, 128, return_lse=True)
    dq, dk, dv = ops.sparse_attention_bwd(qd, kd, vd, lm, out, dod, lse, 128, 128, pools=pools)
    ro, rq, rk, rv = _sdpa_grads(qd, kd, vd, dod, False)
    d = (out.float() - ro.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS
    errs = rel_l2(dq, rq), rel_l2(dk, rk), rel_l2(dv, rv)
    assert max(errs) <= REL_L2, errs


@pytest.mark.parametrize("Hq,Hkv", [(2, 2), (4, 2)])
def test_causal_backward_at_8k_lossless_property(Hq, Hkv):
    """Causal forward + backward at N = 8320 (65 blocks), with and without grouped query heads."""
    from psa_hip import ops

    L, D = 8320, 128
    q, k, v = group_constant_kv(Hkv, L, D, 11 + Hq, Hq=Hq)
    g = torch.Generator().manual_seed(12)
    do = (torch.randn(1, Hq, L, D, generator=g) * 0.05).bfloat16()
    lm = torch.from_numpy(no_skip_map(Hq, 65, 65, 13, causal=True)).to(dev())
    qd, kd, vd, dod = (t.to(dev()) for t in (q, k, v, do))
    out, lse, pools = ops.sparse_attention_fwd(qd, kd, vd, lm, 128, 128, causal=True, return_lse=True)
    dq, dk, dv = ops.sparse_attention_bwd(qd, kd, vd, lm, out, dod, lse, 128, 128, causal=True, pools=pools)
    ro, rq, rk, rv = _sdpa_grads(qd, kd, vd, dod, True, n_rep=Hq // Hkv)
    d = (out.float() - ro.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS
    errs = rel_l2(dq, rq), rel_l2(dk, rk), rel_l2(dv, rv)
    assert max(errs) <= REL_L2, errs


# ------------------------------------------------------------------------------------------------ c5
def test_c5_causal_gqa_at_full_length_lossless_property():
    """Causal forward with LSE at N = 32768, 4 query heads on 2 kv heads, diagonal at level 1, vs causal SDPA."""
    from psa_hip import ops

    L, D, Hq, Hkv = 32768, 128, 4, 2
    q, k, v = group_constant_kv(Hkv, L, D, 21, Hq=Hq)
    lm = torch.from_numpy(no_skip_map(Hq, 256, 256, 22, causal=True)).to(dev())
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    out, lse, _ = ops.sparse_attention_fwd(qd, kd, vd, lm, 128, 128, causal=True, return_lse=True)
    ref = F.scaled_dot_product_attention(qd, kd.repeat_interleave(2, 1), vd.repeat_interleave(2, 1), is_causal=True)
    d = (out.float() - ref.float()).abs()
    assert float(d.max()) <= MAX_ABS and float(d.mean()) <= MEAN_ABS, (float(d.max()), float(d.mean()))
    # LSE of a few rows against the plain definition (fp32 on the GPU)
    rows = torch.tensor([0, 1, 127, 128, 4097, 20000, 32767], device=dev())
    s = torch.einsum("hqd,hkd->hqk", qd[0, :, rows].float(), kd[0].repeat_interleave(2, 0).float()) / D ** 0.5
    s = s.masked_fill(torch.arange(L, device=dev()).view(1, 1, -1) > rows.view(1, -1, 1), float("-inf"))
    torch.testing.assert_close(lse[0][:, rows], torch.logsumexp(s, -1), rtol=2e-3, atol=2e-3)


def test_c5_reduced_prefill_vs_oracle():
    """The causal prefill configuration end to end on 2048 tokens (256 text + 7x16x16 vision), 4 query heads on 2 kv
    heads, antidiagonal estimate with stride 8, energy-bound map: estimate, map (bit-exact from the GPU scores) and
    output against the oracle."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv

    B, Hq, Hkv, D, text = 1, 4, 2, 128, 256
    q, k, v = make_qkv(B, Hq, Hkv, (7, 16, 16), D, seed=31, text_tokens=text, text_first=True)
    L = q.shape[2]
    assert L == 2048
    ratios = {1: (0.0, 0.7), 2: (0.7, 0.8), 4: (0.8, 0.9), 8: (0.9, 0.9), 0: (0.9, 1.0)}
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    est = ops.estimate_xattn(qd, kd, block_size=128, stride=8, causal=True, chunk_size=1024)
    np.testing.assert_allclose(est.cpu().numpy(), O.estimate_xattn(q.float(), k.float(), 128, 8, True, 1024).numpy(), rtol=2e-3, atol=2e-6)
    mp = ops.level_map_qwen(est, ratios, text, "energybound", block_size=128, causal=True, map_dtype=torch.int8)
    ref_map = O.level_map_qwen(est.cpu().numpy(), ratios, text_length=text, mode="energybound", block_size=128, causal=True)
    assert np.array_equal(mp.cpu().numpy(), ref_map)
    out = ops.sparse_attention_fwd(qd, kd, vd, mp, 128, 128, causal=True)
    ref, _ = O.psa_attention_blockwalk(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), ref_map, 128, 128, causal=True)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)


def test_c5_qwen_prefill_full_size_vs_oracle():
    """The causal prefill configuration at its own size: B 1, 28 query heads on 4 kv heads, N 32768 (1024 text tokens first,
    then the first 31744 positions of a 17x44x44 vision grid), D 128, antidiagonal estimate at stride 8, energy-bound map, causal GQA forward through the
    tile schedule.  For the first and the last query head: estimate against the oracle, map rows bit for bit from the
    GPU's estimate, output and LSE of every q-block against the oracle's causal block walk."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv

    B, Hq, Hkv, D, text = 1, 28, 4, 128, 1024
    q, k, v = (t[:, :, :32768].contiguous() for t in make_qkv(B, Hq, Hkv, (17, 44, 44), D, seed=1234, text_tokens=text, text_first=True))
    L = q.shape[2]
    assert L == 32768
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.36), 4: (0.36, 0.42), 8: (0.42, 0.48), 0: (0.48, 1.0)}
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    est = ops.estimate_xattn(qd, kd, block_size=128, stride=8, causal=True)
    mp = ops.level_map_qwen(est, ratios, text, "energybound", block_size=128, causal=True, map_dtype=torch.int8)
    out, lse, _ = ops.sparse_attention_fwd(qd, kd, vd, mp, 128, 128, causal=True, return_lse=True)
    torch.cuda.synchronize()
    dens = float(ops.density(mp, causal=True)[-1])
    assert 0.05 < dens < 0.6, dens
    torch.set_num_threads(min(torch.get_num_threads(), 16))
    for h in (0, 27):
        hk = h // (Hq // Hkv)
        ref_est = O.estimate_xattn(q[:, h:h + 1].float(), k[:, hk:hk + 1].float(), 128, 8, True)
        np.testing.assert_allclose(est[:, h:h + 1].cpu().numpy(), ref_est.numpy(), rtol=2e-3, atol=2e-6)
        ref_map = O.level_map_qwen(est[:, h:h + 1].cpu().numpy(), ratios, text_length=text, mode="energybound", block_size=128, causal=True)
        assert np.array_equal(mp[:, h:h + 1].cpu().numpy(), ref_map)
        ref, ref_lse = O.psa_attention_blockwalk(q[:, h:h + 1], k[:, hk:hk + 1], v[:, hk:hk + 1], ref_map, 128, 128, causal=True)
        mx, mean = attn_errors(out[:, h:h + 1], ref)
        assert mx <= MAX_ABS and mean <= MEAN_ABS, (h, mx, mean)
        assert float((lse[:, h:h + 1].cpu() - ref_lse).abs().max()) <= 5e-3


def test_c5_gqa_ratio_7_forward_lse_backward_vs_oracle():
    """The head ratio of the causal prefill configuration (28 query heads on 4 kv heads = 7 per kv head) at 14 / 2 heads
    and 2048 tokens: causal forward, lse and backward on a random map with skips against the oracle (the backward's
    dK / dV sum seven query heads per kv head)."""
    from psa_hip import ops
    from gpu_util import random_map, rnd

    B, Hq, Hkv, L, D = 1, 14, 2, 2048, 128
    q, k, v = rnd(B, Hq, L, D, seed=71), rnd(B, Hkv, L, D, seed=72), rnd(B, Hkv, L, D, seed=73)
    do = rnd(B, Hq, L, D, seed=74, scale=0.02)
    lmap = random_map(B, Hq, 16, 16, 75)
    idx = np.arange(16)
    lmap[..., idx, idx] = 1  # (the diagonal is always kept at level 1 by the causal map rules)
    qd, kd, vd, dod, md = (t.to(dev()) for t in (q, k, v, do, torch.from_numpy(lmap)))
    out, lse, pools = ops.sparse_attention_fwd(qd, kd, vd, md, 128, 128, causal=True, return_lse=True)
    dq, dk, dv = ops.sparse_attention_bwd(qd, kd, vd, md, out, dod, lse, 128, 128, causal=True, pools=pools)
    torch.cuda.synchronize()
    ref, ref_lse = O.psa_attention_dense(q, k, v, lmap, 128, 128, causal=True)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    fin = torch.isfinite(ref_lse)
    assert float((lse.cpu().double()[fin] - ref_lse[fin]).abs().max()) <= 2e-2
    rdq, rdk, rdv = O.psa_backward_dense(q, k, v, lmap, do, 128, 128, causal=True)
    errs = [rel_l2(a.float().cpu(), b) for a, b in ((dq, rdq), (dk, rdk), (dv, rdv))]
    assert max(errs) <= REL_L2, errs
