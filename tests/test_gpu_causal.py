"""GPU parity of the causal (Qwen2.5-VL style) path: antidiagonal estimator, causal level-map rules, and
the module that chains them with the causal sparse forward."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, attn_errors, dev, rnd

pytestmark = pytest.mark.gpu
QWEN = {1: (0.0, 0.7), 2: (0.7, 0.8), 4: (0.8, 0.9), 8: (0.9, 0.9), 0: (0.9, 1.0)}


@pytest.mark.parametrize("B,Hq,Hkv,L,D,block,stride,chunk,causal",
                         [(1, 2, 2, 2048, 128, 128, 8, 1024, True), (1, 4, 2, 1500, 128, 128, 8, 1024, True),
                          (1, 2, 2, 1024, 64, 128, 16, 2048, True), (1, 1, 1, 2048, 128, 128, 4, 512, False),
                          (2, 2, 1, 700, 64, 64, 8, 1024, True)])
def test_xattn_estimate_matches_oracle(B, Hq, Hkv, L, D, block, stride, chunk, causal):
    from psa_hip import ops

    q, k = rnd(B, Hq, L, D, seed=1), rnd(B, Hkv, L, D, seed=2)
    got = ops.estimate_xattn(q.to(dev()), k.to(dev()), block_size=block, stride=stride, causal=causal, chunk_size=chunk)
    ref = O.estimate_xattn(q.float(), k.float(), block_size=block, stride=stride, causal=causal, chunk_size=chunk)
    assert got.shape == ref.shape
    np.testing.assert_allclose(got.cpu().numpy(), ref.numpy(), rtol=2e-3, atol=2e-6)
    nb = -(-L // block)
    if causal:
        assert float(got.cpu().triu(1).abs().max()) == 0.0  # nothing above the diagonal


@pytest.mark.parametrize("mode", ["energybound", "topk"])
@pytest.mark.parametrize("S,text,causal", [(16, 0, True), (40, 512, True), (33, 300, False), (256, 512, True)])
def test_qwen_level_map_bit_exact(mode, S, text, causal):
    from psa_hip import ops

    rng = np.random.default_rng(S)
    s = (rng.random((2, 3, S, S), dtype=np.float32) ** 6).astype(np.float32)
    if causal:
        s = np.tril(s)
    ratios = QWEN if mode == "energybound" else {1: (0.0, 0.05), 2: (0.05, 0.15), 4: (0.15, 0.25), 8: (0.25, 0.5), 0: (0.5, 1.0)}
    ref = O.level_map_qwen(s, ratios, text_length=text, mode=mode, block_size=128, causal=causal)
    got = ops.level_map_qwen(torch.from_numpy(s).to(dev()), ratios, text, mode, block_size=128, causal=causal)
    assert got.dtype == torch.int32 and np.array_equal(got.cpu().numpy(), ref)
    with pytest.raises(ValueError):
        ops.level_map_qwen(torch.from_numpy(s).to(dev()), {}, text, mode, block_size=128, causal=causal)
    with pytest.raises(ValueError):
        ops.level_map_qwen(torch.from_numpy(s).to(dev()), ratios, text, "thresholdbound", block_size=128, causal=causal)


def test_causal_module_end_to_end_gqa():
    from psa_hip import ops
    from psa_hip.PSA_casual import AttentionConfig, PyramidAdaptiveBlockSparseAttnTrain
    from psa_hip.utils.synthetic import make_qkv

    B, Hq, Hkv, D = 1, 4, 2, 128
    q, k, v = make_qkv(B, Hq, Hkv, (4, 16, 30), D, seed=3, text_tokens=128, text_first=True)  # L = 2048
    L = q.shape[2]
    cfg = AttentionConfig(mask_mode="energybound", mask_ratios=QWEN, xattn_stride=8, xattn_chunk_size=1024, text_length=256,
                          sim_2x_threshold=0.6, sim_4x_threshold=0.5, sim_8x_threshold=0.4)
    mod = PyramidAdaptiveBlockSparseAttnTrain(cfg, layer_idx=0)
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    out = mod(qd, kd, vd, layer_idx=3)
    assert out.shape == q.shape and torch.isfinite(out).all() and mod.layer_idx == 3
    # oracle chain from the GPU's own fp32 estimate (map contract: bit-exact from identical scores)
    est = ops.estimate_xattn(qd, kd, 128, 8, True, 1024)
    np.testing.assert_allclose(est.cpu().numpy(), O.estimate_xattn(q.float(), k.float(), 128, 8, True, 1024).numpy(), rtol=2e-3, atol=2e-6)
    ref_map = O.level_map_qwen(est.cpu().numpy(), QWEN, text_length=256, mode="energybound", block_size=128, causal=True)
    cap = O.k_similarity(k, 128, 0.6, 0.5, 0.4).repeat_interleave(Hq // Hkv, 1).numpy()
    ref_map = np.minimum(ref_map, cap[:, :, None, :])
    got_map = ops.map_min_cap(ops.level_map_qwen(est, QWEN, 256, "energybound", block_size=128, causal=True),
                              ops.k_similarity(kd, 128, 0.6, 0.5, 0.4).repeat_interleave(Hq // Hkv, 1))
    assert np.array_equal(got_map.cpu().numpy(), ref_map)
    ref, _ = O.psa_attention_blockwalk(q, k, v, ref_map, 128, 128, causal=True)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    # warm-up = dense attention WITHOUT a mask, as in the reference (scaled_dot_product_attention(q, k, v);
    # qwen2.5-vl-example/src/attention/PSA_casual/PyramidAdaptiveBlockSparseAttn.py:306-308)
    warm = PyramidAdaptiveBlockSparseAttnTrain(AttentionConfig(warmup_steps=1))
    o2 = warm(qd, kd, vd)
    refc = F.scaled_dot_product_attention(q.float(), k.float().repeat_interleave(2, 1), v.float().repeat_interleave(2, 1))
    mx, mean = attn_errors(o2, refc)
    assert mx <= MAX_ABS and mean <= MEAN_ABS
    with pytest.raises(ValueError):
        AttentionConfig(mask_mode="thresholdbound")
    with pytest.raises(ValueError):
        AttentionConfig(importance_method="pooling")
