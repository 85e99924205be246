"""GPU tests of the reference-compatible Python surface: PSAAttention / psa_attention,
PyramidSparseAttention (warm-up, Hilbert re-ordering, logging), the kernel-module entry points and the
key-similarity cap."""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, attn_errors, dev, rnd

pytestmark = pytest.mark.gpu


def smooth_qkv(B, H, grid, D, seed, text=0):
    from psa_hip.utils.synthetic import make_qkv

    return make_qkv(B, H, H, grid, D, seed=seed, text_tokens=text)


def test_ksim_matches_oracle():
    from psa_hip import ops

    q, k, v = smooth_qkv(2, 3, (4, 8, 20), 128, 3)  # L = 640
    k = torch.cat([k, k[:, :, :37]], 2)              # ragged: 677
    s2, s4, s8 = O.k_similarity_scores(k, 128)
    # thresholds in the middle of the observed range, kept away from every score
    def pick(s):
        vals = np.sort(s.numpy().ravel())
        gaps = np.diff(vals)
        i = int(np.argmax(gaps))
        return float((vals[i] + vals[i + 1]) / 2)
    t2, t4, t8 = pick(s2), pick(s4), pick(s8)
    got = ops.k_similarity(k.to(dev()), 128, t2, t4, t8)
    ref = O.k_similarity(k, 128, t2, t4, t8)
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), ref)
    assert len(set(ref.view(-1).tolist())) >= 2
    for bn, D in ((32, 64), (64, 64)):
        kk = rnd(1, 2, 300, D, seed=bn)
        assert torch.equal(ops.k_similarity(kk.to(dev()), bn, 0.0, 0.0, -1.0).cpu(), O.k_similarity(kk, bn, 0.0, 0.0, -1.0))


@pytest.mark.parametrize("impl,bn,mode,sim", [("new_mask_type", 64, "topk", False), ("new_mask_type", 32, "thresholdbound", False),
                                              ("old_mask_type", 128, "thresholdbound", True), ("old_mask_type", 128, "topk", False)])
def test_psa_attention_module_matches_oracle_layer(impl, bn, mode, sim):
    from psa_hip import PSAAttention, PSAConfig
    from psa_hip.utils.synthetic import sample_offsets

    B, H, D = 1, 2, 128
    q, k, v = smooth_qkv(B, H, (4, 16, 30), D, 5)  # L = 1920
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.45), 4: (0.45, 0.6), 8: (0.6, 0.8), 0: (0.8, 1.0)}
    cfg = PSAConfig(block_m=128, block_n=bn, tile_n=32, mask_ratios=ratios, mask_mode=mode, attn_impl=impl, use_sim_mask=sim,
                    sim_2x_threshold=0.5, sim_4x_threshold=0.4, sim_8x_threshold=0.3)
    psa = PSAAttention(cfg)
    oq, ok = sample_offsets(B, H, 128, 32, 1), sample_offsets(B, H, bn, bn // 4, 2)
    psa.sample_offsets = (oq.to(dev()), ok.to(dev()))
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    out = psa(qd, kd, vd)
    assert out.shape == q.shape and out.dtype == q.dtype
    mask = psa.build_mask(qd, kd, vd)
    # oracle: same scores (GPU fp32 scores feed the oracle's map: the map contract is bit-exact from identical scores)
    from psa_hip import ops

    scores = ops.estimate_sampled(qd, kd, psa.sample_offsets[0], psa.sample_offsets[1], 128, bn, 32, bn // 4).cpu().numpy()
    np.testing.assert_allclose(scores, O.estimate_sampled(q, k, 128, bn, oq, ok).numpy(), rtol=2e-4, atol=1e-9)
    ref_mask = O.level_map(scores, ratios, 0, mode if impl == "old_mask_type" else mode + "_newtype", blocksize=bn, compute_tile=32)
    if sim:
        cap = O.k_similarity(O.pad_replicate(k, bn), bn, 0.5, 0.4, 0.3).numpy()
        ref_mask = np.minimum(ref_mask, cap[:, :, None, :])
    assert np.array_equal(mask.cpu().numpy(), ref_mask)
    dense = ref_mask if impl == "old_mask_type" else O.list_to_dense(ref_mask, -(-q.shape[2] // bn))
    ref, _ = O.psa_attention_blockwalk(q, k, v, dense, 128, bn)
    mx, mean = attn_errors(out, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)


def test_psa_attention_functional_default_runs_and_is_close_to_dense_on_peaky_input():
    from psa_hip import psa_attention

    q, k, v = smooth_qkv(1, 2, (4, 16, 32), 64, 7)
    out = psa_attention(q.to(dev()), k.to(dev()), v.to(dev()))
    assert out.shape == q.shape and torch.isfinite(out).all()
    out2 = psa_attention(q.to(dev()), k.to(dev()), v.to(dev()), mask_ratios={1: (0, 1.0), 2: (1.0, 1.0), 4: (1.0, 1.0), 8: (1.0, 1.0), 0: (1.0, 1.0)},
                         mask_mode="topk", block_n=128)
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float())
    mx, mean = attn_errors(out2, ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS  # every block at level 1 == dense attention


def test_kernel_module_entry_points():
    from psa_hip.kernels.attn_pooling_kernel import attn_with_pooling_optimized
    from psa_hip.utils import calc_density, calc_density_newtype, transfer_attn_to_mask

    sq, sk = rnd(1, 2, 192, 128, seed=1), rnd(1, 2, 128, 128, seed=2)
    _, po = attn_with_pooling_optimized(sq.to(dev()), sk.to(dev()), sk.to(dev()), False, 128 ** -0.5, 32, 32)
    ref = O.estimate_from_sampled(sq, sk, 128 ** -0.5, 32, 32)
    assert po.shape == ref.shape
    np.testing.assert_allclose(po.cpu().numpy(), ref.numpy(), rtol=2e-4, atol=1e-9)
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.5), 4: (0.5, 0.7), 8: (0.7, 0.9), 0: (0.9, 1.0)}
    s = torch.rand(1, 2, 6, 40)
    m = transfer_attn_to_mask(s.to(dev()), ratios, 226, "thresholdbound", blocksize=128, compute_tile=32)
    assert m.dtype == torch.int32
    assert np.array_equal(m.cpu().numpy(), O.level_map(s.numpy(), ratios, 226, "thresholdbound", blocksize=128, compute_tile=32))
    avg, per_head = calc_density(m)
    assert abs(avg - O.density(m.cpu().numpy())) < 1e-6 and len(per_head) == 2
    lst = transfer_attn_to_mask(s.to(dev()), ratios, 0, "topk_newtype", blocksize=128, compute_tile=32)
    avg2, _ = calc_density_newtype(lst)
    assert abs(avg2 - O.density(O.level_map(s.numpy(), ratios, 0, "topk", blocksize=128, compute_tile=32))) < 1e-6


def test_pyramid_sparse_attention_warmup_rearrange_and_logging(tmp_path):
    from psa_hip import AttentionConfig, PyramidSparseAttention
    from psa_hip.config_loader import AttentionConfigLoader

    W, Hh, T, text = 16, 8, 6, 0
    params = AttentionConfigLoader().get_attention_config("Wan2.1_1.3b", "psa_balanced", [W * 16, Hh * 16, T * 4])["params"]
    assert (params["width"], params["height"], params["depth"]) == (W, Hh, T)
    params.update(warmup_steps=1, log_dir=str(tmp_path), enable_logging=True, verbose=False)
    cfg = AttentionConfig(**params)
    layers = 2
    mod = PyramidSparseAttention(cfg, inference_num=4, layer_num=layers, model_type="wan")
    q, k, v = smooth_qkv(1, 2, (T, Hh, W), 128, 11)
    qd, kd, vd = q.to(dev()), k.to(dev()), v.to(dev())
    ref = F.scaled_dot_product_attention(q.float(), k.float(), v.float())
    outs = []
    for step in range(2):            # wan: cond + uncond pass per step -> 2 * layers calls per step
        for _ in range(2):
            for layer in range(layers):
                outs.append(mod(qd, kd, vd, layer))
    # step 0 is warm-up: dense attention in the ORIGINAL token order (rearrange + inverse cancel)
    mx, mean = attn_errors(outs[0], ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS
    # step 1 is sparse: finite, same shape, and not identical to dense
    assert outs[-1].shape == q.shape and torch.isfinite(outs[-1]).all()
    assert float((outs[-1].float().cpu() - ref).abs().mean()) < 0.1
    assert mod.sparsity_counter == 8 and mod.get_current_time() == 2
    mod.close_logger()
    logs = [os.path.join(dp, f) for dp, _, fs in os.walk(tmp_path) for f in fs]
    lines = [json.loads(l) for f in logs if f.endswith("sparsity.jsonl") for l in open(f)]
    assert len(lines) == 8 and lines[0]["is_warmup"] and not lines[-1]["is_warmup"]
    assert 0.0 < lines[-1]["sparsity"] < 1.0 and len(lines[-1]["per_head_density"]) == 2
    # the reference's schema: running step number, time stamp, similarity-cap histogram (this preset uses the cap)
    assert [l["global_step"] for l in lines] == list(range(1, 9)) and all("timestamp" in l for l in lines)
    assert lines[-1]["use_sim_mask"] and abs(sum(lines[-1]["sim_mask_stats"].values()) - 1.0) < 1e-5
    assert sum(lines[0]["sim_mask_stats"].values()) == 0.0  # warm-up calls carry no cap
    summary = [f for f in logs if f.endswith("summary.txt")]
    assert len(summary) == 1 and "Warmup Samples (density=1.0): 4" in open(summary[0]).read()


def test_pyramid_sparse_attention_text_tokens_cogvideo_preset():
    from psa_hip import AttentionConfig, PyramidSparseAttention
    from psa_hip.config_loader import AttentionConfigLoader

    params = AttentionConfigLoader().get_attention_config("CogVideo_5b", "psa_4steps", (16 * 16, 8 * 16, 4 * 4))["params"]
    params.update(enable_logging=False, text_length=226)
    mod = PyramidSparseAttention(AttentionConfig(**params), inference_num=4, layer_num=1, model_type="cogvideo")
    q, k, v = smooth_qkv(2, 2, (4, 8, 16), 64, 13, text=226)  # text tokens are appended at the end by make_qkv
    out = mod(q.to(dev()), k.to(dev()), v.to(dev()), 0)
    assert out.shape == q.shape and torch.isfinite(out).all()


def test_layer_function_equals_the_stages_in_sequence():
    """psa_layer_fwd: map and output must be bit-identical to the stages called one after the other."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    dev = torch.device("cuda:0")
    B, H, D, bm, bn, tn = 1, 3, 128, 128, 128, 32
    q, k, v = make_qkv(B, H, H, (4, 16, 40), D, seed=7, device=dev)  # L = 2560
    off_q = sample_offsets(B, H, bm, bm // 4, 17, device=dev)
    off_k = sample_offsets(B, H, bn, bn // 4, 18, device=dev)
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.4), 4: (0.4, 0.5), 8: (0.5, 0.6), 0: (0.6, 1.0)}
    s = ops.estimate_sampled(q, k, off_q, off_k, bm, bn, bm // 4, bn // 4)
    mp = ops.level_map(s, ratios, 0, "thresholdbound", blocksize=bn, compute_tile=tn, map_dtype=torch.int8)
    ref = ops.sparse_attention_fwd(q, k, v, mp, bm, bn)
    for _ in range(2):
        out, m2 = ops.psa_layer_fwd(q, k, v, off_q, off_k, ratios, "thresholdbound", bm, bn, tn, return_map=True)
        torch.cuda.synchronize()
        assert torch.equal(m2, mp)
        assert torch.equal(out, ref)


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_layer_operator_with_pooling_on_the_second_stream(in_dtype, monkeypatch):
    """psa_layer_fwd runs the pooling pass on a second stream beside the estimator when K is large (>= 16 MiB); here the
    threshold is lowered so that a small layer takes that path: out and map must be the bits of the stage-by-stage
    sequence on one stream, also for fp32 inputs (whose temporary bf16 copies cross the streams)."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn = 1, 4, 128, 128, 128, 32
    q, k, v = make_qkv(B, H, H, (4, 16, 20), D, seed=5)
    oq, ok = sample_offsets(B, H, bm, 32, 6).to(dev()), sample_offsets(B, H, bn, 32, 7).to(dev())
    qd, kd, vd = (t.to(dev()).to(in_dtype) for t in (q, k, v))
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.4), 4: (0.4, 0.5), 8: (0.5, 0.6), 0: (0.6, 1.0)}
    # stage by stage, one stream
    mp_ref = ops.estimate_sampled_map(qd, kd, oq, ok, bm, bn, 32, 32, ratios, 0, "thresholdbound", compute_tile=tn, map_dtype=torch.int8)
    out_ref = ops.sparse_attention_fwd(qd, kd, vd, mp_ref, bm, bn, pools=ops.pool_kv(kd, vd, bn))
    torch.cuda.synchronize()
    monkeypatch.setattr(ops, "_SIDE_STREAM_MIN_BYTES", 0)
    for _ in range(3):  # (an ordering bug between the streams would show up intermittently)
        out, mp = ops.psa_layer_fwd(qd, kd, vd, oq, ok, ratios, "thresholdbound", bm, bn, tn, return_map=True)
        torch.cuda.synchronize()
        assert torch.equal(mp, mp_ref) and torch.equal(out, out_ref) and out.dtype == in_dtype


def test_layer_operator_as_one_graph():
    """psa_layer_fwd_graph: the layer captured into one HIP graph (estimator, reduction + map, schedule, attention; pooling
    on a second branch) gives the eager layer's bits on every replay, with eager work of the program between replays,
    follows the CONTENTS of its input tensors, and captures anew for tensors at other addresses."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    B, H, D, bm, bn, tn = 1, 8, 128, 128, 128, 32
    q, k, v = (t.to(dev()) for t in make_qkv(B, H, H, (8, 16, 32), D, seed=11))  # 4096 tokens: K is 8 MiB
    oq, ok = sample_offsets(B, H, bm, 32, 12).to(dev()), sample_offsets(B, H, bn, 32, 13).to(dev())
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.4), 4: (0.4, 0.5), 8: (0.5, 0.6), 0: (0.6, 1.0)}
    for side_min in (0, 1 << 40):  # with and without the second branch for the pooling pass
        ops._SIDE_STREAM_MIN_BYTES, saved = side_min, ops._SIDE_STREAM_MIN_BYTES
        try:
            ops._LAYER_GRAPHS.clear()
            ref, ref_map = ops.psa_layer_fwd(q, k, v, oq, ok, ratios, "thresholdbound", bm, bn, tn, return_map=True)
            ref, ref_map = ref.clone(), ref_map.clone()
            for rep in range(3):
                junk = torch.randn(1 << 20, device=dev()).sum()
                torch.cuda.synchronize()
                out, mp = ops.psa_layer_fwd_graph(q, k, v, oq, ok, ratios, "thresholdbound", bm, bn, tn, return_map=True)
                torch.cuda.synchronize()
                assert torch.equal(out, ref) and torch.equal(mp, ref_map), (side_min, rep)
                assert torch.isfinite(junk)
            assert len(ops._LAYER_GRAPHS) == 1
            # new contents at the same addresses: the replay computes the new layer
            q2 = torch.roll(q, 17, dims=2).contiguous()
            ref2 = ops.psa_layer_fwd(q2, k, v, oq, ok, ratios, "thresholdbound", bm, bn, tn).clone()
            q_saved = q.clone()
            q.copy_(q2)
            out2, _ = ops.psa_layer_fwd_graph(q, k, v, oq, ok, ratios, "thresholdbound", bm, bn, tn, return_map=True)
            torch.cuda.synchronize()
            assert torch.equal(out2, ref2) and len(ops._LAYER_GRAPHS) == 1
            q.copy_(q_saved)
            # other tensors: another graph
            out3, _ = ops.psa_layer_fwd_graph(q2, k, v, oq, ok, ratios, "thresholdbound", bm, bn, tn, return_map=True)
            torch.cuda.synchronize()
            assert torch.equal(out3, ref2) and len(ops._LAYER_GRAPHS) == 2
        finally:
            ops._SIDE_STREAM_MIN_BYTES = saved
            ops._LAYER_GRAPHS.clear()


def test_token_index_made_under_inference_mode():
    """An index tensor created under torch.inference_mode has no version counter: its contents are checked on every
    call instead of once, and the operators take it like any other."""
    from psa_hip import ops
    from psa_hip.utils.rearranger import GilbertRearranger

    L = 4 * 6 * 8
    k, v = rnd(1, 2, L, 128, seed=1).to(dev()), rnd(1, 2, L, 128, seed=2).to(dev())
    with torch.inference_mode():
        rr = GilbertRearranger(8, 6, 4, 0)
        idx = rr.token_index(dev())
        raw = idx.clone()  # an inference tensor
        assert raw.is_inference() and not idx.is_inference()
        a = ops.pool_kv_indexed(k, v, idx, 32)
        b = ops.pool_kv_indexed(k, v, raw, 32)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    bad = raw.clone()
    with torch.inference_mode():
        worse = bad.clone()
        worse[3] = worse[4]
        with pytest.raises(ValueError):
            ops.pool_kv_indexed(k, v, worse, 32)
