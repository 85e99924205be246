"""GPU parity of the token re-ordering (row gather through the C ABI) against torch index_select + cat, the
formulation of the reference's GilbertRearranger (utils/rearranger.py:14-132).  Pure copies: bit-exact."""
import pytest
import torch

from gpu_util import dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("grid,text,D", [((3, 6, 10), 0, 128), ((4, 5, 7), 33, 64), ((2, 9, 11), 226, 128)])
def test_rearranger_matches_torch_path(dtype, grid, text, D):
    from psa_hip.utils.rearranger import GilbertRearranger

    depth, height, width = grid
    r = GilbertRearranger(width, height, depth, text)
    L = depth * height * width + text
    g = torch.Generator(device="cpu").manual_seed(L + D)
    q = torch.randn(2, 4, L, D, generator=g).to(dtype).to(dev())
    k = torch.randn(2, 2, L, D, generator=g).to(dtype).to(dev())   # fewer heads (GQA)
    v = torch.randn(2, 2, L, D, generator=g).to(dtype).to(dev())
    fwd = r.original_order2gilbert_order_cpu.to(dev())
    inv = r.gilbert_order2original_order_cpu.to(dev())

    def ref_forward(x):  # the reference's formulation: index_select of the video part, text appended
        if text == 0:
            return x.index_select(-2, fwd)
        return torch.cat((x[..., text:, :].index_select(-2, fwd), x[..., :text, :]), dim=-2)

    def ref_backward(x):
        if text == 0:
            return x.index_select(-2, inv)
        return torch.cat((x[..., -text:, :], x[..., :-text, :].index_select(-2, inv)), dim=-2)

    qr, kr, vr = r.rearrange(q, k, v)
    for a, x in ((qr, q), (kr, k), (vr, v)):
        assert torch.equal(a, ref_forward(x))
        assert torch.equal(r.rearrange_single(x), a)
    back = r.reversed_rearrange(qr)
    assert torch.equal(back, ref_backward(qr))
    assert torch.equal(back, q)  # the two orders are inverse permutations
    with pytest.raises(ValueError):
        r.rearrange_single(q.cpu())  # no torch fall-back


def test_gather_rows_strided_views_and_errors():
    from psa_hip import ops

    B, H, L, D = 1, 3, 500, 128
    g = torch.Generator(device="cpu").manual_seed(3)
    x = torch.randn(B, L, H, D, generator=g).to(torch.bfloat16).to(dev()).permute(0, 2, 1, 3)  # [B, H, L, D] view of [B, L, H, D]
    idx = torch.randperm(L, generator=g)[:321].to(torch.int32).to(dev())
    (y,) = ops.gather_rows((x,), idx)
    assert torch.equal(y, x.index_select(2, idx.long()))
    with pytest.raises(ValueError):
        ops.gather_rows((x,), idx.long())
    with pytest.raises(ValueError):
        ops.gather_rows((x, x[:, :, :100]), idx)
    with pytest.raises(Exception):
        ops.gather_rows((x.cpu(),), idx.cpu())


def _layer_inputs(B, Hq, Hkv, L, D, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, Hq, L, D, generator=g).to(torch.bfloat16).to(dev())
    k = torch.randn(B, Hkv, L, D, generator=g).to(torch.bfloat16).to(dev())
    v = torch.randn(B, Hkv, L, D, generator=g).to(torch.bfloat16).to(dev())
    idx = torch.randperm(L, generator=g).to(torch.int32).to(dev())
    inv = torch.empty_like(idx)
    inv[idx.long()] = torch.arange(L, dtype=torch.int32, device=idx.device)
    return q, k, v, idx, inv


@pytest.mark.parametrize("B,Hq,Hkv,L,D,bm,bn", [(1, 4, 4, 1500, 128, 128, 128), (2, 4, 2, 1111, 128, 128, 128),
                                                (1, 3, 3, 1000, 64, 64, 64), (1, 2, 2, 777, 64, 128, 32)])
def test_indexed_kernels_equal_gather_then_kernel(B, Hq, Hkv, L, D, bm, bn):
    """Pooling, estimator and attention forward reading / writing through the token index give, bit for bit, what the
    same kernels give on tensors gathered beforehand (and un-gathered afterwards): they move the same values."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import sample_offsets

    q, k, v, idx, inv = _layer_inputs(B, Hq, Hkv, L, D, seed=L + D)
    qg, kg, vg = (t.index_select(2, idx.long()) for t in (q, k, v))

    kp, vp, ko, vo = ops.pool_kv_indexed(k, v, idx, bn)
    kp_ref, vp_ref = ops.pool_kv(kg, vg, bn)
    assert torch.equal(ko, kg) and torch.equal(vo, vg)
    assert torch.equal(kp, kp_ref) and torch.equal(vp, vp_ref)

    km, kn = bm // 4, bn // 4
    off_q = sample_offsets(B, Hq, bm, km, 5, device=dev())
    off_k = sample_offsets(B, Hkv, bn, kn, 6, device=dev())
    s = ops.estimate_sampled(q, ko, off_q, off_k, bm, bn, km, kn, q_index=idx)
    s_ref = ops.estimate_sampled(qg, kg, off_q, off_k, bm, bn, km, kn)
    assert torch.equal(s, s_ref)

    ratios = {1: (0.0, 0.3), 2: (0.3, 0.5), 4: (0.5, 0.7), 8: (0.7, 0.85), 0: (0.85, 1.0)}
    m = ops.estimate_sampled_map(q, ko, off_q, off_k, bm, bn, km, kn, ratios, 0, "topk", map_dtype=torch.int8, q_index=idx)
    m_ref = ops.estimate_sampled_map(qg, kg, off_q, off_k, bm, bn, km, kn, ratios, 0, "topk", map_dtype=torch.int8)
    assert torch.equal(m, m_ref)
    mp = ops.level_map(s_ref, ratios, 0, "topk", blocksize=bn, compute_tile=min(32, bn), map_dtype=torch.int8)

    for causal in (False, True):
        if causal and bm != bn:
            continue
        o, lse, _ = ops.sparse_attention_fwd(q, ko, vo, mp, bm, bn, causal=causal, pools=(kp, vp), q_index=idx, return_lse=True)
        o_ref, lse_ref, _ = ops.sparse_attention_fwd(qg, kg, vg, mp, bm, bn, causal=causal, pools=(kp_ref, vp_ref), return_lse=True)
        assert torch.equal(o, o_ref.index_select(2, inv.long()))
        assert torch.equal(lse, lse_ref.index_select(2, inv.long()))
    # dense attention (no map) through the index
    o = ops.sparse_attention_fwd(q, ko, vo, None, bm, bn, q_index=idx)
    o_ref = ops.sparse_attention_fwd(qg, kg, vg, None, bm, bn)
    assert torch.equal(o, o_ref.index_select(2, inv.long()))


def test_indexed_argument_errors():
    from psa_hip import ops

    q, k, v, idx, _ = _layer_inputs(1, 2, 2, 300, 128, seed=1)
    with pytest.raises(ValueError):
        ops.pool_kv_indexed(k, v, idx.long(), 128)
    with pytest.raises(ValueError):
        ops.pool_kv_indexed(k, v, idx[:-1], 128)
    with pytest.raises(ValueError):
        ops.sparse_attention_fwd(q, k, v, None, 128, 128, q_index=idx[:10])
    with pytest.raises(RuntimeError):
        ops.pool_kv_indexed(k, v, idx.cpu(), 128)


@pytest.mark.parametrize("impl,mode,blocks", [("new_mask_type", "topk", (64, 64, 32)), ("old_mask_type", "thresholdbound", (128, 128, 32))])
def test_module_reordering_without_gather_passes(impl, mode, blocks, monkeypatch):
    """PyramidSparseAttention with the Gilbert re-ordering read and written by the layer's own kernels: the same bits
    as rearrange -> layer -> reversed_rearrange outside the warm-up steps, close to it during warm-up (dense attention
    in the original order sums over the keys in another order), and the row-gather operator is not called at all."""
    from psa_hip import ops
    from psa_hip.pyramid_sparse_attention import AttentionConfig, PyramidSparseAttention
    from psa_hip.utils.synthetic import sample_offsets

    depth, height, width, text = 4, 12, 20, 70
    L = depth * height * width + text
    cfg = AttentionConfig(width=width, height=height, depth=depth, text_length=text, use_rearrange=True, rearrange_method="Gilbert",
                          attn_impl=impl, mask_mode=mode, warmup_steps=1, block_m=blocks[0], block_n=blocks[1], tile_n=blocks[2], use_sim_mask=(impl == "old_mask_type"),
                          mask_ratios={1: (0.0, 0.4), 2: (0.4, 0.6), 4: (0.6, 0.8), 8: (0.8, 0.9), 0: (0.9, 1.0)})
    g = torch.Generator(device="cpu").manual_seed(9)
    q, k, v = (torch.randn(1, 4, L, 128, generator=g).to(torch.bfloat16).to(dev()) for _ in range(3))
    offs = (sample_offsets(1, 4, cfg.block_m, cfg.block_m // 4, 1, device=dev()),
            sample_offsets(1, 4, cfg.block_n, cfg.block_n // 4, 2, device=dev()))

    def run(fused):
        m = PyramidSparseAttention(cfg, inference_num=4, layer_num=1, model_type="cogvideo")
        m.sample_offsets = offs
        m.fuse_rearrange = fused
        return [m(q, k, v, 0) for _ in range(3)]  # step 0 is warm-up (dense), steps 1 and 2 are sparse

    ref = run(False)
    monkeypatch.setattr(ops, "gather_rows", lambda *a, **kw: (_ for _ in ()).throw(AssertionError("row gather launched")))
    got = run(True)
    assert (got[0].float() - ref[0].float()).abs().max().item() <= 2e-2
    assert torch.equal(got[1], ref[1]) and torch.equal(got[2], ref[2])


@pytest.mark.parametrize("impl,mode,blocks,sim", [("new_mask_type", "topk", (64, 64, 32), False),
                                                  ("old_mask_type", "thresholdbound", (128, 128, 32), True),
                                                  ("old_mask_type", "topk", (128, 128, 32), True)])
def test_module_layer_operator_equals_stage_by_stage(impl, mode, blocks, sim):
    """Without gradients PyramidSparseAttention runs its sparse layer through the layer operator (fused estimate + map,
    similarity cap, token index).  The result must be the same bits as the reference's sequence of separate stages
    (estimate -> transfer_attn_to_mask -> min with the similarity cap -> sparse attention) on gathered tensors."""
    from psa_hip.pyramid_sparse_attention import AttentionConfig, PyramidSparseAttention, adaptive_block_sparse_attn
    from psa_hip.utils.synthetic import sample_offsets

    depth, height, width, text = 3, 10, 24, 40
    L = depth * height * width + text
    cfg = AttentionConfig(width=width, height=height, depth=depth, text_length=text, use_rearrange=True, rearrange_method="Gilbert",
                          attn_impl=impl, mask_mode=mode, warmup_steps=0, use_sim_mask=sim, block_m=blocks[0], block_n=blocks[1],
                          tile_n=blocks[2], sim_2x_threshold=0.3, sim_4x_threshold=0.2, sim_8x_threshold=0.1, enable_logging=False,
                          mask_ratios={1: (0.0, 0.4), 2: (0.4, 0.6), 4: (0.6, 0.8), 8: (0.8, 0.9), 0: (0.9, 1.0)})
    g = torch.Generator(device="cpu").manual_seed(11)
    base = torch.randn(1, 4, 1, 128, generator=g)
    q, k, v = ((base + 0.7 * torch.randn(1, 4, L, 128, generator=g)).to(torch.bfloat16).to(dev()) for _ in range(3))
    offs = (sample_offsets(1, 4, cfg.block_m, cfg.block_m // 4, 1, device=dev()),
            sample_offsets(1, 4, cfg.block_n, cfg.block_n // 4, 2, device=dev()))
    m = PyramidSparseAttention(cfg, inference_num=4, layer_num=1, model_type="cogvideo")
    m.sample_offsets = offs
    with torch.no_grad():
        got = m(q, k, v, 0)
        q_r, k_r, v_r = m.rearranger.rearrange(q, k, v)
        out_r, _, _, cap = adaptive_block_sparse_attn(q_r, k_r, v_r, cfg, m.sparse_attention_fn, sample_offsets=offs)
        ref = m.rearranger.reversed_rearrange(out_r)
    assert torch.equal(got, ref)
    if sim:
        assert cap is not None and int((cap > 1).sum()) > 0  # the cap really acts in this case
