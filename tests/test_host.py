"""CPU-side checks: the C-ABI library loads and exports every declared symbol, configuration
validation, preset loading, the Hilbert-curve rearrangement, and the no-CPU-fallback rule."""
import ctypes
import hashlib
import json
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "pyramid-sparse-attention_amd")
LIB = os.path.join(PKG, "psa_hip", "libpsa_hip.so")


@pytest.fixture(scope="session", autouse=True)
def built_library():
    if not os.path.exists(LIB):
        import build_ext

        build_ext.build(verbose=False)
    assert os.path.exists(LIB)


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "psa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(psa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(LIB)
    syms = declared_symbols()
    assert len(syms) >= 15
    for s in syms:
        assert hasattr(lib, s), s
    from psa_hip import _lib

    assert sorted(_lib.SIGNATURES) == syms  # the Python binding covers exactly the header
    assert _lib.lib.psa_version() >= 100
    assert _lib.lib.psa_pool_elems(1, 12, 32760, 128, 128) == 12 * 32768 * 128 * 7 // 8
    assert _lib.lib.psa_pool_level_offset(1, 12, 32760, 128, 128, 4) == 12 * 32768 * 128 // 2
    assert _lib.lib.psa_pool_level_offset(1, 12, 32760, 128, 128, 3) == -1


def test_no_cpu_path():
    from psa_hip import PSAAttention, ops

    x = torch.randn(1, 1, 128, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.sparse_attention_fwd(x, x, x, None, 128, 128)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.pool_kv(x, x, 128)
    with pytest.raises(RuntimeError, match="GPU only"):
        PSAAttention()(x, x, x)


def test_psa_config_validation():
    from psa_hip import AttentionConfig, PSAConfig

    c = PSAConfig()
    assert (c.block_m, c.block_n, c.tile_n, c.mask_mode, c.attn_impl) == (128, 64, 32, "topk", "new_mask_type")
    assert list(c.mask_ratios) == [1, 2, 4, 8, 0] and c.mask_ratios[8] == (0.15, 0.35)
    with pytest.raises(ValueError, match="use_sim_mask"):
        PSAConfig(use_sim_mask=True)
    with pytest.raises(ValueError, match="block_m=128 and block_n=128"):
        PSAConfig(attn_impl="old_mask_type")
    with pytest.raises(ValueError, match="block_n in"):
        PSAConfig(block_n=16)
    PSAConfig(attn_impl="old_mask_type", block_n=128, use_sim_mask=True)
    with pytest.raises(ValueError, match="use_sim_mask"):
        AttentionConfig()  # defaults: new_mask_type + use_sim_mask=True are incompatible, as in the reference
    a = AttentionConfig(use_sim_mask=False)
    assert a.mask_ratios[1] == (0.0, 0.05) and a.warmup_steps == 12 and a.text_length == 226


def test_kernel_factories_validate():
    from psa_hip.kernels import psa_sparse_attention, psa_sparse_attention_legacy
    from psa_hip.kernels.attn_pooling_kernel import attn_with_pooling_optimized
    from psa_hip.utils import transfer_attn_to_mask

    for bad in ((64, 32, 128), (128, 64, 128), (128, 32, 64)):
        with pytest.raises(ValueError):
            psa_sparse_attention_legacy(*bad)
    with pytest.raises(ValueError):
        psa_sparse_attention(128, 32, 16)
    assert callable(psa_sparse_attention(128, 32, 32)) and callable(psa_sparse_attention_legacy(128, 32, 128, causal=True))
    x = torch.randn(1, 1, 64, 64)
    with pytest.raises(AssertionError):
        attn_with_pooling_optimized(x, x, x, False, 0.1, 3, 16)
    with pytest.raises(ValueError):
        transfer_attn_to_mask(torch.rand(1, 1, 2, 4), None)
    with pytest.raises(ValueError, match="Unknown mode"):
        transfer_attn_to_mask(torch.rand(1, 1, 2, 4), {1: (0, 1.0)}, mode="bogus")


def test_preset_loader_matches_reference_semantics():
    from psa_hip import AttentionConfig
    from psa_hip.config_loader import AttentionConfigLoader

    ld = AttentionConfigLoader()
    assert ld.list_presets("Wan2.1_1.3b") == ["baseline", "psa_balanced", "psa_topk"]
    info = ld.get_attention_config("Wan2.1_1.3b", None, [832, 480, 81])
    assert info["name"] == "psa_balanced" and info["type"] == "psa"
    p = info["params"]
    assert (p["width"], p["height"], p["depth"]) == (52, 30, 21)  # ceil(pixels / 16), ceil(frames / 4)
    assert p["attn_impl"] == "old_mask_type" and p["use_sim_mask"] is True and p["mask_mode"] == "thresholdbound"
    assert (p["block_m"], p["block_n"], p["tile_n"]) == (128, 128, 32)
    assert list(p["mask_ratios"].items()) == [(1, (0.0, 0.5)), (2, (0.5, 0.6)), (4, (0.6, 0.7)), (8, (0.7, 0.8)), (0, (0.8, 1.0))]
    assert (p["sim_2x_threshold"], p["sim_4x_threshold"], p["sim_8x_threshold"]) == (0.7, 0.65, 0.6)
    assert p["warmup_steps"] == 15 and p["text_length"] == 0 and p["rearrange_method"] == "Gilbert"
    cfg = AttentionConfig(**p)
    assert cfg.block_n == 128
    cog = ld.get_attention_config("CogVideo_5b", "psa_4steps", (720, 480, 49))["params"]
    assert cog["text_length"] == 226 and cog["mask_mode"] == "topk" and cog["use_rearrange"] is False and cog["warmup_steps"] == 0
    assert (cog["width"], cog["height"], cog["depth"]) == (45, 30, 13)
    assert ld.get_attention_config("Wan2.2_5B", "baseline", [1280, 704, 121])["type"] == "dense"
    assert ld.get_attention_config("Wan2.2_5B", None, [1280, 704, 121])["params"]["block_n"] == 32
    with pytest.raises(ValueError, match="not found in config"):
        ld.get_attention_config("nope", None, [1, 1, 1])
    with pytest.raises(ValueError, match="Preset 'x' not found"):
        ld.get_attention_config("Wan2.1_14b", "x", [1, 1, 1])
    with pytest.raises(ValueError, match="video_shape"):
        ld.get_attention_config("Wan2.1_14b", None, [1, 1])
    with pytest.raises(FileNotFoundError):
        AttentionConfigLoader("/nonexistent.yaml")


def test_gilbert_curve_golden_and_properties():
    from psa_hip.utils.gilbert3d import gilbert3d

    g = json.load(open(os.path.join(ROOT, "tests", "golden", "gilbert_golden.json")))
    for key, exp in g["full"].items():
        b = tuple(map(int, key.split("x")))
        assert [x + b[0] * (y + b[1] * z) for x, y, z in gilbert3d(*b)] == exp, key
    for key, exp in g["sha256"].items():
        b = tuple(map(int, key.split("x")))
        pts = list(gilbert3d(*b))
        order = [x + b[0] * (y + b[1] * z) for x, y, z in pts]
        assert hashlib.sha256(",".join(map(str, order)).encode()).hexdigest() == exp, key
        assert sorted(order) == list(range(b[0] * b[1] * b[2]))  # every cell exactly once
        steps = [max(abs(p[i] - q[i]) for i in range(3)) for p, q in zip(pts, pts[1:])]
        # locality: consecutive cells touch, except for a handful of length-2 steps on odd-sized boxes
        assert max(steps) <= 2 and sum(st == 2 for st in steps) <= len(steps) // 500


def test_gilbert_rearranger_round_trip_and_text_position():
    """The index vectors the row-gather kernel is driven with (pure index arithmetic, checked here with torch indexing
    on the CPU): text tokens move to the end, the two orders are inverse permutations.  The rearranger itself has no
    CPU path: a CPU tensor is an error."""
    from psa_hip.utils.rearranger import GilbertRearranger

    for text in (0, 5):
        r = GilbertRearranger(6, 4, 3, text)
        n = 72 + text
        x = torch.arange(n, dtype=torch.float32).view(1, 1, n, 1).repeat(1, 2, 1, 3)
        fwd, bwd = r._combined_index("cpu", True).long(), r._combined_index("cpu", False).long()
        q = x.index_select(2, fwd)
        if text:
            assert q[0, 0, -text:, 0].tolist() == list(range(text))  # text moved to the end
        assert sorted(q[0, 0, :, 0].tolist()) == list(range(n))
        assert torch.equal(q.index_select(2, bwd), x)
        # the same as the reference's formulation: index_select of the video part, text appended
        ref = torch.cat((x[:, :, text:].index_select(2, r.original_order2gilbert_order_cpu), x[:, :, :text]), 2)
        assert torch.equal(q, ref)
        with pytest.raises(ValueError):
            r.rearrange(x, x, x)
        with pytest.raises(ValueError):
            r.reversed_rearrange(x)


def test_psa_logger_schema_and_summary(tmp_path):
    """The sparsity log keeps the reference's files and fields (src/psa_triton/utils/psa_logger.py:179-286, 314-515);
    values may arrive as tensors and are only read when the queue is flushed."""
    from psa_hip.pyramid_sparse_attention import AttentionConfig
    from psa_hip.utils.psa_logger import PSALogger

    cfg = AttentionConfig(enable_logging=False, use_sim_mask=True, attn_impl="old_mask_type")
    with PSALogger(str(tmp_path), cfg, "wan", layer_num=2, inference_num=3, session_name="s") as lg:
        cap = torch.tensor([[[1, 2, 2, 8], [4, 4, 1, 1]]])  # 3/8 at 1x, 2/8 at 2x, 2/8 at 4x, 1/8 at 8x
        lg.log_sparsity(0, 0.0, [1.0, 1.0], 100, 1, 2, sim_mask=None, is_warmup=True)
        lg.log_sparsity(0, torch.tensor(0.9), torch.tensor([0.05, 0.15]), 100, 1, 2, sim_mask=cap, is_warmup=False)
        lg.log_sparsity(1, 0.8, [0.2, 0.2], 100, 1, -1, sim_mask=cap, is_warmup=False)
        assert not os.path.getsize(tmp_path / "s" / "sparsity.jsonl")  # nothing is read or written before the flush
    lines = [json.loads(l) for l in open(tmp_path / "s" / "sparsity.jsonl")]
    assert [l["global_step"] for l in lines] == [1, 2, 3]
    keys = {"global_step", "timestamp", "layer_idx", "sparsity", "density", "per_head_density", "sequence_length", "batch_size",
            "num_heads", "is_warmup", "use_sim_mask", "sim_mask_stats"}
    assert all(set(l) == keys for l in lines)
    assert lines[1]["sparsity"] == 0.9 and lines[1]["density"] == 0.1 and lines[1]["per_head_density"] == [0.05, 0.15]
    assert lines[1]["sim_mask_stats"] == {"pool_1x_ratio": 0.375, "pool_2x_ratio": 0.25, "pool_4x_ratio": 0.25, "pool_8x_ratio": 0.125}
    assert lines[0]["is_warmup"] and lines[0]["sim_mask_stats"]["pool_1x_ratio"] == 0.0 and lines[2]["num_heads"] == 2
    summary = open(tmp_path / "s" / "summary.txt").read()
    for needle in ("PSA Sparsity Summary - s", "Total Forward Passes: 3", "Per-Layer Statistics:", "Overall Statistics:",
                   "Non-Warmup Statistics (excluding density=1.0 steps):", "Warmup Samples (density=1.0): 1",
                   "Sim Mask Statistics (Average Pooling Distribution):", "1x Pooling (no pooling):  37.50%", "Total Sim Mask Samples:   2"):
        assert needle in summary, needle
    cfgj = json.load(open(tmp_path / "s" / "config.json"))
    assert cfgj["model_type"] == "wan" and cfgj["layer_num"] == 2 and cfgj["config"]["attn_impl"] == "old_mask_type"


def test_token_index_validator_rejects_what_is_not_a_permutation():
    """A token index that is not a permutation of 0 .. L-1 is refused on the host (the kernels clamp what they read and
    drop what they cannot store, but rows of the output would stay unwritten)."""
    import pytest
    import torch

    from psa_hip import ops

    L = 37
    good = torch.randperm(L, generator=torch.Generator().manual_seed(0)).to(torch.int32)
    ops.validate_token_index(good, L)
    for bad in (good.clone().index_fill_(0, torch.tensor([3]), L),      # past the end
                good.clone().index_fill_(0, torch.tensor([5]), -1),     # negative
                good.clone().index_fill_(0, torch.tensor([7]), int(good[8]))):  # repeated: one row never written
        with pytest.raises(ValueError):
            ops.validate_token_index(bad, L)
    with pytest.raises(ValueError):
        ops.validate_token_index(good.to(torch.int64), L)
    with pytest.raises(ValueError):
        ops.validate_token_index(good[:-1], L)
