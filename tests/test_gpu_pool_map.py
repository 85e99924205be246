"""GPU parity, through the C ABI: pooling (bit-exact bf16), level map (bit-exact integers),
list <-> dense conversion, clamp and density helpers."""
import json
import os

import numpy as np
import pytest
import torch

import psa_oracle as O
from gpu_util import dev, rnd

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden", "level_map_golden.npz")
WAN13 = {1: (0.0, 0.5), 2: (0.5, 0.6), 4: (0.6, 0.7), 8: (0.7, 0.8), 0: (0.8, 1.0)}
PSA_DEFAULT = {1: (0.0, 0.1), 2: (0.1, 0.15), 4: (0.15, 0.15), 8: (0.15, 0.35), 0: (0.35, 1.0)}


@pytest.mark.parametrize("B,H,L,D,bn", [(1, 2, 256, 128, 128), (2, 3, 1000, 64, 128), (1, 1, 77, 128, 32), (1, 2, 4097, 64, 64), (1, 1, 5, 64, 128)])
def test_pool_bit_exact(B, H, L, D, bn):
    from psa_hip import ops

    k, v = rnd(B, H, L, D, seed=1), rnd(B, H, L, D, seed=2)
    kp, vp = ops.pool_kv(k.to(dev()), v.to(dev()), bn)
    torch.cuda.synchronize()
    for src, pool in ((k, kp), (v, vp)):
        lv = ops.pool_levels(pool, B, H, L, D, bn)
        ref = O.pool_kv(src, bn)
        for l in (2, 4, 8):
            assert torch.equal(lv[l].cpu().view(torch.int16), ref[l].view(torch.int16)), (l,)


def test_pool_strided_input_needs_no_copy():
    from psa_hip import ops

    B, H, L, D = 1, 4, 300, 128
    base_k, base_v = rnd(B, L, H, D, seed=3), rnd(B, L, H, D, seed=4)
    k, v = base_k.to(dev()).transpose(1, 2), base_v.to(dev()).transpose(1, 2)  # [B,H,L,D] view of [B,L,H,D]
    kp, _ = ops.pool_kv(k, v, 128)
    ref = O.pool_kv(base_k.transpose(1, 2), 128)
    lv = ops.pool_levels(kp, B, H, L, D, 128)
    for l in (2, 4, 8):
        assert torch.equal(lv[l].cpu().view(torch.int16), ref[l].contiguous().view(torch.int16))


def test_pool_errors():
    from psa_hip import ops

    with pytest.raises(RuntimeError):
        ops.pool_kv(rnd(1, 1, 8, 64), rnd(1, 1, 8, 64), 128)  # CPU tensors: no CPU path
    with pytest.raises(ValueError):
        ops.pool_kv(rnd(1, 1, 8, 64).to(dev()), rnd(1, 1, 9, 64).to(dev()), 128)


@pytest.mark.parametrize("i", range(14))
def test_level_map_golden(i):
    from psa_hip import ops

    g = np.load(GOLD)
    c = json.loads(bytes(g["meta_json"]).decode())[i]
    mr = {int(l): (lo, hi) for l, lo, hi in c["ratios"]}
    s = torch.from_numpy(g[c["name"] + "__scores"]).to(dev())
    got = ops.level_map(s, mr, c["text_length"], c["mode"], blocksize=c["blocksize"], compute_tile=c["compute_tile"])
    assert got.dtype == torch.int32
    assert np.array_equal(got.cpu().numpy(), g[c["name"] + "__mask"])


@pytest.mark.parametrize("mode", ["topk", "thresholdbound", "topk_newtype", "thresholdbound_newtype"])
@pytest.mark.parametrize("Nk,bn,tn", [(256, 128, 32), (139, 128, 32), (1024, 32, 32), (64, 64, 16), (7, 128, 32), (700, 64, 32)])
def test_level_map_random_bit_exact(mode, Nk, bn, tn):
    from psa_hip import ops

    rng = np.random.default_rng(Nk)
    s = (rng.random((2, 3, 9, Nk), dtype=np.float32) ** 8).astype(np.float32)
    s[0, 0, 0, : Nk // 2] = s[0, 0, 0, 0]  # ties -> lower column first
    s[0, 0, 1] = 0.0
    s[0, 0, 1, Nk // 3] = 1.0  # a single spike and many exact zeros
    s[0, 0, 2] = 1.0 / Nk
    s /= s.sum(-1, keepdims=True)
    for ratios, text in ((WAN13, 0), (PSA_DEFAULT, 226)):
        ref = O.level_map(s, ratios, text, mode, blocksize=bn, compute_tile=tn)
        got = ops.level_map(torch.from_numpy(s).to(dev()), ratios, text, mode, blocksize=bn, compute_tile=tn)
        assert np.array_equal(got.cpu().numpy(), ref)
        if not mode.endswith("newtype"):
            got8 = ops.level_map(torch.from_numpy(s).to(dev()), ratios, text, mode, blocksize=bn, compute_tile=tn, map_dtype=torch.int8)
            assert got8.dtype == torch.int8 and np.array_equal(got8.cpu().numpy().astype(np.int32), ref)


def test_level_map_c2_size_properties():
    from psa_hip import ops

    g = torch.Generator().manual_seed(5)
    s = torch.softmax(torch.randn(1, 12, 256, 256, generator=g) * 4, -1)
    m = ops.level_map(s.to(dev()), WAN13, 0, "thresholdbound", blocksize=128, compute_tile=32, map_dtype=torch.int8)
    ref = O.level_map(s.numpy(), WAN13, 0, "thresholdbound", blocksize=128, compute_tile=32)
    assert np.array_equal(m.cpu().numpy().astype(np.int32), ref)
    d = ops.density(m)
    torch.cuda.synchronize()
    assert abs(float(d[-1]) - O.density(ref)) < 1e-6
    for h in range(12):
        assert abs(float(d[h]) - O.density(ref[0, h])) < 1e-6


def test_level_map_errors():
    from psa_hip import ops

    s = torch.rand(1, 1, 2, 8).to(dev())
    with pytest.raises(ValueError):
        ops.level_map(s, None)
    with pytest.raises(ValueError):
        ops.level_map(s, WAN13, mode="nope")
    with pytest.raises(ValueError):
        ops.level_map(s, {3: (0, 1.0)}, 0, "topk")


def test_map_from_list_and_min_cap():
    from psa_hip import ops

    rng = np.random.default_rng(11)
    s = rng.random((1, 2, 5, 300), dtype=np.float32) ** 4
    for mode in ("topk", "thresholdbound"):
        lst = O.level_map(s, WAN13, 0, mode + "_newtype", blocksize=128, compute_tile=32)
        dense = O.level_map(s, WAN13, 0, mode, blocksize=128, compute_tile=32)
        got = ops.map_from_list(torch.from_numpy(lst).to(dev()), 300, torch.int32)
        assert np.array_equal(got.cpu().numpy(), dense)
        assert np.array_equal(got.cpu().numpy(), O.list_to_dense(lst, 300))
    m = torch.from_numpy(dense).to(dev())
    cap = torch.from_numpy(rng.choice([1, 2, 4, 8], size=(1, 2, 300)).astype(np.int32)).to(dev())
    ops.map_min_cap(m, cap)
    assert np.array_equal(m.cpu().numpy(), np.minimum(dense, cap.cpu().numpy()[:, :, None, :]))
    dc = ops.density(m, causal=False)
    assert abs(float(dc[-1]) - O.density(m.cpu().numpy())) < 1e-6


@pytest.mark.parametrize("blocksize,tile", [(32, 32), (128, 32), (64, 32), (128, 64)])
def test_dense_map_to_index_list_bit_exact(blocksize, tile):
    from psa_hip import ops
    from psa_hip.utils import transfer_mask_to_new_type

    rng = np.random.default_rng(blocksize + tile)
    m = rng.choice([0, 1, 2, 4, 8], size=(2, 3, 9, 300), p=(0.4, 0.2, 0.15, 0.15, 0.1)).astype(np.int32)
    m[0, 0, 0] = 0
    m[0, 0, 1] = 1
    m[0, 0, 2] = 8
    for dt in (torch.int32, torch.int8):
        got = transfer_mask_to_new_type(torch.from_numpy(m).to(dt).to(dev()), blocksize, tile)
        assert got.dtype == torch.int32 and tuple(got.shape) == (2, 3, 9, 305)
        assert np.array_equal(got.cpu().numpy(), O.dense_to_list(m, blocksize, tile))
    # and back through the list import
    back = ops.map_from_list(got, 300, torch.int32).cpu().numpy()
    assert np.array_equal(back, O.list_to_dense(O.dense_to_list(m, blocksize, tile), 300))
