"""GPU parity of the sampled block-importance estimator against the oracle (fp32 scores from bf16
inputs; both accumulate in fp32, so only the summation order differs)."""
import numpy as np
import pytest
import torch

import psa_oracle as O
from gpu_util import dev, rnd

pytestmark = pytest.mark.gpu
RTOL = 2e-4  # fp32 scores; accumulation-order differences only


@pytest.mark.parametrize(
    "B,Hq,Hkv,L,D,bm,bn",
    [(1, 2, 2, 1024, 128, 128, 128), (2, 2, 1, 1000, 64, 128, 128), (1, 2, 2, 4096, 64, 64, 64), (1, 1, 1, 520, 128, 128, 32),
     (1, 3, 3, 1111, 128, 128, 64), (1, 1, 1, 64, 64, 64, 64)],
)
def test_estimate_matches_oracle(B, Hq, Hkv, L, D, bm, bn):
    from psa_hip import ops
    from psa_hip.utils.synthetic import sample_offsets

    q, k = rnd(B, Hq, L, D, seed=1), rnd(B, Hkv, L, D, seed=2)
    km, kn = bm // 4, bn // 4
    oq, ok = sample_offsets(B, Hq, bm, km, 5), sample_offsets(B, Hkv, bn, kn, 6)
    got = ops.estimate_sampled(q.to(dev()), k.to(dev()), oq.to(dev()), ok.to(dev()), bm, bn, km, kn)
    ref = O.estimate_sampled(q, k, bm, bn, oq, ok)
    assert got.shape == ref.shape and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), ref.numpy(), rtol=RTOL, atol=1e-9)


def test_estimate_presampled_full_output_like_reference_api():
    from psa_hip import ops

    sq, sk = rnd(1, 2, 96, 128, seed=3), rnd(1, 2, 40, 128, seed=4)  # 96 -> 128 rows (4 groups of 32), 40 -> 64 keys (8 groups of 8)
    ref = O.estimate_from_sampled(sq, sk, 128 ** -0.5, 32, 8)
    got = ops.estimate_sampled(sq.to(dev()), sk.to(dev()), None, None, 32, 8, 32, 8, out_rows=4, out_cols=8)
    np.testing.assert_allclose(got.cpu().numpy(), ref.numpy(), rtol=RTOL, atol=1e-9)
    np.testing.assert_allclose(got.sum(-1).cpu().numpy(), 1.0, rtol=1e-5)


def test_estimate_then_level_map_matches_oracle_map():
    """The level map computed on the GPU from the GPU's own fp32 scores equals the oracle's map from
    those same scores bit for bit (the map contract is defined on identical fp32 scores)."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import make_qkv, sample_offsets

    q, k, _ = make_qkv(1, 2, 2, (4, 16, 32), 128, seed=7)
    oq, ok = sample_offsets(1, 2, 128, 32, 8), sample_offsets(1, 2, 128, 32, 9)
    s = ops.estimate_sampled(q.to(dev()), k.to(dev()), oq.to(dev()), ok.to(dev()), 128, 128, 32, 32)
    ratios = {1: (0.0, 0.5), 2: (0.5, 0.6), 4: (0.6, 0.7), 8: (0.7, 0.8), 0: (0.8, 1.0)}
    m = ops.level_map(s, ratios, 0, "thresholdbound", blocksize=128, compute_tile=32)
    ref = O.level_map(s.cpu().numpy(), ratios, 0, "thresholdbound", blocksize=128, compute_tile=32)
    assert np.array_equal(m.cpu().numpy(), ref)


@pytest.mark.parametrize("mode", ["topk", "thresholdbound"])
@pytest.mark.parametrize(
    "B,Hq,Hkv,L,D,bm,bn,text",
    [(1, 2, 2, 4096, 128, 128, 128, 0), (2, 2, 1, 1000, 64, 128, 128, 226), (1, 2, 2, 4096, 64, 64, 64, 0), (1, 1, 1, 2000, 128, 128, 32, 0),
     (1, 3, 3, 1111, 128, 128, 64, 100), (1, 1, 1, 64, 64, 64, 64, 0), (1, 2, 2, 33000, 128, 128, 128, 0)],
)
def test_fused_estimate_and_map_equals_the_two_calls(mode, B, Hq, Hkv, L, D, bm, bn, text):
    """psa_estimate_sampled_map must return exactly the scores of psa_estimate_sampled and exactly the map
    psa_level_map makes of them (int8 and int32), with and without the scores output."""
    from psa_hip import ops
    from psa_hip.utils.synthetic import sample_offsets

    q, k = rnd(B, Hq, L, D, seed=11).to(dev()), rnd(B, Hkv, L, D, seed=12).to(dev())
    km, kn = bm // 4, bn // 4
    oq, ok = sample_offsets(B, Hq, bm, km, 5).to(dev()), sample_offsets(B, Hkv, bn, kn, 6).to(dev())
    ratios = {1: (0.0, 0.3), 2: (0.3, 0.45), 4: (0.45, 0.6), 8: (0.6, 0.8), 0: (0.8, 1.0)}
    scores = ops.estimate_sampled(q, k, oq, ok, bm, bn, km, kn)
    for dt in (torch.int8, torch.int32):
        ref = ops.level_map(scores, ratios, text, mode, blocksize=bn, compute_tile=min(32, bn), map_dtype=dt)
        s2, m2 = ops.estimate_sampled_map(q, k, oq, ok, bm, bn, km, kn, ratios, text, mode, compute_tile=min(32, bn), map_dtype=dt,
                                          return_scores=True)
        m3 = ops.estimate_sampled_map(q, k, oq, ok, bm, bn, km, kn, ratios, text, mode, compute_tile=min(32, bn), map_dtype=dt)
        assert torch.equal(s2, scores)
        assert m2.dtype == dt and torch.equal(m2, ref) and torch.equal(m3, ref)


def test_fused_estimate_and_map_errors():
    from psa_hip import ops

    q, k = rnd(1, 1, 256, 64, seed=1).to(dev()), rnd(1, 1, 256, 64, seed=2).to(dev())
    with pytest.raises(ValueError):
        ops.estimate_sampled_map(q, k, None, None, 64, 64, 16, 16, None, 0, "topk")
    with pytest.raises(ValueError):
        ops.estimate_sampled_map(q, k, None, None, 64, 64, 16, 16, {1: (0.0, 1.0)}, 0, "topk_newtype")
    with pytest.raises(ValueError):
        ops.estimate_sampled_map(q, k, None, None, 64, 64, 16, 16, {1: (0.0, 1.0)}, 0, "nonsense")


def test_fused_estimate_and_map_very_wide_rows_fall_back_to_two_kernels():
    """6000 key blocks: the row of scores and the level-map scratch exceed LDS together; same results by two kernels."""
    from psa_hip import ops

    L, bm, bn = 192000, 128, 32
    q, k = rnd(1, 1, L, 64, seed=21).to(dev()), rnd(1, 1, L, 64, seed=22).to(dev())
    ratios = {1: (0.0, 0.05), 2: (0.05, 0.1), 4: (0.1, 0.2), 8: (0.2, 0.4), 0: (0.4, 1.0)}
    scores = ops.estimate_sampled(q, k, None, None, bm, bn, 32, 8)
    ref = ops.level_map(scores, ratios, 0, "thresholdbound", blocksize=bn, compute_tile=32, map_dtype=torch.int8)
    got = ops.estimate_sampled_map(q, k, None, None, bm, bn, 32, 8, ratios, 0, "thresholdbound", compute_tile=32, map_dtype=torch.int8)
    assert got.shape == (1, 1, 1500, 6000) and torch.equal(got, ref)


def test_sampling_offsets_drawn_on_the_device():
    """psa_draw_sample_offsets: per (b, h) `keep` distinct offsets inside the block, reproducible from the seed, different
    between heads and seeds, every offset about equally likely (the reference draws rand -> topk: a uniform subset)."""
    from psa_hip import ops

    B, Hq, Hkv = 2, 48, 12
    oq, ok = ops.draw_sample_offsets(B, Hq, Hkv, 128, 32, 64, 16, dev(), seed=1234)
    assert oq.shape == (B, Hq, 32) and ok.shape == (B, Hkv, 16) and oq.dtype == torch.int32
    for o, block, keep in ((oq, 128, 32), (ok, 64, 16)):
        o = o.cpu().numpy().reshape(-1, keep)
        assert o.min() >= 0 and o.max() < block
        assert all(len(set(r)) == keep for r in o)          # distinct
        assert len({tuple(r) for r in o}) == o.shape[0]      # heads differ
    oq2, ok2 = ops.draw_sample_offsets(B, Hq, Hkv, 128, 32, 64, 16, dev(), seed=1234)
    assert torch.equal(oq, oq2) and torch.equal(ok, ok2)
    oq3, _ = ops.draw_sample_offsets(B, Hq, Hkv, 128, 32, 64, 16, dev(), seed=1235)
    assert not torch.equal(oq, oq3)
    # uniformity: 4096 heads x 32 of 128 -> every offset expected 1024 times (sd ~ 28)
    big, _ = ops.draw_sample_offsets(64, 64, 1, 128, 32, 64, 16, dev(), seed=7)
    cnt = np.bincount(big.cpu().numpy().reshape(-1), minlength=128)
    assert cnt.sum() == 4096 * 32 and abs(cnt - 1024).max() < 6 * 28
    # the first offset of a head (the largest random number) is uniform too
    first = np.bincount(big.cpu().numpy().reshape(-1, 32)[:, 0], minlength=128)
    assert abs(first - 32).max() < 6 * 6
    # unseeded draws differ from call to call
    a, _ = ops.draw_sample_offsets(1, 4, 4, 128, 32, 128, 32, dev())
    b, _ = ops.draw_sample_offsets(1, 4, 4, 128, 32, 128, 32, dev())
    assert not torch.equal(a, b)
