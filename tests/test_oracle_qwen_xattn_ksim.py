"""Pins three oracle functions that the GPU parity tests of the causal (Qwen2.5-VL) path and of the
key-similarity cap are measured against:

  O.level_map_qwen     rows worked by hand from the source (both modes, causal on/off, trailing text
                       rows/columns, later-level-overwrites, lower = max(lo, previous hi)) and an
                       independent row-by-row restatement that uses the library calls the reference
                       uses (torch.sort / cumsum / sum on one row at a time) on tie-free rows;
  O.estimate_xattn     brute-force loops over (query group, key group, stride step) in float64, with
                       zero-padded tails (L % chunk != 0), stride 8, non-causal, GQA and Lk > Lq;
  O.k_similarity*      brute-force loops over explicit token pairs (0,1), (0,3), (0,7) of each group of
                       2 / 4 / 8 on random keys with a ragged tail, cross-checked with
                       torch.nn.functional.cosine_similarity on the slices ::2 / 1::2, 0::4 / 3::4, 0::8 / 7::8.

The reference's own files are not imported here: the rules are restated from
qwen2.5-vl-example/src/attention/PSA_casual/PyramidAdaptiveBlockSparseAttn.py:84-168,
qwen2.5-vl-example/src/attention/PSA_casual/kernels/block_importance_kernels.py:6-192,255-323,
qwen2.5-vl-example/src/attention/PSA_casual/utils/block_importance.py:282-462,545-562 and
src/psa_triton/kernels/calc_ksim_kernel.py:66-144, src/psa_triton/attention.py:139-165.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O

QWEN = {1: (0.0, 0.7), 2: (0.7, 0.8), 4: (0.8, 0.9), 8: (0.9, 0.9), 0: (0.9, 1.0)}


# ------------------------------------------------------------------------------------ Qwen level map
def _from_sorted(S, rows):
    """rows: {row index: (column permutation, descending weights)} -> scores [1,1,S,S]; sorted position p of the
    row is column perm[p].  Rows that are not listed get distinct positive weights below the diagonal."""
    s = np.zeros((1, 1, S, S), np.float32)
    for i in range(S):
        s[0, 0, i, : i + 1] = np.arange(i + 1, 0, -1, dtype=np.float32) / 64
    for i, (perm, w) in rows.items():
        s[0, 0, i] = 0
        s[0, 0, i, np.asarray(perm)] = np.asarray(w, np.float32)
    return s


def test_qwen_hand_topk_causal():
    # S = 8, ratios {1:(0,.25), 2:(.25,.5), 4:(.5,.75), 8:(.75,.9), 0:(.9,1)}, valid length of row i = i + 1.
    # Row 7: starts/ends floor(8*r): level 1 [0,2), 2 [2,4), 4 [4,6), 8 [6,7) (floor(7.2) = 7), 0 [7,8).
    #   sorted columns 5,2,7,0,3,6,1,4 -> col5 1, col2 1, col7 2, col0 2, col3 4, col6 4, col1 8, col4 0;
    #   then diagonal (col 7) := 1 and column 0 := 1  ->  [1,8,1,4,0,1,4,1]
    # Row 3 (valid 4): level 1 [0,1), 2 [1,2), 4 [2,3), 8 [3, floor(3.6)=3) empty, 0 [3,4).  Scores 3,9,5,7 in
    #   columns 0..3 (zeros above the diagonal sort last and lie beyond every interval): col1 1, col3 2, col2 4, col0 0;
    #   diagonal (col 3) := 1, column 0 := 1  ->  [1,1,4,1,0,0,0,0]
    ratios = {1: (0.0, 0.25), 2: (0.25, 0.5), 4: (0.5, 0.75), 8: (0.75, 0.9), 0: (0.9, 1.0)}
    s = _from_sorted(8, {7: ([5, 2, 7, 0, 3, 6, 1, 4], [8, 7, 6, 5, 4, 3, 2, 1]), 3: ([1, 3, 2, 0], [9, 7, 5, 3])})
    m = O.level_map_qwen(s, ratios, text_length=0, mode="topk", block_size=128, causal=True)
    assert m[0, 0, 7].tolist() == [1, 8, 1, 4, 0, 1, 4, 1]
    assert m[0, 0, 3].tolist() == [1, 1, 4, 1, 0, 0, 0, 0]
    assert m[0, 0, 0].tolist() == [1, 0, 0, 0, 0, 0, 0, 0]


def test_qwen_hand_topk_noncausal_overwrite_and_text():
    # Non-causal: every row has valid length 8.  Ratios in dict order {2:(0,.5), 1:(0,.25), 0:(.5,1)}: level 2 on
    # sorted positions [0,4), then level 1 OVERWRITES [0,2), level 0 on [4,8).  text_length 200, block 128 ->
    # min(ceil(200/128), 8) = 2 special blocks: last two columns and last two rows := 1.  No triangle is cleared.
    # Row 2 scores by column [1,8,7,6,5,4,3,2] -> sorted columns 1,2,3,4,5,6,7,0: col1 1, col2 1, col3 2, col4 2,
    #   cols 5,6,7,0 -> 0; columns 6,7 := 1; diagonal (col 2) := 1; column 0 := 1  ->  [1,1,1,2,2,0,1,1]
    ratios = {2: (0.0, 0.5), 1: (0.0, 0.25), 0: (0.5, 1.0)}
    s = np.tile(np.array([1, 8, 7, 6, 5, 4, 3, 2], np.float32), (1, 1, 8, 1))
    m = O.level_map_qwen(s, ratios, text_length=200, mode="topk", block_size=128, causal=False)
    assert m[0, 0, 2].tolist() == [1, 1, 1, 2, 2, 0, 1, 1]
    assert m[0, 0, 5].tolist() == [1, 1, 1, 2, 2, 1, 1, 1]  # its diagonal is column 5
    assert m[0, 0, 6].tolist() == [1] * 8 and m[0, 0, 7].tolist() == [1] * 8


def test_qwen_hand_energybound_lower_is_max_of_lo_and_previous_hi():
    # Sorted weights [35,13,8,4,2,1,.5,.5]/64 (sum 1, every prefix sum exact): r = .546875,.75,.875,.9375,.96875,
    # .984375,.9921875,1.  Ratios in dict order {1:(0,.6), 2:(.5,.9), 4:(.9,.95), 8:(.95,.99), 0:(.99,1)}:
    #   level 1: 0 < r <= .6 -> position 0;   level 2: lower = max(.5, previous hi .6) = .6 < r <= .9 -> 1, 2
    #   (with lower = lo = .5 it would also take position 0 and overwrite the 1);  level 4: .9 < r <= .95 -> 3;
    #   level 8: .95 < r <= .99 -> 4, 5;  level 0: .99 < r <= 1 -> 6, 7 (the tie .5/.5: lower column first, same level).
    # Columns by sorted position 4,1,6,3,0,7,2,5; non-causal, row 2: col4 1, col1 2, col6 2, col3 4, col0 8, col7 8,
    #   col2 0, col5 0; diagonal (col 2) := 1, column 0 := 1  ->  [1,2,1,4,1,0,2,8]
    ratios = {1: (0.0, 0.6), 2: (0.5, 0.9), 4: (0.9, 0.95), 8: (0.95, 0.99), 0: (0.99, 1.0)}
    w = np.array([35, 13, 8, 4, 2, 1, 0.5, 0.5], np.float32) / 64
    row = np.zeros(8, np.float32)
    row[[4, 1, 6, 3, 0, 7, 2, 5]] = w
    s = np.tile(row, (1, 1, 8, 1))
    m = O.level_map_qwen(s, ratios, text_length=0, mode="energybound", block_size=128, causal=False)
    assert m[0, 0, 2].tolist() == [1, 2, 1, 4, 1, 0, 2, 8]
    assert m[0, 0, 5].tolist() == [1, 2, 0, 4, 1, 1, 2, 8]  # diagonal at column 5, column 2 keeps its 0


def test_qwen_hand_energybound_causal_text_rows_and_columns():
    # S = 6, block 128, text_length 130 -> 2 special blocks: columns 4,5 := 1 and rows 4,5 := 1, THEN the strict upper
    # triangle := 0, the diagonal := 1, column 0 := 1.
    # Row 3: scores [1,4,3,8]/16 in columns 0..3 -> sorted col3 (.5), col1 (.25), col2 (.1875), col0 (.0625), then the
    #   zero columns 4,5.  r = .5, .75, .9375, 1, 1, 1 with the Qwen ratios {1:(0,.7), 2:(.7,.8), 4:(.8,.9), 8:(.9,.9), 0:(.9,1)}:
    #   position 0 -> 1 (col3), position 1 (.7 < .75 <= .8) -> 2 (col1), position 2 (.9375 > .9) -> 0, the rest 0.
    #   text columns 4,5 := 1, cleared again by the triangle; diagonal (col 3) := 1; column 0 := 1  ->  [1,2,0,1,0,0]
    # Row 4 (a text row): all 1, column 5 cleared by the triangle -> [1,1,1,1,1,0];  row 5: all 1.
    s = _from_sorted(6, {3: ([3, 1, 2, 0], [8 / 16, 4 / 16, 3 / 16, 1 / 16])})
    m = O.level_map_qwen(s, QWEN, text_length=130, mode="energybound", block_size=128, causal=True)
    assert m[0, 0, 3].tolist() == [1, 2, 0, 1, 0, 0]
    assert m[0, 0, 4].tolist() == [1, 1, 1, 1, 1, 0]
    assert m[0, 0, 5].tolist() == [1, 1, 1, 1, 1, 1]


def test_qwen_hand_energybound_zero_row_clamps_total():
    # An all-zero row: the total is clamped to 1e-10, every ratio is 0 and no interval (lower < r) takes it: the row
    # keeps 0 apart from the diagonal and column 0.
    s = np.zeros((1, 1, 4, 4), np.float32)
    m = O.level_map_qwen(s, QWEN, text_length=0, mode="energybound", block_size=128, causal=False)
    assert m[0, 0].tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [1, 0, 1, 0], [1, 0, 0, 1]]


def _qwen_rows_restated(scores, ratios, text_length, mode, block_size, causal):
    """The reference's rules, one row at a time, with the library calls it uses (torch.sort, cumsum, sum,
    tensor-vs-Python-scalar arithmetic and comparisons) applied to a single 1-D row."""
    B, H, S, _ = scores.shape
    out = np.zeros((B, H, S, S), np.int32)
    for b in range(B):
        for h in range(H):
            for i in range(S):
                row = torch.from_numpy(scores[b, h, i].copy())
                w, idx = torch.sort(row, descending=True, stable=True)
                lv_sorted = [0] * S
                if mode == "topk":
                    vl = torch.tensor([i + 1 if causal else S]).float()
                    for lv, (lo, hi) in ratios.items():
                        a = min(int((vl * lo).long()), S)
                        e = min(int((vl * hi).long()), S)
                        for p in range(a, e):
                            lv_sorted[p] = lv
                else:
                    total = row.sum().clamp(min=1e-10)
                    r = torch.cumsum(w, 0) / total
                    prev = 0.0
                    for lv, (lo, hi) in ratios.items():
                        lower = max(lo, prev)
                        prev = hi
                        sel = (r > lower) & (r <= hi)
                        for p in range(S):
                            if bool(sel[p]):
                                lv_sorted[p] = lv
                for p in range(S):
                    out[b, h, i, int(idx[p])] = lv_sorted[p]
    nb = min(math.ceil(text_length / block_size) if text_length > 0 else 0, S)
    for b in range(B):
        for h in range(H):
            m = out[b, h]
            if nb:
                for i in range(S):
                    for j in range(S):
                        if j >= S - nb or i >= S - nb:
                            m[i, j] = 1
            if causal:
                for i in range(S):
                    for j in range(i + 1, S):
                        m[i, j] = 0
            for i in range(S):
                m[i, i] = 1
                m[i, 0] = 1
    return out


def _dyadic_scores(rng, B, H, S, causal):
    """Tie-free rows of multiples of 2^-12 whose every partial sum is exact in fp32, so the row total does not
    depend on the order of summation; above the diagonal 0 when causal (what the causal estimator writes)."""
    s = np.zeros((B, H, S, S), np.float32)
    for b in range(B):
        for h in range(H):
            for i in range(S):
                n = i + 1 if causal else S
                k = rng.choice(np.arange(1, 4096), size=n, replace=False)
                s[b, h, i, :n] = k.astype(np.float32) / 4096
    return s


@pytest.mark.parametrize("mode", ["topk", "energybound"])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("text", [0, 200])
def test_qwen_matches_rowwise_restatement_dyadic(mode, causal, text):
    rng = np.random.default_rng(7 + 2 * causal + text)
    ratio_sets = [QWEN, {1: (0.0, 0.3), 2: (0.2, 0.55), 4: (0.55, 0.7), 8: (0.65, 0.9), 0: (0.9, 1.0)},
                  {2: (0.0, 0.5), 1: (0.0, 0.2), 8: (0.5, 0.8), 0: (0.8, 1.0)}]
    for S in (1, 5, 23):
        s = _dyadic_scores(rng, 1, 2, S, causal)
        for ratios in ratio_sets:
            got = O.level_map_qwen(s, ratios, text_length=text, mode=mode, block_size=128, causal=causal)
            ref = _qwen_rows_restated(s, ratios, text, mode, 128, causal)
            assert np.array_equal(got, ref), (mode, causal, text, S, ratios)


@pytest.mark.parametrize("mode", ["topk", "energybound"])
def test_qwen_matches_rowwise_restatement_softmax_rows(mode):
    """Rows of a causal softmax (generic floats).  The oracle's row total is the last sequential prefix sum, the
    reference's torch.sum of the unsorted row: they may differ in the last place, which could only matter for a
    ratio within one rounding of a bound - none does for these seeds."""
    g = torch.Generator().manual_seed(3)
    S = 40
    z = torch.randn(1, 3, S, S, generator=g) * 2.5
    z = z.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    s = torch.softmax(z, -1).numpy().astype(np.float32)
    for text in (0, 300):
        got = O.level_map_qwen(s, QWEN, text_length=text, mode=mode, block_size=128, causal=True)
        assert np.array_equal(got, _qwen_rows_restated(s, QWEN, text, mode, 128, True))


# ------------------------------------------------------------------------------------ xattn estimate
def _xattn_brute(q, k, block, S, causal, chunk):
    """Plain loops in float64.  q [B,Hq,Lq,D], k [B,Hkv,Lk,D] numpy."""
    B, Hq, Lq, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    rep = Hq // Hkv
    Lqp, Lkp = -(-Lq // chunk) * chunk, -(-Lk // chunk) * chunk
    Mr, Nr, rb = Lqp // S, Lkp // S, block // S
    off = Nr - Mr
    real_rows = -(-Lq // S)
    est = np.zeros((B, Hq, Mr // rb, Nr // rb))
    for b in range(B):
        for h in range(Hq):
            qp = np.zeros((Lqp, D))
            qp[:Lq] = q[b, h]
            kp = np.zeros((Lkp, D))
            kp[:Lk] = k[b, h // rep]
            for m in range(Mr):
                if m >= real_rows:
                    continue  # rows made of padding only contribute nothing
                z = np.full(Nr, -np.inf)
                for n in range(Nr):
                    if causal and n > m + off:
                        continue
                    a = 0.0
                    for i in range(S):
                        a += float(np.dot(qp[m * S + S - 1 - i], kp[n * S + i]))
                    z[n] = a / (math.sqrt(D) * S)  # zero-padded keys keep logit 0: they are NOT masked
                p = np.exp(z - z.max())
                p /= p.sum()
                for n in range(Nr):
                    est[b, h, m // rb, n // rb] += p[n]
    return est[:, :, : -(-Lq // block), : -(-Lk // block)]


@pytest.mark.parametrize(
    "B,Hq,Hkv,Lq,Lk,D,block,S,chunk,causal",
    [
        (1, 2, 1, 40, 40, 8, 16, 8, 32, True),     # ragged tail (zero-padded to 64), stride 8, GQA
        (1, 1, 1, 24, 24, 4, 8, 4, 16, False),     # non-causal, padded keys visible to every row at logit 0
        (2, 4, 2, 44, 44, 8, 16, 8, 32, False),    # non-causal, GQA, L % stride != 0 (a half-padded key group)
        (1, 2, 2, 16, 32, 4, 8, 4, 16, True),      # Lk > Lq: causal offset Nr - Mr
        (1, 1, 1, 32, 32, 4, 8, 2, 32, True),      # the earlier tiny case: no padding, stride 2
    ],
)
def test_xattn_brute_force(B, Hq, Hkv, Lq, Lk, D, block, S, chunk, causal):
    g = torch.Generator().manual_seed(Lq * 7 + S)
    q = torch.randn(B, Hq, Lq, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, Hkv, Lk, D, generator=g, dtype=torch.float64)
    got = O.estimate_xattn(q, k, block_size=block, stride=S, causal=causal, chunk_size=chunk, dtype=torch.float64)
    ref = _xattn_brute(q.numpy(), k.numpy(), block, S, causal, chunk)
    assert tuple(got.shape) == ref.shape
    np.testing.assert_allclose(got.double().numpy(), ref, rtol=1e-6, atol=1e-9)
    # every real query group distributes probability 1: a block row sums to its number of real groups
    rb = block // S
    rows = np.minimum(np.arange(1, ref.shape[2] + 1) * rb, -(-Lq // S)) - np.arange(ref.shape[2]) * rb
    full = ref.shape[3] == -(-(-(-Lk // chunk) * chunk) // block)  # no key block cropped away
    if full:
        np.testing.assert_allclose(got.double().numpy().sum(-1), np.broadcast_to(rows, got.shape[:3]), rtol=1e-6)


def test_xattn_padded_keys_take_mass_when_visible():
    """Non-causal, L = 24 padded to 32 with stride 4: the two all-zero key groups have logit 0 and take part in the
    softmax.  With q = 0 every logit is 0, so each of the 8 groups gets 1/8 and the 2 padded ones fall into block 3,
    which is cropped away: the three real blocks hold 2/8 each per query group."""
    q = torch.zeros(1, 1, 24, 4)
    k = torch.randn(1, 1, 24, 4, generator=torch.Generator().manual_seed(1))
    est = O.estimate_xattn(q, k, block_size=8, stride=4, causal=False, chunk_size=16)
    assert tuple(est.shape) == (1, 1, 3, 3)
    np.testing.assert_allclose(est.numpy(), np.full((1, 1, 3, 3), 2 * 2 / 8), rtol=1e-6)


# ------------------------------------------------------------------------------------ key similarity
def _ksim_brute(k, block_n):
    """Explicit pair loops: group of l tokens -> pair (first, last) = (g*l, g*l + l - 1)."""
    B, H, L, D = k.shape
    nb = -(-L // block_n)
    out = {l: np.zeros((B, H, nb)) for l in (2, 4, 8)}
    for b in range(B):
        for h in range(H):
            for j in range(nb):
                for l in (2, 4, 8):
                    acc = 0.0
                    for g in range(block_n // l):
                        ia, ib = j * block_n + g * l, j * block_n + g * l + l - 1
                        a = k[b, h, min(ia, L - 1)].astype(np.float64)  # tokens past the end replicate the last one
                        c = k[b, h, min(ib, L - 1)].astype(np.float64)
                        acc += float(a @ c) / (math.sqrt(float(a @ a) + 1e-12) * math.sqrt(float(c @ c) + 1e-12) + 1e-6)
                    out[l][b, h, j] = acc / (block_n // l)
    return out[2], out[4], out[8]


@pytest.mark.parametrize("L,block_n", [(64, 32), (100, 32), (200, 64), (130, 128)])
def test_ksim_pair_geometry_brute_force(L, block_n):
    g = torch.Generator().manual_seed(L)
    # distinct rows inside every group, correlated enough that the three similarities differ clearly
    base = torch.randn(1, 2, L, 16, generator=g)
    k = base + 0.7 * torch.roll(base, 1, 2) + 0.4 * torch.roll(base, 3, 2)
    s2, s4, s8 = O.k_similarity_scores(k, block_n)
    b2, b4, b8 = _ksim_brute(k.numpy(), block_n)
    for got, ref in ((s2, b2), (s4, b4), (s8, b8)):
        np.testing.assert_allclose(got.double().numpy(), ref, rtol=2e-5, atol=2e-6)
    # the three pair geometries really differ on this input (so a wrong pair choice cannot pass)
    assert np.abs(b2 - b4).max() > 0.05 and np.abs(b4 - b8).max() > 0.05 and np.abs(b2 - b8).max() > 0.05
    wrong4 = _wrong_pairs(k.numpy(), block_n, 4, 1)  # (0,1) of each group of 4 instead of (0,3)
    assert np.abs(wrong4 - b4).max() > 0.05


def _wrong_pairs(k, block_n, l, second):
    B, H, L, D = k.shape
    nb = -(-L // block_n)
    out = np.zeros((B, H, nb))
    for b in range(B):
        for h in range(H):
            for j in range(nb):
                acc = 0.0
                for g in range(block_n // l):
                    a = k[b, h, min(j * block_n + g * l, L - 1)].astype(np.float64)
                    c = k[b, h, min(j * block_n + g * l + second, L - 1)].astype(np.float64)
                    acc += float(a @ c) / (math.sqrt(float(a @ a)) * math.sqrt(float(c @ c)))
                out[b, h, j] = acc / (block_n // l)
    return out


def test_ksim_matches_library_cosine_on_reference_slices():
    """The slicing of the reference's pure-torch fall-back (::2 vs 1::2, 0::4 vs 3::4, 0::8 vs 7::8) with the library's
    cosine similarity; the two formulas differ only in their epsilons (well below 1e-5 for rows of norm ~ 4)."""
    g = torch.Generator().manual_seed(11)
    k = torch.randn(2, 3, 256, 16, generator=g)
    k = k + 0.8 * torch.roll(k, 1, 2)
    s2, s4, s8 = O.k_similarity_scores(k, 64)
    kc = k.view(2, 3, 4, 64, 16)
    for got, (a, b) in ((s2, (kc[..., ::2, :], kc[..., 1::2, :])), (s4, (kc[..., 0::4, :], kc[..., 3::4, :])),
                        (s8, (kc[..., 0::8, :], kc[..., 7::8, :]))):
        np.testing.assert_allclose(got.numpy(), F.cosine_similarity(a, b, dim=-1).mean(-1).numpy(), rtol=0, atol=2e-5)


def test_ksim_cap_is_the_largest_passing_level():
    """cap = max(1, 2*[s2 > t2], 4*[s4 > t4], 8*[s8 > t8]) with strict comparisons: a later, larger level wins
    whatever the smaller ones say."""
    g = torch.Generator().manual_seed(5)
    k = torch.randn(1, 2, 512, 16, generator=g)
    k = k + 0.9 * torch.roll(k, 1, 2)
    s2, s4, s8 = (t.numpy() for t in O.k_similarity_scores(k, 64))
    t2, t4, t8 = float(np.median(s2)), float(np.median(s4)), float(np.median(s8))
    cap = O.k_similarity(k, 64, t2, t4, t8).numpy()
    want = np.maximum(1, np.maximum(2 * (s2 > t2), np.maximum(4 * (s4 > t4), 8 * (s8 > t8))))
    assert np.array_equal(cap, want)
    assert set(np.unique(cap)) >= {1, 8}
    # strictness: a threshold equal to the similarity does not pass
    one = O.k_similarity(k[:, :1, :64], 64, float(s2[0, 0, 0]), 2.0, 2.0)
    assert one.view(-1).tolist() == [1]
