"""Pins oracle.level_map*: golden vectors written by the reference's own pure-torch
function (tests/golden/make_level_map_golden.py), rows worked by hand from the
source, and invariants."""
import json
import os

import numpy as np
import pytest

import psa_oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden", "level_map_golden.npz")


def _cases():
    g = np.load(GOLD)
    meta = json.loads(bytes(g["meta_json"]).decode())
    return g, meta


@pytest.mark.parametrize("i", range(14))
def test_golden(i):
    g, meta = _cases()
    c = meta[i]
    mr = {int(l): (lo, hi) for l, lo, hi in c["ratios"]}
    got = O.level_map(g[c["name"] + "__scores"], mr, c["text_length"], c["mode"], blocksize=c["blocksize"], compute_tile=c["compute_tile"])
    assert np.array_equal(got, g[c["name"] + "__mask"])


def _row(w):
    return np.asarray(w, dtype=np.float32).reshape(1, 1, 1, -1)


WAN14 = {1: (0.0, 0.4), 2: (0.4, 0.5), 4: (0.5, 0.6), 8: (0.6, 0.8), 0: (0.8, 1.0)}


def test_hand_thresholdbound_d1():
    w = _row([16, 12, 8, 8, 6, 4, 4, 3, 2, 1]) / 64
    m = O.level_map(w, WAN14, 0, "thresholdbound", blocksize=128, compute_tile=32)
    assert m.reshape(-1).tolist() == [1, 1, 2, 4, 8, 8, 0, 0, 0, 0]
    assert abs(O.density(m) - 0.30) < 1e-12
    r2 = dict(WAN14)
    r2[8] = (0.6, 0.7)
    m2 = O.level_map(w, r2, 0, "thresholdbound", blocksize=128, compute_tile=32)
    assert m2.reshape(-1).tolist() == [1, 1, 2, 4, 8, 8, 0, 0, 0, 0]


def test_hand_thresholdbound_round_down_at_boundary():
    w = _row([20, 16, 12, 8, 8]) / 64
    ratios = {1: (0, 0.4), 2: (0.4, 0.5), 4: (0.5, 0.5), 8: (0.5, 0.9), 0: (0.9, 1)}
    m = O.level_map(w, ratios, 0, "thresholdbound", blocksize=128, compute_tile=32)
    assert m.reshape(-1).tolist() == [1, 1, 8, 8, 0]


def test_hand_text_columns_and_permutation():
    w = np.array([16, 12, 8, 8, 6, 4, 4, 3, 2, 1], dtype=np.float32) / 64
    perm = np.array([3, 7, 0, 9, 1, 5, 2, 8, 6, 4])
    s = np.zeros(10, np.float32)
    s[perm] = w  # sorted position p lives at column perm[p]; the tie 8,8 -> lower column first
    m = O.level_map(_row(s), WAN14, 0, "thresholdbound", blocksize=128, compute_tile=32).reshape(-1)
    exp_sorted = [1, 1, 2, 4, 8, 8, 0, 0, 0, 0]
    order = np.argsort(-s, kind="stable")
    assert [int(m[c]) for c in order] == exp_sorted
    mt = O.level_map(_row(s), WAN14, 226, "thresholdbound", blocksize=128, compute_tile=32).reshape(-1)
    assert mt[-2:].tolist() == [1, 1] and np.array_equal(mt[:-2], m[:-2])


PSA_DEFAULT = {1: (0.0, 0.1), 2: (0.1, 0.15), 4: (0.15, 0.15), 8: (0.15, 0.35), 0: (0.35, 1.0)}


def test_hand_topk_d2_and_list_d3():
    w = _row(np.arange(10, 0, -1))
    m = O.level_map(w, PSA_DEFAULT, 0, "topk", blocksize=128, compute_tile=32)
    assert m.reshape(-1).tolist() == [1, 8, 8, 0, 0, 0, 0, 0, 0, 0]
    assert abs(O.density(m) - 0.125) < 1e-12
    lst = O.level_map(w, PSA_DEFAULT, 0, "topk_newtype", blocksize=128, compute_tile=32).reshape(-1)
    assert lst.tolist() == [0, -1, -1, -1, 1, 2, -1, 3, 4, 5, 6, 7, 8, 9, -1]
    assert O.list_to_dense(lst.reshape(1, -1), 10).reshape(-1).tolist() == [1, 8, 8, 0, 0, 0, 0, 0, 0, 0]


def test_topk_counts_at_256():
    rng = np.random.default_rng(0)
    s = rng.random((1, 1, 2, 256), dtype=np.float32)
    m = O.level_map(s, PSA_DEFAULT, 0, "topk", blocksize=128, compute_tile=32)
    for r in m.reshape(-1, 256):
        assert [(r == lv).sum() for lv in (1, 2, 4, 8, 0)] == [25, 13, 0, 52, 166]


@pytest.mark.parametrize("mode", ["topk", "thresholdbound"])
@pytest.mark.parametrize("bn,tn", [(128, 32), (64, 32), (32, 32), (64, 16)])
def test_invariants(mode, bn, tn):
    rng = np.random.default_rng(7)
    Nk = 97
    s = rng.random((2, 3, 5, Nk), dtype=np.float32) ** 6
    m = O.level_map(s, WAN14, 0, mode, blocksize=bn, compute_tile=tn)
    lst = O.level_map(s, WAN14, 0, mode + "_newtype", blocksize=bn, compute_tile=tn)
    assert np.array_equal(O.list_to_dense(lst, Nk), m)  # both formats say the same thing
    order = np.argsort(-s, -1, kind="stable")
    sl = np.take_along_axis(m, order, -1).reshape(-1, Nk)
    rank = {1: 0, 2: 1, 4: 2, 8: 3, 0: 4}
    div = bn // tn
    for r in sl:
        rk = [rank[int(x)] for x in r]
        assert rk == sorted(rk)  # levels monotone in importance order
        if mode == "thresholdbound":
            assert (r == 1).sum() >= min(Nk, int(Nk * 0.06) + 1)
        for lv in (2, 4, 8):
            al = -(-lv // div)
            n = (r == lv).sum()
            assert n % al == 0
    assert np.array_equal(O.level_map(s * np.float32(4.0), WAN14, 0, mode, blocksize=bn, compute_tile=tn), m)


def test_qwen_energybound_hand_d5():
    S = 4
    s = np.zeros((1, 1, S, S), np.float32)
    s[0, 0, 3] = np.array([8, 4, 3, 1], np.float32) / 16
    s[0, 0, 0, 0] = 1
    s[0, 0, 1, :2] = [0.75, 0.25]
    s[0, 0, 2, :3] = [0.5, 0.3, 0.2]
    ratios = {1: (0, 0.7), 2: (0.7, 0.8), 4: (0.8, 0.9), 8: (0.9, 0.9), 0: (0.9, 1)}
    m = O.level_map_qwen(s, ratios, text_length=0, mode="energybound", block_size=128, causal=True)
    assert m[0, 0, 3].tolist() == [1, 2, 0, 1]
    assert np.array_equal(np.triu(m[0, 0], 1), np.zeros((S, S)))
    assert m[0, 0].diagonal().tolist() == [1] * S and m[0, 0, :, 0].tolist() == [1] * S
    m2 = O.level_map_qwen(s, ratios, text_length=512, mode="energybound", block_size=128, causal=True)
    assert np.array_equal(m2[0, 0], np.tril(np.ones((S, S), np.int32)))


def test_errors():
    with pytest.raises(ValueError):
        O.level_map(np.ones((1, 1, 1, 4), np.float32), None)
    with pytest.raises(ValueError):
        O.level_map(np.ones((1, 1, 1, 4), np.float32), WAN14, mode="nope")


def test_dense_to_list_hand_worked_and_round_trip():
    """dense map -> index list (transfer_mask_to_new_type): a hand-worked row with the alignment rule, and the round trip
    through the list-walking rule of the attention kernel."""
    #            j: 0  1  2  3  4  5  6  7  8  9
    row = np.array([1, 0, 2, 8, 1, 2, 4, 2, 1, 8], np.int32)
    # blocksize == compute_tile: level l segments hold multiples of l.  Sorted by level: 1:[0,4,8] 2:[2,5,7] 4:[6] 8:[3,9] 0:[1]
    #   level 1: 3 blocks, multiple of 1 -> [0,4,8]
    #   level 2: 3 blocks -> 2 stay [2,5], block 7 leads the next segment
    #   level 4: [7,6] is 2 blocks -> 0 stay, both move on
    #   level 8: [7,6,3,9] is 4 blocks -> 0 stay, all move to the skipped segment
    lst = O.dense_to_list(row.reshape(1, -1), 32, 32).reshape(-1).tolist()
    assert lst == [0, 4, 8, -1, 2, 5, -1, -1, -1, 7, 6, 3, 9, 1, -1]
    # blocksize 128, compute tile 32: every alignment is ceil(level / 4) -> 1, 1, 1, 2
    lst = O.dense_to_list(row.reshape(1, -1), 128, 32).reshape(-1).tolist()
    assert lst == [0, 4, 8, -1, 2, 5, 7, -1, 6, -1, 3, 9, -1, 1, -1]
    rng = np.random.default_rng(0)
    m = rng.choice([0, 1, 2, 4, 8], size=(2, 3, 7, 40)).astype(np.int32)
    lst = O.dense_to_list(m, 128, 32)
    assert lst.shape == (2, 3, 7, 45) and (lst == -1).sum(-1).min() == 5 and (lst == -1).sum(-1).max() == 5
    back = O.list_to_dense(lst, 40)
    # without excess (alignment 1 for levels 1-4, level-8 segments rounded down to even) the walk reads the map back,
    # except for a level-8 block that moved into the skipped segment
    moved = (back != m)
    assert np.all(m[moved] == 8) and np.all(back[moved] == 0) and moved.sum(-1).max() <= 1
    # every block is listed exactly once
    body = np.sort(np.where(lst == -1, 10 ** 6, lst), -1)[..., :40]
    assert np.array_equal(body, np.broadcast_to(np.arange(40), body.shape))
