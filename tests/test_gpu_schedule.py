"""The prebuilt tile schedule (psa_build_schedule + psa_fwd_scheduled) against the walk that compacts the map row
inside the kernel (psa_fwd): the schedule lists a row's tiles in the order the in-kernel builder produces them, so
outputs and lse must be the same bits.  The in-kernel walk is the one the other forward tests compare with the oracle
at shapes without a schedule; shapes with one (head dim 64 or 128 with 128-token blocks) reach the oracle through the
schedule in test_gpu_fwd / test_gpu_configs."""
import numpy as np
import pytest
import torch

import psa_oracle as O
from gpu_util import MAX_ABS, MEAN_ABS, attn_errors, dev, random_map, rnd

pytestmark = pytest.mark.gpu
D, BM, BN = 128, 128, 128


def _inputs(B, Hq, Hkv, L, seed, D=D):
    return (rnd(B, Hq, L, D, seed=seed).to(dev()), rnd(B, Hkv, L, D, seed=seed + 1).to(dev()), rnd(B, Hkv, L, D, seed=seed + 2).to(dev()))


@pytest.mark.parametrize(
    "B,Hq,Hkv,L,causal,indexed,p",
    [
        (1, 2, 2, 1024, False, False, (0.35, 0.2, 0.15, 0.15, 0.15)),
        (1, 2, 2, 1000, False, False, (0.35, 0.2, 0.15, 0.15, 0.15)),  # ragged last block: the clamped copies
        (1, 3, 3, 2500, False, False, (0.6, 0.1, 0.1, 0.1, 0.1)),
        (1, 2, 2, 2100, False, False, (0.0, 1.0, 0.0, 0.0, 0.0)),      # every pair at level 1, both halves of the ragged block
        (2, 4, 2, 1930, True, False, (0.35, 0.2, 0.15, 0.15, 0.15)),   # causal diagonal, GQA 2
        (1, 7, 1, 2125, True, False, (0.0, 0.4, 0.2, 0.2, 0.2)),       # GQA 7
        (1, 2, 2, 3000, False, True, (0.35, 0.2, 0.15, 0.15, 0.15)),   # query rows through a token index
        (1, 2, 2, 65, False, False, (0.2, 0.2, 0.2, 0.2, 0.2)),
        (1, 1, 1, 4100, False, False, (0.9, 0.025, 0.025, 0.025, 0.025)),  # rows with very few tiles, empty rows
    ],
)
@pytest.mark.parametrize("D", [128, 64])  # the two-group kernel / the one-row kernel
def test_scheduled_walk_equals_map_walk(B, Hq, Hkv, L, causal, indexed, p, D):
    from psa_hip import ops

    q, k, v = _inputs(B, Hq, Hkv, L, seed=L, D=D)
    Mq, Nk = -(-L // BM), -(-L // BN)
    lmap = torch.from_numpy(random_map(B, Hq, Mq, Nk, L + 7, p=p, ensure_row=False)).to(torch.int8).to(dev())
    qi = torch.randperm(L, generator=torch.Generator().manual_seed(L)).to(torch.int32).to(dev()) if indexed else None
    o0, l0, _ = ops.sparse_attention_fwd(q, k, v, lmap, BM, BN, causal=causal, return_lse=True, q_index=qi, schedule=False)
    sched = ops.build_schedule(lmap, Hkv, L, D, BM, BN, causal)
    o1, l1, _ = ops.sparse_attention_fwd(q, k, v, lmap, BM, BN, causal=causal, return_lse=True, q_index=qi, schedule=sched)
    o2, l2, _ = ops.sparse_attention_fwd(q, k, v, lmap, BM, BN, causal=causal, return_lse=True, q_index=qi)  # builds its own
    torch.cuda.synchronize()
    for o, l in ((o1, l1), (o2, l2)):
        assert torch.equal(o0, o)
        assert torch.equal(l0.nan_to_num(neginf=-1e30), l.nan_to_num(neginf=-1e30))


def test_schedule_is_reusable_and_deterministic():
    """Two builds give the same issue order and tiles (equal-cost rows in index order), and one schedule serves
    several forward calls."""
    from psa_hip import ops
    from psa_hip._lib import lib

    B, H, L = 1, 6, 128 * 70 + 40  # 426 rows: more than one row per issue slot, so the order matters
    q, k, v = _inputs(B, H, H, L, seed=3)
    Mq, Nk = -(-L // BM), -(-L // BN)
    lmap = torch.from_numpy(random_map(B, H, Mq, Nk, 11, ensure_row=False)).to(torch.int8).to(dev())
    s1 = ops.build_schedule(lmap, H, L, D, BM, BN)
    s2 = torch.full_like(s1, 0x5A)
    ops.build_schedule(lmap, H, L, D, BM, BN, out=s2)
    rows = B * H * Mq
    # the issue order starts 64 bytes into the buffer
    assert torch.equal(s1[64:64 + 4 * rows], s2[64:64 + 4 * rows])
    order = s1[64:64 + 4 * rows].view(torch.int32).cpu().numpy()
    assert sorted(int(x) for x in order if x >= 0) == sorted(set(int(x) for x in order if x >= 0))
    outs = [ops.sparse_attention_fwd(q, k, v, lmap, BM, BN, schedule=s) for s in (s1, s2, s1)]
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    ref, _ = O.psa_attention_dense(q.cpu(), k.cpu(), v.cpu(), lmap.cpu().numpy().astype(np.int32), BM, BN)
    mx, mean = attn_errors(outs[0], ref)
    assert mx <= MAX_ABS and mean <= MEAN_ABS, (mx, mean)
    # schedules exist for head dims 64 and 128 with 128-token blocks
    assert lib.psa_schedule_bytes(B, H, H, L, 64, BM, BN) > 0
    assert lib.psa_schedule_bytes(B, H, H, L, 32, BM, BN) == 0 and lib.psa_schedule_bytes(B, H, H, L, D, 64, BN) == 0


def test_strided_rows_fall_back_to_the_map_walk():
    """K / V rows that are not D elements apart ([B, L, H, D] storage) use the schedule's order with the map walk."""
    from psa_hip import ops

    B, H, L = 1, 2, 1500
    q, k, v = _inputs(B, H, H, L, seed=5)
    kt = k.transpose(1, 2).contiguous().transpose(1, 2)  # [B, H, L, D] view of [B, L, H, D] storage
    vt = v.transpose(1, 2).contiguous().transpose(1, 2)
    Mq, Nk = -(-L // BM), -(-L // BN)
    lmap = torch.from_numpy(random_map(B, H, Mq, Nk, 5)).to(torch.int8).to(dev())
    o0 = ops.sparse_attention_fwd(q, k, v, lmap, BM, BN)
    o1 = ops.sparse_attention_fwd(q, kt, vt, lmap, BM, BN)
    torch.cuda.synchronize()
    assert kt.stride(2) != D and torch.equal(o0, o1)


@pytest.mark.parametrize("H,Hkv,L", [(3, 3, 128 * 40), (40, 1, 128 * 128), (64, 1, 128 * 300 + 5), (160, 1, 128 * 300)])
def test_issue_order_is_a_stable_sort_of_every_share(H, Hkv, L):
    """The schedule's issue order (layout: 64 bytes | order | cost | tiles | records of 2 Nk + 4 entries of 16 bytes, every
    part padded to 64 bytes): a permutation of the rows in equal shares, each share sorted by decreasing tile count
    with equal counts in index order - for shares of 15 rows (rank counting), 640 and 2408 (radix sort in LDS) and 6020
    (counting sort)."""
    from psa_hip import ops

    B = 1
    Mq = Nk = -(-L // BM)
    rows = B * H * Mq
    g = torch.Generator().manual_seed(H)
    keep = torch.rand(B, H, Mq, 1, generator=g) ** 2  # strongly uneven rows, many ties among the short ones
    lmap = torch.from_numpy(random_map(B, H, Mq, Nk, 5, ensure_row=False))
    lmap = torch.where(torch.rand(B, H, Mq, Nk, generator=g) < keep, lmap, torch.zeros_like(lmap)).to(torch.int8).to(dev())
    from psa_hip._lib import lib

    buf = torch.full((lib.psa_schedule_bytes(B, H, Hkv, L, D, BM, BN),), 0x5A, dtype=torch.uint8, device=dev())
    sched = ops.build_schedule(lmap, Hkv, L, D, BM, BN, out=buf)
    torch.cuda.synchronize()
    words = sched.cpu().view(torch.int32)
    rows_pad = -(-rows // 16) * 16  # every part is padded to 64 bytes
    n_pad = (words.numel() * 4 - 64 - rows_pad * 8 - rows * (2 * Nk + 4) * 16) // 4
    order = words[16:16 + n_pad].numpy()
    while order[-1] == 0x5A5A5A5A:  # the padding behind the last share is never written
        order = order[:-1]
    n_order = len(order)
    tiles = words[16 + n_pad + rows_pad:16 + n_pad + rows_pad + rows].numpy().astype(np.int64)
    live = order[order >= 0]
    assert np.array_equal(np.sort(live), np.arange(rows))
    t = np.where(order >= 0, tiles[np.clip(order, 0, rows - 1)], -1)
    key_a = t[:-1] * (1 << 32) - order[:-1]   # decreasing tiles, then increasing index (pads: -1 tiles, last)
    key_b = t[1:] * (1 << 32) - order[1:]
    breaks = np.nonzero((key_b > key_a) & (order[1:] >= 0))[0] + 1  # where a new share starts
    assert len(breaks) > 0
    chunk = int(np.gcd.reduce(np.append(breaks, n_order)))
    assert n_order % chunk == 0 and (n_order // chunk) % 8 == 0, (chunk, n_order)
    for s0 in range(0, n_order, chunk):
        share = order[s0:s0 + chunk]
        share = share[share >= 0]
        want = sorted(share.tolist(), key=lambda r: (-min(int(tiles[r]), 2047), r))
        assert share.tolist() == want, s0
