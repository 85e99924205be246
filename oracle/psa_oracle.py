"""CPU oracle for the Pyramid Sparse Attention hot path.

THIS IS TEST INFRASTRUCTURE.  It restates, in plain PyTorch-CPU / numpy, the
arithmetic of the reference (ziplab/Pyramid-Sparse-Attention) for the path

    pyramid K/V pooling -> sampled block-importance estimate -> level map
    -> sparse attention forward (non-causal / causal) -> backward

so that the HIP kernels can be checked against it.  Nothing in the shipped
package imports this file; only tests, the smoke check and the CPU-baseline leg
of the benchmark do.

Each function cites the reference file:line it follows (paths relative to the
reference checkout).  How each function is pinned (the reference ships no tests
and no golden vectors of its own):

  pool_kv                closed form (mean of l consecutive replicate-padded rows)
                         + bit-equality with torch.mean chaining on CPU
  estimate_sampled       brute-force closed form on tiny inputs + invariants
                         (rows sum to 1, uniform logits -> 1/Nk)
  level_map_*            hand-worked rows derived from the source, invariants,
                         and golden vectors written by running the reference's
                         pure-torch transfer_attn_to_mask on CPU
                         (tests/golden/make_level_map_golden.py)
  psa_attention_dense    reduces to torch SDPA in special cases (all-1 map,
                         uniform level on pooled+repeated keys, lossless
                         pooling, single retained block, causal all-1)
  psa_backward_dense     torch.autograd through psa_attention_dense (fp64) and
                         finite differences
  level_map_qwen         rows worked by hand from the source (topk and energybound, causal on / off,
                         trailing text rows and columns, later level overwrites, lower bound
                         max(lo, previous hi), all-zero row) and an independent row-by-row
                         restatement built from the library calls the reference uses (torch.sort,
                         cumsum, sum, tensor-vs-scalar arithmetic) on tie-free rows
  estimate_xattn         brute-force loops in float64: zero-padded tails (L % chunk != 0, padded
                         keys at logit 0, padded query rows 0), stride 8, causal and not, grouped
                         heads, Lk > Lq, plus a closed-form case
  k_similarity           brute-force loops over the explicit token pairs (0,1), (0,3), (0,7) on
                         random keys with ragged tails, and the library's cosine similarity on
                         the slices ::2 / 1::2, 0::4 / 3::4, 0::8 / 7::8 of the reference's
                         pure-torch fall-back
(the last three: tests/test_oracle_qwen_xattn_ksim.py)
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

LEVELS = (1, 2, 4, 8)


# --------------------------------------------------------------------------------------
# A.1  pooling          reference: src/psa_triton/kernels/psa_kernel.py:318-349,381-390
# --------------------------------------------------------------------------------------
def pad_replicate(x: torch.Tensor, multiple: int) -> torch.Tensor:
    """Replicate the last token until the sequence length (dim 2) is a multiple.

    reference: src/psa_triton/kernels/psa_kernel.py:318-329 (F.pad mode='replicate').
    """
    L = x.shape[2]
    rem = L % multiple
    if rem == 0:
        return x
    pad = multiple - rem
    return torch.cat([x, x[:, :, -1:, :].expand(-1, -1, pad, -1)], dim=2)


def _mean2(x: torch.Tensor) -> torch.Tensor:
    """Mean of consecutive token pairs, rounded once to x.dtype (what torch.mean
    does for bf16/fp16: fp32 accumulate, one rounding).

    reference: src/psa_triton/kernels/psa_kernel.py:331-349.
    """
    B, H, L, D = x.shape
    assert L % 2 == 0
    xf = (x if x.dtype == torch.float64 else x.float()).view(B, H, L // 2, 2, D)
    return ((xf[:, :, :, 0] + xf[:, :, :, 1]) * 0.5).to(x.dtype)


def pool_kv(x: torch.Tensor, block_n: int) -> Dict[int, torch.Tensor]:
    """Pyramid levels of K or V.  Level 1 is the UN-padded input; level 2 is the
    pairwise mean of the replicate-padded input, level 4 the pairwise mean of the
    (already rounded) level 2, level 8 of level 4.

    reference: src/psa_triton/kernels/psa_kernel.py:381-388.
    """
    xp = pad_replicate(x, block_n)
    l2 = _mean2(xp)
    l4 = _mean2(l2)
    l8 = _mean2(l4)
    return {1: x, 2: l2, 4: l4, 8: l8}


def pool_kv_direct(x: torch.Tensor, block_n: int, level: int) -> torch.Tensor:
    """Closed form used to pin pool_kv: fp64 mean of `level` consecutive padded rows."""
    xp = pad_replicate(x, block_n).double()
    B, H, L, D = xp.shape
    return xp.view(B, H, L // level, level, D).mean(3)


# --------------------------------------------------------------------------------------
# A.2  sampling + block-importance estimate
#      reference: src/psa_triton/attention.py:116-137,178-223
#                 src/psa_triton/kernels/attn_pooling_kernel.py:12-116,285-431
# --------------------------------------------------------------------------------------
def sample_offsets(B: int, H: int, block: int, keep: int, generator: torch.Generator) -> torch.Tensor:
    """`keep` distinct in-block offsets per (b, h), shared by every block of that
    head.  reference: src/psa_triton/attention.py:132-133 (rand -> topk)."""
    r = torch.rand(B, H, block, generator=generator)
    return torch.topk(r, keep, dim=2).indices.to(torch.int32)


def gather_samples(x: torch.Tensor, block: int, offs: torch.Tensor) -> torch.Tensor:
    """Rows `blk*block + offs[b,h,:]` of the replicate-padded x.
    reference: src/psa_triton/attention.py:128-137."""
    xp = pad_replicate(x, block)
    B, H, L, D = xp.shape
    nb = L // block
    keep = offs.shape[-1]
    idx = (torch.arange(nb).view(1, 1, nb, 1) * block + offs.long().view(B, H, 1, keep)).reshape(B, H, nb * keep)
    return torch.gather(xp, 2, idx.unsqueeze(-1).expand(-1, -1, -1, D))


def estimate_from_sampled(
    sq: torch.Tensor,
    sk: torch.Tensor,
    sm_scale: float,
    keep_m: int,
    keep_n: int,
    tile: int = 64,
) -> torch.Tensor:
    """Block-importance estimate from already-sampled rows.

    sq [B,Hq,Ms,D], sk [B,Hkv,Ns,D] -> Po [B,Hq,ceil(Ms_pad/keep_m),ceil(Ns_pad/keep_n)] fp32,
    where *_pad is the length replicate-padded to a multiple of `tile`
    (reference: src/psa_triton/attention.py:214-215).

    R[r,j]  = max_{c in key-group j} (sq_r . sk_c) * sm_scale * log2(e)      (attn_pooling_kernel.py:62-66)
    m[r]    = max_j R[r,j]                                                  (:66-72)
    Po[i,j] = max_{r in q-group i} exp2(R[r,j] - m[r])                      (:93-105; l_i stays 1.0, :218)
    Po     /= Po.sum(-1)                                                    (:428-429)

    Scores stay fp32 (the reference rounds R and Po to the input dtype; the
    level-map contract is defined on fp32 scores).
    """
    sq = pad_replicate(sq, tile)
    sk = pad_replicate(sk, tile)
    B, Hq, Ms, D = sq.shape
    Hkv, Ns = sk.shape[1], sk.shape[2]
    n_rep = Hq // Hkv
    if n_rep > 1:
        sk = sk.repeat_interleave(n_rep, dim=1)  # kv head = q head // n_rep (attn_pooling_kernel.py:171)
    m_d = -(-Ms // keep_m)
    n_d = -(-Ns // keep_n)
    assert Ms % keep_m == 0 and Ns % keep_n == 0
    qk_scale = np.float32(np.float32(sm_scale) * np.float32(1.44269504))
    S = torch.matmul(sq.float(), sk.float().transpose(-1, -2))  # fp32 accumulate
    R = S.view(B, Hq, Ms, n_d, keep_n).amax(-1) * float(qk_scale)
    m = R.amax(-1, keepdim=True)
    E = torch.exp2(R - m)
    Po = E.view(B, Hq, m_d, keep_m, n_d).amax(3)
    return Po / Po.sum(-1, keepdim=True)


def estimate_sampled(
    q: torch.Tensor,
    k: torch.Tensor,
    block_m: int,
    block_n: int,
    off_q: torch.Tensor,
    off_k: torch.Tensor,
    sm_scale: Optional[float] = None,
) -> torch.Tensor:
    """Full estimator of the plug-and-play module: sample block/4 rows per block
    with the given offsets, estimate, crop to [Mq, Nk].
    reference: src/psa_triton/attention.py:178-223."""
    D = q.shape[-1]
    sm_scale = 1.0 / (D ** 0.5) if sm_scale is None else sm_scale
    keep_m, keep_n = off_q.shape[-1], off_k.shape[-1]
    sq = gather_samples(q, block_m, off_q)
    sk = gather_samples(k, block_n, off_k)
    Mq = sq.shape[2] // keep_m
    Nk = sk.shape[2] // keep_n
    Po = estimate_from_sampled(sq, sk, sm_scale, keep_m, keep_n)
    return Po[:, :, :Mq, :Nk]


# --------------------------------------------------------------------------------------
# A.3  level map        reference: src/psa_triton/utils/transfer_attn_to_mask.py:6-507
# --------------------------------------------------------------------------------------
def _sort_desc_stable(scores: np.ndarray) -> np.ndarray:
    """Descending order, ties -> lower kv-block index first (the build's contract;
    the reference calls torch.sort(descending=True), whose tie order is unspecified:
    transfer_attn_to_mask.py:57,130)."""
    return np.argsort(-scores, axis=-1, kind="stable")


def _align(level: int, div: int) -> int:
    return math.ceil(level / div)


def _topk_intervals(mask_ratios: Dict[int, Tuple[float, float]], Nk: int, div: int) -> List[Tuple[int, int, int]]:
    """(level, start, end) per mask_ratios item in insertion order; empty -> start == end.
    reference: transfer_attn_to_mask.py:63-120 (dense) and :282-351 (list format)."""
    out = []
    last_end = 0
    for level, (_lo, hi) in mask_ratios.items():
        align = 1 if level == 0 else _align(level, div)
        start = last_end
        end0 = min(Nk, int(Nk * hi))
        length = end0 - start
        if align > 1 and length > 0:
            rem = length % align
            alen = length + (align - rem) if rem else length
            end = min(start + alen, Nk)
            if end == Nk:
                end = start + ((end - start) // align) * align
        else:
            end = end0
        if start < end:
            out.append((level, start, end))
            last_end = end
        else:
            out.append((level, start, start))
    return out


def _threshold_counts(scores_sorted: np.ndarray, his: Sequence[float]) -> np.ndarray:
    """#{p : r[p] <= fp32(hi + 1e-6)} per row and threshold, with
    r = fp32(cumsum in fp64, each prefix rounded to fp32) / fp32 total.
    reference: transfer_attn_to_mask.py:134-139,156,171 (torch.cumsum on fp32 CPU
    tensors accumulates in double and rounds every prefix; a Python scalar compared
    with an fp32 tensor is rounded to fp32)."""
    w = scores_sorted.astype(np.float32)
    c = np.cumsum(w.astype(np.float64), axis=-1).astype(np.float32)
    r = c / c[..., -1:]
    cnts = []
    for hi in his:
        thr = np.float32(hi + 1e-6)
        cnts.append((r <= thr).sum(-1))
    return np.stack(cnts, -1).astype(np.int64)


def _threshold_intervals(
    cnt: np.ndarray,
    items: List[Tuple[int, Tuple[float, float]]],
    Nk: int,
    div: int,
    min_full_attn_ratio: float,
) -> np.ndarray:
    """Per-row (start, end) for each item (already ordered by upper bound).
    cnt [..., n_items] -> ivals [..., n_items, 2].
    reference: transfer_attn_to_mask.py:150-265."""
    shape = cnt.shape[:-1]
    last = np.zeros(shape, dtype=np.int64)
    iv = np.zeros(shape + (len(items), 2), dtype=np.int64)
    for t, (level, _) in enumerate(items):
        align = _align(level, div)  # level 0 -> 0 -> "no alignment" branch (:152,185,218)
        c = cnt[..., t]
        end0 = np.where(c > 0, c + 1, last)
        start = last
        if align > 1:
            length = np.maximum(end0 - start, 0)
            rem = length % align
            alen = np.where(rem != 0, length + (align - rem), length)
            end = np.minimum(start + alen, Nk)
            at_b = end == Nk
            down = ((end - start) // align) * align
            end = np.where(at_b, start + down, end)
        else:
            end = np.maximum(np.clip(end0, 0, Nk), start)
            if level == 1:
                end = np.maximum(end, min(Nk, int(Nk * min_full_attn_ratio) + 1))
        iv[..., t, 0] = start
        iv[..., t, 1] = end
        last = end
    return iv


def level_map(
    scores: np.ndarray,
    mask_ratios: Dict[int, Tuple[float, float]],
    text_length: int = 226,
    mode: str = "topk",
    min_full_attn_ratio: float = 0.06,
    blocksize: int = 32,
    compute_tile: int = 32,
) -> np.ndarray:
    """scores [B,H,Mq,Nk] fp32 -> int32 level map (dense modes) or index list
    (`*_newtype` modes, [B,H,Mq,Nk+len(mask_ratios)]).

    reference: src/psa_triton/utils/transfer_attn_to_mask.py:6-507.
    """
    if mask_ratios is None:
        raise ValueError("mask_ratios must be provided")
    scores = np.asarray(scores, dtype=np.float32)
    B, H, Mq, Nk = scores.shape
    div = blocksize // compute_tile
    idx = _sort_desc_stable(scores)
    newtype = mode.endswith("_newtype")
    base = mode[: -len("_newtype")] if newtype else mode
    if base == "topk":
        ivs = _topk_intervals(mask_ratios, Nk, div)
        levels = [lv for lv, _, _ in ivs]
        iv = np.zeros((B, H, Mq, len(ivs), 2), dtype=np.int64)
        for t, (_, s, e) in enumerate(ivs):
            iv[..., t, 0] = s
            iv[..., t, 1] = e
    elif base == "thresholdbound":
        items = sorted(mask_ratios.items(), key=lambda x: x[1][1])  # stable (:142)
        levels = [lv for lv, _ in items]
        w = np.take_along_axis(scores, idx, -1)
        cnt = _threshold_counts(w, [hi for _, (_, hi) in items])
        iv = _threshold_intervals(cnt, items, Nk, div, min_full_attn_ratio)
    else:
        raise ValueError(f"Unknown mode: {mode}. Must be 'topk' or 'thresholdbound'")

    pos = np.arange(Nk).reshape(1, 1, 1, Nk)
    if not newtype:
        sorted_lv = np.zeros((B, H, Mq, Nk), dtype=np.int32)
        for t, lv in enumerate(levels):
            sel = (pos >= iv[..., t, 0:1]) & (pos < iv[..., t, 1:2])
            sorted_lv = np.where(sel, np.int32(lv), sorted_lv)
        out = np.zeros((B, H, Mq, Nk), dtype=np.int32)
        np.put_along_axis(out, idx, sorted_lv, -1)
        if text_length > 0:  # process_text_tokens (:40-45)
            tb = (text_length + blocksize - 1) // blocksize
            out[..., -tb:] = 1
        return out

    n_items = len(levels)
    out = np.zeros((B, H, Mq, Nk + n_items), dtype=np.int32)
    for t in range(n_items):
        sel = (pos >= iv[..., t, 0:1]) & (pos < iv[..., t, 1:2])
        seg = out[..., t : t + Nk]
        seg[...] = np.where(sel, idx.astype(np.int32), seg)
        sep = np.clip(iv[..., t, 1] + t, 0, Nk + n_items - 1)
        np.put_along_axis(out, sep[..., None], np.int32(-1), -1)
    return out


def list_to_dense(list_mask: np.ndarray, Nk: int) -> np.ndarray:
    """What the reference's list-walking kernel makes of an index list: the segment
    level starts at 1 and doubles at every -1, the walk stops once it exceeds 8 or
    after `list width` columns.  reference: src/psa_triton/kernels/psa_kernel.py:207-217."""
    lm = np.asarray(list_mask)
    lead = lm.shape[:-1]
    flat = lm.reshape(-1, lm.shape[-1])
    out = np.zeros((flat.shape[0], Nk), dtype=np.int32)
    for r in range(flat.shape[0]):
        mode = 1
        for v in flat[r]:
            if mode > 8:
                break
            if v == -1:
                mode *= 2
            else:
                out[r, v] = mode
    return out.reshape(lead + (Nk,))


def dense_to_list(level_map_dense: np.ndarray, blocksize: int = 32, compute_tile: int = 32) -> np.ndarray:
    """Dense level map [..., Nk] -> index list [..., Nk + 5]: blocks at levels 1, 2, 4, 8, then the skipped ones, a -1
    behind each segment; a segment's length is rounded down to a multiple of ceil(level / (blocksize // compute_tile))
    and the blocks that do not fit lead the next segment.
    reference: src/psa_triton/utils/transfer_attn_to_mask.py:624-750 (transfer_mask_to_new_type).  Blocks of a level
    are listed in ascending order (the reference leaves the order inside a level to torch.sort)."""
    m = np.asarray(level_map_dense)
    lead, Nk = m.shape[:-1], m.shape[-1]
    flat = m.reshape(-1, Nk)
    div = max(1, blocksize // compute_tile)
    out = np.zeros((flat.shape[0], Nk + 5), dtype=np.int32)
    for r in range(flat.shape[0]):
        order = [j for val in (1, 2, 4, 8) for j in range(Nk) if flat[r, j] == val]
        order += [j for j in range(Nk) if flat[r, j] not in (1, 2, 4, 8)]
        counts = [int((flat[r] == val).sum()) for val in (1, 2, 4, 8)]
        counts.append(Nk - sum(counts))
        for t, val in enumerate((1, 2, 4, 8)):
            mult = max(1, -(-val // div))
            rem = counts[t] % mult if mult > 1 else 0
            counts[t] -= rem
            counts[t + 1] += rem
        pos, src = 0, 0
        for t in range(5):
            out[r, pos : pos + counts[t]] = order[src : src + counts[t]]
            pos += counts[t]
            src += counts[t]
            out[r, pos] = -1
            pos += 1
    return out.reshape(lead + (Nk + 5,))


def density(level_map_dense: np.ndarray) -> float:
    """mean(1/level) with skipped blocks counting 0.
    reference: src/psa_triton/utils/transfer_attn_to_mask.py:510-544."""
    m = np.asarray(level_map_dense).astype(np.float64)
    inv = np.where(m > 0, 1.0 / np.maximum(m, 1), 0.0)
    return float(inv.mean())


def level_map_qwen(
    scores: np.ndarray,
    mask_ratios: Dict[int, Tuple[float, float]],
    text_length: int = 512,
    mode: str = "energybound",
    block_size: int = 128,
    causal: bool = True,
) -> np.ndarray:
    """Causal level map of the Qwen2.5-VL example.
    reference: qwen2.5-vl-example/src/attention/PSA_casual/PyramidAdaptiveBlockSparseAttn.py:84-168.
    Sort contract as in level_map (stable, ties -> lower index)."""
    scores = np.asarray(scores, dtype=np.float32)
    B, H, S, S2 = scores.shape
    assert S == S2
    idx = _sort_desc_stable(scores)
    w = np.take_along_axis(scores, idx, -1)
    pos = np.arange(S).reshape(1, 1, 1, S)
    sorted_lv = np.zeros((B, H, S, S), dtype=np.int32)
    if mode == "topk":
        valid = (np.arange(S, dtype=np.float32) + 1.0) if causal else np.full(S, float(S), np.float32)
        valid = valid.reshape(1, 1, S, 1)
        for lv, (lo, hi) in mask_ratios.items():
            s = np.minimum(np.floor(valid * np.float32(lo)).astype(np.int64), S)
            e = np.minimum(np.floor(valid * np.float32(hi)).astype(np.int64), S)
            sel = (pos >= s) & (pos < e)
            sorted_lv = np.where(sel, np.int32(lv), sorted_lv)
    elif mode == "energybound":
        # contract of this build: the row total is the last prefix sum (sequential fp64 accumulation over the sorted
        # row, rounded to fp32); the reference divides by torch's fp32 sum of the unsorted row (:134), whose
        # summation order is an implementation detail of the library
        c = np.cumsum(w.astype(np.float64), -1).astype(np.float32)
        total = np.maximum(c[..., -1:], np.float32(1e-10))
        r = c / total
        prev_hi = 0.0
        for lv, (lo, hi) in mask_ratios.items():
            lower = max(lo, prev_hi)
            sel = (r > np.float32(lower)) & (r <= np.float32(hi))
            sorted_lv = np.where(sel, np.int32(lv), sorted_lv)
            prev_hi = hi
    else:
        raise ValueError(f"unknown mode {mode}")
    out = np.zeros((B, H, S, S), dtype=np.int32)
    np.put_along_axis(out, idx, sorted_lv, -1)
    if text_length > 0:
        nb = min((text_length + block_size - 1) // block_size, S)
        if nb > 0:
            out[..., -nb:] = 1
            out[..., -nb:, :] = 1
    if causal:
        out = np.where(np.triu(np.ones((S, S), dtype=bool), 1), 0, out)
    d = np.arange(S)
    out[..., d, d] = 1
    out[..., 0] = 1
    return out.astype(np.int32)


# --------------------------------------------------------------------------------------
# A.4  sparse attention forward
#      reference: src/psa_triton/kernels/psa_kernel.py:24-316 (list walk),
#                 src/psa_triton/kernels/psa_kernel_legacy.py:34-130,415-799 (dense map, causal)
# --------------------------------------------------------------------------------------
def _expanded_keys(levels_k: Dict[int, torch.Tensor], lmap: torch.Tensor, block_m: int, block_n: int, L: int, causal: bool):
    """Concatenate all four levels along the key axis and build the additive bias
    [B,H,Lq,sum N_l]: +ln(level) where (q-block, kv-block) sits at that level (and the
    key passes the causal rule), -inf elsewhere."""
    B, H, Mq, Nk = lmap.shape
    dev = lmap.device
    qi = torch.arange(L, device=dev)
    qblk = qi // block_m
    biases = []
    for lv in LEVELS:
        N_l = levels_k[lv].shape[2]
        t = torch.arange(N_l, device=dev)
        per = block_n // lv
        kblk = t // per  # kv-block of pooled key t
        sel = lmap[:, :, qblk][:, :, :, kblk] == lv  # [B,H,L,N_l]
        if causal:
            # a pooled key is visible once its last constituent is: (t+1)*lv-1 <= i
            # (psa_kernel_legacy.py:79-81); blocks beyond the diagonal are never visited (:584-586)
            vis = ((t + 1) * lv - 1).view(1, -1) <= qi.view(-1, 1)
            blk_ok = kblk.view(1, -1) < ((qblk + 1) * block_m + block_n - 1).view(-1, 1) // block_n
            sel = sel & (vis & blk_ok).view(1, 1, L, N_l)
        bias = torch.full(sel.shape, float("-inf"), dtype=torch.float64, device=dev)
        bias[sel] = math.log(lv)
        biases.append(bias)
    return torch.cat(biases, -1)


def psa_attention_dense(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lmap,
    block_m: int,
    block_n: int,
    sm_scale: Optional[float] = None,
    causal: bool = False,
    levels_k: Optional[Dict[int, torch.Tensor]] = None,
    levels_v: Optional[Dict[int, torch.Tensor]] = None,
    dtype=torch.float64,
):
    """Reference semantics as ONE dense softmax over the concatenated pyramid:
    logit(i, (l,t)) = scale * q_i.K_l[t] + ln l for retained pairs, one softmax over
    all levels, out = P @ [V_l].  Returns (out [B,H,L,D], lse [B,H,L]) in `dtype`.
    Rows without any key give out = 0 and lse = -inf (psa_kernel_legacy.py:783-788).

    Memory is O(L * 1.875 L): small shapes only.
    """
    lmap = torch.as_tensor(np.asarray(lmap)).long() if not torch.is_tensor(lmap) else lmap.long()
    B, H, L, D = q.shape
    Hkv = k.shape[1]
    sm_scale = 1.0 / (D ** 0.5) if sm_scale is None else sm_scale
    if levels_k is None:
        levels_k = pool_kv(k, block_n)
    if levels_v is None:
        levels_v = pool_kv(v, block_n)
    n_rep = H // Hkv
    Kc = torch.cat([levels_k[lv] for lv in LEVELS], 2).to(dtype)
    Vc = torch.cat([levels_v[lv] for lv in LEVELS], 2).to(dtype)
    if n_rep > 1:
        Kc = Kc.repeat_interleave(n_rep, 1)
        Vc = Vc.repeat_interleave(n_rep, 1)
    bias = _expanded_keys(levels_k, lmap, block_m, block_n, L, causal).to(dtype)
    S = torch.matmul(q.to(dtype), Kc.transpose(-1, -2)) * sm_scale + bias
    # rows without any key: output 0, lse -inf, and (under autograd) zero gradient instead of NaN
    row_ok = (S > float("-inf")).any(-1, keepdim=True)
    S_safe = torch.where(row_ok, S, torch.zeros_like(S))
    lse_safe = torch.logsumexp(S_safe, -1, keepdim=True)
    P = torch.exp(S_safe - lse_safe) * row_ok.to(dtype)
    lse = torch.where(row_ok, lse_safe, torch.full_like(lse_safe, float("-inf"))).squeeze(-1)
    out = torch.matmul(P, Vc)
    return out, lse


def psa_attention_blockwalk(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    lmap,
    block_m: int,
    block_n: int,
    sm_scale: Optional[float] = None,
    causal: bool = False,
    dtype=torch.float32,
    heads: Optional[Sequence[int]] = None,
    qblocks: Optional[Sequence[int]] = None,
):
    """Same semantics, memory O(block_m * L): per (b, h, q-block) gather the retained
    pooled keys/values, two matmuls, one softmax with +ln(level).  Used for large
    shapes and as the CPU baseline.  `heads` / `qblocks` restrict the work (outputs for
    the others stay zero)."""
    lm = np.asarray(lmap.cpu() if torch.is_tensor(lmap) else lmap)
    B, H, L, D = q.shape
    Hkv = k.shape[1]
    n_rep = H // Hkv
    sm_scale = 1.0 / (D ** 0.5) if sm_scale is None else sm_scale
    lk = {lv: t.to(dtype) for lv, t in pool_kv(k, block_n).items()}
    lvv = {lv: t.to(dtype) for lv, t in pool_kv(v, block_n).items()}
    out = torch.zeros(B, H, L, D, dtype=dtype)
    lse = torch.full((B, H, L), float("-inf"), dtype=dtype)
    Mq = lm.shape[2]
    heads = range(H) if heads is None else heads
    qblocks = range(Mq) if qblocks is None else qblocks
    for b in range(B):
        for h in heads:
            hk = h // n_rep
            for I in qblocks:
                q0, q1 = I * block_m, min((I + 1) * block_m, L)
                qi = torch.arange(q0, q1)
                ks, vs, bs, ups = [], [], [], []
                row = lm[b, h, I]
                jmax = min(lm.shape[3], ((I + 1) * block_m + block_n - 1) // block_n) if causal else lm.shape[3]
                for lv in LEVELS:
                    per = block_n // lv
                    N_l = lk[lv].shape[2]
                    js = np.nonzero(row[:jmax] == lv)[0]
                    if js.size == 0:
                        continue
                    t = (torch.as_tensor(js).view(-1, 1) * per + torch.arange(per).view(1, -1)).reshape(-1)
                    t = t[t < N_l]
                    ks.append(lk[lv][b, hk, t])
                    vs.append(lvv[lv][b, hk, t])
                    bs.append(torch.full((t.numel(),), math.log(lv), dtype=dtype))
                    ups.append((t + 1) * lv - 1)
                if not ks:
                    continue
                Kc, Vc, bias = torch.cat(ks), torch.cat(vs), torch.cat(bs)
                S = (q[b, h, q0:q1].to(dtype) @ Kc.T) * sm_scale + bias
                if causal:
                    up = torch.cat(ups)
                    S = torch.where(up.view(1, -1) <= qi.view(-1, 1), S, torch.full_like(S, float("-inf")))
                l = torch.logsumexp(S, -1)
                safe = torch.where(torch.isinf(l), torch.zeros_like(l), l)
                P = torch.exp(S - safe.unsqueeze(-1))
                P = torch.where(torch.isinf(S), torch.zeros_like(P), P)
                out[b, h, q0:q1] = P @ Vc
                lse[b, h, q0:q1] = l
    return out, lse


# --------------------------------------------------------------------------------------
# A.5  backward          reference: src/psa_triton/kernels/psa_kernel_legacy.py:948-1069,
#                                   1072-1234 (kernels), 1280-1320 (pool / un-pool rules)
# --------------------------------------------------------------------------------------
def psa_backward_dense(q, k, v, lmap, do, block_m, block_n, sm_scale=None, causal=False, dtype=torch.float64):
    """dQ, dK, dV by autograd through psa_attention_dense with differentiable pooling
    (replicate pad -> mean over `level` rows), which yields exactly the reference's
    un-pool rule: every constituent token of pooled key t receives dK_l[t]/l and the
    gradient of replicate-pad positions is summed into the last real token
    (psa_kernel_legacy.py:1298-1320).  The level map carries no gradient
    (src/psa_triton/attention.py:276)."""
    qd = q.detach().to(dtype).requires_grad_(True)
    kd = k.detach().to(dtype).requires_grad_(True)
    vd = v.detach().to(dtype).requires_grad_(True)

    def levels(x):
        xp = pad_replicate(x, block_n)
        B, H, Lp, D = xp.shape
        out = {1: x}
        for lv in (2, 4, 8):
            out[lv] = xp.view(B, H, Lp // lv, lv, D).mean(3)
        return out

    out, _ = psa_attention_dense(qd, kd, vd, lmap, block_m, block_n, sm_scale, causal, levels(kd), levels(vd), dtype)
    out.backward(do.to(dtype))
    return qd.grad, kd.grad, vd.grad


# --------------------------------------------------------------------------------------
# A.6  xattn-style estimator of the Qwen example (intended = Triton-kernel semantics)
#      reference: qwen2.5-vl-example/src/attention/PSA_casual/kernels/block_importance_kernels.py:6-192,255-323
#                 qwen2.5-vl-example/src/attention/PSA_casual/utils/block_importance.py:282-462,557-560
# --------------------------------------------------------------------------------------
def estimate_xattn(q, k, block_size=128, stride=8, causal=True, chunk_size=4096, dtype=torch.float32):
    """A[m,n] = sum_{i<S} q[mS+S-1-i] . k[nS+i];  Z = A / (sqrt(D) * S);
    causal keep n <= m (+ offset); row softmax over all strided keys; sum the
    probabilities inside each (block/S)^2 cell.  Zero padding of q, k to a multiple of
    chunk_size; padded q rows give 0; padded keys are NOT masked (logit 0).
    Returns [B,H,ceil(Lq/block),ceil(Lk/block)] fp32."""
    B, H, Lq, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    S = stride
    if H != Hkv:
        k = k.repeat_interleave(H // Hkv, 1)

    def zpad(x, mult):
        L = x.shape[2]
        pad = (-L) % mult
        return F.pad(x, (0, 0, 0, pad)) if pad else x

    qp, kp = zpad(q, chunk_size).to(dtype), zpad(k, chunk_size).to(dtype)
    Lqp, Lkp = qp.shape[2], kp.shape[2]
    Mr, Nr = Lqp // S, Lkp // S
    qr = qp.view(B, H, Mr, S, D).flip(3)  # q[mS + S-1-i] at index i
    kr = kp.view(B, H, Nr, S, D)
    A = torch.einsum("bhmid,bhnid->bhmn", qr, kr)
    Z = A * (1.0 / (math.sqrt(D) * S))
    if causal:
        off = Nr - Mr
        mi = torch.arange(Mr).view(-1, 1)
        ni = torch.arange(Nr).view(1, -1)
        Z = torch.where(ni <= mi + off, Z, torch.full_like(Z, float("-inf")))
    P = torch.softmax(Z, -1)
    real_rows = -(-Lq // S)
    P[:, :, real_rows:, :] = 0
    rb = block_size // S
    E = P.view(B, H, Mr // rb, rb, Nr // rb, rb).sum((3, 5))
    return E[:, :, : -(-Lq // block_size), : -(-Lk // block_size)].float()


# --------------------------------------------------------------------------------------
# K-similarity "sim mask"   reference: src/psa_triton/attention.py:140-164
# --------------------------------------------------------------------------------------
def k_similarity_scores(k: torch.Tensor, block_n: int):
    """(sim2, sim4, sim8) [B,H,Nk] fp32: mean over the block of the cosine similarity of token pairs
    (2g, 2g+1), (4g, 4g+3), (8g, 8g+7), with the GPU kernel's formula
    cos = a.b / (sqrt(|a|^2 + 1e-12) * sqrt(|b|^2 + 1e-12) + 1e-6); tokens past L replicate the last.
    reference: src/psa_triton/kernels/calc_ksim_kernel.py:66-137 (torch fallback: src/psa_triton/attention.py:140-164,
    identical up to the epsilons)."""
    kp = pad_replicate(k, block_n).float()
    B, H, L, D = kp.shape
    nb = L // block_n
    kc = kp.reshape(B, H, nb, block_n, D)
    nrm = torch.sqrt((kc * kc).sum(-1) + 1e-12)

    def sim(step):
        a, b_ = kc[..., 0::step, :], kc[..., step - 1::step, :]
        na, nb_ = nrm[..., 0::step], nrm[..., step - 1::step]
        return ((a * b_).sum(-1) / (na * nb_ + 1e-6)).mean(-1)

    return sim(2), sim(4), sim(8)


def k_similarity(k: torch.Tensor, block_n: int, thr2: float, thr4: float, thr8: float) -> torch.Tensor:
    """Per kv-block cap on the pooling level: the largest l in {2,4,8} whose similarity passes its
    threshold (strict >), at least 1.  reference: src/psa_triton/kernels/calc_ksim_kernel.py:139-144."""
    s2, s4, s8 = k_similarity_scores(k, block_n)
    out = torch.ones_like(s2, dtype=torch.int32)
    out = torch.where(s2 > thr2, torch.full_like(out, 2), out)
    out = torch.where(s4 > thr4, torch.full_like(out, 4), out)
    out = torch.where(s8 > thr8, torch.full_like(out, 8), out)
    return out


# --------------------------------------------------------------------------------------
# whole layer (what PSAAttention.forward does)   reference: src/psa_triton/attention.py:261-310
# --------------------------------------------------------------------------------------
def psa_layer(
    q, k, v, *, block_m, block_n, tile_n, mask_ratios, mask_mode, off_q, off_k,
    text_length=0, causal=False, dtype=torch.float32, dense=False,
):
    """estimate -> level map -> sparse attention; returns (out, lse, level map, scores)."""
    scores = estimate_sampled(q, k, block_m, block_n, off_q, off_k)
    lm = level_map(scores.numpy(), mask_ratios, text_length, mask_mode, blocksize=block_n, compute_tile=tile_n)
    fn = psa_attention_dense if dense else psa_attention_blockwalk
    out, lse = fn(q, k, v, lm, block_m, block_n, None, causal, dtype=dtype)
    return out, lse, lm, scores
