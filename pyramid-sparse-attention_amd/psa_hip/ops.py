"""Torch-facing wrappers of the C-ABI kernels.  PyTorch only supplies device memory and the
current stream; every operator here runs a hand-written HIP kernel and there is no CPU path."""
import ctypes
from typing import Dict, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import Tensor4, check, lib

LEVELS = (1, 2, 4, 8)


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("psa_hip operators run on the GPU only (got a %s tensor); there is no CPU path" % t.device)


_DTYPE_ID = {torch.bfloat16: _lib.PSA_DTYPE_BF16, torch.float16: _lib.PSA_DTYPE_F16, torch.float32: _lib.PSA_DTYPE_F32}


def _kernel_view(x: torch.Tensor, types=(torch.bfloat16, torch.float16, torch.float32)) -> torch.Tensor:
    """[B,H,L,D] tensor usable by the kernels: one of `types` (the element types the operator has kernels for: the
    tensor is computed on in its own type; any other type is rounded to bf16 first), D contiguous, 16-byte aligned
    rows."""
    if x.dim() != 4:
        raise ValueError("expected a [B, H, L, D] tensor, got shape %s" % (tuple(x.shape),))
    if x.dtype not in types:
        x = x.to(torch.bfloat16)
    per16 = 16 // x.element_size()
    ok = x.stride(3) == 1 and all(s % per16 == 0 for s in x.stride()[:3]) and x.data_ptr() % 16 == 0
    return x if ok else x.contiguous()


def _bf16_view(x: torch.Tensor) -> torch.Tensor:
    """For the operators whose kernels take bf16 only (backward, antidiagonal estimate)."""
    return _kernel_view(x, (torch.bfloat16,))


_T16 = (torch.bfloat16, torch.float16)


def _same_type(*ts):
    """Tensors of one call share one element type: anything that differs from the first is converted to it."""
    dt = ts[0].dtype
    return tuple(t if t.dtype == dt else t.to(dt) for t in ts)


def _t4(x: torch.Tensor) -> Tensor4:
    return Tensor4(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2), _DTYPE_ID[x.dtype], 0)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


# ----------------------------------------------------------------------------- pooling
def pool_kv(k: torch.Tensor, v: torch.Tensor, block_n: int, out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
            ) -> Tuple[torch.Tensor, torch.Tensor]:
    """One pass over K and V -> flat pooled buffers holding levels 2, 4, 8 (see pool_levels).  out: the two buffers,
    allocated by the caller (bf16, psa_pool_elems elements each)."""
    _require_gpu(k, v)
    k, v = _same_type(_kernel_view(k), _kernel_view(v))
    B, H, L, D = k.shape
    if v.shape != k.shape:
        raise ValueError("k and v must have the same shape")
    n = lib.psa_pool_elems(B, H, L, D, block_n)
    if out is None:
        kp = torch.empty(n, dtype=k.dtype, device=k.device)
        vp = torch.empty(n, dtype=k.dtype, device=k.device)
    else:
        kp, vp = out
        for t in (kp, vp):
            if t.dtype != k.dtype or t.numel() != n or not t.is_contiguous() or t.device != k.device:
                raise ValueError("pool_kv: out must be two contiguous %s buffers of %d elements on %s" % (k.dtype, n, k.device))
    with torch.cuda.device(k.device):
        check(lib.psa_pool_kv(_t4(k), _t4(v), _ptr(kp), _ptr(vp), B, H, L, D, block_n, _stream(k)), "psa_pool_kv")
    return kp, vp


_VALID_INDEX: Dict[Tuple[int, int, int, int], bool] = {}


def validate_token_index(index: torch.Tensor, L: int) -> None:
    """Raises ValueError unless index is a permutation of 0 .. L-1 (works on CPU and GPU tensors; one small reduction)."""
    if index.dtype != torch.int32 or index.dim() != 1 or index.numel() != L:
        raise ValueError("index must be a 1-D int32 tensor with one entry per token (%d)" % L)
    if L == 0:
        return
    idx = index.to(torch.int64)
    if int(idx.min()) < 0 or int(idx.max()) >= L:
        raise ValueError("token index has entries outside 0 .. %d" % (L - 1))
    seen = torch.zeros(L, dtype=torch.int32, device=index.device)
    seen.index_fill_(0, idx, 1)
    if int(seen.sum()) != L:
        raise ValueError("token index is not a permutation of 0 .. %d: %d positions are never written" % (L - 1, L - int(seen.sum())))


def _check_index(index: torch.Tensor, L: int) -> torch.Tensor:
    """A token index the kernels can use: int32, one entry per token, a permutation of 0 .. L-1.  A bad entry would make
    a kernel read or write another row (the kernels clamp reads and drop stores outside the tensor, so nothing faults,
    but rows of the output would stay unwritten): the contents are checked once per index tensor (keyed on its storage
    and version, so an index built once per model costs one check)."""
    if index.dtype != torch.int32 or index.dim() != 1 or index.numel() != L:
        raise ValueError("index must be a 1-D int32 tensor with one entry per token (%d)" % L)
    index = index.contiguous()
    if index.is_inference():  # no version counter to key a cached verdict on: checked on every call
        validate_token_index(index, L)
        return index
    key = (index.data_ptr(), index._version, L, index.device.index if index.device.index is not None else -1)
    if key not in _VALID_INDEX:
        validate_token_index(index, L)
        if len(_VALID_INDEX) > 64:
            _VALID_INDEX.clear()
        _VALID_INDEX[key] = True
    return index


def pool_kv_indexed(k: torch.Tensor, v: torch.Tensor, index: torch.Tensor, block_n: int):
    """pool_kv of the re-ordered K, V (position i = source row index[i]; index an int32 permutation of 0..L-1) without a
    gather pass of its own: returns (k_pool, v_pool, k_ord, v_ord), the last two being the re-ordered rows [B,H,L,D]."""
    _require_gpu(k, v, index)
    k, v = _same_type(_kernel_view(k), _kernel_view(v))
    B, H, L, D = k.shape
    if v.shape != k.shape:
        raise ValueError("k and v must have the same shape")
    index = _check_index(index, L)
    n = lib.psa_pool_elems(B, H, L, D, block_n)
    kp = torch.empty(n, dtype=k.dtype, device=k.device)
    vp = torch.empty(n, dtype=k.dtype, device=k.device)
    ko, vo = torch.empty_like(k, memory_format=torch.contiguous_format), torch.empty_like(v, memory_format=torch.contiguous_format)
    with torch.cuda.device(k.device):
        check(lib.psa_pool_kv_indexed(_t4(k), _t4(v), _ptr(index), _t4(ko), _t4(vo), _ptr(kp), _ptr(vp), B, H, L, D, block_n,
                                      _stream(k)), "psa_pool_kv_indexed")
    return kp, vp, ko, vo


def pool_levels(pool: torch.Tensor, B: int, H: int, L: int, D: int, block_n: int) -> Dict[int, torch.Tensor]:
    """Views [B,H,Npad/l,D] of the levels inside a pooled buffer."""
    npad = -(-L // block_n) * block_n
    out = {}
    for lv in (2, 4, 8):
        off = lib.psa_pool_level_offset(B, H, L, D, block_n, lv)
        n = B * H * (npad // lv) * D
        out[lv] = pool[off:off + n].view(B, H, npad // lv, D)
    return out


# ----------------------------------------------------------------------------- estimator
_DRAWS = [0]


def draw_sample_offsets(B: int, Hq: int, Hkv: int, block_m: int, keep_m: int, block_n: int, keep_n: int, device,
                        seed: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """(off_q [B,Hq,keep_m], off_k [B,Hkv,keep_n]) int32, drawn on the device in one launch (no host round trip): per
    (b, h) `keep` distinct in-block offsets, the same for every block of the head.  seed None: a new draw per call,
    derived from torch's seed (torch.manual_seed makes a run reproducible) and a call counter."""
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("psa_hip operators run on the GPU only; there is no CPU path")
    if seed is None:
        _DRAWS[0] += 1
        seed = (torch.initial_seed() * 0x9E3779B97F4A7C15 + _DRAWS[0]) & 0xFFFFFFFFFFFFFFFF
    off_q = torch.empty(B, Hq, keep_m, dtype=torch.int32, device=device)
    off_k = torch.empty(B, Hkv, keep_n, dtype=torch.int32, device=device)
    with torch.cuda.device(device):
        check(lib.psa_draw_sample_offsets(_ptr(off_q), _ptr(off_k), B * Hq, B * Hkv, block_m, keep_m, block_n, keep_n,
                                          int(seed) & 0xFFFFFFFFFFFFFFFF, _stream(off_q)), "psa_draw_sample_offsets")
    return off_q, off_k


def estimate_sampled(
    q: torch.Tensor,
    k: torch.Tensor,
    off_q: Optional[torch.Tensor],
    off_k: Optional[torch.Tensor],
    block_m: int,
    block_n: int,
    keep_m: int,
    keep_n: int,
    sm_scale: Optional[float] = None,
    out_rows: Optional[int] = None,
    out_cols: Optional[int] = None,
    q_index: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """fp32 block-importance scores [B,Hq,out_rows,out_cols]; off_* int32 [B,H,keep] in-block offsets
    (None: rows are taken as 0..keep-1 of each block).  q_index (int32 permutation [Lq]): query position i is row
    q_index[i] of q (token re-ordering read on the fly; k is passed already re-ordered)."""
    _require_gpu(q, k, off_q, off_k, q_index)
    q, k = _same_type(_kernel_view(q), _kernel_view(k))
    B, Hq, Lq, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    sm_scale = D ** -0.5 if sm_scale is None else sm_scale
    Mq, Nk = -(-Lq // block_m), -(-Lk // block_n)
    out_rows = Mq if out_rows is None else out_rows
    out_cols = Nk if out_cols is None else out_cols
    for o, H, keep in ((off_q, Hq, keep_m), (off_k, Hkv, keep_n)):
        if o is not None and (o.dtype != torch.int32 or tuple(o.shape) != (B, H, keep) or not o.is_contiguous()):
            raise ValueError("sample offsets must be contiguous int32 [B, H, keep]")
    scores = torch.empty(B, Hq, out_rows, out_cols, dtype=torch.float32, device=q.device)
    ws = torch.empty(lib.psa_estimate_workspace_bytes(B, Hq, Lq, Lk, block_m, block_n, keep_m, keep_n), dtype=torch.uint8, device=q.device)
    tail = (_ptr(off_q), _ptr(off_k), _ptr(scores), _ptr(ws), B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n, float(sm_scale),
            out_rows, out_cols, _stream(q))
    with torch.cuda.device(q.device):
        if q_index is None:
            check(lib.psa_estimate_sampled(_t4(q), _t4(k), *tail), "psa_estimate_sampled")
        else:
            check(lib.psa_estimate_sampled_indexed(_t4(q), _ptr(_check_index(q_index, Lq)), _t4(k), *tail),
                  "psa_estimate_sampled_indexed")
    return scores


def estimate_sampled_map(
    q: torch.Tensor,
    k: torch.Tensor,
    off_q: Optional[torch.Tensor],
    off_k: Optional[torch.Tensor],
    block_m: int,
    block_n: int,
    keep_m: int,
    keep_n: int,
    mask_ratios,
    text_length: int = 226,
    mode: str = "topk",
    min_full_attn_ratio: float = 0.06,
    compute_tile: int = 32,
    map_dtype: torch.dtype = torch.int32,
    sm_scale: Optional[float] = None,
    return_scores: bool = False,
    q_index: Optional[torch.Tensor] = None,
):
    """estimate_sampled + level_map (dense map modes, blocksize = block_n) with the map taken from each row of
    scores while it is still on chip: the same map, bit for bit, in two launches instead of three.  Returns the
    map, or (scores, map) with return_scores."""
    items, m, newtype = _items(mask_ratios, mode)
    if newtype:
        raise ValueError("the fused estimator writes dense maps only")
    if map_dtype not in (torch.int8, torch.int32):
        raise ValueError("map_dtype must be int8 or int32")
    _require_gpu(q, k, off_q, off_k, q_index)
    q, k = _same_type(_kernel_view(q), _kernel_view(k))
    B, Hq, Lq, D = q.shape
    Hkv, Lk = k.shape[1], k.shape[2]
    sm_scale = D ** -0.5 if sm_scale is None else sm_scale
    Mq, Nk = -(-Lq // block_m), -(-Lk // block_n)
    for o, H, keep in ((off_q, Hq, keep_m), (off_k, Hkv, keep_n)):
        if o is not None and (o.dtype != torch.int32 or tuple(o.shape) != (B, H, keep) or not o.is_contiguous()):
            raise ValueError("sample offsets must be contiguous int32 [B, H, keep]")
    div = block_n // compute_tile
    if div < 1:
        raise ValueError("compute_tile must not exceed blocksize")
    n = len(items)
    lv = (ctypes.c_int32 * n)(*[int(i[0]) for i in items])
    hi = (ctypes.c_double * n)(*[float(i[1][1]) for i in items])
    tb = (text_length + block_n - 1) // block_n if text_length > 0 else 0
    # (maps wider than about 5000 columns do not fit the fused kernel's LDS: the library then needs the scores buffer)
    scores = torch.empty(B, Hq, Mq, Nk, dtype=torch.float32, device=q.device) if (return_scores or Nk > 4096) else None
    out = torch.empty(B, Hq, Mq, Nk, dtype=map_dtype, device=q.device)
    ws = torch.empty(lib.psa_estimate_workspace_bytes(B, Hq, Lq, Lk, block_m, block_n, keep_m, keep_n), dtype=torch.uint8, device=q.device)
    tail = (_ptr(off_q), _ptr(off_k), _ptr(scores), _ptr(ws), B, Hq, Hkv, Lq, Lk, D, block_m, block_n, keep_m, keep_n, float(sm_scale),
            Mq, Nk, _ptr(out), out.element_size(), m, n, lv, hi, div, tb, float(min_full_attn_ratio), _stream(q))
    with torch.cuda.device(q.device):
        if q_index is None:
            check(lib.psa_estimate_sampled_map(_t4(q), _t4(k), *tail), "psa_estimate_sampled_map")
        else:
            check(lib.psa_estimate_sampled_map_indexed(_t4(q), _ptr(_check_index(q_index, Lq)), _t4(k), *tail),
                  "psa_estimate_sampled_map_indexed")
    return (scores, out) if return_scores else out


# ----------------------------------------------------------------------------- level map
def _items(mask_ratios, mode: str):
    if mask_ratios is None:
        raise ValueError("mask_ratios must be provided")
    newtype = mode.endswith("_newtype")
    base = mode[: -len("_newtype")] if newtype else mode
    if base == "topk":
        items = list(mask_ratios.items())
        m = _lib.PSA_MODE_TOPK
    elif base == "thresholdbound":
        items = sorted(mask_ratios.items(), key=lambda x: x[1][1])
        m = _lib.PSA_MODE_THRESHOLDBOUND
    else:
        raise ValueError(f"Unknown mode: {mode}. Must be 'topk' or 'thresholdbound'")
    if len(items) > _lib.PSA_MAX_LEVEL_ITEMS:
        raise ValueError("at most %d mask_ratios entries" % _lib.PSA_MAX_LEVEL_ITEMS)
    return items, m, newtype


def level_map(
    scores: torch.Tensor,
    mask_ratios,
    text_length: int = 226,
    mode: str = "topk",
    min_full_attn_ratio: float = 0.06,
    blocksize: int = 32,
    compute_tile: int = 32,
    map_dtype: torch.dtype = torch.int32,
) -> torch.Tensor:
    """Scores [B,H,Mq,Nk] -> level map (dense modes, `map_dtype` int8/int32) or int32 index list
    (`*_newtype` modes)."""
    items, m, newtype = _items(mask_ratios, mode)
    _require_gpu(scores)
    if scores.dim() != 4:
        raise ValueError("scores must be [B, H, Mq, Nk]")
    s = scores.to(torch.float32).contiguous()
    B, H, Mq, Nk = s.shape
    n = len(items)
    lv = (ctypes.c_int32 * n)(*[int(i[0]) for i in items])
    hi = (ctypes.c_double * n)(*[float(i[1][1]) for i in items])
    rows = B * H * Mq
    div = blocksize // compute_tile
    if div < 1:
        raise ValueError("compute_tile must not exceed blocksize")
    with torch.cuda.device(s.device):
        if newtype:
            out = torch.empty(B, H, Mq, Nk + n, dtype=torch.int32, device=s.device)
            rc = lib.psa_level_map(_ptr(s), None, 4, _ptr(out), rows, Nk, m, n, lv, hi, div, 0, float(min_full_attn_ratio), _stream(s))
        else:
            if map_dtype not in (torch.int8, torch.int32):
                raise ValueError("map_dtype must be int8 or int32")
            out = torch.empty(B, H, Mq, Nk, dtype=map_dtype, device=s.device)
            tb = (text_length + blocksize - 1) // blocksize if text_length > 0 else 0
            rc = lib.psa_level_map(_ptr(s), _ptr(out), out.element_size(), None, rows, Nk, m, n, lv, hi, div, tb,
                                   float(min_full_attn_ratio), _stream(s))
    check(rc, "psa_level_map")
    return out


def level_map_qwen(scores: torch.Tensor, mask_ratios, text_length: int, mode: str, *, block_size: int, causal: bool,
                   map_dtype: torch.dtype = torch.int32) -> torch.Tensor:
    """Square causal level map of the Qwen2.5-VL example: scores [B,H,S,S] -> map [B,H,S,S]."""
    if not mask_ratios:
        raise ValueError("mask_ratios must not be empty")
    if mode not in {"topk", "energybound"}:
        raise ValueError("mode must be 'topk' or 'energybound'")
    _require_gpu(scores)
    s = scores.to(torch.float32).contiguous()
    B, H, S, S2 = s.shape
    if S != S2:
        raise ValueError("scores must be square [B, H, S, S]")
    items = list(mask_ratios.items())
    n = len(items)
    lv = (ctypes.c_int32 * n)(*[int(i[0]) for i in items])
    lo = (ctypes.c_double * n)(*[float(i[1][0]) for i in items])
    hi = (ctypes.c_double * n)(*[float(i[1][1]) for i in items])
    special = min(-(-text_length // block_size) if text_length > 0 else 0, S)
    out = torch.empty(B, H, S, S, dtype=map_dtype, device=s.device)
    m = _lib.PSA_MODE_TOPK if mode == "topk" else _lib.PSA_MODE_THRESHOLDBOUND
    with torch.cuda.device(s.device):
        check(lib.psa_level_map_qwen(_ptr(s), _ptr(out), out.element_size(), B * H, S, m, n, lv, lo, hi, special, int(causal), _stream(s)),
              "psa_level_map_qwen")
    return out


def estimate_xattn(q: torch.Tensor, k: torch.Tensor, block_size: int = 128, stride: int = 8, causal: bool = True,
                   chunk_size: int = 4096) -> torch.Tensor:
    """Antidiagonal block-importance estimate, fp32 [B,Hq,ceil(Lq/block),ceil(Lk/block)]."""
    _require_gpu(q, k)
    qb, kb = _bf16_view(q), _bf16_view(k)
    B, Hq, Lq, D = qb.shape
    Hkv, Lk = kb.shape[1], kb.shape[2]
    est = torch.empty(B, Hq, -(-Lq // block_size), -(-Lk // block_size), dtype=torch.float32, device=q.device)
    ws = torch.empty(lib.psa_estimate_xattn_workspace_bytes(B, Hq, Lq, Lk, block_size, stride, chunk_size), dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        check(lib.psa_estimate_xattn(_t4(qb), _t4(kb), _ptr(est), _ptr(ws), B, Hq, Hkv, Lq, Lk, D, block_size, stride, chunk_size,
                                     int(causal), _stream(q)), "psa_estimate_xattn")
    return est


def gather_rows(tensors: Sequence[torch.Tensor], index: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """out[t][b, h, i, :] = tensors[t][b, h, index[i], :] for up to three [B, H, L, D] tensors of one dtype
    (2- or 4-byte elements, D contiguous) that share the int32 index vector: the token re-ordering of
    GilbertRearranger (reference utils/rearranger.py:14-132) in one launch instead of index_select + cat per tensor."""
    _require_gpu(*tensors, index)
    if not 1 <= len(tensors) <= 3:
        raise ValueError("gather_rows takes 1 to 3 tensors")
    t0 = tensors[0]
    B, _, L_src, D = t0.shape
    for t in tensors:
        if t.dim() != 4 or t.dtype != t0.dtype or t.shape[0] != B or t.shape[2] != L_src or t.shape[3] != D:
            raise ValueError("tensors must be [B, H, L, D] with the same dtype, B, L and D")
    if index.dtype != torch.int32 or index.dim() != 1:
        raise ValueError("index must be a 1-D int32 tensor")
    index = index.contiguous()
    srcs = [t if t.stride(3) == 1 else t.contiguous() for t in tensors]
    L_dst = index.numel()
    outs = [torch.empty(B, t.shape[1], L_dst, D, dtype=t.dtype, device=t.device) for t in srcs]
    n = len(srcs)
    a_src = (Tensor4 * 3)(*[_t4(t) for t in srcs], *[_t4(srcs[0])] * (3 - n))
    a_dst = (Tensor4 * 3)(*[_t4(t) for t in outs], *[_t4(outs[0])] * (3 - n))
    heads = (ctypes.c_int * 3)(*[t.shape[1] for t in srcs], *[srcs[0].shape[1]] * (3 - n))
    with torch.cuda.device(t0.device):
        check(lib.psa_gather_rows(a_src, a_dst, heads, n, _ptr(index), B, L_dst, L_src, D, t0.element_size(), _stream(t0)),
              "psa_gather_rows")
    return tuple(outs)


def map_from_list(list_mask: torch.Tensor, Nk: int, map_dtype: torch.dtype = torch.int8) -> torch.Tensor:
    """Index list [..., W] int32 -> dense level map [..., Nk]."""
    _require_gpu(list_mask)
    lm = list_mask.to(torch.int32).contiguous()
    lead, W = lm.shape[:-1], lm.shape[-1]
    rows = lm.numel() // W
    out = torch.empty(*lead, Nk, dtype=map_dtype, device=lm.device)
    with torch.cuda.device(lm.device):
        check(lib.psa_map_from_list(_ptr(lm), _ptr(out), out.element_size(), rows, W, Nk, _stream(lm)), "psa_map_from_list")
    return out


def list_from_map(level_map_: torch.Tensor, blocksize: int = 32, compute_tile: int = 32) -> torch.Tensor:
    """Dense level map [..., Nk] (int8 / int32) -> index list [..., Nk + 5] int32 (levels 1, 2, 4, 8, skipped; -1 behind
    each segment; segment lengths rounded down to the level's alignment)."""
    _require_gpu(level_map_)
    m = level_map_ if level_map_.dtype in (torch.int8, torch.int32) else level_map_.to(torch.int32)
    m = m.contiguous()
    lead, Nk = m.shape[:-1], m.shape[-1]
    div = max(1, blocksize // compute_tile)
    out = torch.empty(*lead, Nk + 5, dtype=torch.int32, device=m.device)
    with torch.cuda.device(m.device):
        check(lib.psa_list_from_map(_ptr(m), m.element_size(), _ptr(out), m.numel() // Nk, Nk, div, _stream(m)), "psa_list_from_map")
    return out


def k_similarity(k: torch.Tensor, block_n: int, thr2: float, thr4: float, thr8: float) -> torch.Tensor:
    """Per kv-block cap on the pooling level, int32 [B,H,Nk] in {1,2,4,8}."""
    _require_gpu(k)
    kb = _kernel_view(k, _T16)
    B, H, L, D = kb.shape
    Nk = -(-L // block_n)
    out = torch.empty(B, H, Nk, dtype=torch.int32, device=k.device)
    with torch.cuda.device(k.device):
        check(lib.psa_ksim(_t4(kb), _ptr(out), B, H, L, D, block_n, float(thr2), float(thr4), float(thr8), _stream(k)), "psa_ksim")
    return out


def map_min_cap(level_map_: torch.Tensor, cap: torch.Tensor) -> torch.Tensor:
    """In place: map[b,h,i,j] = min(map[b,h,i,j], cap[b,h,j])."""
    _require_gpu(level_map_, cap)
    B, H, Mq, Nk = level_map_.shape
    if not level_map_.is_contiguous() or level_map_.dtype not in (torch.int8, torch.int32):
        raise ValueError("level map must be a contiguous int8/int32 tensor")
    cap = cap.to(torch.int32).contiguous()
    if tuple(cap.shape) != (B, H, Nk):
        raise ValueError("cap must be [B, H, Nk]")
    with torch.cuda.device(level_map_.device):
        check(lib.psa_map_min_cap(_ptr(level_map_), level_map_.element_size(), _ptr(cap), B * H, Mq, Nk, _stream(cap)), "psa_map_min_cap")
    return level_map_


def density(level_map_: torch.Tensor, causal: bool = False) -> torch.Tensor:
    """Device-side mean(1/level): returns a float32 tensor [B*H + 1] (per (b,h), then the overall
    mean) without synchronising the host."""
    _require_gpu(level_map_)
    m = level_map_.contiguous()
    B, H, Mq, Nk = m.shape
    out = torch.empty(B * H + 1, dtype=torch.float32, device=m.device)
    with torch.cuda.device(m.device):
        check(lib.psa_density(_ptr(m), m.element_size(), B * H, Mq, Nk, int(causal), _ptr(out), _stream(m)), "psa_density")
    return out


# ----------------------------------------------------------------------------- attention forward
def build_schedule(level_map_: torch.Tensor, Hkv: int, L: int, D: int, block_m: int, block_n: int, causal: bool = False,
                   out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Tile schedule of a level map [B, Hq, Mq, Nk] (int8 / int32): a uint8 buffer for sparse_attention_fwd(schedule=...).
    Exists for D = 64 or 128 and 128 x 128 blocks (ValueError otherwise)."""
    _require_gpu(level_map_)
    if level_map_.dtype not in (torch.int8, torch.int32) or not level_map_.is_contiguous():
        raise ValueError("level map must be a contiguous int8/int32 tensor")
    B, Hq, Mq, Nk = level_map_.shape
    if Mq != -(-L // block_m) or Nk != -(-L // block_n):
        raise ValueError("level map shape does not match L and the block sizes")
    n = lib.psa_schedule_bytes(B, Hq, Hkv, L, D, block_m, block_n)
    if n <= 0:
        raise ValueError("no tile schedule for D=%d, block_m=%d, block_n=%d" % (D, block_m, block_n))
    if out is None:
        out = torch.empty(n, dtype=torch.uint8, device=level_map_.device)
    elif out.dtype != torch.uint8 or out.numel() < n or not out.is_contiguous() or out.device != level_map_.device:
        raise ValueError("schedule buffer must be a contiguous uint8 tensor of at least %d bytes" % n)
    with torch.cuda.device(level_map_.device):
        check(lib.psa_build_schedule(_ptr(level_map_), level_map_.element_size(), _ptr(out), B, Hq, Hkv, L, D, block_m, block_n,
                                     int(causal), _stream(level_map_)), "psa_build_schedule")
    return out


def sparse_attention_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    level_map_: Optional[torch.Tensor],
    block_m: int,
    block_n: int,
    sm_scale: Optional[float] = None,
    causal: bool = False,
    return_lse: bool = False,
    pools: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
    out: Optional[torch.Tensor] = None,
    balance: bool = True,
    q_index: Optional[torch.Tensor] = None,
    schedule=None,
):
    """Pyramid sparse attention forward.  level_map_ None = dense attention.  Returns out (dtype and
    shape of q) or (out, lse fp32 [B,H,L], (k_pool, v_pool)).  balance=True issues the rows of the map
    longest first (same results, shorter tail).  q_index (int32 permutation [L]): k, v, the pools and the map are in
    the re-ordered token order, q is in the original order and read through the index (position i = row q_index[i]),
    and out / lse come back in the original order (row q_index[i] = result of position i).  schedule: a tile schedule
    built from level_map_ with build_schedule (reused across calls on the same map), None to build it here where the
    shape has one, False to walk the map itself."""
    _require_gpu(q, k, v, level_map_, q_index)
    in_dtype = q.dtype
    qb, kb, vb = _same_type(_kernel_view(q), _kernel_view(k), _kernel_view(v))
    B, Hq, L, D = qb.shape
    Hkv = kb.shape[1]
    if kb.shape[2] != L or vb.shape != kb.shape or kb.shape[3] != D:
        raise ValueError("q, k, v must share L and D; k and v must share their shape")
    sm_scale = D ** -0.5 if sm_scale is None else float(sm_scale)
    if not sm_scale > 0:
        raise ValueError("sm_scale must be positive")
    Mq, Nk = -(-L // block_m), -(-L // block_n)
    kp = vp = None
    if level_map_ is not None:
        if level_map_.dtype not in (torch.int8, torch.int32):
            level_map_ = level_map_.to(torch.int32)
        level_map_ = level_map_.contiguous()
        if tuple(level_map_.shape) != (B, Hq, Mq, Nk):
            raise ValueError("level map must be [B, Hq, %d, %d], got %s" % (Mq, Nk, tuple(level_map_.shape)))
        kp, vp = pools if pools is not None else pool_kv(kb, vb, block_n)
        if kp.dtype != kb.dtype or vp.dtype != kb.dtype:
            raise ValueError("the pooled buffers must have the element type of k / v (%s)" % kb.dtype)
    if out is None or out.dtype != qb.dtype:
        o = torch.empty(B, Hq, L, D, dtype=qb.dtype, device=q.device)
    else:
        o = out
    lse = torch.empty(B, Hq, L, dtype=torch.float32, device=q.device) if return_lse else None
    if q_index is not None:
        q_index = _check_index(q_index, L)
    n_sched = 0
    if level_map_ is not None and balance and schedule is not False and qb.dtype in _T16:
        n_sched = lib.psa_schedule_bytes(B, Hq, Hkv, L, D, block_m, block_n)
    if n_sched > 0:
        # the map's tile schedule is built once (one pass over the map) and walked by the kernel
        if not isinstance(schedule, torch.Tensor):
            schedule = build_schedule(level_map_, Hkv, L, D, block_m, block_n, causal)
        with torch.cuda.device(q.device):
            check(lib.psa_fwd_scheduled(_t4(qb), _ptr(q_index), _t4(kb), _t4(vb), _ptr(kp), _ptr(vp), _ptr(level_map_),
                                        level_map_.element_size(), _ptr(schedule), _t4(o), _ptr(lse), B, Hq, Hkv, L, D, block_m, block_n,
                                        sm_scale, int(causal), _stream(q)), "psa_fwd_scheduled")
    else:
        ws = None
        if level_map_ is not None and balance:
            ws = torch.empty(lib.psa_fwd_workspace_bytes(B, Hq, L, block_m) // 4, dtype=torch.int32, device=q.device)
        tail = (_t4(kb), _t4(vb), _ptr(kp), _ptr(vp), _ptr(level_map_), 1 if level_map_ is None else level_map_.element_size(), _t4(o),
                _ptr(lse), B, Hq, Hkv, L, D, block_m, block_n, sm_scale, int(causal), _ptr(ws), _stream(q))
        with torch.cuda.device(q.device):
            if q_index is None:
                check(lib.psa_fwd(_t4(qb), *tail), "psa_fwd")
            else:
                check(lib.psa_fwd_indexed(_t4(qb), _ptr(q_index), *tail), "psa_fwd_indexed")
    res = o if in_dtype == o.dtype else o.to(in_dtype)
    if return_lse:
        return res, lse, (kp, vp)
    return res


_SIDE_STREAMS: Dict[int, "torch.cuda.Stream"] = {}
# below this size of K the fork / join of the second stream costs more than the overlap gains (small layers are bound by
# launch latency: 0.07 ms against 0.13 ms with the fork at B1 H2 N4096 D64)
_SIDE_STREAM_MIN_BYTES = 16 << 20


def _side_stream(device: torch.device) -> "torch.cuda.Stream":
    """One extra stream per device (default priority) for work that does not depend on the main chain."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    if idx not in _SIDE_STREAMS:
        _SIDE_STREAMS[idx] = torch.cuda.Stream(device=idx)
    return _SIDE_STREAMS[idx]


# ----------------------------------------------------------------------------- whole layer, forward only
def psa_layer_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    off_q: torch.Tensor,
    off_k: torch.Tensor,
    mask_ratios,
    mode: str,
    block_m: int,
    block_n: int,
    tile_n: int,
    sm_scale: Optional[float] = None,
    level_cap: Optional[torch.Tensor] = None,
    return_map: bool = False,
    text_length: int = 0,
    token_index: Optional[torch.Tensor] = None,
    sim_thresholds: Optional[Tuple[float, float, float]] = None,
    return_cap: bool = False,
):
    """estimate (+ level map, in the estimator's reduction kernel) -> pooled K/V -> sparse attention, non-causal,
    no gradient, with a dense int8 level map in between (no index-list round trip).  The pooling pass (HBM-bound,
    independent of the estimate) runs on a second stream of default priority beside the estimator and joins the current
    stream before the attention kernel (worth 0.02 ms of 1.0 at the Wan2.1 shape), unless the layer is small.
    sim_thresholds (t2, t4, t8): the key-similarity cap is computed here, on the keys in the order the layer works in
    (after the re-ordering), and applied to the map; level_cap passes a ready cap instead.  Returns out, or
    (out[, map][, cap]) with return_map / return_cap."""
    _require_gpu(q, k, v)
    qb, kb, vb = _same_type(_kernel_view(q), _kernel_view(k), _kernel_view(v))
    keep_m, keep_n = block_m // 4, block_n // 4
    sm_scale = qb.shape[-1] ** -0.5 if sm_scale is None else float(sm_scale)
    if token_index is not None:
        # token re-ordering (int32 permutation: position i = source row token_index[i]) without gather passes: the pooling
        # pass reads K, V through the index and leaves the re-ordered rows behind, the estimator and the attention kernel
        # read Q through it, and the attention kernel writes its rows back to their original places
        kp, vp, kb, vb = pool_kv_indexed(kb, vb, token_index, block_n)
    side = None
    if token_index is None and kb.numel() * 2 >= _SIDE_STREAM_MIN_BYTES:
        # the buffers come from the current stream's allocator; the side stream only runs the kernel
        main = torch.cuda.current_stream(qb.device)
        side = _side_stream(qb.device)
        n_pool = lib.psa_pool_elems(kb.shape[0], kb.shape[1], kb.shape[2], kb.shape[3], block_n)
        kp = torch.empty(n_pool, dtype=kb.dtype, device=kb.device)
        vp = torch.empty(n_pool, dtype=kb.dtype, device=kb.device)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            pool_kv(kb, vb, block_n, out=(kp, vp))
    if sim_thresholds is not None:
        if level_cap is not None:
            raise ValueError("pass either level_cap or sim_thresholds")
        level_cap = k_similarity(kb, block_n, *sim_thresholds)
    mp = estimate_sampled_map(qb, kb, off_q, off_k, block_m, block_n, keep_m, keep_n, mask_ratios, text_length, mode,
                              compute_tile=tile_n, map_dtype=torch.int8, sm_scale=sm_scale, q_index=token_index)
    if level_cap is not None:
        mp = map_min_cap(mp, level_cap)
    if side is not None:
        main.wait_stream(side)
    elif token_index is None:
        kp, vp = pool_kv(kb, vb, block_n)
    out = sparse_attention_fwd(qb, kb, vb, mp, block_m, block_n, sm_scale, pools=(kp, vp), q_index=token_index)
    if out.dtype != q.dtype:
        out = out.to(q.dtype)
    if not (return_map or return_cap):
        return out
    return (out,) + ((mp,) if return_map else ()) + ((level_cap,) if return_cap else ())


# ----------------------------------------------------------------------------- whole layer as one HIP graph
_LAYER_GRAPHS: Dict[tuple, tuple] = {}
_LAYER_GRAPHS_MAX = 16


def psa_layer_fwd_graph(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, off_q: torch.Tensor, off_k: torch.Tensor, mask_ratios,
                        mode: str, block_m: int, block_n: int, tile_n: int, **kwargs):
    """psa_layer_fwd captured into one HIP graph and replayed: the estimator, the reduction + level map, the tile schedule
    and the attention kernel on the main branch, the pooling pass on a second branch beside the estimator - kernel nodes
    only (the library enqueues nothing else: no memset or copy nodes).  For callers that replay graphs anyway; on its own it
    is no faster than the eager operator, whose launches are enqueued far ahead of the GPU.  The graph is tied to the ADDRESSES of q, k, v and the offsets (and to every other
    argument): a call with tensors at the same addresses replays it on their current contents, any other call captures
    a new graph (a few are kept).  The returned tensors belong to the graph and are overwritten by its next replay.
    Same bits as psa_layer_fwd.  Keyword arguments as psa_layer_fwd (tensors among them are part of the key)."""
    _require_gpu(q, k, v, off_q, off_k)

    def keyof(x):
        if isinstance(x, torch.Tensor):
            return ("t", x.data_ptr(), tuple(x.shape), tuple(x.stride()), x.dtype)
        if isinstance(x, dict):
            return tuple(sorted((kk, keyof(vv)) for kk, vv in x.items()))
        if isinstance(x, (list, tuple)):
            return tuple(keyof(e) for e in x)
        return x

    key = (keyof((q, k, v, off_q, off_k)), keyof(mask_ratios), mode, block_m, block_n, tile_n, keyof(kwargs),
           torch.cuda.current_device())
    ent = _LAYER_GRAPHS.get(key)
    if ent is None:
        def run():
            return psa_layer_fwd(q, k, v, off_q, off_k, mask_ratios, mode, block_m, block_n, tile_n, **kwargs)

        # one eager run first (one-time work such as the check of a token index and the library's function attributes
        # must not fall into the capture), on a side stream as torch asks for
        cur = torch.cuda.current_stream(q.device)
        warm = torch.cuda.Stream(device=q.device)
        warm.wait_stream(cur)
        with torch.cuda.stream(warm):
            run()
        cur.wait_stream(warm)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            res = run()
        if len(_LAYER_GRAPHS) >= _LAYER_GRAPHS_MAX:
            _LAYER_GRAPHS.pop(next(iter(_LAYER_GRAPHS)))
        # (the key holds addresses only: keep the tensors alive with the graph so that the addresses stay theirs)
        ent = (graph, res, (q, k, v, off_q, off_k, kwargs))
        _LAYER_GRAPHS[key] = ent
    ent[0].replay()
    return ent[1]


# ----------------------------------------------------------------------------- attention backward
def sparse_attention_bwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    level_map_: Optional[torch.Tensor],
    out: torch.Tensor,
    dout: torch.Tensor,
    lse: torch.Tensor,
    block_m: int,
    block_n: int,
    sm_scale: Optional[float] = None,
    causal: bool = False,
    pools: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
):
    """dq, dk, dv of sparse_attention_fwd (dtype of q / k / v); lse is the fp32 [B,Hq,L] tensor the forward
    returned.  The level map carries no gradient.  bf16 and fp16 tensors are computed on in their own type (fp32
    accumulation); any other type is rounded to bf16 first."""
    _require_gpu(q, k, v, level_map_, out, dout, lse)
    qb, kb, vb, ob, dob = _same_type(*(_kernel_view(t, _T16) for t in (q, k, v, out, dout)))
    B, Hq, L, D = qb.shape
    Hkv = kb.shape[1]
    sm_scale = D ** -0.5 if sm_scale is None else float(sm_scale)
    Mq, Nk = -(-L // block_m), -(-L // block_n)
    kp = vp = None
    if level_map_ is not None:
        if level_map_.dtype not in (torch.int8, torch.int32):
            level_map_ = level_map_.to(torch.int32)
        level_map_ = level_map_.contiguous()
        if tuple(level_map_.shape) != (B, Hq, Mq, Nk):
            raise ValueError("level map must be [B, Hq, %d, %d], got %s" % (Mq, Nk, tuple(level_map_.shape)))
        # (pools of a forward that ran in another element type are of no use to the kernels here)
        reuse = pools is not None and pools[0] is not None and pools[0].dtype == qb.dtype
        kp, vp = pools if reuse else pool_kv(kb, vb, block_n)
    lse = lse.to(torch.float32).contiguous()
    if tuple(lse.shape) != (B, Hq, L):
        raise ValueError("lse must be [B, Hq, L]")
    dq = torch.empty(B, Hq, L, D, dtype=qb.dtype, device=q.device)
    dk = torch.empty(B, Hkv, L, D, dtype=qb.dtype, device=q.device)
    dv = torch.empty(B, Hkv, L, D, dtype=qb.dtype, device=q.device)
    ws = torch.empty(lib.psa_bwd_workspace_bytes(B, Hq, Hkv, L, D, block_n), dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        check(
            lib.psa_bwd(_t4(qb), _t4(kb), _t4(vb), _ptr(kp), _ptr(vp), _ptr(level_map_),
                        1 if level_map_ is None else level_map_.element_size(), _t4(ob), _t4(dob), _ptr(lse), _t4(dq), _t4(dk), _t4(dv),
                        _ptr(ws), B, Hq, Hkv, L, D, block_m, block_n, sm_scale, int(causal), _stream(q)),
            "psa_bwd",
        )
    return dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype)
