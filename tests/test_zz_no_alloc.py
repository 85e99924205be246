"""The allocation-free forward entry point (psa_fwd_noalloc) against the forward operator, through the C ABI: two calls
in a row, the second on a smaller input, each bit-identical to the existing entry point (the row-ordering scratch in
the library's own device array instead of a caller workspace); the driver's free-memory figure does not move across a
call; and the call can be captured into a HIP graph and replayed."""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import dev, random_map, rnd

pytestmark = pytest.mark.gpu


def _call_pair(B, Hq, Hkv, L, D, bm, bn, causal, seed):
    from psa_hip import ops
    from psa_hip._lib import Tensor4, check, lib

    Mq, Nk = -(-L // bm), -(-L // bn)
    assert B * Hq * Mq > 8 * 32  # large enough for the row-ordering kernels (the users of the scratch) to run
    rng = np.random.default_rng(seed)
    lmap = random_map(B, Hq, Mq, Nk, seed)
    keep = rng.random((B, Hq, Mq, 1)) ** 2  # strongly uneven rows, so that the issue order matters
    lmap = np.where(rng.random(lmap.shape) < keep, lmap, 0).astype(np.int8)
    if causal:
        lmap[..., np.arange(Mq), np.arange(Mq)] = 1
    q, k, v = rnd(B, Hq, L, D, seed=seed).to(dev()), rnd(B, Hkv, L, D, seed=seed + 1).to(dev()), rnd(B, Hkv, L, D, seed=seed + 2).to(dev())
    m = torch.from_numpy(lmap).to(dev())
    kp, vp = ops.pool_kv(k, v, bn)
    # the existing entry point, with a caller workspace
    ref_o = torch.full((B, Hq, L, D), float("nan"), dtype=torch.bfloat16, device=dev())
    ref, ref_lse, _ = ops.sparse_attention_fwd(q, k, v, m, bm, bn, causal=causal, return_lse=True, pools=(kp, vp), out=ref_o)
    # the new one: every buffer is allocated here, before the call
    out = torch.full((B, Hq, L, D), float("nan"), dtype=torch.bfloat16, device=dev())
    lse = torch.full((B, Hq, L), float("nan"), dtype=torch.float32, device=dev())
    t4 = lambda x: Tensor4(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2))
    p = lambda x: ctypes.c_void_p(x.data_ptr())

    def call():
        return lib.psa_fwd_noalloc(t4(q), t4(k), t4(v), p(kp), p(vp), p(m), 1, t4(out), p(lse), B, Hq, Hkv, L, D, bm, bn,
                                   float(D ** -0.5), int(causal), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))

    # one warm call (the library looks its scratch array's address up once per device), then the measured one: the
    # driver's own count of free device memory - which any hipMalloc would lower, inside the library as well as
    # in torch - is the same before and after
    check(call(), "psa_fwd_noalloc")
    torch.cuda.synchronize()
    out.fill_(float("nan"))
    lse.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    check(call(), "psa_fwd_noalloc")
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert not torch.isnan(out).any() and not torch.isnan(lse).any()
    assert torch.equal(out, ref) and torch.equal(lse, ref_lse)
    return call, out, lse, ref, ref_lse


def test_noalloc_forward_two_calls_second_smaller():
    _call_pair(1, 5, 5, 128 * 67 + 40, 128, 128, 128, False, 3)   # 340 rows of the map
    _call_pair(1, 4, 2, 128 * 66, 128, 128, 128, True, 4)          # 264 rows: smaller, causal, grouped heads
    _call_pair(2, 3, 3, 128 * 50 + 7, 64, 128, 128, False, 5)      # the one-row kernel (head dim 64), 306 rows


def test_noalloc_forward_under_graph_capture():
    """What the entry point is for: captured into a HIP graph (only kernel nodes: nothing is allocated or cleared inside
    the call) and replayed several times with eager work in between; every replay gives the eager bits."""
    call, out, lse, ref, ref_lse = _call_pair(1, 5, 5, 128 * 67 + 40, 128, 128, 128, False, 7)
    from psa_hip._lib import check

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            check(call(), "psa_fwd_noalloc (captured)")
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        out.fill_(float("nan"))
        lse.fill_(float("nan"))
        junk = torch.randn(1 << 20, device=dev()).sum()  # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref) and torch.equal(lse, ref_lse), rep
        assert torch.isfinite(junk)


def test_noalloc_forward_rejects_oversized_shapes():
    from psa_hip._lib import Tensor4, lib

    assert lib.psa_fwd_noalloc_max_rows() == 65536
    z = Tensor4(1 << 20, 8, 8, 8)
    one = ctypes.c_void_p(1 << 20)
    # 70000 rows of the level map: refused before anything is launched or dereferenced
    rc = lib.psa_fwd_noalloc(z, z, z, one, one, one, 1, z, None, 1, 70000, 70000, 128, 128, 128, 128, 0.1, 0, None)
    assert rc == -2 and b"exceed" in lib.psa_last_error()
