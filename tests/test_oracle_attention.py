"""Pins the oracle's pooling, estimator, attention forward and backward with closed
forms: special cases that reduce to torch's SDPA, brute force on tiny inputs and
finite differences."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import psa_oracle as O

torch.manual_seed(0)


def rnd(*shape, dtype=torch.float64, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float64).to(dtype)


# ---------------------------------------------------------------- pooling
@pytest.mark.parametrize("L,bn", [(256, 128), (250, 128), (77, 32), (129, 64)])
def test_pool_closed_form_and_torch_mean_chain(L, bn):
    x = rnd(2, 3, L, 16, dtype=torch.bfloat16, seed=L)
    lv = O.pool_kv(x, bn)
    Lp = -(-L // bn) * bn
    assert lv[1] is x
    for l in (2, 4, 8):
        assert lv[l].shape == (2, 3, Lp // l, 16) and lv[l].dtype == torch.bfloat16
        direct = O.pool_kv_direct(x, bn, l)
        # <= 1 bf16 ulp per chained rounding step away from the exact mean
        assert (lv[l].double() - direct).abs().max() <= 3 * 2.0 ** -8 * direct.abs().max()
    # bit-equal to what torch.mean does when chained in bf16 (the library op the reference calls)
    xp = O.pad_replicate(x, bn)
    t2 = xp.view(2, 3, -1, 2, 16).mean(3)
    t4 = t2.view(2, 3, -1, 2, 16).mean(3)
    t8 = t4.view(2, 3, -1, 2, 16).mean(3)
    assert torch.equal(lv[2], t2) and torch.equal(lv[4], t4) and torch.equal(lv[8], t8)
    # replicate padding: the last pooled rows only see the last token
    if L % bn and (Lp - L) >= 8:
        assert torch.equal(lv[8][:, :, -1], x[:, :, -1])


# ---------------------------------------------------------------- estimator
def brute_estimate(sq, sk, scale, km, kn):
    B, H, Ms, D = sq.shape
    Ns = sk.shape[2]
    out = np.zeros((B, H, Ms // km, Ns // kn))
    c = scale * 1.44269504
    for b in range(B):
        for h in range(H):
            S = sq[b, h].double().numpy() @ sk[b, h].double().numpy().T
            R = np.zeros((Ms, Ns // kn))
            for r in range(Ms):
                for j in range(Ns // kn):
                    R[r, j] = S[r, j * kn:(j + 1) * kn].max() * c
            E = 2.0 ** (R - R.max(1, keepdims=True))
            for i in range(Ms // km):
                out[b, h, i] = E[i * km:(i + 1) * km].max(0)
            out[b, h] /= out[b, h].sum(1, keepdims=True)
    return out


def test_estimator_brute_force():
    sq, sk = rnd(1, 2, 64, 16, dtype=torch.float32, seed=1), rnd(1, 2, 128, 16, dtype=torch.float32, seed=2)
    po = O.estimate_from_sampled(sq, sk, 0.25, 8, 16)
    assert po.shape == (1, 2, 8, 8)
    np.testing.assert_allclose(po.numpy(), brute_estimate(sq, sk, 0.25, 8, 16), rtol=2e-5)
    np.testing.assert_allclose(po.sum(-1).numpy(), 1.0, rtol=1e-5)


def test_estimator_padding_groups_enter_row_sum():
    # 3 q-blocks of keep 16 -> 48 rows -> padded to 64: one extra q-group; keys 5*8=40 -> 64: 3 extra groups
    sq, sk = rnd(1, 1, 48, 8, dtype=torch.float32, seed=3), rnd(1, 1, 40, 8, dtype=torch.float32, seed=4)
    po = O.estimate_from_sampled(sq, sk, 0.3, 16, 8)
    assert po.shape == (1, 1, 4, 8)
    sqp = torch.cat([sq, sq[:, :, -1:].expand(-1, -1, 16, -1)], 2)
    skp = torch.cat([sk, sk[:, :, -1:].expand(-1, -1, 24, -1)], 2)
    np.testing.assert_allclose(po.numpy(), brute_estimate(sqp, skp, 0.3, 16, 8), rtol=2e-5)


def test_estimator_uniform_logits_and_full_pipeline():
    q = torch.zeros(1, 1, 256, 8)
    k = rnd(1, 1, 256, 8, dtype=torch.float32, seed=5)
    g = torch.Generator().manual_seed(0)
    oq, ok = O.sample_offsets(1, 1, 64, 16, g), O.sample_offsets(1, 1, 64, 16, g)
    assert oq.shape == (1, 1, 16) and len(set(oq.view(-1).tolist())) == 16 and int(oq.max()) < 64
    po = O.estimate_sampled(q, k, 64, 64, oq, ok)
    np.testing.assert_allclose(po.numpy(), 0.25, rtol=1e-6)
    # gather picks rows blk*block + off of the replicate-padded tensor
    x = torch.arange(100.0).view(1, 1, 100, 1)
    s = O.gather_samples(x, 64, torch.tensor([[[3, 60]]], dtype=torch.int32))
    assert s.view(-1).tolist() == [3.0, 60.0, 67.0, 99.0]


# ---------------------------------------------------------------- attention closed forms
def sdpa(q, k, v, **kw):
    return F.scaled_dot_product_attention(q, k, v, **kw)


@pytest.mark.parametrize("L", [256, 200])
def test_all_level1_is_sdpa(L):
    q, k, v = rnd(1, 2, L, 16, seed=1), rnd(1, 2, L, 16, seed=2), rnd(1, 2, L, 16, seed=3)
    lm = np.ones((1, 2, -(-L // 64), -(-L // 64)), np.int32)
    for fn in (O.psa_attention_dense, O.psa_attention_blockwalk):
        out, lse = fn(q, k, v, lm, 64, 64, dtype=torch.float64)
        torch.testing.assert_close(out, sdpa(q, k, v), rtol=1e-9, atol=1e-9)
        ref_lse = torch.logsumexp(q @ k.transpose(-1, -2) / 4.0, -1)
        torch.testing.assert_close(lse, ref_lse, rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("lv", [2, 4, 8])
def test_uniform_level_is_sdpa_on_repeated_pooled(lv):
    L = 256
    q, k, v = rnd(1, 1, L, 8, seed=4), rnd(1, 1, L, 8, seed=5), rnd(1, 1, L, 8, seed=6)
    lm = np.full((1, 1, 4, 4), lv, np.int32)
    kp, vp = O.pool_kv_direct(k, 64, lv), O.pool_kv_direct(v, 64, lv)
    levels_k = {1: k, 2: None, 4: None, 8: None}
    lk = {l: O.pool_kv_direct(k, 64, l) for l in (2, 4, 8)} | {1: k}
    lvv = {l: O.pool_kv_direct(v, 64, l) for l in (2, 4, 8)} | {1: v}
    out, _ = O.psa_attention_dense(q, k, v, lm, 64, 64, levels_k=lk, levels_v=lvv)
    ref = sdpa(q, kp.repeat_interleave(lv, 2), vp.repeat_interleave(lv, 2))
    torch.testing.assert_close(out, ref, rtol=1e-9, atol=1e-9)


def test_lossless_pooling_any_map_is_sdpa():
    L, D = 512, 8
    base_k, base_v = rnd(1, 2, L // 8, D, seed=7), rnd(1, 2, L // 8, D, seed=8)
    k, v = base_k.repeat_interleave(8, 2), base_v.repeat_interleave(8, 2)
    q = rnd(1, 2, L, D, seed=9)
    rng = np.random.default_rng(0)
    lm = rng.choice([1, 2, 4, 8], size=(1, 2, 4, 8)).astype(np.int32)
    for fn in (O.psa_attention_dense, O.psa_attention_blockwalk):
        out, _ = fn(q, k, v, lm, 128, 64, dtype=torch.float64)
        torch.testing.assert_close(out, sdpa(q, k, v), rtol=1e-9, atol=1e-9)


def test_single_block_and_skips_and_empty_rows():
    L, D = 256, 8
    q, k, v = rnd(1, 1, L, D, seed=10), rnd(1, 1, L, D, seed=11), rnd(1, 1, L, D, seed=12)
    lm = np.zeros((1, 1, 4, 4), np.int32)
    lm[0, 0, 0, 2] = 1
    lm[0, 0, 1, 1] = 4
    out, lse = O.psa_attention_dense(q, k, v, lm, 64, 64)
    ref0 = torch.softmax(q[0, 0, :64] @ k[0, 0, 128:192].T / math.sqrt(D), -1) @ v[0, 0, 128:192]
    torch.testing.assert_close(out[0, 0, :64], ref0, rtol=1e-9, atol=1e-9)
    k4, v4 = O.pool_kv_direct(k, 64, 4)[0, 0, 16:32], O.pool_kv_direct(v, 64, 4)[0, 0, 16:32]
    lk = {l: O.pool_kv_direct(k, 64, l) for l in (2, 4, 8)} | {1: k}
    lvv = {l: O.pool_kv_direct(v, 64, l) for l in (2, 4, 8)} | {1: v}
    out, lse = O.psa_attention_dense(q, k, v, lm, 64, 64, levels_k=lk, levels_v=lvv)
    ref1 = torch.softmax(q[0, 0, 64:128] @ k4.T / math.sqrt(D), -1) @ v4
    torch.testing.assert_close(out[0, 0, 64:128], ref1, rtol=1e-9, atol=1e-9)
    assert torch.all(out[0, 0, 128:] == 0) and torch.all(torch.isinf(lse[0, 0, 128:]))
    ob, lb = O.psa_attention_blockwalk(q, k, v, lm, 64, 64, dtype=torch.float64)
    o2, l2 = O.psa_attention_dense(q, k, v, lm, 64, 64)
    torch.testing.assert_close(ob, o2, rtol=1e-9, atol=1e-9)
    torch.testing.assert_close(lb, l2, rtol=1e-9, atol=1e-9)


def test_causal_all1_is_causal_sdpa_and_pooled_visibility():
    L, D = 192, 8
    q, k, v = rnd(1, 2, L, D, seed=13), rnd(1, 2, L, D, seed=14), rnd(1, 2, L, D, seed=15)
    lm = np.tril(np.ones((3, 3), np.int32)).reshape(1, 1, 3, 3).repeat(2, 1)
    for fn in (O.psa_attention_dense, O.psa_attention_blockwalk):
        out, _ = fn(q, k, v, lm, 64, 64, causal=True, dtype=torch.float64)
        torch.testing.assert_close(out, sdpa(q, k, v, is_causal=True), rtol=1e-9, atol=1e-9)
    # an upper-triangle entry is never visited even if the map says so
    lm2 = np.ones((1, 2, 3, 3), np.int32)
    out2, _ = O.psa_attention_dense(q, k, v, lm2, 64, 64, causal=True)
    torch.testing.assert_close(out2, sdpa(q, k, v, is_causal=True), rtol=1e-9, atol=1e-9)
    # diagonal block at level 4: pooled key t visible iff 4t+3 <= i
    lm3 = np.array([[[[4]]]], np.int32)
    q1, k1, v1 = q[:, :1, :64], k[:, :1, :64], v[:, :1, :64]
    out3, _ = O.psa_attention_dense(q1, k1, v1, lm3, 64, 64, causal=True)
    k4, v4 = O.pool_kv(k1, 64)[4][0, 0], O.pool_kv(v1, 64)[4][0, 0]
    i = 10  # sees pooled keys 0,1 (4t+3 <= 10)
    ref = torch.softmax(q1[0, 0, i] @ k4[:2].T / math.sqrt(D), -1) @ v4[:2]
    torch.testing.assert_close(out3[0, 0, i], ref, rtol=1e-9, atol=1e-9)
    assert torch.all(out3[0, 0, :3] == 0)  # rows 0..2 see no pooled key
    ob, _ = O.psa_attention_blockwalk(q1, k1, v1, lm3, 64, 64, causal=True, dtype=torch.float64)
    torch.testing.assert_close(ob, out3, rtol=1e-9, atol=1e-9)


def test_gqa_maps_q_head_to_kv_head():
    L, D = 128, 8
    q, k, v = rnd(1, 4, L, D, seed=16), rnd(1, 2, L, D, seed=17), rnd(1, 2, L, D, seed=18)
    lm = np.ones((1, 4, 2, 2), np.int32)
    out, _ = O.psa_attention_dense(q, k, v, lm, 64, 64)
    ref = sdpa(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1))
    torch.testing.assert_close(out, ref, rtol=1e-9, atol=1e-9)
    ob, _ = O.psa_attention_blockwalk(q, k, v, lm, 64, 64, dtype=torch.float64)
    torch.testing.assert_close(ob, ref, rtol=1e-9, atol=1e-9)


# ---------------------------------------------------------------- backward
def test_backward_all1_matches_sdpa_autograd():
    L, D = 128, 8
    q, k, v, do = (rnd(1, 2, L, D, seed=s) for s in (20, 21, 22, 23))
    lm = np.ones((1, 2, 2, 2), np.int32)
    dq, dk, dv = O.psa_backward_dense(q, k, v, lm, do, 64, 64)
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    sdpa(qq, kk, vv).backward(do)
    for a, b in ((dq, qq.grad), (dk, kk.grad), (dv, vv.grad)):
        torch.testing.assert_close(a, b, rtol=1e-8, atol=1e-10)


def test_backward_lossless_pooling_splits_evenly_and_pad_folds_into_last_token():
    L, D = 120, 4  # padded to 128: the 8 pad rows replicate token 119
    base_k, base_v = rnd(1, 1, 15, D, seed=24), rnd(1, 1, 15, D, seed=25)
    k, v = base_k.repeat_interleave(8, 2), base_v.repeat_interleave(8, 2)
    q, do = rnd(1, 1, L, D, seed=26), rnd(1, 1, L, D, seed=27)
    lm = np.array([[[[8, 2], [4, 8]]]], np.int32)
    dq, dk, dv = O.psa_backward_dense(q, k, v, lm, do, 64, 64)
    # forward equals attention over 16 group keys (15 real + 1 all-pad copy of the last) with weight 8 each
    bk = torch.cat([base_k, base_k[:, :, -1:]], 2).clone().requires_grad_(True)
    bv = torch.cat([base_v, base_v[:, :, -1:]], 2).clone().requires_grad_(True)
    qq = q.clone().requires_grad_(True)
    sdpa(qq, bk, bv).backward(do)
    torch.testing.assert_close(dq, qq.grad, rtol=1e-8, atol=1e-10)
    gk = bk.grad / 8
    exp_dk = gk[:, :, :15].repeat_interleave(8, 2).clone()
    exp_dk[:, :, -1] += 8 * gk[:, :, 15]  # eight pad rows fold into token 119
    torch.testing.assert_close(dk, exp_dk, rtol=1e-8, atol=1e-10)
    gv = bv.grad / 8
    exp_dv = gv[:, :, :15].repeat_interleave(8, 2).clone()
    exp_dv[:, :, -1] += 8 * gv[:, :, 15]
    torch.testing.assert_close(dv, exp_dv, rtol=1e-8, atol=1e-10)


def test_backward_finite_difference_mixed_map():
    L, D = 64, 4
    q, k, v, do = (rnd(1, 1, L, D, seed=s) for s in (30, 31, 32, 33))
    lm = np.array([[[[1, 2, 0, 8], [4, 1, 8, 0], [0, 0, 1, 2], [2, 4, 8, 1]]]], np.int32)
    dq, dk, dv = O.psa_backward_dense(q, k, v, lm, do, 16, 16)

    def loss(qq, kk, vv):
        lk = {l: O.pool_kv_direct(kk, 16, l) for l in (2, 4, 8)} | {1: kk}
        lv_ = {l: O.pool_kv_direct(vv, 16, l) for l in (2, 4, 8)} | {1: vv}
        return (O.psa_attention_dense(qq, kk, vv, lm, 16, 16, levels_k=lk, levels_v=lv_)[0] * do).sum().item()

    eps = 1e-6
    rng = np.random.default_rng(1)
    for name, t, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for _ in range(6):
            i, d = int(rng.integers(L)), int(rng.integers(D))
            tp, tm = t.clone(), t.clone()
            tp[0, 0, i, d] += eps
            tm[0, 0, i, d] -= eps
            args_p = {"q": (tp, k, v), "k": (q, tp, v), "v": (q, k, tp)}[name]
            args_m = {"q": (tm, k, v), "k": (q, tm, v), "v": (q, k, tm)}[name]
            fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
            assert abs(fd - g[0, 0, i, d].item()) < 1e-6 * max(1.0, abs(fd)), (name, i, d)
    # kv-block 2 of level-map column 2... rows of blocks nobody retains get zero dV
    lm0 = lm.copy()
    lm0[..., 3] = 0
    _, dk0, dv0 = O.psa_backward_dense(q, k, v, lm0, do, 16, 16)
    assert torch.all(dv0[0, 0, 48:] == 0) and torch.all(dk0[0, 0, 48:] == 0)


# ---------------------------------------------------------------- xattn + k-similarity
def test_xattn_brute_force():
    L, D, S, blk = 64, 4, 2, 16
    q, k = rnd(1, 1, L, D, dtype=torch.float32, seed=40), rnd(1, 1, L, D, dtype=torch.float32, seed=41)
    est = O.estimate_xattn(q, k, block_size=blk, stride=S, causal=True, chunk_size=32)
    M = L // S
    A = np.zeros((M, M))
    for m in range(M):
        for n in range(M):
            A[m, n] = sum(float(q[0, 0, m * S + S - 1 - i] @ k[0, 0, n * S + i]) for i in range(S))
    Z = A / (math.sqrt(D) * S)
    Z[np.triu_indices(M, 1)] = -np.inf
    P = np.exp(Z - Z.max(1, keepdims=True))
    P /= P.sum(1, keepdims=True)
    rb = blk // S
    E = P.reshape(M // rb, rb, M // rb, rb).sum((1, 3))
    np.testing.assert_allclose(est[0, 0].numpy(), E, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(est.sum(-1).numpy(), rb, rtol=1e-4)


def test_k_similarity_closed_form():
    k = rnd(1, 1, 64, 8, dtype=torch.float32, seed=50).repeat_interleave(2, 2)  # pairs identical -> sim2 = 1
    m = O.k_similarity(k, 64, 0.99, 0.99, 0.99)
    assert m.shape == (1, 1, 2) and m.view(-1).tolist() == [2, 2]
    m = O.k_similarity(k, 64, 0.99, -2.0, 0.99)
    assert m.view(-1).tolist() == [4, 4]
    k8 = rnd(1, 1, 16, 8, dtype=torch.float32, seed=51).repeat_interleave(8, 2)
    assert O.k_similarity(k8, 64, 0.9, 0.9, 0.9).view(-1).tolist() == [8, 8]
    assert O.k_similarity(-k8 * torch.tensor([1.0, -1.0] * 64).view(1, 1, 128, 1), 64, 0.0, 0.0, 0.0).view(-1).tolist() == [1, 1]
