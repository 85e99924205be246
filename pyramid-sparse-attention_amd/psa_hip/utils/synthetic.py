"""Seeded synthetic Q/K/V for tests and benchmarks: smooth low-frequency fields over a (t, h, w)
token grid plus noise, so that attention is concentrated the way video attention is and block
sparsity is meaningful.  Runs on whatever device is asked for (CPU or GPU)."""
import math
from typing import Optional, Tuple

import torch


def smooth_field(
    B: int, H: int, grid: Tuple[int, int, int], D: int, seed: int, *, n_waves: int = 8, noise: float = 0.3,
    device="cpu", text_tokens: int = 0, text_first: bool = False,
) -> torch.Tensor:
    """X[b,h,n,c] = sum_i a_i[h,c] sin(2 pi f_i.(t/T, y/Hh, x/W) + phi_i[h,c]) + noise * eps, fp32,
    n = (t*Hh + y)*W + x; `text_tokens` i.i.d. N(0,1) rows are put after (or before) the grid."""
    T, Hh, W = grid
    g = torch.Generator(device="cpu").manual_seed(seed)
    f = torch.rand(n_waves, 3, generator=g) * 3.0
    amp = torch.randn(n_waves, H, D, generator=g) / math.sqrt(n_waves)
    phi = torch.rand(n_waves, H, D, generator=g) * (2 * math.pi)
    tt, yy, xx = torch.meshgrid(torch.arange(T) / T, torch.arange(Hh) / Hh, torch.arange(W) / W, indexing="ij")
    pos = torch.stack([tt, yy, xx], -1).reshape(-1, 3)  # [N,3]
    f, amp, phi, pos = f.to(device), amp.to(device), phi.to(device), pos.to(device)
    N = pos.shape[0]
    x = torch.zeros(H, N, D, device=device)
    for i in range(n_waves):
        arg = (pos @ f[i]) * (2 * math.pi)  # [N]
        x += amp[i].unsqueeze(1) * torch.sin(arg.view(1, N, 1) + phi[i].unsqueeze(1))
    x = x.unsqueeze(0).repeat(B, 1, 1, 1)
    gn = torch.Generator(device="cpu").manual_seed(seed + 7919)
    x += noise * torch.randn(B, H, N, D, generator=gn).to(device)
    if text_tokens:
        txt = torch.randn(B, H, text_tokens, D, generator=gn).to(device)
        x = torch.cat([txt, x], 2) if text_first else torch.cat([x, txt], 2)
    return x


def make_qkv(
    B: int, Hq: int, Hkv: int, grid: Tuple[int, int, int], D: int, *, seed: int = 1234, dtype=torch.bfloat16, device="cpu",
    logit_std: float = 3.0, text_tokens: int = 0, text_first: bool = False,
):
    """Q [B,Hq,N,D], K, V [B,Hkv,N,D]; Q and K are scaled by a common factor so that
    std(Q K^T / sqrt(D)) ~= logit_std (estimated on a 1024 x 1024 subset)."""
    q = smooth_field(B, Hq, grid, D, seed, device=device, text_tokens=text_tokens, text_first=text_first)
    k = smooth_field(B, Hkv, grid, D, seed + 1, device=device, text_tokens=text_tokens, text_first=text_first)
    v = smooth_field(B, Hkv, grid, D, seed + 2, device=device, text_tokens=text_tokens, text_first=text_first)
    N = q.shape[2]
    g = torch.Generator(device="cpu").manual_seed(seed + 3)
    n = min(N, 1024)
    iq = torch.randperm(N, generator=g)[:n].to(device)
    ik = torch.randperm(N, generator=g)[:n].to(device)
    rep = Hq // Hkv
    s = torch.einsum("hqd,hkd->hqk", q[0, :, iq], k[0].repeat_interleave(rep, 0)[:, ik]) / math.sqrt(D)
    c = math.sqrt(logit_std / float(s.std()))
    return (q * c).to(dtype), (k * c).to(dtype), v.to(dtype)


def sample_offsets(B: int, H: int, block: int, keep: int, seed: int, device="cpu") -> torch.Tensor:
    """`keep` distinct in-block offsets per (b, h): int32 [B,H,keep] (rand -> topk, like the reference)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    r = torch.rand(B, H, block, generator=g)
    return torch.topk(r, keep, dim=2).indices.to(torch.int32).to(device)
