"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

import psa_oracle as O


def dev():
    return torch.device("cuda:0")


def rnd(*shape, seed=0, dtype=torch.bfloat16, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def random_map(B, H, Mq, Nk, seed, p=(0.35, 0.2, 0.15, 0.15, 0.15), ensure_row=True):
    rng = np.random.default_rng(seed)
    m = rng.choice([0, 1, 2, 4, 8], size=(B, H, Mq, Nk), p=p).astype(np.int32)
    if ensure_row:
        m[..., 0] = np.where(m.sum(-1) == 0, 1, m[..., 0])
    return m


def attn_errors(out_gpu, ref):
    d = (out_gpu.float().cpu() - ref.float()).abs()
    return float(d.max()), float(d.mean())


# tolerance of the task statement for bf16 attention outputs
MAX_ABS, MEAN_ABS = 2e-2, 2e-3
