"""Token re-ordering along a 3-D Hilbert-type curve before / after attention.

reference: src/psa_triton/utils/rearranger.py:14-132 (GilbertRearranger).  Tokens of the video grid are
re-ordered so that tokens close in (t, y, x) are close in the sequence, which makes block sparsity
effective; text tokens (first in the input) are moved to the END of the re-ordered sequence, and moved
back to the front when the output is restored.
"""
from typing import Tuple

import torch

from .gilbert3d import gilbert3d


class GilbertRearranger:
    def __init__(self, width: int, height: int, depth: int, text_length: int = 224):
        self.width, self.height, self.depth = width, height, depth
        self.total_elements = width * height * depth
        self.text_length = text_length
        # curve position -> flat token index x + W*(y + H*z), and its inverse
        fwd = [x + width * (y + height * z) for x, y, z in gilbert3d(width, height, depth)]
        inv = [0] * self.total_elements
        for pos, tok in enumerate(fwd):
            inv[tok] = pos
        self.original_order2gilbert_order_cpu = torch.tensor(fwd, dtype=torch.long)
        self.gilbert_order2original_order_cpu = torch.tensor(inv, dtype=torch.long)
        self._cache = {}

    def _indices(self, device, forward: bool) -> torch.Tensor:
        key = (str(device), forward)
        if key not in self._cache:
            src = self.original_order2gilbert_order_cpu if forward else self.gilbert_order2original_order_cpu
            self._cache[key] = src.to(device)
        return self._cache[key]

    def rearrange_single(self, x: torch.Tensor) -> torch.Tensor:
        idx = self._indices(x.device, True)
        if self.text_length == 0:
            return x.index_select(-2, idx)
        text, video = x[..., : self.text_length, :], x[..., self.text_length :, :]
        return torch.cat((video.index_select(-2, idx), text), dim=-2)

    def rearrange(self, q, k, v) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        return self.rearrange_single(q), self.rearrange_single(k), self.rearrange_single(v)

    def reversed_rearrange(self, out: torch.Tensor) -> torch.Tensor:
        idx = self._indices(out.device, False)
        if self.text_length == 0:
            return out.index_select(-2, idx)
        video, text = out[..., : -self.text_length, :], out[..., -self.text_length :, :]
        return torch.cat((text, video.index_select(-2, idx)), dim=-2)
