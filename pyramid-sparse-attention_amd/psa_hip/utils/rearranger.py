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

    def _combined_index(self, device, forward: bool) -> torch.Tensor:
        """int32 [L] source row of every output row, text tokens included: forward moves the text (first
        text_length rows) behind the re-ordered video tokens, backward moves it to the front again."""
        key = (str(device), forward, "combined")
        if key not in self._cache:
            t, n = self.text_length, self.total_elements
            # (built as an ordinary tensor also when first asked for under torch.inference_mode: the operators cache their
            # validity check of an index on its version counter, which inference tensors do not have)
            with torch.inference_mode(False):
                if forward:
                    idx = torch.cat((self.original_order2gilbert_order_cpu + t, torch.arange(t)))
                else:
                    idx = torch.cat((torch.arange(t) + n, self.gilbert_order2original_order_cpu))
                self._cache[key] = idx.to(torch.int32).to(device)
        return self._cache[key]

    def token_index(self, device) -> torch.Tensor:
        """int32 [L]: position i of the re-ordered sequence (video tokens along the curve, then the text) is row
        token_index[i] of the input.  The layer's kernels can read and write through it directly instead of calling
        rearrange() / reversed_rearrange() (ops.pool_kv_indexed, the q_index arguments of the estimator and the
        attention forward)."""
        return self._combined_index(device, True)

    @staticmethod
    def _native(x: torch.Tensor) -> bool:
        # the HIP row gather handles GPU tensors [B, H, L, D] with 2- or 4-byte elements and 16-byte rows
        return (x.is_cuda and x.dim() == 4 and x.element_size() in (2, 4) and (x.shape[-1] * x.element_size()) % 16 == 0
                and 256 % ((x.shape[-1] * x.element_size()) // 16) == 0 and x.data_ptr() % 16 == 0
                and all((s * x.element_size()) % 16 == 0 for s in x.stride()[:3]))

    def _check(self, x: torch.Tensor, what: str) -> None:
        # there is no torch fall-back: tensors the row-gather kernel cannot take are an error, as for every other operator
        if not (self._native(x) and x.shape[-2] == self.total_elements + self.text_length):
            raise ValueError(
                "GilbertRearranger.%s: expected a GPU tensor [B, H, %d, D] with 2- or 4-byte elements, 16-byte aligned rows and "
                "strides (got shape %s on %s)" % (what, self.total_elements + self.text_length, tuple(x.shape), x.device))

    def rearrange_single(self, x: torch.Tensor) -> torch.Tensor:
        from .. import ops

        self._check(x, "rearrange_single")
        return ops.gather_rows((x,), self._combined_index(x.device, True))[0]

    def rearrange(self, q, k, v) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        from .. import ops

        for t in (q, k, v):
            self._check(t, "rearrange")
        if q.dtype == k.dtype == v.dtype and q.shape[0] == k.shape[0] == v.shape[0] and q.shape[-1] == k.shape[-1] == v.shape[-1]:
            return ops.gather_rows((q, k, v), self._combined_index(q.device, True))  # one launch for the three
        return self.rearrange_single(q), self.rearrange_single(k), self.rearrange_single(v)

    def reversed_rearrange(self, out: torch.Tensor) -> torch.Tensor:
        from .. import ops

        self._check(out, "reversed_rearrange")
        return ops.gather_rows((out,), self._combined_index(out.device, False))[0]
