"""GPU parity of the token re-ordering (row gather through the C ABI) against torch index_select + cat, the
formulation of the reference's GilbertRearranger (utils/rearranger.py:14-132).  Pure copies: bit-exact."""
import pytest
import torch

from gpu_util import dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("grid,text,D", [((3, 6, 10), 0, 128), ((4, 5, 7), 33, 64), ((2, 9, 11), 226, 128)])
def test_rearranger_matches_torch_path(dtype, grid, text, D):
    from psa_hip.utils.rearranger import GilbertRearranger

    depth, height, width = grid
    r = GilbertRearranger(width, height, depth, text)
    L = depth * height * width + text
    g = torch.Generator(device="cpu").manual_seed(L + D)
    q = torch.randn(2, 4, L, D, generator=g).to(dtype).to(dev())
    k = torch.randn(2, 2, L, D, generator=g).to(dtype).to(dev())   # fewer heads (GQA)
    v = torch.randn(2, 2, L, D, generator=g).to(dtype).to(dev())
    fwd = r.original_order2gilbert_order_cpu.to(dev())
    inv = r.gilbert_order2original_order_cpu.to(dev())

    def ref_forward(x):  # the reference's formulation: index_select of the video part, text appended
        if text == 0:
            return x.index_select(-2, fwd)
        return torch.cat((x[..., text:, :].index_select(-2, fwd), x[..., :text, :]), dim=-2)

    def ref_backward(x):
        if text == 0:
            return x.index_select(-2, inv)
        return torch.cat((x[..., -text:, :], x[..., :-text, :].index_select(-2, inv)), dim=-2)

    qr, kr, vr = r.rearrange(q, k, v)
    for a, x in ((qr, q), (kr, k), (vr, v)):
        assert torch.equal(a, ref_forward(x))
        assert torch.equal(r.rearrange_single(x), a)
    back = r.reversed_rearrange(qr)
    assert torch.equal(back, ref_backward(qr))
    assert torch.equal(back, q)  # the two orders are inverse permutations
    with pytest.raises(ValueError):
        r.rearrange_single(q.cpu())  # no torch fall-back


def test_gather_rows_strided_views_and_errors():
    from psa_hip import ops

    B, H, L, D = 1, 3, 500, 128
    g = torch.Generator(device="cpu").manual_seed(3)
    x = torch.randn(B, L, H, D, generator=g).to(torch.bfloat16).to(dev()).permute(0, 2, 1, 3)  # [B, H, L, D] view of [B, L, H, D]
    idx = torch.randperm(L, generator=g)[:321].to(torch.int32).to(dev())
    (y,) = ops.gather_rows((x,), idx)
    assert torch.equal(y, x.index_select(2, idx.long()))
    with pytest.raises(ValueError):
        ops.gather_rows((x,), idx.long())
    with pytest.raises(ValueError):
        ops.gather_rows((x, x[:, :, :100]), idx)
    with pytest.raises(Exception):
        ops.gather_rows((x.cpu(),), idx.cpu())
