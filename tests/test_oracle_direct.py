"""The oracle's restatement of the direct form (pieces of one tap on the tile F(1,1)) against the definition of the
convolution: torch's conv2d in fp64, and bit for bit on integers."""
import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow

CASES = [((2, 8, 9, 11), (6, 8, 3, 3), 2, 1), ((1, 5, 12, 12), (4, 5, 7, 7), 2, 3), ((2, 4, 10, 9), (3, 4, 5, 4), 2, (2, 1)),
         ((1, 6, 8, 8), (4, 6, 3, 3), 1, 1), ((2, 3, 7, 9), (5, 3, 1, 1), 2, 0), ((1, 4, 11, 10), (2, 4, 2, 3), 1, 0)]


@pytest.mark.parametrize("xs,ws,stride,pad", CASES)
def test_direct_form_is_the_convolution(xs, ws, stride, pad):
    g = torch.Generator().manual_seed(0)
    x, w, b = torch.randn(*xs, generator=g), torch.randn(*ws, generator=g), torch.randn(ws[0], generator=g)
    ref = F.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    y = ow.direct_conv(x, w, b, stride, pad, "fp64")
    assert y.shape == ref.shape and float((y - ref).abs().max()) < 1e-12
    y32 = ow.direct_conv(x, w, b, stride, pad, "fp32")
    assert float((y32.double() - ref).abs().max() / ref.abs().max()) < 1e-6
    xi, wi = torch.randint(-3, 4, xs, generator=g).double(), torch.randint(-2, 3, ws, generator=g).double()
    for disc in ("fp32", "fp16", "bf16"):
        yi = ow.direct_conv(xi, wi, None, stride, pad, disc)
        assert torch.equal(yi.double(), F.conv2d(xi, wi, stride=stride, padding=pad))
    # the same sum as the decomposed forms of the oracle
    yd = ow.dwm_conv(x, w, b, stride, pad, 2, "fp32")
    assert float((y32 - yd).abs().max() / ref.abs().max()) < 1e-5


CASES_3D = [((2, 3, 5, 8, 9), (4, 3, 3, 3, 3), 1, 1), ((1, 4, 6, 7, 7), (5, 4, 3, 3, 2), 1, (1, 0, 1)), ((1, 2, 4, 6, 5), (3, 2, 2, 3, 3), 2, 1)]


@pytest.mark.parametrize("xs,ws,stride,pad", CASES_3D)
def test_direct_form_is_the_convolution_in_3d(xs, ws, stride, pad):
    """The same restatement with the kernel planes outermost: torch's conv3d in fp64, and bit for bit on integers."""
    g = torch.Generator().manual_seed(1)
    x, w, b = torch.randn(*xs, generator=g), torch.randn(*ws, generator=g), torch.randn(ws[0], generator=g)
    ref = F.conv3d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    y = ow.direct_conv(x, w, b, stride, pad, "fp64")
    assert y.shape == ref.shape and float((y - ref).abs().max()) < 1e-12
    xi, wi = torch.randint(-3, 4, xs, generator=g).double(), torch.randint(-2, 3, ws, generator=g).double()
    for disc in ("fp32", "fp16", "bf16"):
        yi = ow.direct_conv(xi, wi, None, stride, pad, disc)
        assert torch.equal(yi.double(), F.conv3d(xi, wi, stride=stride, padding=pad))
