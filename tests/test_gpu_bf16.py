"""bfloat16 storage (the boundary asks for fp16/bf16 dispatch by tensor dtype; the reference
itself is float-only, pybind/bind.cpp:20-22): every stage and the whole convolution against the
CPU oracle run in the same discipline (bfloat16 storage, fp32 arithmetic, one rounding per stored
value) and against fp64 convolution of the same rounded inputs.

Tolerances, in units of max |reference|: a bfloat16 value carries 8 significant bits, so one
rounding is 2^-9 = 2e-3 relative.
  stage against oracle (same arithmetic, other summation order): 1.2e-2 (a few ulp of the largest value)
  convolution against fp64, output tile 2:  2e-2  (measured 5e-3 .. 7e-3, the fp16 bound of the metric)
  convolution against fp64, output tile 4:  2e-1  (measured 6e-2 .. 1e-1: F(4,r) amplifies the
                                                   rounding of V and M by up to 100; not recommended,
                                                   the modules pick tile 2 for bfloat16)
"""
import pytest
import torch
import torch.nn.functional as F

import pytorch_winoconv_amd as pkg
from oracle import winograd as ow
from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu
BF = torch.bfloat16

CASES = [
    # x shape, w shape, stride, pad, m
    ((2, 16, 13, 12), (24, 16, 3, 3), 1, 1, 2),
    ((2, 16, 13, 12), (24, 16, 3, 3), 1, 1, 4),
    ((2, 8, 12, 13), (8, 8, 5, 5), 1, 2, 2),
    ((1, 8, 15, 14), (4, 8, 7, 7), 2, 3, 4),
    ((1, 6, 6, 9, 8), (8, 6, 3, 3, 3), 1, 1, 2),
    ((2, 64, 28, 28), (64, 64, 3, 3), 1, 1, 2),
    ((2, 256, 14, 14), (256, 256, 3, 3), 1, 1, 4),
]


def _data(xs, ws, seed=0):
    g = torch.Generator().manual_seed(seed)
    fan = 1
    for v in ws[1:]:
        fan *= v
    x = torch.randn(*xs, generator=g).to(BF)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(BF)
    b = torch.randn(ws[0], generator=g).to(BF)
    return x, w, b


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("case", CASES)
def test_stages_against_oracle(dev, case):
    xs, ws, stride, pad, m = case
    x, w, b = _data(xs, ws)
    st = {}
    want = ow.dwm_conv(x, w, b, stride, pad, m, "bf16", st)
    desc = engine.make_desc(xs, ws, BF, stride, pad, m)
    plan = engine.plan_conv(desc)
    C, K = desc.C, desc.K
    U = engine.filter_transform(desc, plan, w.to(dev))
    assert U.dtype == BF and torch.count_nonzero(U[:, :, C:]) == 0
    assert _rel(U[:, :, :C], st["U"]) <= 1.2e-2
    V = engine.input_transform(desc, plan, engine.channel_last(x.to(dev)))
    assert _rel(V[:, :, :C], st["V"]) <= 1.2e-2
    # the next stages are fed the oracle's own buffers so that each is checked on its own
    Cp = U.shape[2]
    Uo = torch.zeros(U.shape, dtype=BF); Uo[:, :, :C] = st["U"]
    Vo = torch.zeros(V.shape, dtype=BF); Vo[:, :, :C] = st["V"]
    M = engine.batched_gemm(Vo.to(dev), Uo.to(dev))
    assert _rel(M[:, :, :K], st["M"]) <= 1.2e-2
    Mo = torch.zeros(M.shape, dtype=BF); Mo[:, :, :K] = st["M"]
    y = engine.output_transform(desc, plan, Mo.to(dev), b.to(dev), desc.N)
    assert _rel(y, st["y_cl"]) <= 1.2e-2
    assert Cp % 32 == 0


@pytest.mark.parametrize("case", CASES)
def test_conv_against_fp64(dev, case):
    xs, ws, stride, pad, m = case
    x, w, b = _data(xs, ws, seed=1)
    conv = F.conv2d if len(xs) == 4 else F.conv3d
    ref = conv(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m)
    assert y.dtype == BF and tuple(y.shape) == tuple(ref.shape)
    err = _rel(y, ref)
    assert err <= (2e-2 if m == 2 else 2e-1), err
    # and no worse than 3x the oracle's own bfloat16 evaluation of the same formula
    yo = ow.dwm_conv(x, w, b, stride, pad, m, "bf16")
    assert err <= 3 * _rel(yo, ref) + 1e-3


def test_batched_gemm_values_and_integer_exactness(dev):
    g = torch.Generator().manual_seed(3)
    V = torch.randn(5, 300, 96, generator=g).to(BF)
    U = (torch.randn(5, 72, 96, generator=g) / 96 ** 0.5).to(BF)
    want = torch.bmm(V.double(), U.double().transpose(1, 2))
    M = engine.batched_gemm(V.to(dev), U.to(dev))
    assert M.dtype == BF and _rel(M[:, :, :72], want) <= 8e-3
    # entries in {-1, 0, 1}: every sum is an integer of magnitude <= 64, exact in bfloat16
    Vi = torch.randint(-1, 2, (6, 333, 64), generator=g).to(BF)
    Ui = torch.randint(-1, 2, (6, 40, 64), generator=g).to(BF)
    Mi = engine.batched_gemm(Vi.to(dev), Ui.to(dev))
    assert torch.equal(Mi[:, :, :40].double().cpu(), torch.bmm(Vi.double(), Ui.double().transpose(1, 2)))


def test_split_concat_and_modules(dev):
    from oracle import tiles as ot
    x = torch.randn(2, 5, 9, 10).to(BF)
    t = pkg.wino_split(x.to(dev), [4, 5, 3, 3], 2)
    assert t.dtype == BF
    assert torch.equal(t.cpu().view(torch.int16), torch.from_numpy(ot.wino_split(x.view(torch.int16).numpy(), (4, 5, 3, 3), 2)))
    o = torch.randn(t.shape[0], 3, 2, 2).to(BF)
    y = pkg.wino_concat(o.to(dev), [7, 8], 2)
    assert torch.equal(y.cpu().view(torch.int16), torch.from_numpy(ot.wino_concat(o.view(torch.int16).numpy(), (7, 8), 2)))
    # the module picks output tile 2 for bfloat16 and stays within the tile-2 bound
    mod = pkg.WinoConv2d(16, 24, 3, 1, 1, dtype=BF, device=dev)
    xx = torch.randn(2, 16, 20, 20).to(BF)
    ref = F.conv2d(xx.double(), mod.weight.detach().double().cpu(), mod.bias.detach().double().cpu(), padding=1)
    assert _rel(mod(xx.to(dev)), ref) <= 2e-2
