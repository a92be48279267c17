"""The benchmark configurations at their full sizes, checked through properties that do not need
a full-size CPU reference:

  * images are independent, so the fp64 torch convolution of ONE image (cheap on the CPU) must
    match that image's slice of the full-batch result within the stated tolerance
    (fp32: 1e-3, fp16: 2e-2 of max |y64|);
  * permuting the batch must permute the output bit for bit (tile indexing, chunking and the
    GEMM's tile partition must not leak between images);
  * linearity: conv(x1 + x2) = conv(x1) + conv(x2) up to rounding.
"""
import pytest
import torch
import torch.nn.functional as F

from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu

H16, F32 = torch.float16, torch.float32
CONFIGS = [
    # name, x shape, w shape, stride, pad, m, dtype
    ("metric F(4,3)", (64, 256, 56, 56), (256, 256, 3, 3), 1, 1, 4, H16),
    ("metric F(2,3)", (64, 256, 56, 56), (256, 256, 3, 3), 1, 1, 2, H16),
    ("c1", (1, 64, 56, 56), (64, 64, 3, 3), 1, 1, 2, F32),
    ("c3 64 @56", (64, 64, 56, 56), (64, 64, 3, 3), 1, 1, 4, H16),
    ("c3 128 @28", (64, 128, 28, 28), (128, 128, 3, 3), 1, 1, 4, H16),
    ("c3 256 @14", (64, 256, 14, 14), (256, 256, 3, 3), 1, 1, 4, H16),
    ("c3 512 @7", (64, 512, 7, 7), (512, 512, 3, 3), 1, 1, 4, H16),
    ("c4 5x5 s1", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 2, H16),
    ("c4 7x7 s1", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 2, H16),
    ("c4 5x5 s1 tile 4", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 4, H16),
    ("c4 7x7 s1 tile 4", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 4, H16),
    ("c4 7x7 s2 tile 4", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 4, H16),
    ("c4 3x3 s2", (32, 128, 112, 112), (128, 128, 3, 3), 2, 1, 2, H16),
    ("c4 7x7 s2", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 2, H16),
    # the same plans with the reference's structure (pieces added after their output transforms); the
    # lines above run the 16-bit default, which adds the pieces in the batched GEMM
    ("c4 5x5 s1 tile 4 piece by piece", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 4, H16),
    ("c4 7x7 s1 piece by piece", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 2, H16),
    ("c4 7x7 s2 tile 4 piece by piece", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 4, H16),
    ("c5 3-D", (8, 128, 16, 56, 56), (128, 128, 3, 3, 3), 1, 1, 2, H16),
    ("c5 3-D tile 2x4x4", (8, 128, 16, 56, 56), (128, 128, 3, 3, 3), 1, 1, 4, H16),
]

# c2: all 13 layers of the VGG-16 stack at N = 8 in fp32, each with both output tiles, F(2x2,3x3) and
# F(4x4,3x3) (layers of equal shape get their own data: the seed is the layer number)
VGG16 = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56), (256, 256, 56),
         (256, 512, 28), (512, 512, 28), (512, 512, 28), (512, 512, 14), (512, 512, 14), (512, 512, 14)]
VGG_SEED = {}
for _i, (_c, _k, _h) in enumerate(VGG16):
    for _m in (2, 4):
        _name = "c2 vgg %d: %d->%d @%d m%d" % (_i + 1, _c, _k, _h, _m)
        VGG_SEED[_name] = _i
        CONFIGS.append((_name, (8, _c, _h, _h), (_k, _c, 3, 3), 1, 1, _m, F32))


def _data(xs, ws, dtype, dev, seed=0):
    g = torch.Generator().manual_seed(seed)
    fan = 1
    for v in ws[1:]:
        fan *= v
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    return x, w


@pytest.mark.parametrize("cfg", CONFIGS, ids=[c[0] for c in CONFIGS])
def test_full_size_config(dev, cfg):
    name, xs, ws, stride, pad, m, dtype = cfg
    x, w = _data(xs, ws, dtype, dev, VGG_SEED.get(name, 0))
    xd, wd = x.to(dev), w.to(dev)
    stacked = False if name.endswith("piece by piece") else None

    def forward(a):
        # the Winograd / DWM plans are what this file covers at full size: the direct form, which the library would
        # take for the stride-2 layers, has its own full-size test (test_gpu_direct.py)
        return engine.conv_forward(a, wd, None, stride, pad, m, stacked=stacked, direct=False)

    y = forward(xd)
    conv = F.conv2d if len(xs) == 4 else F.conv3d
    tol = 1e-3 if dtype == F32 else 2e-2
    # one image against fp64 on the CPU (the last one: it sits in the last, possibly partial, chunk)
    n = xs[0] - 1
    ref = conv(x[n:n + 1].double(), w.double(), stride=stride, padding=pad)
    assert tuple(y.shape[1:]) == tuple(ref.shape[1:])
    err = float((y[n:n + 1].double().cpu() - ref).abs().max() / ref.abs().max())
    assert err <= tol, (name, err)
    if xs[0] > 1:
        perm = torch.randperm(xs[0], generator=torch.Generator().manual_seed(1))
        yp = forward(xd[perm.to(dev)].contiguous())
        assert torch.equal(yp, y[perm.to(dev)]), name
    # linearity on a second input (fp32 accumulate, one rounding of each result)
    x2 = torch.randn(xs, generator=torch.Generator().manual_seed(2)).to(dtype).to(dev)
    if dtype == H16:
        xs_sum = (xd.float() + x2.float()).half()          # what the engine really sees
        lhs = forward(xs_sum).float()
        rhs = forward((xs_sum.float() - x2.float()).half()).float() + forward(x2).float()
        scale = float(rhs.abs().max())
        assert float((lhs - rhs).abs().max()) / scale <= 3e-2, name
    else:
        lhs = forward(xd + x2)
        rhs = y + forward(x2)
        assert float((lhs - rhs).abs().max() / rhs.abs().max()) <= 1e-4, name


def test_stage_calls_beyond_2g_elements(dev):
    """Maximum sizes: V and M hold 2.47e9 elements each (more than 2^31), so every kernel's
    offsets must be 64-bit.  Images are independent, so each stage's slice for one image must
    equal, bit for bit, the same stage run on that image alone; the chunked one-call entry point
    must reproduce the un-chunked stage pipeline; and the last image is checked against fp64."""
    N, C, K, H = 96, 128, 128, 224
    g = torch.Generator().manual_seed(3)
    w = (torch.randn(K, C, 3, 3, generator=g) * (2.0 / (C * 9)) ** 0.5).half().to(dev)
    x = torch.empty(N, H, H, C, dtype=H16, device=dev)                     # channel-last memory
    for b in range(N):
        x[b] = torch.randn(H, H, C, generator=g).half().to(dev)
    desc = engine.make_desc((N, C, H, H), w.shape, H16, 1, 1, 2)
    plan = engine.plan_conv(desc)
    U = engine.filter_transform(desc, plan, w)
    V = engine.input_transform(desc, plan, x)
    assert V.numel() > 2 ** 31
    M = engine.batched_gemm(V, U)
    y = engine.output_transform(desc, plan, M, None, N)
    tiles = V.shape[1] // N
    d1 = engine.make_desc((1, C, H, H), w.shape, H16, 1, 1, 2)
    for b in (0, 41, N - 1):
        V1 = engine.input_transform(d1, plan, x[b:b + 1])
        assert torch.equal(V[:, b * tiles:(b + 1) * tiles], V1), ("input transform", b)
        M1 = engine.batched_gemm(V1, U)
        assert torch.equal(M[:, b * tiles:(b + 1) * tiles], M1), ("batched gemm", b)
        y1 = engine.output_transform(d1, plan, M1, None, 1)
        assert torch.equal(y[b:b + 1], y1), ("output transform", b)
    del V, M
    x_nchw = x.permute(0, 3, 1, 2)                                         # channels_last view, no copy
    yc = engine.conv_forward(x_nchw, w, None, 1, 1, 2)                     # chunked: V + M bounded at 8 GiB
    assert torch.equal(yc.permute(0, 2, 3, 1), y[:, 0])                    # stage output keeps a depth axis of 1
    ref = F.conv2d(x_nchw[N - 1:].double().cpu(), w.double().cpu(), padding=1)
    err = float((yc[N - 1:].double().cpu() - ref).abs().max() / ref.abs().max())
    assert err <= 2e-2, err


def test_stacked_plan_beyond_2g_elements_in_one_pass(dev):
    """7x7 kernel, pieces stacked: V of one pass holds 16 x 125440 x 1152 = 2.3e9 elements.  Images are
    independent, so every image of the batch must equal its own single-image convolution bit for
    bit, and one of them is checked against fp64."""
    N, C, K, H = 40, 128, 128, 112
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(K, C, 7, 7, generator=g) * (2.0 / (C * 49)) ** 0.5).half().to(dev)
    x = torch.randn(N, C, H, H, generator=g).half().to(dev).contiguous(memory_format=torch.channels_last)
    desc = engine.make_desc(x.shape, w.shape, H16, 1, 3, 2, stacked=True)
    plan = engine.plan_conv(desc)
    assert plan.t_total * (N * 56 * 56) * (plan.n_pieces * C) > 2 ** 31
    y = engine.conv_forward(x, w, None, 1, 3, 2, stacked=True)
    for b in (0, 17, N - 1):
        assert torch.equal(y[b:b + 1], engine.conv_forward(x[b:b + 1], w, None, 1, 3, 2, stacked=True)), b
    ref = F.conv2d(x[N - 1:].double().cpu(), w.double().cpu(), padding=3)
    err = float((y[N - 1:].double().cpu() - ref).abs().max() / ref.abs().max())
    assert err <= 2e-2, err


GRAD_CONFIGS = [c for c in CONFIGS if c[0] in ("metric F(4,3)", "metric F(2,3)", "c2 vgg 2: 64->64 @224 m4", "c4 5x5 s1 tile 4",
                                               "c4 7x7 s2", "c5 3-D", "c5 3-D tile 2x4x4")]


@pytest.mark.parametrize("cfg", GRAD_CONFIGS, ids=[c[0] for c in GRAD_CONFIGS])
def test_full_size_gradients_are_the_adjoints_of_the_forward_pass(dev, cfg):
    """The gradients are the adjoints of the two linear maps w -> conv(x, w) and x -> conv(x, w):
    <dw(x, dy), w'> = <dy, conv(x, w')> and <dx(dy, w), x'> = <dy, conv(x', w)>.  With dy set to the
    forward output itself the right-hand sides are squared norms, so the identity is checked to a
    relative bound; the forward pass is the one the tests above check, and no full-size CPU
    reference is needed.  Sums in fp64 on the device.  Measured: 5e-9 in fp32, <= 3e-5 in fp16 (rounding errors average out over the sum)."""
    name, xs, ws, stride, pad, m, dtype = cfg
    x, w = _data(xs, ws, dtype, dev)
    xd, wd = x.to(dev), w.to(dev)
    g = torch.Generator().manual_seed(9)
    w2 = (torch.randn(*ws, generator=g) * float(w.float().std())).to(dtype).to(dev)
    x2 = torch.randn(*xs, generator=g).to(dtype).to(dev)
    tol = 1e-6 if dtype == F32 else 1e-3

    dy = engine.conv_forward(xd, w2, None, stride, pad, m)
    dw = engine.conv_backward_weight(xd, dy, ws, stride, pad, m)
    lhs, rhs = float((dw.double() * w2.double()).sum()), float((dy.double() ** 2).sum())
    assert abs(lhs - rhs) <= tol * rhs, (name, "weight gradient", lhs, rhs)

    dy = engine.conv_forward(x2, wd, None, stride, pad, m)
    dx = engine.conv_backward_input(dy, wd, xs[2:], stride, pad, m)
    lhs, rhs = float((dx.double() * x2.double()).sum()), float((dy.double() ** 2).sum())
    assert abs(lhs - rhs) <= tol * rhs, (name, "input gradient", lhs, rhs)
