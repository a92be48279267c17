"""Seeded random sweep over problem shapes: kernel extents 1..10 per axis (non-square included),
stride 1 and 2, paddings 0..k-1 per axis, odd channel counts, 2-D and 3-D, output tile 2 and 4,
all three storage types - every case against fp64 torch convolution of the same rounded inputs.
Tolerances as everywhere: fp32 1e-3, fp16 2e-2, bf16 2e-2 (tile 2) / 2e-1 (tile 4)."""
import random

import pytest
import torch
import torch.nn.functional as F

from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu


def _cases(seed, n, nd):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        ks = [rng.choice([1, 2, 3, 3, 3, 4, 5, 7, rng.randint(1, 10)]) for _ in range(nd)]
        if nd == 3:
            ks = [min(k, 5) for k in ks]                 # keep the number of pieces (and the runtime) small
        stride = rng.choice([1, 1, 2])
        pad = [rng.randint(0, k - 1) for k in ks]
        sp = [rng.randint(max(k - 2 * p, 1), 14 if nd == 2 else 9) + rng.randint(0, 6) for k, p in zip(ks, pad)]
        N, C, K = rng.randint(1, 3), rng.choice([1, 3, 8, 17, 32, 40]), rng.choice([1, 4, 6, 9, 32, 33])
        m = rng.choice([2, 4])
        if m == 4 and nd == 3 and not (ks == [3, 3, 3] and stride == 1):
            m = 2
        dtype = rng.choice([torch.float32, torch.float16, torch.bfloat16])
        out.append((N, C, K, tuple(sp), tuple(ks), stride, tuple(pad), m, dtype))
    return out


CASES = _cases(2024, 60, 2) + _cases(2025, 30, 3)


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_random_shape(dev, case):
    N, C, K, sp, ks, stride, pad, m, dtype = case
    g = torch.Generator().manual_seed(hash(case[:8]) % (2 ** 31))
    fan = C
    for k in ks:
        fan *= k
    x = torch.randn(N, C, *sp, generator=g).to(dtype)
    w = (torch.randn(K, C, *ks, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(K, generator=g).to(dtype)
    conv = F.conv2d if len(sp) == 2 else F.conv3d
    ref = conv(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m)
    assert tuple(y.shape) == tuple(ref.shape), case
    tol = {torch.float32: 1e-3, torch.float16: 2e-2, torch.bfloat16: 2e-2 if m == 2 else 2e-1}[dtype]
    err = float((y.double().cpu() - ref).abs().max() / ref.abs().max().clamp_min(1e-30))
    assert err <= tol, (case, err)
