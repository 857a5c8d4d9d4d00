"""GPU parity: pool2d / pool2dBackward through the C ABI against the CPU
checker.  fp32 results, argmax bytes and gradients are compared bit for bit."""
import numpy as np
import pytest
import torch

import flashlight_amd as fa
from gpu_util import dev, host, round_to
from oracle import flref
from test_oracle_pool import GEOMS

pytestmark = pytest.mark.gpu

MORE = [
    ((2, 5, 112, 112), (3, 3), (2, 2), (1, 1)),   # ResNet stem pool (W % 4 == 0)
    ((3, 4, 28, 28), (2, 2), (2, 2), (0, 0)),     # MNIST pools
    ((2, 3, 14, 14), (2, 2), (2, 2), (0, 0)),
    ((2, 3, 9, 7), (7, 9), (1, 1), (3, 4)),       # ModuleTest.cpp:398-413: 9x7 SAME stride 1
    ((1, 2, 30, 50), (3, 3), (2, 2), (1, 1)),     # W % 4 != 0
    ((1, 3, 33, 36), (3, 3), (2, 2), (1, 1)),     # odd height
    ((2, 6, 7, 7), (7, 7), (1, 1), (0, 0)),
    ((1, 2, 1, 40), (1, 4), (1, 3), (0, 1)),      # 1-D
    ((3, 7, 56, 280), (3, 3), (2, 2), (1, 1)),    # fast path, rows wider than a wave
    ((2, 3, 37, 24), (3, 3), (2, 2), (1, 1)),     # fast path, odd height, short last strip
    ((5, 3, 2, 4), (3, 3), (2, 2), (1, 1)),       # fast path, tiny planes
    ((1, 2, 18, 8), (3, 3), (2, 2), (1, 1)),
    ((3, 5, 56, 56), (2, 2), (2, 2), (0, 0)),     # 2x2 stride 2: non-overlapping fast path
    ((2, 3, 6, 260), (2, 2), (2, 2), (0, 0)),     # ... rows wider than a wave
    ((2, 3, 7, 8), (2, 2), (2, 2), (0, 0)),       # odd height: generic kernels
    ((2, 3, 8, 6), (2, 2), (2, 2), (0, 0)),       # W % 4 != 0: generic kernels
]
ALL = GEOMS + MORE


def _x(shape, seed):
    return (np.round(np.random.default_rng(seed).standard_normal(shape) * 8) / 8).astype(np.float32)


@pytest.mark.parametrize("geom", ALL)
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_pool_f32_bit_exact(geom, mode):
    xs, win, st, pd = geom
    x = _x(xs, 40)
    d = flref.pool_desc(xs, win, st, pd, mode)
    y_ref, am_ref = flref.pool2d_fwd(d, x)
    dy = np.random.default_rng(41).standard_normal(y_ref.shape).astype(np.float32)
    dx_ref = flref.pool2d_bwd(d, dy, am_ref)
    args = (win[1], win[0], st[1], st[0], pd[1], pd[0])
    y, am = fa.pool2d(dev(x), *args, mode=mode, train=True)
    dx = fa.pool2d_backward(dev(dy), xs, am, *args, mode=mode)
    assert np.array_equal(host(y), y_ref)
    if mode == 0:
        assert am.dtype == torch.uint8 and np.array_equal(am.cpu().numpy(), am_ref)
    else:
        assert am is None
    assert np.array_equal(host(dx), dx_ref)
    # inference (no payload): same values, no argmax
    y2, am2 = fa.pool2d(dev(x), *args, mode=mode, train=False)
    assert am2 is None and np.array_equal(host(y2), y_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("geom", [ALL[0], MORE[0], MORE[1], MORE[4], MORE[12], MORE[14]])
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_pool_16bit_storage(geom, mode, dtype):
    xs, win, st, pd = geom
    x = round_to(_x(xs, 42), dtype)
    d = flref.pool_desc(xs, win, st, pd, mode)
    y_ref, am_ref = flref.pool2d_fwd(d, x)
    dy = round_to(np.random.default_rng(43).standard_normal(y_ref.shape), dtype)
    dx_ref = flref.pool2d_bwd(d, dy, am_ref)
    args = (win[1], win[0], st[1], st[0], pd[1], pd[0])
    y, am = fa.pool2d(dev(x, dtype), *args, mode=mode)
    dx = fa.pool2d_backward(dev(dy, dtype), xs, am, *args, mode=mode)
    assert y.dtype == dtype and dx.dtype == dtype
    if mode == 0:   # selection only: exact
        assert np.array_equal(host(y), y_ref) and np.array_equal(am.cpu().numpy(), am_ref)
    else:
        assert np.allclose(host(y), y_ref, rtol=1e-2, atol=1e-2)
    assert np.allclose(host(dx), dx_ref, rtol=1e-2, atol=1e-2)


def test_missing_trailing_dims_count_as_one():
    # onednn/Pool2D.cpp:95-98: a [W,H] tensor pools as [W,H,1,1]
    x = _x((6, 8), 44)
    y, _ = fa.pool2d(dev(x), 2, 2, 2, 2, 0, 0)
    d = flref.pool_desc((1, 1, 6, 8), (2, 2), (2, 2), (0, 0), 0)
    assert np.array_equal(host(y)[0, 0], flref.pool2d_fwd(d, x)[0][0, 0])


def test_backward_without_payload_raises():
    dy = torch.zeros((1, 1, 4, 4), device="cuda")
    with pytest.raises(ValueError):
        fa.pool2d_backward(dy, (1, 1, 8, 8), None, 2, 2, 2, 2, 0, 0, mode=0)


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_full_size_oracle(mode):
    """configs[2] at its stated size (112x112x64, batch 32, values on a 1/8 grid so that ties
    occur in most windows): values, argmax bytes and the routed gradient bit for bit against
    the CPU checker."""
    rng = np.random.default_rng(46)
    x = (np.round(rng.standard_normal((32, 64, 112, 112), dtype=np.float32) * 8) / 8).astype(np.float32)
    dy = rng.standard_normal((32, 64, 56, 56), dtype=np.float32)
    d = flref.pool_desc(x.shape, (3, 3), (2, 2), (1, 1), mode)
    y_ref, am_ref = flref.pool2d_fwd(d, x)
    dx_ref = flref.pool2d_bwd(d, dy, am_ref)
    y, am = fa.pool2d(dev(x), 3, 3, 2, 2, 1, 1, mode=mode)
    dx = fa.pool2d_backward(dev(dy), x.shape, am, 3, 3, 2, 2, 1, 1, mode=mode)
    assert np.array_equal(host(y), y_ref)
    if mode == 0:
        am_h = am.cpu().numpy()
        assert np.array_equal(am_h, am_ref)
        # the grid does produce ties: count windows whose maximum occurs more than once
        xp = np.pad(x[:2], ((0, 0), (0, 0), (1, 1), (1, 1)), constant_values=-np.inf)
        hits = sum((xp[:, :, kh:kh + 111:2, kw:kw + 111:2] == y_ref[:2]).astype(np.int32)
                   for kh in range(3) for kw in range(3))
        assert (hits >= 2).mean() > 0.05
    assert np.array_equal(host(dx), dx_ref)


def test_full_size_properties():
    # cfg-3 size, independent of the checker: gradient mass is conserved and
    # max-pooling routes every output to a position that holds its value.
    g = torch.Generator(device="cuda").manual_seed(45)
    x = torch.round(torch.randn((32, 64, 112, 112), device="cuda", generator=g) * 8) / 8
    dy = torch.randn((32, 64, 56, 56), device="cuda", generator=g)
    for mode in (0, 2):
        y, am = fa.pool2d(x, 3, 3, 2, 2, 1, 1, mode=mode)
        dx = fa.pool2d_backward(dy, x.shape, am, 3, 3, 2, 2, 1, 1, mode=mode)
        assert abs(dx.double().sum().item() - dy.double().sum().item()) < 1e-2
        if mode == 0:
            # routing dy = y through the argmax and reading x there returns y
            probe = fa.pool2d_backward(torch.ones_like(y), x.shape, am, 3, 3, 2, 2, 1, 1, mode=0)
            assert probe.sum().item() == y.numel()
            assert (x[probe > 0].max() == y.max()).item()
