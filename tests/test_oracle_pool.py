"""Pins oracle/flref.c's pooling (values, tie order, argmax bytes, backward)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import flref
from refmath import brute_pool_bwd, brute_pool_fwd

GEOMS = [
    # x shape, window (y,x), stride, pad
    ((2, 3, 8, 8), (3, 3), (2, 2), (1, 1)),
    ((1, 2, 7, 9), (2, 2), (2, 2), (0, 0)),
    ((1, 2, 9, 7), (3, 2), (1, 2), (1, 0)),
    ((2, 1, 6, 6), (2, 3), (1, 1), (1, 1)),
    ((1, 1, 3, 3), (2, 2), (1, 1), (0, 0)),   # AutogradTest.cpp:333-337
    ((1, 4, 7, 7), (7, 7), (1, 1), (0, 0)),   # global average, Resnet.cpp:225
]


def _x(shape, seed):
    # values on a 1/8 grid so that equal maxima occur inside windows
    return (np.round(np.random.default_rng(seed).standard_normal(shape) * 8) / 8).astype(np.float32)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("mode", [0, 1, 2])
def test_brute_force_bit_exact(geom, mode):
    xs, win, st, pd = geom
    x = _x(xs, 11)
    d = flref.pool_desc(xs, win, st, pd, mode)
    y, am = flref.pool2d_fwd(d, x)
    yb, amb = brute_pool_fwd(x, win, st, pd, mode)
    assert np.array_equal(y, yb)
    if mode == 0:
        assert np.array_equal(am, amb)
    dy = np.random.default_rng(12).standard_normal(y.shape).astype(np.float32)
    dx = flref.pool2d_bwd(d, dy, am)
    assert np.array_equal(dx, brute_pool_bwd(dy, amb, xs, win, st, pd, mode))


def test_ties_take_first_in_scan_order():
    x = np.zeros((1, 1, 4, 4), np.float32)      # every window is all ties
    d = flref.pool_desc(x.shape, (3, 3), (1, 1), (1, 1), 0)
    _, am = flref.pool2d_fwd(d, x)
    # first in-bounds position: top row of outputs skips kh=0, left column skips kw=0
    assert am[0, 0, 0, 0] == 1 * 3 + 1
    assert am[0, 0, 0, 1] == 1 * 3 + 0
    assert am[0, 0, 1, 0] == 0 * 3 + 1
    assert am[0, 0, 2, 2] == 0
    x[0, 0, 1, 1] = 1; x[0, 0, 1, 2] = 1; x[0, 0, 2, 1] = 1
    _, am = flref.pool2d_fwd(d, x)
    assert am[0, 0, 2, 2] == 0                  # (1,1) seen first
    assert am[0, 0, 1, 3] == 1 * 3 + 0          # window cols 2..4: (1,2) first


@pytest.mark.parametrize("geom", GEOMS)
def test_max_against_library_indices(geom):
    # ATen max_pool2d_with_indices and oneDNN's pooling both keep the first
    # maximum; ATen's index is the flat input offset ih*W+iw.
    xs, win, st, pd = geom
    x = _x(xs, 13)
    d = flref.pool_desc(xs, win, st, pd, 0)
    y, am = flref.pool2d_fwd(d, x)
    yt, it = F.max_pool2d(torch.tensor(x), win, st, pd, return_indices=True)
    assert np.array_equal(y, yt.numpy())
    oh, ow = np.meshgrid(np.arange(y.shape[2]), np.arange(y.shape[3]), indexing="ij")
    ih = oh * st[0] - pd[0] + am // win[1]
    iw = ow * st[1] - pd[1] + am % win[1]
    assert np.array_equal(ih * xs[3] + iw, it.numpy())


@pytest.mark.parametrize("geom", GEOMS[:4])
def test_max_against_onednn_through_mkldnn_tensor(geom):
    xs, win, st, pd = geom
    x = _x(xs, 14)
    d = flref.pool_desc(xs, win, st, pd, 0)
    y, am = flref.pool2d_fwd(d, x)
    dy = np.random.default_rng(15).standard_normal(y.shape).astype(np.float32)
    xt = torch.tensor(x, requires_grad=True)
    yt = torch.max_pool2d(xt.to_mkldnn(), win, st, pd).to_dense()
    yt.backward(torch.tensor(dy))
    assert np.array_equal(y, yt.detach().numpy())
    assert np.allclose(flref.pool2d_bwd(d, dy, am), xt.grad.numpy(), rtol=0, atol=1e-6)


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("mode", [1, 2])
def test_avg_against_library(geom, mode):
    xs, win, st, pd = geom
    x = _x(xs, 16)
    d = flref.pool_desc(xs, win, st, pd, mode)
    y, _ = flref.pool2d_fwd(d, x)
    xt = torch.tensor(x, requires_grad=True)
    yt = F.avg_pool2d(xt, win, st, pd, count_include_pad=(mode == 1))
    assert np.allclose(y, yt.detach().numpy(), rtol=1e-6, atol=1e-6)
    dy = np.random.default_rng(17).standard_normal(y.shape).astype(np.float32)
    yt.backward(torch.tensor(dy))
    assert np.allclose(flref.pool2d_bwd(d, dy), xt.grad.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("mode", [0, 2])
def test_gradient_mass_is_conserved(mode):
    xs, win, st, pd = GEOMS[0]
    x = _x(xs, 18)
    d = flref.pool_desc(xs, win, st, pd, mode)
    y, am = flref.pool2d_fwd(d, x)
    dy = np.random.default_rng(19).standard_normal(y.shape).astype(np.float32)
    dx = flref.pool2d_bwd(d, dy, am)
    assert abs(dx.astype(np.float64).sum() - dy.astype(np.float64).sum()) < 1e-4
