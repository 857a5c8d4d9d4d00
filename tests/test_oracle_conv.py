"""Pins oracle/flref.c's convolution against definitions that share no code with it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import flref
from refmath import brute_conv_bwd, brute_conv_fwd, rel_l2

CASES = [
    # x shape (N,C,H,W), w shape (K,C/g,KH,KW), stride, pad, dil, groups
    ((2, 3, 7, 6), (4, 3, 3, 3), (1, 1), (1, 1), (1, 1), 1),
    ((1, 4, 8, 9), (6, 2, 3, 2), (2, 1), (0, 2), (1, 1), 2),
    ((2, 2, 9, 9), (2, 2, 3, 3), (1, 2), (2, 1), (2, 2), 1),
    ((1, 6, 6, 11), (3, 2, 1, 5), (1, 3), (0, 2), (1, 2), 3),
    ((3, 1, 5, 5), (2, 1, 5, 5), (1, 1), (2, 2), (1, 1), 1),
    ((1, 3, 10, 4), (5, 3, 1, 1), (2, 2), (0, 0), (1, 1), 1),
]


def _mk(case, seed=0, bias=True):
    xs, ws, st, pd, dl, g = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(xs).astype(np.float32)
    w = rng.standard_normal(ws).astype(np.float32)
    b = rng.standard_normal(ws[0]).astype(np.float32) if bias else None
    d = flref.conv_desc(xs, ws, st, pd, dl, g)
    return x, w, b, d


@pytest.mark.parametrize("case", CASES)
def test_brute_force(case):
    x, w, b, d = _mk(case)
    _, _, st, pd, dl, g = case
    y = flref.conv2d_fwd(d, x, w, b)
    yb = brute_conv_fwd(x, w, b, st, pd, dl, g)
    assert y.shape == yb.shape
    assert rel_l2(y, yb) < 1e-6
    dy = np.random.default_rng(1).standard_normal(y.shape).astype(np.float32)
    gx, gw, gb = brute_conv_bwd(x, w, dy, st, pd, dl, g)
    assert rel_l2(flref.conv2d_bwd_data(d, dy, w), gx) < 1e-6
    dw, db = flref.conv2d_bwd_filter(d, x, dy)
    assert rel_l2(dw, gw) < 1e-6
    assert rel_l2(db, gb) < 1e-6


@pytest.mark.parametrize("case", CASES)
def test_adjoint_identities(case):
    # <conv(x,w), dy> == <x, bwdData(dy,w)> == <w, bwdFilter(x,dy)>
    x, w, _, d = _mk(case, seed=3, bias=False)
    y = flref.conv2d_fwd(d, x, w, None).astype(np.float64)
    dy = np.random.default_rng(4).standard_normal(y.shape).astype(np.float32)
    lhs = float((y * dy).sum())
    dx = flref.conv2d_bwd_data(d, dy, w).astype(np.float64)
    dw, db = flref.conv2d_bwd_filter(d, x, dy)
    scale = np.abs(y * dy).sum()
    assert abs(lhs - float((dx * x).sum())) < 1e-5 * scale
    assert abs(lhs - float((dw.astype(np.float64) * w).sum())) < 1e-5 * scale
    assert np.allclose(db, dy.sum(axis=(0, 2, 3)), rtol=1e-5, atol=1e-5)


def test_1x1_is_gemm():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 8, 5, 7)).astype(np.float32)
    w = rng.standard_normal((6, 8, 1, 1)).astype(np.float32)
    d = flref.conv_desc(x.shape, w.shape)
    y = flref.conv2d_fwd(d, x, w, None)
    ref = np.einsum("kc,nchw->nkhw", w[:, :, 0, 0].astype(np.float64), x.astype(np.float64))
    assert rel_l2(y, ref) < 1e-6


def test_batching_invariance():
    # flashlight/fl/test/nn/ModuleTest.cpp:338-353: 30->50 channels, 9x7 kernel,
    # stride 2x3, pad 3x2 — the batched result equals the per-sample results.
    rng = np.random.default_rng(6)
    x = rng.standard_normal((4, 30, 17, 20)).astype(np.float32)
    w = rng.standard_normal((50, 30, 7, 9)).astype(np.float32)
    b = rng.standard_normal(50).astype(np.float32)
    d = flref.conv_desc(x.shape, w.shape, (3, 2), (2, 3))
    y = flref.conv2d_fwd(d, x, w, b)
    for n in range(4):
        d1 = flref.conv_desc((1,) + x.shape[1:], w.shape, (3, 2), (2, 3))
        y1 = flref.conv2d_fwd(d1, x[n:n + 1], w, b)
        assert np.array_equal(y1[0], y[n])


LIB_CASES = CASES + [
    # flashlight/fl/test/autograd/AutogradConv2DTest.cpp:21-74: input [10,9,8,7],
    # weights [4,3,8,6], px=2, py=1 (row-major: x (7,8,9,10), w (6,8,3,4)).
    ((7, 8, 9, 10), (6, 8, 3, 4), (1, 1), (1, 2), (1, 1), 1),
    # :137-162 groups = 2 ; :164-213 dilation 2
    ((7, 8, 9, 10), (6, 4, 3, 4), (1, 1), (1, 2), (1, 1), 2),
    ((7, 8, 9, 10), (6, 8, 3, 4), (1, 1), (1, 2), (2, 2), 1),
    ((2, 16, 14, 14), (24, 16, 3, 3), (2, 2), (1, 1), (1, 1), 1),
]


@pytest.mark.parametrize("case", LIB_CASES)
def test_against_library_routine(case):
    # PyTorch-CPU's convolution (oneDNN v3.7.1 direct convolution on this image)
    x, w, b, d = _mk(case, seed=7)
    _, _, st, pd, dl, g = case
    xt = torch.tensor(x, requires_grad=True)
    wt = torch.tensor(w, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    yt = F.conv2d(xt, wt, bt, stride=st, padding=pd, dilation=dl, groups=g)
    y = flref.conv2d_fwd(d, x, w, b)
    assert rel_l2(y, yt.detach().numpy()) < 1e-5
    dy = np.random.default_rng(8).standard_normal(y.shape).astype(np.float32)
    yt.backward(torch.tensor(dy))
    assert rel_l2(flref.conv2d_bwd_data(d, dy, w), xt.grad.numpy()) < 1e-5
    dw, db = flref.conv2d_bwd_filter(d, x, dy)
    assert rel_l2(dw, wt.grad.numpy()) < 1e-5
    assert rel_l2(db, bt.grad.numpy()) < 1e-5


def test_finite_difference_jacobian():
    # flashlight/fl/test/autograd/AutogradTestUtils.h:32-70: central differences,
    # perturbation 1e-4 (done here in float64 on the brute-force forward).
    case = ((1, 2, 5, 4), (3, 2, 3, 2), (1, 1), (1, 0), (1, 1), 1)
    x, w, b, d = _mk(case, seed=9)
    _, _, st, pd, dl, g = case
    dy = np.random.default_rng(10).standard_normal(flref.conv2d_fwd(d, x, w, b).shape).astype(np.float32)
    dx = flref.conv2d_bwd_data(d, dy, w)
    dw, _ = flref.conv2d_bwd_filter(d, x, dy)
    h = 1e-4

    def loss(xx, ww):
        return float((brute_conv_fwd(xx, ww, b, st, pd, dl, g) * dy).sum())

    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    for idx in [(0, 0, 0, 0), (0, 1, 2, 3), (0, 1, 4, 1)]:
        xp, xm = x64.copy(), x64.copy()
        xp[idx] += h; xm[idx] -= h
        assert abs((loss(xp, w64) - loss(xm, w64)) / (2 * h) - dx[idx]) < 1e-3
    for idx in [(0, 0, 0, 0), (2, 1, 2, 1)]:
        wp, wm = w64.copy(), w64.copy()
        wp[idx] += h; wm[idx] -= h
        assert abs((loss(x64, wp) - loss(x64, wm)) / (2 * h) - dw[idx]) < 1e-3


def test_out_dims_and_same_padding():
    # flashlight/fl/nn/Utils.cpp:87-100 (SAME) with onednn/Conv2D.cpp:179-188
    def same_pad(n, k, s, dl):
        rem = n % s
        return max(((k - 1) * dl - (s if rem == 0 else rem) + 1 + 1) // 2, 0)
    for n, k, s in [(56, 3, 1), (224, 7, 2), (56, 1, 2), (1500, 21, 2), (28, 5, 1), (112, 3, 2)]:
        p = same_pad(n, k, s, 1)
        d = flref.conv_desc((1, 1, n, n), (1, 1, k, k), (s, s), (p, p))
        assert flref.conv_out(d) == (-(-n // s), -(-n // s))
