"""Pins oracle/flref.c's batch normalisation."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import flref
from refmath import rel_l2


def _to_whcn(a):
    """row-major N,C,H,W array -> numpy array indexed [w,h,c,n] (Flashlight order)."""
    return np.transpose(a, (3, 2, 1, 0))


def test_view_rule():
    # flashlight/fl/autograd/tensor/backend/onednn/BatchNorm.cpp:40-71
    assert flref.bn_view([13, 13, 3, 8], [2]) == (8, 3, 169)
    assert flref.bn_view([13, 13, 4, 8], [0, 1, 2]) == (8, 676, 1)
    assert flref.bn_view([5, 6, 7, 8], [1, 2]) == (8, 42, 5)
    assert flref.bn_view([5, 6, 7, 8], [0, 1, 2, 3]) == (1, 1680, 1)
    with pytest.raises(ValueError):
        flref.bn_view([5, 6, 7, 8], [0, 2])


def test_train_closed_form_single_axis():
    # AutogradNormalizationTest.cpp:158-189: [13,13,3,8], axes {2}, population
    # variance, eps 1e-5, tolerance 1e-5.
    rng = np.random.default_rng(20)
    x = rng.random((8, 3, 13, 13)).astype(np.float32)
    g = rng.random(3).astype(np.float32); b = rng.random(3).astype(np.float32)
    outer, C, inner = flref.bn_view([13, 13, 3, 8], [2])
    y, mean, var = flref.bn_fwd_train(outer, C, inner, x, g, b, 1e-5)
    x64 = x.astype(np.float64)
    mu = x64.mean(axis=(0, 2, 3), keepdims=True)
    v = x64.var(axis=(0, 2, 3), keepdims=True)
    exp = (x64 - mu) / np.sqrt(v + 1e-5) * g.reshape(1, 3, 1, 1) + b.reshape(1, 3, 1, 1)
    assert np.allclose(y, exp, atol=1e-5, rtol=0)
    assert np.allclose(mean, mu.ravel(), atol=1e-6) and np.allclose(var, v.ravel(), atol=1e-6)


def test_train_closed_form_multi_axis():
    # AutogradNormalizationTest.cpp:191-226: [13,13,4,8], axes {0,1,2}: one
    # feature per (w,h,c), statistics over the batch only.
    rng = np.random.default_rng(21)
    x = rng.random((8, 4, 13, 13)).astype(np.float32)
    nf = 13 * 13 * 4
    g = rng.random(nf).astype(np.float32); b = rng.random(nf).astype(np.float32)
    outer, C, inner = flref.bn_view([13, 13, 4, 8], [0, 1, 2])
    y, _, _ = flref.bn_fwd_train(outer, C, inner, x, g, b, 1e-5)
    xw, yw = _to_whcn(x).astype(np.float64), _to_whcn(y)
    for i in range(0, nf, 37):
        sel = (i % 13, (i // 13) % 13, (i // 13) // 13)
        t = xw[sel]
        exp = (t - t.mean()) / np.sqrt(t.var() + 1e-5) * g[i] + b[i]
        assert np.allclose(yw[sel], exp, atol=1e-5, rtol=0)


def test_eval_closed_form():
    # AutogradNormalizationTest.cpp:37-92 (single axis, with and without affine)
    rng = np.random.default_rng(22)
    x = rng.random((16, 3, 13, 13)).astype(np.float32)
    rm, rv, g, b = (rng.random(3).astype(np.float32) for _ in range(4))
    outer, C, inner = flref.bn_view([13, 13, 3, 16], [2])
    sh = (1, 3, 1, 1)
    y = flref.bn_fwd_infer(outer, C, inner, x, g, b, rm, rv, 1e-5)
    exp = (x - rm.reshape(sh)) / np.sqrt(rv.reshape(sh) + 1e-5) * g.reshape(sh) + b.reshape(sh)
    assert np.allclose(y, exp, atol=1e-5, rtol=0)
    y = flref.bn_fwd_infer(outer, C, inner, x, None, None, rm, rv, 1e-5)
    assert np.allclose(y, (x - rm.reshape(sh)) / np.sqrt(rv.reshape(sh) + 1e-5), atol=1e-5, rtol=0)


@pytest.mark.parametrize("shape,axes", [((5, 4, 6, 7), [2]), ((3, 5, 4, 6), [0, 1, 2]), ((6, 3, 2, 5), [1, 2])])
def test_backward_against_autograd_of_closed_form(shape, axes):
    # shape is row-major N,C,H,W; Flashlight shape is its reverse.
    rng = np.random.default_rng(23)
    whcn = list(shape[::-1])
    outer, C, inner = flref.bn_view(whcn, axes)
    x = (rng.standard_normal(shape) * 1.5 + 0.5).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    b = rng.standard_normal(C).astype(np.float32)
    y, mean, var = flref.bn_fwd_train(outer, C, inner, x, g, b, 1e-5)
    dx, dg, db = flref.bn_bwd(outer, C, inner, x, dy, g, mean, var, 1e-5)
    xt = torch.tensor(x, dtype=torch.float64).reshape(outer, C, inner).requires_grad_(True)
    gt = torch.tensor(g, dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(b, dtype=torch.float64, requires_grad=True)
    mu = xt.mean(dim=(0, 2), keepdim=True)
    v = ((xt - mu) ** 2).mean(dim=(0, 2), keepdim=True)
    yt = (xt - mu) / torch.sqrt(v + 1e-5) * gt.reshape(1, C, 1) + bt.reshape(1, C, 1)
    assert rel_l2(y, yt.detach().numpy().reshape(shape)) < 1e-6
    yt.backward(torch.tensor(dy, dtype=torch.float64).reshape(outer, C, inner))
    assert rel_l2(dx, xt.grad.numpy().reshape(shape)) < 1e-5
    assert rel_l2(dg, gt.grad.numpy()) < 1e-5
    assert rel_l2(db, bt.grad.numpy()) < 1e-5
    # invariants of the formula: dx is orthogonal to 1 and to xhat per feature
    d3 = dx.astype(np.float64).reshape(outer, C, inner)
    xh = ((x.reshape(outer, C, inner) - mean.reshape(1, C, 1)) / np.sqrt(var.reshape(1, C, 1) + 1e-5))
    assert np.abs(d3.sum(axis=(0, 2))).max() < 1e-4
    # (exactly so only for eps -> 0: sum(xhat^2) = M*var/(var+eps))
    assert (np.abs((d3 * xh).sum(axis=(0, 2))) <= 1e-4 + 1e-2 * np.abs(d3 * xh).sum(axis=(0, 2))).all()
    assert np.allclose(db, dy.reshape(outer, C, inner).sum(axis=(0, 2)), atol=1e-4)


def test_against_library_routine():
    # F.batch_norm on CPU (fwd + autograd backward), spatial mode
    rng = np.random.default_rng(24)
    x = (rng.standard_normal((6, 5, 7, 9)) * np.sqrt(2) + 0.5).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(5)).astype(np.float32)
    b = rng.standard_normal(5).astype(np.float32)
    dy = rng.standard_normal(x.shape).astype(np.float32)
    y, mean, var = flref.bn_fwd_train(6, 5, 63, x, g, b, 1e-5)
    xt = torch.tensor(x, requires_grad=True); gt = torch.tensor(g, requires_grad=True)
    bt = torch.tensor(b, requires_grad=True)
    rm, rv = torch.zeros(5), torch.ones(5)
    yt = F.batch_norm(xt, rm, rv, gt, bt, True, 0.1, 1e-5)
    yt.backward(torch.tensor(dy))
    assert rel_l2(y, yt.detach().numpy()) < 1e-5
    dx, dg, db = flref.bn_bwd(6, 5, 63, x, dy, g, mean, var, 1e-5)
    assert rel_l2(dx, xt.grad.numpy()) < 1e-4
    assert rel_l2(dg, gt.grad.numpy()) < 1e-5 and rel_l2(db, bt.grad.numpy()) < 1e-5
    # running statistics with momentum: PyTorch blends with the unbiased variance,
    # the same rule cuDNN applies
    r_m, r_v = flref.bn_running_update(6 * 63, mean, var, 0.1, np.zeros(5), np.ones(5))
    assert np.allclose(r_m, rm.numpy(), atol=1e-6) and np.allclose(r_v, rv.numpy(), atol=1e-6)
    # momentum 0: the oneDNN extension leaves the batch statistics in the buffers
    r_m, r_v = flref.bn_running_update(6 * 63, mean, var, 0.0, np.zeros(5), np.ones(5))
    assert np.array_equal(r_m, mean) and np.array_equal(r_v, var)


def test_against_onednn_batchnorm_through_mkldnn_tensor():
    rng = np.random.default_rng(25)
    x = (rng.standard_normal((4, 3, 6, 5)) + 0.5).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(3)).astype(np.float32)
    b = rng.standard_normal(3).astype(np.float32)
    y, _, _ = flref.bn_fwd_train(4, 3, 30, x, g, b, 1e-5)
    yt = F.batch_norm(torch.tensor(x).to_mkldnn(), torch.zeros(3), torch.ones(3),
                      torch.tensor(g), torch.tensor(b), True, 0.0, 1e-5).to_dense()
    assert np.allclose(y, yt.numpy(), atol=1e-5, rtol=0)
