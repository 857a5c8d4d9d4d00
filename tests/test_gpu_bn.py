"""GPU parity: batchnorm / batchnormBackward through the C ABI against the CPU
checker (fp32 relative L2 <= 1e-4; bf16 storage <= 2e-2)."""
import numpy as np
import pytest
import torch

import flashlight_amd as fa
from gpu_util import bf16_round, dev, host, round_to
from oracle import flref
from refmath import rel_l2

pytestmark = pytest.mark.gpu

# (row-major shape N,C,H,W ; Flashlight feature axes)
CASES = [
    ((8, 3, 13, 13), [2]),          # AutogradNormalizationTest.cpp:158-189
    ((8, 4, 13, 13), [0, 1, 2]),    # :191-226 per-activation
    ((4, 16, 14, 14), [2]),         # inner % 4 == 0
    ((2, 5, 3, 7), [1, 2]),         # features over (H,C)
    ((1, 7, 5, 6), [0, 1, 2, 3]),   # LayerNorm-style: every element its own feature
    ((16, 250, 1, 75), [2]),        # speech stack shape [T,1,250,B]
    ((6, 300, 2, 2), [2]),          # many features, tiny inner
    ((64, 10), [0]),                # 2-D, per-activation
    ((3, 2, 56, 56), [2]),          # long rows
    ((8, 8, 130, 3), [2]),          # one workgroup per feature, mostly idle lanes
    ((28, 28, 128, 9), [2]),        # one workgroup of 256 threads per feature
    ((28, 28, 128, 20), [2]),       # one workgroup of 1024 threads per feature, 8 vectors per thread
    ((56, 56, 128, 11), [2]),       # ... 16 vectors per thread
    ((56, 56, 128, 22), [2]),       # ... 25 vectors per thread, part of dy re-read
    # rows that are not 16-byte friendly: element-wise resident kernels
    ((4, 130, 7, 7), [2]),          # 256 threads, mostly idle slots
    ((32, 128, 7, 7), [2]),         # the 7x7 planes of the last ResNet stage
    ((12, 128, 1, 750), [2]),       # speech rows after the stride-2 layer, 16 elements per thread
    ((5, 128, 53, 101), [2]),       # 32 elements per thread
    ((3, 64, 9, 9), [2]),           # forward resident, backward split (fewer than 128 features)
    # bf16 storage: the 8-wide resident kernels (rows of a multiple of 8 elements) with 256 threads, and with
    # 8 / 16 / 25 vectors per thread; fp32 takes the two-pass kernels for the largest
    ((4, 128, 16, 16), [2]),
    ((20, 128, 56, 56), [2]),
    ((40, 128, 56, 56), [2]),
    ((48, 128, 56, 56), [2]),
    # configs[3] at its stated size: [T, 1, 250, B] with T = 1500 and, after the stride-2 layer, 750
    ((16, 250, 1, 1500), [2]),
    ((16, 250, 1, 750), [2]),
    # configs[4] at batch 64: features beyond one workgroup's registers (fp32 56x56 planes, the stem's
    # 112x112 planes in both storage types)
    ((64, 256, 56, 56), [2]),
    ((64, 64, 112, 112), [2]),
]


def _data(shape, axes, seed, dtype):
    rng = np.random.default_rng(seed)
    outer, C, inner = flref.bn_view(list(shape[::-1]), axes)
    x = (rng.standard_normal(shape) * np.sqrt(2) + 0.5).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    x, dy = round_to(x, dtype), round_to(dy, dtype)
    g = (1 + 0.1 * rng.standard_normal(C)).astype(np.float32)
    b = rng.standard_normal(C).astype(np.float32)
    return outer, C, inner, x, dy, g, b


# f16 storage takes the kernels of the other two types with its own loads, stores and conversions (the 8-wide resident
# kernels hold bf16 and f16 alike as raw words): the shapes up to 20M elements, which reach every vector count of those
TYPED_CASES = ([(s, a, dt) for s, a in CASES for dt in (torch.float32, torch.bfloat16)] +
               [(s, a, torch.float16) for s, a in CASES if int(np.prod(s)) <= 20 << 20])


@pytest.mark.parametrize("shape,axes,dtype", TYPED_CASES)
def test_train_forward_backward(shape, axes, dtype):
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    outer, C, inner, x, dy, g, b = _data(shape, axes, 50, dtype)
    y_ref, mean, var = flref.bn_fwd_train(outer, C, inner, x, g, b, 1e-5)
    dx_ref, dg_ref, db_ref = flref.bn_bwd(outer, C, inner, x, dy, g, mean, var, 1e-5)
    rm, rv = dev(np.zeros(C, np.float32)), dev(np.ones(C, np.float32))
    xd, dyd = dev(x, dtype), dev(dy, dtype)
    y, sm, si = fa.batchnorm(xd, dev(g), dev(b), rm, rv, axes, True, 0.1, 1e-5)
    dx, dg, db = fa.batchnorm_backward(dyd, xd, dev(g), sm, si, axes)
    assert rel_l2(host(y), y_ref) <= tol
    assert np.allclose(host(sm), mean, rtol=1e-5, atol=1e-6)
    assert np.allclose(host(si), 1 / np.sqrt(var.astype(np.float64) + 1e-5), rtol=1e-4)
    rm_ref, rv_ref = flref.bn_running_update(outer * inner, mean, var, 0.1, np.zeros(C), np.ones(C))
    assert np.allclose(host(rm), rm_ref, rtol=1e-5, atol=1e-6)
    assert np.allclose(host(rv), rv_ref, rtol=1e-4, atol=1e-6)
    # (a feature with a single sample has dx == 0 exactly: absolute check there)
    assert rel_l2(host(dx), dx_ref) <= tol or np.abs(host(dx) - dx_ref).max() <= 1e-4
    # with bf16 storage the checker sees the same rounded inputs; parameter
    # gradients are fp32 sums
    assert rel_l2(host(dg), dg_ref) <= 1e-4 or np.abs(host(dg) - dg_ref).max() <= 1e-4
    assert rel_l2(host(db), db_ref) <= 1e-4


def test_momentum_zero_overwrites_running_stats_like_onednn():
    # onednn/BatchNorm.cpp:154-157
    shape, axes = CASES[0]
    outer, C, inner, x, _, g, b = _data(shape, axes, 51, torch.float32)
    _, mean, var = flref.bn_fwd_train(outer, C, inner, x, g, b, 1e-5)
    rm, rv = dev(np.full(C, 7, np.float32)), dev(np.full(C, 9, np.float32))
    fa.batchnorm(dev(x), dev(g), dev(b), rm, rv, axes, True, 0.0, 1e-5)
    assert np.allclose(host(rm), mean, rtol=1e-5, atol=1e-6)
    assert np.allclose(host(rv), var, rtol=1e-4, atol=1e-6)


def test_no_affine_and_no_running_stats():
    shape, axes = CASES[2]
    outer, C, inner, x, dy, _, _ = _data(shape, axes, 52, torch.float32)
    y_ref, mean, var = flref.bn_fwd_train(outer, C, inner, x, None, None, 1e-5)
    y, sm, si = fa.batchnorm(dev(x), None, None, None, None, axes, True, 0.0, 1e-5)
    assert rel_l2(host(y), y_ref) <= 1e-4
    dx_ref, _, _ = flref.bn_bwd(outer, C, inner, x, dy, None, mean, var, 1e-5)
    dx, _, _ = fa.batchnorm_backward(dev(dy), dev(x), None, sm, si, axes)
    assert rel_l2(host(dx), dx_ref) <= 1e-4


@pytest.mark.parametrize("shape,axes", CASES[:3])
def test_inference(shape, axes):
    # AutogradNormalizationTest.cpp:37-156
    outer, C, inner, x, _, g, b = _data(shape, axes, 53, torch.float32)
    rng = np.random.default_rng(54)
    rm, rv = rng.random(C).astype(np.float32), rng.random(C).astype(np.float32)
    y_ref = flref.bn_fwd_infer(outer, C, inner, x, g, b, rm, rv, 1e-5)
    y, sm, si = fa.batchnorm(dev(x), dev(g), dev(b), dev(rm), dev(rv), axes, False, 0.0, 1e-5)
    assert sm is None and si is None
    assert np.allclose(host(y), y_ref, atol=1e-5, rtol=1e-5)


def test_large_mean_small_variance():
    # a shifted-sum variance must survive mean >> std
    rng = np.random.default_rng(55)
    x = (1000.0 + 0.01 * rng.standard_normal((4, 8, 16, 16))).astype(np.float32)
    y_ref, mean, var = flref.bn_fwd_train(4, 8, 256, x, None, None, 1e-5)
    y, sm, si = fa.batchnorm(dev(x), None, None, None, None, [2], True, 0.0, 1e-5)
    # the fp32 mean itself is only known to 6e-5 here (ulp of 1000), 0.6% of the std
    assert rel_l2(host(y), y_ref) <= 1e-2
    assert np.allclose(host(sm), mean, rtol=1e-6)
    assert np.allclose(host(si), 1 / np.sqrt(var.astype(np.float64) + 1e-5), rtol=1e-3)


def test_errors():
    x = torch.zeros((2, 3, 4, 4), device="cuda")
    with pytest.raises(ValueError):
        fa.batchnorm(x, None, None, None, None, [0, 2], True, 0.0, 1e-5)   # axes not contiguous
    with pytest.raises(ValueError):
        fa.batchnorm_backward(x, x, None, None, None, [2])                 # no payload
    with pytest.raises(ValueError):
        fa.batchnorm(x, torch.zeros(5, device="cuda"), None, None, None, [2], True, 0.0, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_full_size_oracle(dtype):
    """configs[2] at its stated size (56x56x256, batch 32, values N(0.5, 2), gamma N(1, 0.1),
    eps 1e-5, momentum 0.1): y, saved statistics, running statistics, dx, dgamma, dbeta
    against the CPU checker, whole tensors."""
    rng = np.random.default_rng(57)
    N, Cc, HW = 32, 256, 56 * 56
    x = (rng.standard_normal((N, Cc, 56, 56), dtype=np.float32) * np.float32(2 ** 0.5) + np.float32(0.5))
    dy = rng.standard_normal((N, Cc, 56, 56), dtype=np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(Cc)).astype(np.float32)
    beta = np.zeros(Cc, np.float32)
    lo = dtype != torch.float32
    if lo:
        x, dy = round_to(x, dtype), round_to(dy, dtype)
    y_ref, mean, var = flref.bn_fwd_train(N, Cc, HW, x, gamma, beta, 1e-5)
    dx_ref, dg_ref, db_ref = flref.bn_bwd(N, Cc, HW, x, dy, gamma, mean, var, 1e-5)
    rm, rv = torch.zeros(Cc, device="cuda"), torch.ones(Cc, device="cuda")
    xd, dyd = dev(x, dtype), dev(dy, dtype)
    y, sm, si = fa.batchnorm(xd, dev(gamma), dev(beta), rm, rv, [2], True, 0.1, 1e-5)
    dx, dg, db = fa.batchnorm_backward(dyd, xd, dev(gamma), sm, si, [2])
    tol = 4e-3 if lo else 1e-4
    assert rel_l2(host(y), y_ref) <= tol
    assert rel_l2(host(dx), dx_ref) <= tol
    assert rel_l2(host(dg), dg_ref) <= 1e-4 and rel_l2(host(db), db_ref) <= 1e-4
    assert rel_l2(host(sm), mean) <= 1e-5
    assert rel_l2(host(si), 1 / np.sqrt(var.astype(np.float64) + 1e-5)) <= 1e-5
    M = N * HW
    assert rel_l2(host(rm), 0.1 * mean) <= 1e-5
    assert rel_l2(host(rv), 0.9 + 0.1 * var.astype(np.float64) * M / (M - 1)) <= 1e-5


def test_full_size_invariants():
    # cfg-3 shape: per-feature sums of dx and of dx*xhat vanish; y has zero mean
    # and unit variance per feature.
    g = torch.Generator(device="cuda").manual_seed(56)
    x = torch.randn((32, 256, 56, 56), device="cuda", generator=g) * (2 ** 0.5) + 0.5
    dy = torch.randn((32, 256, 56, 56), device="cuda", generator=g)
    gamma = 1 + 0.1 * torch.randn(256, device="cuda", generator=g)
    y, sm, si = fa.batchnorm(x, gamma, None, None, None, [2], True, 0.1, 1e-5)
    ym = y.double().mean(dim=(0, 2, 3)); yv = y.double().var(dim=(0, 2, 3), unbiased=False)
    assert ym.abs().max().item() < 1e-4
    assert torch.allclose(yv, gamma.double() ** 2, rtol=1e-3)
    dx, dg, db = fa.batchnorm_backward(dy, x, gamma, sm, si, [2])
    assert torch.allclose(db.double(), dy.double().sum(dim=(0, 2, 3)), rtol=1e-4, atol=1e-2)
    s = dx.double().sum(dim=(0, 2, 3)).abs().max().item()
    assert s < 1e-1, s     # 1e5 elements per feature of magnitude ~1
    xh = (x.double() - sm.double().view(1, -1, 1, 1)) * si.double().view(1, -1, 1, 1)
    assert (dx.double() * xh).sum(dim=(0, 2, 3)).abs().max().item() < 1.0


# ---- batch norm fused with ReLU and the residual add ---------------------------------------
# against the checker's composition batchnorm -> (+ residual) -> relu and relu' -> batchnormBackward,
# over every kernel family (resident 4-wide with 8 / 16 / 25 vectors, element-wise resident, split)
FUSED = [
    ((4, 16, 14, 14), [2]),         # small: resident, 256 threads
    ((28, 28, 128, 20)[::-1], [2]),
    ((56, 56, 128, 11)[::-1], [2]),  # 16 vectors per thread
    ((56, 56, 128, 22)[::-1], [2]),  # 25 vectors per thread, part of dy (and of the mask) re-read
    ((32, 128, 7, 7), [2]),         # element-wise resident
    ((3, 64, 9, 9), [2]),           # forward resident, backward split
    ((2, 5, 3, 7), [1, 2]),         # split, element-wise
    ((6, 8, 60, 60), [2]),          # split, 4-wide
    ((48, 128, 56, 56), [2]),       # bf16: 8-wide resident with 25 vectors per thread, part of dy and y re-read
    ((40, 128, 56, 56), [2]),       # bf16: 16 vectors
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_residual", [False, True])
@pytest.mark.parametrize("shape,axes", FUSED)
def test_fused_bn_relu(shape, axes, with_residual, dtype):
    from flashlight_amd import ops
    rng = np.random.default_rng(len(shape) + shape[1] + int(with_residual))
    lo = dtype != torch.float32
    rnd = lambda a: round_to(a, dtype)
    x = rnd((rng.standard_normal(shape) * 1.5 + 0.3).astype(np.float32))
    res = rnd(rng.standard_normal(shape).astype(np.float32)) if with_residual else None
    dy = rnd(rng.standard_normal(shape).astype(np.float32))
    outer, Cc, inner = ops.bn_view(shape, axes)
    gamma = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32)
    beta = (0.3 * rng.standard_normal(Cc)).astype(np.float32)
    yb, mean, var = flref.bn_fwd_train(outer, Cc, inner, x, gamma, beta, 1e-5)
    pre = yb + (res if with_residual else 0)
    y_ref = flref.relu_fwd(pre)
    y, sm, si = ops.batchnorm_relu(dev(x, dtype), dev(gamma), dev(beta), None, None, axes, 0.1, 1e-5,
                                   None if res is None else dev(res, dtype))
    tol = 4e-3 if lo else 1e-4
    assert rel_l2(host(y), y_ref) <= tol
    assert rel_l2(host(sm), mean) <= 1e-5
    # backward on the device's own forward result (its mask), like the tape does
    yh = host(y)
    dz_ref = flref.relu_bwd(dy, yh)
    dx_ref, dg_ref, db_ref = flref.bn_bwd(outer, Cc, inner, x, dz_ref, gamma, mean, var, 1e-5)
    dx, dg, db, dr = ops.batchnorm_relu_backward(dev(dy, dtype), dev(x, dtype), y, dev(gamma), sm, si, axes,
                                                 want_residual_grad=with_residual)
    assert rel_l2(host(dx), dx_ref) <= tol
    assert rel_l2(host(dg), dg_ref) <= 1e-4 and rel_l2(host(db), db_ref) <= 1e-4
    if with_residual:
        assert np.array_equal(host(dr), dz_ref.reshape(shape))
    # the same pair with the ReLU's mask kept as one byte per 4 elements: same forward result, the
    # bytes hold y > 0 bit by bit, and the backward pass that reads them gives the same bits as
    # the one that reads y
    args = (dev(x, dtype), dev(gamma), dev(beta), None, None, axes, 0.1, 1e-5, None if res is None else dev(res, dtype))
    if inner % 4 == 0:
        ym, _, _, mask = ops.batchnorm_relu(*args, want_mask=True)
        assert torch.equal(ym, y)
        bits = (yh.reshape(-1, 4) > 0).astype(np.uint8)
        assert np.array_equal(mask.cpu().numpy(), bits[:, 0] | bits[:, 1] << 1 | bits[:, 2] << 2 | bits[:, 3] << 3)
        got = ops.batchnorm_relu_backward(dev(dy, dtype), dev(x, dtype), None, dev(gamma), sm, si, axes,
                                          want_residual_grad=with_residual, mask=mask)
        for a, b in zip(got, (dx, dg, db, dr)):
            assert (a is None and b is None) or torch.equal(a, b)
    else:
        with pytest.raises(ValueError):
            ops.batchnorm_relu(*args, want_mask=True)
    # relu == 0: batch norm plus residual only
    y2, _, _ = ops.batchnorm_relu(dev(x, dtype), dev(gamma), dev(beta), None, None, axes, 0.1, 1e-5,
                                  None if res is None else dev(res, dtype), relu=False)
    assert rel_l2(host(y2), pre) <= tol


def test_fused_bn_relu_refuses_per_activation_mode():
    from flashlight_amd import ops
    x = torch.zeros((4, 3, 5, 5), device="cuda")
    with pytest.raises(ValueError):
        ops.batchnorm_relu(x, None, None, None, None, [0, 1, 2], 0.1, 1e-5)
