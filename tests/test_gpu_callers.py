"""GPU parity of the caller-closure operations (ReLU, Linear's matrix products, bias
reduction, logSoftmax, categorical cross-entropy) against oracle/flref.c, through the C
ABI, and one training step of the README MNIST convnet (configs[0]) end to end."""
import numpy as np
import pytest
import torch

import flashlight_amd as fa
from flashlight_amd import ops
from gpu_util import dev, host, round_to
from oracle import flref
from refmath import rel_l2

pytestmark = pytest.mark.gpu
DT = [torch.float32, torch.bfloat16, torch.float16]


def _tol(dtype):
    return 1e-4 if dtype == torch.float32 else 2e-2


def _round(a, dtype):
    return round_to(a, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("n", [5000, 4, 5, 7, 4099, 1 << 20])
def test_relu(dtype, n):
    rng = np.random.default_rng(60)
    x = _round(rng.standard_normal(n).astype(np.float32), dtype)
    x[:4] = [0.0, -0.0, np.inf, -np.inf]
    dy = _round(rng.standard_normal(n).astype(np.float32), dtype)
    assert np.array_equal(host(ops.relu(dev(x, dtype))), flref.relu_fwd(x))
    assert np.array_equal(host(ops.relu_backward(dev(dy, dtype), dev(x, dtype))), flref.relu_bwd(dy, x))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("fin,fout,batch", [(3136, 1024, 16), (1024, 10, 64), (37, 21, 9), (5, 130, 1), (200, 1, 70),
                                             (96, 80, 300), (130, 67, 1000)])
def test_linear(fin, fout, batch, dtype):
    rng = np.random.default_rng(fin + fout + batch)
    x = _round(rng.standard_normal((batch, fin)).astype(np.float32), dtype)
    w = _round((rng.standard_normal((fin, fout)) / np.sqrt(fin)).astype(np.float32), dtype)
    b = rng.standard_normal(fout).astype(np.float32)
    dy = _round(rng.standard_normal((batch, fout)).astype(np.float32), dtype)
    tol = _tol(dtype)
    y = ops.linear(dev(x, dtype), dev(w, dtype), dev(b))
    assert rel_l2(host(y), flref.matmul(fout, batch, fin, w, x, False, False, b)) <= tol
    y0 = ops.linear(dev(x, dtype), dev(w, dtype), None)
    assert rel_l2(host(y0), flref.matmul(fout, batch, fin, w, x)) <= tol
    dx, dw, db = ops.linear_backward(dev(dy, dtype), dev(x, dtype), dev(w, dtype))
    assert rel_l2(host(dx), flref.matmul(fin, batch, fout, w, dy, True, False)) <= tol
    assert rel_l2(host(dw), flref.matmul(fout, fin, batch, dy, x, False, True)) <= tol
    assert rel_l2(host(db), flref.sum_columns(fout, batch, dy)) <= 1e-5


@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (64, 64, 16), (70, 33, 129), (1, 9, 200), (130, 67, 300)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_matmul_all_forms_through_the_c_abi(M, N, K, ta, tb, with_bias):
    """flhip_matmul: C = op(A) op(B) (+ bias per row) in all four transposition forms, whichever
    kernel takes them (1x1-convolution GEMMs, the A * B^T kernel, the tiled vector-ALU kernel)."""
    import ctypes as C
    from flashlight_amd import capi
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    A = rng.standard_normal((M, K) if ta else (K, M)).astype(np.float32)   # storage as in the oracle's test
    B = rng.standard_normal((K, N) if tb else (N, K)).astype(np.float32)
    bias = rng.standard_normal(M).astype(np.float32) if with_bias else None
    want = flref.matmul(M, N, K, A, B, ta, tb, bias)
    Ad, Bd, Cd = dev(A), dev(B), torch.empty(N, M, device="cuda")
    bd = dev(bias) if with_bias else None
    P = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = capi.lib().flhip_matmul(P(Ad), P(Bd), P(Cd), M, N, K, int(ta), int(tb), P(bd), capi.F32, S)
    assert rc == 0
    assert rel_l2(host(Cd), want) <= 1e-5


def _matmul_through_c_abi(A, B, M, N, K, ta, tb, bias, dtype):
    import ctypes as C
    from flashlight_amd import capi
    Ad, Bd, Cd = dev(A, dtype), dev(B, dtype), torch.empty(N, M, device="cuda", dtype=dtype)
    bd = dev(bias) if bias is not None else None
    P = lambda t: C.c_void_p(t.data_ptr()) if t is not None else None
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    code = {torch.float32: capi.F32, torch.bfloat16: capi.BF16, torch.float16: capi.F16}[dtype]
    rc = capi.lib().flhip_matmul(P(Ad), P(Bd), P(Cd), M, N, K, int(ta), int(tb), P(bd), code, S)
    assert rc == 0
    return host(Cd)


# shapes around the edges of the 16-bit matrix-instruction kernels: rows that are no multiple of the 8-row cells
# (and fewer than 8: another kernel's), columns that are no multiple of the 64/128-column tiles, contractions of
# a partial last stage (40, 72, 200), of no whole cell (67, 1001: not for A B, which then takes another kernel)
# and of many stages
LO16_MATMUL = [(67, 130, 40), (8, 257, 72), (9, 129, 200), (135, 1000, 67), (300, 131, 1001), (5, 300, 64),
               (128, 256, 32), (257, 513, 1000), (1000, 200, 8), (64, 2000, 96)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", LO16_MATMUL)
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True)])
def test_matmul_in_16_bit_storage(M, N, K, ta, tb, dtype):
    """The three products fl::linear needs, in 16-bit storage with more than 128 columns: they run on the
    16-bit matrix instructions.  Every element is compared: one rounding of the exact sum, plus what an fp32
    accumulation over K terms may add."""
    rng = np.random.default_rng(M * 1000 + N * 10 + K + int(ta) + 2 * int(tb))
    A = _round(rng.standard_normal((M, K) if ta else (K, M)).astype(np.float32), dtype)
    B = _round(rng.standard_normal((K, N) if tb else (N, K)).astype(np.float32), dtype)
    for bias in ([None] if tb else [None, rng.standard_normal(M).astype(np.float32)]):
        want = flref.matmul(M, N, K, A, B, ta, tb, bias)
        got = _matmul_through_c_abi(A, B, M, N, K, ta, tb, bias, dtype)
        half_ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
        slack = 1.01 * half_ulp * np.abs(want) + 2e-6 * K + (0 if dtype == torch.bfloat16 else 6e-8)
        bad = np.abs(got.astype(np.float64) - want) > slack
        assert not bad.any(), (int(bad.sum()), np.argwhere(bad)[:4].tolist())


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("M,N,K,part", [(128, 80, 5000, 1.0), (2000, 80, 12000, 1.0), (1024, 1024, 12000, 1.0),
                                        (67, 130, 3001, 1.0), (256, 64, 4096, 0.5), (300, 200, 70, 1.0)])
def test_matmul_with_a_workspace_cuts_a_long_contraction(M, N, K, part, dtype):
    """flhip_matmul_ws: A * B^T of few tiles over a long contraction (the weight gradient of a layer over many
    frames) in slices whose partial products are added in slice order; with part < 1 the caller brings less than
    flhip_matmul_workspace_bytes asks for (fewer slices, or none).  Checked against numpy's float64 product of the
    same rounded operands; two calls give the same bits."""
    import ctypes as C
    from flashlight_amd import capi
    rng = np.random.default_rng(M + N + K)
    A = _round(rng.standard_normal((K, M)).astype(np.float32), dtype)
    B = _round(rng.standard_normal((K, N)).astype(np.float32), dtype)
    want = B.astype(np.float64).T @ A.astype(np.float64)                       # stored [n][m]
    code = {torch.float32: capi.F32, torch.bfloat16: capi.BF16, torch.float16: capi.F16}[dtype]
    lib = capi.lib()
    assert lib.flhip_matmul_workspace_bytes(M, N, K, 0, 0, code) == 0          # only A * B^T has a use for one
    assert lib.flhip_matmul_workspace_bytes(M, N, K, 1, 0, code) == 0
    need = lib.flhip_matmul_workspace_bytes(M, N, K, 0, 1, code)
    if K >= 3000 and M * N <= 1024 * 1024 and (dtype == torch.float32 or N % 2 == 0):
        assert need >= 2 * M * N * 4
    nws = int(need * part) // 4 * 4
    ws = torch.full((max(nws, 4),), 0xff, dtype=torch.uint8, device="cuda")
    Ad, Bd = dev(A, dtype), dev(B, dtype)
    P = lambda t: C.c_void_p(t.data_ptr())
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for _ in range(2):
        Cd = torch.empty(N, M, device="cuda", dtype=dtype)
        assert lib.flhip_matmul_ws(P(Ad), P(Bd), P(Cd), M, N, K, 0, 1, None, code, P(ws) if nws else None, nws, S) == 0
        outs.append(host(Cd))
    assert np.array_equal(outs[0], outs[1])
    half_ulp = {torch.float32: 2.0 ** -24, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    bad = np.abs(outs[0].astype(np.float64) - want) > 1.01 * half_ulp * np.abs(want) + 2e-6 * K
    assert not bad.any(), (int(bad.sum()), np.argwhere(bad)[:4].tolist())


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows,cols,part", [(2000, 12000, 1.0), (80, 12000, 1.0), (67, 5000, 1.0), (129, 333, 1.0), (1, 4096, 1.0),
                                            (1024, 64, 1.0), (512, 3000, 0.5), (130, 100000, 1.0)])
def test_sum_columns_with_a_workspace(rows, cols, part, dtype):
    """flhip_sum_columns_ws (the bias gradient of fl::linear over many frames): the columns in slices, added in slice
    order; against the oracle's sums (float64 accumulation), two calls bit-equal, and with less workspace than asked
    for the one-pass kernel's result."""
    import ctypes as C
    from flashlight_amd import capi
    rng = np.random.default_rng(rows + cols)
    x = _round(rng.standard_normal((cols, rows)).astype(np.float32), dtype)
    want = flref.sum_columns(rows, cols, x)
    code = {torch.float32: capi.F32, torch.bfloat16: capi.BF16, torch.float16: capi.F16}[dtype]
    lib = capi.lib()
    need = lib.flhip_sum_columns_workspace_bytes(rows, cols, code)
    if cols >= 3000 and rows * cols >= 1 << 21:
        assert need >= 2 * rows * 4
    nws = int(need * part) // 4 * 4
    ws = torch.full((max(nws, 4),), 0xff, dtype=torch.uint8, device="cuda")
    xd = dev(x, dtype)
    P = lambda t: C.c_void_p(t.data_ptr())
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for _ in range(2):
        out = torch.full((rows,), float("nan"), device="cuda")
        assert lib.flhip_sum_columns_ws(P(xd), P(out), rows, cols, code, P(ws) if nws else None, nws, S) == 0
        outs.append(host(out))
    assert np.array_equal(outs[0], outs[1])
    assert np.allclose(outs[0], want, rtol=1e-5, atol=2e-6 * cols)


@pytest.mark.parametrize("planes", [7, 0, None])
@pytest.mark.parametrize("M,N,K", LO16_MATMUL + [(256, 200, 64), (512, 4100, 36), (1027, 1030, 130)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True)])
def test_matmul_fp32_with_a_matrix_as_one_plane(M, N, K, ta, tb, planes):
    """fp32 products on the 1x1 kernels with a matrix as one image's plane (option MATMUL_PLANES: 7 = whatever the
    shape, 0 = never, unset = by shape), every element against the oracle."""
    from flashlight_amd import capi
    rng = np.random.default_rng(M * 1000 + N * 10 + K + int(ta) + 2 * int(tb))
    A = rng.standard_normal((M, K) if ta else (K, M)).astype(np.float32)
    B = rng.standard_normal((K, N) if tb else (N, K)).astype(np.float32)
    capi.set_option("MATMUL_PLANES", planes)
    try:
        for bias in ([None] if tb else [None, rng.standard_normal(M).astype(np.float32)]):
            want = flref.matmul(M, N, K, A, B, ta, tb, bias)
            got = _matmul_through_c_abi(A, B, M, N, K, ta, tb, bias, torch.float32)
            bad = np.abs(got.astype(np.float64) - want) > 1e-5 * np.abs(want) + 2e-6 * K
            assert not bad.any(), (int(bad.sum()), np.argwhere(bad)[:4].tolist())
    finally:
        capi.set_option("MATMUL_PLANES", None)


def test_matmul_fp32_at_the_size_of_a_speech_model():
    """2000 x 2000 weights against 4000 frames in fp32 (the plane mapping by shape), against numpy's float64 product."""
    M, N, K = 2000, 4000, 2000
    rng = np.random.default_rng(78)
    for ta, tb in [(False, False), (True, False), (False, True)]:
        A = rng.standard_normal((M, K) if ta else (K, M)).astype(np.float32)
        B = rng.standard_normal((K, N) if tb else (N, K)).astype(np.float32)
        A64 = A.astype(np.float64) if ta else A.astype(np.float64).T
        B64 = B.astype(np.float64) if tb else B.astype(np.float64).T
        want = (A64 @ B64).T
        bias = rng.standard_normal(M).astype(np.float32) if not (ta or tb) else None
        if bias is not None:
            want = want + bias[None, :]
        got = _matmul_through_c_abi(A, B, M, N, K, ta, tb, bias, torch.float32)
        bad = np.abs(got.astype(np.float64) - want) > 1e-5 * np.abs(want) + 2e-6 * K
        assert not bad.any(), (ta, tb, int(bad.sum()), np.argwhere(bad)[:4].tolist())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matmul_in_16_bit_storage_at_the_size_of_a_speech_model(dtype):
    """2000 x 2000 weights against 4000 frames, the three products of a layer's step; checked against numpy's
    float64 product of the same rounded operands (the oracle's loops would take minutes here)."""
    M, N, K = 2000, 4000, 2000
    rng = np.random.default_rng(77)
    half_ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    for ta, tb in [(False, False), (True, False), (False, True)]:
        A = _round(rng.standard_normal((M, K) if ta else (K, M)).astype(np.float32), dtype)
        B = _round(rng.standard_normal((K, N) if tb else (N, K)).astype(np.float32), dtype)
        A64 = A.astype(np.float64) if ta else A.astype(np.float64).T            # M x K
        B64 = B.astype(np.float64) if tb else B.astype(np.float64).T            # K x N
        want = (A64 @ B64).T                                                     # stored [n][m]
        got = _matmul_through_c_abi(A, B, M, N, K, ta, tb, None, dtype)
        bad = np.abs(got.astype(np.float64) - want) > 1.01 * half_ulp * np.abs(want) + 2e-6 * K
        assert not bad.any(), (ta, tb, int(bad.sum()), np.argwhere(bad)[:4].tolist())


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("classes,cols", [(10, 64), (1000, 7), (1, 5), (65, 3)])
def test_logsoftmax(classes, cols, dtype):
    rng = np.random.default_rng(classes + cols)
    x = _round((rng.standard_normal((cols, classes)) * 4).astype(np.float32), dtype)
    dy = _round(rng.standard_normal((cols, classes)).astype(np.float32), dtype)
    y_ref = flref.logsoftmax_fwd(x)
    y = ops.log_softmax(dev(x, dtype))
    if dtype == torch.float32:
        assert np.allclose(host(y), y_ref, atol=2e-6, rtol=1e-5)
    else:
        assert np.allclose(host(y), y_ref, atol=0.06, rtol=1e-2)
    yq = _round(y_ref, dtype)
    dx = ops.log_softmax_backward(dev(dy, dtype), dev(yq, dtype))
    dx_ref = flref.logsoftmax_bwd(dy, yq)
    assert np.allclose(host(dx), dx_ref, atol=_tol(dtype) * 10, rtol=_tol(dtype))


@pytest.mark.parametrize("reduction", [ops.REDUCE_NONE, ops.REDUCE_MEAN, ops.REDUCE_SUM])
def test_cross_entropy(reduction):
    rng = np.random.default_rng(70 + reduction)
    logp = np.log(rng.dirichlet(np.ones(10), size=300)).astype(np.float32)
    target = rng.integers(0, 10, 300).astype(np.int32)
    target[[5, 17, 200]] = -1
    per, s, mean, count, bad = flref.cce_fwd(logp, target)
    loss, stats = ops.categorical_cross_entropy(dev(logp), dev(target), reduction)
    want = [per, np.float32(mean), np.float32(s)][reduction]
    assert np.allclose(host(loss).reshape(np.shape(want)), want, rtol=1e-5, atol=1e-6)
    g = rng.standard_normal(300 if reduction == ops.REDUCE_NONE else 1).astype(np.float32)
    dx = ops.categorical_cross_entropy_backward(dev(g), logp.shape, torch.float32, dev(target), stats,
                                                reduction)
    assert np.allclose(host(dx), flref.cce_bwd(logp.shape, g, target, count, reduction), rtol=1e-6,
                       atol=1e-7)
    with pytest.raises(ValueError):
        ops.categorical_cross_entropy(dev(logp), dev(np.full(300, 10, np.int32)))


def _mnist_params(rng):
    """Conv2D / Linear initialisation of the reference (nn/modules/Conv2D.cpp:177-194,
    Linear.cpp:62-74): Kaiming-uniform weights, bias U(+-sqrt(1/fanIn))."""
    def ku(shape, fan_in):
        return rng.uniform(-np.sqrt(3.0 / fan_in), np.sqrt(3.0 / fan_in), shape).astype(np.float32)

    def bu(n, fan_in):
        return rng.uniform(-np.sqrt(1.0 / fan_in), np.sqrt(1.0 / fan_in), n).astype(np.float32)
    return dict(w1=ku((32, 1, 5, 5), 25), b1=bu(32, 25), w2=ku((64, 32, 5, 5), 800), b2=bu(64, 800),
                w3=ku((3136, 1024), 3136), b3=bu(1024, 3136), w4=ku((1024, 10), 1024), b4=bu(10, 1024))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("outer,mid,inner,scalar", [(3, 5, 7, False), (1, 600, 1, False), (40, 9, 1, False),
                                                    (1, 8, 5000, False), (2, 3, 4, True),
                                                    (1, 1, 300000, True), (64, 512, 1, False)])
def test_affine(outer, mid, inner, scalar, dtype):
    rng = np.random.default_rng(outer + mid + inner)
    x = _round(rng.standard_normal((outer, mid, inner)).astype(np.float32), dtype)
    dy = _round(rng.standard_normal((outer, mid, inner)).astype(np.float32), dtype)
    n = 1 if scalar else mid
    w = _round(rng.standard_normal(n).astype(np.float32), dtype)
    b = _round(rng.standard_normal(n).astype(np.float32), dtype)
    view = (outer, mid, inner, scalar)
    tol = _tol(dtype)
    y = ops.affine(dev(x, dtype), dev(w, dtype), dev(b, dtype), view)
    assert rel_l2(host(y), flref.affine_fwd(outer, mid, inner, scalar, x, w, b)) <= tol
    dx, dw, db = ops.affine_backward(dev(dy, dtype), dev(x, dtype), dev(w, dtype), view)
    rdx, rdw, rdb = flref.affine_bwd(outer, mid, inner, scalar, dy, x, w)
    assert rel_l2(host(dx), rdx) <= tol
    # the sums accumulate in fp32 whatever the storage type
    assert rel_l2(host(dw), rdw) <= 1e-4 and rel_l2(host(db), rdb) <= 1e-4


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("idx_shape,dim,tokens", [((1,), 1, 1), ((7,), 5, 3), ((50, 4), 16, 9), ((200, 16), 33, 1000),
                                                  ((64,), 8, 2), ((300, 40), 512, 10000), ((9,), 2500, 5), ((129,), 300, 1)])
def test_embedding(idx_shape, dim, tokens, dtype):
    """fl::embedding forward (bit-exact: a gather) and the table's gradient (sums in the order of the positions, fp32,
    one rounding), with tokens that repeat, tokens that never occur and two indices outside the table."""
    rng = np.random.default_rng(dim + tokens + len(idx_shape))
    idx = rng.integers(0, tokens, size=idx_shape).astype(np.int32)
    if idx.size > 4:
        idx.ravel()[1] = tokens
        idx.ravel()[-2] = -3
    w = _round(rng.standard_normal((tokens, dim)).astype(np.float32), dtype)
    dy = _round(rng.standard_normal(idx_shape + (dim,)).astype(np.float32), dtype)
    idx_d = torch.from_numpy(idx).cuda()
    y = ops.embedding(idx_d, dev(w, dtype))
    assert tuple(y.shape) == idx_shape + (dim,)
    assert np.array_equal(host(y).reshape(-1, dim), flref.embedding_fwd(idx, w))
    dw = ops.embedding_backward(dev(dy, dtype), idx_d, tokens)
    want = flref.embedding_bwd(idx, dy.reshape(-1, dim), tokens)
    if dtype == torch.float32:
        assert np.allclose(host(dw), want, rtol=1e-5, atol=1e-5 * max(1, idx.size / tokens) ** 0.5)
    else:
        assert np.allclose(host(dw), want, rtol=2.0 ** -7, atol=1e-3)
    dw2 = ops.embedding_backward(dev(dy, dtype), idx_d, tokens)
    assert torch.equal(dw, dw2)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("shape,scalar", [((3, 5, 7), True), ((3, 5, 7), False), ((1, 600), False), ((40, 9, 1), True),
                                          ((64, 3, 56, 56), True), ((8, 250, 1, 300), False), ((300001,), True)])
def test_prelu(shape, scalar, dtype):
    """fl::PReLU forward, input gradient and parameter gradient against the checker: a single parameter or one per
    index of the fastest dimension, sizes from one workgroup's slice to many slices per parameter; exact zeros in x
    (the mask is x >= 0)."""
    rng = np.random.default_rng(len(shape) * 100 + shape[-1])
    x = _round(rng.standard_normal(shape).astype(np.float32), dtype)
    x.flat[::5] = 0.0
    dy = _round(rng.standard_normal(shape).astype(np.float32), dtype)
    d0 = shape[-1]
    w = _round(rng.uniform(0.05, 0.95, 1 if scalar else d0).astype(np.float32), dtype)
    tol = _tol(dtype)
    y = ops.prelu(dev(x, dtype), dev(w, dtype))
    assert rel_l2(host(y), flref.prelu_fwd(x, w, d0)) <= tol
    dx, dw = ops.prelu_backward(dev(dy, dtype), dev(x, dtype), dev(w, dtype))
    rdx, rdw = flref.prelu_bwd(dy, x, w, d0)
    assert rel_l2(host(dx), rdx) <= tol
    assert rel_l2(host(dw), rdw) <= 1e-4           # fp32 sums whatever the storage type
    assert np.array_equal(host(dx).flat[::5], dy.flat[::5])
    # twice the same call: the same bits (fixed order of the two-stage sum)
    dx2, dw2 = ops.prelu_backward(dev(dy, dtype), dev(x, dtype), dev(w, dtype))
    assert torch.equal(dw, dw2) and torch.equal(dx, dx2)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("whcn,norm,params", [
    ((6, 5, 4, 3), (0, 1, 2), "per"),        # LayerNorm over {0,1,2} of WHCN
    ((6, 5, 4, 3), (0, 1, 2), "scalar"),
    ((512, 50, 8), (0,), "per"),             # [C, T, B], normalise C
    ((512, 50, 8), (0,), None),
    ((20, 4, 3, 16), (3,), "per"),
    ((56, 56, 64, 4), (0, 1, 2), "per"),
    # non-contiguous complement: through the device reorder (LayerNorm.cpp:63-86)
    ((6, 5, 4, 3), (1,), "per"),
    ((6, 5, 4, 3), (1, 2), None),
    ((6, 5, 4, 3), (0, 2), "scalar"),
    ((4, 7, 3, 2), (1, 3), "per"),
    ((32, 50, 16), (1,), "per"),
    ((40, 30, 8, 6), (0, 3), "per"),
])
def test_layer_norm(whcn, norm, params, dtype):
    # fl::LayerNorm::forward (nn/modules/LayerNorm.cpp:42-131) = the extension's batchnorm
    # over the complement axes + the broadcast scale and shift
    rng = np.random.default_rng(sum(whcn) + len(norm))
    tshape = tuple(whcn[::-1])
    x = _round((rng.standard_normal(tshape) * 2 + 0.5).astype(np.float32), dtype)
    dy = _round(rng.standard_normal(tshape).astype(np.float32), dtype)
    w = b = None
    if params == "per":
        n = int(np.prod([whcn[a] for a in norm]))
        w = _round(rng.standard_normal(n).astype(np.float32), dtype)
        b = _round(rng.standard_normal(n).astype(np.float32), dtype)
    elif params == "scalar":
        w, b = _round(np.array([1.7], np.float32), dtype), _round(np.array([-0.3], np.float32), dtype)
    eps = 1e-5
    ry, rxhat, rmean, rvar = flref.layer_norm_fwd(x, whcn, norm, eps, w, b)
    rdx, rdw, rdb = flref.layer_norm_bwd(dy, x, rxhat, rmean, rvar, whcn, norm, eps, w)
    dw_ = None if w is None else dev(w, dtype)
    db_ = None if b is None else dev(b, dtype)
    y, ctx = ops.layer_norm(dev(x, dtype), norm, eps, dw_, db_)
    tol = _tol(dtype)
    assert tuple(y.shape) == tshape
    assert rel_l2(host(y), ry.reshape(tshape)) <= tol
    dx, dw, db = ops.layer_norm_backward(dev(dy, dtype), ctx, dw_)
    assert rel_l2(host(dx), rdx.reshape(tshape)) <= (1e-4 if dtype == torch.float32 else 3e-2)
    if w is not None:
        assert rel_l2(host(dw), rdw) <= tol and rel_l2(host(db), rdb) <= tol


def test_layer_norm_argument_errors():
    with pytest.raises(ValueError):
        ops.layer_norm(dev(np.zeros((2, 2, 2, 2, 2), np.float32)), (0,))
    with pytest.raises(ValueError):
        ops.layer_norm(dev(np.zeros((2, 3, 4, 5), np.float32)), (0, 1, 2, 3))   # nothing left to batch over


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("whcn,perm", [((6, 5, 4, 3), (1, 0, 2, 3)), ((6, 5, 4, 3), (3, 2, 1, 0)),
                                       ((7, 1, 9, 2), (2, 3, 0, 1)), ((64, 33, 1, 1), (1, 0, 2, 3)),
                                       ((5, 4, 3), (0, 2, 1, 3))])
def test_reorder_is_a_transpose(whcn, perm, dtype):
    # fl::reorder: result dimension k = input dimension perm[k]; bit-exact copy
    rng = np.random.default_rng(sum(whcn))
    w4 = list(whcn) + [1] * (4 - len(whcn))
    x = _round(rng.standard_normal(tuple(w4[::-1])).astype(np.float32), dtype)
    y = ops.reorder(dev(x, dtype).reshape(tuple(whcn[::-1])), perm)
    want = x.transpose([3 - p for p in perm][::-1])
    assert tuple(y.shape) == want.shape
    assert np.array_equal(host(y), want)
    with pytest.raises(ValueError):
        ops.reorder(dev(x, dtype), (0, 0, 1, 2))



@pytest.mark.parametrize("B", [16, 64])
def test_mnist_convnet_training_step(B):
    """configs[0]: View, Conv2D 1->32 5x5 SAME, ReLU, Pool2D max 2x2 s2, Conv2D 32->64 5x5
    SAME, ReLU, Pool2D, View, Linear 3136->1024, ReLU, Linear 1024->10, LogSoftmax, then
    categoricalCrossEntropy (reference README); dropout left out (it is a random mask, not
    part of the path).  Forward and the gradient closures in tape order, device against
    oracle, every parameter gradient compared."""
    rng = np.random.default_rng(80)       # batch 64 is the size configs[0] states
    x = rng.standard_normal((B, 1, 28, 28)).astype(np.float32)
    labels = rng.integers(0, 10, B).astype(np.int32)
    P = _mnist_params(rng)
    pad = fa.derive_padding(28, 5, 1, -1)          # SAME
    assert pad == 2 and fa.derive_padding(14, 5, 1, -1) == 2
    MAXP = fa.PoolingMode.MAX

    # ---- oracle -----------------------------------------------------------------
    d1 = flref.conv_desc(x.shape, P["w1"].shape, (1, 1), (2, 2))
    a1 = flref.conv2d_fwd(d1, x, P["w1"], P["b1"]); r1 = flref.relu_fwd(a1)
    pd1 = flref.pool_desc(r1.shape, (2, 2), (2, 2), (0, 0), 0); p1, am1 = flref.pool2d_fwd(pd1, r1)
    d2 = flref.conv_desc(p1.shape, P["w2"].shape, (1, 1), (2, 2))
    a2 = flref.conv2d_fwd(d2, p1, P["w2"], P["b2"]); r2 = flref.relu_fwd(a2)
    pd2 = flref.pool_desc(r2.shape, (2, 2), (2, 2), (0, 0), 0); p2, am2 = flref.pool2d_fwd(pd2, r2)
    f = p2.reshape(B, 3136)
    a3 = flref.matmul(1024, B, 3136, P["w3"], f, False, False, P["b3"]); r3 = flref.relu_fwd(a3)
    a4 = flref.matmul(10, B, 1024, P["w4"], r3, False, False, P["b4"])
    lp = flref.logsoftmax_fwd(a4)
    _, _, loss_ref, count, bad = flref.cce_fwd(lp, labels)
    assert bad == 0
    g = flref.cce_bwd(lp.shape, np.ones(1, np.float32), labels, count, 1)
    g = flref.logsoftmax_bwd(g, lp)
    R = {"b4": flref.sum_columns(10, B, g), "w4": flref.matmul(10, 1024, B, g, r3, False, True)}
    g = flref.relu_bwd(flref.matmul(1024, B, 10, P["w4"], g, True, False), a3)
    R["b3"] = flref.sum_columns(1024, B, g); R["w3"] = flref.matmul(1024, 3136, B, g, f, False, True)
    g = flref.matmul(3136, B, 1024, P["w3"], g, True, False).reshape(p2.shape)
    g = flref.relu_bwd(flref.pool2d_bwd(pd2, g, am2), a2)
    R["w2"], R["b2"] = flref.conv2d_bwd_filter(d2, p1, g)
    g = flref.relu_bwd(flref.pool2d_bwd(pd1, flref.conv2d_bwd_data(d2, g, P["w2"]), am1), a1)
    R["w1"], R["b1"] = flref.conv2d_bwd_filter(d1, x, g)

    # ---- device ------------------------------------------------------------------
    D = {k: dev(v) for k, v in P.items()}
    xd, ld = dev(x), dev(labels)
    A1 = ops.conv2d(xd, D["w1"], D["b1"], 1, 1, 2, 2); R1 = ops.relu(A1)
    P1, AM1 = ops.pool2d(R1, 2, 2, 2, 2, 0, 0, MAXP)
    A2 = ops.conv2d(P1, D["w2"], D["b2"], 1, 1, 2, 2); R2 = ops.relu(A2)
    P2, AM2 = ops.pool2d(R2, 2, 2, 2, 2, 0, 0, MAXP)
    Fl = P2.reshape(B, 3136)
    A3 = ops.linear(Fl, D["w3"], D["b3"]); R3 = ops.relu(A3)
    A4 = ops.linear(R3, D["w4"], D["b4"])
    LP = ops.log_softmax(A4)
    loss, stats = ops.categorical_cross_entropy(LP, ld)
    assert abs(float(loss.item()) - loss_ref) <= 1e-5 * max(1.0, abs(loss_ref))
    G = ops.categorical_cross_entropy_backward(dev(np.ones(1, np.float32)), LP.shape, torch.float32, ld,
                                               stats)
    G = ops.log_softmax_backward(G, LP)
    G, dw4, db4 = ops.linear_backward(G, R3, D["w4"])
    G, dw3, db3 = ops.linear_backward(ops.relu_backward(G, A3), Fl, D["w3"])
    G = ops.pool2d_backward(G.reshape(P2.shape), R2.shape, AM2, 2, 2, 2, 2, 0, 0, MAXP)
    G = ops.relu_backward(G, A2)
    dw2, db2 = ops.conv2d_backward_filter_bias(G, P1, D["w2"].shape, True, 1, 1, 2, 2)
    G = ops.conv2d_backward_data(G, P1.shape, D["w2"], 1, 1, 2, 2)
    G = ops.relu_backward(ops.pool2d_backward(G, R1.shape, AM1, 2, 2, 2, 2, 0, 0, MAXP), A1)
    dw1, db1 = ops.conv2d_backward_filter_bias(G, xd, D["w1"].shape, True, 1, 1, 2, 2)
    got = dict(w1=dw1, b1=db1, w2=dw2, b2=db2, w3=dw3, b3=db3, w4=dw4, b4=db4)
    for k in sorted(R):
        assert rel_l2(host(got[k]), R[k]) <= 1e-4, (k, rel_l2(host(got[k]), R[k]))


def test_astype_many_equals_astype():
    """flhip_convert_many: every tensor converted as flhip_convert would, whatever its length
    (empty, shorter than a piece of 2048 elements, several pieces), more tensors than fit in one launch."""
    rng = np.random.default_rng(77)
    sizes = [0, 1, 7, 2047, 2048, 2049, 5000, 64 * 64 * 9, 100003] + [int(v) for v in rng.integers(1, 9000, 70)]
    xs = [dev(rng.standard_normal(n).astype(np.float32)) for n in sizes]
    many = ops.astype_many(xs, torch.bfloat16)
    for x, m in zip(xs, many):
        assert m.dtype == torch.bfloat16 and torch.equal(m, ops.astype(x, torch.bfloat16))
        assert torch.equal(m, x.to(torch.bfloat16))           # round to nearest even
    back = ops.astype_many(many, torch.float32)
    for m, b in zip(many, back):
        assert torch.equal(b, m.float())
    assert ops.astype_many([], torch.bfloat16) == []


@pytest.mark.parametrize("src,dst", [(torch.float32, torch.float16), (torch.float16, torch.float32),
                                     (torch.bfloat16, torch.float16), (torch.float16, torch.bfloat16),
                                     (torch.float16, torch.float16)])
def test_astype_with_f16(src, dst):
    """Tensor::astype to and from f16 storage: round to nearest even, overflow to infinity, subnormal results,
    NaN kept; between the two 16-bit types through the fp32 value."""
    rng = np.random.default_rng(78)
    v = rng.standard_normal(10007).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 10007).astype(np.float32)
    v[:8] = [0.0, -0.0, np.inf, -np.inf, np.nan, 65504.0, 65520.0, 5.9604645e-8]
    x = dev(v).to(src)
    got = ops.astype(x, dst)
    ref = x.float().to(dst)
    assert got.dtype == dst
    nan = torch.isnan(ref)
    assert torch.equal(torch.isnan(got), nan) and int(nan.sum()) == 1
    bits = torch.int32 if dst == torch.float32 else torch.int16
    assert torch.equal(got.view(bits)[~nan], ref.view(bits)[~nan])
    many = ops.astype_many([x, x[:5], x[:0]], dst)
    assert torch.equal(many[0].float().nan_to_num(7.0), got.float().nan_to_num(7.0)) and many[2].numel() == 0


# ---- activations, gated linear unit, dropout (nn/modules/Activations.cpp, Functions.cpp:1567-1610, 1777-1785) ----
_ACTS = [(ops.ACT_ELU, 1.0, 0.0), (ops.ACT_ELU, 0.3, 0.0), (ops.ACT_CLAMP, 0.0, 6.0), (ops.ACT_CLAMP, -1.0, 1.0),
         (ops.ACT_TANH, 0.0, 0.0), (ops.ACT_LOG, 0.0, 0.0), (ops.ACT_SWISH, 1.0, 0.0), (ops.ACT_SWISH, 1.7, 0.0),
         (ops.ACT_SIGMOID, 0.0, 0.0), (ops.ACT_SCALE, -0.37, 0.0), (ops.ACT_LEAKY, 0.01, 0.0), (ops.ACT_LEAKY, 1.5, 0.0),
         (ops.ACT_THRESHOLD, 0.7, 0.0)]


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("op,a,b", _ACTS)
@pytest.mark.parametrize("n", [4099, 1 << 18, 3])
def test_activations(op, a, b, n, dtype):
    rng = np.random.default_rng(70 + op)
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    if op == ops.ACT_LOG:
        x = np.abs(x) + 0.05
    if op == ops.ACT_CLAMP and n >= 4:
        x[:4] = [a, b, np.nextafter(np.float32(a), np.float32(9)), np.nextafter(np.float32(b), np.float32(-9))]
    x = _round(x, dtype)
    dy = _round(rng.standard_normal(n).astype(np.float32), dtype)
    y = host(ops.activation(op, dev(x, dtype), a, b))
    dx = host(ops.activation_backward(op, dev(dy, dtype), dev(x, dtype), a, b))
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    assert rel_l2(y, flref.act_fwd(op, x, a, b)) <= tol
    assert rel_l2(dx, flref.act_bwd(op, dy, x, a, b)) <= tol
    if op == ops.ACT_CLAMP:      # selections and copies: exact
        assert np.array_equal(y, flref.act_fwd(op, x, a, b))
        assert np.array_equal(dx, flref.act_bwd(op, dy, x, a, b))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("shape,dim", [((3, 8, 5), 1), ((4, 6), 1), ((10, 7), 0), ((2, 3, 4, 6), 3), ((16, 400, 1, 150), 1)])
def test_gated_linear_unit(shape, dim, dtype):
    rng = np.random.default_rng(80 + dim)
    x = _round(rng.standard_normal(shape).astype(np.float32), dtype)
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    m = shape[dim] // 2 * int(np.prod(shape[dim + 1:], dtype=np.int64))
    y_ref = flref.glu_fwd(x, outer, m)
    dy = _round(rng.standard_normal(y_ref.shape).astype(np.float32), dtype)
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    y = ops.gated_linear_unit(dev(x, dtype), dim)
    assert tuple(y.shape) == tuple(s // 2 if i == dim else s for i, s in enumerate(shape))
    assert rel_l2(host(y).ravel(), y_ref) <= tol
    dx = ops.gated_linear_unit_backward(dev(dy.reshape(y.shape), dtype), dev(x, dtype), dim)
    assert rel_l2(host(dx).ravel(), flref.glu_bwd(dy, x, outer, m).ravel()) <= tol
    with pytest.raises(ValueError):
        ops.gated_linear_unit(dev(np.zeros((3, 5), np.float32), dtype), 1)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("p", [0.0, 0.2, 0.75])
def test_dropout_mask_matches_the_checker(p, dtype):
    rng = np.random.default_rng(90)
    x = _round(rng.standard_normal(100003).astype(np.float32), dtype)
    seed = (77 << 32) | 12345
    y = host(ops.dropout(dev(x, dtype), p, seed))
    ref = flref.dropout(x, p, 12345, 77)
    assert np.array_equal(y == 0, ref == 0)            # the same mask
    assert rel_l2(y, ref) <= (1e-6 if dtype == torch.float32 else 4e-3)
    assert np.array_equal(y, host(ops.dropout(dev(x, dtype), p, seed)))


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("shape,dim", [((13, 1, 80, 200), 3), ((1816, 30), 0), ((7, 3, 5, 11), 3), ((13, 40), 0), ((70, 2), 0),
                                       ((1, 1, 300, 3), 3)])
def test_weightnorm(shape, dim, dtype):
    # WeightNorm.cpp:45-72 over Conv2D (dim 3) and Linear (dim 0) weights in Flashlight's order
    rng = np.random.default_rng(100 + dim)
    rows = shape[dim]
    cols = int(np.prod(shape)) // rows
    rows_fast = dim == 0
    v = _round(rng.standard_normal(int(np.prod(shape))).astype(np.float32), dtype)
    g = _round((1 + 0.3 * rng.standard_normal(rows)).astype(np.float32), dtype)
    dw = _round(rng.standard_normal(v.size).astype(np.float32), dtype)
    tol = 1e-5 if dtype == torch.float32 else 6e-3
    assert rel_l2(host(ops.rownorm(dev(v, dtype), rows, cols, rows_fast)), flref.rownorm(v, rows, cols, rows_fast)) <= tol
    assert rel_l2(host(ops.weightnorm(dev(v, dtype), dev(g, dtype), rows, cols, rows_fast)),
                  flref.weightnorm_fwd(v, g, rows, cols, rows_fast)) <= tol
    dv, dg = ops.weightnorm_backward(dev(dw, dtype), dev(v, dtype), dev(g, dtype), rows, cols, rows_fast)
    dv_ref, dg_ref = flref.weightnorm_bwd(dw, v, g, rows, cols, rows_fast)
    assert rel_l2(host(dv), dv_ref) <= tol
    assert rel_l2(host(dg), dg_ref) <= (1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("dims,before,after", [((5, 4, 3, 2), (1, 0, 2, 0), (0, 3, 0, 1)), ((1500, 1, 80, 4), (170, 0, 0, 0), (0, 0, 0, 0)),
                                               ((7, 1, 1, 1), (2, 0, 0, 0), (5, 0, 0, 0)), ((3, 3, 2, 2), (0, 0, 0, 0), (0, 0, 0, 0))])
def test_padding(dims, before, after, dtype):
    rng = np.random.default_rng(110)
    x = _round(rng.standard_normal(int(np.prod(dims))).astype(np.float32), dtype)
    y_ref = flref.pad_fwd(x, dims, before, after, 0.25)
    assert np.array_equal(host(ops.padding(dev(x, dtype), dims, before, after, 0.25)), y_ref)
    dy = _round(rng.standard_normal(y_ref.size).astype(np.float32), dtype)
    assert np.array_equal(host(ops.padding_backward(dev(dy, dtype), dims, before, after)), flref.pad_bwd(dy, dims, before, after))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mu,wd,nesterov", [(0.0, 0.0, False), (0.9, 1e-2, False), (0.8, 5e-3, True)])
def test_sgd_many(mu, wd, nesterov, dtype):
    # several tensors (more than one launch holds), three steps; fp32 against the checker step by step
    rng = np.random.default_rng(120)
    sizes = [1, 5, 2048, 2049, 70001] + [int(rng.integers(1, 3000)) for _ in range(60)]
    ws = [_round(rng.standard_normal(n).astype(np.float32), dtype) for n in sizes]
    vs = [np.zeros(n, np.float32) for n in sizes] if mu else None
    wd_ = [dev(w, dtype) for w in ws]
    vd_ = [dev(v, dtype) for v in vs] if mu else None
    for step in range(3):
        gs = [_round(rng.standard_normal(n).astype(np.float32), dtype) for n in sizes]
        ops.sgd_step(wd_, [dev(g, dtype) for g in gs], vd_, 0.05, mu, wd, nesterov)
        for i in range(len(sizes)):
            ws[i], nv = flref.sgd(ws[i], gs[i], vs[i] if mu else None, 0.05, mu, wd, nesterov)
            if mu:
                vs[i] = _round(nv, dtype)
            ws[i] = _round(ws[i], dtype)
        tol = 2e-6 if dtype == torch.float32 else 8e-3
        for i in range(len(sizes)):
            assert rel_l2(host(wd_[i]), ws[i]) <= tol, (step, i, sizes[i])
            if mu:
                assert rel_l2(host(vd_[i]), vs[i]) <= tol, (step, i)


@pytest.mark.parametrize("wd", [0.0, 0.05])
def test_adam_many(wd):
    rng = np.random.default_rng(130)
    sizes = [1, 7, 2048, 2049, 50001] + [int(rng.integers(1, 3000)) for _ in range(40)]
    ws = [rng.standard_normal(n).astype(np.float32) for n in sizes]
    ms = [np.zeros(n, np.float32) for n in sizes]
    vs = [np.zeros(n, np.float32) for n in sizes]
    wd_, md_, vd_ = [dev(w) for w in ws], [dev(m) for m in ms], [dev(v) for v in vs]
    for t in range(1, 4):
        gs = [rng.standard_normal(n).astype(np.float32) for n in sizes]
        ops.adam_step(wd_, [dev(g) for g in gs], md_, vd_, 0.01, 0.9, 0.99, 1e-6, wd, t)
        for i in range(len(sizes)):
            ws[i], ms[i], vs[i] = flref.adam(ws[i], gs[i], ms[i], vs[i], 0.01, 0.9, 0.99, 1e-6, wd, t)
            assert rel_l2(host(wd_[i]), ws[i]) <= 2e-6 and rel_l2(host(md_[i]), ms[i]) <= 2e-6 and rel_l2(host(vd_[i]), vs[i]) <= 2e-6
