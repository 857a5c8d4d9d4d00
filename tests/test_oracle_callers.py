"""Pins the caller-closure functions of oracle/flref.c (ReLU, the matrix products of
Linear, logSoftmax, categorical cross-entropy) against PyTorch-CPU library routines in
float64 and against closed forms.  Arrays are row-major with the Flashlight shape
reversed: a Flashlight [features, batch] matrix is a numpy [batch, features] array."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import flref
from refmath import rel_l2


def test_relu_and_mask():
    # Functions.cpp:329-338, 1787-1789; AutogradTest checks relu by its Jacobian
    x = np.array([-2.0, -0.0, 0.0, 1e-30, 3.5, np.nan, -np.inf, np.inf], np.float32)
    y = flref.relu_fwd(x)
    assert np.array_equal(y, np.array([0, 0, 0, 1e-30, 3.5, 0, 0, np.inf], np.float32))
    dy = np.arange(1, 9, dtype=np.float32)
    assert np.array_equal(flref.relu_bwd(dy, x), np.array([0, 0, 0, 4, 5, 0, 0, 8], np.float32))
    rng = np.random.default_rng(1)
    x = rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(flref.relu_fwd(x), F.relu(torch.from_numpy(x)).numpy())


@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (64, 64, 16), (70, 33, 129), (1, 9, 200), (10, 1, 1)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_against_float64(M, N, K, ta, tb):
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    opA = rng.standard_normal((M, K))          # mathematical op(A), op(B)
    opB = rng.standard_normal((K, N))
    bias = rng.standard_normal(M).astype(np.float32)
    # storage: column-major M x K == numpy [K, M]; transposed storage K x M == numpy [M, K]
    A = np.ascontiguousarray(opA if ta else opA.T, dtype=np.float32)
    B = np.ascontiguousarray(opB if tb else opB.T, dtype=np.float32)
    a64 = (A.astype(np.float64) if ta else A.astype(np.float64).T)
    b64 = (B.astype(np.float64) if tb else B.astype(np.float64).T)
    want = a64 @ b64 + bias[:, None]
    got = flref.matmul(M, N, K, A, B, ta, tb, bias)          # numpy [N, M]
    assert rel_l2(got.T, want) < 1e-6


def test_linear_forward_backward_like_torch():
    # fl::linear (Functions.cpp:1255-1309): y = W x + b; dX = W^T dY; dW = dY X^T; db = sum dY
    rng = np.random.default_rng(3)
    fin, fout, batch = 37, 21, 9
    x = rng.standard_normal((batch, fin)).astype(np.float32)          # Flashlight [in, batch]
    w = rng.standard_normal((fin, fout)).astype(np.float32)           # Flashlight [out, in]
    b = rng.standard_normal(fout).astype(np.float32)
    dy = rng.standard_normal((batch, fout)).astype(np.float32)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    wt = torch.from_numpy(w).double().requires_grad_(True)            # [in, out]
    bt = torch.from_numpy(b).double().requires_grad_(True)
    yt = xt @ wt + bt
    yt.backward(torch.from_numpy(dy).double())
    y = flref.matmul(fout, batch, fin, w, x, False, False, b)
    assert rel_l2(y, yt.detach().numpy()) < 1e-6
    dx = flref.matmul(fin, batch, fout, w, dy, True, False)
    assert rel_l2(dx, xt.grad.numpy()) < 1e-6
    dw = flref.matmul(fout, fin, batch, dy, x, False, True)            # numpy [in, out]
    assert rel_l2(dw, wt.grad.numpy()) < 1e-6
    db = flref.sum_columns(fout, batch, dy)
    assert rel_l2(db, bt.grad.numpy()) < 1e-6


def test_logsoftmax_like_torch():
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((13, 10)) * 5).astype(np.float32)
    x[0, 3] = 80.0          # large logits: the max subtraction must keep this finite
    dy = rng.standard_normal((13, 10)).astype(np.float32)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    yt = torch.log_softmax(xt, dim=-1)
    yt.backward(torch.from_numpy(dy).double())
    y = flref.logsoftmax_fwd(x)
    assert np.allclose(y, yt.detach().numpy(), atol=1e-5, rtol=1e-6)
    assert np.allclose(np.exp(y.astype(np.float64)).sum(-1), 1.0, atol=1e-5)
    dx = flref.logsoftmax_bwd(dy, y)
    assert rel_l2(dx, xt.grad.numpy()) < 1e-5


@pytest.mark.parametrize("reduction", [0, 1, 2])
def test_cross_entropy_like_torch(reduction):
    # Functions.cpp:1078-1154, ignoreIndex = -1 by default
    rng = np.random.default_rng(5 + reduction)
    logp = np.log(rng.dirichlet(np.ones(10), size=17)).astype(np.float32)
    target = rng.integers(0, 10, 17).astype(np.int32)
    target[[2, 11]] = -1                                   # ignored columns
    per, s, mean, count, bad = flref.cce_fwd(logp, target)
    assert bad == 0 and count == 15
    lt = torch.from_numpy(logp).double().requires_grad_(True)
    tt = torch.from_numpy(target).long()
    mode = ["none", "mean", "sum"][reduction]
    want = F.nll_loss(lt, tt, ignore_index=-1, reduction=mode)
    got = [per, mean, s][reduction]
    assert np.allclose(got, want.detach().numpy(), rtol=1e-6, atol=1e-6)
    g = rng.standard_normal(17 if reduction == 0 else 1).astype(np.float32)
    want.backward(torch.from_numpy(g).double() if reduction == 0 else torch.tensor(float(g[0]), dtype=torch.float64))
    dx = flref.cce_bwd(logp.shape, g, target, count, reduction)
    assert np.allclose(dx, lt.grad.numpy(), rtol=1e-6, atol=1e-7)


def test_cross_entropy_flags_bad_targets():
    logp = np.zeros((4, 3), np.float32)
    assert flref.cce_fwd(logp, np.array([0, 3, 2, -2], np.int32))[4] == 2


@pytest.mark.parametrize("outer,mid,inner,scalar", [(3, 5, 7, False), (1, 6, 1, False), (4, 9, 1, False),
                                                    (1, 8, 5, False), (2, 3, 4, True)])
def test_affine_against_numpy_broadcast(outer, mid, inner, scalar):
    # tileAs(weight) * x + tileAs(bias) and the gradients of the broadcasts
    # (LayerNorm.cpp:110-128), written with numpy broadcasting in float64
    rng = np.random.default_rng(outer * 100 + mid * 10 + inner)
    x = rng.standard_normal((outer, mid, inner)).astype(np.float32)
    dy = rng.standard_normal((outer, mid, inner)).astype(np.float32)
    n = 1 if scalar else mid
    w, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    wb = w.astype(np.float64).reshape(1, n, 1)
    bb = b.astype(np.float64).reshape(1, n, 1)
    y = flref.affine_fwd(outer, mid, inner, scalar, x, w, b)
    assert rel_l2(y, wb * x + bb) < 1e-6
    dx, dw, db = flref.affine_bwd(outer, mid, inner, scalar, dy, x, w)
    assert rel_l2(dx, wb * dy) < 1e-6
    red = (0, 1, 2) if scalar else (0, 2)
    assert rel_l2(dw, (dy.astype(np.float64) * x).sum(axis=red).reshape(-1)) < 1e-6
    assert rel_l2(db, dy.astype(np.float64).sum(axis=red).reshape(-1)) < 1e-6


@pytest.mark.parametrize("whcn,norm,params", [
    ((6, 5, 4, 3), (0, 1, 2), "per"),      # the reference's LayerNorm test: axes {0,1,2} of WHCN
    ((6, 5, 4, 3), (0, 1, 2), "scalar"),
    ((16, 7, 3), (0,), "per"),             # transformer use: [C, T, B], normalise C
    ((16, 7, 3), (0,), None),
    ((5, 4, 3, 2), (3,), "per"),
    ((8, 3), (0, 1), "scalar"),
    # non-contiguous complement: the reorder branch (LayerNorm.cpp:63-86)
    ((6, 5, 4, 3), (1,), "per"),
    ((6, 5, 4, 3), (1, 2), None),
    ((6, 5, 4, 3), (0, 2), "scalar"),
    ((4, 7, 3, 2), (1, 3), "per"),
    ((5, 4, 6), (1,), "per"),
    ((6, 5, 4, 3), (0, 3), "per"),         # contiguous complement, parameters over axes that are not
])
def test_layer_norm_restated_on_batchnorm_is_layer_norm(whcn, norm, params):
    # LayerNorm.cpp:42-131 against torch.nn.functional.layer_norm (float64) and its autograd
    rng = np.random.default_rng(sum(whcn) + len(norm))
    tshape = tuple(whcn[::-1])                       # torch shape = reversed Flashlight shape
    x = (rng.standard_normal(tshape) * 2 + 0.5).astype(np.float32)
    dy = rng.standard_normal(tshape).astype(np.float32)
    w = b = None
    norm_t = sorted(len(whcn) - 1 - a for a in norm)    # torch dims that are normalised
    nshape = [whcn[a] for a in sorted(norm)][::-1]
    if params == "per":
        w = rng.standard_normal(int(np.prod(nshape))).astype(np.float32)
        b = rng.standard_normal(int(np.prod(nshape))).astype(np.float32)
    elif params == "scalar":
        w, b = np.array([1.7], np.float32), np.array([-0.3], np.float32)
    eps = 1e-5
    y, xhat, mean, var = flref.layer_norm_fwd(x, whcn, norm, eps, w, b)
    dx, dw, db = flref.layer_norm_bwd(dy, x, xhat, mean, var, whcn, norm, eps, w)
    # torch: move the normalised dims last (they are contiguous here), normalise, move back
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    keep = [d for d in range(len(tshape)) if d not in norm_t]
    perm = keep + norm_t
    xp = xt.permute(perm)
    yp = F.layer_norm(xp, xp.shape[len(keep):], eps=eps)
    inv = [perm.index(d) for d in range(len(tshape))]
    yt = yp.permute(inv)
    params_t = []
    if params == "per":
        bshape = [tshape[d] if d in norm_t else 1 for d in range(len(tshape))]
        wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
        bt = torch.tensor(b, dtype=torch.float64, requires_grad=True)
        yt = yt * wt.reshape(bshape) + bt.reshape(bshape)
        params_t = [wt, bt]
    elif params == "scalar":
        wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
        bt = torch.tensor(b, dtype=torch.float64, requires_grad=True)
        yt = yt * wt + bt
        params_t = [wt, bt]
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    assert rel_l2(y.reshape(tshape), yt.detach().numpy()) < 1e-5
    assert rel_l2(dx.reshape(tshape), xt.grad.numpy()) < 1e-4
    if params_t:
        assert rel_l2(dw, params_t[0].grad.numpy().reshape(-1)) < 1e-5
        assert rel_l2(db, params_t[1].grad.numpy().reshape(-1)) < 1e-5


# ---- the element-wise activations of nn/modules/Activations.cpp, gatedlinearunit, dropout ----
# (op, a, b, torch function in float64); log gets positive inputs
_ACTS = [
    (flref.ACT_ELU, 1.0, 0.0, lambda t: F.elu(t, alpha=1.0)),
    (flref.ACT_ELU, 0.3, 0.0, lambda t: F.elu(t, alpha=0.3)),
    (flref.ACT_CLAMP, 0.0, 6.0, lambda t: F.relu6(t)),
    (flref.ACT_CLAMP, -1.0, 1.0, lambda t: F.hardtanh(t)),
    (flref.ACT_TANH, 0.0, 0.0, torch.tanh),
    (flref.ACT_LOG, 0.0, 0.0, torch.log),
    (flref.ACT_SWISH, 1.0, 0.0, F.silu),
    (flref.ACT_SWISH, 1.7, 0.0, lambda t: t * torch.sigmoid(1.7 * t)),
    (flref.ACT_SIGMOID, 0.0, 0.0, torch.sigmoid),
    (flref.ACT_SCALE, -0.37, 0.0, lambda t: -0.37 * t),
    (flref.ACT_LEAKY, 0.01, 0.0, lambda t: F.leaky_relu(t, 0.01)),
    (flref.ACT_LEAKY, 0.3, 0.0, lambda t: torch.maximum(t, 0.3 * t)),
    (flref.ACT_LEAKY, 1.5, 0.0, lambda t: torch.where(t > 1.5 * t, t, 1.5 * t)),       # a slope above 1: still max(x, a x)
    (flref.ACT_THRESHOLD, 0.7, 0.0, lambda t: F.threshold(t, 0.7, 0.0) + 0.0 * t),
]


@pytest.mark.parametrize("op,a,b,fn", _ACTS)
def test_activations_against_torch_float64(op, a, b, fn):
    rng = np.random.default_rng(300 + op)
    x = (rng.standard_normal(4000) * 3).astype(np.float32)
    if op == flref.ACT_LOG:
        x = np.abs(x) + 0.05
    dy = rng.standard_normal(4000).astype(np.float32)
    t = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    y = fn(t)
    y.backward(torch.from_numpy(dy.astype(np.float64)))
    assert rel_l2(flref.act_fwd(op, x, a, b), y.detach().numpy()) <= 1e-6
    assert rel_l2(flref.act_bwd(op, dy, x, a, b), t.grad.numpy()) <= 1e-6


def test_clamp_passes_the_gradient_strictly_inside():
    # Functions.cpp:471: (result > lo) && (result < hi) — nothing at the bounds themselves
    x = np.array([-2.0, -1.0, -0.5, 0.0, 1.0, 1.5, 6.0, 7.0], np.float32)
    dy = np.arange(1, 9, dtype=np.float32)
    assert np.array_equal(flref.act_fwd(flref.ACT_CLAMP, x, -1.0, 1.0), np.array([-1, -1, -0.5, 0, 1, 1, 1, 1], np.float32))
    assert np.array_equal(flref.act_bwd(flref.ACT_CLAMP, dy, x, -1.0, 1.0), np.array([0, 0, 3, 4, 0, 0, 0, 0], np.float32))
    assert np.array_equal(flref.act_bwd(flref.ACT_CLAMP, dy, x, 0.0, 6.0), np.array([0, 0, 0, 0, 5, 6, 0, 0], np.float32))


@pytest.mark.parametrize("shape,dim", [((3, 8, 5), 1), ((4, 6), 1), ((10, 7), 0), ((2, 3, 4, 6), 3), ((2, 4, 3, 5), 1)])
def test_glu_against_torch_float64(shape, dim):
    # Functions.cpp:1567-1610; a torch dimension `dim` of a contiguous array: halves are blocks of m per outer index
    rng = np.random.default_rng(310 + dim)
    x = rng.standard_normal(shape).astype(np.float32)
    outer = int(np.prod(shape[:dim], dtype=np.int64))
    m = shape[dim] // 2 * int(np.prod(shape[dim + 1:], dtype=np.int64))
    t = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    y = F.glu(t, dim)
    dy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(torch.from_numpy(dy.astype(np.float64)))
    assert rel_l2(flref.glu_fwd(x, outer, m).reshape(y.shape), y.detach().numpy()) <= 1e-6
    assert rel_l2(flref.glu_bwd(dy, x, outer, m).reshape(shape), t.grad.numpy()) <= 1e-6


@pytest.mark.parametrize("n,dim,tokens", [(1, 1, 1), (7, 5, 3), (50, 16, 9), (200, 33, 1000), (64, 8, 2)])
def test_embedding_against_torch_float64(n, dim, tokens):
    """The checker's embedding against torch.nn.functional.embedding, forward and autograd (float64): a gather of
    table rows and a scatter-add of the deltas; tokens that occur twice and tokens that never occur both appear.
    Indices outside the table (which torch refuses) give zero columns and take no gradient."""
    import torch
    rng = np.random.default_rng(n + dim + tokens)
    idx = rng.integers(0, tokens, size=n).astype(np.int32)
    w = rng.standard_normal((tokens, dim)).astype(np.float32)
    dy = rng.standard_normal((n, dim)).astype(np.float32)
    wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    yt = torch.nn.functional.embedding(torch.tensor(idx, dtype=torch.int64), wt)
    yt.backward(torch.tensor(dy, dtype=torch.float64))
    assert np.array_equal(flref.embedding_fwd(idx, w), yt.detach().numpy().astype(np.float32))
    assert np.allclose(flref.embedding_bwd(idx, dy, tokens), wt.grad.numpy(), rtol=1e-6, atol=1e-6)
    # out of range: zeros forward, nothing backward
    bad = idx.copy()
    bad[0] = tokens
    if n > 1:
        bad[-1] = -1
    y = flref.embedding_fwd(bad, w)
    assert not y[0].any() and (n == 1 or not y[-1].any())
    keep = (bad >= 0) & (bad < tokens)
    want = np.zeros((tokens, dim))
    np.add.at(want, bad[keep], dy[keep].astype(np.float64))
    assert np.allclose(flref.embedding_bwd(bad, dy, tokens), want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape,size", [((4, 3, 10), 1), ((4, 3, 10), 10), ((5, 12), 12), ((2, 3, 4, 6), 1), ((7, 8), 4)])
def test_prelu_against_torch_float64(shape, size):
    # nn/modules/Activations.cpp:116-124: the parameter tiled along Flashlight's first dimension = the last one of
    # the contiguous array.  torch.nn.functional.prelu puts its parameter on dimension 1, so the pin is written with
    # torch's own operators (where / broadcasting) and autograd in float64; size 4 over extent 8 is tileAs' repeat.
    rng = np.random.default_rng(320 + size)
    x = rng.standard_normal(shape).astype(np.float32)
    x.flat[::7] = 0.0                                  # the mask is x >= 0: a zero passes the gradient whole
    w = rng.uniform(0.1, 0.9, size).astype(np.float32)
    d0 = shape[-1]
    t = torch.from_numpy(x.astype(np.float64)).requires_grad_(True)
    tw = torch.from_numpy(w.astype(np.float64)).requires_grad_(True)
    y = torch.where(t >= 0, t, t * tw.repeat(d0 // size))
    dy = rng.standard_normal(shape).astype(np.float32)
    y.backward(torch.from_numpy(dy.astype(np.float64)))
    assert rel_l2(flref.prelu_fwd(x, w, d0), y.detach().numpy()) <= 1e-6
    dx, dw = flref.prelu_bwd(dy, x, w, d0)
    assert rel_l2(dx, t.grad.numpy()) <= 1e-6 and rel_l2(dw, tw.grad.numpy()) <= 1e-6
    if size == 1 and len(shape) == 2:
        # the one case the library routine states the same way: a single parameter
        assert rel_l2(flref.prelu_fwd(x, w, d0), F.prelu(torch.from_numpy(x), torch.from_numpy(w)).numpy()) <= 1e-6
    assert np.array_equal(dx.flat[::7], dy.flat[::7])


def test_dropout_mask_rate_scale_and_determinism():
    # Functions.cpp:1777-1785: zero with probability p, the rest scaled by 1 / (1 - p); the mask is a function of
    # (seed, index) only
    x = np.ones(200000, np.float32)
    for p in (0.2, 0.5, 0.9):
        y = flref.dropout(x, p, 123, 456)
        kept = y != 0
        assert np.allclose(y[kept], 1.0 / (1.0 - p), rtol=1e-6)
        assert abs(kept.mean() - (1.0 - p)) < 4 * np.sqrt(p * (1 - p) / x.size)
        assert np.array_equal(y, flref.dropout(x, p, 123, 456))
        assert not np.array_equal(y, flref.dropout(x, p, 124, 456))
    assert np.array_equal(flref.dropout(x, 0.0, 1, 2), x)


@pytest.mark.parametrize("shape,dim", [((7, 3, 5, 11), 3), ((13, 40), 0), ((1, 1, 9, 4), 3), ((64, 3), 0)])
def test_weightnorm_against_torch_float64(shape, dim):
    # WeightNorm.cpp:45-72 on a Flashlight (column-major) weight of `shape`: numpy holds it with the shape reversed
    rng = np.random.default_rng(320 + dim)
    rows = shape[dim]
    cols = int(np.prod(shape)) // rows
    rows_fast = dim == 0
    v = rng.standard_normal(shape[::-1]).astype(np.float32)          # numpy [d3, d2, d1, d0]
    g = (1 + 0.3 * rng.standard_normal(rows)).astype(np.float32)
    dw = rng.standard_normal(v.shape).astype(np.float32)
    tv = torch.from_numpy(v.astype(np.float64)).requires_grad_(True)
    tg = torch.from_numpy(g.astype(np.float64)).requires_grad_(True)
    ax = v.ndim - 1 - dim                                            # the kept numpy axis
    other = tuple(a for a in range(v.ndim) if a != ax)
    bshape = [1] * v.ndim
    bshape[ax] = rows
    nrm = torch.sqrt((tv * tv).sum(dim=other, keepdim=True))
    w = tv * (tg.reshape(bshape) / nrm)
    w.backward(torch.from_numpy(dw.astype(np.float64)))
    assert rel_l2(flref.rownorm(v, rows, cols, rows_fast), nrm.detach().numpy().ravel()) <= 1e-6
    assert rel_l2(flref.weightnorm_fwd(v, g, rows, cols, rows_fast), w.detach().numpy()) <= 1e-6
    dv, dg = flref.weightnorm_bwd(dw, v, g, rows, cols, rows_fast)
    assert rel_l2(dv, tv.grad.numpy()) <= 1e-6
    assert rel_l2(dg, tg.grad.numpy()) <= 1e-6


@pytest.mark.parametrize("dims,before,after", [((5, 4, 3, 2), (1, 0, 2, 0), (0, 3, 0, 1)), ((7, 1, 1, 1), (2, 0, 0, 0), (5, 0, 0, 0)),
                                               ((3, 3, 2, 2), (0, 0, 0, 0), (0, 0, 0, 0))])
def test_padding_against_numpy(dims, before, after):
    # Functions.cpp:1751-1775: the input inside a tensor of `val`; the gradient is the inner box
    rng = np.random.default_rng(330)
    x = rng.standard_normal(dims[::-1]).astype(np.float32)           # numpy [d3, d2, d1, d0]
    widths = [(before[k], after[k]) for k in (3, 2, 1, 0)]
    ref = np.pad(x, widths, constant_values=-1.5)
    assert np.array_equal(flref.pad_fwd(x, dims, before, after, -1.5).reshape(ref.shape), ref)
    dy = rng.standard_normal(ref.shape).astype(np.float32)
    sl = tuple(slice(b, b + n) for (b, _), n in zip(widths, x.shape))
    assert np.array_equal(flref.pad_bwd(dy, dims, before, after).reshape(x.shape), dy[sl])


@pytest.mark.parametrize("mu,wd,nesterov", [(0.0, 0.0, False), (0.9, 0.0, False), (0.9, 1e-2, False), (0.8, 5e-3, True), (0.0, 1e-2, False)])
def test_sgd_against_torch_optim(mu, wd, nesterov):
    # optim/SGDOptimizer.cpp:38-68 is torch.optim.SGD's update (dampening 0): three steps with fresh gradients
    rng = np.random.default_rng(340)
    w = rng.standard_normal(500).astype(np.float32)
    tw = torch.nn.Parameter(torch.from_numpy(w.astype(np.float64)))
    opt = torch.optim.SGD([tw], lr=0.05, momentum=mu, weight_decay=wd, nesterov=nesterov)
    v = np.zeros_like(w) if mu else None
    for step in range(3):
        g = rng.standard_normal(500).astype(np.float32)
        tw.grad = torch.from_numpy(g.astype(np.float64))
        opt.step()
        w, v = flref.sgd(w, g, v, 0.05, mu, wd, nesterov)
        assert rel_l2(w, tw.detach().numpy()) <= 1e-6


@pytest.mark.parametrize("wd", [0.0, 0.05])
def test_adam_against_torch_adamw(wd):
    # optim/AdamOptimizer.cpp:45-79: decoupled decay and lr sqrt(1 - b2^t) / (1 - b1^t) m / (sqrt(v) + eps).  torch's
    # AdamW divides by sqrt(v) / sqrt(1 - b2^t) + eps', the same update for eps' = eps / sqrt(1 - b2^t): each step is
    # checked against one step of a torch optimizer given the state before it and that epsilon.
    rng = np.random.default_rng(350)
    lr, b1, b2, eps = 0.01, 0.9, 0.99, 1e-6
    w = rng.standard_normal(400).astype(np.float32)
    m, v = np.zeros_like(w), np.zeros_like(w)
    for t in range(1, 5):
        g = rng.standard_normal(400).astype(np.float32)
        tw = torch.nn.Parameter(torch.from_numpy(w.astype(np.float64)))
        opt = torch.optim.AdamW([tw], lr=lr, betas=(b1, b2), eps=eps / np.sqrt(1 - b2 ** t), weight_decay=wd)
        opt.state[tw] = {"step": torch.tensor(float(t - 1)), "exp_avg": torch.from_numpy(m.astype(np.float64)),
                         "exp_avg_sq": torch.from_numpy(v.astype(np.float64))}
        tw.grad = torch.from_numpy(g.astype(np.float64))
        opt.step()
        w, m, v = flref.adam(w, g, m, v, lr, b1, b2, eps, wd, t)
        assert rel_l2(w, tw.detach().numpy()) <= 2e-6
        assert rel_l2(m, opt.state[tw]["exp_avg"].numpy()) <= 1e-6
        assert rel_l2(v, opt.state[tw]["exp_avg_sq"].numpy()) <= 1e-6
