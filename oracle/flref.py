"""ctypes binding of the CPU checker (libflref.so).

Test infrastructure only: imported by tests/, by the smoke check and by the
CPU-baseline leg of bench.py — never by the flashlight_amd package.
Arrays are numpy float32, C-contiguous, in the reference's layout (row-major
N,C,H,W == Flashlight [W,H,C,N]).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "C", "H", "W", "K", "KH", "KW", "sy", "sx", "py", "px",
        "dil_y", "dil_x", "groups")]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "C", "H", "W", "wy", "wx", "sy", "sx", "py", "px", "mode")]


def build(force=False):
    so = os.path.join(_HERE, "libflref.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libflref.so"],
                              stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        _LIB = C.CDLL(build())
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def conv_desc(x_shape, w_shape, stride=(1, 1), pad=(0, 0), dil=(1, 1), groups=1):
    """stride/pad/dil are (y, x)."""
    N, Cc, H, W = x_shape
    K, Cg, KH, KW = w_shape
    assert Cg * groups == Cc, (x_shape, w_shape, groups)
    return ConvDesc(N, Cc, H, W, K, KH, KW, stride[0], stride[1], pad[0], pad[1],
                    dil[0], dil[1], groups)


def conv_out(d):
    oh, ow = C.c_int32(), C.c_int32()
    if lib().flref_conv_out(C.byref(d), C.byref(oh), C.byref(ow)):
        raise ValueError("invalid conv geometry")
    return oh.value, ow.value


def conv2d_fwd(d, x, w, b=None):
    x, w, b = _f32(x), _f32(w), _f32(b)
    oh, ow = conv_out(d)
    y = np.empty((d.N, d.K, oh, ow), np.float32)
    lib().flref_conv2d_fwd(C.byref(d), _p(x), _p(w), _p(b), _p(y))
    return y


def conv2d_bwd_data(d, dy, w):
    dy, w = _f32(dy), _f32(w)
    dx = np.empty((d.N, d.C, d.H, d.W), np.float32)
    lib().flref_conv2d_bwd_data(C.byref(d), _p(dy), _p(w), _p(dx))
    return dx


def conv2d_bwd_filter(d, x, dy, want_bias=True):
    x, dy = _f32(x), _f32(dy)
    dw = np.empty((d.K, d.C // d.groups, d.KH, d.KW), np.float32)
    db = np.empty((d.K,), np.float32) if want_bias else None
    lib().flref_conv2d_bwd_filter(C.byref(d), _p(x), _p(dy), _p(dw), _p(db))
    return dw, db


def pool_desc(x_shape, window, stride, pad, mode):
    """window/stride/pad are (y, x); mode 0 max, 1 avg-include, 2 avg-exclude."""
    N, Cc, H, W = x_shape
    return PoolDesc(N, Cc, H, W, window[0], window[1], stride[0], stride[1],
                    pad[0], pad[1], mode)


def pool_out(d):
    oh, ow = C.c_int32(), C.c_int32()
    if lib().flref_pool_out(C.byref(d), C.byref(oh), C.byref(ow)):
        raise ValueError("invalid pool geometry")
    return oh.value, ow.value


def pool2d_fwd(d, x):
    x = _f32(x)
    oh, ow = pool_out(d)
    y = np.empty((d.N, d.C, oh, ow), np.float32)
    am = np.zeros((d.N, d.C, oh, ow), np.uint8) if d.mode == 0 else None
    lib().flref_pool2d_fwd(C.byref(d), _p(x), _p(y), _p(am))
    return y, am


def pool2d_bwd(d, dy, argmax=None):
    dy = _f32(dy)
    if argmax is not None:
        argmax = np.ascontiguousarray(argmax, dtype=np.uint8)
    dx = np.empty((d.N, d.C, d.H, d.W), np.float32)
    lib().flref_pool2d_bwd(C.byref(d), _p(dy), _p(argmax), _p(dx))
    return dx


def _i64(v):
    return C.c_int64(int(v))


def bn_fwd_train(outer, Cc, inner, x, gamma, beta, eps):
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    y = np.empty_like(x)
    mean = np.empty((Cc,), np.float32)
    var = np.empty((Cc,), np.float32)
    lib().flref_bn_fwd_train(_i64(outer), _i64(Cc), _i64(inner), _p(x), _p(gamma),
                             _p(beta), C.c_double(eps), _p(y), _p(mean), _p(var))
    return y, mean, var


def bn_fwd_infer(outer, Cc, inner, x, gamma, beta, mean, var, eps):
    x, gamma, beta, mean, var = map(_f32, (x, gamma, beta, mean, var))
    y = np.empty_like(x)
    lib().flref_bn_fwd_infer(_i64(outer), _i64(Cc), _i64(inner), _p(x), _p(gamma),
                             _p(beta), _p(mean), _p(var), C.c_double(eps), _p(y))
    return y


def bn_bwd(outer, Cc, inner, x, dy, gamma, mean, var, eps):
    x, dy, gamma, mean, var = map(_f32, (x, dy, gamma, mean, var))
    dx = np.empty_like(x)
    dg = np.empty((Cc,), np.float32)
    db = np.empty((Cc,), np.float32)
    lib().flref_bn_bwd(_i64(outer), _i64(Cc), _i64(inner), _p(x), _p(dy), _p(gamma),
                       _p(mean), _p(var), C.c_double(eps), _p(dx), _p(dg), _p(db))
    return dx, dg, db


def bn_running_update(M, mean, var, momentum, run_mean, run_var):
    mean, var = _f32(mean), _f32(var)
    rm, rv = _f32(run_mean).copy(), _f32(run_var).copy()
    lib().flref_bn_running_update(_i64(mean.size), _i64(M), _p(mean), _p(var),
                                  C.c_double(momentum), _p(rm), _p(rv))
    return rm, rv


def bn_view(shape_whcn, axes):
    """(outer, C, inner) of the view the oneDNN extension builds from a Flashlight
    shape [d0,d1,...] (column-major) and feature axes
    (flashlight/fl/autograd/tensor/backend/onednn/BatchNorm.cpp:40-71,124-130)."""
    axes = sorted(axes)
    if axes != list(range(axes[0], axes[-1] + 1)):
        raise ValueError("axis array should be continuous")
    nfeat = 1
    for a in axes:
        nfeat *= shape_whcn[a]
    total = 1
    for s in shape_whcn:
        total *= s
    if axes[0] == 0:
        return total // nfeat, nfeat, 1
    outer = 1
    for s in shape_whcn[axes[-1] + 1:]:
        outer *= s
    return outer, nfeat, total // (nfeat * outer)


# ---- caller closures; matrices column-major (numpy: pass arrays whose reversed shape is
# the Flashlight shape, i.e. [cols, rows] row-major) ----------------------------------------

def relu_fwd(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().flref_relu_fwd(_i64(x.size), _p(x), _p(y))
    return y


ACT_ELU, ACT_CLAMP, ACT_TANH, ACT_LOG, ACT_SWISH, ACT_SIGMOID, ACT_SCALE, ACT_LEAKY, ACT_THRESHOLD = range(9)


def act_fwd(op, x, a=0.0, b=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    lib().flref_act_fwd(C.c_int(op), _i64(x.size), _p(x), C.c_double(a), C.c_double(b), _p(y))
    return y


def act_bwd(op, dy, x, a=0.0, b=0.0):
    dy, x = _f32(dy), _f32(x)
    dx = np.empty_like(x)
    lib().flref_act_bwd(C.c_int(op), _i64(x.size), _p(dy), _p(x), C.c_double(a), C.c_double(b), _p(dx))
    return dx


def glu_fwd(x, outer, m):
    """x: any array of outer * 2 * m elements in memory order [outer][2][m]."""
    x = _f32(x)
    y = np.empty(outer * m, np.float32)
    lib().flref_glu_fwd(_i64(outer), _i64(m), _p(x), _p(y))
    return y


def glu_bwd(dy, x, outer, m):
    dy, x = _f32(dy), _f32(x)
    dx = np.empty_like(x)
    lib().flref_glu_bwd(_i64(outer), _i64(m), _p(dy), _p(x), _p(dx))
    return dx


def embedding_fwd(idx, w):
    """idx: int array of n indices; w: [tokens, dim] (numpy order of the column-major dim x tokens) -> [n, dim]."""
    idx, w = np.ascontiguousarray(idx, dtype=np.int32).ravel(), _f32(w)
    y = np.empty((idx.size, w.shape[1]), dtype=np.float32)
    lib().flref_embedding_fwd(_i64(idx.size), _i64(w.shape[1]), _i64(w.shape[0]), idx.ctypes.data_as(C.c_void_p), _p(w), _p(y))
    return y


def embedding_bwd(idx, dy, tokens):
    idx, dy = np.ascontiguousarray(idx, dtype=np.int32).ravel(), _f32(dy)
    dw = np.empty((tokens, dy.shape[1]), dtype=np.float32)
    lib().flref_embedding_bwd(_i64(idx.size), _i64(dy.shape[1]), _i64(tokens), idx.ctypes.data_as(C.c_void_p), _p(dy), _p(dw))
    return dw


def prelu_fwd(x, w, d0):
    """x: any array whose fastest dimension has d0 elements; w: 1-D parameter whose size divides d0."""
    x, w = _f32(x), _f32(w)
    y = np.empty_like(x)
    lib().flref_prelu_fwd(_i64(x.size), _i64(d0), _i64(w.size), _p(x), _p(w), _p(y))
    return y


def prelu_bwd(dy, x, w, d0):
    dy, x, w = _f32(dy), _f32(x), _f32(w)
    dx, dw = np.empty_like(x), np.empty_like(w)
    lib().flref_prelu_bwd(_i64(x.size), _i64(d0), _i64(w.size), _p(dy), _p(x), _p(w), _p(dx), _p(dw))
    return dx, dw


def dropout(x, p, seed_lo, seed_hi):
    x = _f32(x)
    y = np.empty_like(x)
    lib().flref_dropout(_i64(x.size), _p(x), C.c_double(p), C.c_uint32(seed_lo), C.c_uint32(seed_hi), _p(y))
    return y


def rownorm(v, rows, cols, rows_fast):
    v = _f32(v)
    n = np.empty(rows, np.float32)
    lib().flref_rownorm(_i64(rows), _i64(cols), C.c_int(int(rows_fast)), _p(v), _p(n))
    return n


def weightnorm_fwd(v, g, rows, cols, rows_fast):
    v, g = _f32(v), _f32(g)
    w = np.empty_like(v)
    lib().flref_weightnorm_fwd(_i64(rows), _i64(cols), C.c_int(int(rows_fast)), _p(v), _p(g), _p(w))
    return w


def weightnorm_bwd(dw, v, g, rows, cols, rows_fast):
    dw, v, g = _f32(dw), _f32(v), _f32(g)
    dv, dg = np.empty_like(v), np.empty(rows, np.float32)
    lib().flref_weightnorm_bwd(_i64(rows), _i64(cols), C.c_int(int(rows_fast)), _p(dw), _p(v), _p(g), _p(dv), _p(dg))
    return dv, dg


def _pad_args(dims, before, after):
    return ((C.c_int64 * 4)(*dims), (C.c_int32 * 4)(*before), (C.c_int32 * 4)(*after))


def pad_fwd(x, dims, before, after, value):
    """dims / before / after: four column-major entries (dims[0] fastest); x in memory order."""
    x = _f32(x)
    d, b, a = _pad_args(dims, before, after)
    y = np.empty(int(np.prod([dims[k] + before[k] + after[k] for k in range(4)])), np.float32)
    lib().flref_pad_fwd(d, b, a, C.c_double(value), _p(x), _p(y))
    return y


def pad_bwd(dy, dims, before, after):
    dy = _f32(dy)
    d, b, a = _pad_args(dims, before, after)
    dx = np.empty(int(np.prod(dims)), np.float32)
    lib().flref_pad_bwd(d, b, a, _p(dy), _p(dx))
    return dx


def sgd(w, g, v, lr, mu, wd, nesterov):
    """One SGD step; returns (w, v) as new arrays (v None when mu == 0)."""
    w = _f32(w).copy()
    g = _f32(g)
    v = _f32(v).copy() if v is not None else None
    lib().flref_sgd(_i64(w.size), _p(w), _p(g), _p(v) if v is not None else None, C.c_double(lr), C.c_double(mu),
                    C.c_double(wd), C.c_int(int(nesterov)))
    return w, v


def adam(w, g, m, v, lr, b1, b2, eps, wd, step):
    """One Adam step; returns new (w, m, v)."""
    w, m, v = _f32(w).copy(), _f32(m).copy(), _f32(v).copy()
    g = _f32(g)
    lib().flref_adam(_i64(w.size), _p(w), _p(g), _p(m), _p(v), C.c_double(lr), C.c_double(b1), C.c_double(b2),
                     C.c_double(eps), C.c_double(wd), _i64(step))
    return w, m, v


def relu_bwd(dy, x):
    dy, x = _f32(dy), _f32(x)
    dx = np.empty_like(x)
    lib().flref_relu_bwd(_i64(x.size), _p(dy), _p(x), _p(dx))
    return dx


def matmul(M, N, K, A, B, ta=False, tb=False, bias=None):
    """C (M x N, column-major, returned as a numpy [N, M] array)."""
    A, B = _f32(A), _f32(B)
    b = None if bias is None else _f32(bias)
    out = np.empty((N, M), np.float32)
    lib().flref_matmul(C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(int(ta)), C.c_int(int(tb)), _p(A),
                       _p(B), None if b is None else _p(b), _p(out))
    return out


def sum_columns(rows, cols, x):
    x = _f32(x)
    out = np.empty((rows,), np.float32)
    lib().flref_sum_columns(C.c_int(rows), C.c_int(cols), _p(x), _p(out))
    return out


def affine_fwd(outer, mid, inner, scalar, x, w, b):
    x, w, b = _f32(x), _f32(w), _f32(b)
    y = np.empty_like(x)
    lib().flref_affine_fwd(_i64(outer), _i64(mid), _i64(inner), C.c_int(int(scalar)), _p(x), _p(w),
                           _p(b), _p(y))
    return y


def affine_bwd(outer, mid, inner, scalar, dy, x, w):
    """-> (dx, dw, db)"""
    dy, x, w = _f32(dy), _f32(x), _f32(w)
    n = 1 if scalar else mid
    dx = np.empty_like(x)
    dw, db = np.empty((n,), np.float32), np.empty((n,), np.float32)
    lib().flref_affine_bwd(_i64(outer), _i64(mid), _i64(inner), C.c_int(int(scalar)), _p(dy), _p(x),
                           _p(w), _p(dx), _p(dw), _p(db))
    return dx, dw, db


def logsoftmax_fwd(x):
    """x: numpy [cols, classes] (Flashlight [classes, cols])."""
    x = _f32(x)
    y = np.empty_like(x)
    lib().flref_logsoftmax_fwd(C.c_int(x.shape[-1]), C.c_int(x.size // x.shape[-1]), _p(x), _p(y))
    return y


def logsoftmax_bwd(dy, y):
    dy, y = _f32(dy), _f32(y)
    dx = np.empty_like(y)
    lib().flref_logsoftmax_bwd(C.c_int(y.shape[-1]), C.c_int(y.size // y.shape[-1]), _p(dy), _p(y),
                               _p(dx))
    return dx


def cce_fwd(logp, target, ignore=-1):
    """-> (per_column, loss_sum, loss_mean, count, bad)."""
    logp = _f32(logp)
    t = np.ascontiguousarray(target, dtype=np.int32)
    per = np.empty((t.size,), np.float32)
    loss = np.empty((2,), np.float32)
    cnt = C.c_float()
    bad = lib().flref_cce_fwd(C.c_int(logp.shape[-1]), C.c_int(t.size), _p(logp),
                              t.ctypes.data_as(C.c_void_p), C.c_int(ignore), _p(per), _p(loss),
                              C.byref(cnt))
    return per, float(loss[0]), float(loss[1]), cnt.value, bad


def cce_bwd(shape, grad, target, count, reduction=1, ignore=-1):
    g = _f32(np.atleast_1d(grad))
    t = np.ascontiguousarray(target, dtype=np.int32)
    dx = np.empty(shape, np.float32)
    lib().flref_cce_bwd(C.c_int(shape[-1]), C.c_int(t.size), _p(g), t.ctypes.data_as(C.c_void_p),
                        C.c_int(ignore), C.c_int(reduction), C.c_float(count), _p(dx))
    return dx


# ---- fl::LayerNorm::forward (flashlight/fl/nn/modules/LayerNorm.cpp:42-131) restated on
# the functions above: the shape is padded to 4 dimensions, batchnorm runs in train mode
# over the complement of the normalised axes with no parameters, then the broadcast
# scale and shift.  A non-contiguous complement goes through the reference's reorder
# (numpy transposes here), LayerNorm.cpp:63-86 and 98-108.
def layer_norm_plan(shape_whcn, norm_axes, nparam):
    whcn = list(shape_whcn) + [1] * (4 - len(shape_whcn))
    norm = sorted(norm_axes)
    comp = [d for d in range(4) if d not in norm]
    if comp != list(range(comp[0], comp[-1] + 1)):
        raise ValueError("non-contiguous complement")
    view = None
    if nparam == 1:
        view = (1, 1, int(np.prod(whcn)), True)
    elif nparam:
        inner = int(np.prod(whcn[:norm[0]]))
        mid = int(np.prod(whcn[norm[0]:norm[-1] + 1]))
        outer = int(np.prod(whcn[norm[-1] + 1:]))
        assert mid == nparam and norm == list(range(norm[0], norm[-1] + 1))
        view = (outer, mid, inner, False)
    return bn_view(whcn, comp), view


def _ln_reorder(shape_whcn, norm_axes, nparam=0):
    """The reorder of LayerNorm.cpp:63-86 for a non-contiguous complement, or None: Flashlight
    dims = normalised axes (ascending) then the complement; batchnorm then runs over the
    last len(comp) dims.  Returned as numpy axes of the row-major array (reversed order).
    Per-element parameters over normalised axes that are not contiguous take this general
    path too (the transposes cancel; the broadcast is then plain numpy)."""
    whcn = list(shape_whcn) + [1] * (4 - len(shape_whcn))
    norm = sorted(norm_axes)
    comp = [d for d in range(4) if d not in norm]
    norm_ok = nparam <= 1 or norm == list(range(norm[0], norm[-1] + 1))
    if comp == list(range(comp[0], comp[-1] + 1)) and norm_ok:
        return None
    order = norm + comp                                   # Flashlight dim i of the result = dim order[i]
    np_axes = [3 - d for d in order][::-1]                # numpy (row-major) axes of the result
    new_whcn = [whcn[d] for d in order]
    return whcn, norm, comp, np_axes, new_whcn


def _ln_bshape(whcn, norm):
    """numpy broadcast shape of per-element parameters: the tensor's shape with the complement
    axes set to 1 (LayerNorm.cpp:113-124)."""
    return [whcn[d] if d in norm else 1 for d in range(4)][::-1]


def layer_norm_fwd(x, shape_whcn, norm_axes, eps, w=None, b=None):
    """-> (y, xhat, mean, var); x is the flat/any-shape array of the tensor's memory."""
    ro = _ln_reorder(shape_whcn, norm_axes, 0 if w is None else np.size(w))
    if ro is None:
        bnv, view = layer_norm_plan(shape_whcn, norm_axes, 0 if w is None else np.size(w))
        ones, zeros = np.ones(bnv[1], np.float32), np.zeros(bnv[1], np.float32)
        xhat, mean, var = bn_fwd_train(*bnv, x, ones, zeros, eps)
        y = xhat if w is None else affine_fwd(*view, xhat, w, b)
        return y, xhat, mean, var
    whcn, norm, comp, np_axes, new_whcn = ro
    x4 = np.asarray(x, np.float32).reshape(whcn[::-1])
    xr = np.ascontiguousarray(x4.transpose(np_axes))                       # reorder(input, reorderDims)
    bnv = bn_view(new_whcn, list(range(len(norm), 4)))
    ones, zeros = np.ones(bnv[1], np.float32), np.zeros(bnv[1], np.float32)
    xh_r, mean, var = bn_fwd_train(*bnv, xr, ones, zeros, eps)
    xhat = np.ascontiguousarray(xh_r.reshape(xr.shape).transpose(np.argsort(np_axes)))   # restore
    y = xhat
    if w is not None:
        if np.size(w) == 1:
            y = (np.float32(w.reshape(-1)[0]) * xhat + np.float32(b.reshape(-1)[0])).astype(np.float32)
        else:
            bs = _ln_bshape(whcn, norm)
            y = (np.asarray(w, np.float32).reshape(bs) * xhat + np.asarray(b, np.float32).reshape(bs)).astype(np.float32)
    return y, xhat, mean, var


def layer_norm_bwd(dy, x, xhat, mean, var, shape_whcn, norm_axes, eps, w=None):
    """-> (dx, dw, db)"""
    ro = _ln_reorder(shape_whcn, norm_axes, 0 if w is None else np.size(w))
    if ro is None:
        bnv, view = layer_norm_plan(shape_whcn, norm_axes, 0 if w is None else np.size(w))
        dw = db = None
        g = dy
        if w is not None:
            g, dw, db = affine_bwd(*view, dy, xhat, w)
        dx, _, _ = bn_bwd(*bnv, x, g, np.ones(bnv[1], np.float32), mean, var, eps)
        return dx, dw, db
    whcn, norm, comp, np_axes, new_whcn = ro
    shape = whcn[::-1]
    dy4 = np.asarray(dy, np.float32).reshape(shape)
    xh4 = np.asarray(xhat, np.float32).reshape(shape)
    dw = db = None
    g = dy4
    if w is not None:
        d64, h64 = dy4.astype(np.float64), xh4.astype(np.float64)
        if np.size(w) == 1:
            dw = np.array([(d64 * h64).sum()], np.float32)
            db = np.array([d64.sum()], np.float32)
            g = (np.float32(np.asarray(w).reshape(-1)[0]) * dy4).astype(np.float32)
        else:
            red = tuple(3 - d for d in comp)
            dw = (d64 * h64).sum(axis=red).reshape(-1).astype(np.float32)
            db = d64.sum(axis=red).reshape(-1).astype(np.float32)
            g = (np.asarray(w, np.float32).reshape(_ln_bshape(whcn, norm)) * dy4).astype(np.float32)
    xr = np.ascontiguousarray(np.asarray(x, np.float32).reshape(shape).transpose(np_axes))
    gr = np.ascontiguousarray(g.transpose(np_axes))
    bnv = bn_view(new_whcn, list(range(len(norm), 4)))
    dx_r, _, _ = bn_bwd(*bnv, xr, gr, np.ones(bnv[1], np.float32), mean, var, eps)
    dx = np.ascontiguousarray(dx_r.reshape(xr.shape).transpose(np.argsort(np_axes)))
    return dx, dw, db


# ---- rnn / rnnBackward (cuDNN semantics, flat cuDNN weight order; see flref.h) ------------
RNN_RELU, RNN_TANH, RNN_LSTM, RNN_GRU = 0, 1, 2, 3


class RnnDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("input_size", "hidden", "layers", "bidirectional", "mode", "T", "B")] + [
        ("dropout", C.c_float), ("seed_lo", C.c_uint32), ("seed_hi", C.c_uint32)]


def rnn_desc(input_size, hidden, layers, bidirectional, mode, T, B, dropout=0.0, seed=0):
    return RnnDesc(input_size, hidden, layers, int(bool(bidirectional)), mode, T, B, float(dropout),
                   seed & 0xffffffff, (seed >> 32) & 0xffffffff)


def dropout_keep(seed, layer, n, dropout):
    """the keep mask of the first n elements of the output of `layer` (bool array)"""
    f = lib().flref_dropout_keep
    f.restype = C.c_int
    f.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_float]
    return np.array([f(seed & 0xffffffff, (seed >> 32) & 0xffffffff, layer, i, dropout) for i in range(n)], bool)


def rnn_param_count(d):
    f = lib().flref_rnn_param_count
    f.restype = C.c_int64
    return int(f(C.byref(d)))


def _opt(a):
    return None if a is None else _f32(a)


def rnn_fwd(d, x, w, hx=None, cx=None):
    """x [T, B, input], hx / cx [layers*dirs, B, hidden] or None -> (y, hy, cy or None)"""
    x, w, hx, cx = _f32(x), _f32(w), _opt(hx), _opt(cx)
    D = 2 if d.bidirectional else 1
    y = np.empty((d.T, d.B, D * d.hidden), np.float32)
    hy = np.empty((d.layers * D, d.B, d.hidden), np.float32)
    cy = np.empty_like(hy) if d.mode == RNN_LSTM else None
    lib().flref_rnn_fwd(C.byref(d), _p(x), _p(hx) if hx is not None else None, _p(cx) if cx is not None else None,
                        _p(w), _p(y), _p(hy), _p(cy) if cy is not None else None)
    return y, hy, cy


def rnn_bwd(d, x, w, hx=None, cx=None, dy=None, dhy=None, dcy=None):
    """-> (dx, dhx, dcx or None, dw)"""
    x, w, hx, cx, dy, dhy, dcy = _f32(x), _f32(w), _opt(hx), _opt(cx), _opt(dy), _opt(dhy), _opt(dcy)
    D = 2 if d.bidirectional else 1
    dx = np.empty_like(x)
    dhx = np.empty((d.layers * D, d.B, d.hidden), np.float32)
    dcx = np.empty_like(dhx) if d.mode == RNN_LSTM else None
    dw = np.empty_like(w)
    q = lambda a: _p(a) if a is not None else None
    lib().flref_rnn_bwd(C.byref(d), _p(x), q(hx), q(cx), _p(w), q(dy), q(dhy), q(dcy), _p(dx), _p(dhx), q(dcx),
                        _p(dw))
    return dx, dhx, dcx, dw
