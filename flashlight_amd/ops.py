"""Operator-level binding over torch device tensors.

Argument order and meaning follow fl::AutogradExtension
(flashlight/fl/autograd/tensor/AutogradExtension.h:58-164): ints in x-then-y
order, `axes` as Flashlight dimension indices of the column-major shape
[W,H,C,N].  A contiguous torch tensor of shape (N,C,H,W) is byte-identical to
that Flashlight tensor, so torch is used here only as the owner of device
memory and of the stream.
"""
import ctypes as C
import enum

import torch

from . import capi


class PoolingMode(enum.IntEnum):
    """fl::PoolingMode (flashlight/fl/common/Defines.h:53-64)."""
    MAX = 0
    AVG_INCLUDE_PADDING = 1
    AVG_EXCLUDE_PADDING = 2


def derive_padding(in_size, filter_size, stride, pad, dilation=1):
    """fl::derivePadding (flashlight/fl/nn/Utils.cpp:87-100); pad == -1 is SAME."""
    if pad == -1:
        rem = in_size % stride
        p = ((filter_size - 1) * dilation - (stride if rem == 0 else rem) + 1 + 1) // 2
        return max(p, 0)
    return pad


def _dtype_tag(t):
    if t.dtype == torch.float32:
        return capi.F32
    if t.dtype == torch.bfloat16:
        return capi.BF16
    if t.dtype == torch.float16:
        return capi.F16
    raise RuntimeError("flashlight_amd: unsupported dtype %s" % t.dtype)


_TAG_OF = {torch.float32: capi.F32, torch.bfloat16: capi.BF16, torch.float16: capi.F16}


def _dev(t, name):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("%s must live on the GPU" % name)
    if not t.is_contiguous():
        # fl::DevicePtr refuses non-contiguous tensors (flashlight/fl/common/DevicePtr.cpp:16-33)
        raise ValueError("%s must be contiguous" % name)
    return t


def _ptr(t):
    return None if t is None or t.numel() == 0 else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _as4(t):
    """Missing trailing Flashlight dims count as 1 (onednn/Pool2D.cpp:95-98);
    in row-major terms: missing LEADING dims."""
    if t.dim() > 4:
        raise ValueError("at most 4 dimensions")
    return (1,) * (4 - t.dim()) + tuple(t.shape)


def _conv_desc(x_shape, w_shape, sx, sy, px, py, dx, dy, groups, tag):
    N, Cc, H, W = x_shape
    K, Cg, KH, KW = w_shape
    if Cg * groups != Cc:
        raise ValueError("conv2d: weight/input channel mismatch")
    return capi.ConvDesc(N, Cc, H, W, K, KH, KW, sy, sx, py, px, dy, dx, groups, tag)


def _ws(nbytes, device):
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def conv2d(input, weights, bias, sx=1, sy=1, px=0, py=0, dx=1, dy=1, groups=1, keep_gathered=False):
    """AutogradExtension::conv2d.  bias may be None or empty.
    keep_gathered: returns (output, gathered) - what the closure's payload carries to the backward pass:
    the gathered input that the forward pass of a strided bf16 layer leaves in its workspace (None for
    geometries that gather nothing), to be given to conv2d_backward_filter_bias(gathered=...)."""
    x, w = _dev(input, "input"), _dev(weights, "weights")
    if x.dim() != 4 or w.dim() != 4:
        raise ValueError("conv2d: input and weights must have 4 dimensions")
    if x.dtype != w.dtype:
        raise ValueError("conv2d: input and weights must have the same type")
    tag = _dtype_tag(x)
    d = _conv_desc(x.shape, w.shape, sx, sy, px, py, dx, dy, groups, tag)
    oh, ow = C.c_int32(), C.c_int32()
    capi.check(capi.lib().flhip_conv2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)))
    b = None
    if bias is not None and bias.numel() > 0:
        if bias.numel() != d.K:
            raise ValueError("conv2d: bias must have one element per output channel")
        b = _dev(bias, "bias").float().contiguous()
    y = torch.empty((d.N, d.K, oh.value, ow.value), dtype=x.dtype, device=x.device)
    nws = capi.lib().flhip_conv2d_workspace_bytes(C.byref(d), capi.CONV_FWD)
    ws = _ws(nws, x.device)
    capi.check(capi.lib().flhip_conv2d_fwd(C.byref(d), _ptr(x), _ptr(w), _ptr(b), _ptr(y),
                                           _ptr(ws), nws, _stream()))
    if keep_gathered:
        ngb = capi.lib().flhip_conv2d_gathered_bytes(C.byref(d))
        return y, (ws[:ngb] if ngb > 0 else None)
    return y


def conv2d_backward_data(grad_output, input_shape, weights, sx=1, sy=1, px=0, py=0, dx=1, dy=1,
                         groups=1, addend=None):
    """AutogradExtension::conv2dBackwardData; only the input's shape is needed
    (onednn/Conv2D.cpp:285).  addend: a gradient the input already holds; the result is then
    addend + the pass's result (Variable::addGrad), in one pass where the kernel allows it."""
    g, w = _dev(grad_output, "gradOutput"), _dev(weights, "weights")
    tag = _dtype_tag(g)
    d = _conv_desc(tuple(input_shape), w.shape, sx, sy, px, py, dx, dy, groups, tag)
    oh, ow = C.c_int32(), C.c_int32()
    capi.check(capi.lib().flhip_conv2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)))
    if tuple(g.shape) != (d.N, d.K, oh.value, ow.value):
        raise ValueError("conv2dBackwardData: gradOutput shape does not match the geometry")
    out = torch.empty(tuple(input_shape), dtype=g.dtype, device=g.device)
    nws = capi.lib().flhip_conv2d_workspace_bytes(C.byref(d), capi.CONV_BWD_DATA)
    ws = _ws(nws, g.device)
    if addend is not None:
        a = _dev(addend, "addend")
        if tuple(a.shape) != tuple(input_shape) or a.dtype != g.dtype:
            raise ValueError("conv2dBackwardData: addend must have the input's shape and the gradient's type")
        capi.check(capi.lib().flhip_conv2d_bwd_data_add(C.byref(d), _ptr(g), _ptr(w), _ptr(a), _ptr(out),
                                                        _ptr(ws), nws, _stream()))
        return out
    capi.check(capi.lib().flhip_conv2d_bwd_data(C.byref(d), _ptr(g), _ptr(w), _ptr(out),
                                                _ptr(ws), nws, _stream()))
    return out


def conv2d_backward_filter_bias(grad_output, input, weights_shape, want_bias, sx=1, sy=1, px=0,
                                py=0, dx=1, dy=1, groups=1, gathered=None):
    """AutogradExtension::conv2dBackwardFilterBias -> (gradWeights, gradBias or None).
    Gradients are fp32 (the master-weight precision) for both storage types.
    gathered: what conv2d(keep_gathered=True) returned for this layer (the payload); the pass then
    skips gathering the input again."""
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    tag = _dtype_tag(x)
    d = _conv_desc(x.shape, tuple(weights_shape), sx, sy, px, py, dx, dy, groups, tag)
    oh, ow = C.c_int32(), C.c_int32()
    capi.check(capi.lib().flhip_conv2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)))
    if tuple(g.shape) != (d.N, d.K, oh.value, ow.value):
        raise ValueError("conv2dBackwardFilterBias: gradOutput shape does not match the geometry")
    dw = torch.empty(tuple(weights_shape), dtype=torch.float32, device=x.device)
    db = torch.empty((d.K,), dtype=torch.float32, device=x.device) if want_bias else None
    nws = capi.lib().flhip_conv2d_workspace_bytes(C.byref(d), capi.CONV_BWD_FILTER)
    ws = _ws(nws, x.device)
    if gathered is not None:
        if gathered.numel() != capi.lib().flhip_conv2d_gathered_bytes(C.byref(d)):
            raise ValueError("conv2dBackwardFilterBias: gathered input of another geometry")
        capi.check(capi.lib().flhip_conv2d_bwd_filter_gathered(C.byref(d), _ptr(gathered), _ptr(g), _ptr(dw),
                                                           _ptr(db), _ptr(ws), nws, _stream()))
        return dw, db
    capi.check(capi.lib().flhip_conv2d_bwd_filter(C.byref(d), _ptr(x), _ptr(g), _ptr(dw), _ptr(db),
                                                  _ptr(ws), nws, _stream()))
    return dw, db


def conv2d_backward_filter_bias_static(grad_output, input, dw, db, sx=1, sy=1, px=0, py=0, dx=1,
                                       dy=1, groups=1):
    """flhip_conv2d_bwd_filter_static: the filter / bias gradient written into the
    caller's fp32 tensors `dw` (weight shape) and `db` (or None), with the partial
    results in the library's static buffer.  Neither this wrapper nor the library
    allocates device memory."""
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    if dw.dtype != torch.float32 or (db is not None and db.dtype != torch.float32):
        raise ValueError("conv2dBackwardFilterBias: gradients are fp32")
    d = _conv_desc(x.shape, tuple(dw.shape), sx, sy, px, py, dx, dy, groups, _dtype_tag(x))
    oh, ow = C.c_int32(), C.c_int32()
    capi.check(capi.lib().flhip_conv2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)))
    if tuple(g.shape) != (d.N, d.K, oh.value, ow.value):
        raise ValueError("conv2dBackwardFilterBias: gradOutput shape does not match the geometry")
    capi.check(capi.lib().flhip_conv2d_bwd_filter_static(C.byref(d), _ptr(x), _ptr(g), _ptr(dw),
                                                         _ptr(db), _stream()))
    return dw, db


def _pool_desc(x_shape4, wx, wy, sx, sy, px, py, mode, tag):
    N, Cc, H, W = x_shape4
    return capi.PoolDesc(N, Cc, H, W, wy, wx, sy, sx, py, px, int(mode), tag)


def pool2d(input, wx, wy, sx, sy, px, py, mode=PoolingMode.MAX, train=True):
    """AutogradExtension::pool2d -> (output, argmax).  argmax (uint8, one
    window-relative index per output) is returned for MAX when train is set —
    the reference keeps the equivalent oneDNN workspace in its payload only when
    a payload exists (onednn/Pool2D.cpp:88-92,150-161)."""
    x = _dev(input, "input")
    s4 = _as4(x)
    d = _pool_desc(s4, wx, wy, sx, sy, px, py, mode, _dtype_tag(x))
    oh, ow = C.c_int32(), C.c_int32()
    capi.check(capi.lib().flhip_pool2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)))
    oshape = (s4[0], s4[1], oh.value, ow.value)
    y = torch.empty(oshape, dtype=x.dtype, device=x.device)
    am = None
    if train and int(mode) == PoolingMode.MAX:
        am = torch.empty(oshape, dtype=torch.uint8, device=x.device)
    capi.check(capi.lib().flhip_pool2d_fwd(C.byref(d), _ptr(x), _ptr(y), _ptr(am), _stream()))
    return y, am


def pool2d_backward(grad_output, input_shape, argmax, wx, wy, sx, sy, px, py,
                    mode=PoolingMode.MAX):
    """AutogradExtension::pool2dBackward.  The result has the type of
    gradOutput."""
    g = _dev(grad_output, "gradOutput")
    s4 = (1,) * (4 - len(input_shape)) + tuple(input_shape)
    d = _pool_desc(s4, wx, wy, sx, sy, px, py, mode, _dtype_tag(g))
    if int(mode) == PoolingMode.MAX and argmax is None:
        raise ValueError("pool2dBackward: max pooling needs the forward payload")
    am = _dev(argmax, "argmax") if argmax is not None else None
    out = torch.empty(s4, dtype=g.dtype, device=g.device)
    capi.check(capi.lib().flhip_pool2d_bwd(C.byref(d), _ptr(g), _ptr(am), _ptr(out), _stream()))
    return out


def bn_view(shape_nchw, axes):
    """(outer, C, inner) from Flashlight feature axes; the rule of
    onednn/BatchNorm.cpp:40-71 and the contiguity check of :124-130."""
    whcn = list(shape_nchw)[::-1]
    axes = sorted(int(a) for a in axes)
    if not axes or axes != list(range(axes[0], axes[-1] + 1)) or axes[-1] >= len(whcn):
        raise ValueError("axis array should be continuous")
    nfeat = 1
    for a in axes:
        nfeat *= whcn[a]
    total = 1
    for s in whcn:
        total *= s
    if axes[0] == 0:
        return total // nfeat, nfeat, 1
    outer = 1
    for s in whcn[axes[-1] + 1:]:
        outer *= s
    return outer, nfeat, total // (nfeat * outer)


def _f32vec(t, n, name):
    if t is None or t.numel() == 0:
        return None
    if t.numel() != n:
        raise ValueError("batchnorm: %s must have one element per feature" % name)
    t = _dev(t, name)
    return t if t.dtype == torch.float32 else t.float()


def batchnorm(input, weight, bias, running_mean, running_var, axes, train, momentum, epsilon):
    """AutogradExtension::batchnorm -> (output, saveMean, saveInvStd).

    Train mode: batch statistics; running_mean/running_var (fp32, updated in
    place) follow the rule documented at flhip_bn_fwd_train.  Inference: uses the
    running statistics and returns (output, None, None)."""
    x = _dev(input, "input")
    outer, Cc, inner = bn_view(x.shape, axes)
    d = capi.BnDesc(outer, Cc, inner, _dtype_tag(x))
    g, b = _f32vec(weight, Cc, "weight"), _f32vec(bias, Cc, "bias")
    y = torch.empty_like(x)
    if not train:
        if running_mean is None or running_var is None:
            raise ValueError("batchnorm: inference needs running statistics")
        rm, rv = _f32vec(running_mean, Cc, "runningMean"), _f32vec(running_var, Cc, "runningVar")
        capi.check(capi.lib().flhip_bn_fwd_infer(C.byref(d), _ptr(x), _ptr(g), _ptr(b), _ptr(rm),
                                                 _ptr(rv), float(epsilon), _ptr(y), _stream()))
        return y, None, None
    for t, name in ((running_mean, "runningMean"), (running_var, "runningVar")):
        if t is not None and (t.dtype != torch.float32 or t.numel() != Cc):
            raise ValueError("batchnorm: %s must be fp32 with one element per feature" % name)
    sm = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    si = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    nws = capi.lib().flhip_bn_workspace_bytes(C.byref(d))
    ws = _ws(nws, x.device)
    capi.check(capi.lib().flhip_bn_fwd_train(
        C.byref(d), _ptr(x), _ptr(g), _ptr(b), _ptr(y), _ptr(sm), _ptr(si),
        _ptr(_dev(running_mean, "runningMean")), _ptr(_dev(running_var, "runningVar")),
        float(momentum), float(epsilon), _ptr(ws), nws, _stream()))
    return y, sm, si


def batchnorm_backward(grad_output, input, weight, save_mean, save_invstd, axes):
    """AutogradExtension::batchnormBackward -> (gradInput, gradWeight, gradBias)."""
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    if g.dtype != x.dtype or g.shape != x.shape:
        raise ValueError("batchnormBackward: gradOutput must match the input")
    if save_mean is None or save_invstd is None:
        raise ValueError("batchnormBackward: needs the forward payload")
    outer, Cc, inner = bn_view(x.shape, axes)
    d = capi.BnDesc(outer, Cc, inner, _dtype_tag(x))
    w = _f32vec(weight, Cc, "weight")
    dx = torch.empty_like(x)
    dg = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    db = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    nws = capi.lib().flhip_bn_workspace_bytes(C.byref(d))
    ws = _ws(nws, x.device)
    capi.check(capi.lib().flhip_bn_bwd(C.byref(d), _ptr(x), _ptr(g), _ptr(w), _ptr(save_mean),
                                       _ptr(save_invstd), _ptr(dx), _ptr(dg), _ptr(db), _ptr(ws),
                                       nws, _stream()))
    return dx, dg, db


def batchnorm_relu(input, weight, bias, running_mean, running_var, axes, momentum, epsilon,
                   residual=None, relu=True, want_mask=False):
    """flhip_bn_act_fwd_train: relu(batchnorm(input) + residual) in train mode, one pass over
    the tensor -> (output, saveMean, saveInvStd).  residual is optional.  want_mask: through
    flhip_bn_act_fwd_train_mask, with a fourth result, the ReLU's mask as bytes (one per 4
    elements) for batchnorm_relu_backward; rows must hold a multiple of 4 elements."""
    x = _dev(input, "input")
    outer, Cc, inner = bn_view(x.shape, axes)
    d = capi.BnDesc(outer, Cc, inner, _dtype_tag(x))
    g, b = _f32vec(weight, Cc, "weight"), _f32vec(bias, Cc, "bias")
    r = _dev(residual, "residual")
    if r is not None and (r.shape != x.shape or r.dtype != x.dtype):
        raise ValueError("batchnormRelu: the residual must match the input")
    y = torch.empty_like(x)
    sm = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    si = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    nws = capi.lib().flhip_bn_workspace_bytes(C.byref(d))
    ws = _ws(nws, x.device)
    rm, rv = _dev(running_mean, "runningMean"), _dev(running_var, "runningVar")
    if want_mask:
        nmask = capi.lib().flhip_bn_act_mask_bytes(C.byref(d))
        if nmask == 0:
            raise ValueError("batchnormRelu: the mask form needs rows of a multiple of 4 elements")
        mask = torch.empty((nmask,), dtype=torch.uint8, device=x.device)
        capi.check(capi.lib().flhip_bn_act_fwd_train_mask(
            C.byref(d), _ptr(x), _ptr(g), _ptr(b), _ptr(r), int(bool(relu)), _ptr(y), _ptr(mask), _ptr(sm),
            _ptr(si), _ptr(rm), _ptr(rv), float(momentum), float(epsilon), _ptr(ws), nws, _stream()))
        return y, sm, si, mask
    capi.check(capi.lib().flhip_bn_act_fwd_train(
        C.byref(d), _ptr(x), _ptr(g), _ptr(b), _ptr(r), int(bool(relu)), _ptr(y), _ptr(sm), _ptr(si),
        _ptr(rm), _ptr(rv), float(momentum), float(epsilon), _ptr(ws), nws, _stream()))
    return y, sm, si


def batchnorm_relu_backward(grad_output, input, output, weight, save_mean, save_invstd, axes,
                            want_residual_grad=False, mask=None):
    """flhip_bn_act_bwd -> (gradInput, gradWeight, gradBias, gradResidual or None): the
    gradient passes the ReLU mask of `output` (the forward result), then batchnormBackward.
    With `mask` (the fourth result of batchnorm_relu(want_mask=True)) the call goes through
    flhip_bn_act_bwd_mask and `output` is not read (it may be None)."""
    g, x, y = _dev(grad_output, "gradOutput"), _dev(input, "input"), _dev(output, "output")
    if g.dtype != x.dtype or g.shape != x.shape:
        raise ValueError("batchnormReluBackward: gradOutput must match the input")
    if mask is None and (y is None or y.dtype != x.dtype or y.shape != x.shape):
        raise ValueError("batchnormReluBackward: output must match the input")
    outer, Cc, inner = bn_view(x.shape, axes)
    d = capi.BnDesc(outer, Cc, inner, _dtype_tag(x))
    w = _f32vec(weight, Cc, "weight")
    dx = torch.empty_like(x)
    dr = torch.empty_like(x) if want_residual_grad else None
    dg = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    db = torch.empty((Cc,), dtype=torch.float32, device=x.device)
    nws = capi.lib().flhip_bn_workspace_bytes(C.byref(d))
    ws = _ws(nws, x.device)
    if mask is not None:
        m = _dev(mask, "mask")
        if m.dtype != torch.uint8 or m.numel() != capi.lib().flhip_bn_act_mask_bytes(C.byref(d)) or m.numel() == 0:
            raise ValueError("batchnormReluBackward: the mask must be the byte tensor of the forward call")
        capi.check(capi.lib().flhip_bn_act_bwd_mask(C.byref(d), _ptr(x), _ptr(g), _ptr(m), _ptr(w), _ptr(save_mean),
                                                    _ptr(save_invstd), _ptr(dx), _ptr(dr), _ptr(dg), _ptr(db),
                                                    _ptr(ws), nws, _stream()))
        return dx, dg, db, dr
    capi.check(capi.lib().flhip_bn_act_bwd(C.byref(d), _ptr(x), _ptr(g), _ptr(y), _ptr(w), _ptr(save_mean),
                                           _ptr(save_invstd), _ptr(dx), _ptr(dr), _ptr(dg), _ptr(db),
                                           _ptr(ws), nws, _stream()))
    return dx, dg, db, dr


# ---- operations of the caller closures (flashlight/fl/autograd/Functions.cpp) -------
# Shapes follow the rule of the rest of this module: a torch tensor's shape is the
# Flashlight shape reversed (same memory).  A Flashlight [features, batch] matrix is a
# torch [batch, features] tensor.

def astype(input, dtype):
    """Tensor::astype between fp32 and bf16 (round to nearest even)."""
    x = _dev(input, "input")
    out = torch.empty_like(x, dtype=dtype)
    capi.check(capi.lib().flhip_convert(_ptr(x), _dtype_tag(x), _ptr(out), _dtype_tag(out), x.numel(), _stream()))
    return out


def astype_many(inputs, dtype):
    """The same conversion of a list of tensors of one type, in one launch per 64 of them."""
    xs = [_dev(t, "input") for t in inputs]
    if not xs:
        return []
    if any(x.dtype != xs[0].dtype for x in xs):
        raise ValueError("astype_many: the tensors must share a type")
    outs = [torch.empty_like(x, dtype=dtype) for x in xs]
    n = len(xs)
    src = (C.c_void_p * n)(*[x.data_ptr() for x in xs])
    dst = (C.c_void_p * n)(*[o.data_ptr() for o in outs])
    cnt = (C.c_size_t * n)(*[x.numel() for x in xs])
    capi.check(capi.lib().flhip_convert_many(src, dst, cnt, n, _dtype_tag(xs[0]), _dtype_tag(outs[0]), _stream()))
    return outs


def relu(input):
    """fl::relu (Functions.cpp:1787-1789)."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    capi.check(capi.lib().flhip_relu_fwd(_ptr(x), _ptr(y), x.numel(), _dtype_tag(x), _stream()))
    return y


def relu_backward(grad_output, input):
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    if g.shape != x.shape or g.dtype != x.dtype:
        raise ValueError("relu backward: gradOutput must match the input")
    dx = torch.empty_like(x)
    capi.check(capi.lib().flhip_relu_bwd(_ptr(g), _ptr(x), _ptr(dx), x.numel(), _dtype_tag(x),
                                         _stream()))
    return dx


ACT_ELU, ACT_CLAMP, ACT_TANH, ACT_LOG, ACT_SWISH, ACT_SIGMOID, ACT_SCALE, ACT_LEAKY, ACT_THRESHOLD = range(9)


def activation(op, input, a=0.0, b=0.0):
    """flhip_act_fwd: the element-wise activations of nn/modules/Activations.cpp (ELU(a), clamp(a, b) = ReLU6 /
    HardTanh, tanh, log, swish(a), sigmoid)."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    capi.check(capi.lib().flhip_act_fwd(int(op), _ptr(x), _ptr(y), x.numel(), float(a), float(b), _dtype_tag(x),
                                        _stream()))
    return y


def activation_backward(op, grad_output, input, a=0.0, b=0.0):
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    if g.shape != x.shape or g.dtype != x.dtype:
        raise ValueError("activation backward: gradOutput must match the input")
    dx = torch.empty_like(x)
    capi.check(capi.lib().flhip_act_bwd(int(op), _ptr(g), _ptr(x), _ptr(dx), x.numel(), float(a), float(b),
                                        _dtype_tag(x), _stream()))
    return dx


def _glu_view(shape, dim):
    """(outer, m) of fl::gatedlinearunit along torch dimension `dim` of a contiguous tensor."""
    if shape[dim] % 2:
        raise ValueError("halving dimension must be even for GLU")
    outer = 1
    for v in shape[:dim]:
        outer *= v
    m = shape[dim] // 2
    for v in shape[dim + 1:]:
        m *= v
    return outer, m


def gated_linear_unit(input, dim):
    """fl::gatedlinearunit (Functions.cpp:1567-1610) along torch dimension `dim`."""
    x = _dev(input, "input")
    outer, m = _glu_view(tuple(x.shape), dim)
    shape = list(x.shape)
    shape[dim] //= 2
    y = torch.empty(shape, dtype=x.dtype, device=x.device)
    capi.check(capi.lib().flhip_glu_fwd(_ptr(x), _ptr(y), outer, m, _dtype_tag(x), _stream()))
    return y


def gated_linear_unit_backward(grad_output, input, dim):
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    outer, m = _glu_view(tuple(x.shape), dim)
    if g.numel() * 2 != x.numel() or g.dtype != x.dtype:
        raise ValueError("GLU backward: gradOutput must have half the input's elements")
    dx = torch.empty_like(x)
    capi.check(capi.lib().flhip_glu_bwd(_ptr(g), _ptr(x), _ptr(dx), outer, m, _dtype_tag(x), _stream()))
    return dx


def dropout(input, p, seed):
    """fl::dropout (Functions.cpp:1777-1785) with the counter-based mask of (seed, element index); the backward pass
    is the same call on the gradient."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    capi.check(capi.lib().flhip_dropout(_ptr(x), _ptr(y), x.numel(), float(p), int(seed) & 0xffffffff,
                                        (int(seed) >> 32) & 0xffffffff, _dtype_tag(x), _stream()))
    return y


def rownorm(v, rows, cols, rows_fast):
    """flhip_rownorm: ||v_r|| of a rows x cols view (rows_fast: element (r, j) at r + j * rows)."""
    x = _dev(v, "v")
    n = torch.empty(rows, dtype=x.dtype, device=x.device)
    capi.check(capi.lib().flhip_rownorm(_ptr(x), _ptr(n), rows, cols, int(rows_fast), _dtype_tag(x), _stream()))
    return n


def weightnorm(v, g, rows, cols, rows_fast):
    """fl::WeightNorm's weight (WeightNorm.cpp:45-66): v * g[r] / ||v_r||."""
    x, gg = _dev(v, "v"), _dev(g, "g")
    w = torch.empty_like(x)
    capi.check(capi.lib().flhip_weightnorm_fwd(_ptr(x), _ptr(gg), _ptr(w), rows, cols, int(rows_fast), _dtype_tag(x),
                                               _stream()))
    return w


def weightnorm_backward(dw, v, g, rows, cols, rows_fast):
    d, x, gg = _dev(dw, "dw"), _dev(v, "v"), _dev(g, "g")
    dv, dg = torch.empty_like(x), torch.empty_like(gg)
    capi.check(capi.lib().flhip_weightnorm_bwd(_ptr(d), _ptr(x), _ptr(gg), _ptr(dv), _ptr(dg), rows, cols,
                                               int(rows_fast), _dtype_tag(x), _stream()))
    return dv, dg


def _pad_args(dims, before, after):
    return ((C.c_int64 * 4)(*dims), (C.c_int32 * 4)(*before), (C.c_int32 * 4)(*after))


def padding(input, dims, before, after, value=0.0):
    """fl::padding (Functions.cpp:1751-1775); dims / before / after: four column-major entries (dims[0] fastest) of a
    contiguous tensor with prod(dims) elements.  Returns a flat tensor in the padded shape's memory order."""
    x = _dev(input, "input")
    d, b, a = _pad_args(dims, before, after)
    n = 1
    for k in range(4):
        n *= dims[k] + before[k] + after[k]
    y = torch.empty(n, dtype=x.dtype, device=x.device)
    capi.check(capi.lib().flhip_pad_fwd(_ptr(x), _ptr(y), d, b, a, float(value), _dtype_tag(x), _stream()))
    return y


def padding_backward(grad_output, dims, before, after):
    g = _dev(grad_output, "gradOutput")
    d, b, a = _pad_args(dims, before, after)
    n = 1
    for k in range(4):
        n *= dims[k]
    dx = torch.empty(n, dtype=g.dtype, device=g.device)
    capi.check(capi.lib().flhip_pad_bwd(_ptr(g), _ptr(dx), d, b, a, _dtype_tag(g), _stream()))
    return dx


def sgd_step(params, grads, velocities, lr, momentum=0.0, weight_decay=0.0, nesterov=False):
    """fl::SGDOptimizer::step (optim/SGDOptimizer.cpp:38-68) over lists of tensors of one dtype, in place."""
    ps = [_dev(p, "param") for p in params]
    gs = [_dev(g, "grad") for g in grads]
    vs = [_dev(v, "velocity") for v in velocities] if velocities is not None else None
    n = len(ps)
    if n == 0:
        return
    pa = (C.c_void_p * n)(*[p.data_ptr() for p in ps])
    ga = (C.c_void_p * n)(*[g.data_ptr() for g in gs])
    va = (C.c_void_p * n)(*[v.data_ptr() for v in vs]) if vs is not None else None
    cnt = (C.c_size_t * n)(*[p.numel() for p in ps])
    capi.check(capi.lib().flhip_sgd_many(pa, ga, va, cnt, n, float(lr), float(momentum), float(weight_decay),
                                         int(bool(nesterov)), _dtype_tag(ps[0]), _stream()))


def adam_step(params, grads, first, second, lr, beta1, beta2, epsilon, weight_decay, step):
    """fl::AdamOptimizer::step (optim/AdamOptimizer.cpp:45-79) over lists of tensors of one dtype, in place."""
    lists = [[_dev(t, "tensor") for t in l] for l in (params, grads, first, second)]
    n = len(lists[0])
    if n == 0:
        return
    arrs = [(C.c_void_p * n)(*[t.data_ptr() for t in l]) for l in lists]
    cnt = (C.c_size_t * n)(*[t.numel() for t in lists[0]])
    capi.check(capi.lib().flhip_adam_many(arrs[0], arrs[1], arrs[2], arrs[3], cnt, n, float(lr), float(beta1), float(beta2),
                                          float(epsilon), float(weight_decay), int(step), _dtype_tag(lists[0][0]), _stream()))


def linear(input, weight, bias=None):
    """fl::linear (Functions.cpp:1255-1309): input [..., in] (Flashlight [in, ...]), weight
    torch [in, out] (Flashlight [out, in]), bias [out] or None -> [..., out]."""
    x, w = _dev(input, "input"), _dev(weight, "weight")
    if w.dim() != 2 or x.shape[-1] != w.shape[0] or x.dtype != w.dtype:
        raise ValueError("linear: input [.., in] and weight [in, out] of one type expected")
    fin, fout = w.shape
    frames = x.numel() // fin
    b = None
    if bias is not None and bias.numel() > 0:
        if bias.numel() != fout:
            raise ValueError("linear: bias must have one element per output feature")
        b = _dev(bias, "bias").float().contiguous()
    y = torch.empty(tuple(x.shape[:-1]) + (fout,), dtype=x.dtype, device=x.device)
    capi.check(capi.lib().flhip_matmul(_ptr(w), _ptr(x), _ptr(y), fout, frames, fin, 0, 0, _ptr(b),
                                       _dtype_tag(x), _stream()))
    return y


def linear_backward(grad_output, input, weight, want_bias=True):
    """-> (gradInput, gradWeight, gradBias or None), the three branches of the gradient
    closure of fl::linear (Functions.cpp:1276-1303)."""
    g, x, w = _dev(grad_output, "gradOutput"), _dev(input, "input"), _dev(weight, "weight")
    fin, fout = w.shape
    frames = x.numel() // fin
    tag = _dtype_tag(x)
    dx = torch.empty_like(x)
    capi.check(capi.lib().flhip_matmul(_ptr(w), _ptr(g), _ptr(dx), fin, frames, fout, 1, 0, None, tag,
                                       _stream()))
    dw = torch.empty_like(w)
    nws = capi.lib().flhip_matmul_workspace_bytes(fout, fin, frames, 0, 1, tag)
    ws = torch.empty((nws,), dtype=torch.uint8, device=x.device) if nws else None
    capi.check(capi.lib().flhip_matmul_ws(_ptr(g), _ptr(x), _ptr(dw), fout, fin, frames, 0, 1, None, tag,
                                          _ptr(ws) if nws else None, nws, _stream()))
    db = None
    if want_bias:
        db = torch.empty((fout,), dtype=torch.float32, device=x.device)
        nws = capi.lib().flhip_sum_columns_workspace_bytes(fout, frames, tag)
        ws = torch.empty((nws,), dtype=torch.uint8, device=x.device) if nws else None
        capi.check(capi.lib().flhip_sum_columns_ws(_ptr(g), _ptr(db), fout, frames, tag, _ptr(ws) if nws else None,
                                                   nws, _stream()))
    return dx, dw, db


def log_softmax(input):
    """fl::logSoftmax over Flashlight dimension 0 (Functions.cpp:1044-1070): torch [..., classes]."""
    x = _dev(input, "input")
    y = torch.empty_like(x)
    classes = x.shape[-1]
    capi.check(capi.lib().flhip_logsoftmax_fwd(_ptr(x), _ptr(y), classes, x.numel() // classes,
                                               _dtype_tag(x), _stream()))
    return y


def log_softmax_backward(grad_output, output):
    g, y = _dev(grad_output, "gradOutput"), _dev(output, "output")
    dx = torch.empty_like(y)
    classes = y.shape[-1]
    capi.check(capi.lib().flhip_logsoftmax_bwd(_ptr(g), _ptr(y), _ptr(dx), classes,
                                               y.numel() // classes, _dtype_tag(y), _stream()))
    return dx


REDUCE_NONE, REDUCE_MEAN, REDUCE_SUM = 0, 1, 2


def categorical_cross_entropy(input, targets, reduction=REDUCE_MEAN, ignore_index=-1):
    """fl::categoricalCrossEntropy (Functions.cpp:1078-1154) on log-probabilities
    [..., classes] and int32 targets [...] -> (loss, stats); stats feeds the backward.
    Raises ValueError for targets outside [0, classes), as the reference throws."""
    x, t = _dev(input, "input"), _dev(targets, "targets")
    if t.dtype != torch.int32 or tuple(t.shape) != tuple(x.shape[:-1]):
        raise ValueError("categoricalCrossEntropy: int32 targets with one dimension fewer expected")
    classes = x.shape[-1]
    cols = t.numel()
    stats = torch.empty((4,), dtype=torch.float32, device=x.device)
    per = torch.empty((cols,), dtype=torch.float32, device=x.device) if reduction == REDUCE_NONE else None
    capi.check(capi.lib().flhip_cce_fwd(_ptr(x), _ptr(t), _ptr(stats), _ptr(per), classes, cols,
                                        ignore_index, _dtype_tag(x), _stream()))
    if float(stats[2].item()) != 0.0:
        raise ValueError("target contains elements out of valid range [0, num_categories) "
                         "in categorical cross entropy")
    if reduction == REDUCE_NONE:
        return per.reshape(t.shape), stats
    return (stats[3:4] if reduction == REDUCE_MEAN else stats[0:1]), stats


def categorical_cross_entropy_backward(grad_output, input_shape, dtype, targets, stats,
                                       reduction=REDUCE_MEAN, ignore_index=-1):
    g, t = _dev(grad_output, "gradOutput").float().contiguous(), _dev(targets, "targets")
    dx = torch.empty(tuple(input_shape), dtype=dtype, device=t.device)
    classes = input_shape[-1]
    tag = _TAG_OF[dtype]
    capi.check(capi.lib().flhip_cce_bwd(_ptr(g), _ptr(t), _ptr(stats), _ptr(dx), classes, t.numel(),
                                        reduction, ignore_index, tag, _stream()))
    return dx


# ---- LayerNorm = batchnorm over the complement axes + broadcast scale and shift -------
def _affine_view(whcn, norm_axes, nparam):
    """(outer, mid, inner, scalar) of the parameter broadcast of LayerNorm.cpp:110-126:
    one element, or one per position along the (contiguous) normalised axes."""
    if nparam == 1:
        return 1, 1, 1, True
    axes = sorted(norm_axes)
    if axes != list(range(axes[0], axes[-1] + 1)):
        raise ValueError("LayerNorm: per-element parameters need contiguous normalised axes")
    mid = inner = outer = 1
    for d, s in enumerate(whcn):
        if d < axes[0]:
            inner *= s
        elif d <= axes[-1]:
            mid *= s
        else:
            outer *= s
    if mid != nparam:
        raise ValueError("[LayerNorm] Input size along the norm axis doesn't with axisSize.")
    return outer, mid, inner, False


def affine(input, weight, bias, view):
    """y = tileAs(weight) * input + tileAs(bias) on the [outer][mid][inner] view."""
    x = _dev(input, "input")
    outer, mid, inner, scalar = view
    if scalar:
        outer, mid, inner = 1, 1, x.numel()
    w, b = _dev(weight, "weight").to(x.dtype), _dev(bias, "bias").to(x.dtype)
    y = torch.empty_like(x)
    capi.check(capi.lib().flhip_affine_fwd(_ptr(x), _ptr(w), _ptr(b), _ptr(y), outer, mid, inner,
                                           int(scalar), _dtype_tag(x), _stream()))
    return y


def affine_backward(grad_output, input, weight, view):
    """-> (gradInput, gradWeight fp32, gradBias fp32) of `affine`."""
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    outer, mid, inner, scalar = view
    if scalar:
        outer, mid, inner = 1, 1, x.numel()
    w = _dev(weight, "weight").to(x.dtype)
    n = 1 if scalar else mid
    dx = torch.empty_like(x)
    dw = torch.empty((n,), dtype=torch.float32, device=x.device)
    db = torch.empty((n,), dtype=torch.float32, device=x.device)
    nws = capi.lib().flhip_affine_bwd_workspace_bytes(outer, mid, inner, int(scalar))
    ws = _ws(nws, x.device)
    capi.check(capi.lib().flhip_affine_bwd(_ptr(g), _ptr(x), _ptr(w), _ptr(dx), _ptr(dw), _ptr(db),
                                           outer, mid, inner, int(scalar), _dtype_tag(x), _ptr(ws),
                                           nws, _stream()))
    return dx, dw, db


def embedding(indices, table):
    """fl::embedding: `indices` int32 (any shape), `table` [tokens, dim] -> indices.shape + [dim]."""
    idx, w = _dev(indices, "indices"), _dev(table, "table")
    if idx.dtype != torch.int32:
        raise ValueError("embedding: indices must be int32")
    tokens, dim = w.shape
    y = torch.empty(tuple(idx.shape) + (dim,), dtype=w.dtype, device=w.device)
    capi.check(capi.lib().flhip_embedding_fwd(_ptr(idx), _ptr(w), _ptr(y), idx.numel(), dim, tokens, _dtype_tag(w),
                                              _stream()))
    return y


def embedding_backward(grad_output, indices, tokens):
    """-> the gradient of the table, [tokens, dim]."""
    g, idx = _dev(grad_output, "gradOutput"), _dev(indices, "indices")
    dim = g.shape[-1]
    dw = torch.empty((tokens, dim), dtype=g.dtype, device=g.device)
    capi.check(capi.lib().flhip_embedding_bwd(_ptr(idx), _ptr(g), _ptr(dw), idx.numel(), dim, tokens, _dtype_tag(g),
                                              _stream()))
    return dw


def prelu(input, weight):
    """fl::PReLU: `weight` has one element, or as many as the input's fastest (last torch) dimension."""
    x = _dev(input, "input")
    w = _dev(weight, "weight").to(x.dtype).contiguous()
    d0 = x.shape[-1]
    if w.numel() not in (1, d0):
        raise ValueError("prelu: the parameter has 1 element or one per index of the first dimension")
    y = torch.empty_like(x)
    capi.check(capi.lib().flhip_prelu_fwd(_ptr(x), _ptr(w), _ptr(y), x.numel() // d0, d0, int(w.numel() == 1),
                                          _dtype_tag(x), _stream()))
    return y


def prelu_backward(grad_output, input, weight):
    """-> (gradInput, gradWeight fp32) of `prelu`."""
    g, x = _dev(grad_output, "gradOutput"), _dev(input, "input")
    w = _dev(weight, "weight").to(x.dtype).contiguous()
    d0 = x.shape[-1]
    scalar = int(w.numel() == 1)
    dx = torch.empty_like(x)
    dw = torch.empty((w.numel(),), dtype=torch.float32, device=x.device)
    nws = capi.lib().flhip_prelu_bwd_workspace_bytes(x.numel() // d0, d0, scalar)
    ws = _ws(nws, x.device)
    capi.check(capi.lib().flhip_prelu_bwd(_ptr(g), _ptr(x), _ptr(w), _ptr(dx), _ptr(dw), x.numel() // d0, d0, scalar,
                                          _dtype_tag(x), _ptr(ws), nws, _stream()))
    return dx, dw


def reorder(input, perm_whcn):
    """fl::reorder on the Flashlight view of `input` (torch shape reversed, padded to four
    dimensions): Flashlight dimension k of the result is dimension perm_whcn[k] of the
    input.  -> a new contiguous tensor (torch shape = reversed result shape)."""
    x = _dev(input, "input")
    whcn = list(x.shape)[::-1]
    whcn += [1] * (4 - len(whcn))
    perm = [int(v) for v in perm_whcn]
    if sorted(perm) != [0, 1, 2, 3]:
        raise ValueError("reorder: not a permutation of the four dimensions")
    out = torch.empty([whcn[k] for k in perm][::-1], dtype=x.dtype, device=x.device)
    dims = (C.c_int64 * 4)(*whcn)
    pm = (C.c_int32 * 4)(*perm)
    capi.check(capi.lib().flhip_reorder(_ptr(x), _ptr(out), dims, pm, _dtype_tag(x), _stream()))
    return out


def _layer_norm_axes(shape, norm_axes):
    whcn = list(shape)[::-1]
    if len(whcn) > 4:
        raise ValueError("LayerNorm::forward - input must be 4 or fewer dimensions.")
    whcn += [1] * (4 - len(whcn))
    norm = sorted(int(a) for a in norm_axes)
    comp = [d for d in range(4) if d not in norm]
    if not comp:
        raise ValueError("LayerNorm: no axis left to batch over")
    contiguous = comp == list(range(comp[0], comp[-1] + 1))
    return whcn, norm, comp, contiguous


def layer_norm(input, norm_axes, epsilon=1e-5, weight=None, bias=None):
    """fl::LayerNorm::forward (nn/modules/LayerNorm.cpp:42-131): batchnorm in train mode
    over the complement of the normalised axes with no parameters and no running
    statistics, then the broadcast scale and shift.  When the complement axes are not
    contiguous the tensor is reordered first (normalised axes, then the complement) and
    the result reordered back, as the reference does; the scale and shift are then
    applied in the reordered layout, where the normalised axes are the leading ones.
    -> (output, ctx for the backward)."""
    x = _dev(input, "input")
    whcn, norm, comp, contiguous = _layer_norm_axes(x.shape, norm_axes)
    if weight is not None and weight.numel() > 1 and norm != list(range(norm[0], norm[-1] + 1)):
        contiguous = False       # the broadcast of per-element parameters needs leading normalised axes too
    x4 = x.reshape(whcn[::-1])
    ctx = {"view": None, "perm": None, "shape": tuple(x.shape)}
    if contiguous:
        bn_axes, w4 = comp, whcn
    else:
        ctx["perm"] = norm + comp
        x4 = reorder(x4, ctx["perm"])
        w4 = [whcn[k] for k in ctx["perm"]]
        bn_axes = list(range(len(norm), 4))
        norm = list(range(len(norm)))
    xhat, sm, si = batchnorm(x4, None, None, None, None, bn_axes, True, 0.0, epsilon)
    ctx.update({"x4": x4, "xhat": xhat, "sm": sm, "si": si, "comp": bn_axes})
    out = xhat
    if weight is not None:
        ctx["view"] = _affine_view(w4, norm, weight.numel())
        out = affine(xhat, weight, bias, ctx["view"])
    if ctx["perm"] is not None:
        inv = [ctx["perm"].index(k) for k in range(4)]
        out = reorder(out, inv)
    return out.reshape(x.shape), ctx


def layer_norm_backward(grad_output, ctx, weight=None):
    """-> (gradInput, gradWeight, gradBias) of `layer_norm` (the last two None without
    parameters)."""
    g = _dev(grad_output, "gradOutput")
    if ctx["perm"] is not None:
        whcn = list(g.shape)[::-1]
        whcn += [1] * (4 - len(whcn))
        g = reorder(g.reshape(whcn[::-1]), ctx["perm"])
    g = g.reshape(ctx["x4"].shape)
    dw = db = None
    if ctx["view"] is not None:
        g, dw, db = affine_backward(g, ctx["xhat"], weight, ctx["view"])
    dx, _, _ = batchnorm_backward(g, ctx["x4"], None, ctx["sm"], ctx["si"], ctx["comp"])
    if ctx["perm"] is not None:
        dx = reorder(dx, [ctx["perm"].index(k) for k in range(4)])
    return dx.reshape(grad_output.shape), dw, db


# ---- rnn / rnnBackward -----------------------------------------------------------------
RNN_RELU, RNN_TANH, RNN_LSTM, RNN_GRU = 0, 1, 2, 3


def _rnn_desc(x, hidden_size, num_layers, mode, bidirectional, dropout=0.0, seed=0):
    if x.dim() != 3 or x.dtype != torch.float32:
        raise ValueError("rnn: input must be fp32 [seq, batch, input] (Flashlight [input, batch, seq])")
    if not 0.0 <= dropout < 1.0:
        raise ValueError("rnn: dropout must be in [0, 1)")
    T, B, I = x.shape
    # dropout acts between layers only (backend/cudnn/RNN.cpp:83-90)
    return capi.RnnDesc(I, hidden_size, num_layers, int(bool(bidirectional)), int(mode), T, B, capi.F32,
                        float(dropout) if num_layers > 1 else 0.0, seed & 0xffffffff, (seed >> 32) & 0xffffffff)


def rnn_param_count(input_size, hidden_size, num_layers, mode, bidirectional):
    d = capi.RnnDesc(input_size, hidden_size, num_layers, int(bool(bidirectional)), int(mode), 1, 1, capi.F32)
    return capi.lib().flhip_rnn_param_count(C.byref(d))


def rnn(input, hidden_state, cell_state, weights, hidden_size, num_layers, mode, bidirectional,
        dropout=0.0, seed=0):
    """AutogradExtension::rnn -> (output, hiddenOut, cellOut or None, reserve).  Tensors are
    torch views of the Flashlight ones (shape reversed): input [seq, batch, input], states
    [layers*dirs, batch, hidden], output [seq, batch, dirs*hidden]; weights flat in cuDNN's
    order.  reserve goes to rnn_backward (the payload of the reference's closure), together
    with the same dropout and seed (the mask between layers is a function of the seed)."""
    x, w = _dev(input, "input"), _dev(weights, "weights")
    d = _rnn_desc(x, hidden_size, num_layers, mode, bidirectional, dropout, seed)
    L = capi.lib()
    if w.numel() != L.flhip_rnn_param_count(C.byref(d)):
        raise ValueError("invalid # of parameters or wrong input shape for RNN")
    D = 2 if bidirectional else 1
    sshape = (num_layers * D, d.batch, hidden_size)
    for t, name in ((hidden_state, "hidden"), (cell_state, "cell")):
        if t is not None and t.numel() and tuple(t.shape) != sshape:
            raise ValueError("invalid %s state dims for RNN" % name)
    if cell_state is not None and cell_state.numel() and mode != RNN_LSTM:
        raise ValueError("invalid cell state dims for RNN")
    hx = _dev(hidden_state, "hiddenState") if hidden_state is not None and hidden_state.numel() else None
    cx = _dev(cell_state, "cellState") if cell_state is not None and cell_state.numel() else None
    y = torch.empty((d.seq_len, d.batch, D * hidden_size), dtype=torch.float32, device=x.device)
    hy = torch.empty(sshape, dtype=torch.float32, device=x.device)
    cy = torch.empty(sshape, dtype=torch.float32, device=x.device) if mode == RNN_LSTM else None
    nres, nws = L.flhip_rnn_reserve_bytes(C.byref(d)), L.flhip_rnn_workspace_bytes(C.byref(d))
    reserve, ws = _ws(nres, x.device), _ws(nws, x.device)
    capi.check(L.flhip_rnn_fwd(C.byref(d), _ptr(x), _ptr(hx), _ptr(cx), _ptr(w), _ptr(y), _ptr(hy), _ptr(cy),
                               _ptr(reserve), nres, _ptr(ws), nws, _stream()))
    return y, hy, cy, reserve


def rnn_backward(input, weights, reserve, hidden_size, num_layers, mode, bidirectional,
                 grad_output=None, grad_hidden=None, grad_cell=None, dropout=0.0, seed=0):
    """AutogradExtension::rnnBackward -> (gradInput, gradHidden, gradCell or None, gradWeights);
    missing output gradients count as zero (Functions.cpp:1677-1699)."""
    x, w = _dev(input, "input"), _dev(weights, "weights")
    d = _rnn_desc(x, hidden_size, num_layers, mode, bidirectional, dropout, seed)
    L = capi.lib()
    D = 2 if bidirectional else 1
    sshape = (num_layers * D, d.batch, hidden_size)
    dx = torch.empty_like(x)
    dhx = torch.empty(sshape, dtype=torch.float32, device=x.device)
    dcx = torch.empty(sshape, dtype=torch.float32, device=x.device) if mode == RNN_LSTM else None
    dw = torch.empty_like(w)
    nres, nws = L.flhip_rnn_reserve_bytes(C.byref(d)), L.flhip_rnn_workspace_bytes(C.byref(d))
    if reserve is None or reserve.numel() < nres:
        raise ValueError("rnnBackward: needs the reserve buffer of the forward pass")
    ws = _ws(nws, x.device)
    opt = lambda t, n: _ptr(_dev(t, n)) if t is not None and t.numel() else None
    capi.check(L.flhip_rnn_bwd(C.byref(d), _ptr(x), _ptr(w), opt(grad_output, "gradOutput"),
                               opt(grad_hidden, "gradHidden"), opt(grad_cell, "gradCell"), _ptr(reserve), nres,
                               _ptr(dx), _ptr(dhx), _ptr(dcx), _ptr(dw), _ptr(ws), nws, _stream()))
    return dx, dhx, dcx, dw
