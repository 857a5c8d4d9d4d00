"""ctypes declarations of include/flhip.h."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libflhip.so")

OK, INVALID_ARGUMENT, RUNTIME_ERROR, DECLINED = 0, 1, 2, 3
F32, BF16, F16 = 0, 1, 2
CONV_FWD, CONV_BWD_DATA, CONV_BWD_FILTER = 0, 1, 2
STATIC_SCRATCH_BYTES = 40 << 20      # FLHIP_STATIC_SCRATCH_BYTES


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "C", "H", "W", "K", "KH", "KW", "sy", "sx", "py", "px",
        "dil_y", "dil_x", "groups", "dtype")]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "N", "C", "H", "W", "wy", "wx", "sy", "sx", "py", "px", "mode", "dtype")]


class BnDesc(C.Structure):
    _fields_ = [("outer", C.c_int64), ("C", C.c_int64), ("inner", C.c_int64),
                ("dtype", C.c_int32)]


class RnnDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("input_size", "hidden_size", "num_layers", "bidirectional", "mode",
                                         "seq_len", "batch", "dtype")] + [
        ("dropout", C.c_float), ("seed_lo", C.c_uint32), ("seed_hi", C.c_uint32)]


# every symbol include/flhip.h declares: name -> (restype, argtypes)
_VP, _SZ, _I32P = C.c_void_p, C.c_size_t, C.POINTER(C.c_int32)
SYMBOLS = {
    "flhip_last_error": (C.c_char_p, []),
    "flhip_version": (C.c_int, []),
    "flhip_conv2d_plan_count": (C.c_int, [C.c_int]),
    "flhip_conv2d_plan_name": (C.c_char_p, [C.c_int, C.c_int]),
    "flhip_conv2d_bwd_data_plan": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _SZ, C.c_int, _VP]),
    "flhip_conv2d_bwd_filter_plan": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _VP, _SZ, C.c_int, _VP]),
    "flhip_convert_many_launches": (C.c_int, [C.POINTER(C.c_size_t), C.c_int, _I32P]),
    "flhip_arch": (C.c_char_p, []),
    "flhip_set_option": (C.c_int, [C.c_char_p, C.c_char_p]),
    "flhip_conv2d_out_dims": (C.c_int, [C.POINTER(ConvDesc), _I32P, _I32P]),
    "flhip_pool2d_out_dims": (C.c_int, [C.POINTER(PoolDesc), _I32P, _I32P]),
    "flhip_conv2d_workspace_bytes": (_SZ, [C.POINTER(ConvDesc), C.c_int]),
    "flhip_conv2d_fwd": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "flhip_conv2d_bwd_data": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _SZ, _VP]),
    "flhip_conv2d_bwd_data_add": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "flhip_conv2d_bwd_filter": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "flhip_conv2d_bwd_filter_static": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _VP]),
    "flhip_conv2d_gathered_bytes": (_SZ, [C.POINTER(ConvDesc)]),
    "flhip_conv2d_bwd_filter_gathered": (C.c_int, [C.POINTER(ConvDesc), _VP, _VP, _VP, _VP, _VP, _SZ, _VP]),
    "flhip_pool2d_fwd": (C.c_int, [C.POINTER(PoolDesc), _VP, _VP, _VP, _VP]),
    "flhip_pool2d_bwd": (C.c_int, [C.POINTER(PoolDesc), _VP, _VP, _VP, _VP]),
    "flhip_bn_workspace_bytes": (_SZ, [C.POINTER(BnDesc)]),
    "flhip_bn_fwd_train": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                      C.c_double, C.c_double, _VP, _SZ, _VP]),
    "flhip_bn_fwd_infer": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, _VP, C.c_double,
                                      _VP, _VP]),
    "flhip_bn_bwd": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                _SZ, _VP]),
    "flhip_bn_act_fwd_train": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, C.c_int, _VP, _VP, _VP, _VP, _VP,
                                          C.c_double, C.c_double, _VP, _SZ, _VP]),
    "flhip_bn_act_bwd": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                    _SZ, _VP]),
    "flhip_bn_act_mask_bytes": (_SZ, [C.POINTER(BnDesc)]),
    "flhip_bn_act_fwd_train_mask": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, C.c_int, _VP, _VP, _VP, _VP, _VP,
                                               _VP, C.c_double, C.c_double, _VP, _SZ, _VP]),
    "flhip_bn_act_bwd_mask": (C.c_int, [C.POINTER(BnDesc), _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP,
                                         _SZ, _VP]),
    "flhip_copy_bytes": (C.c_int, [_VP, _VP, _SZ, _VP]),
    "flhip_convert": (C.c_int, [_VP, C.c_int, _VP, C.c_int, _SZ, _VP]),
    "flhip_convert_many": (C.c_int, [C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_SZ), C.c_int, C.c_int, C.c_int, _VP]),
    "flhip_fill": (C.c_int, [_VP, C.c_double, _SZ, C.c_int, _VP]),
    "flhip_add": (C.c_int, [_VP, _VP, _VP, _SZ, C.c_int, _VP]),
    "flhip_relu_fwd": (C.c_int, [_VP, _VP, _SZ, C.c_int, _VP]),
    "flhip_relu_bwd": (C.c_int, [_VP, _VP, _VP, _SZ, C.c_int, _VP]),
    "flhip_act_fwd": (C.c_int, [C.c_int, _VP, _VP, _SZ, C.c_double, C.c_double, C.c_int, _VP]),
    "flhip_act_bwd": (C.c_int, [C.c_int, _VP, _VP, _VP, _SZ, C.c_double, C.c_double, C.c_int, _VP]),
    "flhip_glu_fwd": (C.c_int, [_VP, _VP, C.c_int64, C.c_int64, C.c_int, _VP]),
    "flhip_glu_bwd": (C.c_int, [_VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int, _VP]),
    "flhip_sgd_many": (C.c_int, [C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_SZ), C.c_int, C.c_double,
                                 C.c_double, C.c_double, C.c_int, C.c_int, _VP]),
    "flhip_adam_many": (C.c_int, [C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_VP), C.POINTER(_SZ), C.c_int,
                                  C.c_double, C.c_double, C.c_double, C.c_double, C.c_double, C.c_int64, C.c_int, _VP]),
    "flhip_dropout": (C.c_int, [_VP, _VP, _SZ, C.c_double, C.c_uint32, C.c_uint32, C.c_int, _VP]),
    "flhip_rownorm": (C.c_int, [_VP, _VP, C.c_int64, C.c_int64, C.c_int, C.c_int, _VP]),
    "flhip_weightnorm_fwd": (C.c_int, [_VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int, C.c_int, _VP]),
    "flhip_weightnorm_bwd": (C.c_int, [_VP, _VP, _VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int, C.c_int, _VP]),
    "flhip_pad_fwd": (C.c_int, [_VP, _VP, C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.c_double, C.c_int, _VP]),
    "flhip_pad_bwd": (C.c_int, [_VP, _VP, C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.c_int, _VP]),
    "flhip_matmul": (C.c_int, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int, C.c_int, _VP,
                               C.c_int, _VP]),
    "flhip_matmul_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int32, C.c_int, C.c_int, C.c_int]),
    "flhip_matmul_ws": (C.c_int, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int, C.c_int, _VP,
                                  C.c_int, _VP, C.c_size_t, _VP]),
    "flhip_sum_columns": (C.c_int, [_VP, _VP, C.c_int32, C.c_int32, C.c_int, _VP]),
    "flhip_sum_columns_workspace_bytes": (C.c_size_t, [C.c_int32, C.c_int32, C.c_int]),
    "flhip_sum_columns_ws": (C.c_int, [_VP, _VP, C.c_int32, C.c_int32, C.c_int, _VP, C.c_size_t, _VP]),
    "flhip_logsoftmax_fwd": (C.c_int, [_VP, _VP, C.c_int32, C.c_int32, C.c_int, _VP]),
    "flhip_logsoftmax_bwd": (C.c_int, [_VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int, _VP]),
    "flhip_cce_fwd": (C.c_int, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int32, C.c_int, _VP]),
    "flhip_cce_bwd": (C.c_int, [_VP, _VP, _VP, _VP, C.c_int32, C.c_int32, C.c_int, C.c_int32, C.c_int,
                                _VP]),
    "flhip_rnn_param_count": (C.c_size_t, [_VP]),
    "flhip_rnn_reserve_bytes": (C.c_size_t, [_VP]),
    "flhip_rnn_workspace_bytes": (C.c_size_t, [_VP]),
    "flhip_rnn_fwd": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, _VP, C.c_size_t, _VP, C.c_size_t, _VP]),
    "flhip_rnn_bwd": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, _VP, C.c_size_t, _VP, _VP, _VP, _VP, _VP,
                                C.c_size_t, _VP]),
    "flhip_reorder": (C.c_int, [_VP, _VP, C.POINTER(C.c_int64), C.POINTER(C.c_int32), C.c_int, _VP]),
    "flhip_affine_fwd": (C.c_int, [_VP, _VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int64, C.c_int, C.c_int,
                                   _VP]),
    "flhip_affine_bwd_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int64, C.c_int]),
    "flhip_affine_bwd": (C.c_int, [_VP, _VP, _VP, _VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int64, C.c_int,
                                   C.c_int, _VP, C.c_size_t, _VP]),
    "flhip_embedding_fwd": (C.c_int, [_VP, _VP, _VP, C.c_int64, C.c_int32, C.c_int32, C.c_int, _VP]),
    "flhip_embedding_bwd": (C.c_int, [_VP, _VP, _VP, C.c_int64, C.c_int32, C.c_int32, C.c_int, _VP]),
    "flhip_prelu_fwd": (C.c_int, [_VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int, C.c_int, _VP]),
    "flhip_prelu_bwd_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int]),
    "flhip_prelu_bwd": (C.c_int, [_VP, _VP, _VP, _VP, _VP, C.c_int64, C.c_int64, C.c_int, C.c_int, _VP, C.c_size_t,
                                  _VP]),
}

_lib = None


def lib():
    """Loads libflhip.so; there is no fallback when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "flashlight_amd: %s is missing; build it with "
                "`python -m flashlight_amd.build` (needs hipcc)" % LIB_PATH)
        h = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            f = getattr(h, name)
            f.restype = res
            f.argtypes = args
        _lib = h
    return _lib


def check(rc):
    """Maps a status to the exception kinds of the reference boundary."""
    if rc == OK:
        return
    msg = lib().flhip_last_error().decode()
    if rc == INVALID_ARGUMENT:
        raise ValueError(msg)      # std::invalid_argument
    raise RuntimeError(msg)        # std::runtime_error


def set_option(name, value=None):
    """flhip_set_option: a measurement / debugging switch (value None = default)."""
    check(lib().flhip_set_option(name.encode(), None if value is None else str(value).encode()))
