"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and the argument checks that need no GPU behave as documented."""
import ctypes as C
import os
import re

import pytest

from flashlight_amd import capi
from flashlight_amd.ops import bn_view, derive_padding

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_exported_and_bound():
    text = open(os.path.join(ROOT, "include", "flhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = set(re.findall(r"\b(flhip_[a-z0-9_]+)\s*\(", text))
    assert declared, "no declarations parsed"
    lib = capi.lib()
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(capi.SYMBOLS)


def test_version_and_arch():
    text = open(os.path.join(ROOT, "include", "flhip.h")).read()
    declared = int(re.search(r"#define\s+FLHIP_VERSION\s+(\d+)", text).group(1))
    assert capi.lib().flhip_version() == declared >= 200
    assert capi.lib().flhip_arch() == b"gfx950"


def test_convert_many_launch_split():
    """How flhip_convert_many cuts a list of tensors into launches: 64 tensors or 2^31 - 1
    pieces of 2048 elements per launch, whichever comes first; empty tensors take no slot."""
    lib = capi.lib()

    def plan(sizes):
        n = (C.c_size_t * len(sizes))(*sizes)
        where = (C.c_int32 * len(sizes))()
        launches = lib.flhip_convert_many_launches(n, len(sizes), where)
        return launches, list(where)

    assert plan([]) == (0, [])
    assert plan([0, 0]) == (0, [-1, -1])
    assert plan([5] * 64) == (1, [0] * 64)
    assert plan([5] * 65) == (2, [0] * 64 + [1])
    assert plan([5, 0] * 65)[0] == 2
    big = (1 << 40) - 1                       # 2^29 pieces
    launches, where = plan([big] * 9)         # three fit under 2^31 - 1, the fourth does not
    assert launches == 3 and where == [0, 0, 0, 1, 1, 1, 2, 2, 2]
    # exactly the grid limit fits, one more piece does not
    limit = (1 << 31) - 1
    rest = limit - 3 * (1 << 29)
    assert plan([big] * 3 + [rest * 2048])[0] == 1
    assert plan([big] * 3 + [rest * 2048 + 1])[0] == 2
    assert plan([1 << 40])[0] == -1           # refused, like the call itself


def test_conv_out_dims_and_errors():
    lib = capi.lib()
    oh, ow = C.c_int32(), C.c_int32()
    d = capi.ConvDesc(32, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, capi.F32)
    assert lib.flhip_conv2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)) == capi.OK
    assert (oh.value, ow.value) == (56, 56)
    d = capi.ConvDesc(64, 3, 224, 224, 64, 7, 7, 2, 2, 3, 3, 1, 1, 1, capi.F32)
    assert lib.flhip_conv2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)) == capi.OK
    assert (oh.value, ow.value) == (112, 112)
    bad = capi.ConvDesc(1, 3, 8, 8, 4, 3, 3, 1, 1, 0, 0, 1, 1, 2, capi.F32)   # groups !| C
    assert lib.flhip_conv2d_out_dims(C.byref(bad), C.byref(oh), C.byref(ow)) == capi.INVALID_ARGUMENT
    with pytest.raises(ValueError):
        capi.check(capi.INVALID_ARGUMENT)
    assert b"groups" in lib.flhip_last_error()
    bad = capi.ConvDesc(1, 3, 2, 2, 4, 5, 5, 1, 1, 0, 0, 1, 1, 1, capi.F32)   # kernel > input
    assert lib.flhip_conv2d_out_dims(C.byref(bad), C.byref(oh), C.byref(ow)) == capi.INVALID_ARGUMENT


def test_pool_out_dims_and_errors():
    lib = capi.lib()
    oh, ow = C.c_int32(), C.c_int32()
    d = capi.PoolDesc(32, 64, 112, 112, 3, 3, 2, 2, 1, 1, 0, capi.F32)
    assert lib.flhip_pool2d_out_dims(C.byref(d), C.byref(oh), C.byref(ow)) == capi.OK
    assert (oh.value, ow.value) == (56, 56)
    bad = capi.PoolDesc(1, 1, 8, 8, 2, 2, 2, 2, 2, 2, 0, capi.F32)            # pad >= window
    assert lib.flhip_pool2d_out_dims(C.byref(bad), C.byref(oh), C.byref(ow)) == capi.INVALID_ARGUMENT
    bad = capi.PoolDesc(1, 1, 8, 8, 2, 2, 2, 2, 0, 0, 7, capi.F32)            # unknown mode
    assert lib.flhip_pool2d_out_dims(C.byref(bad), C.byref(oh), C.byref(ow)) == capi.INVALID_ARGUMENT


def test_null_arguments_are_rejected_before_any_launch():
    lib = capi.lib()
    d = capi.PoolDesc(1, 1, 8, 8, 2, 2, 2, 2, 0, 0, 0, capi.F32)
    assert lib.flhip_pool2d_fwd(C.byref(d), None, None, None, None) == capi.INVALID_ARGUMENT
    # max-pool backward without the forward argmax: the reference throws
    # std::invalid_argument (onednn/Pool2D.cpp:190-193)
    assert lib.flhip_pool2d_bwd(C.byref(d), C.c_void_p(16), None, C.c_void_p(16), None) == capi.INVALID_ARGUMENT
    b = capi.BnDesc(4, 3, 10, capi.F32)
    assert lib.flhip_bn_workspace_bytes(C.byref(b)) > 0
    assert lib.flhip_bn_bwd(C.byref(b), C.c_void_p(16), C.c_void_p(16), None, None, None,
                            C.c_void_p(16), None, None, None, 0, None) == capi.INVALID_ARGUMENT
    assert lib.flhip_copy_bytes(C.c_void_p(16), C.c_void_p(32), 24, None) == capi.INVALID_ARGUMENT


def test_bn_view_and_same_padding():
    assert bn_view((8, 3, 13, 13), [2]) == (8, 3, 169)
    assert bn_view((8, 4, 13, 13), [0, 1, 2]) == (8, 676, 1)
    with pytest.raises(ValueError):
        bn_view((8, 4, 13, 13), [0, 2])
    # fl::derivePadding (flashlight/fl/nn/Utils.cpp:87-100)
    assert derive_padding(56, 3, 1, -1) == 1
    assert derive_padding(224, 7, 2, -1) == 3
    assert derive_padding(56, 1, 2, -1) == 0
    assert derive_padding(1500, 21, 1, -1) == 10
    assert derive_padding(1500, 21, 2, -1) == 10
    assert derive_padding(28, 5, 1, -1) == 2
    assert derive_padding(112, 3, 2, -1) == 1
    assert derive_padding(9, 3, 1, 4) == 4


def test_plan_lists():
    """The kernel families of the backward passes have names; the forward pass has no plans."""
    lib = capi.lib()
    for pas in (capi.CONV_BWD_DATA, capi.CONV_BWD_FILTER):
        n = lib.flhip_conv2d_plan_count(pas)
        assert n >= 2
        names = [lib.flhip_conv2d_plan_name(pas, i) for i in range(n)]
        assert all(names) and len(set(names)) == n
        assert lib.flhip_conv2d_plan_name(pas, n) is None and lib.flhip_conv2d_plan_name(pas, -1) is None
    assert lib.flhip_conv2d_plan_count(capi.CONV_FWD) == 0
