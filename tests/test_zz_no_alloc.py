"""flhip_conv2d_bwd_filter_static (the entry point that allocates nothing) against
flhip_conv2d_bwd_filter with a caller workspace: bit-identical dw / db through the
C ABI, on calls in a row that share the library's static buffer, later calls with
smaller inputs (so stale partials of an earlier call sit behind the live ones)."""
import ctypes as C

import numpy as np
import pytest
import torch

import flashlight_amd as fa
from flashlight_amd import capi
from gpu_util import dev
from oracle import flref
from refmath import rel_l2

pytestmark = pytest.mark.gpu

# (x shape, w shape, stride, pad): first the large call, then smaller ones
SEQUENCE = [
    ((8, 64, 56, 56), (64, 64, 3, 3), (1, 1), (1, 1)),     # row-slab kernel, 128-way split
    ((2, 64, 28, 28), (64, 64, 3, 3), (1, 1), (1, 1)),     # the same kernel, fewer partials
    ((3, 96, 14, 14), (160, 96, 1, 1), (2, 2), (0, 0)),    # 1x1 strided
    ((2, 3, 32, 32), (16, 3, 7, 7), (2, 2), (3, 3)),       # gather filter gradient
]


def _both(x, dy, wshape, stride, pad, want_bias=True):
    geo = dict(sx=stride[1], sy=stride[0], px=pad[1], py=pad[0])
    dw_ref, db_ref = fa.conv2d_backward_filter_bias(dy, x, wshape, want_bias, **geo)
    dw = torch.full(wshape, float("nan"), dtype=torch.float32, device="cuda")
    db = torch.full((wshape[0],), float("nan"), dtype=torch.float32, device="cuda") if want_bias else None
    fa.conv2d_backward_filter_bias_static(dy, x, dw, db, **geo)
    torch.cuda.synchronize()
    return dw, db, dw_ref, db_ref


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_static_scratch_matches_workspace_entry_point(dtype):
    rng = np.random.default_rng(11)
    for xs, ws, stride, pad in SEQUENCE:
        d = flref.conv_desc(xs, ws, stride, pad)
        x = rng.standard_normal(xs).astype(np.float32)
        oh, ow_ = flref.conv_out(d)
        dy = rng.standard_normal((xs[0], ws[0], oh, ow_)).astype(np.float32)
        xd, dyd = dev(x, dtype), dev(dy, dtype)
        dw, db, dw_ref, db_ref = _both(xd, dyd, ws, stride, pad)
        assert torch.equal(dw, dw_ref), (xs, ws)
        assert torch.equal(db, db_ref), (xs, ws)
        # and against the CPU checker on the values the device saw
        ow, ob = flref.conv2d_bwd_filter(d, xd.float().cpu().numpy(), dyd.float().cpu().numpy())
        assert rel_l2(dw.cpu().numpy(), ow) <= 1e-4
        assert rel_l2(db.cpu().numpy(), ob) <= 1e-4


def test_static_scratch_allocates_nothing():
    rng = np.random.default_rng(12)
    xs, ws = (4, 64, 28, 28), (64, 64, 3, 3)
    x, dy = dev(rng.standard_normal(xs).astype(np.float32)), dev(rng.standard_normal(xs).astype(np.float32))
    dw = torch.empty(ws, dtype=torch.float32, device="cuda")
    db = torch.empty((64,), dtype=torch.float32, device="cuda")
    fa.conv2d_backward_filter_bias_static(dy, x, dw, db, px=1, py=1)    # first call: symbol lookup
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    stats0 = torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(3):
        fa.conv2d_backward_filter_bias_static(dy, x, dw, db, px=1, py=1)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == stats0
    assert free1 == free0


def test_static_scratch_refuses_oversize():
    # the bf16 stride-2 3x3 filter gradient at batch 64 wants > 100 MB of gathered taps
    d = capi.ConvDesc(64, 128, 56, 56, 128, 3, 3, 2, 2, 1, 1, 1, 1, 1, capi.BF16)
    need = capi.lib().flhip_conv2d_workspace_bytes(C.byref(d), capi.CONV_BWD_FILTER)
    assert need > capi.STATIC_SCRATCH_BYTES
    one = torch.zeros(16, device="cuda")
    rc = capi.lib().flhip_conv2d_bwd_filter_static(C.byref(d), C.c_void_p(one.data_ptr()),
                                                   C.c_void_p(one.data_ptr()), C.c_void_p(one.data_ptr()),
                                                   None, None)
    assert rc == capi.INVALID_ARGUMENT
    assert b"static buffer" in capi.lib().flhip_last_error()
