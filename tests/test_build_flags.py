"""The build's device-code flags do what they are there for: with the flags of flashlight_amd/build.py
the gfx950 pass emits no packed fp32 arithmetic for code that would otherwise get it; the
x86-64 host pass of the same command only notes that it does not know the feature."""
import os
import subprocess

from flashlight_amd import build

PROBE = """
#include <hip/hip_runtime.h>
__global__ void probe(float2* a, const float2* b, const float2* c) {
  const int i = threadIdx.x + blockIdx.x * 256;
  const float2 x = b[i], y = c[i];
  a[i] = make_float2(x.x * y.x + 1.0f, x.y * y.y + 1.0f);
}
"""
PACKED = ("v_pk_fma_f32", "v_pk_mul_f32", "v_pk_add_f32")


def _device_asm(tmp_path, flags):
    src = tmp_path / "probe.hip"
    src.write_text(PROBE)
    out = tmp_path / "probe.s"
    r = subprocess.run([build.HIPCC] + flags + ["--cuda-device-only", "-S", str(src), "-o", str(out)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return out.read_text(), r.stdout + r.stderr


def test_packed_fp32_is_off_in_the_device_pass(tmp_path):
    flags = [f for f in build.FLAGS if not f.startswith("-I")]
    with_flag, log = _device_asm(tmp_path, flags)
    assert not any(op in with_flag for op in PACKED)
    assert "not a recognized feature" not in log          # the device pass knows the feature
    drop = {"-Xclang", "-target-feature", "-packed-fp32-ops"}
    without, _ = _device_asm(tmp_path, [f for f in flags if f not in drop])
    assert any(op in without for op in PACKED), "the probe no longer shows what the flag changes"
