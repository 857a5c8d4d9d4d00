"""Runs the C++ test programs of the host layer (HipTensor, registration,
HipAutogradExtension, caller closures, modules, Jacobians) on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin", "test_host_extension")


@pytest.mark.gpu
def test_host_extension_program():
    assert os.path.exists(BIN), "build it with `python -m flashlight_amd.build`"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "all host extension checks passed" in r.stdout


@pytest.mark.gpu
def test_resnet50_step_program():
    """configs[4] at batch 2, fp32 and bf16 storage: every operation of a real ResNet-50 step
    (conv / batch norm / pooling forward and backward, ReLU, residual adds, casts, the
    classifier and the loss) replayed on the CPU checker with the operation's own device
    inputs, at the stated tolerances; shapes, gradients for all 161 parameter tensors,
    run-to-run bit identity."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_resnet_step")
    assert os.path.exists(exe), "build it with `python -m flashlight_amd.build`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "ResNet-50 step checks passed" in r.stdout


@pytest.mark.gpu
def test_jacobian_program():
    """The reference's finite-difference Jacobian tests of conv2d, pool2d, batchnorm (one and
    several feature axes, the LayerNorm axes) and rnn, with its shapes and tolerances
    (AutogradConv2DTest.cpp:21-74,137-213, AutogradTest.cpp:333-337,
    AutogradNormalizationTest.cpp:228-256,294-324,365-383, AutogradRnnTest.cpp:24-160)."""
    exe = os.path.join(ROOT, "tests", "cpp", "bin", "test_jacobian")
    assert os.path.exists(exe), "build it with `python -m flashlight_amd.build`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "all Jacobian checks passed" in r.stdout


def test_host_library_is_built_and_links_the_c_abi():
    lib = os.path.join(ROOT, "flashlight_amd", "lib", "libflhip_host.so")
    assert os.path.exists(lib)
    out = subprocess.run(["nm", "-D", "--defined-only", lib], capture_output=True, text=True).stdout
    for sym in ("HipAutogradExtension", "getAutogradExtension", "conv2dBackwardFilterBias",
                "batchnormBackward", "pool2dBackward"):
        assert sym in out, sym
    und = subprocess.run(["nm", "-D", "--undefined-only", lib], capture_output=True, text=True).stdout
    assert "flhip_conv2d_bwd_filter" in und and "flhip_bn_bwd" in und
