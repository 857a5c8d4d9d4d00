"""Compiles the HIP sources in csrc/ for gfx950 into flashlight_amd/lib/libflhip.so."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "_obj")
LIB = os.path.join(LIBDIR, "libflhip.so")

SOURCES = ["api.hip", "callers.hip", "rnn.hip", "pool2d.hip", "batchnorm.hip", "conv2d.hip", "conv2d_mfma_gather.hip", "conv2d_mfma_wgrad.hip",
           "conv2d_mfma_slab.hip", "conv2d_mfma_pointwise.hip", "conv2d_mfma_pointwise_bf16.hip", "conv2d_mfma_wgrad_slab.hip", "conv2d_mfma_slab_bf16.hip",
           "conv2d_mfma_wgrad_slab_bf16.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    if out.strip():
        sys.stderr.write(out + "\n")
    return obj


HOST = os.path.join(HERE, "host")
HOST_LIB = os.path.join(LIBDIR, "libflhip_host.so")
HOST_SOURCES = ["HipTensor.cpp", "HipAutogradExtension.cpp", "Functions.cpp", "Modules.cpp", "Resnet.cpp",
                "SequentialBuilder.cpp"]
HOST_TEST_SRC = os.path.join(ROOT, "tests", "cpp", "test_host_extension.cpp")
HOST_TEST_BIN = os.path.join(ROOT, "tests", "cpp", "bin", "test_host_extension")


def build_host(verbose=True):
    """The C++ host layer (HipTensor, HipAutogradExtension, caller closures) and its
    test program; both link libflhip.so, the test also links the CPU checker."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cxx = [os.environ.get("CXX", "g++"), "-O2", "-g", "-rdynamic", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(rocm, "include"), "-I" + os.path.join(ROOT, "include"), "-I" + HOST]
    hiplibs = ["-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    cmd = cxx + ["-fPIC", "-shared", "-o", HOST_LIB]
    cmd += [os.path.join(HOST, f) for f in HOST_SOURCES]
    cmd += ["-L" + LIBDIR, "-lflhip", "-Wl,-rpath,$ORIGIN"] + hiplibs
    subprocess.check_call(cmd)
    if os.path.exists(HOST_TEST_SRC):
        os.makedirs(os.path.dirname(HOST_TEST_BIN), exist_ok=True)
        oracle = os.path.join(ROOT, "oracle")
        subprocess.check_call(["make", "-C", oracle, "libflref.so"], stdout=subprocess.DEVNULL)
        cmd = cxx + ["-I" + oracle, "-o", HOST_TEST_BIN, HOST_TEST_SRC,
                     "-L" + LIBDIR, "-lflhip_host", "-lflhip", "-L" + oracle, "-lflref",
                     "-Wl,-rpath,$ORIGIN/../../../flashlight_amd/lib",
                     "-Wl,-rpath,$ORIGIN/../../../oracle"] + hiplibs
        subprocess.check_call(cmd)
        # the ResNet-50 step program needs no CPU checker
        rsrc = os.path.join(os.path.dirname(HOST_TEST_SRC), "test_resnet_step.cpp")
        rbin = os.path.join(os.path.dirname(HOST_TEST_BIN), "test_resnet_step")
        cmd = cxx + ["-o", rbin, rsrc, "-L" + LIBDIR, "-lflhip_host", "-lflhip",
                     "-Wl,-rpath,$ORIGIN/../../../flashlight_amd/lib"] + hiplibs
        subprocess.check_call(cmd)
        # neither do the finite-difference Jacobian tests
        jsrc = os.path.join(os.path.dirname(HOST_TEST_SRC), "test_jacobian.cpp")
        jbin = os.path.join(os.path.dirname(HOST_TEST_BIN), "test_jacobian")
        cmd = cxx + ["-o", jbin, jsrc, "-L" + LIBDIR, "-lflhip_host", "-lflhip",
                     "-Wl,-rpath,$ORIGIN/../../../flashlight_amd/lib"] + hiplibs
        subprocess.check_call(cmd)
    if verbose:
        print("built", HOST_LIB)
    return HOST_LIB


def build(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB)
    build_host(verbose)
    return LIB


if __name__ == "__main__":
    build()
