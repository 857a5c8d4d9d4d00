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
           "conv2d_mfma_wgrad_slab_bf16.hip", "conv2d_mfma_strip_bf16.hip", "conv2d_mfma_first_bf16.hip", "conv2d_mfma_cells.hip",
           "conv2d_mfma_pointwise_dma_bf16.hip", "conv2d_mfma_wgrad_dma_bf16.hip", "conv2d_mfma_tap1d.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


# hipcc compiles a .hip file twice.  The device pass (amdgcn, gfx950) knows the target feature
# packed-fp32-ops and honours its removal (tests/test_build_flags.py compiles a probe to assembly
# with and without it).  The host pass (x86-64) has no such feature and says so once per -Xclang
# pair: "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)".  That
# one line is counted and reported as such; every other diagnostic is printed as it is.
_HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"
_host_pass_notes = 0


def _compile(src):
    global _host_pass_notes
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    lines = (r.stdout + r.stderr).splitlines()
    _host_pass_notes += sum(1 for l in lines if l.strip() == _HOST_PASS_NOTE)
    out = "\n".join(l for l in lines if l.strip() != _HOST_PASS_NOTE)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, out))
    if out.strip():
        sys.stderr.write(out + "\n")
    return obj


HOST = os.path.join(HERE, "host")
HOST_LIB = os.path.join(LIBDIR, "libflhip_host.so")
STEP_BENCH = os.path.join(LIBDIR, "flhip_step_bench")
HOST_SOURCES = ["HipTensor.cpp", "HipAutogradExtension.cpp", "Functions.cpp", "Modules.cpp", "Optimizers.cpp", "Resnet.cpp",
                "SequentialBuilder.cpp"]
TESTS_DIR = os.path.join(ROOT, "tests", "cpp")
TESTS_BIN = os.path.join(TESTS_DIR, "bin")
# test program -> links the CPU checker?
TEST_PROGRAMS = {"test_host_extension": True, "test_resnet_step": True, "test_jacobian": False}


def _host_cxx():
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cxx = [os.environ.get("CXX", "g++"), "-O2", "-g", "-rdynamic", "-std=c++17", "-Wall", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(rocm, "include"), "-I" + os.path.join(ROOT, "include"), "-I" + HOST]
    hiplibs = ["-L" + os.path.join(rocm, "lib"), "-lamdhip64", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    return cxx, hiplibs


def build_host(verbose=True):
    """The C++ host layer (HipTensor, HipAutogradExtension, caller closures, modules):
    libflhip_host.so, linked against libflhip.so.  Needs nothing outside the package."""
    cxx, hiplibs = _host_cxx()
    cmd = cxx + ["-fPIC", "-shared", "-o", HOST_LIB]
    cmd += [os.path.join(HOST, f) for f in HOST_SOURCES]
    cmd += ["-L" + LIBDIR, "-lflhip", "-Wl,-rpath,$ORIGIN"] + hiplibs
    subprocess.check_call(cmd)
    # the whole-step benchmark program bench.py runs for its step workloads
    cmd = cxx + ["-o", STEP_BENCH, os.path.join(HOST, "step_bench.cpp"), "-L" + LIBDIR, "-lflhip_host", "-lflhip",
                 "-Wl,-rpath,$ORIGIN"] + hiplibs
    subprocess.check_call(cmd)
    if verbose:
        print("built", HOST_LIB, "and", STEP_BENCH)
    return HOST_LIB


def build_tests(verbose=True):
    """The C++ test programs under tests/cpp (not part of the product): they link the two
    libraries above and, where they compare with it, the CPU checker oracle/libflref.so."""
    cxx, hiplibs = _host_cxx()
    os.makedirs(TESTS_BIN, exist_ok=True)
    oracle = os.path.join(ROOT, "oracle")
    subprocess.check_call(["make", "-C", oracle, "libflref.so"], stdout=subprocess.DEVNULL)

    def one(item):
        name, with_checker = item
        cmd = cxx + ["-o", os.path.join(TESTS_BIN, name), os.path.join(TESTS_DIR, name + ".cpp"),
                     "-L" + LIBDIR, "-lflhip_host", "-lflhip", "-Wl,-rpath,$ORIGIN/../../../flashlight_amd/lib"]
        if with_checker:
            cmd += ["-I" + oracle, "-L" + oracle, "-lflref", "-Wl,-rpath,$ORIGIN/../../../oracle"]
        subprocess.check_call(cmd + hiplibs)
        return name
    with ThreadPoolExecutor(max_workers=3) as ex:
        names = list(ex.map(one, TEST_PROGRAMS.items()))
    if verbose:
        print("built", ", ".join(names))


def build(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    if verbose:
        print("built", LIB)
        if _host_pass_notes:
            print("note: the x86-64 host pass of hipcc ignored the device-only feature flag "
                  "-packed-fp32-ops (%d notices); the gfx950 pass applies it" % _host_pass_notes)
    build_host(verbose)
    return LIB


if __name__ == "__main__":
    build()
    if os.path.isdir(TESTS_DIR):
        build_tests()
