"""Builds the two native artefacts of the backend, in-tree under goinfer_amd/lib/:

  rocmdecode_gfx950.hsaco   the gfx950 code object (hipcc --genco, cross-compiles without a GPU)
  librocmdecode.so          the C-ABI host library (g++; binds libamdhip64 at run time with dlopen)
  librocmdecode_static.so   the allocation-free top-K entry point (hipcc; links the HIP runtime; opened by the library above)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "lib")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HSACO = os.path.join(LIB, "rocmdecode_gfx950.hsaco")
SO = os.path.join(LIB, "librocmdecode.so")
HOST_SOURCES = ["hipdyn.cc", "device.cc", "ops.cc", "model.cc", "bench.cc"]


def build_kernels(verbose=False):
    os.makedirs(LIB, exist_ok=True)
    src = os.path.join(HERE, "csrc", "kernels", "rocmdecode.hip")
    cmd = [os.path.join(ROCM, "bin", "hipcc"), "--genco", "--offload-arch=gfx950", "-O3", "-std=c++17",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           # MFMA results that the VALU reads next (the int8 dots before their f32 fold) stay in ordinary VGPRs
           "-mllvm", "-amdgpu-mfma-vgpr-form=1", "-o", HSACO, src]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return HSACO


def build_host(verbose=False):
    os.makedirs(LIB, exist_ok=True)
    srcs = [os.path.join(HERE, "csrc", "host", s) for s in HOST_SOURCES]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-Wno-unused-parameter",
           "-D__HIP_PLATFORM_AMD__=1", "-I" + os.path.join(ROCM, "include"), "-o", SO] + srcs + ["-ldl", "-lpthread"]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return SO


STATIC_SO = os.path.join(LIB, "librocmdecode_static.so")


def build_static(verbose=False):
    """The allocation-free entry point's library: one hipcc translation unit (host and gfx950 device code) that links the HIP runtime."""
    os.makedirs(LIB, exist_ok=True)
    src = os.path.join(HERE, "csrc", "static", "topk_static.hip")
    cmd = [os.path.join(ROCM, "bin", "hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", STATIC_SO, src]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return STATIC_SO


SYNTH = os.path.join(LIB, "libgoinfer_synth.so")


def build_synth(verbose=False):
    os.makedirs(LIB, exist_ok=True)
    cmd = ["g++", "-O3", "-march=x86-64-v2", "-std=c++17", "-fPIC", "-shared", "-fopenmp", "-ffp-contract=off", "-Wall",
           "-o", SYNTH, os.path.join(HERE, "csrc", "host", "synth.cc")]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return SYNTH


def build_all(verbose=False):
    return build_kernels(verbose), build_host(verbose), build_static(verbose), build_synth(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", HSACO, SO, SYNTH)
