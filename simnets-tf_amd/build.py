"""Compiles the HIP sources under csrc/ into libsimnets_hip.so next to this file (gfx950 only).

Run as a script (`python simnets-tf_amd/build.py`) or call build().  hipcc cross-compiles, so no
GPU is needed.  Packed FP32 VALU instructions are switched off for the device pass.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsimnets_hip.so")
NATIVE = os.path.join(HERE, "_simnets_native.so")
BENCH = os.path.join(HERE, "simnets_bench")
OBJDIR = os.path.join(HERE, "build")

SOURCES = ["host_logic.cpp", "capi.hip", "similarity_direct.hip", "similarity_mfma.hip", "mex.hip",
           "similarity_grad.hip", "mex_grad.hip", "mex_pool.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = ["-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-Wall",
          "-Wno-unused-function"]
DEVICE = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-fno-fast-math",
          "-fno-gpu-rdc"]


# hipcc hands the -target-feature switch to its host pass as well, which does not know an AMDGPU feature and says so
# once per file; the switch only matters to (and is honoured by) the device pass, so that one line is dropped.
_HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target"


def _run(cmd):
    r = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    noise = [ln for ln in r.stderr.splitlines() if _HOST_PASS_NOTE not in ln]
    if noise:
        print("\n".join(noise), file=sys.stderr)
    if r.returncode != 0:
        raise subprocess.CalledProcessError(r.returncode, cmd)


def _compile(src, extra):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    path = os.path.join(CSRC, src)
    if src.endswith(".hip"):
        cmd = [HIPCC, "-c", path, "-o", obj] + COMMON + DEVICE + extra
    else:
        cmd = [HIPCC, "-x", "c++", "-c", path, "-o", obj] + COMMON + extra
    _run(cmd)
    return obj


def build(extra=(), verbose=False):
    os.makedirs(OBJDIR, exist_ok=True)
    extra = list(extra)
    with ThreadPoolExecutor(max_workers=min(len(SOURCES), 8)) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), SOURCES))
    subprocess.run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs, check=True)
    # standalone C++ harness, linked against the product library only
    bench_src = os.path.join(HERE, "bench", "simnets_bench.hip")
    _run([HIPCC, bench_src, "-o", BENCH] + COMMON + DEVICE + extra +
         ["-L" + HERE, "-lsimnets_hip", "-Wl,-rpath,$ORIGIN"])
    build_op_layer()
    if verbose:
        print("built", LIB, ",", NATIVE, "and", BENCH)
    return LIB


def build_op_layer():
    """The compiled operator layer (csrc/op_layer.cpp): host code only, built with the host compiler against torch's
    headers and linked to libsimnets_hip.so next to it."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-o", NATIVE,
           os.path.join(CSRC, "op_layer.cpp"), "-I" + os.path.join(ROOT, "include")]
    cmd += ["-I" + p for p in ce.include_paths()] + ["-I" + sysconfig.get_paths()["include"], "-I/opt/rocm/include"]
    cmd += ["-DUSE_ROCM=1", "-D__HIP_PLATFORM_AMD__=1", "-DHIPBLAS_V2", "-DTORCH_EXTENSION_NAME=_simnets_native",
            "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
            "-Wall", "-Wno-unused-function"]
    cmd += ["-L" + tlib, "-L" + HERE, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-lsimnets_hip", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    _run(cmd)
    return NATIVE


if __name__ == "__main__":
    build(sys.argv[1:], verbose=True)
