"""Builds the native libraries in-tree (run on the build host; hipcc cross-compiles gfx950
without a GPU):

    decx_amd/lib/libdecx_hip.so        HIP kernels + the C ABI (include/decx_hip.h)
    decx_amd/lib/libDECX_BLAS_HIP.so   C++ host layer: the de:: objects and entry points

    python -m decx_amd.build
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(PKG, "lib", "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
             # No packed-fp32 VALU forms (v_pk_fma_f32, v_pk_mul_f32, v_pk_add_f32) in the device code.  The feature
             # switch reaches both passes of hipcc: the gfx950 pass applies it (tests/test_cabi_cpu.py compiles a
             # float2 multiply-add both ways and looks at the instructions), the x86 host pass does not know the
             # feature and says "ignoring feature" once per module: harmless, and dropped from the output below.
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument"]
HIP_SOURCES = ["gemm_f32.hip", "gemm_f32_dma.hip", "gemm_f16.hip", "gemm_f16_dma.hip", "gemm_f64.hip", "gemm_complex.hip", "gemv.hip", "conv_direct.hip", "capi.hip"]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wextra",
              "-I" + os.path.join(ROOT, "include")]


def _run(cmd):
    done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in done.stdout.splitlines()
                    if "'-packed-fp32-ops' is not a recognized feature for this target" not in l)
    if done.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + log)
        raise RuntimeError("build step failed: " + cmd[-1])
    return log


def build_hip(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    objs = [os.path.join(OBJ, s.replace(".hip", ".o")) for s in HIP_SOURCES]
    cmds = [[HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(HIP_SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(_run, cmds))
    out = os.path.join(LIB, "libdecx_hip.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", out] + objs)
    if verbose:
        print("built", out)
    return out


def build_host(verbose=False):
    srcs = sorted(f for f in os.listdir(HOST) if f.endswith(".cpp")) if os.path.isdir(HOST) else []
    if not srcs:
        return None
    out = os.path.join(LIB, "libDECX_BLAS_HIP.so")
    _run(["g++"] + HOST_FLAGS + ["-shared", "-o", out] + [os.path.join(HOST, s) for s in srcs] +
         ["-L" + LIB, "-ldecx_hip", "-Wl,-rpath,$ORIGIN"])
    if verbose:
        print("built", out)
    return out


def build_api_test(verbose=False):
    """The C++ program the tests drive the public de:: API with (tests/cpp/de_api_test)."""
    src = os.path.join(ROOT, "tests", "cpp", "de_api_test.cpp")
    out = os.path.join(ROOT, "tests", "cpp", "de_api_test")
    _run(["g++", "-O1", "-std=c++17", "-Wall", "-pthread", "-I" + os.path.join(ROOT, "include"), src, "-o", out,
          "-L" + LIB, "-lDECX_BLAS_HIP", "-ldecx_hip", "-Wl,-rpath," + LIB, "-Wl,-rpath,$ORIGIN/../../decx_amd/lib"])
    if verbose:
        print("built", out)
    return out


def build_all(verbose=False):
    build_hip(verbose)
    build_host(verbose)
    build_api_test(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
