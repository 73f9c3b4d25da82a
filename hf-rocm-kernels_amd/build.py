"""Build the two shared objects of this package, in-tree, for gfx950 only.

  hf_rocm_kernels/libhfrk_gfx950.so   HIP kernels + C ABI (include/hfrk_gfx950.h); depends on the HIP runtime only
  hf_rocm_kernels/_HFRK_C.abi3.so     torch.ops._HFRK_C registration, a thin caller of the C ABI
  hf_rocm_kernels/benchmarks/libhfrk_bench_probes.so   measurement probes for `bench.py --workload floor` (bench_probes/probe.hip);
                                      not part of the product library

Plain hipcc / g++ command lines: no cmake, no hipify, no CUDA-compat headers (the reference's CMakeLists.txt,
cmake/utils.cmake and cmake/hipify.py have no counterpart here).  hipcc cross-compiles, so no GPU is needed.

Usage:  python hf-rocm-kernels_amd/build.py [--no-torch]
"""
import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
PKG = os.path.join(HERE, "hf_rocm_kernels")
OBJ = os.path.join(HERE, "build")
INCLUDE = os.path.join(ROOT, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["hfrk_common.hip", "skinny_gemm.hip", "skinny_gemm_plan.hip", "skinny_gemm_stream.hip", "skinny_gemm_rows.hip", "skinny_gemm_rows_tiled.hip", "skinny_gemm_ksplit.hip", "residual_rms.hip", "swiglu.hip",
               "dynamic_quant.hip", "pack_weight.hip", "plan_table_file.hip"]
PROBE_SOURCE = os.path.join(HERE, "bench_probes", "probe.hip")
PROBE_LIB = os.path.join(PKG, "benchmarks", "libhfrk_bench_probes.so")
LIB_NAME = "libhfrk_gfx950.so"
EXT_NAME = "_HFRK_C.abi3.so"

# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I" + INCLUDE, "-I" + CSRC,
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), proc.stdout))
    return proc.stdout


def lib_path():
    return os.path.join(PKG, LIB_NAME)


def ext_path():
    return os.path.join(PKG, EXT_NAME)


def _compile_hip(src):
    hipcc = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    _run([hipcc] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
    return obj


def _compile_torch_bindings():
    import torch
    from torch.utils import cpp_extension

    cxx = shutil.which("g++") or "g++"
    obj = os.path.join(OBJ, "torch_bindings.o")
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-c",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-DPy_LIMITED_API=0x03090000"]
    for inc in cpp_extension.include_paths() + [os.path.join(ROCM, "include"), sysconfig.get_paths()["include"], INCLUDE]:
        cmd.append("-I" + inc)
    _run(cmd + [os.path.join(CSRC, "torch_bindings.cpp"), "-o", obj])
    return obj


def _build_probes():
    hipcc = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    _run([hipcc] + HIPCC_FLAGS + ["-shared", PROBE_SOURCE, "-o", PROBE_LIB, "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return PROBE_LIB


def _link_library(objs):
    hipcc = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path()] + objs +
         ["-Wl,-rpath," + os.path.join(ROCM, "lib"), "-Wl,--no-undefined"])
    return lib_path()


def _link_torch_extension(obj):
    import torch

    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cxx = shutil.which("g++") or "g++"
    _run([cxx, "-shared", "-fPIC", obj, "-o", ext_path(),
          "-L" + torch_lib, "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
          "-L" + PKG, "-l:" + LIB_NAME, "-Wl,-rpath,$ORIGIN"])
    return ext_path()


def build_all(with_torch=True):
    """Compile everything, every time it is called: objects in parallel, then the two links."""
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=6) as pool:
        hip_jobs = [pool.submit(_compile_hip, s) for s in HIP_SOURCES]
        ext_job = pool.submit(_compile_torch_bindings) if with_torch else None
        probe_job = pool.submit(_build_probes)
        objs = [j.result() for j in hip_jobs]
        probe_job.result()
        _link_library(objs)
        if ext_job is not None:
            _link_torch_extension(ext_job.result())
    return lib_path(), (ext_path() if with_torch else None)


if __name__ == "__main__":
    paths = build_all(with_torch="--no-torch" not in sys.argv)
    print("built:", *[p for p in paths if p])
