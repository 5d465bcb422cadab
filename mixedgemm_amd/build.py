"""Builds the HIP library (C-ABI) and the pybind11/torch extension module.

    python -m mixedgemm_amd.build            # build what is missing or stale
    python -m mixedgemm_amd.build --force    # rebuild everything

Outputs (kept out of git, shipped with the tree):
    mixedgemm_amd/lib/libmixedgemm_hip.so   hand-written gfx950 kernels + extern "C" entry points
    mixedgemm_amd/lib/libmixedgemm_bench.so measurement kernels bench.py times next to the library (not the product)
    build/mixedgemm.so                      torch extension with the reference's operator surface
    build/abi_driver                        torch-free host program (tests/c_host) on the C-ABI
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libmixedgemm_hip.so")
EXT_DIR = os.path.join(ROOT, "build")
EXT_PATH = os.path.join(EXT_DIR, "mixedgemm.so")
DRIVER_SRC = os.path.join(ROOT, "tests", "c_host", "abi_driver.cpp")
DRIVER_PATH = os.path.join(EXT_DIR, "abi_driver")

BENCH_LIB_PATH = os.path.join(LIB_DIR, "libmixedgemm_bench.so")
OBJ_DIR = os.path.join(EXT_DIR, "obj")

HIP_SOURCES = ["abi.hip", "reorder_quant.hip", "mixed_gemm.hip", "mixed_gemm_256.hip", "calibrate.hip"]
BENCH_SOURCES = ["bench_kernels.hip"]
HIP_HEADERS = ["mg_common.h", os.path.join(ROOT, "include", "mixedgemm_abi.h")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed FP32 VALU forms are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
]


def _stale(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


# Kernels whose loads and LDS copies are inline assembly that the compiler does not count: a register such a load
# is still to fill must never be moved or spilled, so these kernels must compile without scratch memory.  (The
# whole-tile GEMM is listed for speed: a spill inside its K loop costs more than anything else there.)
NO_SCRATCH_KERNELS = ("mixed_gemm_decode_kernel", "reorder_quant_dma_kernel", "mixed_gemm_256_kernel",
                      "mixed_gemm_256_tail_kernel")


# ... except the quantizer for K > 20480 (run-time workgroup size, up to 1024 lanes of 128 registers): it spills, and
# reads its index and its gathered channels through loads the compiler sees instead.
MAY_SPILL = ("reorder_quant_dma_kernelILi32ELi0E",)


def _split_remarks(stderr: str) -> tuple[str, str]:
    """(resource-usage remarks, everything else) of a hipcc run with -Rpass-analysis=kernel-resource-usage."""
    remarks, other, skip = [], [], 0
    for line in stderr.splitlines():
        if "-Rpass-analysis=kernel-resource-usage" in line:
            remarks.append(line)
            skip = 2          # the source line and the caret that follow a remark
        elif skip and ("remark" not in line) and (line.strip().startswith(("|", "^")) or "|" in line[:8]):
            skip -= 1
        else:
            other.append(line)
    return "\n".join(remarks), "\n".join(other)


def _check_no_scratch(src: str, remarks: str) -> None:
    import re
    name, bad = None, []
    for line in remarks.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
        m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name and int(m.group(1)) and any(k in name for k in NO_SCRATCH_KERNELS) and not any(k in name for k in MAY_SPILL):
            bad.append(f"{name}: {m.group(1)} bytes of scratch per lane")
    if bad:
        raise RuntimeError(f"{os.path.basename(src)}: kernels that must not spill do:\n  " + "\n  ".join(bad))


def _compile_and_link(sources: list[str], target: str, force: bool, verbose: bool) -> str:
    """One object per source, compiled side by side, then one link."""
    from concurrent.futures import ThreadPoolExecutor

    srcs = [os.path.join(CSRC, s) for s in sources]
    hdrs = [h if os.path.isabs(h) else os.path.join(CSRC, h) for h in HIP_HEADERS]
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, os.path.basename(s) + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        if force or _stale(obj, [src] + hdrs):
            cmd = ["hipcc", *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", src, "-o", obj]
            if verbose:
                print(" ".join(cmd), flush=True)
            done = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
            remarks, other = _split_remarks(done.stderr)
            if other.strip():
                print(other, file=sys.stderr, flush=True)
            if done.returncode != 0:
                raise subprocess.CalledProcessError(done.returncode, cmd)
            try:
                _check_no_scratch(src, remarks)
            except Exception:
                os.remove(obj)
                raise

    with ThreadPoolExecutor(max_workers=min(len(srcs), 6)) as pool:
        list(pool.map(compile_one, zip(srcs, objs)))
    if force or _stale(target, objs):
        cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", target, *objs]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return target


def build_hip_library(force: bool = False, verbose: bool = False) -> str:
    return _compile_and_link(HIP_SOURCES, LIB_PATH, force, verbose)


def build_bench_library(force: bool = False, verbose: bool = False) -> str:
    """Measurement kernels for bench.py (MFMA register loop, plain copy, empty launch): their own
    shared object, so that the product library holds the hot path only."""
    return _compile_and_link(BENCH_SOURCES, BENCH_LIB_PATH, force, verbose)


def build_torch_extension(force: bool = False, verbose: bool = False) -> str:
    """g++ build of csrc/bindings.cpp against torch + pybind11; links the HIP
    library through its C-ABI only (no HIP headers on this side)."""
    import torch
    from torch.utils import cpp_extension

    src = os.path.join(CSRC, "bindings.cpp")
    deps = [src, os.path.join(ROOT, "include", "mixedgemm_abi.h"), LIB_PATH]
    if force or _stale(EXT_PATH, deps):
        os.makedirs(EXT_DIR, exist_ok=True)
        torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
        inc = [f"-I{p}" for p in cpp_extension.include_paths()]
        inc += [f"-I{sysconfig.get_paths()['include']}", f"-I{os.path.join(ROOT, 'include')}"]
        cmd = [
            "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
            "-DTORCH_EXTENSION_NAME=mixedgemm", "-DTORCH_API_INCLUDE_EXTENSION_H",
            "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-I/opt/rocm/include",
            f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
            *inc, src, "-o", EXT_PATH,
            f"-L{LIB_DIR}", "-lmixedgemm_hip", f"-Wl,-rpath,{LIB_DIR}", "-Wl,-rpath,$ORIGIN/../mixedgemm_amd/lib",
            f"-L{torch_lib}", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_python", f"-Wl,-rpath,{torch_lib}",
        ]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return EXT_PATH


def build_c_host_driver(force: bool = False, verbose: bool = False) -> str:
    """The torch-free host program of tests/c_host (HIP runtime + the C-ABI only)."""
    deps = [DRIVER_SRC, os.path.join(ROOT, "include", "mixedgemm_abi.h"), LIB_PATH]
    if force or _stale(DRIVER_PATH, deps):
        os.makedirs(EXT_DIR, exist_ok=True)
        cmd = ["hipcc", "-O2", "-std=c++17", f"-I{os.path.join(ROOT, 'include')}", DRIVER_SRC, "-o", DRIVER_PATH,
               f"-L{LIB_DIR}", "-lmixedgemm_hip", f"-Wl,-rpath,{LIB_DIR}", "-Wl,-rpath,$ORIGIN/../mixedgemm_amd/lib"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return DRIVER_PATH


def build_all(force: bool = False, verbose: bool = False) -> None:
    build_hip_library(force, verbose)
    build_bench_library(force, verbose)
    build_torch_extension(force, verbose)
    build_c_host_driver(force, verbose)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv, verbose=True)
