"""Builds the HIP library in-tree: rivoli_amd/csrc/*.hip -> rivoli_amd/csrc/librivoli_kvcache.so.

Mirrors how the reference builds its kernels (crates/backend/build.rs:103-183: hipcc,
--offload-arch from the environment, -O3 -fPIC, link amdhip64), except that the default
architecture here is gfx950 and the product is one shared library behind a C ABI.
"""
from __future__ import annotations

import os
import re
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(CSRC, "librivoli_kvcache.so")
HOST_LIB_PATH = os.path.join(CSRC, "librivoli_pagepool.so")
KERNELS = ["kv_append.hip", "kv_gather.hip", "index_topk.hip", "index_score.hip", "mla_attend.hip",
           "act_quant.hip", "kv_compress.hip", "kv_ring.hip", "gather_attn.hip", "hash_rows.hip",
           "block_index.hip"]
# Matrix-instruction results in ordinary registers: the 8-bit attention kernel keeps its 128
# accumulators there and its q terms in the accumulation registers (mla_attend_f8.hpp); the bf16
# kernels of the same file time the same either way.
EXTRA_FLAGS = {"mla_attend.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}
HOST_SOURCES = ["pagepool.cpp"]
# Kernels whose design rests on "no scratch memory": source file -> (substring of the mangled
# name, suffix of it). The 8-bit attention kernels run one wave per SIMD on the whole register
# file and order their own LDS transfers (hand-placed waits, an m0 swap around each transfer): a
# build of them that spills is a different program, so the build refuses to produce one (a
# compile without EXTRA_FLAGS, an ablation with a piece compiled out).
NO_SCRATCH = {"mla_attend.hip": ("mla_attend_paged_kernel", "Lb1EEEvNS_10AttendArgsE")}


def check_resources(k: str, report: str) -> None:
    """Raises when a kernel of NO_SCRATCH[k] in hipcc's resource report uses scratch memory or
    more LDS than a compute unit has."""
    if k not in NO_SCRATCH:
        return
    part, suffix = NO_SCRATCH[k]
    seen = 0
    for block in re.split(r"remark: Function Name: ", report)[1:]:
        name = block.split()[0]
        if part not in name or not name.endswith(suffix):
            continue
        seen += 1
        scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", block).group(1))
        lds = int(re.search(r"LDS Size \[bytes/block\]: (\d+)", block).group(1))
        if scratch or lds > 160 * 1024:
            raise RuntimeError(f"{k}: {name} uses {scratch} bytes of scratch per lane and {lds} bytes of LDS; "
                               "this kernel must compile to 0 and at most 163840")
    if not seen:
        raise RuntimeError(f"{k}: no kernel matching {part}...{suffix} in the resource report")


def hipcc() -> str:
    return os.environ.get("HIPCC", "hipcc")


def offload_arch() -> str:
    return os.environ.get("RIVOLI_OFFLOAD_ARCH", "gfx950")


def build_kernels(verbose: bool = False) -> str:
    """Every source to an object of its own (in parallel, under build/), then one link."""
    from concurrent.futures import ThreadPoolExecutor

    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    common = [hipcc(), f"--offload-arch={offload_arch()}", "-O3", "-std=c++17", "-fPIC",
              # packed-f32 instructions stay off: plain f32 math only
              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
              "-I", os.path.join(os.path.dirname(CSRC), "..", "include")]

    def compile_one(k: str) -> str:
        obj = os.path.join(objdir, k.replace(".hip", ".o"))
        report = ["-Rpass-analysis=kernel-resource-usage"] if k in NO_SCRATCH else []
        res = subprocess.run(common + EXTRA_FLAGS.get(k, []) + report + ["-c", os.path.join(CSRC, k), "-o", obj],
                             capture_output=True, text=True)
        if res.returncode != 0 or (verbose and not report):
            sys.stderr.write(res.stdout + res.stderr)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed compiling " + k)
        try:
            check_resources(k, res.stderr)
        except RuntimeError:
            os.remove(obj)  # never link it
            raise
        return obj

    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        objs = list(pool.map(compile_one, KERNELS))
    res = subprocess.run([hipcc(), f"--offload-arch={offload_arch()}", "-shared", "-fPIC", "-o", LIB_PATH] + objs,
                         capture_output=True, text=True)
    if verbose or res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed linking " + LIB_PATH)
    return LIB_PATH


def build_host(verbose: bool = False) -> str:
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
           "-I", os.path.join(os.path.dirname(CSRC), "..", "include"),
           "-o", HOST_LIB_PATH] + [os.path.join(CSRC, s) for s in HOST_SOURCES]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
    if res.returncode != 0:
        raise RuntimeError("g++ failed building " + HOST_LIB_PATH)
    return HOST_LIB_PATH


def build_all(verbose: bool = False) -> None:
    build_kernels(verbose)
    build_host(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print(LIB_PATH)
    print(HOST_LIB_PATH)
