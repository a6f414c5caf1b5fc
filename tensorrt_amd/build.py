"""Builds libtrtamd_bert_plugins.so (HIP kernels + C-ABI + IPluginV3 hosts) for gfx950 with hipcc.

Usage: ``python -m tensorrt_amd.build`` (or ``build_library()``).  hipcc cross-compiles without a
GPU; every source is recompiled on each call.
"""
from __future__ import annotations

import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
INCLUDE = os.path.join(os.path.dirname(ROOT), "include")
LIB_DIR = os.path.join(ROOT, "lib")
LIB_NAME = "libtrtamd_bert_plugins.so"
MICROBENCH_LIB_NAME = "libtrtamd_microbench.so"   # instruction-rate probes for bench.py; not part of the plugin library
ABLATION_LIB_NAME = "libtrtamd_ablation.so"       # the plugin library with the attention MFMAs left out (timing only)
OBJ_DIR = os.path.join(CSRC, "_obj")

ARCH = "gfx950"
# packed-fp32 code generation is switched off: hipcc -O3 otherwise forms v_pk_*_f32 by itself
COMMON_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}", f"-I{CSRC}", f"-I{os.path.join(CSRC, 'plugin')}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build the library")
    return exe


def sources() -> list[str]:
    pats = ["*.hip", "*.cpp", os.path.join("plugin", "*.cpp"), os.path.join("plugin", "*.hip"),
            os.path.join("runtime", "*.cpp")]
    out: list[str] = []
    for p in pats:
        out += sorted(glob.glob(os.path.join(CSRC, p)))
    return out


def _compile(src: str, extra: tuple = (), suffix: str = "") -> str:
    obj = os.path.join(OBJ_DIR, os.path.relpath(src, CSRC).replace(os.sep, "_") + suffix + ".o")
    cmd = [_hipcc(), *COMMON_FLAGS, *extra, "-x", "hip", "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the AMDGPU feature name and says so; that line is noise
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(jobs: int | None = None, verbose: bool = False) -> str:
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, len(srcs), os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    out = os.path.join(LIB_DIR, LIB_NAME)
    tmp = out + ".tmp"
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs, "-ldl", "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, out)
    if verbose:
        print(f"built {out} from {len(srcs)} sources")
    return out


def build_microbench(verbose: bool = False) -> str:
    """The instruction-rate microbenchmarks (csrc/bench/microbench.hip) as a library of their own."""
    os.makedirs(LIB_DIR, exist_ok=True)
    src = os.path.join(CSRC, "bench", "microbench.hip")
    out = os.path.join(LIB_DIR, MICROBENCH_LIB_NAME)
    tmp = out + ".tmp"
    cmd = [_hipcc(), *COMMON_FLAGS, "-x", "hip", "-shared", src, "-o", tmp]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    os.replace(tmp, out)
    if verbose:
        print(f"built {out}")
    return out


def build_ablation(verbose: bool = False) -> str:
    """A diagnostic copy of the plugin library whose cu_seqlens attention kernels leave their MFMAs out
    (csrc/fused_mha.hip built with -DTRTAMD_ABLATE_ATTENTION_MFMA, every other object as in the plugin library, which
    must have been built): wrong results, and the time the kernels would take if the matrix work were free.
    `python -m tensorrt_amd.kernel_bench --ablation` times it; nothing else loads it."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    fused = os.path.join(CSRC, "fused_mha.hip")
    ablated = _compile(fused, ("-DTRTAMD_ABLATE_ATTENTION_MFMA",), ".ablated")
    plain = os.path.join(OBJ_DIR, os.path.relpath(fused, CSRC).replace(os.sep, "_") + ".o")
    objs = []
    for src in sources():
        obj = os.path.join(OBJ_DIR, os.path.relpath(src, CSRC).replace(os.sep, "_") + ".o")
        if not os.path.exists(obj):
            raise RuntimeError(f"{obj} is missing: build the plugin library first")
        objs.append(ablated if obj == plain else obj)
    out = os.path.join(LIB_DIR, ABLATION_LIB_NAME)
    cmd = [_hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", out + ".tmp", *objs, "-ldl", "-lpthread"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(out + ".tmp", out)
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    build_library(verbose=True)
    build_microbench(verbose=True)
    if "--ablation" in sys.argv[1:]:
        build_ablation(verbose=True)
