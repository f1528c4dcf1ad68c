"""Compile the HIP sources in csrc/ into lazy_amd/_lib/liblazyattn.so for gfx950, and the host helper
csrc/host/callkey.cpp into lazy_amd/_lib/_callkey.so.

Usage: python build.py [--jobs N].  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lazy_amd", "_lib")
LIB = os.path.join(OUT_DIR, "liblazyattn.so")
SOURCES = ["prefill_mfma_bf16.hip", "prefill_mfma_bf16_e4m3.hip", "prefill_mfma_bf16_e5m2.hip", "prefill_mfma_f16.hip",
           "prefill_mfma_f16_e4m3.hip", "prefill_mfma_f16_e5m2.hip", "api.hip", "prefill_generic.hip", "prefill_mfma.hip", "paged_decode.hip", "rope_cache_write.hip", "rotation_metadata.hip", "block_reposition.hip", "rope_table.hip"]
# packed-fp32 VALU forms are kept off on purpose: some have produced wrong results on
# this hardware pool; scalar fp32 code is used throughout.
# No -ffast-math: the fp32 kernel needs IEEE expf/division and every kernel relies on
# infinities; the MFMA kernel asks for hardware exp2 explicitly where it wants it.
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-Wno-inline-asm"]


def _compile(src: str, extra: list[str]) -> str:
    obj = os.path.join(OUT_DIR, src.replace(".hip", ".o"))
    cmd = ["hipcc", *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    subprocess.check_call(cmd)
    return obj


def build_library(jobs: int = 4, extra: list[str] | None = None, verbose: bool = True) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    extra = extra or []
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), SOURCES))
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB])
    if verbose:
        print(f"built {LIB}", file=sys.stderr)
    return LIB


def build_callkey(verbose: bool = True) -> str:
    """The host helper csrc/host/callkey.cpp (a CPython module, no GPU code): g++ against torch's headers."""
    import sysconfig
    from torch.utils import cpp_extension as ce
    import torch
    os.makedirs(OUT_DIR, exist_ok=True)
    out = os.path.join(OUT_DIR, "_callkey.so")
    libdirs = ce.library_paths()
    cmd = ["g++", "-O2", "-shared", "-fPIC", "-std=c++17", "-w",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{d}" for d in ce.include_paths()], f"-I{sysconfig.get_paths()['include']}",
           os.path.join(CSRC, "host", "callkey.cpp"), "-o", out,
           *[f"-L{d}" for d in libdirs], "-ltorch_python", *[f"-Wl,-rpath,{d}" for d in libdirs]]
    subprocess.check_call(cmd)
    if verbose:
        print(f"built {out}", file=sys.stderr)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("--save-temps", action="store_true")
    a = ap.parse_args()
    build_library(a.jobs, ["-save-temps=obj"] if a.save_temps else [])
    build_callkey()
