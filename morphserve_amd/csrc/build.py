"""Build libmorphkv.so (the C-ABI HIP library) in-tree with hipcc for gfx950.

Usage: ``python -m morphserve_amd.csrc.build`` or ``build_library()``.
The shared object lands next to the sources so that it travels with the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(ROOT, "include")
LIB_NAME = "libmorphkv.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = [
    "core.hip",
    "kv_append.hip",
    "rope.hip",
    "paged_attn_decode.hip",
    "prefill_attn.hip",
    "block_pool.hip",
    "migrate.hip",
    "vmm_arena.hip",
    "diag.hip",
]

# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE,
    "-I" + HERE,
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the morphkv library cannot be built")
    return exe


def _compile(src: str, obj_dir: str) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stderr}")
    return obj


def build_library(verbose: bool = True, jobs: int = 6) -> str:
    """Compile every source and link ``libmorphkv.so``; always rebuilds."""
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({os.path.getsize(LIB_PATH) / 1024:.0f} KiB)")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
