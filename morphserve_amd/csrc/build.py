"""Build the C-ABI HIP libraries in-tree with hipcc for gfx950.

``libmorphkv.so`` is the product: it exports exactly what ``include/morphkv.h`` declares.
``libmorphkv_diag.so`` is its diagnostic twin, built from the same sources with ``-DMKV_DIAG=1``
plus ``diag.hip``: the same entry points and, on top, the switches and measurement hooks of
``include/morphkv_diag.h`` (kernel variants, per-launch event timing, per-workgroup time stamps,
calibration loops).  Benchmarks and tests that need those load the twin; the package never does.

Usage: ``python -m morphserve_amd.csrc.build`` or ``build_library()``.
The shared objects land next to the sources so that they travel with the tree.
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
DIAG_LIB_PATH = os.path.join(HERE, "libmorphkv_diag.so")

SOURCES = [
    "core.hip",
    "kv_append.hip",
    "rope.hip",
    "paged_attn_decode.hip",
    "prefill_attn.hip",
    "block_pool.hip",
    "migrate.hip",
    "vmm_arena.hip",
]
DIAG_SOURCES = SOURCES + ["diag.hip"]

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


def _compile(src: str, obj_dir: str, defines=()) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *defines, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{res.stderr}")
    return obj


def _link(objs, out: str) -> None:
    tmp = out + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC",
           "-Wl,--version-script=" + os.path.join(HERE, "exports.map"), "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, out)


def build_library(verbose: bool = True, jobs: int = 8, diag: bool = True) -> str:
    """Compile every source and link ``libmorphkv.so`` (and, with ``diag``, its diagnostic twin);
    always rebuilds."""
    obj_dir = os.path.join(HERE, "build")
    diag_dir = os.path.join(obj_dir, "diag")
    os.makedirs(diag_dir if diag else obj_dir, exist_ok=True)
    work = [(s, obj_dir, ("-DMKV_DIAG=0",)) for s in SOURCES]
    if diag:
        work += [(s, diag_dir, ("-DMKV_DIAG=1",)) for s in DIAG_SOURCES]
    # the two attention files dominate the build: start them first
    work.sort(key=lambda w: 0 if "attn" in w[0] else 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda w: (w[1], _compile(*w)), work))
    _link([o for d, o in objs if d == obj_dir], LIB_PATH)
    if diag:
        _link([o for d, o in objs if d == diag_dir], DIAG_LIB_PATH)
    if verbose:
        for path in (LIB_PATH, DIAG_LIB_PATH) if diag else (LIB_PATH,):
            print(f"built {path} ({os.path.getsize(path) / 1024:.0f} KiB)")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
