"""Compile the oracle's C restatement (``oracle/oracle.c``) with gcc.

TEST INFRASTRUCTURE ONLY.  The reference's own native sources
(csrc/src/block_swapping.cpp, memory_manager.cpp) include <torch/extension.h>
and <cuda_runtime.h> and call cudaMemcpyAsync; without a CUDA toolkit they do
not compile here, so no ``oracle/_ref`` build exists and the oracle is pinned
by the checks listed in ``oracle/ref_cpu.py``.
"""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")


def build_oracle(verbose: bool = True) -> str:
    cmd = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-o", LIB_PATH + ".tmp",
           os.path.join(HERE, "oracle.c"), "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"gcc failed for oracle.c:\n{res.stderr}")
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_oracle()
