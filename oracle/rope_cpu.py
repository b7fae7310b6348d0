"""CPU oracle of the rotary embedding step (TEST INFRASTRUCTURE ONLY -- nothing in the
product may import this file).

Restates MorphServe/worker/kernels/rotary_emb.py:7-42 (the kernel body) and
MorphServe/worker/model.py:230-241 (the cos / sin cache).

Rounding.  q, k, cos and sin are all fp16 in the reference, so ``q0*cos - q1*sin`` and
``q0*sin + q1*cos`` are fp16 expressions.  The statement below is one rounded fp16 product
under one fp16 fused multiply-add,
    out0 = fma(q0, cos, -rn16(q1*sin))      out1 = fma(q0, sin, rn16(q1*cos)),
the usual contraction of ``a*b -/+ c*d``.  PARITY UNPINNED for that choice: the reference
kernel is Triton, cannot run here, ships no vectors, and whether its compiler contracts,
and which product it keeps apart, is not visible in its source.  Every candidate (no
contraction, the other product kept apart, fp32 throughout) differs from this one by at
most one fp16 unit in the last place per output; the tests pin index pairing, signs and
table row selection independently and bound the distance to exact arithmetic.
"""
from __future__ import annotations

from typing import Tuple

import numpy as np


def rotary_tables(head_dim: int, max_position_embeddings: int, rope_theta: float = 10000.0,
                  rope_scaling: float = 1.0) -> Tuple[np.ndarray, np.ndarray]:
    """model.py:230-241 in float32: ``[max_position_embeddings * scaling + 128, head_dim / 2]`` fp16."""
    max_seq_len = max_position_embeddings * rope_scaling
    expo = np.arange(0, head_dim, 2, dtype=np.float32) / np.float32(head_dim)
    inv_freq = (np.float32(1.0) / np.power(np.float32(rope_theta), expo, dtype=np.float32)).astype(np.float32)
    t = (np.arange(int(max_seq_len + 128), dtype=np.float32) / np.float32(rope_scaling)).astype(np.float32)
    freqs = np.outer(t, inv_freq).astype(np.float32)
    return np.cos(freqs).astype(np.float16), np.sin(freqs).astype(np.float16)


def _fma16(a: np.ndarray, b: np.ndarray, c: np.ndarray) -> np.ndarray:
    """rn16(a*b + c) for fp16 inputs.  a*b is exact in float64 (22 significant bits); the sum
    is rounded once to float64 and once more to fp16 -- a double rounding that can only differ
    from the single one when c is more than 2^40 times smaller than a*b and a*b sits on an
    fp16 rounding boundary, which the oracle's callers do not produce."""
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float16)


def _mul16(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    return (a.astype(np.float64) * b.astype(np.float64)).astype(np.float16)       # exact product, one rounding


def rotate_rows(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x [T, H, D] fp16, cos / sin [T, D/2] fp16 -> rotated copy (rotary_emb.py:26-42:
    pairs are (d, d + D/2), every head of token t uses row t of the tables)."""
    assert x.dtype == np.float16 and cos.dtype == np.float16 and sin.dtype == np.float16
    half = x.shape[2] // 2
    x0, x1 = x[:, :, :half], x[:, :, half:]
    c, s = cos[:, None, :], sin[:, None, :]
    c = np.broadcast_to(c, x0.shape)
    s = np.broadcast_to(s, x0.shape)
    out = np.empty_like(x)
    out[:, :, :half] = _fma16(x0, c, -_mul16(x1, s))
    out[:, :, half:] = _fma16(x0, s, _mul16(x1, c))
    return out


def rotary_embedding_inplace(q: np.ndarray, k: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> None:
    q[...] = rotate_rows(q, cos, sin)
    k[...] = rotate_rows(k, cos, sin)
