"""Seeded scenario builders shared by the CPU (oracle) and GPU (parity) tests."""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence

import numpy as np

from oracle import ref_cpu as R


class Cfg:
    """Duck-typed stand-in for the reference's model / engine config objects."""

    def __init__(self, **kw):
        self.__dict__.update(kw)


@dataclasses.dataclass
class Case:
    L: int
    Hq: int
    Hkv: int
    B: int
    D: int
    num_blocks: int
    max_seqs: int
    max_blocks_per_seq: int
    seq_ids: np.ndarray          # [n] int32
    seq_lens: np.ndarray         # [n] int32
    block_table: np.ndarray      # [max_seqs, max_blocks_per_seq] int32
    n_alloc: np.ndarray          # [max_seqs] int32
    is_free: np.ndarray          # [num_blocks] bool
    arena: np.ndarray            # flat fp16: K pool then V pool
    lay: R.PoolLayout

    @property
    def k_pool(self):
        n = self.num_blocks * self.lay.block_elems
        return self.arena[:n].reshape(self.num_blocks, self.L, self.Hkv, self.B, self.D)

    @property
    def v_pool(self):
        n = self.num_blocks * self.lay.block_elems
        return self.arena[n:2 * n].reshape(self.num_blocks, self.L, self.Hkv, self.B, self.D)


def make_case(seed: int, L: int, Hq: int, Hkv: int, lens: Sequence[int], num_blocks: int,
              B: int = 16, D: int = 128, max_seqs: Optional[int] = None,
              max_blocks_per_seq: Optional[int] = None, permute: bool = True,
              fill: str = "live") -> Case:
    """Sequences with the given lengths own blocks dealt from a seeded permutation
    of the pool (``permute=False``: ascending ids).  ``fill='live'`` puts N(0,1)
    values in the owned blocks and zeros elsewhere; ``'all'`` fills every block."""
    rng = np.random.default_rng(seed)
    n = len(lens)
    lens = np.asarray(lens, dtype=np.int32)
    max_seqs = max_seqs or max(2 * n, 4)
    need = (lens.astype(np.int64) + B - 1) // B
    max_blocks_per_seq = max_blocks_per_seq or int(max(need.max(initial=1) + 2, 4))
    assert need.sum() <= num_blocks
    order = rng.permutation(num_blocks) if permute else np.arange(num_blocks)
    seq_ids = rng.permutation(max_seqs)[:n].astype(np.int32)
    table = np.full((max_seqs, max_blocks_per_seq), -1, dtype=np.int32)
    n_alloc = np.zeros(max_seqs, dtype=np.int32)
    is_free = np.ones(num_blocks, dtype=bool)
    pos = 0
    for i in range(n):
        ids = order[pos:pos + need[i]]
        pos += need[i]
        table[seq_ids[i], :need[i]] = ids
        n_alloc[seq_ids[i]] = need[i]
        is_free[ids] = False
    lay = R.plain_layout(num_blocks, L, Hkv, B, D)
    arena = np.zeros(2 * num_blocks * lay.block_elems, dtype=np.float16)
    if fill == "all":
        arena[:] = rng.standard_normal(arena.shape[0], dtype=np.float32).astype(np.float16)
    else:
        live = np.nonzero(~is_free)[0]
        for which in ("k", "v"):
            for b in live:
                o = lay.block_offset(which, int(b))
                arena[o:o + lay.block_elems] = rng.standard_normal(lay.block_elems, dtype=np.float32).astype(np.float16)
    return Case(L, Hq, Hkv, B, D, num_blocks, max_seqs, max_blocks_per_seq, seq_ids, lens,
                table, n_alloc, is_free, arena, lay)


def rand_f16(rng, *shape):
    return rng.standard_normal(shape, dtype=np.float32).astype(np.float16)


def attn_err(got: np.ndarray, want: np.ndarray):
    """(max abs error, max of abs error / max(|want|, 1)) in float64."""
    g = got.astype(np.float64)
    w = want.astype(np.float64)
    ae = np.abs(g - w)
    return float(ae.max(initial=0.0)), float((ae / np.maximum(np.abs(w), 1.0)).max(initial=0.0))


# The attention tolerance of the path: fp16 output, fp32 accumulation.  Both bounds hold together:
# every element within ATTN_MAX_ABS of the oracle, and -- where the oracle's value is large enough for
# a relative error to mean something (|want| >= ATTN_REL_FLOOR; below it the absolute bound is the
# tighter one, 2e-3 / 0.2 = 1e-2) -- within ATTN_MAX_REL of it as well.
ATTN_MAX_ABS = 2e-3
ATTN_MAX_REL = 1e-2
ATTN_REL_FLOOR = 0.2


def assert_attn_close(got: np.ndarray, want: np.ndarray, what: str = "", report: bool = False):
    g = got.astype(np.float64)
    w = want.astype(np.float64)
    assert np.isfinite(g).all(), f"{what}: non-finite output"
    ae = np.abs(g - w)
    big = np.abs(w) >= ATTN_REL_FLOOR
    max_abs = float(ae.max(initial=0.0))
    max_rel = float((ae[big] / np.abs(w[big])).max(initial=0.0))
    if report:
        print(f"[attn parity] {what}: max abs err {max_abs:.3e}, max rel err (|want| >= {ATTN_REL_FLOOR}) {max_rel:.3e}")
    assert max_abs <= ATTN_MAX_ABS, f"{what}: max abs err {max_abs:.3e} > {ATTN_MAX_ABS}"
    assert max_rel <= ATTN_MAX_REL, f"{what}: max rel err {max_rel:.3e} > {ATTN_MAX_REL} (max abs {max_abs:.3e})"
    return max_abs, max_rel
