"""Moves seeded scenarios onto the GPU and reads the state back for bit-exact comparison."""
from __future__ import annotations

import numpy as np
import torch

from helpers import Case, Cfg
from morphserve_amd import BlockManager, build_infer_state


def to_gpu(case: Case, dev):
    k = torch.from_numpy(case.k_pool.copy()).to(dev)
    v = torch.from_numpy(case.v_pool.copy()).to(dev)
    bt = torch.from_numpy(case.block_table.copy()).to(dev)
    return k, v, bt


def configs(case: Case, max_blocks_per_seq=None):
    model = Cfg(num_layers=case.L, num_q_heads=case.Hq, num_kv_heads=case.Hkv, head_dim=case.D)
    engine = Cfg(block_size=case.B, max_blocks_per_seq=max_blocks_per_seq or case.max_blocks_per_seq)
    return model, engine


def load_manager(case: Case, dev) -> BlockManager:
    bm = BlockManager("GPU", case.num_blocks, case.max_seqs, case.max_blocks_per_seq, case.B)
    bm.block_table.copy_(torch.from_numpy(case.block_table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(case.n_alloc))
    bm.is_block_free.copy_(torch.from_numpy(case.is_free))
    bm.num_free_blocks = int(case.is_free.sum())
    return bm


def manager_state(bm: BlockManager) -> dict:
    return dict(block_table=bm.block_table.cpu().numpy(),
                num_seq_allocated_blocks=bm.num_seq_allocated_blocks.cpu().numpy(),
                is_block_free=bm.is_block_free.cpu().numpy(),
                num_blocks=int(bm.num_blocks), num_free_blocks=int(bm.num_free_blocks))


def assert_state_equal(got: dict, want: dict, what=""):
    for key in want:
        assert np.array_equal(got[key], want[key]), f"{what}: {key} differs"


def bits(t) -> np.ndarray:
    """fp16 tensor / array -> uint16 bit patterns (NaN-safe, sign-of-zero-exact compare)."""
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t).view(np.uint16)
