"""A block manager whose tables live in (pinned) host memory.

The reference creates its "CPU" block manager -- the one that hands out blocks of the host swap space --
with GPU tensors like the other one (MorphServe/worker/model.py:214-227), and every eviction reads its
results back (:481-489).  The swap space is host memory and the sequences to move arrive as host lists,
so this manager keeps ``block_table``, ``num_seq_allocated_blocks`` and ``is_block_free`` on the host and
does its few operations there, in the reference's order (lowest free ids ascending, dealt to the batch
rows in order; stale rows after a free: MorphServe/worker/block_manager.py:64-129).  Same attribute and
method names as ``BlockManager``; ids come back as host arrays.
"""
from __future__ import annotations

from typing import Sequence

import numpy as np
import torch

from .block_manager import BlockCount


class HostBlockManager:
    def __init__(self, device_name: str, num_blocks: int, max_seqs_in_block_table: int, max_blocks_per_seq: int,
                 block_size: int, pinned: bool = True):
        self.device_name = device_name
        self._num_free_blocks = BlockCount(num_blocks)
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.num_free_blocks_org = num_blocks
        self.num_blocks_org = num_blocks
        pin = bool(pinned and torch.cuda.is_available())
        self.num_seq_allocated_blocks = torch.zeros((max_seqs_in_block_table,), dtype=torch.int32, pin_memory=pin)
        self.block_table = torch.full((max_seqs_in_block_table, max_blocks_per_seq), -1, dtype=torch.int32,
                                      pin_memory=pin)
        self.is_block_free = torch.ones((num_blocks,), dtype=torch.bool, pin_memory=pin)
        self._n_alloc = self.num_seq_allocated_blocks.numpy()
        self._table = self.block_table.numpy()
        self._free = self.is_block_free.numpy()
        self._first_maybe_free = 0          # no free id lies below this one

    @property
    def num_free_blocks(self) -> BlockCount:
        return self._num_free_blocks

    @num_free_blocks.setter
    def num_free_blocks(self, value) -> None:
        self._num_free_blocks = BlockCount(int(value))

    def get_num_used_blocks(self) -> int:
        return self.num_blocks - self.num_free_blocks

    def _ids(self, seq_ids: Sequence[int]) -> np.ndarray:
        ids = np.asarray(seq_ids, dtype=np.int64).reshape(-1)
        if ids.size and (ids.min() < 0 or ids.max() >= self._n_alloc.shape[0]):
            raise ValueError(f"(On {self.device_name}) a sequence id is outside the block table")
        return ids

    def allocate_blocks_for_seqs(self, seq_ids: Sequence[int], target_lens: Sequence[int]) -> np.ndarray:
        """Newly allocated ids (int64, ascending), dealt to the rows in batch order."""
        ids = self._ids(seq_ids)
        targets = -(-np.asarray(target_lens, dtype=np.int64).reshape(-1) // self.block_size)
        if targets.size and targets.max() > self._table.shape[1]:
            raise ValueError(f"(On {self.device_name}) a target length needs more than {self._table.shape[1]} "
                             "blocks per sequence")
        have = self._n_alloc[ids].astype(np.int64)
        need = targets - have
        assert not (need < 0).any(), \
            f"(On {self.device_name}) Logic error: Some sequences have more blocks already allocated than needed."
        total = int(need.sum())
        if total > self.num_free_blocks:
            raise RuntimeError(f"No enough free blocks available on {self.device_name} ({self.num_blocks} in total, "
                               f"{self.num_free_blocks} free, {total} requested)")
        if total == 0:
            return np.empty(0, dtype=np.int64)
        lo = self._first_maybe_free
        new = lo + np.flatnonzero(self._free[lo:])[:total]
        assert len(new) == total, "the free counter and the free map disagree"
        self._free[new] = False
        self._first_maybe_free = int(new[-1]) + 1
        start = 0
        for row, h, n in zip(ids, have, need):
            if n:
                self._table[row, h:h + n] = new[start:start + n]
                self._n_alloc[row] = h + n
                start += n
        self.num_free_blocks -= total
        return new.astype(np.int64)

    def gather_allocated_blocks_and_free(self, seq_ids: Sequence[int]) -> np.ndarray:
        """Ids owned by the sequences (int32, sequence-major); they become free, the rows keep their entries."""
        ids = self._ids(seq_ids)
        parts = [self._table[row, :self._n_alloc[row]] for row in ids]
        out = np.concatenate(parts).astype(np.int32) if parts else np.empty(0, dtype=np.int32)
        if out.size:
            self._free[out] = True
            self._first_maybe_free = min(self._first_maybe_free, int(out.min()))
        self._n_alloc[ids] = 0
        self.num_free_blocks += len(out)
        return out

    def free_blocks_for_seqs(self, seq_ids: Sequence[int]) -> None:
        self.gather_allocated_blocks_and_free(seq_ids)

    def get_num_allocated_blocks(self, seq_ids: Sequence[int]) -> np.ndarray:
        return self._n_alloc[self._ids(seq_ids)].copy()

    host_num_allocated_blocks = get_num_allocated_blocks
