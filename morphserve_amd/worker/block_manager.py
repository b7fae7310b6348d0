"""Device-resident block manager with the reference's interface.

Mirrors ``BlockManager`` of MorphServe/worker/block_manager.py:18-136: same
constructor, attributes and methods, same allocation order (lowest free ids,
ascending, dealt to the batch rows in order), same stale rows after a free.
Each method is one HIP launch plus, where the result's size is data dependent,
one small host read.
"""
from __future__ import annotations

import torch

from .. import _capi
from .kernels.block_mgmt import (gather_allocated_blocks_and_unset,
                                 set_block_table_and_num_seq_alloc_blocks,
                                 unset_block_table_and_num_seq_alloc_blocks)


class BlockCount(int):
    """An ``int`` that also answers ``.item()``: callers of the reference use the
    free-block counter both ways (MorphServe/server/engine.py:239,
    MorphServe/server/scheduler.py:83)."""

    def item(self) -> int:
        return int(self)

    def __add__(self, other):
        return BlockCount(int(self) + int(other))

    __radd__ = __add__

    def __sub__(self, other):
        return BlockCount(int(self) - int(other))

    def __rsub__(self, other):
        return BlockCount(int(other) - int(self))


class BlockManager:
    """``block_table`` (seq, logical block) -> block id, ``num_seq_allocated_blocks``
    and the ``is_block_free`` map live on the GPU; ``num_blocks`` /
    ``num_free_blocks`` are host counters that outside code may adjust when the
    pool grows or shrinks."""

    def __init__(self, device_name: str, num_blocks: int, max_seqs_in_block_table: int,
                 max_blocks_per_seq: int, block_size: int, device: str = "cuda"):
        _capi.lib()
        self.device_name = device_name
        self._num_free_blocks = BlockCount(num_blocks)
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.num_free_blocks_org = num_blocks
        self.num_blocks_org = num_blocks

        self.num_seq_allocated_blocks = torch.zeros((max_seqs_in_block_table,), dtype=torch.int32, device=device)
        self.block_table = torch.full((max_seqs_in_block_table, max_blocks_per_seq), -1,
                                      dtype=torch.int32, device=device)
        self.is_block_free = torch.ones((num_blocks,), dtype=torch.bool, device=device)
        self._result = torch.zeros(4, dtype=torch.int64, device=device)

    # the counter stays usable as a number and through .item() whatever is assigned to it
    @property
    def num_free_blocks(self) -> BlockCount:
        return self._num_free_blocks

    @num_free_blocks.setter
    def num_free_blocks(self, value) -> None:
        self._num_free_blocks = BlockCount(int(value))

    def get_num_used_blocks(self) -> int:
        return self.num_blocks - self.num_free_blocks

    def _allocate_blocks(self, num_blocks: int) -> torch.Tensor:
        """The ``num_blocks`` lowest free ids, ascending; marks them used."""
        num_blocks = int(num_blocks)
        if num_blocks > self.num_free_blocks:
            raise RuntimeError(f"No enough free blocks available on {self.device_name} ({self.num_blocks} in total, {self.num_free_blocks} free, {num_blocks} requested)")
        out = torch.empty(num_blocks, dtype=torch.int64, device=self.is_block_free.device)
        _capi.check(_capi.lib().mkv_bm_take_first_free(
            self.is_block_free.data_ptr(), self.is_block_free.shape[0], num_blocks,
            out.data_ptr(), self._result.data_ptr(), _capi.current_stream()))
        found, status = self._result[:2].tolist()
        if status != 0:
            raise RuntimeError(f"No enough free blocks available on {self.device_name} ({self.num_blocks} in total, {found} free in the map, {num_blocks} requested)")
        self.num_free_blocks -= num_blocks
        return out

    def _free_blocks(self, block_ids: torch.Tensor) -> None:
        self.num_free_blocks += len(block_ids)
        self.is_block_free[block_ids] = True

    def allocate_blocks_for_seqs(self, seq_ids: torch.Tensor, target_lens: torch.Tensor) -> torch.Tensor:
        """Ensure sequence ``seq_ids[i]`` owns ``ceil(target_lens[i] / block_size)``
        blocks; returns the newly allocated ids (int64), empty when none were needed."""
        assert seq_ids.dtype == torch.int32 and target_lens.dtype == torch.int32
        seq_ids = seq_ids.contiguous()
        target_lens = target_lens.contiguous()
        dev = self.is_block_free.device
        batch = seq_ids.shape[0]
        upper = min(int(self.is_block_free.shape[0]), batch * self.block_table.shape[1])
        new_ids = torch.empty(max(upper, 1), dtype=torch.int64, device=dev)
        # the kernel refuses (and modifies nothing) when the request exceeds this capacity: bounding it by
        # the host's free counter keeps the device state untouched whenever the call is going to raise
        cap = min(new_ids.shape[0], int(self.num_free_blocks))
        _capi.check(_capi.lib().mkv_bm_allocate(
            self.num_seq_allocated_blocks.data_ptr(), self.num_seq_allocated_blocks.shape[0],
            self.block_table.data_ptr(), self.block_table.shape[1],
            self.is_block_free.data_ptr(), self.is_block_free.shape[0],
            seq_ids.data_ptr(), target_lens.data_ptr(), batch, self.block_size,
            new_ids.data_ptr(), cap, self._result.data_ptr(), _capi.current_stream()))
        total, status, found = self._result[:3].tolist()
        if status == _capi.MKV_EINVAL:
            raise ValueError(f"(On {self.device_name}) a sequence id is outside the block table or a target "
                             f"length needs more than {self.block_table.shape[1]} blocks per sequence")
        assert status != _capi.MKV_ELOGIC, \
            f"(On {self.device_name}) Logic error: Some sequences have more blocks already allocated than needed. seq_ids: {seq_ids}, target_lens: {target_lens}"
        if status == _capi.MKV_ENOSPC:
            raise RuntimeError(f"No enough free blocks available on {self.device_name} ({self.num_blocks} in total, {self.num_free_blocks} free, {total} requested)")
        if total == 0:
            return torch.empty(0, device=dev, dtype=torch.int64)
        self.num_free_blocks -= total
        return new_ids[:total]

    def free_blocks_for_seqs(self, seq_ids: torch.Tensor) -> None:
        assert seq_ids.dtype == torch.int32
        seq_ids = seq_ids.contiguous()
        unset_block_table_and_num_seq_alloc_blocks(
            self.num_seq_allocated_blocks, self.block_table, seq_ids, self.is_block_free,
            freed_total=self._result[3:4])
        self.num_free_blocks += int(self._result[3].item())

    def gather_allocated_blocks_and_free(self, seq_ids: torch.Tensor) -> torch.Tensor:
        """Ids owned by the sequences (int32, sequence-major) -- they become free."""
        gathered = gather_allocated_blocks_and_unset(
            self.num_seq_allocated_blocks, self.block_table, seq_ids.contiguous(), self.is_block_free)
        self.num_free_blocks += len(gathered)
        return gathered

    def get_num_allocated_blocks(self, seq_ids: torch.Tensor) -> torch.Tensor:
        return self.num_seq_allocated_blocks[seq_ids.long()]
