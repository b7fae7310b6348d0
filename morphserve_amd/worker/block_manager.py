"""Device-resident block manager with the reference's interface.

Mirrors ``BlockManager`` of MorphServe/worker/block_manager.py:18-136: same
constructor, attributes and methods, same allocation order (lowest free ids,
ascending, dealt to the batch rows in order), same stale rows after a free.
Each method is one HIP launch plus, where the result's size is data dependent,
one small host read.

That host read is the reference's own (``nonzero``, ``.item()``: block_manager.py:75, block_mgmt.py:116)
and stalls the caller until the stream has drained.  A caller that still HAS the batch as host lists --
the step preparation (MorphServe/worker/model.py:318-368) and ``_swap`` (:468-505) do -- can pass them
as ``seq_ids_host`` / ``target_lens_host``: the manager keeps a host copy of every row's block count,
so the sizes, the free counter and every error check are then computed on the host before the launch
and nothing waits for the GPU.  The results are the same tensors either way.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
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
                 max_blocks_per_seq: int, block_size: int, device: str = "cuda", reserve_blocks: int = 0):
        """``reserve_blocks``: the largest number of blocks the pool may grow to, when known: the free map
        is then allocated once at that size and growing the pool allocates nothing."""
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
        self._free_map_store = torch.ones((max(num_blocks, int(reserve_blocks)),), dtype=torch.bool, device=device)
        self.is_block_free = self._free_map_store[:num_blocks]
        self._result = torch.zeros(4, dtype=torch.int64, device=device)
        # host copy of num_seq_allocated_blocks: exact as long as every change went through a call that was
        # given host lists (or re-read from the device by _host_counts after one that was not)
        self._host_n_alloc = np.zeros(max_seqs_in_block_table, dtype=np.int64)
        self._host_n_alloc_valid = True
        # torch counts the in-place operations on a tensor: a change of that count means that code outside the
        # manager wrote the device counts (a state loaded with copy_, an indexed assignment), and the host
        # copy is re-read; the manager's own kernels write through the raw pointer and do not move it
        self._host_n_alloc_version = self.num_seq_allocated_blocks._version

    # -- the host copy of the rows' block counts ------------------------------------------------------------
    def _host_counts(self) -> np.ndarray:
        version = self.num_seq_allocated_blocks._version
        if not self._host_n_alloc_valid or version != self._host_n_alloc_version:
            # a call without host lists, or code outside the manager, changed the counts: one read back
            self._host_n_alloc = self.num_seq_allocated_blocks.cpu().numpy().astype(np.int64)
            self._host_n_alloc_valid = True
            self._host_n_alloc_version = version
        return self._host_n_alloc

    def invalidate_host_counts(self) -> None:
        """For code that writes ``num_seq_allocated_blocks`` directly (the kernels of ``kernels.block_mgmt``
        called by hand, a state loaded from elsewhere): the host copy is re-read before its next use."""
        self._host_n_alloc_valid = False

    def _host_ids(self, seq_ids_host: Sequence[int]) -> np.ndarray:
        ids = np.asarray(seq_ids_host, dtype=np.int64).reshape(-1)
        if ids.size and (ids.min() < 0 or ids.max() >= self._host_n_alloc.shape[0]):
            raise ValueError(f"(On {self.device_name}) a sequence id is outside the block table")
        return ids

    # -- the free map when the pool grows or shrinks (MorphServe/server/memory_utils.py:409-411, :648) --------
    def grow_free_map(self, num_new_blocks: int) -> None:
        """``is_block_free = cat(is_block_free, ones(num_new_blocks))`` without the reallocation: the map
        is a view of a buffer with spare room; only when that room runs out is a larger buffer (twice the
        size) allocated and the old map copied over, on the device."""
        old = int(self.is_block_free.shape[0])
        new = old + int(num_new_blocks)
        store = self._free_map_store
        if self.is_block_free.data_ptr() != store.data_ptr() or new > store.shape[0]:
            # outside code replaced the map, or the room ran out
            store = torch.empty((max(new, 2 * old),), dtype=torch.bool, device=self.is_block_free.device)
            store[:old].copy_(self.is_block_free)
            self._free_map_store = store
        store[old:new] = True
        self.is_block_free = store[:new]

    def shrink_free_map(self, new_num_blocks: int) -> None:
        """``is_block_free = is_block_free[:new_num_blocks]`` (a view: nothing is copied)."""
        self.is_block_free = self.is_block_free[:int(new_num_blocks)]

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

    def allocate_blocks_for_seqs(self, seq_ids: torch.Tensor, target_lens: torch.Tensor,
                                 seq_ids_host: Optional[Sequence[int]] = None,
                                 target_lens_host: Optional[Sequence[int]] = None) -> torch.Tensor:
        """Ensure sequence ``seq_ids[i]`` owns ``ceil(target_lens[i] / block_size)``
        blocks; returns the newly allocated ids (int64), empty when none were needed.
        With the two host lists (the same values as the tensors) nothing waits for the GPU."""
        assert seq_ids.dtype == torch.int32 and target_lens.dtype == torch.int32
        seq_ids = seq_ids.contiguous()
        target_lens = target_lens.contiguous()
        dev = self.is_block_free.device
        batch = seq_ids.shape[0]
        if seq_ids_host is not None and target_lens_host is not None:
            return self._allocate_from_host_lists(seq_ids, target_lens, seq_ids_host, target_lens_host)
        self._host_n_alloc_valid = False
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

    def _allocate_from_host_lists(self, seq_ids, target_lens, seq_ids_host, target_lens_host) -> torch.Tensor:
        """The same call with every decision taken on the host: the needs come from the host copy of the
        rows' counts, the errors are raised before anything is launched, and the result tensor has its
        final size from the start -- no read back, no wait."""
        dev = self.is_block_free.device
        counts = self._host_counts()
        ids = self._host_ids(seq_ids_host)
        targets = -(-np.asarray(target_lens_host, dtype=np.int64).reshape(-1) // self.block_size)
        if ids.shape[0] != seq_ids.shape[0] or targets.shape[0] != target_lens.shape[0]:
            raise ValueError("the host lists must hold the same values as the tensors")
        if targets.size and targets.max() > self.block_table.shape[1]:
            raise ValueError(f"(On {self.device_name}) a sequence id is outside the block table or a target "
                             f"length needs more than {self.block_table.shape[1]} blocks per sequence")
        need = targets - counts[ids]
        assert not (need < 0).any(), \
            f"(On {self.device_name}) Logic error: Some sequences have more blocks already allocated than needed. seq_ids: {seq_ids_host}, target_lens: {target_lens_host}"
        total = int(need.sum())
        if total > self.num_free_blocks:
            raise RuntimeError(f"No enough free blocks available on {self.device_name} ({self.num_blocks} in total, {self.num_free_blocks} free, {total} requested)")
        if total == 0:
            return torch.empty(0, device=dev, dtype=torch.int64)
        new_ids = torch.empty(total, dtype=torch.int64, device=dev)
        _capi.check(_capi.lib().mkv_bm_allocate(
            self.num_seq_allocated_blocks.data_ptr(), self.num_seq_allocated_blocks.shape[0],
            self.block_table.data_ptr(), self.block_table.shape[1],
            self.is_block_free.data_ptr(), self.is_block_free.shape[0],
            seq_ids.data_ptr(), target_lens.data_ptr(), seq_ids.shape[0], self.block_size,
            new_ids.data_ptr(), total, self._result.data_ptr(), _capi.current_stream()))
        counts[ids] = targets
        self.num_free_blocks -= total
        return new_ids

    def free_blocks_for_seqs(self, seq_ids: torch.Tensor, seq_ids_host: Optional[Sequence[int]] = None) -> None:
        assert seq_ids.dtype == torch.int32
        seq_ids = seq_ids.contiguous()
        if seq_ids_host is not None:                      # the count is known on the host: nothing to read back
            counts = self._host_counts()
            ids = self._host_ids(seq_ids_host)
            unset_block_table_and_num_seq_alloc_blocks(
                self.num_seq_allocated_blocks, self.block_table, seq_ids, self.is_block_free)
            self.num_free_blocks += int(np.minimum(counts[ids], self.block_table.shape[1]).sum())
            counts[ids] = 0
            return
        self._host_n_alloc_valid = False
        unset_block_table_and_num_seq_alloc_blocks(
            self.num_seq_allocated_blocks, self.block_table, seq_ids, self.is_block_free,
            freed_total=self._result[3:4])
        self.num_free_blocks += int(self._result[3].item())

    def gather_allocated_blocks_and_free(self, seq_ids: torch.Tensor,
                                         seq_ids_host: Optional[Sequence[int]] = None) -> torch.Tensor:
        """Ids owned by the sequences (int32, sequence-major) -- they become free."""
        if seq_ids_host is not None:
            counts = self._host_counts()
            ids = self._host_ids(seq_ids_host)
            total = int(np.minimum(counts[ids], self.block_table.shape[1]).sum())
            gathered = gather_allocated_blocks_and_unset(
                self.num_seq_allocated_blocks, self.block_table, seq_ids.contiguous(), self.is_block_free,
                total=total)
            counts[ids] = 0
        else:
            self._host_n_alloc_valid = False
            gathered = gather_allocated_blocks_and_unset(
                self.num_seq_allocated_blocks, self.block_table, seq_ids.contiguous(), self.is_block_free)
        self.num_free_blocks += len(gathered)
        return gathered

    def host_num_allocated_blocks(self, seq_ids_host: Sequence[int]) -> np.ndarray:
        """``get_num_allocated_blocks`` from the host copy (no device read once the copy is valid)."""
        return self._host_counts()[self._host_ids(seq_ids_host)].copy()

    def get_num_allocated_blocks(self, seq_ids: torch.Tensor) -> torch.Tensor:
        return self.num_seq_allocated_blocks[seq_ids.long()]
