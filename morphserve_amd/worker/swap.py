"""Sequence eviction: MorphServe/worker/model.py:468-534 (``_swap``, ``swap_in_seqs``,
``swap_out_seqs``, ``free_seqs_resources``) and the swap space of :195-204.

Flow, as in the reference: block counts of the sequences on the source manager ->
``gather_allocated_blocks_and_free`` there -> ``allocate_blocks_for_seqs`` on the
destination manager -> copy block ``src[i]`` to block ``dst[i]``.  Two differences:
the swap space is PINNED host memory (the reference's is pageable), and the id lists
never leave the device -- the copy is one kernel reading both lists where the reference
does ``.tolist()`` twice and issues a memcpy pair per run of consecutive ids.
``use_kernel=False`` keeps the reference's route (host lists, memcpy runs) for pageable
swap space.

``cpu_tables="host"`` keeps the "CPU" block manager's tables in pinned host memory
(``HostBlockManager``; the reference's live on the GPU, model.py:214-227): its side of a swap is then
plain host work and its id list reaches the copy kernel through a pinned staging buffer.  Measured
against the device-resident manager (``bench.py --workload eviction``) the two are equal within a
percent -- a swap is bound by the PCIe copy, not by either manager -- so the device-resident one
stays the default, as in the reference.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional, Sequence

import torch

from .. import _capi, swiftllm_c
from ..elastic_pool import ElasticKVPool
from .block_manager import BlockManager
from .host_block_manager import HostBlockManager
from .kernels import _deferred


class KVSwapper:
    def __init__(self, pool: ElasticKVPool, num_cpu_blocks: int, cpu_block_manager: Optional[BlockManager] = None,
                 pinned: bool = True, cpu_tables: str = "device"):
        if cpu_tables not in ("device", "host"):
            raise ValueError('cpu_tables must be "device" or "host"')
        bm = pool.block_manager
        self.pool = pool
        self.gpu_block_manager = bm
        if cpu_block_manager is not None:
            self.cpu_block_manager = cpu_block_manager
        elif cpu_tables == "host":
            self.cpu_block_manager = HostBlockManager("CPU", num_cpu_blocks, bm.block_table.shape[0],
                                                      bm.block_table.shape[1], bm.block_size)
        else:
            self.cpu_block_manager = BlockManager("CPU", num_cpu_blocks, bm.block_table.shape[0],
                                                  bm.block_table.shape[1], bm.block_size, device=str(pool.device))
        self._host_tables = isinstance(self.cpu_block_manager, HostBlockManager)
        shape = (num_cpu_blocks, *pool.shape_tail)
        self.k_swap = torch.zeros(shape, dtype=torch.float16, device="cpu", pin_memory=pinned)
        self.v_swap = torch.zeros(shape, dtype=torch.float16, device="cpu", pin_memory=pinned)
        self.pinned = pinned
        self.block_swap = 0          # blocks moved so far (model.py:478)
        # (sequence ids | lengths) of a call travel to the device through pinned staging, two buffers in turn
        rows = bm.block_table.shape[0]
        on_gpu = pool.device.type == "cuda"
        self._stage_host = [torch.empty((2, rows), dtype=torch.int32, pin_memory=on_gpu) for _ in range(2)]
        self._stage_dev = [torch.empty((2, rows), dtype=torch.int32, device=pool.device) for _ in range(2)]
        self._stage_done = [None, None]
        self._stage_turn = 0
        if self._host_tables:                         # the host manager's id lists travel the same way
            self._ids_host = [torch.empty(num_cpu_blocks, dtype=torch.int64, pin_memory=on_gpu) for _ in range(2)]
            self._ids_dev = [torch.empty(num_cpu_blocks, dtype=torch.int64, device=pool.device) for _ in range(2)]
            self._ids_done = [None, None]
            self._ids_turn = 0

    def _stage_ids(self, ids) -> torch.Tensor:
        """A host id list as an int64 device tensor (asynchronous copy from pinned memory)."""
        n = len(ids)
        slot = self._ids_turn
        self._ids_turn ^= 1
        if self._ids_done[slot] is not None:
            self._ids_done[slot].synchronize()
        self._ids_host[slot].numpy()[:n] = ids
        self._ids_dev[slot][:n].copy_(self._ids_host[slot][:n], non_blocking=True)
        if self._ids_dev[slot].is_cuda:
            self._ids_done[slot] = torch.cuda.Event()
            self._ids_done[slot].record()
        return self._ids_dev[slot][:n]

    def _stage(self, ids_host, lens_host):
        """Device views of the two lists, copied asynchronously from pinned memory on the current stream."""
        n = len(ids_host)
        if n > self._stage_host[0].shape[1]:
            raise ValueError("more sequences than the block table has rows")
        slot = self._stage_turn
        self._stage_turn ^= 1
        if self._stage_done[slot] is not None:
            self._stage_done[slot].synchronize()             # the copy that last read this buffer (long finished)
        host, dev = self._stage_host[slot], self._stage_dev[slot]
        host.numpy()[0, :n] = ids_host
        host.numpy()[1, :n] = lens_host
        dev[:, :n].copy_(host[:, :n], non_blocking=True)
        if dev.is_cuda:
            self._stage_done[slot] = torch.cuda.Event()
            self._stage_done[slot].record()
        return dev[0, :n], dev[1, :n]

    def _swap(self, seq_ids_list: Sequence[int], is_swap_in: bool, use_kernel: Optional[bool] = None) -> int:
        if use_kernel is None:
            use_kernel = self.pinned
        if use_kernel and not self.k_swap.is_pinned():       # before any manager state changes
            raise ValueError("the one-kernel route needs a pinned swap space (pinned=True)")
        src_mgr = self.cpu_block_manager if is_swap_in else self.gpu_block_manager
        dst_mgr = self.gpu_block_manager if is_swap_in else self.cpu_block_manager
        ids_host = list(seq_ids_list)
        # block counts from the managers' host copies: the id lists get their sizes without a device read
        # (model.py:481-489 reads them back three times)
        lens_host = src_mgr.host_num_allocated_blocks(ids_host) * self.gpu_block_manager.block_size
        seq_ids, seq_lengths = self._stage(ids_host, lens_host)
        src_host = dst_host = None
        if self._host_tables and is_swap_in:           # the host manager gives, the device manager takes
            src_host = src_mgr.gather_allocated_blocks_and_free(ids_host)
            dst_ids = dst_mgr.allocate_blocks_for_seqs(seq_ids, seq_lengths, seq_ids_host=ids_host,
                                                       target_lens_host=lens_host)
            src_ids = self._stage_ids(src_host) if use_kernel else None
            n = len(src_host)
        elif self._host_tables:
            src_ids = src_mgr.gather_allocated_blocks_and_free(seq_ids, seq_ids_host=ids_host)
            dst_host = dst_mgr.allocate_blocks_for_seqs(ids_host, lens_host)
            dst_ids = self._stage_ids(dst_host) if use_kernel else None
            n = len(dst_host)
        else:
            src_ids = src_mgr.gather_allocated_blocks_and_free(seq_ids, seq_ids_host=ids_host)    # int32, sequence-major
            dst_ids = dst_mgr.allocate_blocks_for_seqs(seq_ids, seq_lengths, seq_ids_host=ids_host,
                                                       target_lens_host=lens_host)             # int64, lowest free ids
            n = int(src_ids.numel())
            assert int(dst_ids.numel()) == n
        self.block_swap += n
        if n == 0:
            return 0
        if use_kernel:
            desc = self.pool.descriptor()
            _deferred.flush()
            _capi.check(_capi.lib().mkv_swap_blocks_device_ids(
                src_ids.to(torch.int64).data_ptr(), dst_ids.data_ptr(), n, 1 if is_swap_in else 0,
                C.byref(desc), self.k_swap.data_ptr(), self.v_swap.data_ptr(), self.k_swap.shape[0],
                _capi.current_stream()))
            # Nothing waits here: the id tensors are torch allocations on this stream, which hands their
            # memory to later work of the same stream only; like the reference's asynchronous copies
            # (block_swapping.cpp:51-80) the blocks have arrived once the stream has reached this point.
        else:
            desc = self.pool.descriptor()
            cnt = C.c_int64(0)
            src_l = src_host.tolist() if src_host is not None else src_ids.tolist()
            dst_l = dst_host.tolist() if dst_host is not None else dst_ids.tolist()
            _capi.check(_capi.lib().mkv_swap_blocks(
                swiftllm_c._ids(src_l), swiftllm_c._ids(dst_l), n, 1 if is_swap_in else 0, C.byref(desc),
                self.k_swap.data_ptr(), self.v_swap.data_ptr(), C.byref(cnt), _capi.current_stream()))
            torch.cuda.current_stream().synchronize()
        return n

    def swap_in_seqs(self, seq_ids_list: List[int], use_kernel: Optional[bool] = None) -> int:
        """CPU swap space -> GPU pool for the given sequences."""
        return self._swap(seq_ids_list, True, use_kernel)

    def swap_out_seqs(self, seq_ids_list: List[int], use_kernel: Optional[bool] = None) -> int:
        """GPU pool -> CPU swap space for the given sequences."""
        return self._swap(seq_ids_list, False, use_kernel)

    def free_seqs_resources(self, seq_ids_list: List[int]) -> None:
        ids_host = list(seq_ids_list)
        seq_ids, _ = self._stage(ids_host, [0] * len(ids_host))
        self.gpu_block_manager.free_blocks_for_seqs(seq_ids, seq_ids_host=ids_host)
        if self._host_tables:
            self.cpu_block_manager.free_blocks_for_seqs(ids_host)
        else:
            self.cpu_block_manager.free_blocks_for_seqs(seq_ids, seq_ids_host=ids_host)
