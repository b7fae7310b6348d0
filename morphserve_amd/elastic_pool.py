"""Elastic KV pool: grow by segments, shrink with on-device migration of live blocks.

Growing and the bookkeeping of a shrink follow the reference
(MorphServe/server/memory_utils.py:369-420 ``update_kvcache_after_replacing_layer``,
:529-544 ``if_kv_cache_unused``, :644-651 tail of ``quant2org_and_update_kvcache``).
The reference refuses to shrink while any block of the tail segment is live
(:623-624); ``shrink_to`` lifts that by relocating live blocks below the cut:
plan (device scan) -> batched block copy -> block-table rewrite -> truncate.
"""
from __future__ import annotations

import ctypes as C
import time
from typing import List, Optional, Tuple

import torch

from . import _capi
from .kv_placement import allocate_kv_caches
from .worker.block_manager import BlockManager
from .worker.kernels import _deferred


class PoolTooFullError(RuntimeError):
    """A shrink was asked for whose live blocks do not fit below the cut; nothing was changed."""


class ElasticKVPool:
    """Base pool ``[num_blocks, L, Hkv, B, D]`` (K and V) plus equally sized
    extension segments, with a ``BlockManager`` over the whole id range."""

    def __init__(self, num_blocks: int, num_layers: int, num_kv_heads: int, block_size: int,
                 head_dim: int, max_seqs_in_block_table: int, max_blocks_per_seq: int,
                 device: str = "cuda", zero_init: bool = True, tune_placement: bool = False,
                 reserve_blocks: int = 0):
        """``tune_placement``: let ``kv_placement.allocate_kv_caches`` time a few starting offsets for the V
        tensor and keep the fastest (off by default).  ``reserve_blocks``: the largest size the pool may grow
        to, when known (the free map is then allocated once)."""
        _capi.lib()
        self.device = torch.device(device)
        self.shape_tail = (num_layers, num_kv_heads, block_size, head_dim)
        # K and V as the reference creates them (model.py:187-190); on request the V base may sit a few KiB
        # into its allocation where the decode gather measures faster that way (kv_placement)
        self.k_cache, self.v_cache, self.kv_placement = allocate_kv_caches(
            num_blocks, self.shape_tail, device, zero_init=zero_init, tune=tune_placement)
        self.k_cache_new: List[torch.Tensor] = []
        self.v_cache_new: List[torch.Tensor] = []
        self.kv_cache_new_block_size = 0
        self.block_manager = BlockManager("GPU", num_blocks, max_seqs_in_block_table,
                                          max_blocks_per_seq, block_size, device=device,
                                          reserve_blocks=reserve_blocks)
        self._result = torch.zeros(4, dtype=torch.int64, device=device)
        self._init_timing()

    def _init_timing(self) -> None:
        # measurement on request: with time_kernels set, the migration copy of a shrink and the zero fill of a
        # growth are bracketed by an event pair on their stream; the elapsed times land in last_migrate_ms /
        # last_fill_ms (the fill's when the caller next reads it: see fill_ms())
        self.time_kernels = False
        self.last_migrate_ms: Optional[float] = None
        self.last_relocate_s: Optional[float] = None     # host time of the last relocation, its final wait included
        self._fill_events: List[Tuple[torch.cuda.Event, torch.cuda.Event]] = []

    def fill_ms(self) -> float:
        """GPU time of the zero fills recorded since the last call (synchronises their events)."""
        total = 0.0
        for e0, e1 in self._fill_events:
            e1.synchronize()
            total += e0.elapsed_time(e1)
        self._fill_events = []
        return total

    def _fill_zero(self, ptr: int, nbytes: int, stream: int) -> None:
        timed = self.time_kernels
        if timed:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
        _capi.check(_capi.lib().mkv_fill_zero(ptr, nbytes, stream))
        if timed:
            e1.record()
            self._fill_events.append((e0, e1))

    # -- description ---------------------------------------------------------------
    @property
    def block_bytes(self) -> int:
        l, h, b, d = self.shape_tail
        return l * h * b * d * 2

    @property
    def num_blocks(self) -> int:
        return self.block_manager.num_blocks

    def descriptor(self) -> _capi.MkvPool:
        return _capi.make_pool(self.k_cache, self.v_cache, self.k_cache_new, self.v_cache_new,
                               num_blocks_org=self.block_manager.num_blocks_org,
                               seg_blocks=self.kv_cache_new_block_size)

    # -- grow ------------------------------------------------------------------------
    def expand(self, seg_blocks: int, k_seg: Optional[torch.Tensor] = None,
               v_seg: Optional[torch.Tensor] = None) -> None:
        """Add one segment of ``seg_blocks`` blocks (all segments share one size).
        The segment memory is given (e.g. views from ``acquire_new_kvcache``) or
        allocated here; either way it is zero filled by the HIP fill kernel."""
        if self.k_cache_new and seg_blocks != self.kv_cache_new_block_size:
            raise ValueError("all extension segments must have the same number of blocks")
        if len(self.k_cache_new) >= _capi.MKV_MAX_SEGMENTS:
            raise RuntimeError(f"at most {_capi.MKV_MAX_SEGMENTS} extension segments")
        lib = _capi.lib()
        stream = _capi.current_stream()
        if k_seg is None:
            shape = (seg_blocks, *self.shape_tail)
            k_seg = torch.empty(shape, dtype=torch.float16, device=self.device)
            off = self.kv_placement["v_offset_bytes"] // 2       # the base pool's K-to-V stagger serves its segments too
            numel = k_seg.numel()
            v_seg = torch.empty(numel + off, dtype=torch.float16, device=self.device)[off:].view(shape)
        assert tuple(k_seg.shape) == (seg_blocks, *self.shape_tail) and k_seg.is_contiguous()
        assert tuple(v_seg.shape) == (seg_blocks, *self.shape_tail) and v_seg.is_contiguous()
        nbytes = seg_blocks * self.block_bytes
        self._fill_zero(k_seg.data_ptr(), nbytes, stream)
        self._fill_zero(v_seg.data_ptr(), nbytes, stream)
        self.k_cache_new.append(k_seg)
        self.v_cache_new.append(v_seg)
        self.kv_cache_new_block_size = seg_blocks
        bm = self.block_manager
        bm.num_blocks += seg_blocks
        bm.num_free_blocks += seg_blocks
        bm.grow_free_map(seg_blocks)

    # -- shrink ------------------------------------------------------------------------
    def tail_segment_unused(self) -> bool:
        """True when no block of the last segment is live."""
        assert self.k_cache_new, "no extension segment to check"
        bm = self.block_manager
        s = self.kv_cache_new_block_size
        lo = bm.num_blocks_org + s * (len(self.k_cache_new) - 1)
        _capi.check(_capi.lib().mkv_bm_count_live(bm.is_block_free.data_ptr(), lo, lo + s,
                                                  self._result.data_ptr(), _capi.current_stream()))
        return int(self._result[0].item()) == 0

    def shrink_tail_if_unused(self) -> bool:
        """The reference's shrink: drop the last segment, refused when it holds a live block."""
        if not self.tail_segment_unused():
            return False
        self._drop_segments(1)
        return True

    def _drop_segments(self, count: int) -> None:
        bm = self.block_manager
        s = self.kv_cache_new_block_size
        for _ in range(count):
            del self.k_cache_new[-1]
            del self.v_cache_new[-1]
            bm.num_blocks -= s
            bm.num_free_blocks -= s
        bm.shrink_free_map(bm.num_blocks)
        if not self.k_cache_new:
            self.kv_cache_new_block_size = 0

    def shrink_to(self, new_num_blocks: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """Shrink to ``new_num_blocks`` (base pool plus a whole number of segments),
        first moving every live block with id >= ``new_num_blocks`` into the lowest
        free ids below it and rewriting the block table.  Returns the move lists
        ``(src, dst)``; raises ``PoolTooFullError`` (state untouched) when the live
        blocks do not fit."""
        bm = self.block_manager
        s = self.kv_cache_new_block_size
        org = bm.num_blocks_org
        if not (org <= new_num_blocks <= bm.num_blocks) or (s and (new_num_blocks - org) % s):
            raise ValueError(f"new size {new_num_blocks} must be {org} + k * {s} and at most {bm.num_blocks}")
        drop = (bm.num_blocks - new_num_blocks) // s if s else 0
        if drop == 0:
            e = torch.empty(0, dtype=torch.int64, device=self.device)
            return e, e
        src, dst = self._relocate_live_blocks(new_num_blocks)
        self._drop_segments(drop)
        return src, dst

    def _relocate_live_blocks(self, new_num_blocks: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """Plan (device scan) -> batched block copy -> block-table rewrite, then wait: when
        this returns no live block has an id >= ``new_num_blocks`` and the memory behind
        those ids is no longer read.  Raises ``PoolTooFullError`` (state untouched) when the
        live blocks do not fit below the cut; a failing launch raises ``MorphKVError``."""
        t_start = time.perf_counter()
        _deferred.flush()
        bm = self.block_manager
        lib = _capi.lib()
        stream = _capi.current_stream()
        cap = bm.num_blocks - new_num_blocks
        src = torch.empty(cap, dtype=torch.int64, device=self.device)
        dst = torch.empty(cap, dtype=torch.int64, device=self.device)
        remap = torch.empty(bm.num_blocks, dtype=torch.int32, device=self.device)
        _capi.check(lib.mkv_pool_plan_shrink(bm.is_block_free.data_ptr(), bm.num_blocks,
                                             new_num_blocks, src.data_ptr(), dst.data_ptr(), cap,
                                             remap.data_ptr(), self._result.data_ptr(), stream))
        moves, status, free_below = self._result[:3].tolist()
        if status != 0:
            raise PoolTooFullError(f"cannot shrink to {new_num_blocks} blocks: {moves} live blocks to move, "
                               f"{free_below} free below the cut")
        events = None
        if moves:
            pool = self.descriptor()
            if self.time_kernels:
                events = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                events[0].record()
            _capi.check(lib.mkv_pool_migrate(C.byref(pool), src.data_ptr(), dst.data_ptr(), moves, stream))
            if events:
                events[1].record()
            _capi.check(lib.mkv_bt_remap(bm.block_table.data_ptr(), bm.block_table.shape[1],
                                         bm.num_seq_allocated_blocks.data_ptr(),
                                         bm.num_seq_allocated_blocks.shape[0], remap.data_ptr(),
                                         bm.num_blocks, stream))
        # the memory above the cut must outlive the copy that reads it
        torch.cuda.current_stream().synchronize()
        self.last_migrate_ms = events[0].elapsed_time(events[1]) if events else None
        self.last_relocate_s = time.perf_counter() - t_start
        return src[:moves], dst[:moves]
