"""KV pool backed by HIP virtual memory: one contiguous ``[num_blocks, L, Hkv, B, D]``
tensor (K, and one for V) that grows and shrinks in place.

The reference grows its pool with extra tensors carved from freed weight memory
(MorphServe/server/memory_utils.py:369-420) and can only drop the last of them when it
is empty (:529-544, :617-651); every kernel then needs the segment arithmetic of
MorphServe/worker/kernels/kvcache_mgmt.py:169-183.  Here the address range of the
largest pool is reserved once and physical memory is mapped at its end chunk by chunk:
block ids are plain indices, ``k_cache_new`` stays empty, growing copies nothing, and a
shrink first relocates the live blocks above the cut (as ``ElasticKVPool.shrink_to``).
Same ``BlockManager`` and bookkeeping as ``ElasticKVPool``.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional, Tuple

import torch

from . import _capi
from .elastic_pool import ElasticKVPool
from .swiftllm_c import _RawDeviceMemory
from .worker.block_manager import BlockManager


class _Arena:
    def __init__(self, reserve_bytes: int, chunk_bytes: int):
        self.handle = C.c_void_p()
        _capi.check(_capi.lib().mkv_arena_create(reserve_bytes, chunk_bytes, C.byref(self.handle)))
        base = C.c_void_p()
        _capi.check(_capi.lib().mkv_arena_info(self.handle, C.byref(base), None, None, None))
        self.base = int(base.value)

    def resize(self, mapped_bytes: int) -> None:
        rc = _capi.lib().mkv_arena_resize(self.handle, mapped_bytes)
        if rc == _capi.MKV_ENOSPC:
            raise MemoryError("the device has no memory left for the pool to grow")
        _capi.check(rc)

    def mapped_bytes(self) -> int:
        n = C.c_uint64(0)
        _capi.check(_capi.lib().mkv_arena_info(self.handle, None, None, None, C.byref(n)))
        return int(n.value)

    def move_tail_to(self, other: "_Arena", nbytes: int) -> None:
        """Hand the physical memory behind the last ``nbytes`` mapped here over to the end of ``other``."""
        _capi.check(_capi.lib().mkv_arena_move_tail(self.handle, other.handle, nbytes))

    def close(self) -> None:
        if self.handle:
            _capi.check(_capi.lib().mkv_arena_destroy(self.handle))
            self.handle = C.c_void_p()


class LayerArena(_Arena):
    """Device memory of one replaceable transformer layer, in chunks a ``VmmKVPool`` can take over.

    The reference keeps a layer's fp16 weights in one range, copies the quantized twin to the START of that
    range when the layer is replaced and turns the rest into KV tensors (csrc/src/memory_manager.cpp:69-176);
    restoring the layer copies the fp16 weights back from the host (memory_utils.py:635).  Here the range is
    an arena of ``nbytes`` rounded up to whole chunks, all mapped; ``VmmKVPool.expand_from`` moves the chunks
    behind ``keep_bytes`` to the end of the pool and ``VmmKVPool.shrink_into`` brings them back."""

    def __init__(self, nbytes: int, chunk_bytes: int, device: str = "cuda"):
        self.chunk_bytes = chunk_bytes
        self.capacity = -(-nbytes // chunk_bytes) * chunk_bytes
        super().__init__(self.capacity, chunk_bytes)
        self.device = torch.device(device, torch.cuda.current_device()) if device == "cuda" else torch.device(device)
        try:
            self.resize(self.capacity)
        except Exception:
            self.close()
            raise

    def tensor(self, offset_bytes: int, shape, dtype=torch.float16) -> torch.Tensor:
        """A tensor over ``[offset_bytes, offset_bytes + size)`` of the arena; the range must be mapped for
        as long as the tensor is used."""
        shape = tuple(int(x) for x in shape)
        nbytes = torch.empty((), dtype=dtype).element_size()
        for x in shape:
            nbytes *= x
        if offset_bytes < 0 or offset_bytes + nbytes > self.mapped_bytes():
            raise ValueError(f"[{offset_bytes}, {offset_bytes + nbytes}) is outside the {self.mapped_bytes()} mapped bytes")
        typestrs = {torch.float16: "<f2", torch.uint8: "|u1", torch.int8: "|i1", torch.int32: "<i4", torch.float32: "<f4"}
        if dtype not in typestrs:
            raise ValueError(f"{dtype}: take a uint8 tensor and .view() it")
        typestr = typestrs[dtype]
        return torch.as_tensor(_RawDeviceMemory(self.base + offset_bytes, shape, self, typestr), device=self.device)


class VmmKVPool(ElasticKVPool):
    """``num_blocks`` blocks now, room for ``max_blocks``; sizes move in multiples of
    ``chunk_blocks`` (one physical allocation per chunk and per tensor; a chunk above 2 MiB must be a
    multiple of 2 MiB, the library refuses others).

    ``placement="groups"`` (the default) lets ``mkv_arena_pair_grow`` choose the physical memory: K chunks
    from one memory group of the device and V chunks from another, told apart by a store-rate measurement
    at creation and at every growth (chunks of 256 MiB per tensor and more; smaller ones cannot be measured
    and grow in the driver's order).  ``placement="plain"`` always takes the driver's order."""

    def __init__(self, num_blocks: int, max_blocks: int, num_layers: int, num_kv_heads: int, block_size: int,
                 head_dim: int, max_seqs_in_block_table: int, max_blocks_per_seq: int, chunk_blocks: int = 64,
                 device: str = "cuda", v_stagger_bytes: int = 0, placement: str = "groups",
                 placement_budget_bytes: int = 0):
        """``v_stagger_bytes``: how far into its range the V tensor starts (a multiple of 4 KiB below the chunk
        size; it costs one more mapped chunk).  ``placement_budget_bytes``: the most device memory a growth may
        hold at once while it looks for chunks of the right groups (0: all that is free but 4 GiB)."""
        _capi.lib()
        if placement not in ("groups", "plain"):
            raise ValueError('placement must be "groups" or "plain"')
        self.device = torch.device(device, torch.cuda.current_device()) if device == "cuda" else torch.device(device)
        self.shape_tail = (num_layers, num_kv_heads, block_size, head_dim)
        self.chunk_blocks = chunk_blocks
        if num_blocks % chunk_blocks or max_blocks % chunk_blocks or not 0 < num_blocks <= max_blocks:
            raise ValueError(f"num_blocks and max_blocks must be multiples of chunk_blocks ({chunk_blocks})")
        self.max_blocks = max_blocks
        chunk = chunk_blocks * self.block_bytes
        if v_stagger_bytes < 0 or v_stagger_bytes % 4096 or v_stagger_bytes >= chunk:
            raise ValueError("v_stagger_bytes must be a multiple of 4096 below the chunk size")
        self.placement = placement
        self.placement_budget_bytes = int(placement_budget_bytes)
        self._v_off = int(v_stagger_bytes)
        self._v_pad = chunk if self._v_off else 0            # the V range is mapped one chunk further
        self._k_arena = _Arena(max_blocks * self.block_bytes, chunk)
        self._v_arena = _Arena(max_blocks * self.block_bytes + self._v_pad, chunk)
        self.k_cache_new, self.v_cache_new = [], []          # never used: the pool is one tensor
        self.kv_cache_new_block_size = 0
        self.kv_placement: Dict = {"v_offset_bytes": self._v_off, "placement": placement, "growths": []}
        self.block_manager = BlockManager("GPU", num_blocks, max_seqs_in_block_table, max_blocks_per_seq,
                                          block_size, device=device, reserve_blocks=max_blocks)
        self._result = torch.zeros(4, dtype=torch.int64, device=device)
        self._init_timing()
        self._map(num_blocks)
        self._zero(0, num_blocks)

    # -- mapping ---------------------------------------------------------------------
    def _map(self, num_blocks: int) -> None:
        """Map (or unmap) so that both tensors hold ``num_blocks`` blocks."""
        nbytes = num_blocks * self.block_bytes
        k_have, v_have = self._k_arena.mapped_bytes(), self._v_arena.mapped_bytes()
        k_add, v_add = nbytes - k_have, nbytes + self._v_pad - v_have
        if self.placement == "groups" and k_add > 0 and v_add > 0:
            info = _capi.MkvPairInfo()
            rc = _capi.lib().mkv_arena_pair_grow(self._k_arena.handle, self._v_arena.handle, k_add, v_add,
                                                 self.placement_budget_bytes, _capi.current_stream(), C.byref(info))
            if rc == _capi.MKV_ENOSPC:
                raise MemoryError("the device has no memory left for the pool to grow")
            _capi.check(rc)
            self.kv_placement["growths"].append({f: getattr(info, f) for f, _ in info._fields_ if f != "_pad"})
        else:
            self._k_arena.resize(nbytes)
            try:
                self._v_arena.resize(nbytes + self._v_pad)
            except Exception:
                self._k_arena.resize(k_have)
                raise
        self._make_views(num_blocks)

    def _make_views(self, num_blocks: int) -> None:
        shape = (num_blocks, *self.shape_tail)
        self.k_cache = torch.as_tensor(_RawDeviceMemory(self._k_arena.base, shape, self._k_arena), device=self.device)
        self.v_cache = torch.as_tensor(_RawDeviceMemory(self._v_arena.base + self._v_off, shape, self._v_arena),
                                       device=self.device)

    def _zero(self, first: int, count: int) -> None:
        stream = _capi.current_stream()
        off, nbytes = first * self.block_bytes, count * self.block_bytes
        self._fill_zero(self._k_arena.base + off, nbytes, stream)
        self._fill_zero(self._v_arena.base + self._v_off + off, nbytes, stream)

    def descriptor(self) -> _capi.MkvPool:
        return _capi.make_pool(self.k_cache, self.v_cache)

    # -- grow / shrink ---------------------------------------------------------------
    def expand(self, num_new_blocks: int, k_seg=None, v_seg=None) -> None:
        """Map ``num_new_blocks`` more blocks at the end (zero filled, all free)."""
        assert k_seg is None and v_seg is None, "a virtual-memory pool maps its own memory"
        bm = self.block_manager
        if num_new_blocks <= 0 or num_new_blocks % self.chunk_blocks:
            raise ValueError(f"the pool grows in multiples of {self.chunk_blocks} blocks")
        if bm.num_blocks + num_new_blocks > self.max_blocks:
            raise ValueError(f"at most {self.max_blocks} blocks were reserved")
        self._map(bm.num_blocks + num_new_blocks)
        self._grew_by(num_new_blocks)

    def _grew_by(self, num_new_blocks: int) -> None:
        bm = self.block_manager
        old = bm.num_blocks
        self._zero(old, num_new_blocks)
        bm.num_blocks += num_new_blocks
        bm.num_free_blocks += num_new_blocks
        bm.grow_free_map(num_new_blocks)

    def blocks_available_from(self, donor: "LayerArena", keep_bytes: int) -> int:
        """How many blocks ``expand_from(donor, keep_bytes)`` would add: the donor's mapped chunks behind
        ``keep_bytes`` split evenly between K and V, capped by the reservation."""
        if donor.chunk_bytes != self.chunk_blocks * self.block_bytes:
            raise ValueError("the donor's chunks must have the pool's chunk size")
        keep_chunks = -(-keep_bytes // donor.chunk_bytes)
        free_chunks = donor.mapped_bytes() // donor.chunk_bytes - keep_chunks
        room = (self.max_blocks - self.block_manager.num_blocks) // self.chunk_blocks
        return max(0, min(free_chunks // 2, room)) * self.chunk_blocks

    def expand_from(self, donor: "LayerArena", keep_bytes: int) -> int:
        """Grow by the memory ``donor`` no longer needs once its first ``keep_bytes`` hold the quantized
        layer (``acquire_new_kvcache``, csrc/src/memory_manager.cpp:69-176, followed by
        ``update_kvcache_after_replacing_layer``, memory_utils.py:369-420): the donor's chunks behind
        ``keep_bytes`` move to the end of K and of V (half each), are zero filled and join the free map.
        Nothing is allocated or copied.  Returns the number of new blocks (0: nothing to take)."""
        n = self.blocks_available_from(donor, keep_bytes)
        if n == 0:
            return 0
        nbytes = n * self.block_bytes
        torch.cuda.synchronize(self.device)                          # nothing may still use the donor's tail
        have = self.block_manager.num_blocks
        k_had, v_had = self._k_arena.mapped_bytes(), self._v_arena.mapped_bytes()
        self.k_cache = self.v_cache = None
        try:
            donor.move_tail_to(self._k_arena, nbytes)
            donor.move_tail_to(self._v_arena, nbytes)
        except Exception:
            # a move stops at the chunk that failed and leaves the earlier ones moved: hand back whatever
            # either tensor received, so that the pool and the donor are as they were
            self._give_back(donor, k_had, v_had)
            self._make_views(have)
            raise
        self._make_views(have + n)
        self._grew_by(n)
        return n

    def _give_back(self, donor: "LayerArena", k_had: int, v_had: int) -> None:
        """Return to ``donor`` the chunks the two arenas hold beyond ``k_had`` / ``v_had`` mapped bytes (V's
        first, the reverse of the order they were taken in).  Best effort: a second failure is left to the
        caller's exception."""
        for arena, had in ((self._v_arena, v_had), (self._k_arena, k_had)):
            extra = arena.mapped_bytes() - had
            if extra > 0:
                try:
                    arena.move_tail_to(donor, extra)
                except Exception:
                    pass

    def shrink_into(self, donor: "LayerArena", new_num_blocks: int) -> Tuple[torch.Tensor, torch.Tensor]:
        """``shrink_to(new_num_blocks)`` with the memory above the cut handed back to ``donor`` instead of
        the driver (the restored layer's weights are copied there next, memory_utils.py:635)."""
        return self.shrink_to(new_num_blocks, donor)

    def tail_unused(self, num_blocks: int) -> bool:
        """True when none of the last ``num_blocks`` blocks is live."""
        bm = self.block_manager
        _capi.check(_capi.lib().mkv_bm_count_live(bm.is_block_free.data_ptr(), bm.num_blocks - num_blocks,
                                                  bm.num_blocks, self._result.data_ptr(), _capi.current_stream()))
        return int(self._result[0].item()) == 0

    def shrink_to(self, new_num_blocks: int, donor: "LayerArena" = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Shrink to ``new_num_blocks``: live blocks above the cut move to the lowest free ids
        below it, the block table is rewritten, the memory above the cut is unmapped (or, with a
        ``donor``, mapped back at the end of that arena).
        Returns the move lists; raises ``RuntimeError`` (state untouched) when they do not fit."""
        bm = self.block_manager
        if donor is not None:
            if donor.chunk_bytes != self.chunk_blocks * self.block_bytes:
                raise ValueError("the donor's chunks must have the pool's chunk size")
            if donor.mapped_bytes() + 2 * (bm.num_blocks - new_num_blocks) * self.block_bytes > donor.capacity:
                raise ValueError("the donor has no room for that many chunks")
        if not 0 < new_num_blocks <= bm.num_blocks or new_num_blocks % self.chunk_blocks:
            raise ValueError(f"new size {new_num_blocks} must be a positive multiple of {self.chunk_blocks} "
                             f"and at most {bm.num_blocks}")
        removed = bm.num_blocks - new_num_blocks
        if removed == 0:
            e = torch.empty(0, dtype=torch.int64, device=self.device)
            return e, e
        src, dst = self._relocate_live_blocks(new_num_blocks)        # synchronises the stream
        torch.cuda.synchronize(self.device)                          # nothing may still read the tail
        if donor is None:
            self._map(new_num_blocks)
        else:
            k_had, v_had = self._k_arena.mapped_bytes(), self._v_arena.mapped_bytes()
            d_had = donor.mapped_bytes()
            self.k_cache = self.v_cache = None
            try:
                self._v_arena.move_tail_to(donor, removed * self.block_bytes)
                self._k_arena.move_tail_to(donor, removed * self.block_bytes)
            except Exception:
                # take back what the donor received (K's chunks lie behind V's there), so that the pool still
                # holds every block its counters speak of; the relocation stays (it is valid at either size)
                self._take_back(donor, d_had, k_had, v_had)
                self._make_views(bm.num_blocks)
                raise
            self._make_views(new_num_blocks)
        # the counters follow the memory: only now is the pool smaller
        bm.num_blocks -= removed
        bm.num_free_blocks -= removed
        bm.shrink_free_map(new_num_blocks)
        return src, dst

    def _take_back(self, donor: "LayerArena", d_had: int, k_had: int, v_had: int) -> None:
        """Undo a partial hand-over to ``donor``: chunks it received beyond ``d_had`` return to the arenas that
        are short of ``k_had`` / ``v_had`` (K's were mapped last, so they come back first).  Best effort."""
        for arena, had in ((self._k_arena, k_had), (self._v_arena, v_had)):
            short = had - arena.mapped_bytes()
            if short > 0 and donor.mapped_bytes() - d_had >= short:
                try:
                    donor.move_tail_to(arena, short)
                except Exception:
                    pass

    # the segment-based entry points of the parent do not apply
    def tail_segment_unused(self) -> bool:
        raise NotImplementedError("a virtual-memory pool has no segments; use tail_unused(num_blocks)")

    def shrink_tail_if_unused(self) -> bool:
        raise NotImplementedError("a virtual-memory pool has no segments; use shrink_to(num_blocks)")

    def close(self) -> None:
        """Unmap everything and free the address ranges (the tensors must not be used afterwards)."""
        self.k_cache = self.v_cache = None
        self._k_arena.close()
        self._v_arena.close()
