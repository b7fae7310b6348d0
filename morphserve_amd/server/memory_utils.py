"""KV side of MorphServe/server/memory_utils.py: what growing and shrinking the pool
does to the block manager, the segment lists and the scheduler's block budget.

The reference grows the pool as a side effect of swapping a transformer layer for
its quantized twin (``org2quant_and_update_kvcache``, :93-116) and shrinks it when
the layer is restored (``quant2org_and_update_kvcache``, :617-659).  The weight
swap itself is not part of this package; where the freed bytes come from is a
callable ``acquire_segment(layer_id) -> (k_seg, v_seg) | None`` (``None``: let the
pool allocate a segment of ``seg_blocks`` blocks itself) or, for a pool over virtual
memory, a ``LayerArena`` per replaceable layer whose chunks behind the quantized copy
move into the pool and back (``layer_arenas``, ``quant_layer_bytes``).  Everything else -- the
order of the bookkeeping, the layer counters the scheduler reads, the refusal of a
shrink whose tail segment still holds live blocks -- follows the reference; the
``migrate`` switch replaces that refusal by an on-device relocation of the live
blocks (``ElasticKVPool.shrink_to``).
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

from ..elastic_pool import ElasticKVPool, PoolTooFullError


class _Model:
    """The attributes of ``engine.model`` that scheduler.py and memory_utils.py touch."""

    def __init__(self, pool: ElasticKVPool, num_layers: int, seg_blocks: int):
        self.pool = pool
        self.num_layers = num_layers
        self.kv_cache_new_block_size = seg_blocks     # survives a shrink to zero segments (model.py:77)
        self.next_unquantized_layer = num_layers - 1  # layers are replaced last to first (model.py:81)
        self.layer_quant_list: List[int] = []
        self.is_layer_quant_list = [False] * num_layers

    gpu_block_manager = property(lambda self: self.pool.block_manager)
    k_cache = property(lambda self: self.pool.k_cache)
    v_cache = property(lambda self: self.pool.v_cache)
    k_cache_new = property(lambda self: self.pool.k_cache_new)
    v_cache_new = property(lambda self: self.pool.v_cache_new)


class PoolEngine:
    """Stands where the reference passes its ``Engine`` into the scheduler and the two
    functions below: ``.model`` (pool + layer counters), ``.engine_config``, ``.scheduler``."""

    def __init__(self, pool: ElasticKVPool, engine_config, num_layers: int, seg_blocks: int,
                 acquire_segment: Optional[Callable] = None, migrate: bool = True,
                 layer_arenas: Optional[Dict[int, object]] = None, quant_layer_bytes: int = 0):
        self.model = _Model(pool, num_layers, seg_blocks)
        self.engine_config = engine_config
        self.acquire_segment = acquire_segment
        self.layer_arenas = layer_arenas or {}       # layer id -> LayerArena (virtual-memory pools only)
        self.quant_layer_bytes = quant_layer_bytes   # what the quantized twin keeps at the start of its arena
        self.migrate = migrate
        self.scheduler = None        # set by the owner once the Scheduler exists
        self.migrated_blocks = 0     # live blocks relocated by shrinks so far
        # blocks each replaced layer gave to the pool: arenas may differ in what they can spare (their size,
        # the pool's remaining reservation), so a restored layer takes back exactly what IT gave
        self.blocks_from_layer: Dict[int, int] = {}


class _ShrinkInto:
    """A virtual-memory pool whose ``shrink_to`` hands the memory above the cut to ``arena``."""

    def __init__(self, pool, arena):
        self._pool, self._arena = pool, arena

    def __getattr__(self, name):
        return getattr(self._pool, name)

    def shrink_to(self, new_num_blocks: int):
        return self._pool.shrink_to(new_num_blocks, self._arena)


def update_kvcache_after_replacing_layer(engine: PoolEngine, layer_id: int) -> None:
    """memory_utils.py:369-420: append the new segment; ``num_blocks``, ``num_free_blocks``,
    the free map and the scheduler's budget all grow by its block count."""
    model = engine.model
    arena = engine.layer_arenas.get(layer_id)
    seg = engine.acquire_segment(layer_id) if engine.acquire_segment and arena is None else None
    if arena is not None:
        n = model.pool.expand_from(arena, engine.quant_layer_bytes)
        if n == 0:                                   # memory_manager.cpp:96-98
            raise RuntimeError("No space available for new KV cache blocks")
        model.kv_cache_new_block_size = n
    elif seg is None:
        model.pool.expand(model.kv_cache_new_block_size)
    else:
        model.pool.expand(int(seg[0].shape[0]), seg[0], seg[1])
        model.kv_cache_new_block_size = int(seg[0].shape[0])
    engine.blocks_from_layer[layer_id] = model.kv_cache_new_block_size
    if engine.scheduler is not None:
        engine.scheduler.num_gpu_blocks += model.kv_cache_new_block_size


def org2quant_and_update_kvcache(engine: PoolEngine, update_kvcache: bool = True) -> None:
    """memory_utils.py:93-116 without the weight swap: layer ``next_unquantized_layer`` is
    marked replaced and its bytes become one more KV segment."""
    model = engine.model
    layer_id = model.next_unquantized_layer
    if layer_id < 0:
        raise RuntimeError("every layer has already been replaced")
    if update_kvcache:
        update_kvcache_after_replacing_layer(engine, layer_id)
    model.is_layer_quant_list[layer_id] = True
    model.layer_quant_list.append(layer_id)
    model.next_unquantized_layer -= 1


def quant2org_and_update_kvcache(engine: PoolEngine, update_kvcache: bool = True) -> bool:
    """memory_utils.py:617-659 without the weight swap: the most recently replaced layer
    comes back and the LAST segment is dropped.  Reference behaviour (``migrate`` off):
    False, nothing changed, while any block of that segment is live (:529-544, :623-624).
    With ``migrate`` the live blocks are first moved into the lowest free ids below the cut
    and the block table is rewritten; False only when they do not fit."""
    model = engine.model
    layer_id = model.next_unquantized_layer + 1
    if not model.layer_quant_list:
        raise RuntimeError("no replaced layer to restore")
    if update_kvcache:
        pool = model.pool
        contiguous = hasattr(pool, "tail_unused")          # a virtual-memory pool: no segments to pop
        arena = engine.layer_arenas.get(layer_id)
        if arena is not None:                              # the memory goes back to the layer it came from
            pool = _ShrinkInto(pool, arena)
        # what this layer gave (the reference's segments all have one size, so there the latest value does)
        given = engine.blocks_from_layer.get(layer_id, model.kv_cache_new_block_size)
        if contiguous and pool.tail_unused(given):
            pool.shrink_to(pool.num_blocks - given)
        elif not contiguous and pool.shrink_tail_if_unused():
            pass
        elif not engine.migrate:
            return False
        else:
            try:
                src, _ = pool.shrink_to(pool.num_blocks - given)
            except PoolTooFullError:       # does not fit: an ordinary refusal; a failed launch propagates
                return False
            engine.migrated_blocks += int(src.numel())
        engine.blocks_from_layer.pop(layer_id, None)
        if engine.scheduler is not None:
            engine.scheduler.num_gpu_blocks -= given
    model.is_layer_quant_list[layer_id] = False
    model.layer_quant_list.remove(layer_id)
    model.next_unquantized_layer = layer_id
    return True
