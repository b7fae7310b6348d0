"""Turns the operators' cache arguments into the ``mkv_pool`` descriptor."""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Tuple

import torch

from ... import _capi

_cache: Dict[Tuple, _capi.MkvPool] = {}
_CACHE_LIMIT = 64


def pool_from_args(k_cache: torch.Tensor, v_cache: torch.Tensor,
                   k_cache_new: List[torch.Tensor], v_cache_new: List[torch.Tensor],
                   infer_state) -> _capi.MkvPool:
    """Base pool plus the extension segments in ``k_cache_new`` / ``v_cache_new``.

    Each segment tensor's own address is used, which in the reference's memory
    layout equals its "segment 0 minus j * org_layer_param_size elements" rule
    (MorphServe/worker/kernels/kvcache_mgmt.py:177-183).  Ids at or beyond
    ``infer_state.num_blocks_org`` address the segments, each
    ``infer_state.kv_cache_new_block_size`` blocks long.
    """
    nseg = len(k_cache_new)
    org = k_cache.shape[0]
    seg_blocks = 0
    if nseg:
        org = infer_state.num_blocks_org if infer_state.num_blocks_org is not None else org
        seg_blocks = int(infer_state.kv_cache_new_block_size)
    key = (k_cache.data_ptr(), v_cache.data_ptr(), tuple(k_cache.shape), org, seg_blocks,
           tuple(t.data_ptr() for t in k_cache_new), tuple(t.data_ptr() for t in v_cache_new))
    pool = _cache.get(key)
    if pool is None:
        if len(_cache) >= _CACHE_LIMIT:
            _cache.clear()
        pool = _capi.make_pool(k_cache, v_cache, k_cache_new, v_cache_new,
                               num_blocks_org=org, seg_blocks=seg_blocks)
        _cache[key] = pool
    return pool


def pool_strided(k_cache: torch.Tensor, v_cache: torch.Tensor, k_cache_new0: torch.Tensor,
                 v_cache_new0: torch.Tensor, num_blocks_org: int, org_layer_param_size: int,
                 kv_cache_new_block_size: int, elem_bytes: int, num_segments: int) -> _capi.MkvPool:
    """The reference's calling convention: only segment 0 is passed, segment j is
    ``j * org_layer_param_size`` elements below it (csrc/src/block_swapping.cpp:156-160)."""
    pool = _capi.make_pool(k_cache, v_cache, num_blocks_org=num_blocks_org)
    pool.seg_blocks = int(kv_cache_new_block_size)
    _capi.check(_capi.lib().mkv_pool_set_strided(
        C.byref(pool), k_cache_new0.data_ptr(), v_cache_new0.data_ptr(),
        int(org_layer_param_size), int(elem_bytes), int(num_segments)))
    return pool
