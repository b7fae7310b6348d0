"""``store_kvcache``: append this step's K/V to the paged cache.

Operator surface of MorphServe/worker/kernels/kvcache_mgmt.py:298-414; the work
is done by the HIP kernels behind ``mkv_append_prefill`` / ``mkv_append_decode``.
"""
from __future__ import annotations

import ctypes as C
from typing import List

import torch

from ... import _capi
from . import _deferred
from ._pool import pool_from_args


def store_kvcache(
    k: torch.Tensor,                    # [num_tokens, num_kv_heads, head_dim]
    v: torch.Tensor,
    k_cache: torch.Tensor,              # [num_blocks, num_layers, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    k_cache_new: List[torch.Tensor],    # extension segments, same trailing shape
    v_cache_new: List[torch.Tensor],
    block_table: torch.Tensor,          # [max_seqs, max_blocks_per_seq] int32
    model_config,
    engine_config,
    infer_state,
    cur_layer: int,
) -> None:
    """Prefill rows (``[:num_prefill_tokens]``) are scattered block by block, decode
    rows (the tail) one token each at position ``len - 1``; both in one call for a
    mixed batch.  Whether a block id lives in the base pool or in an extension
    segment is decided per id inside the kernel, so the table is never scanned
    (the reference scans it and synchronises, kvcache_mgmt.py:381-383).
    """
    assert k.is_contiguous()
    assert v.is_contiguous()
    assert k_cache.is_contiguous()
    assert v_cache.is_contiguous()
    assert block_table.is_contiguous()
    assert infer_state.seq_ids.is_contiguous()
    assert infer_state.decoding_seq_lens.is_contiguous()
    assert k.dtype == torch.float16 and k_cache.dtype == torch.float16

    lib = _capi.lib()
    _deferred.flush()                   # an append remembered by an earlier call goes out first
    pool = pool_from_args(k_cache, v_cache, k_cache_new, v_cache_new, infer_state)
    stream = _capi.current_stream()
    max_blocks_per_seq = block_table.shape[1]
    row_elems = k.shape[1] * k.shape[2]

    if infer_state.num_prefill_seqs > 0:
        _capi.check(lib.mkv_append_prefill(
            k.data_ptr(), v.data_ptr(), C.byref(pool), block_table.data_ptr(), max_blocks_per_seq,
            infer_state.seq_ids.data_ptr(), infer_state.prefill_seq_start_locs.data_ptr(),
            infer_state.prefill_seq_lens.data_ptr(), infer_state.num_prefill_seqs,
            infer_state.max_prefill_len, cur_layer, stream))

    if infer_state.num_decoding_seqs > 0:
        tok_off = infer_state.num_prefill_tokens * row_elems * k.element_size()
        ids_off = infer_state.num_prefill_seqs * infer_state.seq_ids.element_size()
        if _deferred.ENABLED:           # the paged_attention that follows appends these rows inside its launch
            _deferred.remember(k, v, k.data_ptr() + tok_off, v.data_ptr() + tok_off, pool,
                               (k_cache, v_cache, list(k_cache_new), list(v_cache_new)), k_cache, v_cache,
                               block_table, infer_state, infer_state.seq_ids.data_ptr() + ids_off,
                               infer_state.num_decoding_seqs, cur_layer)
            return
        _capi.check(lib.mkv_append_decode(
            k.data_ptr() + tok_off, v.data_ptr() + tok_off, C.byref(pool),
            block_table.data_ptr(), max_blocks_per_seq,
            infer_state.seq_ids.data_ptr() + ids_off, infer_state.decoding_seq_lens.data_ptr(),
            infer_state.num_decoding_seqs, cur_layer, stream))
