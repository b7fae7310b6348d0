"""Causal prefill attention.

``prefill_attention`` keeps the operator surface of
MorphServe/worker/kernels/prefill_attn.py:102-139 (whole prompts over the batch's
own contiguous q, k, v -- what the live ``flash_attn_varlen_func`` call computes,
MorphServe/worker/layers/transformer_layer.py:154-164).
``chunked_prefill_attention`` is the variant the reference lacks: a chunk of
queries attending to a prefix that is already in the paged cache.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Optional

import torch

from ... import _capi
from . import _deferred
from ._pool import pool_from_args


def prefill_attention(
    q: torch.Tensor,    # [num_prefill_tokens, num_q_heads, head_dim]
    k: torch.Tensor,    # [num_prefill_tokens, num_kv_heads, head_dim]
    v: torch.Tensor,    # [num_prefill_tokens, num_kv_heads, head_dim]
    o: torch.Tensor,    # [num_prefill_tokens, num_q_heads, head_dim], written
    model_config,
    engine_config,
    infer_state,
) -> None:
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous() and o.is_contiguous()
    assert q.dtype == torch.float16 and o.dtype == torch.float16
    if infer_state.num_prefill_seqs == 0:
        return
    _capi.check(_capi.lib().mkv_prefill_attn(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
        infer_state.prefill_seq_start_locs.data_ptr(), infer_state.prefill_seq_lens.data_ptr(),
        infer_state.num_prefill_seqs, infer_state.max_prefill_len,
        model_config.num_q_heads, model_config.num_kv_heads, model_config.head_dim,
        float(infer_state.softmax_scale), _capi.current_stream()))


def chunked_prefill_attention(
    q: torch.Tensor,                    # [num_chunk_tokens, num_q_heads, head_dim]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_cache_new: List[torch.Tensor],
    v_cache_new: List[torch.Tensor],
    block_table: torch.Tensor,
    model_config,
    engine_config,
    infer_state,
    cur_layer: int,
    o: torch.Tensor,                    # [num_chunk_tokens, num_q_heads, head_dim], written
    prefix_lens: Optional[torch.Tensor] = None,   # [num_prefill_seqs] int32 cached tokens before each chunk
    max_prefix_len: int = 0,            # host-side upper bound of prefix_lens (0 = unknown): picks the launch shape only
) -> None:
    """Chunk b = rows ``prefill_seq_start_locs[b] : +prefill_seq_lens[b]`` of ``q``
    at positions ``prefix_lens[b] ..`` of sequence ``seq_ids[b]``.  The chunk's own
    K/V must have been appended to the cache first; row at position p attends to
    cached positions <= p."""
    assert q.is_contiguous() and o.is_contiguous() and block_table.is_contiguous()
    assert q.dtype == torch.float16 and o.dtype == torch.float16
    if infer_state.num_prefill_seqs == 0:
        return
    pool = pool_from_args(k_cache, v_cache, k_cache_new, v_cache_new, infer_state)
    _deferred.flush()
    _capi.check(_capi.lib().mkv_prefill_attn_paged(
        q.data_ptr(), o.data_ptr(), C.byref(pool), block_table.data_ptr(), block_table.shape[1],
        infer_state.seq_ids.data_ptr(), infer_state.prefill_seq_start_locs.data_ptr(),
        infer_state.prefill_seq_lens.data_ptr(), _capi.ptr(prefix_lens),
        infer_state.num_prefill_seqs, infer_state.max_prefill_len, int(max_prefix_len), model_config.num_q_heads,
        float(infer_state.softmax_scale), cur_layer, _capi.current_stream()))
