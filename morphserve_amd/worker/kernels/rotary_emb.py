"""Rotary position embedding, alone or fused with the KV append.

``rotary_embedding_inplace`` keeps the operator surface of
MorphServe/worker/kernels/rotary_emb.py:44-58.  ``rotary_embedding_and_store_kvcache``
is the pair the transformer layer runs back to back
(MorphServe/worker/layers/transformer_layer.py:93-126) in ONE launch: q and k are
rotated in place (prefill attention still reads the batch's own k) and the rotated k
and v rows go straight to their cache slots, prefill and decode rows alike.
``rotary_tables`` builds the cos / sin cache of MorphServe/worker/model.py:230-241.
"""
from __future__ import annotations

import ctypes as C
from typing import List, Tuple

import torch

from ... import _capi
from . import _deferred
from ._pool import pool_from_args


def rotary_tables(head_dim: int, max_position_embeddings: int, rope_theta: float = 10000.0,
                  rope_scaling: float = 1.0, device: str = "cuda") -> Tuple[torch.Tensor, torch.Tensor]:
    """``(_cos_cached, _sin_cached)``: fp16 ``[max_position_embeddings * scaling + 128, head_dim / 2]``."""
    max_seq_len = max_position_embeddings * rope_scaling
    inv_freq = 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, device=device, dtype=torch.float32) / head_dim))
    t = torch.arange(max_seq_len + 128, device=device, dtype=torch.float32) / rope_scaling
    freqs = torch.outer(t, inv_freq)
    return torch.cos(freqs).to(torch.float16), torch.sin(freqs).to(torch.float16)


def _check(q, k, infer_state):
    assert q.is_contiguous() and k.is_contiguous() and q.dtype == torch.float16 and k.dtype == torch.float16
    cos, sin = infer_state.position_cos, infer_state.position_sin
    assert cos is not None and sin is not None, "infer_state carries no position_cos / position_sin"
    assert cos.is_contiguous() and sin.is_contiguous() and cos.dtype == torch.float16
    assert cos.shape == (q.shape[0], q.shape[2] // 2) == sin.shape, "one cos / sin row per token"
    assert k.shape[0] == q.shape[0] and k.shape[2] == q.shape[2]
    return cos, sin


def rotary_embedding_inplace(
    q: torch.Tensor,    # [num_tokens, num_q_heads, head_dim]
    k: torch.Tensor,    # [num_tokens, num_kv_heads, head_dim]
    infer_state,
) -> None:
    cos, sin = _check(q, k, infer_state)
    _capi.check(_capi.lib().mkv_rope_store_kvcache(
        q.data_ptr(), k.data_ptr(), None, cos.data_ptr(), sin.data_ptr(), None, None, 0, None, None, None, None,
        0, q.shape[0], 0, q.shape[1], k.shape[1], q.shape[2], 0, 0, _capi.current_stream()))


def rotary_embedding_and_store_kvcache(
    q: torch.Tensor,    # [num_tokens, num_q_heads, head_dim], rotated in place
    k: torch.Tensor,    # [num_tokens, num_kv_heads, head_dim], rotated in place
    v: torch.Tensor,    # [num_tokens, num_kv_heads, head_dim]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_cache_new: List[torch.Tensor],
    v_cache_new: List[torch.Tensor],
    block_table: torch.Tensor,
    model_config,
    engine_config,
    infer_state,
    cur_layer: int,
) -> None:
    cos, sin = _check(q, k, infer_state)
    assert v.is_contiguous() and v.shape == k.shape and block_table.is_contiguous()
    assert q.shape[0] == infer_state.num_tokens
    pool = pool_from_args(k_cache, v_cache, k_cache_new, v_cache_new, infer_state)
    st = infer_state
    _deferred.flush()
    _capi.check(_capi.lib().mkv_rope_store_kvcache(
        q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(), C.byref(pool),
        block_table.data_ptr(), block_table.shape[1], st.seq_ids.data_ptr(),
        _capi.ptr(st.prefill_seq_start_locs), _capi.ptr(st.prefill_seq_lens), _capi.ptr(st.decoding_seq_lens),
        st.num_prefill_seqs, st.num_prefill_tokens, st.num_decoding_seqs, q.shape[1], k.shape[1], q.shape[2],
        cur_layer, 1, _capi.current_stream()))
