"""The attention section of ``LlamaTransformerLayer.forward`` (and of ``AWQTransformerLayer.forward``):
everything between the QKV projection and the output projection
(MorphServe/worker/layers/transformer_layer.py:93-191, :427-504).

The reference runs, per layer: ``rotary_embedding_inplace(q, k)`` -> ``store_kvcache(k, v, ...)`` + an event ->
``flash_attn_varlen_func`` over the prefill tokens into ``o[:P]`` -> on a second ("piggyback") stream that waits
for the event, ``paged_attention`` over the decoding sequences into ``o[P:]`` -> the first stream waits for it.
``attention_section`` is that sequence with this package's launches, in as few of them as the batch allows:

* decode-only batch: ONE launch (rotary of the new q and k rows, append, attention);
* a batch with prefill sequences: rotary + append of every row in one launch, the causal prefill kernel, then
  the paged decode kernel -- on the calling stream, or on ``decoding_piggyback_stream`` behind an event as in the
  reference (the prefill kernel fills every CU, so the second stream gains nothing measurable here; the default
  is one stream).

Results are the reference's: ``o`` rows in batch order (prefill tokens first), the cache holding the rotated k
and the v of every token of the batch.  One side effect differs in the one-launch decode path only: q and k stay
unrotated in memory, which nothing after the attention reads; ``keep_rotated_inputs=True`` takes the two-launch
route that rotates them in place as the reference does.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..kernels.kvcache_mgmt import store_kvcache
from ..kernels.paged_attn import decode_append_and_attend, decode_rope_append_and_attend, paged_attention
from ..kernels.prefill_attn import prefill_attention
from ..kernels.rotary_emb import rotary_embedding_and_store_kvcache, rotary_embedding_inplace


def attention_section(
    q: torch.Tensor,                    # [num_tokens, num_q_heads, head_dim], unrotated
    k: torch.Tensor,                    # [num_tokens, num_kv_heads, head_dim], unrotated
    v: torch.Tensor,                    # [num_tokens, num_kv_heads, head_dim]
    o: torch.Tensor,                    # [num_tokens, num_q_heads * head_dim], written
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    k_cache_new: List[torch.Tensor],
    v_cache_new: List[torch.Tensor],
    block_table: Optional[torch.Tensor],
    model_config,
    engine_config,
    infer_state,
    layer_id: int,
    *,
    rotary: bool = True,
    keep_rotated_inputs: bool = False,
    decoding_piggyback_stream: Optional[torch.cuda.Stream] = None,
) -> None:
    st = infer_state
    ignore_kvcache = bool(getattr(st, "ignore_kvcache", False))
    num_prefill_tokens = st.num_prefill_tokens
    assert q.shape[0] == k.shape[0] == v.shape[0] == o.shape[0] == num_prefill_tokens + st.num_decoding_seqs
    assert o.dim() == 2 and o.shape[1] == q.shape[1] * q.shape[2] and o.is_contiguous()

    if st.num_prefill_seqs == 0 and st.num_decoding_seqs > 0 and not keep_rotated_inputs:
        assert not ignore_kvcache                           # transformer_layer.py:175
        fused = decode_rope_append_and_attend if rotary else decode_append_and_attend
        fused(k, v, q, k_cache, v_cache, k_cache_new, v_cache_new, block_table, model_config, engine_config, st,
              layer_id, o)
        return

    if ignore_kvcache:                                      # the forged batch of profile_num_blocks: no cache at all
        if rotary:
            rotary_embedding_inplace(q, k, st)
    elif rotary:
        rotary_embedding_and_store_kvcache(q, k, v, k_cache, v_cache, k_cache_new, v_cache_new, block_table,
                                           model_config, engine_config, st, layer_id)
    else:
        store_kvcache(k, v, k_cache, v_cache, k_cache_new, v_cache_new, block_table, model_config, engine_config,
                      st, layer_id)

    stored = None
    if decoding_piggyback_stream is not None and st.num_decoding_seqs > 0:
        stored = torch.cuda.Event()
        stored.record()                                     # transformer_layer.py:129-133

    if st.num_prefill_seqs > 0:
        prefill_attention(q[:num_prefill_tokens], k[:num_prefill_tokens], v[:num_prefill_tokens],
                          o[:num_prefill_tokens], model_config, engine_config, st)

    if st.num_decoding_seqs > 0:
        assert not ignore_kvcache
        if stored is None:
            paged_attention(q[num_prefill_tokens:], k_cache, v_cache, k_cache_new, v_cache_new, block_table,
                            model_config, engine_config, st, layer_id, o[num_prefill_tokens:])
        else:
            main = torch.cuda.current_stream()
            with torch.cuda.stream(decoding_piggyback_stream):
                torch.cuda.current_stream().wait_event(stored)
                paged_attention(q[num_prefill_tokens:], k_cache, v_cache, k_cache_new, v_cache_new, block_table,
                                model_config, engine_config, st, layer_id, o[num_prefill_tokens:])
                done = torch.cuda.Event()
                done.record()
            main.wait_event(done)                           # transformer_layer.py:188-191
