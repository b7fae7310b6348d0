"""``paged_attention``: decode attention over the paged cache.

Operator surface of MorphServe/worker/kernels/paged_attn.py:700-1015 (phase 1
:59-240 / :243-437, phase 2 :658-696) on top of ``mkv_paged_attn_decode``.
"""
from __future__ import annotations

import ctypes as C
import os
from collections import OrderedDict
from typing import List, Optional, Tuple

import torch

from ... import _capi
from . import _deferred
from ._pool import pool_from_args

# Scratch for the per-split partials, grown on demand and reused across calls
# (the reference allocates it on every call, paged_attn.py:780-793).  One buffer per
# (device, stream): calls on one stream are ordered, calls on different streams may overlap.
# At most MAX_SCRATCH_BUFFERS are kept; the least recently used one is dropped (its memory goes
# back to torch's allocator, which keeps it valid for work already queued on its stream).
MAX_SCRATCH_BUFFERS = 8
_scratch: "OrderedDict[Tuple[int, int, int], Tuple[torch.Tensor, torch.Tensor]]" = OrderedDict()

# "auto": split length chosen here for the MI355X grid; "reference": use the
# caller's infer_state.seq_block_size as the reference kernels do.
SPLIT_POLICY = os.environ.get("MORPHKV_SPLIT_POLICY", "auto")
# Workgroups a decode launch should hold: None = two per compute unit of the device (512 on an
# MI355X); a number here or in the environment overrides that.
TARGET_WORKGROUPS: Optional[int] = (int(os.environ["MORPHKV_TARGET_WGS"])
                                    if os.environ.get("MORPHKV_TARGET_WGS") else None)
_target_wgs_by_device = {}
# The grid takes the batch rows in an order that gives every CU about the same number of tokens
# (``mkv_decode_order``); "0" keeps the rows' own order.
BALANCED_ORDER = os.environ.get("MORPHKV_DECODE_ORDER", "1") != "0"


def target_workgroups(device=None) -> int:
    if TARGET_WORKGROUPS is not None:
        return int(TARGET_WORKGROUPS)
    if not torch.cuda.is_available():
        return 512                      # host-only use (tests of the split arithmetic): an MI355X's figure
    idx = torch.cuda.current_device() if device is None or device.index is None else device.index
    wgs = _target_wgs_by_device.get(idx)
    if wgs is None:
        wgs = 2 * torch.cuda.get_device_properties(idx).multi_processor_count
        _target_wgs_by_device[idx] = wgs
    return wgs


def choose_split(n: int, num_kv_heads: int, max_len: int, block_size: int,
                 target_wgs: Optional[int] = None) -> Tuple[int, int]:
    """``(tokens_per_split, max_splits)``: enough (split, kv head, sequence)
    workgroups to put two on each compute unit of the device, and no more: every
    extra split costs a partial write and the phase-2 launch, and a sequence that
    is not split at all is written straight to ``o``.  Each split is a multiple
    of four blocks (one per wave) and never shorter than 128 tokens."""
    target = target_workgroups() if target_wgs is None else target_wgs
    unit = 4 * block_size
    max_len = max(int(max_len), 1)
    want = max(1, -(-target // max(1, n * num_kv_heads)))
    most = max(1, max_len // (2 * unit))
    splits = min(want, most)
    tps = -(-max_len // splits)
    tps = -(-tps // unit) * unit
    return tps, -(-max_len // tps)


def _get_scratch(device: torch.device, n: int, hq: int, splits: int, d: int):
    need_lse = n * hq * splits
    key = (device.index or 0, _capi.current_stream(), d)
    cur = _scratch.get(key)
    if cur is None or cur[1].numel() < need_lse:
        grow = max(need_lse, 2 * cur[1].numel() if cur else 0)
        cur = (torch.empty(grow * d, dtype=torch.float32, device=device),
               torch.empty(grow, dtype=torch.float32, device=device))
        _scratch[key] = cur
        while len(_scratch) > MAX_SCRATCH_BUFFERS:
            _scratch.popitem(last=False)
    _scratch.move_to_end(key)
    return cur


def _decode_order(infer_state, lens: torch.Tensor, n: int, num_kv_heads: int, splits: int) -> Optional[torch.Tensor]:
    """The balanced order of this batch's rows, computed by one small launch the first time a layer asks
    for it and kept on ``infer_state`` for the other layers of the step (it depends on the lengths only).
    An order that has gone stale -- lengths updated in place -- is still a permutation, so the outputs
    do not depend on it; only the balance does.  A batch that is cut into splits needs none: its workgroups
    carry equal token counts already.

    An order whose launch was only RECORDED into a graph holds nothing until that graph runs, so an
    entry made during a stream capture serves that capture alone: an eager call, or another capture,
    computes its own (an abandoned capture can therefore never hand anyone an unwritten buffer)."""
    if not BALANCED_ORDER or n < 2 or n > 4096 or splits > 1:
        return None
    key = (lens.data_ptr(), n, num_kv_heads)
    stream = torch.cuda.current_stream()
    capture = _capi.capture_id(stream.cuda_stream)          # None outside a capture
    cached = getattr(infer_state, "_morphkv_decode_order", None)
    if cached is None or cached[0] != key or cached[4] != capture:
        order = torch.empty(n, dtype=torch.int32, device=lens.device)
        cached = [key, order, None, stream.cuda_stream, capture]
        try:
            infer_state._morphkv_decode_order = cached
        except AttributeError:          # nowhere to keep it: a launch per layer would cost more than it brings
            return None
        _capi.check(_capi.lib().mkv_decode_order(lens.data_ptr(), n, num_kv_heads, order.data_ptr(),
                                                 stream.cuda_stream))
        if capture is None:
            cached[2] = torch.cuda.Event()
            cached[2].record(stream)
    elif cached[3] != stream.cuda_stream and cached[2] is not None and capture is None:
        stream.wait_event(cached[2])    # computed on another stream
    return cached[1]


def _split_for(infer_state, model_config, engine_config):
    n = infer_state.num_decoding_seqs
    max_len = infer_state.num_seq_blocks * infer_state.seq_block_size
    known = getattr(infer_state, "max_decoding_len", 0)
    if known:
        max_len = min(max_len, int(known)) if max_len > 0 else int(known)
    if SPLIT_POLICY == "reference":
        return infer_state.seq_block_size, max(1, infer_state.num_seq_blocks)
    return choose_split(n, model_config.num_kv_heads, max_len, engine_config.block_size)


def decode_append_and_attend(
    k: torch.Tensor,                    # [num_tokens, num_kv_heads, head_dim]; decode rows are the tail
    v: torch.Tensor,
    q: torch.Tensor,                    # [num_decoding_seqs, num_q_heads, head_dim]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_cache_new: List[torch.Tensor],
    v_cache_new: List[torch.Tensor],
    block_table: torch.Tensor,
    model_config,
    engine_config,
    infer_state,
    cur_layer: int,
    o: torch.Tensor,
) -> None:
    """``store_kvcache`` followed by ``paged_attention`` for a decode-only batch
    (MorphServe/worker/layers/transformer_layer.py:116-126, :181-187) as a single
    kernel launch per layer: the new token is written to its cache slot by the
    workgroup that attends over the sequence's last block."""
    assert infer_state.num_prefill_seqs == 0, "the fused call covers decode-only batches"
    assert k.is_contiguous() and v.is_contiguous() and q.is_contiguous() and o.is_contiguous()
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and block_table.is_contiguous()
    assert infer_state.seq_block_size % engine_config.block_size == 0
    assert q.dtype == torch.float16 and o.dtype == torch.float16 and k.dtype == torch.float16
    n = infer_state.num_decoding_seqs
    if n == 0:
        return
    _deferred.flush()
    hq, d = model_config.num_q_heads, model_config.head_dim
    tps, splits = _split_for(infer_state, model_config, engine_config)
    pool = pool_from_args(k_cache, v_cache, k_cache_new, v_cache_new, infer_state)
    mid_o, mid_lse = (None, None)
    if splits > 1:
        mid_o, mid_lse = _get_scratch(q.device, n, hq, splits, d)
    order = _decode_order(infer_state, infer_state.decoding_seq_lens, n, model_config.num_kv_heads, splits)
    _capi.check(_capi.lib().mkv_decode_attn_ordered(
        q.data_ptr(), o.data_ptr(), C.byref(pool), block_table.data_ptr(), block_table.shape[1],
        infer_state.seq_ids.data_ptr(), infer_state.decoding_seq_lens.data_ptr(), _capi.ptr(order), n, hq,
        float(infer_state.softmax_scale), cur_layer, tps, splits, _capi.ptr(mid_o), _capi.ptr(mid_lse),
        k.data_ptr(), v.data_ptr(), None, None, _capi.current_stream()))


def decode_rope_append_and_attend(
    k: torch.Tensor,                    # [num_decoding_seqs, num_kv_heads, head_dim], NOT yet rotated
    v: torch.Tensor,
    q: torch.Tensor,                    # [num_decoding_seqs, num_q_heads, head_dim], NOT yet rotated
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    k_cache_new: List[torch.Tensor],
    v_cache_new: List[torch.Tensor],
    block_table: torch.Tensor,
    model_config,
    engine_config,
    infer_state,                        # with position_cos / position_sin, one row per decoding sequence
    cur_layer: int,
    o: torch.Tensor,
) -> None:
    """``rotary_embedding_inplace`` + ``store_kvcache`` + ``paged_attention`` of a decode-only
    batch (MorphServe/worker/layers/transformer_layer.py:93-126, :181-187) as ONE launch per
    layer.  q and k are rotated on their way into the kernel and are left unrotated in
    memory; the cache receives the rotated k row."""
    assert infer_state.num_prefill_seqs == 0, "the fused call covers decode-only batches"
    assert k.is_contiguous() and v.is_contiguous() and q.is_contiguous() and o.is_contiguous()
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and block_table.is_contiguous()
    assert q.dtype == torch.float16 and o.dtype == torch.float16 and k.dtype == torch.float16
    cos, sin = infer_state.position_cos, infer_state.position_sin
    n = infer_state.num_decoding_seqs
    if n == 0:
        return
    hq, d = model_config.num_q_heads, model_config.head_dim
    assert cos is not None and sin is not None and cos.is_contiguous() and sin.is_contiguous()
    assert cos.dtype == torch.float16 and tuple(cos.shape) == (n, d // 2) == tuple(sin.shape)
    _deferred.flush()
    tps, splits = _split_for(infer_state, model_config, engine_config)
    pool = pool_from_args(k_cache, v_cache, k_cache_new, v_cache_new, infer_state)
    mid_o, mid_lse = (None, None)
    if splits > 1:
        mid_o, mid_lse = _get_scratch(q.device, n, hq, splits, d)
    order = _decode_order(infer_state, infer_state.decoding_seq_lens, n, model_config.num_kv_heads, splits)
    _capi.check(_capi.lib().mkv_decode_attn_ordered(
        q.data_ptr(), o.data_ptr(), C.byref(pool), block_table.data_ptr(), block_table.shape[1],
        infer_state.seq_ids.data_ptr(), infer_state.decoding_seq_lens.data_ptr(), _capi.ptr(order), n, hq,
        float(infer_state.softmax_scale), cur_layer, tps, splits, _capi.ptr(mid_o), _capi.ptr(mid_lse),
        k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(), _capi.current_stream()))


def paged_attention(
    q: torch.Tensor,                    # [num_decoding_seqs, num_q_heads, head_dim]
    k_cache: torch.Tensor,              # [num_blocks, num_layers, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    k_cache_new: List[torch.Tensor],
    v_cache_new: List[torch.Tensor],
    block_table: torch.Tensor,          # [max_seqs, max_blocks_per_seq] int32
    model_config,
    engine_config,
    infer_state,
    cur_layer: int,
    o: torch.Tensor,                    # [num_decoding_seqs, num_q_heads*head_dim] (or 3-D), written
) -> None:
    assert q.is_contiguous()
    assert k_cache.is_contiguous()
    assert v_cache.is_contiguous()
    assert block_table.is_contiguous()
    assert infer_state.seq_block_size % engine_config.block_size == 0
    assert o.is_contiguous()
    assert q.dtype == torch.float16 and o.dtype == torch.float16

    n = infer_state.num_decoding_seqs
    if n == 0:
        return
    hq = model_config.num_q_heads
    d = model_config.head_dim
    block_size = engine_config.block_size

    tps, splits = _split_for(infer_state, model_config, engine_config)

    lib = _capi.lib()
    pool = pool_from_args(k_cache, v_cache, k_cache_new, v_cache_new, infer_state)
    mid_o, mid_lse = (None, None)
    if splits > 1:
        mid_o, mid_lse = _get_scratch(q.device, n, hq, splits, d)
    ids_off = infer_state.num_prefill_seqs * infer_state.seq_ids.element_size()
    seq_ids_ptr = infer_state.seq_ids.data_ptr() + ids_off
    lens_ptr = infer_state.decoding_seq_lens.data_ptr()
    pending = _deferred.take(k_cache, v_cache, block_table, seq_ids_ptr, lens_ptr, n, cur_layer)
    order = _decode_order(infer_state, infer_state.decoding_seq_lens, n, model_config.num_kv_heads, splits)
    # a pending append: the decode rows store_kvcache was given for this layer are appended by this launch
    _capi.check(lib.mkv_decode_attn_ordered(
        q.data_ptr(), o.data_ptr(), C.byref(pool), block_table.data_ptr(), block_table.shape[1], seq_ids_ptr,
        lens_ptr, _capi.ptr(order), n, hq, float(infer_state.softmax_scale), cur_layer, tps, splits,
        _capi.ptr(mid_o), _capi.ptr(mid_lse), pending.k_ptr if pending is not None else None,
        pending.v_ptr if pending is not None else None, None, None, _capi.current_stream()))
