"""Optional deferral of the decode rows of ``store_kvcache`` into the ``paged_attention`` that follows.

The reference's decode layer calls ``store_kvcache`` and then ``paged_attention``
(MorphServe/worker/layers/transformer_layer.py:116-126, :181-187): two launches, the first of which
moves a few hundred KiB and costs a launch latency.  With the deferral switched on, ``store_kvcache``
only REMEMBERS the decode rows of its call; the next ``paged_attention`` for the same layer, cache and
block table appends them inside its own launch (``mkv_decode_append_attn``).  Anything else that reads
or writes the cache through this package first issues the remembered append as a launch of its own
(``flush``), on the stream ``store_kvcache`` was called on.

The pending append is kept per host thread (the reference's engine issues its GPU work from one
executor thread at a time, MorphServe/server/engine.py:43-48, :314-319): a thread only ever sees and
flushes what it remembered itself, so two threads driving two pools never hand each other's rows on.
A thread that reads a cache another thread still has a pending append for must be ordered after that
thread's attention call (or ``flush_pending_appends()``) by the caller, exactly as it must be ordered
after the other thread's launches.

Off by default: while an append is pending the cache does not hold the new token yet, which a caller
that inspects the cache tensors directly (not through this package) between the two calls would see,
and the decode rows of ``k`` and ``v`` are read when the append is finally issued, so they must not be
overwritten before the attention call (or ``flush_pending_appends()``).
``MORPHKV_DEFER_DECODE_APPEND=1`` or ``enable_deferred_decode_append(True)`` turns it on.
"""
from __future__ import annotations

import ctypes as C
import os
import threading
from typing import Optional

import torch

from ... import _capi

ENABLED = os.environ.get("MORPHKV_DEFER_DECODE_APPEND", "0") == "1"


class _Pending:
    __slots__ = ("k", "v", "k_ptr", "v_ptr", "pool", "keep", "block_table", "seq_ids", "seq_ids_ptr", "lens", "n",
                 "layer", "stream_obj", "key")


class _State(threading.local):
    pending: Optional[_Pending] = None


_state = _State()


def pending() -> Optional[_Pending]:
    """The calling thread's remembered append, if any."""
    return _state.pending


def enable_deferred_decode_append(on: bool) -> None:
    global ENABLED
    flush()
    ENABLED = bool(on)


def _key(k_cache, v_cache, block_table, seq_ids_ptr, lens_ptr, n, layer):
    return (k_cache.data_ptr(), v_cache.data_ptr(), block_table.data_ptr(), seq_ids_ptr, lens_ptr, n, layer)


def remember(k, v, k_ptr, v_ptr, pool, keep, k_cache, v_cache, block_table, infer_state, seq_ids_ptr, n, layer) -> None:
    """Called by ``store_kvcache`` in place of the decode-row launch."""
    flush()
    p = _Pending()
    p.k, p.v, p.k_ptr, p.v_ptr = k, v, k_ptr, v_ptr          # the tensors are kept alive until the append is issued
    p.pool, p.keep = pool, keep
    p.block_table, p.seq_ids, p.lens = block_table, infer_state.seq_ids, infer_state.decoding_seq_lens
    p.seq_ids_ptr, p.n, p.layer = seq_ids_ptr, n, layer
    p.stream_obj = torch.cuda.current_stream()
    p.key = _key(k_cache, v_cache, block_table, seq_ids_ptr, p.lens.data_ptr(), n, layer)
    _state.pending = p


def take(k_cache, v_cache, block_table, seq_ids_ptr, lens_ptr, n, layer) -> Optional[_Pending]:
    """The pending append if it is exactly what this attention call needs; any other pending append is
    issued first."""
    p = _state.pending
    if p is None:
        return None
    if p.key == _key(k_cache, v_cache, block_table, seq_ids_ptr, lens_ptr, n, layer):
        _state.pending = None
        return p
    flush()
    return None


def flush() -> None:
    """Issue the remembered append, if any, as a launch of its own on the stream it was remembered on."""
    p = _state.pending
    if p is None:
        return
    _state.pending = None
    _capi.check(_capi.lib().mkv_append_decode(
        p.k_ptr, p.v_ptr, C.byref(p.pool), p.block_table.data_ptr(), p.block_table.shape[1], p.seq_ids_ptr,
        p.lens.data_ptr(), p.n, p.layer, p.stream_obj.cuda_stream))
