"""Per-step argument bundle of the paged-KV operators.

Mirrors ``LlamaInferState`` (MorphServe/worker/infer_state.py:4-32) field for
field and restates how ``LlamaModel.forward`` fills it
(MorphServe/worker/model.py:318-436).
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Sequence, Tuple

import numpy as np
import torch


@dataclasses.dataclass
class LlamaInferState:
    batch_size: int
    num_tokens: int

    seq_ids: torch.Tensor            # [batch_size] int32; prefill sequences first, then decoding ones
    softmax_scale: float             # head_dim ** -0.5

    num_prefill_seqs: int
    num_prefill_tokens: int
    prefill_seq_start_locs: torch.Tensor            # [num_prefill_seqs] int32
    prefill_seq_start_locs_with_end: torch.Tensor   # [num_prefill_seqs + 1] int32
    prefill_seq_lens: torch.Tensor                  # [num_prefill_seqs] int32
    max_prefill_len: int

    num_decoding_seqs: int
    decoding_seq_lens: torch.Tensor  # [num_decoding_seqs] int32, the token being appended included
    max_decoding_len: int

    seq_block_size: int
    num_seq_blocks: int

    num_blocks_org: Optional[int]    # first id of the extension segments
    kv_cache_new_block_size: int     # blocks per extension segment
    org_layer_param_size: int        # elements between consecutive segments

    position_cos: Optional[torch.Tensor] = None
    position_sin: Optional[torch.Tensor] = None

    ignore_kvcache: bool = False


def select_seq_block_size(num_kv_heads: int, decoding_seq_lens: Sequence[int]) -> Tuple[int, int]:
    """Split-KV chunk length and chunk count the reference would pick
    (MorphServe/worker/model.py:397-402, :426)."""
    size = 512
    total = sum(decoding_seq_lens)
    longest = max(decoding_seq_lens) if len(decoding_seq_lens) else 0
    while (num_kv_heads * (total / size) < 1024 and size // 2 >= 64
           and longest / (size // 2) <= 128):
        size //= 2
    return size, (longest + size - 1) // size


def build_infer_state(prefill_lens: Sequence[int], seq_ids_list: Sequence[int],
                      decoding_seq_lens_list: Sequence[int], num_kv_heads: int, head_dim: int,
                      num_blocks_org: Optional[int] = None, kv_cache_new_block_size: int = 0,
                      org_layer_param_size: int = 0, device: str = "cuda") -> LlamaInferState:
    """What ``LlamaModel.forward`` builds from its host lists
    (MorphServe/worker/model.py:318-341, :397-436), without the rotary tables."""
    prefill_lens = [int(x) for x in prefill_lens]
    dec = [int(x) for x in decoding_seq_lens_list]
    num_prefill_seqs = len(prefill_lens)
    batch_size = num_prefill_seqs + len(dec)
    assert len(seq_ids_list) == batch_size
    num_prefill_tokens = sum(prefill_lens)
    num_tokens = num_prefill_tokens + len(dec)
    seq_ids = torch.tensor(list(seq_ids_list), dtype=torch.int32, device=device)
    p_lens = torch.tensor(prefill_lens, dtype=torch.int32, device=device)
    starts = torch.cumsum(p_lens, dim=0, dtype=torch.int32) - p_lens
    sbs, nsb = select_seq_block_size(num_kv_heads, dec)
    return LlamaInferState(
        batch_size=batch_size,
        num_tokens=num_tokens,
        seq_ids=seq_ids,
        softmax_scale=head_dim ** -0.5,
        num_prefill_seqs=num_prefill_seqs,
        num_prefill_tokens=num_prefill_tokens,
        prefill_seq_start_locs=starts,
        prefill_seq_start_locs_with_end=torch.cat(
            [starts, torch.tensor([num_tokens], dtype=torch.int32, device=device)]),
        prefill_seq_lens=p_lens,
        max_prefill_len=max(prefill_lens) if prefill_lens else 0,
        num_decoding_seqs=len(dec),
        decoding_seq_lens=torch.tensor(dec, dtype=torch.int32, device=device),
        max_decoding_len=max(dec) if dec else 0,
        seq_block_size=sbs,
        num_seq_blocks=nsb,
        num_blocks_org=num_blocks_org,
        kv_cache_new_block_size=kv_cache_new_block_size,
        org_layer_param_size=org_layer_param_size,
    )


class StepStateBuilder:
    """``LlamaModel.forward``'s per-step preparation (MorphServe/worker/model.py:318-436) with ONE host-to-device
    copy: the reference turns each host list into a device tensor of its own (seven ``torch.tensor(..., device=
    "cuda")`` calls, an ``arange`` per prefill sequence and two ``cat``), each a synchronous copy from pageable
    memory.  Here every list is written into one pinned int32 staging buffer --

        seq_ids[B] | seq_lengths[B] | prefill_lens[P] | prefill_starts[P] , end | decoding_lens[n] | positions[T]

    -- which goes to the device as one asynchronous copy on the current stream; the fields of the returned
    ``LlamaInferState`` are views of the device copy.  ``position_cos / position_sin`` are gathered from the cached
    tables by the positions (``:343-362``, ``:431-432``) when tables were given, and the blocks the step needs are
    allocated (``:364-368``) when a block manager is passed.

    ``slots`` staging/device buffer pairs are used in turn, so a state stays valid until ``slots`` further
    states have been built (the reference's states live as long as they are referenced); before a pair is
    reused the builder waits for the copy that last read its staging half.
    """

    def __init__(self, max_batch_size: int, max_tokens_in_batch: int, num_kv_heads: int, head_dim: int,
                 cos_cached: Optional[torch.Tensor] = None, sin_cached: Optional[torch.Tensor] = None,
                 device: str = "cuda", slots: int = 2):
        self.num_kv_heads, self.head_dim = num_kv_heads, head_dim
        self.cos_cached, self.sin_cached = cos_cached, sin_cached
        self.device = torch.device(device)
        self.max_batch_size, self.max_tokens = max_batch_size, max_tokens_in_batch
        cap = 5 * max_batch_size + 1 + max_tokens_in_batch
        on_gpu = self.device.type == "cuda"
        self._host = [torch.empty(cap, dtype=torch.int32, pin_memory=on_gpu) for _ in range(slots)]
        self._dev = [torch.empty(cap, dtype=torch.int32, device=self.device) for _ in range(slots)]
        self._copied = [None] * slots
        self._turn = 0

    def build(self, prefill_lens: Sequence[int], seq_ids_list: Sequence[int], decoding_seq_lens_list: Sequence[int],
              block_manager=None, ignore_kvcache: bool = False, kv_cache_new_block_size: int = 0,
              org_layer_param_size: int = 0) -> LlamaInferState:
        P, n = len(prefill_lens), len(decoding_seq_lens_list)
        B = P + n
        if len(seq_ids_list) != B:
            raise ValueError("one sequence id per prefill and per decoding sequence")
        slot = self._turn
        self._turn = (self._turn + 1) % len(self._host)
        if self._copied[slot] is not None:
            self._copied[slot].synchronize()                 # the staging half may be overwritten now
        host = self._host[slot].numpy()
        o_ids, o_len, o_pl, o_ps, o_dl = 0, B, 2 * B, 2 * B + P, 2 * B + 2 * P + 1
        o_pos = o_dl + n
        host[o_ids:o_ids + B] = seq_ids_list
        host[o_pl:o_pl + P] = prefill_lens
        host[o_dl:o_dl + n] = decoding_seq_lens_list
        p_lens = host[o_pl:o_pl + P]
        d_lens = host[o_dl:o_dl + n]
        num_prefill_tokens = int(p_lens.sum())
        T = num_prefill_tokens + n
        if B > self.max_batch_size or T > self.max_tokens:
            raise ValueError(f"batch of {B} sequences / {T} tokens exceeds the builder's {self.max_batch_size} / "
                             f"{self.max_tokens}")
        host[o_len:o_len + P] = p_lens
        host[o_len + P:o_len + B] = d_lens
        starts = host[o_ps:o_ps + P + 1]
        starts[0:1] = 0
        if P:
            starts[1:P + 1] = p_lens.cumsum()
        starts_only = starts[:P].copy()
        starts[P] = T                                        # the reference's "with end" closes on num_tokens (:416-419)
        pos = host[o_pos:o_pos + T]
        if P:                                                # 0 .. len-1 per prefill sequence, then len-1 per decoding one
            idx = np.arange(num_prefill_tokens, dtype=np.int32)
            pos[:num_prefill_tokens] = idx - np.repeat(starts_only, p_lens)
        pos[num_prefill_tokens:] = d_lens - 1
        used = o_pos + T
        dev = self._dev[slot]
        dev[:used].copy_(self._host[slot][:used], non_blocking=True)
        if self.device.type == "cuda":
            ev = torch.cuda.Event()
            ev.record()
            self._copied[slot] = ev
        seq_ids, seq_lengths = dev[o_ids:o_ids + B], dev[o_len:o_len + B]
        if block_manager is not None and not ignore_kvcache:
            # the lists are at hand: the manager sizes and checks the request on the host and nothing waits
            block_manager.allocate_blocks_for_seqs(seq_ids, seq_lengths, seq_ids_host=host[o_ids:o_ids + B],
                                                   target_lens_host=host[o_len:o_len + B])
        dec = [int(x) for x in decoding_seq_lens_list]
        sbs, nsb = select_seq_block_size(self.num_kv_heads, dec)
        positions = dev[o_pos:o_pos + T]
        with_tables = self.cos_cached is not None and self.sin_cached is not None
        return LlamaInferState(
            batch_size=B,
            num_tokens=T,
            seq_ids=seq_ids,
            softmax_scale=self.head_dim ** -0.5,
            num_prefill_seqs=P,
            num_prefill_tokens=num_prefill_tokens,
            prefill_seq_start_locs=dev[o_ps:o_ps + P],
            prefill_seq_start_locs_with_end=dev[o_ps:o_ps + P + 1],
            prefill_seq_lens=dev[o_pl:o_pl + P],
            max_prefill_len=int(p_lens.max()) if P else 0,
            num_decoding_seqs=n,
            decoding_seq_lens=dev[o_dl:o_dl + n],
            max_decoding_len=max(dec) if dec else 0,
            seq_block_size=sbs,
            num_seq_blocks=nsb,
            num_blocks_org=block_manager.num_blocks_org if block_manager is not None else None,
            kv_cache_new_block_size=kv_cache_new_block_size,
            org_layer_param_size=org_layer_param_size,
            position_cos=self.cos_cached[positions] if with_tables else None,
            position_sin=self.sin_cached[positions] if with_tables else None,
            ignore_kvcache=ignore_kvcache,
        )
