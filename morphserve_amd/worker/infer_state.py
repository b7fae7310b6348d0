"""Per-step argument bundle of the paged-KV operators.

Mirrors ``LlamaInferState`` (MorphServe/worker/infer_state.py:4-32) field for
field and restates how ``LlamaModel.forward`` fills it
(MorphServe/worker/model.py:318-436).
"""
from __future__ import annotations

import dataclasses
from typing import Optional, Sequence, Tuple

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
