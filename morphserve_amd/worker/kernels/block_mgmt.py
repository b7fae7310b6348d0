"""Block-table row operations.

Operator surface of MorphServe/worker/kernels/block_mgmt.py:26-46, :66-80,
:106-125, each one single-workgroup HIP launch.
"""
from __future__ import annotations

import torch

from ... import _capi


def set_block_table_and_num_seq_alloc_blocks(
    num_seq_allocated_blocks: torch.Tensor,   # [max_seqs] int32
    block_table: torch.Tensor,                # [max_seqs, max_blocks_per_seq] int32
    candidate_blocks: torch.Tensor,           # [sum(block_needed)] int64
    seq_ids: torch.Tensor,                    # [batch] int32
    block_needed: torch.Tensor,               # [batch] int32 or int64
) -> None:
    """Row ``seq_ids[i]`` receives the next ``block_needed[i]`` candidate ids after
    its current entries and its count grows by that much (batch order)."""
    assert candidate_blocks.dtype == torch.int64 and candidate_blocks.is_contiguous()
    assert seq_ids.dtype == torch.int32 and seq_ids.is_contiguous()
    assert block_needed.dtype in (torch.int32, torch.int64) and block_needed.is_contiguous()
    _capi.check(_capi.lib().mkv_bt_append(
        num_seq_allocated_blocks.data_ptr(), num_seq_allocated_blocks.shape[0],
        block_table.data_ptr(), block_table.shape[1], candidate_blocks.data_ptr(),
        seq_ids.data_ptr(), block_needed.data_ptr(),
        1 if block_needed.dtype == torch.int64 else 0, seq_ids.shape[0], _capi.current_stream()))


def unset_block_table_and_num_seq_alloc_blocks(
    num_seq_allocated_blocks: torch.Tensor,
    block_table: torch.Tensor,
    seq_ids: torch.Tensor,
    is_block_free: torch.Tensor,              # [num_blocks] bool
    freed_total: torch.Tensor = None,         # optional [1] int64: receives the number released
) -> None:
    """Marks the blocks of the given sequences free and zeroes their counts; the
    row contents stay as they are."""
    assert seq_ids.dtype == torch.int32 and seq_ids.is_contiguous()
    _capi.check(_capi.lib().mkv_bt_release(
        num_seq_allocated_blocks.data_ptr(), num_seq_allocated_blocks.shape[0],
        block_table.data_ptr(), block_table.shape[1], seq_ids.data_ptr(), seq_ids.shape[0],
        is_block_free.data_ptr(), is_block_free.shape[0], _capi.ptr(freed_total),
        _capi.current_stream()))


def gather_allocated_blocks_and_unset(
    num_seq_allocated_blocks: torch.Tensor,
    block_table: torch.Tensor,
    seq_ids: torch.Tensor,
    is_block_free: torch.Tensor,
    total: int = None,
) -> torch.Tensor:
    """As the release above, and returns the released ids (int32, sequence-major,
    logical block order).  One host read of the total sizes the result -- unless the
    caller knows ``total`` (the sum of the rows' counts): then the result has its size
    from the start and nothing is read back."""
    assert seq_ids.dtype == torch.int32 and seq_ids.is_contiguous()
    dev = block_table.device
    if total is not None:
        out = torch.empty(int(total), dtype=torch.int32, device=dev)
        result = torch.empty(2, dtype=torch.int64, device=dev)
        _capi.check(_capi.lib().mkv_bt_gather_release(
            num_seq_allocated_blocks.data_ptr(), num_seq_allocated_blocks.shape[0],
            block_table.data_ptr(), block_table.shape[1], seq_ids.data_ptr(), seq_ids.shape[0],
            is_block_free.data_ptr(), int(is_block_free.shape[0]), out.data_ptr(), int(total), result.data_ptr(),
            _capi.current_stream()))
        return out
    cap = int(is_block_free.shape[0])
    out = torch.empty(cap, dtype=torch.int32, device=dev)
    result = torch.zeros(2, dtype=torch.int64, device=dev)
    _capi.check(_capi.lib().mkv_bt_gather_release(
        num_seq_allocated_blocks.data_ptr(), num_seq_allocated_blocks.shape[0],
        block_table.data_ptr(), block_table.shape[1], seq_ids.data_ptr(), seq_ids.shape[0],
        is_block_free.data_ptr(), cap, out.data_ptr(), cap, result.data_ptr(),
        _capi.current_stream()))
    total, status = result.tolist()
    if status != 0:
        raise RuntimeError(f"gather_allocated_blocks_and_unset: {total} ids do not fit {cap}")
    return out[:total]
