"""The KV-cache entries of the reference's native module ``swiftllm_c``
(csrc/src/entrypoints.cpp:7-8, :9-12, :19-22), same names and arguments:

* ``swap_blocks`` / ``swap_blocks_new_kv_combined``  csrc/src/block_swapping.cpp:22-85, :88-202
* ``register_kv_cache_info`` / ``acquire_new_kvcache`` csrc/src/memory_manager.cpp:57-66, :69-176
* ``register_layer_memory_org_gpu`` / ``register_layer_memory_quant`` (:16-35) -- only as
  the bookkeeping ``acquire_new_kvcache`` reads.

The weight-swapping entries (``replace_layer_*`` and friends) are not part of
the KV path and raise ``NotImplementedError``.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Sequence, Tuple

import torch

from . import _capi
from .worker.kernels import _deferred
from .worker.kernels._pool import pool_strided

_kv_info: Dict[str, int] = {}
_layer_org_gpu: Dict[int, Tuple[int, int]] = {}
_layer_quant: Dict[int, Tuple[int, int]] = {}


def _ids(xs: Sequence[int]):
    arr = (C.c_int64 * len(xs))(*[int(x) for x in xs])
    return arr


def swap_blocks(source_block_ids: List[int], target_block_ids: List[int], is_swap_in: bool,
                k_cache: torch.Tensor, v_cache: torch.Tensor,
                k_swap: torch.Tensor, v_swap: torch.Tensor) -> int:
    """Copy blocks ``source[i] -> target[i]`` between the GPU pool and the CPU swap
    tensors on the current stream; consecutive runs become one copy pair.
    Returns the number of copy pairs issued."""
    assert len(source_block_ids) == len(target_block_ids)
    pool = _capi.make_pool(k_cache, v_cache)
    n = C.c_int64(0)
    _deferred.flush()
    _capi.check(_capi.lib().mkv_swap_blocks(
        _ids(source_block_ids), _ids(target_block_ids), len(source_block_ids),
        1 if is_swap_in else 0, C.byref(pool), k_swap.data_ptr(), v_swap.data_ptr(),
        C.byref(n), _capi.current_stream()))
    return n.value


def swap_blocks_new_kv_combined(source_block_ids: List[int], target_block_ids: List[int],
                                is_swap_in: bool, num_blocks_org: int, org_layer_param_size: int,
                                kv_cache_new_block_size: int, k_cache_element_size: int,
                                k_cache: torch.Tensor, v_cache: torch.Tensor,
                                k_swap: torch.Tensor, v_swap: torch.Tensor,
                                k_cache_new: torch.Tensor, v_cache_new: torch.Tensor) -> int:
    """As ``swap_blocks`` with GPU ids at or beyond ``num_blocks_org`` living in
    extension segments: segment j starts ``j * org_layer_param_size`` elements
    below ``k_cache_new`` (segment 0).  On swap-in the GPU address comes from the
    TARGET id."""
    assert len(source_block_ids) == len(target_block_ids)
    dev_ids = target_block_ids if is_swap_in else source_block_ids
    top = max((int(x) for x in dev_ids), default=-1)
    nseg = 0
    if top >= num_blocks_org:
        nseg = (top - num_blocks_org) // int(kv_cache_new_block_size) + 1
    pool = pool_strided(k_cache, v_cache, k_cache_new, v_cache_new, num_blocks_org,
                        org_layer_param_size, kv_cache_new_block_size, k_cache_element_size, nseg)
    n = C.c_int64(0)
    _deferred.flush()
    _capi.check(_capi.lib().mkv_swap_blocks(
        _ids(source_block_ids), _ids(target_block_ids), len(source_block_ids),
        1 if is_swap_in else 0, C.byref(pool), k_swap.data_ptr(), v_swap.data_ptr(),
        C.byref(n), _capi.current_stream()))
    return n.value


def register_kv_cache_info(num_layers: int, num_kv_heads: int, block_size: int, head_dim: int) -> None:
    _kv_info.update(num_layers=int(num_layers), num_kv_heads=int(num_kv_heads),
                    block_size=int(block_size), head_dim=int(head_dim))


def register_layer_memory_org_gpu(layer_id: int, start_addr_int: int, size: int) -> None:
    _layer_org_gpu[int(layer_id)] = (int(start_addr_int), int(size))


def register_layer_memory_quant(layer_id: int, start_addr_int: int, size: int) -> None:
    _layer_quant[int(layer_id)] = (int(start_addr_int), int(size))


class _RawDeviceMemory:
    """Non-owning view of device memory for ``torch.as_tensor``."""

    def __init__(self, address: int, shape: Tuple[int, ...], keepalive=None, typestr: str = "<f2"):
        self.__cuda_array_interface__ = {
            "shape": tuple(shape), "typestr": typestr, "data": (int(address), False),
            "version": 2, "strides": None,
        }
        self._keepalive = keepalive


def carve_segment(layer_base: int, org_bytes: int, quant_bytes: int):
    """``(k_start, num_blocks, v_start)`` for the registered cache geometry."""
    if not _kv_info:
        raise RuntimeError("KV cache info not registered")
    k0, s, v0 = C.c_uint64(0), C.c_int64(0), C.c_uint64(0)
    rc = _capi.lib().mkv_pool_carve_segment(
        layer_base, org_bytes, quant_bytes, _kv_info["num_layers"], _kv_info["num_kv_heads"],
        _kv_info["block_size"], _kv_info["head_dim"], C.byref(k0), C.byref(s), C.byref(v0))
    if rc == _capi.MKV_ENOSPC:
        raise RuntimeError("No space available for new KV cache blocks")
    _capi.check(rc)
    return k0.value, s.value, v0.value


def acquire_new_kvcache(layer_id: int, keepalive=None):
    """K and V segment tensors ``[S, L, Hkv, B, D]`` (non-owning views, zeroed)
    carved from the tail of a weight layer's memory that quantisation freed."""
    layer_id = int(layer_id)
    if layer_id not in _layer_org_gpu or layer_id not in _layer_quant:
        raise RuntimeError("Layer not found in memory maps")
    base, org_bytes = _layer_org_gpu[layer_id]
    _, quant_bytes = _layer_quant[layer_id]
    k0, s, v0 = carve_segment(base, org_bytes, quant_bytes)
    shape = (s, _kv_info["num_layers"], _kv_info["num_kv_heads"], _kv_info["block_size"],
             _kv_info["head_dim"])
    dev = torch.device("cuda", torch.cuda.current_device())
    k = torch.as_tensor(_RawDeviceMemory(k0, shape, keepalive), device=dev)
    v = torch.as_tensor(_RawDeviceMemory(v0, shape, keepalive), device=dev)
    nbytes = k.numel() * 2
    stream = _capi.current_stream()
    _capi.check(_capi.lib().mkv_fill_zero(k0, nbytes, stream))
    _capi.check(_capi.lib().mkv_fill_zero(v0, nbytes, stream))
    return k, v


def _not_kv_path(name):
    def fn(*_a, **_k):
        raise NotImplementedError(f"swiftllm_c.{name} belongs to weight-layer swapping, outside the paged-KV path")
    fn.__name__ = name
    return fn


for _n in ("register_layer_memory_org_cpu", "register_layer_memory_tensor_map_quant",
           "register_layer_memory_tensor_map_org", "replace_layer_org2quant",
           "replace_layer_quant2org", "get_freed_memory_size", "verify_tensor_continuity"):
    globals()[_n] = _not_kv_path(_n)
