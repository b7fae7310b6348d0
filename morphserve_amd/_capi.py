"""ctypes binding of ``libmorphkv.so`` (see ``include/morphkv.h``).

The library is the only compute path of this package: when it cannot be loaded
the import of any operator raises; there is no CPU or eager fallback.

``diag_lib()`` loads ``libmorphkv_diag.so``, the diagnostic twin built from the same sources
(``include/morphkv_diag.h``: kernel-variant switches, per-launch event timing, per-workgroup time
stamps, calibration loops).  Nothing in this package calls it; benchmarks and tests do, either
directly or by routing the package's operators through it for a while with ``use_diag_library()``.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import os
from typing import Optional, Sequence

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmorphkv.so")
DIAG_LIB_PATH = os.path.join(_HERE, "csrc", "libmorphkv_diag.so")

MKV_OK, MKV_EINVAL, MKV_EHIP, MKV_ENOSPC, MKV_ELOGIC = 0, -1, -2, -3, -4
MKV_MAX_SEGMENTS = 128

K_APPEND_DECODE, K_APPEND_PREFILL, K_ATTN_PHASE1, K_ATTN_PHASE2 = 0, 1, 2, 3
K_MIGRATE, K_PREFILL_ATTN, K_FILL_ZERO, K_SWAP, K_ROPE_STORE = 4, 5, 6, 7, 8


class MkvPool(C.Structure):
    _fields_ = [
        ("k_base", C.c_void_p),
        ("v_base", C.c_void_p),
        ("num_blocks_org", C.c_int64),
        ("seg_blocks", C.c_int64),
        ("num_segments", C.c_int32),
        ("num_layers", C.c_int32),
        ("num_kv_heads", C.c_int32),
        ("block_size", C.c_int32),
        ("head_dim", C.c_int32),
        ("_pad", C.c_int32),
        ("k_seg", C.c_void_p * MKV_MAX_SEGMENTS),
        ("v_seg", C.c_void_p * MKV_MAX_SEGMENTS),
    ]


class MkvPairInfo(C.Structure):
    """``mkv_pair_info``: what a memory-group aware growth found (include/morphkv.h)."""
    _fields_ = [
        ("groups_found", C.c_int32),
        ("candidates", C.c_int32),
        ("k_chunks", C.c_int32),
        ("v_chunks", C.c_int32),
        ("k_in_group", C.c_int32),
        ("v_in_group", C.c_int32),
        ("probes", C.c_int32),
        ("_pad", C.c_int32),
        ("probe_ms", C.c_double),
        ("total_ms", C.c_double),
        ("released_bytes", C.c_uint64),
    ]


_P = C.c_void_p
_I32 = C.c_int32
_I64 = C.c_int64
_U64 = C.c_uint64
_F32 = C.c_float
_PP = C.POINTER(MkvPool)

# name -> argtypes (restype is int unless listed in _RESTYPES)
PROTOTYPES = {
    "mkv_last_error": [],
    "mkv_version": [],
    "mkv_sizeof_pool": [],
    "mkv_pool_set_strided": [_PP, _P, _P, _I64, _I32, _I32],
    "mkv_append_decode": [_P, _P, _PP, _P, _I64, _P, _P, _I32, _I32, _P],
    "mkv_append_prefill": [_P, _P, _PP, _P, _I64, _P, _P, _P, _I32, _I32, _I32, _P],
    "mkv_paged_attn_scratch_bytes": [_I32, _I32, _I32, _I32, C.POINTER(_I64), C.POINTER(_I64)],
    "mkv_paged_attn_decode": [_P, _P, _PP, _P, _I64, _P, _P, _I32, _I32, _F32, _I32, _I32, _I32, _P, _P, _P],
    "mkv_decode_order": [_P, _I32, _I32, _P, _P],
    "mkv_decode_attn_ordered": [_P, _P, _PP, _P, _I64, _P, _P, _P, _I32, _I32, _F32, _I32, _I32, _I32, _P, _P, _P, _P,
                                _P, _P, _P],
    "mkv_paged_attn_decode_static": [_P, _P, _PP, _P, _I64, _P, _P, _I32, _I32, _F32, _I32, _I32, _I32, _P],
    "mkv_decode_append_attn": [_P, _P, _P, _P, _PP, _P, _I64, _P, _P, _I32, _I32, _F32, _I32, _I32, _I32, _P, _P, _P],
    "mkv_decode_rope_append_attn": [_P, _P, _P, _P, _P, _P, _PP, _P, _I64, _P, _P, _I32, _I32, _F32, _I32, _I32, _I32,
                                    _P, _P, _P],
    "mkv_prefill_attn": [_P, _P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _F32, _P],
    "mkv_prefill_attn_paged": [_P, _P, _PP, _P, _I64, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _F32, _I32, _P],
    "mkv_bm_allocate": [_P, _I64, _P, _I64, _P, _I64, _P, _P, _I32, _I32, _P, _I64, _P, _P],
    "mkv_bm_take_first_free": [_P, _I64, _I64, _P, _P, _P],
    "mkv_bt_append": [_P, _I64, _P, _I64, _P, _P, _P, _I32, _I32, _P],
    "mkv_bt_release": [_P, _I64, _P, _I64, _P, _I32, _P, _I64, _P, _P],
    "mkv_bt_gather_release": [_P, _I64, _P, _I64, _P, _I32, _P, _I64, _P, _I64, _P, _P],
    "mkv_pool_carve_segment": [_U64, _U64, _U64, _I32, _I32, _I32, _I32, C.POINTER(_U64),
                               C.POINTER(_I64), C.POINTER(_U64)],
    "mkv_fill_zero": [_P, _U64, _P],
    "mkv_bm_count_live": [_P, _I64, _I64, _P, _P],
    "mkv_pool_plan_shrink": [_P, _I64, _I64, _P, _P, _I64, _P, _P, _P],
    "mkv_pool_migrate": [_PP, _P, _P, _I64, _P],
    "mkv_bt_remap": [_P, _I64, _P, _I64, _P, _I64, _P],
    "mkv_arena_create": [_U64, _U64, C.POINTER(_P)],
    "mkv_arena_info": [_P, C.POINTER(_P), C.POINTER(_U64), C.POINTER(_U64), C.POINTER(_U64)],
    "mkv_arena_resize": [_P, _U64],
    "mkv_arena_destroy": [_P],
    "mkv_arena_move_tail": [_P, _P, _U64],
    "mkv_arena_pair_grow": [_P, _P, _U64, _U64, _U64, _P, C.POINTER(MkvPairInfo)],
    "mkv_rope_store_kvcache": [_P, _P, _P, _P, _P, _PP, _P, _I64, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32,
                               _I32, _I32, _I32, _P],
    "mkv_swap_blocks": [_P, _P, _I64, _I32, _PP, _P, _P, C.POINTER(_I64), _P],
    "mkv_swap_blocks_device_ids": [_P, _P, _I64, _I32, _PP, _P, _P, _I64, _P],
}
# entries of the diagnostic twin only (include/morphkv_diag.h)
DIAG_PROTOTYPES = {
    "mkv_set_decode_variant": [_I32],
    "mkv_set_prefill_variant": [_I32],
    "mkv_diag_mfma_loop": [_I32, _I32, _P, _P, C.POINTER(C.c_double), _P],
    "mkv_diag_timeline": [_P, _I64],
    "mkv_diag_slab_gather": [_P, _P, _U64, _I32, _I32, _I32, _I32, _I32, C.c_uint32, _P, _P],
    "mkv_diag_split_by_rate": [C.POINTER(C.c_double), _I64, C.c_double, C.POINTER(C.c_uint8)],
    "mkv_prof_enable": [_I32],
    "mkv_prof_reset": [],
    "mkv_prof_collect": [_I32, C.POINTER(_I64), C.POINTER(C.c_double)],
}
_RESTYPES = {"mkv_last_error": C.c_char_p}

_lib: Optional[C.CDLL] = None
_diag_lib: Optional[C.CDLL] = None


class MorphKVError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"morphkv error {code}: {message}")
        self.code = code


def _load(path: str, prototypes) -> C.CDLL:
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m morphserve_amd.csrc.build` "
            "(there is no fallback path)")
    handle = C.CDLL(path)
    for name, argtypes in prototypes.items():
        fn = getattr(handle, name)
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, C.c_int)
    if handle.mkv_sizeof_pool() != C.sizeof(MkvPool):
        raise ImportError("mkv_pool layout of the library does not match this binding")
    return handle


def lib() -> C.CDLL:
    """Load the library (once).  Raises when it has not been built."""
    global _lib
    if _lib is None:
        path = os.environ.get("MORPHKV_LIBRARY") or LIB_PATH     # another build of the same ABI, for A/B runs
        _lib = _load(path, PROTOTYPES)
    return _lib


def diag_lib() -> C.CDLL:
    """Load the diagnostic twin (once): every entry of ``lib()`` plus ``DIAG_PROTOTYPES``."""
    global _diag_lib
    if _diag_lib is None:
        _diag_lib = _load(os.environ.get("MORPHKV_DIAG_LIBRARY") or DIAG_LIB_PATH,
                          {**PROTOTYPES, **DIAG_PROTOTYPES})
    return _diag_lib


@contextlib.contextmanager
def use_diag_library():
    """Route every call of this package through the diagnostic twin inside the ``with`` block
    (measurement and tests; process-wide, so not while other threads are issuing calls)."""
    global _lib
    lib()
    saved, _lib = _lib, diag_lib()
    try:
        yield _lib
    finally:
        _lib = saved


def check(rc: int) -> None:
    if rc != MKV_OK:
        raise MorphKVError(rc, lib().mkv_last_error().decode("utf-8", "replace"))


def current_stream() -> int:
    import torch
    return torch.cuda.current_stream().cuda_stream


_hip_runtime = None


def capture_id(stream: int) -> Optional[int]:
    """Id of the graph capture ``stream`` is recording into, ``None`` when it is not capturing
    (``hipStreamGetCaptureInfo`` of the HIP runtime torch has already loaded)."""
    global _hip_runtime
    if _hip_runtime is None:
        _hip_runtime = C.CDLL("libamdhip64.so")
        _hip_runtime.hipStreamGetCaptureInfo.argtypes = [_P, C.POINTER(C.c_int), C.POINTER(C.c_ulonglong)]
        _hip_runtime.hipStreamGetCaptureInfo.restype = C.c_int
    status = C.c_int(0)
    cid = C.c_ulonglong(0)
    rc = _hip_runtime.hipStreamGetCaptureInfo(stream, C.byref(status), C.byref(cid))
    if rc != 0:
        raise MorphKVError(MKV_EHIP, f"hipStreamGetCaptureInfo failed with HIP error {rc}")
    return int(cid.value) if status.value == 1 else None      # 1 = hipStreamCaptureStatusActive


def ptr(t) -> int:
    """Device (or host) address of a tensor's first element; views keep their offset."""
    return 0 if t is None else t.data_ptr()


def make_pool(k_cache, v_cache, k_segments: Sequence = (), v_segments: Sequence = (),
              num_blocks_org: Optional[int] = None, seg_blocks: int = 0) -> MkvPool:
    """Describe a pool: base tensors ``[blocks, L, Hkv, B, D]`` plus extension
    segments given as tensors (their own addresses are used)."""
    assert k_cache.dim() == 5 and v_cache.shape == k_cache.shape
    p = MkvPool()
    p.k_base = k_cache.data_ptr()
    p.v_base = v_cache.data_ptr()
    p.num_blocks_org = k_cache.shape[0] if num_blocks_org is None else num_blocks_org
    p.num_layers, p.num_kv_heads, p.block_size, p.head_dim = (int(x) for x in k_cache.shape[1:])
    nseg = len(k_segments)
    if nseg > MKV_MAX_SEGMENTS:
        raise ValueError(f"at most {MKV_MAX_SEGMENTS} extension segments are supported")
    p.num_segments = nseg
    p.seg_blocks = int(seg_blocks) if nseg else 0
    for j in range(nseg):
        p.k_seg[j] = k_segments[j].data_ptr()
        p.v_seg[j] = v_segments[j].data_ptr()
    return p


def prof_enable(on: bool) -> None:
    """Per-launch event timing of the DIAGNOSTIC twin (calls must go through it: ``use_diag_library()``)."""
    check(diag_lib().mkv_prof_enable(1 if on else 0))


def prof_reset() -> None:
    check(diag_lib().mkv_prof_reset())


def prof_collect(kernel_id: int):
    """(launches, total_ms) of one instrumented kernel since the last reset."""
    n = _I64(0)
    ms = C.c_double(0.0)
    check(diag_lib().mkv_prof_collect(kernel_id, C.byref(n), C.byref(ms)))
    return n.value, ms.value
