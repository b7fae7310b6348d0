"""ctypes loader for the C restatement.  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import ref_cpu as R

_lib = None


class OraLayout(C.Structure):
    _fields_ = [(n, C.c_int64) for n in ("num_layers", "num_kv_heads", "block_size", "head_dim",
                                         "k_base", "v_base", "num_blocks_org", "seg_blocks",
                                         "num_segments")] + [("k_seg", C.c_void_p), ("v_seg", C.c_void_p)]


def lib():
    global _lib
    if _lib is None:
        from .build import LIB_PATH, build_oracle
        if not os.path.exists(LIB_PATH):
            build_oracle(verbose=False)
        _lib = C.CDLL(LIB_PATH)
        _lib.ora_take_first_free.restype = C.c_int64
        _lib.ora_block_offset.restype = C.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class CLayout:
    """Keeps the per-segment offset arrays alive next to the C struct."""

    def __init__(self, lay: R.PoolLayout, num_segments: int = 0):
        if lay.k_seg is not None:
            ks, vs = list(lay.k_seg), list(lay.v_seg)
        else:
            ks = [lay.k_new0 - j * lay.org_layer_param_size for j in range(num_segments)]
            vs = [lay.v_new0 - j * lay.org_layer_param_size for j in range(num_segments)]
        self.ks = np.asarray(ks, dtype=np.int64)
        self.vs = np.asarray(vs, dtype=np.int64)
        self.c = OraLayout(lay.num_layers, lay.num_kv_heads, lay.block_size, lay.head_dim,
                           lay.k_base, lay.v_base, lay.num_blocks_org, lay.seg_blocks, len(ks),
                           _p(self.ks), _p(self.vs))

    def ref(self):
        return C.byref(self.c)


def append_decode(arena, cl, k, v, table, seq_ids, seq_lens, layer):
    lib().ora_append_decode(_p(arena), cl.ref(), _p(np.ascontiguousarray(k)), _p(np.ascontiguousarray(v)),
                            _p(table), C.c_int64(table.shape[1]), _p(seq_ids), _p(seq_lens),
                            C.c_int64(len(seq_ids)), C.c_int64(layer))


def append_prefill(arena, cl, k, v, table, seq_ids, starts, lens, layer):
    lib().ora_append_prefill(_p(arena), cl.ref(), _p(np.ascontiguousarray(k)), _p(np.ascontiguousarray(v)),
                             _p(table), C.c_int64(table.shape[1]), _p(seq_ids), _p(starts), _p(lens),
                             C.c_int64(len(seq_ids)), C.c_int64(layer))


def paged_attention(q, arena, cl, table, seq_ids, seq_lens, scale, layer):
    q = np.ascontiguousarray(q)
    o = np.empty_like(q)
    lib().ora_paged_attention(_p(q), _p(o), _p(arena), cl.ref(), _p(table), C.c_int64(table.shape[1]),
                              _p(seq_ids), _p(seq_lens), C.c_int64(q.shape[0]), C.c_int64(q.shape[1]),
                              C.c_float(scale), C.c_int64(layer))
    return o


def take_first_free(is_free_u8, n):
    out = np.empty(max(n, 1), dtype=np.int64)
    found = lib().ora_take_first_free(_p(is_free_u8), C.c_int64(len(is_free_u8)), C.c_int64(n), _p(out))
    return out[:min(found, n)], found


def migrate(arena, cl, src, dst):
    src = np.ascontiguousarray(src, dtype=np.int64)
    dst = np.ascontiguousarray(dst, dtype=np.int64)
    lib().ora_migrate(_p(arena), cl.ref(), _p(src), _p(dst), C.c_int64(len(src)))
