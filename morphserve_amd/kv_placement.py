"""Where the V pool starts relative to the K pool.

The reference creates ``k_cache`` and ``v_cache`` as two allocations of the same shape
(MorphServe/worker/model.py:187-190).  A decode workgroup reads the K slab and the V slab of one
block back to back, at the SAME offset of the two pools; when the two bases also agree in their low
address bits the two reads meet in the same part of the memory system, and the gather over a large
pool runs 1-2 % slower than with the V pool a few KiB further on (which offset is the slow one depends
on where the driver placed the allocations, so it is measured, not assumed).

``allocate_kv_caches`` allocates V with a few KiB of slack, times the decode gather for a handful of
V offsets on the freshly allocated memory and returns V as the view that was fastest.  The tensors
have the reference's shapes and are contiguous; only ``v_cache.data_ptr()`` differs from a plain
allocation.  Off by default (``tune=False``: two plain allocations); ``tune=True`` does it for any pool of at
least ``MIN_BLOCKS_TO_TUNE`` blocks -- the effect was measured on 64-186 GiB pools; on a pool of a few hundred
MiB the probe only sees its own noise.  The decision is relative (a candidate against offset 0 on the same
allocation), no rate is assumed.

Which PHYSICAL memory backs the two tensors matters more than this offset and is not something two plain
allocations can choose: a pool that owns its memory (``vmm_pool.VmmKVPool``) places K and V in different memory
groups of the device instead (``mkv_arena_pair_grow``).
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, Sequence, Tuple

import torch

from . import _capi

# candidate V offsets in bytes (multiples of 4 KiB keep every slab's alignment)
CANDIDATE_OFFSETS = (0, 4096, 8192, 12288, 20480)
SLACK_BYTES = 32768
MIN_BLOCKS_TO_TUNE = 4096


def _probe_us(k_cache: torch.Tensor, v_cache: torch.Tensor, probe, layers: Sequence[int]) -> float:
    """Microseconds per launch of the decode attention over the probe batch (unsplit, no append)."""
    lib = _capi.lib()
    bt, ids, lens_t, q, o, n, hq = probe
    pool = _capi.make_pool(k_cache, v_cache)
    stream = _capi.current_stream()

    def run():
        for layer in layers:
            _capi.check(lib.mkv_paged_attn_decode(
                q.data_ptr(), o.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], ids.data_ptr(),
                lens_t.data_ptr(), n, hq, 0.088, layer, bt.shape[1] * 16, 1, None, None, stream))
    run()
    run()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(4):
        run()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (4 * len(layers))


def allocate_kv_caches(num_blocks: int, shape_tail: Tuple[int, int, int, int], device, zero_init: bool = True,
                       tune: bool = False, seed: int = 0) -> Tuple[torch.Tensor, torch.Tensor, Dict]:
    """``(k_cache, v_cache, info)`` with ``k_cache, v_cache : [num_blocks, L, Hkv, B, D]`` fp16."""
    L, hkv, bsz, d = shape_tail
    device = torch.device(device)
    supported = bsz == 16 and d == 128 and device.type == "cuda"
    tune = bool(tune and supported and num_blocks >= MIN_BLOCKS_TO_TUNE)
    return _allocate_and_probe(num_blocks, shape_tail, device, zero_init, tune, seed)


def _make_probe(num_blocks: int, shape_tail, device, seed: int):
    """The probe batch: as many sequences as put two workgroups on every CU, 64 blocks each, block ids drawn over
    the whole pool; one q head per kv head (the vector-ALU kernel reads memory exactly as the matrix one does)."""
    L, hkv, bsz, d = shape_tail
    n = max(1, 512 // hkv)
    per_seq = min(64, num_blocks // n)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    bt = torch.randperm(num_blocks, generator=gen)[:n * per_seq].to(torch.int32).view(n, per_seq).to(device)
    ids = torch.arange(n, dtype=torch.int32, device=device)
    lens_t = torch.full((n,), per_seq * 16, dtype=torch.int32, device=device)
    q = torch.zeros((n, hkv, d), dtype=torch.float16, device=device)
    o = torch.empty((n, hkv, d), dtype=torch.float16, device=device)
    layers = list(range(0, L, max(1, L // 4)))[:4]
    probe_bytes = n * per_seq * hkv * 2 * bsz * d * 2                 # every K and V slab of the probe batch once
    return (bt, ids, lens_t, q, o, n, hkv), layers, probe_bytes


def probe_gather_GBs(k_cache: torch.Tensor, v_cache: torch.Tensor, seed: int = 0) -> float:
    """GB/s of the probe gather over an existing pool (best of three passes): the figure ``allocate_kv_caches``
    compares with its threshold, for pools whose memory is obtained in another way."""
    num_blocks = int(k_cache.shape[0])
    shape_tail = tuple(int(x) for x in k_cache.shape[1:])
    probe, layers, probe_bytes = _make_probe(num_blocks, shape_tail, k_cache.device, seed)
    best = min(_probe_us(k_cache, v_cache, probe, layers) for _ in range(3))
    return round(probe_bytes / best / 1e3, 1)


def _allocate_and_probe(num_blocks: int, shape_tail, device, zero_init: bool, tune: bool, seed: int):
    L, hkv, bsz, d = shape_tail
    alloc = torch.zeros if zero_init else torch.empty
    shape = (num_blocks, L, hkv, bsz, d)
    numel = num_blocks * L * hkv * bsz * d
    k_cache = alloc(shape, dtype=torch.float16, device=device)
    info: Dict = {"v_offset_bytes": 0, "tuned": False}
    if not tune:
        return k_cache, alloc(shape, dtype=torch.float16, device=device), info
    v_flat = alloc(numel + SLACK_BYTES // 2, dtype=torch.float16, device=device)
    probe, layers, probe_bytes = _make_probe(num_blocks, shape_tail, device, seed)
    timings = {off: float("inf") for off in CANDIDATE_OFFSETS}
    for _ in range(3):                              # candidates in turn, three times over: the best of each
        for off in CANDIDATE_OFFSETS:
            v_view = v_flat[off // 2: off // 2 + numel].view(shape)
            timings[off] = min(timings[off], _probe_us(k_cache, v_view, probe, layers))
    best = min(timings, key=timings.get)
    if timings[best] > 0.995 * timings[0]:          # within the noise of the probe: keep the plain placement
        best = 0
    info = {"v_offset_bytes": best, "tuned": True,
            "probe_us_per_launch": {str(k): round(v, 2) for k, v in timings.items()},
            "probe_GBs": round(probe_bytes / timings[best] / 1e3, 1)}
    return k_cache, v_flat[best // 2: best // 2 + numel].view(shape), info
