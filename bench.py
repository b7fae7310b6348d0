"""Benchmark of the paged-KV hot path on one MI355X.

Default workload (``cfg2_llama3_8b_decode``): Llama-3-8B-shaped decode -- 32
layers, GQA 32 q / 8 kv heads, head_dim 128, block_size 16, batch 64, contexts
uniform in [1024, 1536], KV pool of 65 536 blocks (128 GiB) with randomly
permuted block tables, Q/K/V ~ N(0,1).  One step = for every layer: append one
token per sequence to the paged cache, then paged decode attention.

Prints ONE JSON line: whole-step throughput in algorithmic HBM GB/s (inputs
resident in HBM), the roofline of the dominant kernel (decode attention phase 1,
timed per launch with HIP events on its own stream) and a CPU baseline (the
oracle's torch-CPU statement of the same path on a bounded sample).  The default
line also carries the pool resize of config 3 (``"resize"``), measured in the same
process.

``--workload cfg3_resize`` measures the elastic pool alone: grow 32k -> 96k
blocks (zero fill), scatter ~24.5k live blocks, shrink to 40k with migration.
``--workload placement_ab`` creates, measures (decode and resize) and frees pools
with and without memory-group placement several times in ONE process, at once
and after a pause: the evidence that the figures do not hang on allocation history.

The pool is a ``VmmKVPool`` with K and V placed in different memory groups of the
device (``--pool-backing torch`` / ``--placement plain`` give the other layouts).
Everything that is timed runs on ``libmorphkv.so``; per-kernel breakdowns of steps
that launch several kernels go through its diagnostic twin and are labelled so.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.modules.setdefault("bench", sys.modules[__name__])     # bench_workloads imports this module by name, run as a script or not

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_per_launch.md")


def measured_traffic(key):
    """HBM bytes per launch of a workload's dominant kernel, from the committed table of FETCH_SIZE /
    WRITE_SIZE counter runs (counters cannot be collected from inside this process); None when the
    table has no row for exactly this workload and arguments."""
    try:
        for line in open(TRAFFIC_TABLE):
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) >= 3 and cells[0] == key:
                return int(cells[2].replace(" ", "").replace(",", ""))
    except OSError:
        pass
    return None


class Cfg:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg2_llama3_8b_decode",
                    choices=["cfg2_llama3_8b_decode", "cfg1_llama2_7b_layer", "cfg5_codellama34b_decode", "cfg3_resize",
                             "cfg4_mixed", "cfg4_serving", "cfg5_pressure_shrink", "placement_ab", "copy_calibration",
                             "mfma_calibration", "eviction", "prefill_shapes", "layer_handover", "step_state",
                             "allocator"])
    ap.add_argument("--pool-blocks", type=int, default=0, help="0 = the workload's own pool size")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of a HIP graph replay")
    ap.add_argument("--unfused", action="store_true",
                    help="time store_kvcache + paged_attention as two calls per layer (default: the fused "
                         "one-launch-per-layer call)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ctx", type=int, nargs=2, default=None, metavar=("LO", "HI"),
                    help="decode workloads: context lengths are uniform in [LO, HI] (default: the workload's, "
                         "[1024, 1536] or, for cfg1, [64, 512])")
    ap.add_argument("--no-resize", action="store_true",
                    help="default workload only: skip the pool-resize measurement that follows the decode one")
    ap.add_argument("--batch", type=int, default=0, help="decode workloads: number of sequences (0 = the workload's)")
    ap.add_argument("--tables", choices=["permuted", "identity"], default="permuted",
                    help="decode workloads: block tables dealt from a seeded permutation of the pool (the "
                         "benchmark's definition) or in id order (diagnostic only)")
    ap.add_argument("--pool-backing", choices=["vmm", "torch"], default="vmm",
                    help="the pool is one tensor over HIP virtual memory whose physical chunks the library places "
                         "(VmmKVPool, default) or two torch allocations plus segments (ElasticKVPool)")
    ap.add_argument("--placement", choices=["groups", "plain"], default="groups",
                    help="with --pool-backing vmm: K and V chunks from different memory groups of the device "
                         "(default) or in the order the driver hands them out")
    ap.add_argument("--vmm-chunk-blocks", type=int, default=0,
                    help="with --pool-backing vmm: blocks per physical allocation (must divide the pool size; "
                         "0 = the largest divisor that keeps a chunk at or under 1 GiB per tensor)")
    ap.add_argument("--v-stagger-bytes", type=int, default=0,
                    help="with --pool-backing vmm: how far into its range the V tensor starts (a multiple of 4096)")
    ap.add_argument("--no-wipe-wait", action="store_true",
                    help="decode workloads, diagnostic: start measuring right after pool creation instead of waiting for "
                         "the driver to wipe the candidate memory that creation gave back")
    ap.add_argument("--ab-pause", type=float, default=10.0,
                    help="placement_ab workload: seconds between the second free and the third allocation")
    ap.add_argument("--prefill-shapes", default="8x512,4x4096,2x8192,1x16384",
                    help="prefill_shapes workload: comma-separated SEQSxTOKENS prompt batches; SEQSxTOKENS+PREFIX is a "
                         "batch of chunks over PREFIX tokens already in a paged cache")
    ap.add_argument("--prefill-data", choices=["randn", "zeros"], default="randn",
                    help="prefill_shapes workload: N(0,1) inputs (default) or all-zero inputs -- the same instruction "
                         "stream without switching activity in the matrix pipe, to show what the power limit costs")
    ap.add_argument("--prefill-variants", default="0",
                    help="prefill_shapes workload: workgroup shapes to time (0 = the library's own choice by prompt "
                         "length, on the product library; 4 = four waves / 128 query rows, 8 = eight waves / 256 query "
                         "rows: forced through the diagnostic twin)")
    ap.add_argument("--seed", type=int, default=2)
    args = ap.parse_args()
    if args.ctx is None:
        args.ctx = [64, 512] if args.workload == "cfg1_llama2_7b_layer" else [1024, 1536]
    return args


# ---------------------------------------------------------------------------------
def decode_bytes_per_layer(lens, n, hq, hkv, d, b):
    """Algorithmic HBM bytes of one layer: every K/V slab once, q, o, table; plus the append."""
    lens = np.asarray(lens, dtype=np.int64)
    attn = int(lens.sum()) * 2 * hkv * d * 2 + 2 * n * hq * d * 2 + int(((lens + b - 1) // b).sum()) * 4
    append = 2 * (n * 2 * hkv * d * 2)            # read k, v rows + write them into the cache
    return attn, append


def auto_chunk_blocks(num_blocks, bytes_per_block_and_tensor):
    """Blocks per chunk for a pool of num_blocks: the largest count whose chunk is a multiple of 2 MiB and at
    most 1 GiB per tensor, a divisor of num_blocks when one exists that gives chunks of 256 MiB and more (what
    placement by memory groups needs), else the largest such count (the pool then maps whole chunks past
    num_blocks)."""
    target = max(1, (1 << 30) // bytes_per_block_and_tensor)
    aligned = [c for c in range(min(target, num_blocks), 0, -1) if (c * bytes_per_block_and_tensor) % (2 << 20) == 0]
    if not aligned:
        return 1
    for c in aligned:
        if num_blocks % c == 0 and c * bytes_per_block_and_tensor >= (256 << 20):
            return c
    return aligned[0]


def make_pool(args, num_blocks, max_blocks, L, HKV, B, D, max_seqs, max_blocks_per_seq):
    """The KV pool of a workload by --pool-backing / --placement; (pool, description).  A virtual-memory pool
    holds whole chunks: its block counts are the workload's rounded up to the chunk."""
    from morphserve_amd import ElasticKVPool, VmmKVPool
    if args.pool_backing == "vmm":
        per_tensor = L * HKV * B * D * 2
        chunk = args.vmm_chunk_blocks or auto_chunk_blocks(int(np.gcd(num_blocks, max_blocks)), per_tensor)
        asked = num_blocks
        num_blocks, max_blocks = -(-num_blocks // chunk) * chunk, -(-max_blocks // chunk) * chunk
        pool = VmmKVPool(num_blocks, max_blocks, L, HKV, B, D, max_seqs, max_blocks_per_seq, chunk_blocks=chunk,
                         placement=args.placement, v_stagger_bytes=args.v_stagger_bytes)
        what = (f"VmmKVPool, chunks of {chunk} blocks ({chunk * per_tensor / 2**20:.0f} MiB per tensor), placement "
                f"{args.placement}" + (f", {num_blocks} blocks mapped for the {asked} used" if num_blocks != asked else ""))
    else:
        pool = ElasticKVPool(num_blocks, L, HKV, B, D, max_seqs, max_blocks_per_seq, reserve_blocks=max_blocks)
        what = "ElasticKVPool: two torch allocations, growth by segments"
    return pool, what


WIPE_SECONDS_PER_GIB = 0.04
PROCESS_START = time.perf_counter()
_wipe_done_at = None          # when the driver will have wiped everything this process knows to have been released


def note_release(nbytes):
    """Memory went back to the driver just now: it is wiped in the background, one release after the other."""
    global _wipe_done_at
    now = time.perf_counter()
    _wipe_done_at = max(_wipe_done_at or now, now) + nbytes / 2 ** 30 * WIPE_SECONDS_PER_GIB


def pool_bytes(pool):
    return 2 * pool.num_blocks * pool.block_bytes


def wait_for_driver_wipe(pool):
    """The driver wipes released memory in the background (about 30 ms per GiB on this system; an allocation
    that needs such memory waits for it, which is how the rate shows), and while that runs every kernel is a
    few per cent slower: a measurement that starts right after a release would time the driver's wipe, not the
    pool.  Releases happen when a pool is created with memory-group placement (the candidate chunks it did
    not keep), when this program closes a pool, and when a process that ended just before this one gave its
    memory back, which nothing here can see.  A server creates its pool long before the first request; the
    benchmark waits here until all of that would be wiped: a time computed from the bytes released and, for
    the invisible case, from the size of the whole device counted from this process's own start.  Nothing is
    measured or compared to decide it.  Returns the seconds waited."""
    import torch
    note_release(sum(g.get("released_bytes", 0) for g in pool.kv_placement.get("growths", [])))
    whole_device = PROCESS_START + torch.cuda.mem_get_info()[1] / 2 ** 30 * WIPE_SECONDS_PER_GIB
    wait = max(_wipe_done_at, whole_device) - time.perf_counter()
    if wait > 0:
        time.sleep(wait)
    return round(max(wait, 0.0), 2)


def diag_kernel_times(fn, kernel_ids):
    """{kernel id: (launches, total ms)} of one pass of fn() routed through the DIAGNOSTIC twin of the library,
    which brackets every launch of the listed kernels with an event pair (same sources, same kernels; the
    figures that are reported as results are always timed on the product library)."""
    import torch
    from morphserve_amd import _capi
    with _capi.use_diag_library():
        _capi.prof_reset()
        _capi.prof_enable(True)
        try:
            fn()
            torch.cuda.synchronize()
            out = {kid: _capi.prof_collect(kid) for kid in kernel_ids}
        finally:
            _capi.prof_enable(False)
            _capi.prof_reset()
    return out


def _balanced_order():
    from morphserve_amd.worker.kernels import paged_attn as PA
    return bool(PA.BALANCED_ORDER)


def bench_decode(args):
    import torch
    from morphserve_amd import (_capi, build_infer_state, decode_append_and_attend, paged_attention,
                                store_kvcache)

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.workload == "cfg5_codellama34b_decode":
        # 48 layers, GQA 64 q / 8 kv heads, batch 128, pool ~200 GB of 3 MiB blocks
        L, HQ, HKV, D, B, N = 48, 64, 8, 128, 16, 128
        default_blocks = 63578
    elif args.workload == "cfg1_llama2_7b_layer":
        # one Llama-2-7B-shaped layer: MHA 32 / 32 heads, batch 8, pool of 4096 blocks of 256 KiB (1 GiB)
        L, HQ, HKV, D, B, N = 1, 32, 32, 128, 16, 8
        default_blocks = 4096
    else:
        L, HQ, HKV, D, B, N = 32, 32, 8, 128, 16, 64
        default_blocks = 65536
    rng = np.random.default_rng(args.seed)
    if args.batch:
        N = args.batch
    lens = rng.integers(args.ctx[0], args.ctx[1] + 1, size=N).astype(np.int32)
    nblk = (lens.astype(np.int64) + B - 1) // B
    num_blocks = args.pool_blocks or default_blocks
    max_blocks_per_seq = max(128, -(-args.ctx[1] // B))
    max_seqs = max(256, N)

    # block tables: a seeded permutation of the whole pool dealt in order
    perm = rng.permutation(num_blocks)
    if args.tables == "identity":                 # diagnostic: blocks in id order, no gather scatter
        perm = np.arange(num_blocks)
    seq_ids = rng.permutation(max_seqs)[:N].astype(np.int32)
    table = np.full((max_seqs, max_blocks_per_seq), -1, dtype=np.int32)
    pos = 0
    for i in range(N):
        table[seq_ids[i], :nblk[i]] = perm[pos:pos + nblk[i]]
        pos += nblk[i]
    live = perm[:pos].copy()

    shape = (num_blocks, L, HKV, B, D)
    t_pool = time.perf_counter()
    kv_pool, pool_what = make_pool(args, num_blocks, num_blocks, L, HKV, B, D, max_seqs, max_blocks_per_seq)
    torch.cuda.synchronize()
    pool_creation_s = time.perf_counter() - t_pool
    wiped_s = 0.0 if args.no_wipe_wait else wait_for_driver_wipe(kv_pool)
    k_cache, v_cache = kv_pool.k_cache, kv_pool.v_cache
    kv_placement = kv_pool.kv_placement
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    live_t = torch.from_numpy(live).to(dev)
    for c0 in range(0, len(live), 256):           # N(0,1) in the live blocks, 256 blocks at a time
        idx = live_t[c0:c0 + 256]
        k_cache[idx] = torch.randn((len(idx), *shape[1:]), dtype=torch.float16, device=dev, generator=g)
        v_cache[idx] = torch.randn((len(idx), *shape[1:]), dtype=torch.float16, device=dev, generator=g)
    bt = torch.from_numpy(table).to(dev)
    q = torch.randn((L, N, HQ, D), dtype=torch.float16, device=dev, generator=g)
    k_new = torch.randn((L, N, HKV, D), dtype=torch.float16, device=dev, generator=g)
    v_new = torch.randn((L, N, HKV, D), dtype=torch.float16, device=dev, generator=g)
    o = torch.empty((L, N, HQ * D), dtype=torch.float16, device=dev)

    model = Cfg(num_layers=L, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    engine = Cfg(block_size=B, max_blocks_per_seq=max_blocks_per_seq)
    st = build_infer_state([], seq_ids.tolist(), lens.tolist(), HKV, D)

    def new_step():
        # a serving loop builds its infer_state per step: what the wrappers keep on it (the balanced row
        # order, one small launch) is recomputed in every timed step, inside the graph too
        st.__dict__.pop("_morphkv_decode_order", None)

    def step_two_calls():
        new_step()
        for layer in range(L):
            store_kvcache(k_new[layer], v_new[layer], k_cache, v_cache, [], [], bt, model, engine, st, layer)
            paged_attention(q[layer], k_cache, v_cache, [], [], bt, model, engine, st, layer, o[layer])

    def step_fused():
        new_step()
        for layer in range(L):
            decode_append_and_attend(k_new[layer], v_new[layer], q[layer], k_cache, v_cache, [], [], bt,
                                     model, engine, st, layer, o[layer])

    step = step_two_calls if args.unfused else step_fused
    other = step_fused if args.unfused else step_two_calls

    # -- warmup, then the timed region --------------------------------------------------
    for _ in range(max(args.warmup, 1)):
        step()
    torch.cuda.synchronize()

    graph = None
    # a one-layer step is two or three launches: replaying it as a graph costs more than launching it
    if not args.no_graph and args.workload != "cfg1_llama2_7b_layer":
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        graph.replay()
        torch.cuda.synchronize()
    run = graph.replay if graph is not None else step

    def timed_ms(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    ms_per_step = timed_ms(run)
    # the other call shape under the same conditions (a graph of its own), for the record
    other_graph_ms = None
    if graph is not None:
        other()
        torch.cuda.synchronize()
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2):
            other()
        graph2.replay()
        torch.cuda.synchronize()
        other_graph_ms = timed_ms(graph2.replay)
        del graph2
    # the two-call shape with store_kvcache's decode rows deferred into the paged_attention that follows
    deferred_graph_ms = None
    if graph is not None:
        import morphserve_amd
        morphserve_amd.enable_deferred_decode_append(True)
        try:
            step_two_calls()
            torch.cuda.synchronize()
            graph3 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph3):
                step_two_calls()
            graph3.replay()
            torch.cuda.synchronize()
            deferred_graph_ms = timed_ms(graph3.replay)
            del graph3
        finally:
            morphserve_amd.enable_deferred_decode_append(False)

    # eager step time too (CPU launch overhead included), and the other call shape, for the record
    reps = max(3, args.steps // 4)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) * 1e3 / reps
    other()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        other()
    torch.cuda.synchronize()
    other_ms = (time.perf_counter() - t0) * 1e3 / reps

    # -- dominant kernel: per-launch duration with HIP events on its stream -------------
    # Which kernels a step launches, and each one's share, from one pass through the diagnostic twin
    # (every launch bracketed by its own event pair, the pair's own cost included) ...
    def three_steps():
        for _ in range(3):
            step()
    kt = diag_kernel_times(three_steps, (_capi.K_ATTN_PHASE1, _capi.K_ATTN_PHASE2, _capi.K_APPEND_DECODE))
    (launches, total_ms), (p2_launches, p2_ms), (ap_launches, ap_ms) = (
        kt[_capi.K_ATTN_PHASE1], kt[_capi.K_ATTN_PHASE2], kt[_capi.K_APPEND_DECODE])
    bracketed_ms = total_ms / max(launches, 1)
    # ... and, when a step is nothing but launches of that kernel (fused call, one split), the figure that
    # is reported: one event pair around whole steps of the PRODUCT library, elapsed / launches
    phase1_ms = bracketed_ms
    timing = "event pair around every launch (diagnostic twin of the library)"
    if not args.unfused and p2_launches == 0 and ap_launches == 0:
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.steps):
            step()
        e1.record()
        torch.cuda.synchronize()
        phase1_ms = e0.elapsed_time(e1) / (args.steps * L)
        launches = args.steps * L
        timing = "one event pair around back-to-back launches of this kernel only"

    attn_bytes, append_bytes = decode_bytes_per_layer(lens, N, HQ, HKV, D, B)
    step_bytes = (attn_bytes + append_bytes) * L
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = attn_bytes / (phase1_ms * 1e-3) / 1e9

    out = {
        "metric": "paged decode-attn+KV-append HBM GB/s (% of peak) and decode tokens/s, 1 MI355X",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {L} layers, GQA {HQ}q/{HKV}kv, head_dim 128, block 16, "
                               f"batch {N}, ctx U[{args.ctx[0]},{args.ctx[1]}], pool {num_blocks} blocks "
                               f"({num_blocks * 2 * L * HKV * B * D * 2 / 2**30:.0f} GiB), {args.tables} tables",
                   "pool": pool_what,
                   "calls_per_layer": "store_kvcache + paged_attention (2 calls)" if args.unfused
                                      else "decode_append_and_attend (1 fused launch)",
                   "timed_as": "eager launches" if graph is None else "HIP graph replay of one step",
                   "row_order": ("the grid takes the batch's rows in the balanced order, computed once per step "
                                 "inside the timed region" if _balanced_order() and getattr(st, "_morphkv_decode_order", None)
                                 else "the grid takes the rows as given (a split batch needs no order)" if _balanced_order()
                                 else "the grid takes the rows as given"),
                   "pool_creation": f"outside the timed region, {pool_creation_s:.2f} s (kv_placement says what the "
                                    f"memory-group measurement found), then {wiped_s} s of waiting for the driver to "
                                    "have wiped what was released before (creation's unused candidates, pools this "
                                    "program closed, at most the whole device by a process that ended just before)"},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "kv_placement": kv_placement,
        "decode_tokens_per_s": round(N / (ms_per_step * 1e-3), 1),
        "us_per_step": round(ms_per_step * 1e3, 2),
        **({"note": "latency-bound: one layer moves a few tens of MB, so a step is a few launch latencies long and "
                    "the HBM fraction says little; us_per_step is the figure to read"}
           if args.workload == "cfg1_llama2_7b_layer" else {}),
        "eager_ms_per_step": round(eager_ms, 4),
        ("fused_eager_ms_per_step" if args.unfused else "two_call_eager_ms_per_step"): round(other_ms, 4),
        ("fused_graph_ms_per_step" if args.unfused else "two_call_graph_ms_per_step"):
            round(other_graph_ms, 4) if other_graph_ms else None,
        ("fused_graph_pct_of_hbm_peak" if args.unfused else "two_call_graph_pct_of_hbm_peak"):
            round(100.0 * step_bytes / (other_graph_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2) if other_graph_ms else None,
        "two_call_deferred_append_graph_ms_per_step": round(deferred_graph_ms, 4) if deferred_graph_ms else None,
        "two_call_deferred_append_graph_pct_of_hbm_peak":
            round(100.0 * step_bytes / (deferred_graph_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2) if deferred_graph_ms else None,
        "step_algorithmic_bytes": step_bytes,
        "roofline": {"bound": "hbm",
                     "kernel": (f"attn_decode_phase1_mfma<{HQ // HKV}, false>" if HQ // HKV >= 4
                                else f"attn_decode_phase1<{HQ // HKV}, false>"),
                     "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(
                         f"{args.workload} pool={num_blocks} batch={N} ctx={args.ctx[0]}-{args.ctx[1]} "
                         f"tables={args.tables} seed={args.seed}"),
                     "avg_launch_ms": round(phase1_ms, 5), "launches_timed": launches,
                     "timing": timing, "avg_launch_ms_bracketed": round(bracketed_ms, 5),
                     "algorithmic_bytes_per_launch": attn_bytes,
                     "phase2_avg_ms": round(p2_ms / max(p2_launches, 1), 5) if p2_launches else None,
                     "append_avg_ms": round(ap_ms / max(ap_launches, 1), 5) if ap_launches else None},
    }

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_decode(k_cache, v_cache, live, table, seq_ids, lens, q, k_new, v_new,
                                                  HQ, HKV, D, B, attn_bytes + append_bytes, L)
    del graph, k_cache, v_cache
    if hasattr(kv_pool, "close"):
        torch.cuda.synchronize()
        note_release(pool_bytes(kv_pool))
        kv_pool.close()                           # the memory goes back to the driver before the next workload
    return out


def cpu_baseline_decode(k_cache, v_cache, live, table, seq_ids, lens, q, k_new, v_new, HQ, HKV, D, B,
                        bytes_per_layer, L):
    """The oracle's torch-CPU path (append + paged attention as the reference's own
    PyTorch statement) on ONE layer of the same batch; the pool on the host holds
    only the live blocks, renumbered."""
    import torch
    from oracle import ref_cpu as R

    layer = 0
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    pool_bytes = 2 * k_cache.numel() * 2
    full_size = pool_bytes <= (4 << 30)
    if full_size:
        # the whole pool on the host, the block table as it is
        lay = R.plain_layout(k_cache.shape[0], k_cache.shape[1], HKV, B, D)
        arena = np.concatenate([k_cache.cpu().numpy().reshape(-1), v_cache.cpu().numpy().reshape(-1)])
        t2 = table.copy()
    else:
        live_sorted = np.sort(live)
        renum = {int(b): j for j, b in enumerate(live_sorted)}
        idx = torch.from_numpy(live_sorted).to(k_cache.device)
        kl = k_cache[idx, layer].cpu().numpy()          # [nlive, Hkv, B, D]
        vl = v_cache[idx, layer].cpu().numpy()
        nlive = len(live_sorted)
        lay = R.plain_layout(nlive, 1, HKV, B, D)
        arena = np.concatenate([kl.reshape(-1), vl.reshape(-1)])
        t2 = table.copy()
        for s in seq_ids:
            row = t2[s]
            for j in range(len(row)):
                if row[j] >= 0:
                    row[j] = renum[int(row[j])]
    qh = q[layer].cpu().numpy()
    kh = k_new[layer].cpu().numpy()
    vh = v_new[layer].cpu().numpy()
    reps, t_total = 0, 0.0
    while t_total < 10.0 and reps < 400:           # about ten seconds of host work
        t0 = time.perf_counter()
        R.append_decode(arena, lay, kh, vh, t2, seq_ids, lens, 0)
        R.paged_attention(qh, arena, lay, t2, seq_ids, lens, D ** -0.5, 0)
        t_total += time.perf_counter() - t0
        reps += 1
    per_layer = t_total / reps
    return {"value": round(bytes_per_layer / per_layer / 1e9, 3), "unit": "GB/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": (f"full size: the whole {pool_bytes / 2**30:.1f} GiB pool on the host, all {L} layer(s) of the same batch "
                       f"({len(lens)} seqs, ctx {int(min(lens))}-{int(max(lens))}), {reps} repetitions, "
                       f"{per_layer * L * 1e3:.2f} ms per step") if full_size and L == 1 else
                      (f"1 of {L} layers of the same batch ({len(lens)} seqs, ctx {int(min(lens))}-{int(max(lens))}), {reps} repetitions, "
                       f"{per_layer * 1e3:.1f} ms per layer; x{L} layers = {per_layer * L * 1e3:.0f} ms per step (extrapolated)"),
            "host_cpu_count": os.cpu_count()}


def cpu_baseline_resize(rng):
    """The oracle's shrink with migration (plan, NumPy block copies, table rewrite) on a pool
    scaled down to 1536 blocks of the same 2 MiB geometry, 60 % of the kept blocks live."""
    from oracle import ref_cpu as R
    L, HKV, D, B = 32, 8, 128, 16
    total, new_n = 1536, 640
    lay = R.plain_layout(total, L, HKV, B, D)
    arena = np.ones(2 * total * lay.block_elems, dtype=np.float16)        # 3 GiB of host memory
    dt, moved, moves, reps = 0.0, 0, 0, 0
    while dt < 10.0 and reps < 2000:          # about ten seconds of host work, a fresh live set each time
        bm = R.BlockManagerOracle("GPU", total, 64, 64, B)
        live = rng.permutation(total)[:int(0.6 * new_n)]
        for s_ in range(len(live) // 48):
            bm.block_table[s_, :48] = live[s_ * 48:(s_ + 1) * 48]
            bm.num_seq_allocated_blocks[s_] = 48
        live = live[:(len(live) // 48) * 48]
        bm.is_block_free[live] = False
        bm.num_free_blocks = total - len(live)
        t0 = time.perf_counter()
        src, _ = R.apply_migration(arena, lay, bm, new_n)
        dt += time.perf_counter() - t0
        moved += len(src) * 2 * lay.block_elems * 2
        moves += len(src)
        reps += 1
    return {"value": round(2 * moved / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} shrinks of a {total}-block pool of 2 MiB blocks to {new_n} ({len(live)} live, "
                      f"{moves // reps} moves each), {dt:.1f} s in all, NumPy copies on one core",
            "host_cpu_count": os.cpu_count()}


# ---------------------------------------------------------------------------------
def _warm_resize_kernels(dev, L, HKV, B, D):
    """One small resize with live blocks above the cut: a kernel's first launch in a process loads its code
    object (a few hundred microseconds each for the plan, copy and table-rewrite kernels), which is not part of
    a resize."""
    import torch
    from morphserve_amd import ElasticKVPool
    small = ElasticKVPool(64, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=64)
    small.expand(64)
    small.block_manager.allocate_blocks_for_seqs(torch.arange(4, dtype=torch.int32, device=dev),
                                                 torch.full((4,), 24 * B, dtype=torch.int32, device=dev))
    small.block_manager.free_blocks_for_seqs(torch.arange(3, dtype=torch.int32, device=dev))
    src, _ = small.shrink_to(64)
    assert src.numel() == 24


def bench_resize(args, with_cpu_baseline=True):
    """Config 3: grow 32k -> 96k blocks of 2 MiB in eight steps (zero fill), scatter 24.5k live blocks over
    the 96k range, shrink to 40k: plan, migration copy, block-table rewrite, release of the tail."""
    import torch

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, HKV, D, B = 32, 8, 128, 16
    ORG, SEG, NSEG, KEEP = 32768, 8192, 8, 1          # 32k -> 96k -> 40k blocks of 2 MiB
    rng = np.random.default_rng(args.seed)
    _warm_resize_kernels(dev, L, HKV, B, D)
    t0 = time.perf_counter()
    if not args.vmm_chunk_blocks:
        args = argparse.Namespace(**{**vars(args), "vmm_chunk_blocks": SEG})     # one physical allocation per segment and tensor
    pool, pool_what = make_pool(args, ORG, ORG + NSEG * SEG, L, HKV, B, D, 512, 256)
    torch.cuda.synchronize()
    create_s = time.perf_counter() - t0
    pool.time_kernels = True
    blk_bytes = pool.block_bytes
    pool.fill_ms()                                     # drop the base pool's own zero fill from the record
    t0 = time.perf_counter()
    for _ in range(NSEG):
        pool.expand(SEG)
    torch.cuda.synchronize()
    expand_s = time.perf_counter() - t0
    fz_ms = pool.fill_ms()
    grown = NSEG * SEG
    fill_gbs = grown * 2 * blk_bytes / (fz_ms * 1e-3) / 1e9

    total = ORG + grown
    new_n = ORG + KEEP * SEG
    n_live = int(0.6 * new_n)                          # 24 576 live blocks scattered over the 96k range
    live = rng.permutation(total)[:n_live]
    bm = pool.block_manager
    per_seq = 192
    n_seq = n_live // per_seq
    table = np.full((512, 256), -1, dtype=np.int32)
    n_alloc = np.zeros(512, dtype=np.int32)
    for s in range(n_seq):
        table[s, :per_seq] = live[s * per_seq:(s + 1) * per_seq]
        n_alloc[s] = per_seq
    live = live[:n_seq * per_seq]
    free = np.ones(total, dtype=bool)
    free[live] = False
    bm.block_table.copy_(torch.from_numpy(table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(n_alloc))
    bm.is_block_free.copy_(torch.from_numpy(free))
    bm.num_free_blocks = int(free.sum())
    moves_expected = int((live >= new_n).sum())

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    blocks_before = pool.num_blocks
    src, dst = pool.shrink_to(new_n)
    torch.cuda.synchronize()
    shrink_s = time.perf_counter() - t0
    if hasattr(pool, "close"):                         # a virtual-memory pool gives the tail back to the driver
        note_release(2 * (blocks_before - new_n) * pool.block_bytes)
    mg_ms = pool.last_migrate_ms
    moves = int(src.numel())
    assert moves == moves_expected
    # what the caller waits for before the pool is usable again: plan + copy + table rewrite + sync; giving the
    # tail's memory back to the driver (unmapping the chunks / freeing the segments) follows it
    relocate_s = getattr(pool, "last_relocate_s", None) or shrink_s
    moved_bytes = moves * 2 * blk_bytes
    traffic = 2 * moved_bytes                          # read + write
    achieved = traffic / (mg_ms * 1e-3) / 1e9
    whole = traffic / relocate_s / 1e9
    kv_placement = pool.kv_placement
    del src, dst
    if hasattr(pool, "close"):
        note_release(pool_bytes(pool))
        pool.close()
    cpu = None
    if with_cpu_baseline and not args.no_cpu_baseline:
        cpu = cpu_baseline_resize(rng)
    return {
        **({"cpu_baseline": cpu} if cpu else {}),
        "metric": "pool resize + live-block migration HBM GB/s (read+write), 1 MI355X",
        "value": round(whole, 1), "unit": "GB/s", "n_gpus": 1, "steps": 1, "warmup": 0,
        "ms_per_step": round(relocate_s * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"cfg3_resize: 2 MiB blocks (32 layers x 8 kv heads x 16 x 128 fp16, K+V), "
                               f"grow {ORG}->{total} (zero fill), {len(live)} live scattered, shrink to {new_n}",
                   "pool": pool_what,
                   "timed": "shrink_to up to the point where every live block has its new place and the table is "
                            "rewritten (plan + migration copy + table rewrite + stream sync); shrink_ms_with_release "
                            "adds the release of the memory above the cut"},
        "moves": moves, "moved_GiB": round(moved_bytes / 2 ** 30, 2), "kv_placement": kv_placement,
        "pool_creation_s": round(create_s, 3),
        "expand_s": round(expand_s, 4), "zero_fill_GBs": round(fill_gbs, 1),
        "shrink_ms_with_release": round(shrink_s * 1e3, 3),
        "pct_of_hbm_peak": round(100 * whole / HBM_PEAK_GBS, 2),
        "roofline": {"bound": "hbm", "kernel": "pool_migrate_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(f"cfg3_resize moves={moves}"),
                     "avg_launch_ms": round(mg_ms, 4),
                     "algorithmic_bytes_per_launch": traffic},
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU's throughput; this build uses a single GPU "
              f"(--gpus {args.gpus} is not supported)", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from morphserve_amd import _capi
    _capi.lib()
    table = {"cfg2_llama3_8b_decode": bench_decode, "cfg5_codellama34b_decode": bench_decode,
             "cfg1_llama2_7b_layer": bench_decode, "cfg3_resize": bench_resize}
    if args.workload not in table:
        import bench_workloads
        table = bench_workloads.WORKLOADS
    out = table[args.workload](args)
    if args.workload == "cfg2_llama3_8b_decode" and not args.no_resize and not args.pool_blocks:
        # the second target of the path in the same process and the same JSON line: the decode pool has been
        # closed, the resize workload builds its own
        import gc
        gc.collect()
        r = bench_resize(args)
        out["resize"] = {"workload": r["config"]["workload"], "metric": r["metric"], "value": r["value"],
                         "unit": r["unit"], "ms": r["ms_per_step"], "pct_of_hbm_peak": r["pct_of_hbm_peak"],
                         "moves": r["moves"], "moved_GiB": r["moved_GiB"], "expand_s": r["expand_s"],
                         "shrink_ms_with_release": r["shrink_ms_with_release"], "pool": r["config"]["pool"],
                         "timed": r["config"]["timed"], "kv_placement": r["kv_placement"],
                         "zero_fill_GBs": r["zero_fill_GBs"], "dtype": r["dtype"], "roofline": r["roofline"],
                         **({"cpu_baseline": r["cpu_baseline"]} if "cpu_baseline" in r else {})}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
