"""The secondary workloads of ``bench.py`` (``--workload ...``): the mixed and serving steps of config 4, config 5's
pressure-driven shrink, prefill shapes, the allocator, eviction, the placement A/B, the hand-over of a layer's
memory, step preparation and the two calibration loops.  ``bench.py`` imports this module when one of them is
asked for; everything shared (pool construction, traffic table, the decode and resize benchmarks the A/B
repeats) lives in ``bench.py``."""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

from bench import (Cfg, HBM_PEAK_GBS, _warm_resize_kernels, bench_decode, bench_resize, decode_bytes_per_layer, diag_kernel_times, make_pool, measured_traffic)


def bench_pressure_shrink(args):
    """Config 5 with its mid-run shrink: CodeLlama-34B-shaped decode on a ~200 GB pool, and
    mid-run the scheduler's own give-back rule releases 25 % of the blocks (63 578 -> 47 684)
    while a quarter of the live blocks sit above the cut and have to move."""
    import torch
    from morphserve_amd import build_infer_state, decode_append_and_attend, paged_attention
    from morphserve_amd.server import PoolEngine, Request, Scheduler

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, HQ, HKV, D, B, N = 48, 64, 8, 128, 16, 128
    KEEP, SEG = 47684, 15894                       # 63 578 blocks of 3 MiB (K+V) = 186 GiB
    if args.pool_backing == "vmm":                 # whole chunks of 512 blocks (768 MiB per tensor): 63 488 -> 47 616
        KEEP, SEG = 47616, 15872
        if not args.vmm_chunk_blocks:
            args = argparse.Namespace(**{**vars(args), "vmm_chunk_blocks": 512})
    total = KEEP + SEG
    rng = np.random.default_rng(args.seed)
    lens = rng.integers(args.ctx[0], args.ctx[1] + 1, size=N).astype(np.int32)
    nblk = (lens.astype(np.int64) + B - 1) // B
    max_seqs, max_bps = 256, 128
    _warm_resize_kernels(dev, L, HKV, B, D)
    pool, pool_what = make_pool(args, KEEP, total, L, HKV, B, D, max_seqs, max_bps)
    pool.expand(SEG)
    pool.time_kernels = True
    perm = rng.permutation(total)
    seq_ids = rng.permutation(max_seqs)[:N].astype(np.int32)
    table = np.full((max_seqs, max_bps), -1, dtype=np.int32)
    n_alloc = np.zeros(max_seqs, dtype=np.int32)
    pos = 0
    for i in range(N):
        table[seq_ids[i], :nblk[i]] = perm[pos:pos + nblk[i]]
        n_alloc[seq_ids[i]] = nblk[i]
        pos += nblk[i]
    live = perm[:pos].copy()
    free = np.ones(total, dtype=bool)
    free[live] = False
    bm = pool.block_manager
    bm.block_table.copy_(torch.from_numpy(table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(n_alloc))
    bm.is_block_free.copy_(torch.from_numpy(free))
    bm.num_free_blocks = int(free.sum())
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    tail = (L, HKV, B, D)
    parts = (((live, pool.k_cache, pool.v_cache, 0),) if not pool.k_cache_new else
             ((live[live < KEEP], pool.k_cache, pool.v_cache, 0),
              (live[live >= KEEP], pool.k_cache_new[0], pool.v_cache_new[0], KEEP)))
    for ids, kt, vt, off in parts:
        idt = torch.from_numpy(ids - off).to(dev)
        for c0 in range(0, len(ids), 128):
            idx = idt[c0:c0 + 128]
            kt[idx] = torch.randn((len(idx), *tail), dtype=torch.float16, device=dev, generator=g)
            vt[idx] = torch.randn((len(idx), *tail), dtype=torch.float16, device=dev, generator=g)
    q = torch.randn((L, N, HQ, D), dtype=torch.float16, device=dev, generator=g)
    k_new = torch.randn((L, N, HKV, D), dtype=torch.float16, device=dev, generator=g)
    v_new = torch.randn((L, N, HKV, D), dtype=torch.float16, device=dev, generator=g)
    o = torch.empty((L, N, HQ * D), dtype=torch.float16, device=dev)
    model = Cfg(num_layers=L, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    ecfg = Cfg(block_size=B, max_blocks_per_seq=max_bps, max_batch_size=256, max_tokens_in_batch=1 << 20,
               num_cpu_blocks=0, max_seqs_in_block_table=max_seqs, quant_serve=True, num_layers_to_quantize=1,
               num_layers_to_quantize_max=0)

    def state():
        return build_infer_state([], seq_ids.tolist(), lens.tolist(), HKV, D, num_blocks_org=bm.num_blocks_org,
                                 kv_cache_new_block_size=pool.kv_cache_new_block_size)

    def step(st):
        for layer in range(L):
            decode_append_and_attend(k_new[layer], v_new[layer], q[layer], pool.k_cache, pool.v_cache,
                                     pool.k_cache_new, pool.v_cache_new, bm.block_table, model, ecfg, st, layer,
                                     o[layer])

    def timed_steps(st):
        for _ in range(max(args.warmup, 1)):
            step(st)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step(st)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    def probe(st):                                  # attention only (no append) on three layers
        out = torch.empty((3, N, HQ * D), dtype=torch.float16, device=dev)
        for j, layer in enumerate((0, 17, 47)):
            paged_attention(q[layer], pool.k_cache, pool.v_cache, pool.k_cache_new, pool.v_cache_new,
                            bm.block_table, model, ecfg, st, layer, out[j])
        return out

    st = state()
    before_ms = timed_steps(st)
    ref = probe(st)

    # the scheduler decides: running sequences only, nothing waiting, plenty of free blocks
    engine = PoolEngine(pool, ecfg, num_layers=L, seg_blocks=SEG, migrate=True)
    engine.model.layer_quant_list.append(L - 1)     # the segment came from replacing the last layer
    engine.model.is_layer_quant_list[L - 1] = True
    engine.model.next_unquantized_layer = L - 2
    sched = Scheduler(model, ecfg, total)
    engine.scheduler = sched
    for i in range(N):
        sched.running_q.append(Request(prompt_len=int(lens[i]) - 1, output_len=1, request_id=int(seq_ids[i])))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sched.get_next_batch(engine)
    torch.cuda.synchronize()
    shrink_ms = (time.perf_counter() - t0) * 1e3
    mg_ms = pool.last_migrate_ms or 0.0
    relocate_ms = (pool.last_relocate_s or 0.0) * 1e3
    assert pool.num_blocks == KEEP and not pool.k_cache_new and sched.num_gpu_blocks == KEEP, "no give-back happened"
    moves = engine.migrated_blocks
    assert moves == int((live >= KEEP).sum())

    st = state()
    got = probe(st)
    identical = bool(torch.equal(got, ref))
    assert identical, "attention outputs changed across the shrink"
    after_ms = timed_steps(st)

    attn_bytes, append_bytes = decode_bytes_per_layer(lens, N, HQ, HKV, D, B)
    step_bytes = L * (attn_bytes + append_bytes)
    moved = moves * 2 * pool.block_bytes
    return {
        "metric": "decode step around a pressure-driven pool shrink with live migration, 1 MI355X",
        "value": round(step_bytes / (after_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(after_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"cfg5_pressure_shrink: 48 layers, GQA 64q/8kv, batch {N}, ctx U[{args.ctx[0]},"
                               f"{args.ctx[1]}], pool {total} -> {KEEP} blocks of 3 MiB, eager launches",
                   "pool": pool_what},
        "ms_per_step_before": round(before_ms, 4), "ms_per_step_after": round(after_ms, 4),
        "pct_of_hbm_peak_before": round(100 * step_bytes / (before_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "pct_of_hbm_peak_after": round(100 * step_bytes / (after_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 2),
        "shrink": {"decided_by": "Scheduler.get_next_batch -> try_quant2org -> quant2org_and_update_kvcache(migrate)",
                   "ms": round(shrink_ms, 3), "relocation_ms": round(relocate_ms, 3),
                   "live_blocks_moved": moves, "moved_GiB": round(moved / 2 ** 30, 2),
                   "GBs_read_plus_write": round(2 * moved / (max(relocate_ms, 1e-9) * 1e-3) / 1e9, 1),
                   "migrate_kernel_ms": round(mg_ms, 3),
                   "attention_outputs_bit_identical_across_shrink": identical},
        "roofline": {"bound": "hbm", "kernel": "pool_migrate_kernel",
                     "achieved": round(2 * moved / (mg_ms * 1e-3) / 1e9, 1) if mg_ms else None,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(2 * moved / (mg_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if mg_ms else None,
                     "traffic": None},
    }


def bench_mixed(args):
    """Config 4: Llama-2-7B MHA shapes, 32 layers; one step = eight 512-token prefill
    chunks + 120 decode sequences (contexts lognormal(6.2, 0.6) clipped to [16, 768]):
    per layer store_kvcache (prefill + decode rows), prefill attention, decode attention."""
    import torch
    from morphserve_amd import _capi, build_infer_state, paged_attention, prefill_attention, store_kvcache

    dev = torch.device("cuda:0")
    L, HQ, HKV, D, B = 32, 32, 32, 128, 16
    rng = np.random.default_rng(args.seed)
    p_lens = [512] * 8
    d_lens = np.clip(rng.lognormal(6.2, 0.6, size=120), 16, 768).astype(np.int32)
    lens = np.concatenate([np.asarray(p_lens, dtype=np.int32), d_lens])
    nblk = (lens.astype(np.int64) + B - 1) // B
    num_blocks = args.pool_blocks or 8192                       # 8 MiB per block (K+V): 64 GiB
    perm = rng.permutation(num_blocks)
    n_seq = len(lens)
    seq_ids = rng.permutation(256)[:n_seq].astype(np.int32)
    table = np.full((256, 64), -1, dtype=np.int32)
    pos = 0
    for i in range(n_seq):
        table[seq_ids[i], :nblk[i]] = perm[pos:pos + nblk[i]]
        pos += nblk[i]
    shape = (num_blocks, L, HKV, B, D)
    k_cache = torch.zeros(shape, dtype=torch.float16, device=dev)
    v_cache = torch.zeros(shape, dtype=torch.float16, device=dev)
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    live_t = torch.from_numpy(perm[:pos].copy()).to(dev)
    for c0 in range(0, pos, 64):
        idx = live_t[c0:c0 + 64]
        k_cache[idx] = torch.randn((len(idx), *shape[1:]), dtype=torch.float16, device=dev, generator=g)
        v_cache[idx] = torch.randn((len(idx), *shape[1:]), dtype=torch.float16, device=dev, generator=g)
    bt = torch.from_numpy(table).to(dev)
    T = sum(p_lens)
    n_tok = T + len(d_lens)
    q = torch.randn((n_tok, HQ, D), dtype=torch.float16, device=dev, generator=g)
    k = torch.randn((n_tok, HKV, D), dtype=torch.float16, device=dev, generator=g)
    v = torch.randn((n_tok, HKV, D), dtype=torch.float16, device=dev, generator=g)
    o = torch.empty((n_tok, HQ * D), dtype=torch.float16, device=dev)
    model = Cfg(num_layers=L, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    engine = Cfg(block_size=B, max_blocks_per_seq=64)
    st = build_infer_state(p_lens, seq_ids.tolist(), d_lens.tolist(), HKV, D)

    def step():
        for layer in range(L):
            store_kvcache(k, v, k_cache, v_cache, [], [], bt, model, engine, st, layer)
            prefill_attention(q[:T], k[:T], v[:T], o[:T].view(T, HQ, D), model, engine, st)
            paged_attention(q[T:], k_cache, v_cache, [], [], bt, model, engine, st, layer, o[T:])

    # the reference's layer runs the decode attention on a second stream that waits for store_kvcache only, so it
    # may overlap the prefill attention of the same layer (transformer_layer.py:151-191)
    side = torch.cuda.Stream()

    def step_two_streams():
        main = torch.cuda.current_stream()
        for layer in range(L):
            store_kvcache(k, v, k_cache, v_cache, [], [], bt, model, engine, st, layer)
            stored = torch.cuda.Event()
            stored.record(main)
            prefill_attention(q[:T], k[:T], v[:T], o[:T].view(T, HQ, D), model, engine, st)
            with torch.cuda.stream(side):
                side.wait_event(stored)
                paged_attention(q[T:], k_cache, v_cache, [], [], bt, model, engine, st, layer, o[T:])
                done = torch.cuda.Event()
                done.record(side)
            main.wait_event(done)

    def time_steps(fn):
        for _ in range(max(args.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / args.steps

    ms_per_step = time_steps(step)
    ms_two_streams = time_steps(step_two_streams)
    # the step's kernels one by one: a pass through the diagnostic twin, every launch bracketed by an event pair
    names = (("prefill_attn", _capi.K_PREFILL_ATTN), ("append_prefill", _capi.K_APPEND_PREFILL),
             ("append_decode", _capi.K_APPEND_DECODE), ("attn_phase1", _capi.K_ATTN_PHASE1),
             ("attn_phase2", _capi.K_ATTN_PHASE2))
    kt = diag_kernel_times(step, [kid for _, kid in names])
    avg = {name: (kt[kid][1] / kt[kid][0] if kt[kid][0] else None) for name, kid in names}

    # the step before the append: rotary embedding of q and k, separate or fused with it
    from morphserve_amd import rotary_embedding_and_store_kvcache, rotary_embedding_inplace, rotary_tables
    cos_t, sin_t = rotary_tables(D, 4096, device="cuda")
    positions = np.concatenate([np.arange(n) for n in p_lens] + [np.asarray(d_lens) - 1])
    pos_t = torch.from_numpy(positions).to(dev)
    st.position_cos, st.position_sin = cos_t[pos_t].contiguous(), sin_t[pos_t].contiguous()

    def timed(fn, reps=20, warm_s=0.0):
        fn()
        t_warm = time.perf_counter()           # matrix work settles on its clock only after tens of milliseconds
        while time.perf_counter() - t_warm < warm_s:
            for _ in range(8):
                fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    def rope_then_store():
        rotary_embedding_inplace(q, k, st)
        store_kvcache(k, v, k_cache, v_cache, [], [], bt, model, engine, st, 0)

    rope_two_ms = timed(rope_then_store)
    # the prefill kernel on its own: one event pair around back-to-back launches (the per-launch brackets above add
    # the event records' own cost to a 40 us kernel and run it between kernels that evict its inputs)
    prefill_b2b_ms = timed(lambda: prefill_attention(q[:T], k[:T], v[:T], o[:T].view(T, HQ, D), model, engine, st), reps=50,
                            warm_s=0.06)
    rope_fused_ms = timed(lambda: rotary_embedding_and_store_kvcache(q, k, v, k_cache, v_cache, [], [], bt, model,
                                                                      engine, st, 0))
    # chunked prefill over the paged cache: the second 256 tokens of every prompt as a chunk
    # whose first 256 tokens are already cached (the cache holds the prompts after step())
    from morphserve_amd import chunked_prefill_attention
    half = p_lens[0] // 2
    n_p = len(p_lens)
    st_chunk = build_infer_state([half] * n_p, seq_ids[:n_p].tolist(), [], HKV, D)
    q_chunk = torch.randn((n_p * half, HQ, D), dtype=torch.float16, device=dev, generator=g)
    o_chunk = torch.empty_like(q_chunk)
    prefix_t = torch.full((n_p,), half, dtype=torch.int32, device=dev)
    chunk_ms = timed(lambda: chunked_prefill_attention(q_chunk, k_cache, v_cache, [], [], bt, model, engine,
                                                       st_chunk, 0, o_chunk, prefix_t))
    chunk_flops = n_p * HQ * 4 * D * (half * half + half * half / 2)
    row = D * 2
    rope_bytes =n_tok * (2 * HQ * row + 2 * HKV * row + HKV * row + 2 * HKV * row + 2 * (D // 2) * 2)
    flops = sum(HQ * 4 * D * (n * n) / 2 for n in p_lens)                  # causal half, QK^T + PV
    tflops = flops / (prefill_b2b_ms * 1e-3) / 1e12
    tflops_in_step = flops / (avg["prefill_attn"] * 1e-3) / 1e12
    prefill_bytes = T * (2 * HQ + 2 * HKV) * D * 2                        # q + o, k + v
    append_bytes = 2 * T * 2 * HKV * D * 2
    dec_bytes, _ = decode_bytes_per_layer(d_lens, len(d_lens), HQ, HKV, D, B)
    return {
        "metric": "mixed chunked-prefill + decode step, 1 MI355X", "value": round(ms_per_step, 3), "unit": "ms/step",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "cfg4_mixed: 32 layers, MHA 32/32, head_dim 128, 8 x 512-token prefill + 120 decode "
                               f"(ctx lognormal(6.2,0.6) in [16,768]), pool {num_blocks} blocks"},
        "kernel_avg_ms": {kk: (round(vv, 5) if vv is not None else None) for kk, vv in avg.items()},
        "two_stream_ms_per_step": round(ms_two_streams, 4),
        "prefill_attn_TFLOPs": round(tflops, 1), "prefill_attn_TFLOPs_inside_the_step_bracketed": round(tflops_in_step, 1),
        "prefill_attn_ms_back_to_back": round(prefill_b2b_ms, 5), "prefill_flops_per_layer": flops,
        "append_prefill_GBs": round(append_bytes / (avg["append_prefill"] * 1e-3) / 1e9, 1),
        "decode_attn_GBs": round(dec_bytes / (avg["attn_phase1"] * 1e-3) / 1e9, 1),
        "chunked_prefill_ms": round(chunk_ms, 5),
        "chunked_prefill": f"{n_p} chunks of {half} tokens over a {half}-token cached prefix: "
                           f"{chunk_flops / (chunk_ms * 1e-3) / 1e12:.1f} TFLOP/s",
        "rotary_then_store_ms": round(rope_two_ms, 5), "rotary_store_fused_ms": round(rope_fused_ms, 5),
        "rotary_store_fused_GBs": round(rope_bytes / (rope_fused_ms * 1e-3) / 1e9, 1),
        "roofline": {"bound": "mfma", "kernel": "prefill_attn_kernel<false, 4, false>", "achieved": round(tflops, 1),
                     "peak": 2500.0, "unit": "TFLOP/s", "frac": round(tflops / 2500.0, 4),
                     "timing": "one event pair around 50 back-to-back launches of this kernel only",
                     "traffic": measured_traffic(f"cfg4_mixed prefill=8x512 seed={args.seed}")},
        # q, k, v read once and o written once: at 512-token prompts with 32 kv heads the kernel's arithmetic
        # intensity is below the machine's (2500 TFLOP/s / 8 TB/s = 312 FLOP per byte), so the HBM roofline is the
        # lower of the two ceilings for this shape
        "prefill_attn_hbm_view": {
            "algorithmic_bytes_per_launch": prefill_bytes, "flop_per_byte": round(flops / prefill_bytes, 1),
            "achieved_GBs": round(prefill_bytes / (prefill_b2b_ms * 1e-3) / 1e9, 1),
            "frac_of_8000": round(prefill_bytes / (prefill_b2b_ms * 1e-3) / 1e9 / 8000.0, 4),
            "tflops_at_hbm_peak": round(flops / (prefill_bytes / 8e12) / 1e12, 1)},
    }


def bench_serving(args):
    """Config 4 as a serving loop on the KV path only (no GEMMs): bursty arrivals (gamma
    inter-arrival, shape 0.5), 512-token prompts admitted by the scheduler as prefill batches,
    decode batches in between, sequences finishing at random lengths and freeing their blocks.
    Every step runs scheduler -> block allocation -> rotary + append -> attention for all 32
    layers -> frees.  Reports where the time of a step goes."""
    import torch
    from morphserve_amd import (ElasticKVPool, build_infer_state, decode_rope_append_and_attend, prefill_attention,
                                rotary_embedding_and_store_kvcache, rotary_tables)
    from morphserve_amd.server import PoolEngine, Request, Scheduler

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, HQ, HKV, D, B = 32, 32, 32, 128, 16
    num_blocks = args.pool_blocks or 8192
    max_seqs, max_bps = 256, 64
    rng = np.random.default_rng(args.seed)
    pool = ElasticKVPool(num_blocks, L, HKV, B, D, max_seqs_in_block_table=max_seqs, max_blocks_per_seq=max_bps,
                         zero_init=False)
    bm = pool.block_manager
    model = Cfg(num_layers=L, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    ecfg = Cfg(block_size=B, max_blocks_per_seq=max_bps, max_batch_size=160, max_tokens_in_batch=8 * 512,
               num_cpu_blocks=0, max_seqs_in_block_table=max_seqs, quant_serve=False, num_layers_to_quantize=0,
               num_layers_to_quantize_max=0)
    engine = PoolEngine(pool, ecfg, num_layers=L, seg_blocks=0)
    sched = Scheduler(model, ecfg, num_blocks)
    engine.scheduler = sched
    cos_t, sin_t = rotary_tables(D, 4096, device="cuda")
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    max_tok = 8 * 512
    q = torch.randn((max_tok, HQ, D), dtype=torch.float16, device=dev, generator=g)
    k = torch.randn((max_tok, HKV, D), dtype=torch.float16, device=dev, generator=g)
    v = torch.randn((max_tok, HKV, D), dtype=torch.float16, device=dev, generator=g)
    o = torch.empty((max_tok, HQ * D), dtype=torch.float16, device=dev)

    n_steps = max(args.steps, 1) * 40
    # arrivals: gamma(0.5) gaps with a mean of 5 steps per burst of 8 prompts -> ~115 sequences in flight
    arrival_step, t = [], 0.0
    while t < n_steps:
        t += rng.gamma(0.5, 10.0)
        arrival_step.append(int(t))
    next_arrival = 0
    spent = {"schedule": 0.0, "allocate": 0.0, "allocate_call_host": 0.0, "kernels": 0.0, "free": 0.0}
    counts = {"prefill_steps": 0, "decode_steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "finished": 0,
              "allocate_calls": 0, "blocks_allocated": 0, "max_running": 0}

    def dev_i32(x):
        return torch.tensor(x, dtype=torch.int32, device=dev)

    torch.cuda.synchronize()
    t_begin = time.perf_counter()
    for step_no in range(n_steps):
        while next_arrival < len(arrival_step) and arrival_step[next_arrival] <= step_no:
            sched.on_requests_arrival([Request(prompt_len=512, max_output_len=int(rng.integers(32, 257)))
                                       for _ in range(8)])
            next_arrival += 1
        t0 = time.perf_counter()
        batch, swapped_in, swapped_out = sched.get_next_batch(engine)
        assert not swapped_in and not swapped_out, "the pool is sized so that nothing is evicted"
        t1 = time.perf_counter()
        reqs = list(batch)
        if not reqs:
            spent["schedule"] += t1 - t0
            continue
        prefill = batch is not sched.running_q
        ids = [r.request_id for r in reqs]
        lens = [r.prompt_len + r.output_len for r in reqs]
        ids_t, lens_t = dev_i32(ids), dev_i32(lens)
        t1a = time.perf_counter()
        # the lists the scheduler already holds go along: every check and the size of the result come from the
        # manager's host copy of its counters, nothing is read back from the device
        new_ids = bm.allocate_blocks_for_seqs(ids_t, lens_t, seq_ids_host=ids, target_lens_host=lens)
        t1b = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        spent["allocate_call_host"] += t1b - t1a
        if prefill:
            p_lens, d_lens = [r.prompt_len for r in reqs], []
            positions = np.concatenate([np.arange(n) for n in p_lens])
        else:
            p_lens, d_lens = [], lens
            positions = np.asarray(lens) - 1
        n_tok = len(positions)
        st = build_infer_state(p_lens, ids, d_lens, HKV, D)
        pos_t = torch.from_numpy(positions).to(dev)
        st.position_cos, st.position_sin = cos_t[pos_t].contiguous(), sin_t[pos_t].contiguous()
        for layer in range(L):
            if prefill:       # rotary + append in one launch, then causal attention over the batch's own k, v
                rotary_embedding_and_store_kvcache(q[:n_tok], k[:n_tok], v[:n_tok], pool.k_cache, pool.v_cache,
                                                   [], [], bm.block_table, model, ecfg, st, layer)
                prefill_attention(q[:n_tok], k[:n_tok], v[:n_tok], o[:n_tok].view(n_tok, HQ, D), model, ecfg, st)
            else:             # rotary + append + attention in one launch
                decode_rope_append_and_attend(k[:n_tok], v[:n_tok], q[:n_tok], pool.k_cache, pool.v_cache, [], [],
                                              bm.block_table, model, ecfg, st, layer, o[:n_tok])
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        for r in reqs:
            r.output_len += 1
        done = [r.request_id for r in reqs if r.is_finished()]
        if done:
            bm.free_blocks_for_seqs(dev_i32(done), seq_ids_host=done)
            torch.cuda.synchronize()
        sched.on_batch_finish(reqs)
        t4 = time.perf_counter()
        spent["schedule"] += t1 - t0
        spent["allocate"] += t2 - t1
        spent["kernels"] += t3 - t2
        spent["free"] += t4 - t3
        counts["prefill_steps" if prefill else "decode_steps"] += 1
        counts["prefill_tokens" if prefill else "decode_tokens"] += n_tok
        counts["finished"] += len(done)
        counts["allocate_calls"] += 1
        counts["blocks_allocated"] += int(new_ids.numel())
        counts["max_running"] = max(counts["max_running"], len(sched.running_q))
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_begin

    # conservation: every block is free or owned by exactly one running sequence
    owned = int(bm.num_seq_allocated_blocks.sum().item())
    free_now = int(bm.is_block_free.sum().item())
    assert owned + free_now == num_blocks == int(bm.num_free_blocks) + owned, "block accounting drifted"
    assert owned == sum(-(-(r.prompt_len + r.output_len - 1) // B) for r in sched.running_q), \
        "running sequences own a different number of blocks than their lengths need"
    steps_run = counts["prefill_steps"] + counts["decode_steps"]
    tokens = counts["prefill_tokens"] + counts["decode_tokens"]
    return {
        "metric": "KV-path serving loop (scheduler + allocator + rotary/append + attention, 32 layers), 1 MI355X",
        "value": round(tokens / wall, 1), "unit": "tokens/s (KV path only)", "n_gpus": 1, "steps": steps_run,
        "warmup": 0, "ms_per_step": round(wall * 1e3 / max(steps_run, 1), 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": f"cfg4_serving: MHA 32/32, head_dim 128, 32 layers, pool {num_blocks} blocks of 8 MiB, "
                               "bursts of 8 x 512-token prompts with gamma(0.5) gaps, outputs U[32,256], "
                               f"{n_steps} scheduler steps, eager launches with a sync per phase for the breakdown"},
        **counts,
        "share_of_wall": {kk: round(vv / wall, 4) for kk, vv in spent.items()},
        "avg_ms": {"schedule": round(spent["schedule"] * 1e3 / n_steps, 4),
                   "allocate_call_host": round(spent["allocate_call_host"] * 1e3 / max(counts["allocate_calls"], 1), 4),
                   "allocate_incl_input_copy_and_sync": round(spent["allocate"] * 1e3 / max(counts["allocate_calls"], 1), 4),
                   "kernels_per_step": round(spent["kernels"] * 1e3 / max(steps_run, 1), 4),
                   "free_and_bookkeeping": round(spent["free"] * 1e3 / max(steps_run, 1), 4)},
        "roofline": None,
    }


def bench_mfma_calibration(args):
    """What the matrix pipe sustains with nothing else in the way: the prefill kernel's 64 matrix
    instructions per wave and round, (0) on constant register operands, (1) on N(0,1) register
    operands, (2) on N(0,1) operands read from LDS in the prefill kernel's fragment pattern."""
    import ctypes as C
    import torch
    from morphserve_amd import _capi

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    data = torch.randn(64 * 1024, dtype=torch.float16, device=dev, generator=g)
    sink = torch.empty(512 * 256, dtype=torch.float32, device=dev)
    lib = _capi.diag_lib()                     # the calibration loop lives in the diagnostic twin
    iters = 2000
    out = {}
    for mode, name in ((0, "registers_constant_operands"), (1, "registers_normal_operands"), (2, "lds_normal_operands")):
        flops = C.c_double(0.0)
        _capi.check(lib.mkv_diag_mfma_loop(mode, 10, data.data_ptr(), sink.data_ptr(), None, _capi.current_stream()))
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(max(args.steps, 1)):
            _capi.check(lib.mkv_diag_mfma_loop(mode, iters, data.data_ptr(), sink.data_ptr(), C.byref(flops),
                                               _capi.current_stream()))
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / max(args.steps, 1)
        out[name] = round(flops.value / (ms * 1e-3) / 1e12, 1)
    best = out["registers_normal_operands"]
    return {"metric": "matrix-pipe calibration, v_mfma_f32_16x16x32_f16, TFLOP/s", "value": best, "unit": "TFLOP/s",
            "n_gpus": 1, "steps": args.steps, "warmup": 0, "ms_per_step": None, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
            "config": {"workload": "mfma_calibration: 512 workgroups x 4 waves x 2000 rounds x 64 matrix instructions"},
            "tflops": out, "published_peak_tflops": 2500.0}


def bench_prefill_shapes(args):
    """Causal prefill attention (MHA 32 / 32 heads, head_dim 128) for a list of prompt batches -- whole prompts
    over the batch's own contiguous q, k, v ("8x512"), or chunks over a prefix already in a paged cache
    ("8x512+2048") -- and every workgroup shape of the kernel: microseconds per launch and TFLOP/s (causal
    half of the chunk plus the whole prefix, QK^T + PV).  `value` is the library's own choice on the first shape."""
    import torch
    from morphserve_amd import _capi

    import contextlib
    dev = torch.device("cuda:0")
    H, D = 32, 128
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    variants = [int(x) for x in args.prefill_variants.split(",")]
    rows = {}
    for shape in args.prefill_shapes.split(","):
        # "NxL": N whole prompts of L tokens over their own k, v; "NxL+P": N chunks of L tokens whose sequences
        # already hold P tokens in a paged cache (one layer, blocks dealt from a seeded permutation of the pool)
        body, _, pfx = shape.partition("+")
        prefix = int(pfx) if pfx else 0
        paged = pfx != ""
        HKV = H
        nseq, ln = (int(x) for x in body.split("x"))
        T = nseq * ln
        if args.prefill_data == "zeros":
            q = torch.zeros((T, H, D), dtype=torch.float16, device=dev)
            k, v = (torch.zeros((T, HKV, D), dtype=torch.float16, device=dev) for _ in range(2))
        else:
            q = torch.randn((T, H, D), dtype=torch.float16, device=dev, generator=g)
            k = torch.randn((T, HKV, D), dtype=torch.float16, device=dev, generator=g)
            v = torch.randn((T, HKV, D), dtype=torch.float16, device=dev, generator=g)
        starts = torch.arange(nseq, dtype=torch.int32, device=dev) * ln
        lens = torch.full((nseq,), ln, dtype=torch.int32, device=dev)
        flops = nseq * H * 4 * D * (ln * prefix + ln * ln / 2)
        if paged:
            from morphserve_amd import build_infer_state, chunked_prefill_attention
            per_seq = (prefix + ln + 15) // 16
            nb = nseq * per_seq + 64
            rng = np.random.default_rng(args.seed)
            table = rng.permutation(nb)[:nseq * per_seq].reshape(nseq, per_seq).astype(np.int32)
            bt = torch.from_numpy(table).to(dev)
            if args.prefill_data == "zeros":
                k_cache = torch.zeros((nb, 1, H, 16, D), dtype=torch.float16, device=dev)
                v_cache = torch.zeros((nb, 1, H, 16, D), dtype=torch.float16, device=dev)
            else:
                k_cache = torch.randn((nb, 1, H, 16, D), dtype=torch.float16, device=dev, generator=g)
                v_cache = torch.randn((nb, 1, H, 16, D), dtype=torch.float16, device=dev, generator=g)
            model = Cfg(num_layers=1, num_q_heads=H, num_kv_heads=H, head_dim=D)
            engine = Cfg(block_size=16, max_blocks_per_seq=per_seq)
            st = build_infer_state([ln] * nseq, list(range(nseq)), [], H, D)
            prefix_t = torch.full((nseq,), prefix, dtype=torch.int32, device=dev)
        outs, row = {}, {}
        for var in variants:
            # 0 = the product library and its own choice; a forced shape exists in the diagnostic twin only
            with (_capi.use_diag_library() if var else contextlib.nullcontext(_capi.lib())) as lib:
                if var:
                    _capi.check(lib.mkv_set_prefill_variant(var))
                o = torch.full_like(q, float("nan"))

                def run():
                    if paged:
                        chunked_prefill_attention(q, k_cache, v_cache, [], [], bt, model, engine, st, 0, o, prefix_t, prefix)
                    else:
                        _capi.check(lib.mkv_prefill_attn(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                         starts.data_ptr(), lens.data_ptr(), nseq, ln, H, HKV, D, D ** -0.5,
                                                         _capi.current_stream()))
                # warm up by time, not by count: after the set-up kernels (random fills) the first few tens of
                # milliseconds of matrix work run at another clock, and a timing taken there reads 10-15 % low
                t_warm = time.perf_counter()
                n_warm = 0
                while n_warm < max(args.warmup, 1) or time.perf_counter() - t_warm < 0.06:
                    run()
                    n_warm += 1
                    if n_warm % 8 == 0:
                        torch.cuda.synchronize()
                torch.cuda.synchronize()
                reps = max(args.steps, 5)
                blocks = []
                for _ in range(3):                       # median of three timed blocks of `reps` launches
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(reps):
                        run()
                    e1.record()
                    torch.cuda.synchronize()
                    blocks.append(e0.elapsed_time(e1) / reps)
                ms = sorted(blocks)[1]
                outs[var] = o
                row[f"variant_{var}"] = {"us": round(ms * 1e3, 2), "TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1),
                                         "frac_of_2500": round(flops / (ms * 1e-3) / 1e12 / 2500.0, 4)}
                if var:
                    _capi.check(lib.mkv_set_prefill_variant(0))
        base = outs[variants[0]].float()
        assert torch.isfinite(base).all()
        row["max_abs_diff_between_variants"] = max(float((outs[x].float() - base).abs().max()) for x in variants)
        rows[shape] = row
    first = rows[args.prefill_shapes.split(",")[0]]
    best = first[f"variant_{variants[0]}"]
    return {"metric": "causal prefill attention TFLOP/s (fp16 MFMA, fp32 accumulate), 1 MI355X", "value": best["TFLOPs"],
            "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": best["us"] / 1e3,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)",
            "data": "synthetic",
            "config": {"workload": f"prefill_shapes: 32 q / 32 kv heads, head_dim 128, prompt batches {args.prefill_shapes}, "
                                   f"workgroup shapes {args.prefill_variants}, inputs {args.prefill_data}"},
            "shapes": rows,
            "roofline": {"bound": "mfma", "kernel": "prefill_attn_kernel",
                         "achieved": best["TFLOPs"], "peak": 2500.0, "unit": "TFLOP/s",
                         "frac": round(best["TFLOPs"] / 2500.0, 4), "traffic": None}}


def bench_copy_calibration(args):
    """A plain device copy of known size (the migration kernel moving 512 blocks of
    2 MiB: 1 GiB read, 1 GiB written) -- the yardstick the FETCH_SIZE / WRITE_SIZE
    counters of the other kernels are scaled by."""
    import ctypes as C
    import torch
    from morphserve_amd import _capi

    dev = torch.device("cuda:0")
    L, HKV, D, B = 32, 8, 128, 16
    nb, moves = 2048, 512
    k = torch.zeros((nb, L, HKV, B, D), dtype=torch.float16, device=dev)
    v = torch.zeros_like(k)
    pool = _capi.make_pool(k, v)
    src = torch.arange(1024, 1024 + moves, dtype=torch.int64, device=dev)
    dst = torch.arange(0, moves, dtype=torch.int64, device=dev)
    stream = _capi.current_stream()
    _capi.check(_capi.lib().mkv_pool_migrate(C.byref(pool), src.data_ptr(), dst.data_ptr(), moves, stream))
    launches = max(args.steps, 1)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(launches):
        _capi.check(_capi.lib().mkv_pool_migrate(C.byref(pool), src.data_ptr(), dst.data_ptr(), moves, stream))
    e1.record()
    torch.cuda.synchronize()
    moved = moves * 2 * (L * HKV * B * D * 2)
    avg = e0.elapsed_time(e1) / launches
    return {"metric": "plain device copy GB/s (read+write)", "value": round(2 * moved / (avg * 1e-3) / 1e9, 1),
            "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": 0, "ms_per_step": round(avg, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
            "config": {"workload": "copy_calibration: pool_migrate_kernel, 512 moves x 2 MiB (K+V)"},
            "bytes_read_per_launch": moved, "bytes_written_per_launch": moved}


def bench_placement_ab(args):
    """Does a figure depend on when and where its pool was allocated?  ONE process creates a pool, measures the
    decode step of config 2 on it and the resize of config 3, and frees it -- for the memory-group placement
    and for the plain order, three times each: at once, again at once, and after a pause (the driver hands
    out different memory for some seconds after a large free).  Every figure of the table should sit on one
    level per placement."""
    import gc
    import torch
    rows = []
    base = {**vars(args), "no_cpu_baseline": True, "no_resize": True, "pool_backing": "vmm",
            "workload": "cfg2_llama3_8b_decode", "vmm_chunk_blocks": 0}
    base["no_wipe_wait"] = False
    schedule = [("first", 0.0), ("again at once", 0.0), (f"after {args.ab_pause:g} s", args.ab_pause)]
    for when, pause in schedule:
        for placement in ("groups", "plain", "groups, measured without waiting for the driver's wipe"):
            if pause:
                time.sleep(pause)
            a = argparse.Namespace(**{**base, "placement": placement.split(",")[0],
                                      "no_wipe_wait": "without waiting" in placement})
            d = bench_decode(a)
            gc.collect()
            r = bench_resize(a, with_cpu_baseline=False)
            gc.collect()
            rows.append({"when": when, "placement": placement,
                         "decode_pct_of_hbm_peak": d["pct_of_hbm_peak"], "decode_ms_per_step": d["ms_per_step"],
                         "decode_kernel_frac": d["roofline"]["frac"],
                         "resize_pct_of_hbm_peak": r["pct_of_hbm_peak"], "resize_ms": r["ms_per_step"],
                         "migrate_kernel_frac": r["roofline"]["frac"], "zero_fill_GBs": r["zero_fill_GBs"],
                         "decode_pool_creation": d["config"]["pool_creation"],
                         "decode_pool_growths": d["kv_placement"]["growths"],
                         "resize_pool_growths": r["kv_placement"]["growths"]})
            print(json.dumps({k: v for k, v in rows[-1].items() if not k.endswith("growths")}), file=sys.stderr, flush=True)
    g = [x for x in rows if x["placement"] == "groups"]
    p = [x for x in rows if x["placement"] == "plain"]
    return {"metric": "decode and resize, % of HBM peak, over repeated pool creations in one process", "unit": "%",
            "value": min(x["decode_pct_of_hbm_peak"] for x in g), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": max(x["decode_ms_per_step"] for x in g), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16 / u8", "data": "synthetic",
            "config": {"workload": "placement_ab: config 2 decode and config 3 resize on a VmmKVPool, memory-group "
                                   "placement against the plain order, allocate -> measure -> free three times each"},
            "range_with_groups": {"decode_pct": [min(x["decode_pct_of_hbm_peak"] for x in g), max(x["decode_pct_of_hbm_peak"] for x in g)],
                                  "resize_pct": [min(x["resize_pct_of_hbm_peak"] for x in g), max(x["resize_pct_of_hbm_peak"] for x in g)]},
            "range_plain": {"decode_pct": [min(x["decode_pct_of_hbm_peak"] for x in p), max(x["decode_pct_of_hbm_peak"] for x in p)],
                            "resize_pct": [min(x["resize_pct_of_hbm_peak"] for x in p), max(x["resize_pct_of_hbm_peak"] for x in p)]},
            "rows": rows}


def bench_allocator(args):
    """Launch times of the block manager's kernels on maps of config-2 and config-3 size (rocprofv3 --kernel-trace
    gives the per-kernel durations of this workload), and the host time of allocate_blocks_for_seqs with and
    without host lists."""
    import torch
    from morphserve_amd import BlockManager, ElasticKVPool

    dev = torch.device("cuda:0")
    out = {}
    rng = np.random.default_rng(args.seed)
    for num_blocks, fill in ((65536, 0.08), (65536, 0.9), (98304, 0.25)):
        bm = BlockManager("GPU", num_blocks, 512, 256, 16)
        used = rng.random(num_blocks) < fill
        bm.is_block_free.copy_(torch.from_numpy(~used))
        bm.num_free_blocks = int((~used).sum())
        ids = torch.arange(64, dtype=torch.int32, device=dev)
        ids_h = list(range(64))
        cur = np.zeros(64, dtype=np.int64)
        times = {}
        for mode in ("host lists", "device read"):
            for _ in range(3):                             # warm-up: code objects, torch's allocator, the host copy
                cur += 16
                tgt = torch.from_numpy(cur.astype(np.int32)).to(dev)
                if mode == "host lists":
                    bm.allocate_blocks_for_seqs(ids, tgt, seq_ids_host=ids_h, target_lens_host=cur)
                else:
                    bm.allocate_blocks_for_seqs(ids, tgt)
            reps = max(args.steps, 20)
            host_s = 0.0
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(reps):
                cur += 16                                  # one more block per sequence
                tgt = torch.from_numpy(cur.astype(np.int32)).to(dev)
                t0 = time.perf_counter()
                if mode == "host lists":
                    bm.allocate_blocks_for_seqs(ids, tgt, seq_ids_host=ids_h, target_lens_host=cur)
                else:
                    bm.allocate_blocks_for_seqs(ids, tgt)
                host_s += time.perf_counter() - t0
            e1.record()
            torch.cuda.synchronize()
            times[mode] = {"host_us_per_call": round(host_s / reps * 1e6, 1),
                           "stream_us_per_call_incl_input_copy": round(e0.elapsed_time(e1) / reps * 1e3, 1)}
        out[f"{num_blocks} blocks, {int(fill * 100)} % used"] = times
    # shrink planning on the config-3 map
    pool = ElasticKVPool(64, 1, 1, 16, 128, max_seqs_in_block_table=8, max_blocks_per_seq=8)
    bm = pool.block_manager
    total, new_n = 98304, 40960
    free = torch.ones(total, dtype=torch.bool, device=dev)
    live = torch.from_numpy(rng.permutation(total)[:24576]).to(dev)
    src = torch.empty(total - new_n, dtype=torch.int64, device=dev)
    dst = torch.empty_like(src)
    remap = torch.empty(total, dtype=torch.int32, device=dev)
    res = torch.zeros(4, dtype=torch.int64, device=dev)
    from morphserve_amd import _capi
    reps = max(args.steps, 20)
    tot_ms = 0.0
    for _ in range(reps):
        free.fill_(True)
        free[live] = False
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _capi.check(_capi.lib().mkv_pool_plan_shrink(free.data_ptr(), total, new_n, src.data_ptr(), dst.data_ptr(),
                                                     total - new_n, remap.data_ptr(), res.data_ptr(),
                                                     _capi.current_stream()))
        e1.record()
        torch.cuda.synchronize()
        tot_ms += e0.elapsed_time(e1)
    out["pool_plan_shrink 98304 -> 40960, 24576 live"] = {"event_us_per_launch": round(tot_ms / reps * 1e3, 1),
                                                          "moves": int(res[0].item())}
    del pool, bm
    first = out["65536 blocks, 8 % used"]["host lists"]
    return {"metric": "block manager: host microseconds per allocate_blocks_for_seqs call", "unit": "us",
            "value": first["host_us_per_call"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": first["host_us_per_call"] / 1e3, "higher_is_better": False, "scaling": "weak",
            "vs_baseline": None, "dtype": "int32", "data": "synthetic",
            "config": {"workload": "allocator: 64 decoding sequences take one more block each per call; free maps "
                                   "of 65 536 and 98 304 entries"},
            "cases": out}


def bench_step_state(args):
    """Host time of a step's preparation (MorphServe/worker/model.py:318-436): the reference's way -- one device
    tensor per host list, an arange per prefill sequence, two gathers -- against ``StepStateBuilder`` (one pinned
    staging buffer, one asynchronous copy, two gathers), block allocation excluded from both."""
    import torch
    from morphserve_amd import StepStateBuilder, build_infer_state

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    rng = np.random.default_rng(args.seed)
    cos = torch.randn((4096 + 128, 64), dtype=torch.float16, device=dev)
    sin = torch.randn_like(cos)
    builder = StepStateBuilder(256, 16384, 8, 128, cos_cached=cos, sin_cached=sin)

    def reference_way(p, ids, d):
        st = build_infer_state(p, ids, d, 8, 128)
        pos = torch.cat((
            torch.concat([torch.arange(0, x, device=dev, dtype=torch.int32) for x in p])
            if p else torch.empty(0, device=dev, dtype=torch.int32), st.decoding_seq_lens - 1), dim=0)
        st.position_cos, st.position_sin = cos[pos], sin[pos]
        return st

    shapes = {"cfg2 decode step (64 decoding)": ([], rng.integers(1024, 1537, size=64).tolist()),
              "cfg4 mixed step (8 x 512 prefill + 120 decoding)": ([512] * 8, rng.integers(16, 769, size=120).tolist()),
              "cfg5 decode step (128 decoding)": ([], rng.integers(1024, 1537, size=128).tolist())}
    out = {}
    for name, (p, d) in shapes.items():
        ids = list(range(len(p) + len(d)))
        row = {}
        for label, fn in (("one_tensor_per_list_us", reference_way), ("one_staging_copy_us", builder.build)):
            for _ in range(max(args.warmup, 3)):
                fn(p, ids, d)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps * 5):
                fn(p, ids, d)
            host = (time.perf_counter() - t0) / (args.steps * 5) * 1e6       # until the calls return
            torch.cuda.synchronize()
            row[label] = round(host, 1)
        a, b = reference_way(p, ids, d), builder.build(p, ids, d)
        assert torch.equal(a.position_cos, b.position_cos) and torch.equal(a.seq_ids, b.seq_ids)
        out[name] = row
    first = out["cfg2 decode step (64 decoding)"]
    return {
        "metric": "host time to prepare one step's LlamaInferState (lists -> device tensors, positions, rotary rows)",
        "value": first["one_staging_copy_us"], "unit": "us", "n_gpus": 1, "steps": args.steps * 5, "warmup": args.warmup,
        "ms_per_step": round(first["one_staging_copy_us"] / 1e3, 4), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "int32", "data": "synthetic",
        "config": {"workload": "step_state: the preparation of model.py:318-436 for three batch shapes"},
        "shapes": out, "roofline": None,
    }


def bench_layer_handover(args):
    """A replaced layer's memory becoming pool blocks and going back (config-2 geometry: 1 MiB per block and
    tensor): ``VmmKVPool.expand_from`` / ``shrink_into`` against ``expand`` / ``shrink_to``, which allocate and
    free the same amount through the driver.  Llama-3-8B layer: 436 MB in fp16, 116 MB as its 4-bit twin."""
    import time
    import torch
    from morphserve_amd import LayerArena, VmmKVPool

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, HKV, B, D = 32, 8, 16, 128
    org = args.pool_blocks or 8192
    layer_bytes, quant_bytes = 436_207_616, 116_000_000

    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3

    by_chunk = {}
    for cb in (16, 32, 64):
        pool = VmmKVPool(org, org + 4096, L, HKV, B, D, max_seqs_in_block_table=64, max_blocks_per_seq=128, chunk_blocks=cb)
        chunk = cb * pool.block_bytes
        layer = LayerArena(layer_bytes, chunk)
        n = pool.blocks_available_from(layer, quant_bytes)
        rows = {"hand_over_in_ms": [], "hand_over_back_ms": [], "allocate_ms": [], "free_ms": []}
        for it in range(args.warmup + args.steps):
            a = timed(lambda: pool.expand_from(layer, quant_bytes))
            assert pool.num_blocks == org + n
            b = timed(lambda: pool.shrink_into(layer, org))
            c = timed(lambda: pool.expand(n))
            d = timed(lambda: pool.shrink_to(org))
            if it >= args.warmup:
                for k, v in zip(rows, (a, b, c, d)):
                    rows[k].append(v)
        by_chunk[f"{chunk >> 20} MiB"] = {"new_blocks": n, "chunks_moved": 2 * n // cb,
                                          **{k: round(sorted(v)[len(v) // 2], 3) for k, v in rows.items()}}
        layer.close()
        pool.close()
    best = by_chunk["64 MiB"]
    return {
        "metric": "pool growth out of a replaced layer's memory and back, ms per hand-over, 1 MI355X",
        "value": best["hand_over_in_ms"], "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": best["hand_over_in_ms"], "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"layer_handover: layer {layer_bytes} B, quantized twin {quant_bytes} B, pool of {org} "
                               "blocks of 2 MiB (K+V), chunks of 64 MiB; empty tail on the way back"},
        "by_chunk_size": by_chunk, "zero_fill_included": True, "roofline": None,
    }


def bench_eviction(args):
    """Swap sequences out to host swap space and back (config-2 block geometry, 2 MiB per
    block): whole ``_swap`` calls -- block-manager work, copy, synchronisation -- as PCIe GB/s."""
    import torch
    from morphserve_amd import ElasticKVPool, KVSwapper, _capi

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    small = _eviction_routes(args, 1, 32, args.pool_blocks or 8192, 32, 40)     # config-1 geometry: 256 KiB blocks
    torch.cuda.empty_cache()
    results, gbytes, n_seq, blocks_per_seq, num_blocks = _eviction_routes(args, 32, 8, args.pool_blocks or 4096, 16, 80)
    best = results["kernel_pinned"]
    return {
        "metric": "KV eviction (swap out + swap in of 16 sequences), PCIe GB/s, 1 MI355X",
        "value": round(2 * gbytes / ((best["swap_out_ms"] + best["swap_in_ms"]) * 1e-3), 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(best["swap_out_ms"] + best["swap_in_ms"], 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"eviction: 2 MiB blocks (K+V), {n_seq} sequences x {blocks_per_seq} scattered blocks "
                               f"= {gbytes:.2f} GB each way, pool {num_blocks} blocks"},
        "routes": results,
        "routes_256KiB_blocks": {"workload": f"{small[2]} sequences x {small[3]} scattered blocks = "
                                             f"{small[1]:.2f} GB each way", **small[0]},
        "roofline": None,
    }


def _eviction_routes(args, L, HKV, num_blocks, n_seq, blocks_per_seq):
    import torch
    from morphserve_amd import ElasticKVPool, KVSwapper
    D, B = 128, 16
    rng = np.random.default_rng(args.seed)
    pool = ElasticKVPool(num_blocks, L, HKV, B, D, max_seqs_in_block_table=64, max_blocks_per_seq=128,
                         zero_init=False)
    bm = pool.block_manager
    # scattered ownership: blocks dealt from a permutation of the pool
    perm = rng.permutation(num_blocks)[:n_seq * blocks_per_seq]
    table = np.full(tuple(bm.block_table.shape), -1, dtype=np.int32)
    for s_ in range(n_seq):
        table[s_, :blocks_per_seq] = perm[s_ * blocks_per_seq:(s_ + 1) * blocks_per_seq]
    bm.block_table.copy_(torch.from_numpy(table))
    bm.num_seq_allocated_blocks[:n_seq] = blocks_per_seq
    free = np.ones(num_blocks, dtype=bool)
    free[perm] = False
    bm.is_block_free.copy_(torch.from_numpy(free))
    bm.num_free_blocks = int(free.sum())
    seqs = list(range(n_seq))
    moved = n_seq * blocks_per_seq
    gbytes = moved * pool.block_bytes * 2 / 1e9
    results = {}
    for name, pinned, use_kernel, cpu_tables in (("kernel_pinned", True, True, "device"),
                                                 ("kernel_pinned_host_tables", True, True, "host"),
                                                 ("memcpy_runs_pinned", True, False, "device"),
                                                 ("memcpy_runs_pinned_host_tables", True, False, "host"),
                                                 ("memcpy_runs_pageable", False, False, "device")):
        sw = KVSwapper(pool, moved + 64, pinned=pinned, cpu_tables=cpu_tables)
        out_ms, in_ms = [], []
        for rep in range(max(args.warmup, 1) + args.steps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            sw.swap_out_seqs(seqs, use_kernel=use_kernel)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            sw.swap_in_seqs(seqs, use_kernel=use_kernel)
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            if rep >= max(args.warmup, 1):
                out_ms.append((t1 - t0) * 1e3)
                in_ms.append((t2 - t1) * 1e3)
        results[name] = {"swap_out_ms": round(float(np.mean(out_ms)), 3), "swap_in_ms": round(float(np.mean(in_ms)), 3),
                         "swap_out_GBs": round(gbytes / (np.mean(out_ms) * 1e-3), 2),
                         "swap_in_GBs": round(gbytes / (np.mean(in_ms) * 1e-3), 2)}
        del sw
    del pool
    return results, gbytes, n_seq, blocks_per_seq, num_blocks


WORKLOADS = {"cfg4_mixed": bench_mixed, "cfg4_serving": bench_serving, "cfg5_pressure_shrink": bench_pressure_shrink,
             "placement_ab": bench_placement_ab, "allocator": bench_allocator,
             "copy_calibration": bench_copy_calibration, "mfma_calibration": bench_mfma_calibration,
             "eviction": bench_eviction, "prefill_shapes": bench_prefill_shapes,
             "layer_handover": bench_layer_handover, "step_state": bench_step_state}
