"""Config 4's arrival / finish interleave at length, against the oracle step by step.

MorphServe/worker/model.py:302-466 (a step: lists -> state -> block allocation -> per layer rotary, append,
prefill attention, decode attention) and :507-534 (finished sequences give their blocks back), driven for a
few hundred steps by a bursty arrival process -- gamma(shape 0.5) inter-arrival times, prompt lengths
lognormal(6.2, 0.6) clipped to [16, 768], MHA -- with ``StepStateBuilder`` + ``attention_section`` on the GPU and
``BlockManagerOracle`` / ``R.store_kvcache`` on the CPU.  The allocator state is compared after EVERY step, the
pool bytes and the attention outputs every few steps and at the end.
"""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from oracle import rope_cpu as RO
from helpers import Cfg, assert_attn_close, rand_f16
from gpu_helpers import assert_state_equal, bits, manager_state
from morphserve_amd import ElasticKVPool, StepStateBuilder
from morphserve_amd.worker.layers import attention_section

pytestmark = pytest.mark.gpu


def _positions(p_lens, d_lens):
    pos = [np.arange(n) for n in p_lens] + [np.asarray([n - 1]) for n in d_lens]
    return np.concatenate(pos) if pos else np.zeros(0, dtype=np.int64)


@pytest.mark.parametrize("seed,steps", [(4, 220)])
def test_bursty_serving_loop_matches_the_oracle(cuda, seed, steps):
    L, H, D, B = 2, 4, 128, 16                      # MHA: as many kv heads as q heads
    NB, ROWS, MAX_BLOCKS, MAX_RUNNING, CHECK_EVERY = 1100, 48, 56, 20, 10
    rng = np.random.default_rng(seed)
    pool = ElasticKVPool(NB, L, H, B, D, max_seqs_in_block_table=ROWS, max_blocks_per_seq=MAX_BLOCKS)
    bm = pool.block_manager
    ob = R.BlockManagerOracle("GPU", NB, ROWS, MAX_BLOCKS, B)
    lay = R.plain_layout(NB, L, H, B, D)
    arena = np.zeros(2 * NB * lay.block_elems, dtype=np.float16)
    half = NB * lay.block_elems
    ct, st_ = RO.rotary_tables(D, MAX_BLOCKS * B)
    builder = StepStateBuilder(ROWS, 8192, H, D, torch.from_numpy(ct).to(cuda), torch.from_numpy(st_).to(cuda))
    model, engine = Cfg(num_layers=L, num_q_heads=H, num_kv_heads=H, head_dim=D), Cfg(block_size=B, max_blocks_per_seq=MAX_BLOCKS)

    # arrivals: bursty, in units of steps; every request: (prompt length, tokens to generate)
    t, waiting = 0.0, []
    while t < steps:
        t += rng.gamma(0.5, 3.0)
        prompt = int(np.clip(rng.lognormal(6.2, 0.6), 16, 768))
        waiting.append((t, prompt, int(rng.integers(1, 40))))
    waiting.reverse()                               # pop() takes the earliest
    lens, left = {}, {}                             # running: row -> context length / tokens still to generate
    free_rows = list(range(ROWS))[::-1]
    served = finished_total = checked = 0
    for step in range(steps):
        # sequences that are done give their blocks back (model.py:507-534)
        done = sorted(r for r in lens if left[r] == 0)
        if done:
            bm.free_blocks_for_seqs(torch.tensor(done, dtype=torch.int32, device=cuda), seq_ids_host=done)
            ob.free_blocks_for_seqs(np.asarray(done))
            for r in done:
                del lens[r], left[r]
                free_rows.append(r)
            finished_total += len(done)
        # admission: what has arrived by now, as long as rows, batch slots and blocks last (decode growth first)
        budget = ob.num_free_blocks - sum(1 for r in lens if lens[r] % B == 0)
        new = []
        while waiting and waiting[-1][0] <= step and free_rows and len(lens) + len(new) < MAX_RUNNING:
            _, prompt, gen = waiting[-1]
            need = -(-prompt // B)
            if need > budget or prompt + gen > MAX_BLOCKS * B:
                break
            waiting.pop()
            budget -= need
            new.append((free_rows.pop(), prompt, gen))
        running = sorted(lens)
        p_lens = [p for _, p, _ in new]
        d_lens = [lens[r] + 1 for r in running]
        ids = [r for r, _, _ in new] + running
        if not ids:
            continue
        state = builder.build(p_lens, ids, d_lens, block_manager=bm)
        ob.allocate_blocks_for_seqs(np.asarray(ids), np.asarray(p_lens + d_lens))
        assert_state_equal(manager_state(bm), ob.snapshot(), f"step {step}: allocator state")
        check = step % CHECK_EVERY == 0 or step == steps - 1
        P, n = sum(p_lens), len(d_lens)
        T = P + n
        pos = _positions(p_lens, d_lens)
        cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
        starts = np.cumsum(p_lens) - np.asarray(p_lens) if p_lens else np.zeros(0, dtype=np.int64)
        for layer in range(L):
            q, k, v = rand_f16(rng, T, H, D), rand_f16(rng, T, H, D), rand_f16(rng, T, H, D)
            qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
            o = torch.full((T, H * D), float("nan"), dtype=torch.float16, device=cuda)
            attention_section(qg, kg, vg, o, pool.k_cache, pool.v_cache, pool.k_cache_new, pool.v_cache_new,
                              bm.block_table, model, engine, state, layer)
            RO.rotary_embedding_inplace(q, k, cos, sin)
            R.store_kvcache(arena, lay, k, v, ob.block_table, np.asarray(ids), len(p_lens), P, starts,
                            np.asarray(p_lens), np.asarray(d_lens), layer)
            if check:
                got = o.cpu().numpy().reshape(T, H, D)
                if P:
                    want = R.prefill_attention(q[:P], k[:P], v[:P], starts, np.asarray(p_lens), D ** -0.5, math="np32")
                    assert_attn_close(got[:P], np.asarray(want), f"step {step} layer {layer}: prefill rows")
                if n:
                    want = R.paged_attention(q[P:], arena, lay, ob.block_table, np.asarray(running), np.asarray(d_lens),
                                             D ** -0.5, layer)
                    assert_attn_close(got[P:], np.asarray(want), f"step {step} layer {layer}: decode rows")
        if check:
            torch.cuda.synchronize()
            assert np.array_equal(bits(pool.k_cache).reshape(-1), arena[:half].view(np.uint16)), f"step {step}: K pool"
            assert np.array_equal(bits(pool.v_cache).reshape(-1), arena[half:].view(np.uint16)), f"step {step}: V pool"
            checked += 1
        for r, prompt, gen in new:
            lens[r], left[r] = prompt, gen
            served += 1
        for r in running:
            lens[r] += 1
            left[r] -= 1
    # the run was a real interleave: many requests came and went, the pool was under load, checks happened
    assert served >= 40 and finished_total >= 25 and checked >= steps // CHECK_EVERY
    assert int(bm.num_free_blocks) == ob.num_free_blocks
