"""A small serving loop driven by the scheduler's own pressure arithmetic: prompts that do
not fit grow the pool by segments, sequences finish, and with nothing waiting the scheduler
gives segments back -- relocating the live blocks they hold.  Block-manager state, every
cache byte and the logical KV of every live sequence are checked against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, rand_f16
from gpu_helpers import assert_state_equal, bits, manager_state
from morphserve_amd import ElasticKVPool, VmmKVPool, build_infer_state, store_kvcache
from morphserve_amd.server import (PoolEngine, Request, Scheduler, org2quant_and_update_kvcache,
                                   quant2org_and_update_kvcache)

pytestmark = pytest.mark.gpu

L, HKV, D, B = 2, 2, 128, 16
ORG, S, MAX_SEG = 16, 8, 4


class Mirror:
    """Oracle-side twin of the pool: arena with room for MAX_SEG segments + block manager."""

    def __init__(self, contiguous=False):
        blk = L * HKV * B * D
        self.contiguous = contiguous
        if contiguous:                       # one K tensor and one V tensor with room for every segment
            self.lay = R.plain_layout(ORG + MAX_SEG * S, L, HKV, B, D)
            self.arena = np.zeros(2 * (ORG + MAX_SEG * S) * blk, dtype=np.float16)
            self.bm = R.BlockManagerOracle("GPU", ORG, 16, 32, B)
            self.nseg = 0
            return
        self.lay = R.PoolLayout(L, HKV, B, D, k_base=0, v_base=ORG * blk, num_blocks_org=ORG, seg_blocks=S,
                                k_seg=[2 * ORG * blk + j * 2 * S * blk for j in range(MAX_SEG)],
                                v_seg=[2 * ORG * blk + j * 2 * S * blk + S * blk for j in range(MAX_SEG)])
        self.arena = np.zeros(2 * (ORG + MAX_SEG * S) * blk, dtype=np.float16)
        self.bm = R.BlockManagerOracle("GPU", ORG, 16, 32, B)
        self.nseg = 0


def _pool_bytes(pool):
    parts = [pool.k_cache.reshape(-1), pool.v_cache.reshape(-1)]
    for k, v in zip(pool.k_cache_new, pool.v_cache_new):
        parts += [k.reshape(-1), v.reshape(-1)]
    return bits(torch.cat(parts))


@pytest.mark.parametrize("backing", ["segments", "virtual_memory"])
def test_pressure_driven_growth_and_migrating_give_back(cuda, backing):
    rng = np.random.default_rng(11)
    vmm = backing == "virtual_memory"
    ecfg = Cfg(block_size=B, max_batch_size=8, max_tokens_in_batch=4096, num_cpu_blocks=64,
               max_seqs_in_block_table=16, max_blocks_per_seq=32, quant_serve=True,
               num_layers_to_quantize=2, num_layers_to_quantize_max=0)
    mcfg = Cfg(num_layers=L, num_q_heads=HKV, num_kv_heads=HKV, head_dim=D)
    if vmm:
        pool = VmmKVPool(ORG, ORG + MAX_SEG * S, L, HKV, B, D, max_seqs_in_block_table=16, max_blocks_per_seq=32,
                         chunk_blocks=S)
    else:
        pool = ElasticKVPool(ORG, L, HKV, B, D, max_seqs_in_block_table=16, max_blocks_per_seq=32)
    engine = PoolEngine(pool, ecfg, num_layers=6, seg_blocks=S, migrate=True)
    mir = Mirror(contiguous=vmm)
    events = []

    def grow(e):
        org2quant_and_update_kvcache(e)
        mir.bm.expand(S)
        mir.nseg += 1
        events.append("grow")

    def give_back(e):
        before = pool.num_blocks
        moved_before = e.migrated_blocks
        ok = quant2org_and_update_kvcache(e)
        if ok:
            if mir.bm.tail_segment_unused(S, mir.nseg):
                assert mir.bm.shrink(S, mir.nseg) and e.migrated_blocks == moved_before
                events.append("drop")
            else:
                src, _ = R.apply_migration(mir.arena, mir.lay, mir.bm, before - S)
                assert e.migrated_blocks - moved_before == len(src) > 0
                events.append(f"migrate{len(src)}")
            mir.nseg -= 1
        return ok

    sched = Scheduler(mcfg, ecfg, ORG, grow=grow, give_back=give_back)
    engine.scheduler = sched
    bm = pool.block_manager
    history = {}                       # request -> [k rows, v rows] per layer, appended so far

    def dev_i32(x):
        return torch.tensor(list(x), dtype=torch.int32, device=cuda)

    def append(reqs, p_lens, d_lens):
        ids = [r.request_id for r in reqs]
        T = int(sum(p_lens))
        st = build_infer_state(p_lens, ids, d_lens, HKV, D, num_blocks_org=ORG,
                               kv_cache_new_block_size=pool.kv_cache_new_block_size)
        starts = np.cumsum(p_lens) - np.asarray(p_lens) if len(p_lens) else np.zeros(0, dtype=np.int64)
        for layer in range(L):
            k = rand_f16(rng, T + len(d_lens), HKV, D)
            v = rand_f16(rng, T + len(d_lens), HKV, D)
            R.store_kvcache(mir.arena, mir.lay, k, v, mir.bm.block_table, np.asarray(ids, dtype=np.int32),
                            len(p_lens), T, starts, np.asarray(p_lens), np.asarray(d_lens), layer)
            store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), pool.k_cache, pool.v_cache,
                          pool.k_cache_new, pool.v_cache_new, bm.block_table, mcfg, ecfg, st, layer)
            pos = 0
            for j, r in enumerate(reqs):
                n = p_lens[j] if j < len(p_lens) else 1
                h = history.setdefault(id(r), [[[], []] for _ in range(L)])
                h[layer][0].append(k[pos:pos + n])
                h[layer][1].append(v[pos:pos + n])
                pos += n

    def step():
        batch, swapped_in, swapped_out = sched.get_next_batch(engine)
        assert not swapped_in and not swapped_out
        prefill = batch is not sched.running_q
        reqs = list(batch)
        if not reqs:
            return
        lens = [r.prompt_len + r.output_len for r in reqs]     # a decode row's length counts its new token
        ids = [r.request_id for r in reqs]
        got = bm.allocate_blocks_for_seqs(dev_i32(ids), dev_i32(lens))
        want = mir.bm.allocate_blocks_for_seqs(ids, lens)
        assert got.cpu().tolist() == want.tolist()
        if prefill:
            append(reqs, [r.prompt_len for r in reqs], [])
        else:
            append(reqs, [], lens)
        for r in reqs:
            r.output_len += 1
        done = [r for r in reqs if r.is_finished()]
        if done:
            bm.free_blocks_for_seqs(dev_i32([r.request_id for r in done]))
            mir.bm.free_blocks_for_seqs([r.request_id for r in done])
            for r in done:
                history.pop(id(r))
        sched.on_batch_finish(reqs)
        torch.cuda.synchronize()
        assert_state_equal(manager_state(bm), mir.bm.snapshot(), f"after step ({events})")

    r0 = Request(prompt_len=200, max_output_len=3)          # 13 blocks
    r1 = Request(prompt_len=100, max_output_len=40)         # 7 blocks: 20 > 16 -> two segments
    r2 = Request(prompt_len=120, max_output_len=40)         # 8 blocks
    sched.on_requests_arrival([r0, r1, r2])
    step()                                                  # prefill of all three after growth
    assert events == ["grow", "grow"] and pool.num_blocks == 32 and sched.num_gpu_blocks == 32
    assert [r.request_id for r in (r0, r1, r2)] == [0, 1, 2]
    step()
    step()                                                  # r0 finishes: 13 blocks free again
    assert r0.is_finished() and sched.running_q == [r1, r2]
    step()   # 17 free >= 2 segments' worth, nothing waiting: both segments go, live blocks move below 16
    assert events == ["grow", "grow", "migrate4", "migrate8"], events
    assert pool.num_blocks == 16 and sched.num_gpu_blocks == 16 and len(pool.k_cache_new) == 0
    assert tuple(pool.k_cache.shape)[0] == 16
    assert engine.model.next_unquantized_layer == 5 and engine.model.layer_quant_list == []
    for _ in range(3):
        step()                                              # appends keep landing through the rewritten tables
    sched.on_requests_arrival([Request(prompt_len=60, max_output_len=2)])   # 15 + 4 > 16: grows again
    step()
    assert events[4:] == ["grow", "grow"] and pool.num_blocks == 32
    step()
    step()

    # every byte of the pool, and the logical KV of each live sequence through its table
    if vmm:
        nb, cap, be = pool.num_blocks, ORG + MAX_SEG * S, mir.lay.block_elems
        assert pool.k_cache_new == [] and nb in (16, 32)
        assert np.array_equal(bits(pool.k_cache).reshape(-1), mir.arena[:nb * be].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache).reshape(-1), mir.arena[cap * be:(cap + nb) * be].view(np.uint16))
    else:
        keep = 2 * ORG * mir.lay.block_elems + len(pool.k_cache_new) * 2 * S * mir.lay.block_elems
        assert np.array_equal(_pool_bytes(pool), mir.arena[:keep].view(np.uint16))
    table = bm.block_table.cpu().numpy()
    caches = {"k": [pool.k_cache] + pool.k_cache_new, "v": [pool.v_cache] + pool.v_cache_new}
    for r in sched.running_q:
        n = r.prompt_len + r.output_len - 1                 # the newest token has not been appended yet
        for layer in range(L):
            for w, which in enumerate("kv"):
                want = np.concatenate(history[id(r)][layer][w], axis=0)
                assert want.shape[0] == n
                rows = []
                for j in range((n + B - 1) // B):
                    pid = int(table[r.request_id, j])
                    seg, local = (0, pid) if (vmm or pid < ORG) else (1 + (pid - ORG) // S, (pid - ORG) % S)
                    blkt = caches[which][seg][local, layer].cpu().numpy()        # [Hkv, B, D]
                    rows.append(np.transpose(blkt, (1, 0, 2)))
                got = np.concatenate(rows, axis=0)[:n]
                assert np.array_equal(bits(got), bits(want)), (r.request_id, layer, which)
    if vmm:
        pool.close()
