"""Config 5 at its own geometry: CodeLlama-34B shapes (48 layers x 8 kv heads, 3 MiB blocks), a pool of
63 578 blocks (186 GiB) and a pressure-driven release of 25 % of them with live migration.

The release is decided by the scheduler's own rule (MorphServe/server/scheduler.py:75-89 ``try_quant2org`` ->
MorphServe/server/memory_utils.py:617-662 ``quant2org_and_update_kvcache``, with the refusal at :623-624
replaced by the relocation).  Checked: the move lists equal the CPU plan element by element, every
sequence's blocks carry the same bytes afterwards, the free map and counters equal the oracle's, and decode
attention on three layers AFTER the shrink matches ``R.paged_attention`` on a compacted host copy.
"""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, assert_attn_close
from gpu_helpers import assert_state_equal, manager_state
from morphserve_amd import ElasticKVPool, build_infer_state, paged_attention
from morphserve_amd.server import PoolEngine, Request, Scheduler

pytestmark = pytest.mark.gpu


def _free_gib():
    import gc
    gc.collect()
    torch.cuda.empty_cache()
    return torch.cuda.mem_get_info()[0] / 2 ** 30


def test_config5_pressure_shrink_at_full_size(cuda):
    if _free_gib() < 200:
        pytest.skip("needs 200 GiB of free device memory: the pool alone is 186 GiB")
    L, HQ, HKV, D, B, N = 48, 64, 8, 128, 16, 128
    KEEP, SEG = 47684, 15894
    total = KEEP + SEG
    max_seqs, max_bps = 256, 128
    rng = np.random.default_rng(55)
    lens = rng.integers(1024, 1537, size=N).astype(np.int32)
    nblk = (lens.astype(np.int64) + B - 1) // B
    pool = ElasticKVPool(KEEP, L, HKV, B, D, max_seqs_in_block_table=max_seqs, max_blocks_per_seq=max_bps)
    pool.expand(SEG)
    bm = pool.block_manager
    # seeded live set over the whole 63 578-block range, loaded into the manager and into the oracle
    ob = R.BlockManagerOracle("GPU", KEEP, max_seqs, max_bps, B)
    ob.expand(SEG)
    perm = rng.permutation(total)
    seq_ids = rng.permutation(max_seqs)[:N].astype(np.int32)
    pos = 0
    for i in range(N):
        ob.block_table[seq_ids[i], :nblk[i]] = perm[pos:pos + nblk[i]]
        ob.num_seq_allocated_blocks[seq_ids[i]] = nblk[i]
        pos += nblk[i]
    live = perm[:pos].copy()
    ob.is_block_free[live] = False
    ob.num_free_blocks = total - len(live)
    bm.block_table.copy_(torch.from_numpy(ob.block_table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(ob.num_seq_allocated_blocks))
    bm.is_block_free.copy_(torch.from_numpy(ob.is_block_free))
    bm.num_free_blocks = ob.num_free_blocks
    assert int((live >= KEEP).sum()) > 2000            # a quarter of the live blocks sit above the cut

    # N(0,1) in every live block, all layers
    gen = torch.Generator(device=cuda)
    gen.manual_seed(7)
    tail = (L, HKV, B, D)
    for ids, kt, vt, off in ((live[live < KEEP], pool.k_cache, pool.v_cache, 0),
                             (live[live >= KEEP], pool.k_cache_new[0], pool.v_cache_new[0], KEEP)):
        idt = torch.from_numpy(ids - off).to(cuda)
        for c0 in range(0, len(ids), 128):
            idx = idt[c0:c0 + 128]
            kt[idx] = torch.randn((len(idx), *tail), dtype=torch.float16, device=cuda, generator=gen)
            vt[idx] = torch.randn((len(idx), *tail), dtype=torch.float16, device=cuda, generator=gen)

    weights = torch.arange(1, 4097, dtype=torch.int64, device=cuda)

    def rows_of(ids):
        """int16 views [n, block elems] of K and V for global block ids (base pool or the one segment)."""
        ids = torch.as_tensor(np.asarray(ids), device=cuda).long()
        nseg = len(pool.k_cache_new)
        outk = torch.empty((len(ids), L * HKV * B * D), dtype=torch.int16, device=cuda)
        outv = torch.empty_like(outk)
        low = ids < KEEP
        if bool(low.any()):
            outk[low] = pool.k_cache.view(torch.int16).reshape(KEEP, -1)[ids[low]]
            outv[low] = pool.v_cache.view(torch.int16).reshape(KEEP, -1)[ids[low]]
        if bool((~low).any()):
            assert nseg == 1
            outk[~low] = pool.k_cache_new[0].view(torch.int16).reshape(SEG, -1)[ids[~low] - KEEP]
            outv[~low] = pool.v_cache_new[0].view(torch.int16).reshape(SEG, -1)[ids[~low] - KEEP]
        return outk, outv

    def checksums(ids):
        out = []
        for c0 in range(0, len(ids), 256):
            kk, vv = rows_of(ids[c0:c0 + 256])
            sk = (kk.view(len(kk), -1, 4096).to(torch.int64) * weights).sum(dim=(1, 2))
            sv = (vv.view(len(vv), -1, 4096).to(torch.int64) * weights).sum(dim=(1, 2))
            out.append(sk * 31 + sv)
        return torch.cat(out)

    logical = np.concatenate([ob.block_table[seq_ids[i], :nblk[i]] for i in range(N)])      # sequence-major
    before = checksums(logical)

    # the scheduler decides: running sequences only, nothing waiting, plenty of free blocks
    model = Cfg(num_layers=L, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    ecfg = Cfg(block_size=B, max_blocks_per_seq=max_bps, max_batch_size=256, max_tokens_in_batch=1 << 20,
               num_cpu_blocks=0, max_seqs_in_block_table=max_seqs, quant_serve=True, num_layers_to_quantize=1,
               num_layers_to_quantize_max=0)
    engine = PoolEngine(pool, ecfg, num_layers=L, seg_blocks=SEG, migrate=True)
    engine.model.layer_quant_list.append(L - 1)        # the segment came from replacing the last layer
    engine.model.is_layer_quant_list[L - 1] = True
    engine.model.next_unquantized_layer = L - 2
    sched = Scheduler(model, ecfg, total)
    engine.scheduler = sched
    for i in range(N):
        sched.running_q.append(Request(prompt_len=int(lens[i]) - 1, output_len=1, request_id=int(seq_ids[i])))
    moves = {}
    plain_shrink = pool.shrink_to

    def recording_shrink(new_n):
        moves["src"], moves["dst"] = plain_shrink(new_n)
        return moves["src"], moves["dst"]
    pool.shrink_to = recording_shrink
    want_src, want_dst = R.plan_migration(ob.is_block_free, KEEP)
    sched.get_next_batch(engine)
    torch.cuda.synchronize()
    assert pool.num_blocks == KEEP and not pool.k_cache_new and sched.num_gpu_blocks == KEEP, "no give-back happened"
    assert moves["src"].cpu().tolist() == want_src.tolist() and moves["dst"].cpu().tolist() == want_dst.tolist()
    assert engine.migrated_blocks == len(want_src) == int((live >= KEEP).sum())

    # the oracle's bookkeeping of the same shrink (a layout without payload: tables, map and counters only)
    R.apply_migration(np.zeros(0, dtype=np.float16), R.plain_layout(total, 0, HKV, B, D), ob, KEEP)
    assert_state_equal(manager_state(bm), ob.snapshot(), "after the pressure shrink")
    now = np.concatenate([ob.block_table[seq_ids[i], :nblk[i]] for i in range(N)])
    assert now.max() < KEEP and len(np.unique(now)) == len(now)
    assert torch.equal(checksums(now), before), "a sequence's KV changed during the migration"

    # decode attention after the shrink, three layers, against the oracle on a compacted host copy
    st = build_infer_state([], seq_ids.tolist(), lens.tolist(), HKV, D, num_blocks_org=bm.num_blocks_org,
                           kv_cache_new_block_size=pool.kv_cache_new_block_size)
    now_t = torch.from_numpy(now).to(cuda).long()
    small_table = np.full((max_seqs, max_bps), -1, dtype=np.int32)
    pos = 0
    for i in range(N):
        small_table[seq_ids[i], :nblk[i]] = np.arange(pos, pos + nblk[i])
        pos += nblk[i]
    lay = R.plain_layout(len(now), 1, HKV, B, D)
    for layer in (0, 17, 47):
        q = torch.randn((N, HQ, D), dtype=torch.float16, device=cuda, generator=gen)
        o = torch.full((N, HQ * D), float("nan"), dtype=torch.float16, device=cuda)
        paged_attention(q, pool.k_cache, pool.v_cache, pool.k_cache_new, pool.v_cache_new, bm.block_table, model,
                        ecfg, st, layer, o)
        torch.cuda.synchronize()
        arena = np.concatenate([pool.k_cache[now_t, layer].reshape(-1).cpu().numpy(),
                                pool.v_cache[now_t, layer].reshape(-1).cpu().numpy()])
        want = R.paged_attention(q.cpu().numpy(), arena, lay, small_table, seq_ids, lens, D ** -0.5, 0)
        assert_attn_close(o.cpu().numpy().reshape(N, HQ, D), np.asarray(want), f"layer {layer} after the shrink")
