"""The virtual-memory pool (one contiguous tensor that grows and shrinks in place): fixed
address, data kept across resizes, fresh blocks zero, shrink with relocation and every
kernel of the path working on its memory -- all bit-exact against the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, assert_attn_close, rand_f16
from gpu_helpers import assert_state_equal, bits, manager_state
from morphserve_amd import VmmKVPool, build_infer_state, paged_attention, store_kvcache

pytestmark = pytest.mark.gpu

L, HKV, D, B = 2, 2, 128, 16


def _i32(x, dev):
    return torch.tensor(list(x), dtype=torch.int32, device=dev)


def _mirror(pool, num_blocks, rng):
    """Random bytes in the pool and the oracle's arena (plain layout: K then V)."""
    blk = L * HKV * B * D
    arena = rng.standard_normal(2 * num_blocks * blk, dtype=np.float32).astype(np.float16)
    pool.k_cache.copy_(torch.from_numpy(arena[:num_blocks * blk]).view_as(pool.k_cache))
    pool.v_cache.copy_(torch.from_numpy(arena[num_blocks * blk:]).view_as(pool.v_cache))
    return arena


def test_grow_and_shrink_in_place(cuda):
    pool = VmmKVPool(32, 128, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=64, chunk_blocks=16)
    try:
        rng = np.random.default_rng(0)
        k_addr, v_addr = pool.k_cache.data_ptr(), pool.v_cache.data_ptr()
        assert float(pool.k_cache.abs().sum()) == 0.0 and float(pool.v_cache.abs().sum()) == 0.0
        arena = _mirror(pool, 32, rng)
        ob = R.BlockManagerOracle("GPU", 32, 8, 64, B)
        pool.expand(48)
        ob.expand(48)
        assert pool.num_blocks == 80 and tuple(pool.k_cache.shape) == (80, L, HKV, B, D)
        assert pool.k_cache.data_ptr() == k_addr and pool.v_cache.data_ptr() == v_addr and pool.k_cache_new == []
        blk = L * HKV * B * D
        assert np.array_equal(bits(pool.k_cache[:32]), arena[:32 * blk].view(np.uint16).reshape(32, L, HKV, B, D))
        assert np.array_equal(bits(pool.v_cache[:32]), arena[32 * blk:].view(np.uint16).reshape(32, L, HKV, B, D))
        assert float(pool.k_cache[32:].abs().sum()) == 0.0 and float(pool.v_cache[32:].abs().sum()) == 0.0
        assert_state_equal(manager_state(pool.block_manager), ob.snapshot(), "grown")
        assert pool.block_manager.num_blocks_org == 32
        with pytest.raises(ValueError):
            pool.expand(8)                    # not a multiple of the chunk
        with pytest.raises(ValueError):
            pool.expand(64)                   # beyond the reservation
        pool.k_cache[32:] = 3.0               # dirty the tail, drop it, map it again: zero
        assert pool.tail_unused(48)
        pool.shrink_to(32)
        assert pool.num_blocks == 32 and pool.k_cache.data_ptr() == k_addr
        assert np.array_equal(bits(pool.k_cache), arena[:32 * blk].view(np.uint16).reshape(32, L, HKV, B, D))
        pool.expand(16)
        assert float(pool.k_cache[32:].abs().sum()) == 0.0
    finally:
        pool.close()


@pytest.mark.parametrize("seed,total,keep,live_frac", [(0, 64, 32, 0.3), (1, 96, 16, 0.12), (2, 48, 32, 0.6)])
def test_shrink_with_relocation_bit_exact(cuda, seed, total, keep, live_frac):
    pool = VmmKVPool(total, 128, L, HKV, B, D, max_seqs_in_block_table=24, max_blocks_per_seq=total, chunk_blocks=16)
    try:
        rng = np.random.default_rng(seed)
        arena = _mirror(pool, total, rng)
        lay = R.plain_layout(total, L, HKV, B, D)
        n_live = int(live_frac * total)
        live = np.random.default_rng(seed + 100).permutation(total)[:n_live]
        ob = R.BlockManagerOracle("GPU", total, 24, total, B)
        cuts = np.sort(rng.choice(np.arange(1, n_live), size=min(7, n_live - 1), replace=False))
        for s, ids in enumerate(np.split(live, cuts)):
            ob.block_table[s, :len(ids)] = ids
            ob.num_seq_allocated_blocks[s] = len(ids)
        ob.is_block_free[live] = False
        ob.num_free_blocks = total - n_live
        ob.block_table[20, :2] = [total - 1, 0]              # stale ids of a freed row stay
        bm = pool.block_manager
        bm.block_table.copy_(torch.from_numpy(ob.block_table))
        bm.num_seq_allocated_blocks.copy_(torch.from_numpy(ob.num_seq_allocated_blocks))
        bm.is_block_free.copy_(torch.from_numpy(ob.is_block_free))
        bm.num_free_blocks = ob.num_free_blocks
        want_src, want_dst = R.apply_migration(arena, lay, ob, keep)
        src, dst = pool.shrink_to(keep)
        assert src.cpu().tolist() == want_src.tolist() and dst.cpu().tolist() == want_dst.tolist()
        assert_state_equal(manager_state(bm), ob.snapshot(), "after shrink")
        blk = lay.block_elems
        assert np.array_equal(bits(pool.k_cache).reshape(-1), arena[:keep * blk].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache).reshape(-1), arena[total * blk:(total + keep) * blk].view(np.uint16))
    finally:
        pool.close()


def test_shrink_refused_when_it_does_not_fit(cuda):
    pool = VmmKVPool(32, 32, L, HKV, B, D, max_seqs_in_block_table=4, max_blocks_per_seq=32, chunk_blocks=16)
    try:
        bm = pool.block_manager
        bm.allocate_blocks_for_seqs(_i32([1], cuda), _i32([16 * 20], cuda))
        before = manager_state(bm)
        with pytest.raises(RuntimeError, match="cannot shrink"):
            pool.shrink_to(16)
        assert_state_equal(manager_state(bm), before, "refused") and pool.num_blocks == 32
    finally:
        pool.close()


def test_append_and_attention_on_mapped_memory(cuda):
    """The kernels address a grown pool as one tensor: ids beyond the first size are plain
    indices (no extension segments)."""
    pool = VmmKVPool(16, 64, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=32, chunk_blocks=16)
    try:
        pool.expand(32)
        bm = pool.block_manager
        lens = [200, 33, 17, 120]
        ids = [3, 0, 5, 1]
        ob = R.BlockManagerOracle("GPU", 48, 8, 32, B)
        got = bm.allocate_blocks_for_seqs(_i32(ids, cuda), _i32(lens, cuda))
        want = ob.allocate_blocks_for_seqs(ids, lens)
        assert got.cpu().tolist() == want.tolist() and int(want.max()) >= 16
        lay = R.plain_layout(48, L, HKV, B, D)
        arena = np.zeros(2 * 48 * lay.block_elems, dtype=np.float16)
        rng = np.random.default_rng(3)
        model = Cfg(num_layers=L, num_q_heads=2 * HKV, num_kv_heads=HKV, head_dim=D)
        engine = Cfg(block_size=B, max_blocks_per_seq=32)
        st = build_infer_state(lens, ids, [], HKV, D)
        T = sum(lens)
        starts = np.cumsum(lens) - np.asarray(lens)
        for layer in range(L):
            k, v = rand_f16(rng, T, HKV, D), rand_f16(rng, T, HKV, D)
            R.store_kvcache(arena, lay, k, v, ob.block_table, np.asarray(ids, np.int32), len(lens), T, starts,
                            np.asarray(lens), np.zeros(0, np.int64), layer)
            store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), pool.k_cache, pool.v_cache,
                          [], [], bm.block_table, model, engine, st, layer)
        torch.cuda.synchronize()
        blk = lay.block_elems
        assert np.array_equal(bits(pool.k_cache).reshape(-1), arena[:48 * blk].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache).reshape(-1), arena[48 * blk:].view(np.uint16))
        q = rand_f16(rng, len(lens), 2 * HKV, D)
        dst = build_infer_state([], ids, lens, HKV, D)
        o = torch.empty((len(lens), 2 * HKV * D), dtype=torch.float16, device=cuda)
        paged_attention(torch.from_numpy(q).to(cuda), pool.k_cache, pool.v_cache, [], [], bm.block_table, model,
                        engine, dst, 1, o)
        want_o = R.paged_attention(q, arena, lay, ob.block_table, np.asarray(ids, np.int32), np.asarray(lens),
                                   D ** -0.5, 1)
        assert_attn_close(o.cpu().numpy().reshape(len(lens), 2 * HKV, D), np.asarray(want_o), "attention on the grown pool")
    finally:
        pool.close()


def test_eviction_on_a_virtual_memory_pool(cuda):
    """KVSwapper over a grown VmmKVPool: ids beyond the first size are swapped like any other."""
    from morphserve_amd import KVSwapper
    pool = VmmKVPool(16, 64, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=32, chunk_blocks=16)
    try:
        pool.expand(16)
        rng = np.random.default_rng(9)
        arena = _mirror(pool, 32, rng)
        lay = R.plain_layout(32, L, HKV, B, D)
        bm = pool.block_manager
        ob = R.BlockManagerOracle("GPU", 32, 8, 32, B)
        ids, lens = [2, 5, 0], [16 * 9, 16 * 12, 40]
        bm.allocate_blocks_for_seqs(_i32(ids, cuda), _i32(lens, cuda))
        ob.allocate_blocks_for_seqs(ids, lens)
        sw = KVSwapper(pool, 24)
        ocpu = R.BlockManagerOracle("CPU", 24, 8, 32, B)
        ks, vs = np.zeros(sw.k_swap.shape, np.float16), np.zeros(sw.v_swap.shape, np.float16)

        def oracle_swap(src_bm, dst_bm, seqs, is_in):
            ln = src_bm.get_num_allocated_blocks(seqs) * B
            src = src_bm.gather_allocated_blocks_and_free(seqs)
            dst = dst_bm.allocate_blocks_for_seqs(seqs, ln)
            R.swap_blocks(arena, lay, ks, vs, src, dst, is_in)
            return len(src)

        assert sw.swap_out_seqs([5, 2]) == oracle_swap(ob, ocpu, [5, 2], False) == 21
        bm.allocate_blocks_for_seqs(_i32([7], cuda), _i32([16 * 5], cuda))     # takes some freed low ids
        ob.allocate_blocks_for_seqs([7], [16 * 5])
        assert sw.swap_in_seqs([2, 5]) == oracle_swap(ocpu, ob, [2, 5], True)
        torch.cuda.synchronize()
        assert_state_equal(manager_state(bm), ob.snapshot(), "gpu manager")
        assert_state_equal(manager_state(sw.cpu_block_manager), ocpu.snapshot(), "cpu manager")
        assert np.array_equal(bits(sw.k_swap), bits(ks)) and np.array_equal(bits(sw.v_swap), bits(vs))
        blk = lay.block_elems
        assert np.array_equal(bits(pool.k_cache).reshape(-1), arena[:32 * blk].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache).reshape(-1), arena[32 * blk:].view(np.uint16))
    finally:
        pool.close()
