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


@pytest.fixture(autouse=True, params=[0, 8192], ids=["plain", "v_staggered"])
def _v_stagger(request, monkeypatch):
    """Every test of this file runs twice: with the V tensor at the start of its range and 8 KiB into it (the
    placement a large pool may choose for itself; it maps one chunk more)."""
    import morphserve_amd.vmm_pool as VP
    orig = VP.VmmKVPool.__init__

    def init(self, *a, **k):
        k.setdefault("v_stagger_bytes", request.param)
        orig(self, *a, **k)
    monkeypatch.setattr(VP.VmmKVPool, "__init__", init)
    return request.param


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


# ---- a layer's memory moving into the pool and back ---------------------------------------------------------
def _free_device_bytes():
    import gc
    gc.collect()              # pools of earlier tests that are garbage by now release their memory here, not later
    torch.cuda.synchronize()
    return torch.cuda.mem_get_info()[0]


def test_pool_grows_out_of_a_replaced_layers_memory_and_gives_it_back(cuda):
    """``acquire_new_kvcache`` (csrc/src/memory_manager.cpp:69-176) over virtual memory: the chunks of a
    layer's arena behind the quantized copy become pool blocks (zero filled, free), the quantized bytes at
    the start of the arena and every old pool byte stay as they were, no device memory is allocated or
    freed on the way, and ``shrink_into`` (with live blocks above the cut) returns the memory to the layer."""
    from morphserve_amd import LayerArena
    cb, org = 64, 64
    pool = VmmKVPool(org, 256, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=32, chunk_blocks=cb)
    chunk = cb * pool.block_bytes                      # 1 MiB
    layer_bytes = 9 * chunk - 1000                     # fp16 layer: 9 chunks (the last one partly used)
    quant_bytes = 2 * chunk + 6                        # its quantized twin: needs 3 chunks
    layer = LayerArena(layer_bytes, chunk)
    try:
        rng = np.random.default_rng(5)
        blk = L * HKV * B * D
        mapped = lambda: layer.mapped_bytes() + pool._k_arena.mapped_bytes() + pool._v_arena.mapped_bytes()
        assert layer.capacity == 9 * chunk and layer.mapped_bytes() == 9 * chunk
        w = layer.tensor(0, (layer_bytes // 2,), torch.float16)
        w.copy_(torch.from_numpy(rng.standard_normal(layer_bytes // 2, dtype=np.float32).astype(np.float16)))
        head = bits(layer.tensor(0, (quant_bytes // 2,), torch.float16))
        arena = _mirror(pool, org, rng)
        k_addr, v_addr = pool.k_cache.data_ptr(), pool.v_cache.data_ptr()
        ob = R.BlockManagerOracle("GPU", org, 8, 32, B)
        total_mapped, free_before = mapped(), _free_device_bytes()

        assert pool.blocks_available_from(layer, quant_bytes) == 3 * cb              # (9 - 3) // 2 chunks each
        n = pool.expand_from(layer, quant_bytes)
        ob.expand(n)
        assert n == 192 and pool.num_blocks == 256 and layer.mapped_bytes() == 3 * chunk
        assert mapped() == total_mapped and abs(_free_device_bytes() - free_before) < 4 * chunk   # 6 chunks moved
        assert pool.k_cache.data_ptr() == k_addr and pool.v_cache.data_ptr() == v_addr
        assert np.array_equal(bits(pool.k_cache[:org]).reshape(-1), arena[:org * blk].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache[:org]).reshape(-1), arena[org * blk:].view(np.uint16))
        assert not pool.k_cache[org:].any() and not pool.v_cache[org:].any()         # the old weights are gone
        assert_state_equal(manager_state(pool.block_manager), ob.snapshot(), "grown out of the layer")
        assert np.array_equal(bits(layer.tensor(0, (quant_bytes // 2,), torch.float16)), head)   # the twin is untouched
        with pytest.raises(ValueError):
            layer.tensor(3 * chunk, (16,), torch.float16)                             # no longer the layer's

        # sequences that live in the new blocks; then the layer comes back and they move below the cut
        bm = pool.block_manager
        lens = [16 * 30, 16 * 30, 16 * 25, 16 * 9, 40]
        ids = list(range(len(lens)))
        bm.allocate_blocks_for_seqs(_i32(ids, cuda), _i32(lens, cuda))
        ob.allocate_blocks_for_seqs(np.array(ids), np.array(lens))
        bm.free_blocks_for_seqs(_i32([0, 1], cuda))
        ob.free_blocks_for_seqs(np.array([0, 1]))
        lens2 = [16 * 12, 16 * 3]
        bm.allocate_blocks_for_seqs(_i32([5, 6], cuda), _i32(lens2, cuda))
        ob.allocate_blocks_for_seqs(np.array([5, 6]), np.array(lens2))
        total = pool.num_blocks
        full = _mirror(pool, total, rng)
        lay = R.plain_layout(total, L, HKV, B, D)
        want_src, want_dst = R.apply_migration(full, lay, ob, org)
        src, dst = pool.shrink_into(layer, org)
        assert len(want_src) > 0 and src.cpu().tolist() == want_src.tolist() and dst.cpu().tolist() == want_dst.tolist()
        assert_state_equal(manager_state(bm), ob.snapshot(), "after the layer came back")
        assert np.array_equal(bits(pool.k_cache).reshape(-1), full[:org * blk].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache).reshape(-1), full[total * blk:(total + org) * blk].view(np.uint16))
        assert layer.mapped_bytes() == 9 * chunk and mapped() == total_mapped
        assert abs(_free_device_bytes() - free_before) < 4 * chunk
        assert np.array_equal(bits(layer.tensor(0, (quant_bytes // 2,), torch.float16)), head)
        w = layer.tensor(0, (layer_bytes // 2,), torch.float16)                      # the restored weights fit again
        w.fill_(1.5)
        assert float(w.min()) == 1.5 and pool.k_cache.data_ptr() == k_addr
        assert np.array_equal(bits(pool.k_cache).reshape(-1), full[:org * blk].view(np.uint16))
    finally:
        layer.close()
        pool.close()


def test_hand_over_limits(cuda):
    from morphserve_amd import LayerArena, _capi
    pool = VmmKVPool(32, 64, L, HKV, B, D, max_seqs_in_block_table=4, max_blocks_per_seq=16, chunk_blocks=16)
    chunk = 16 * pool.block_bytes
    layer = LayerArena(10 * chunk, chunk)
    other = LayerArena(chunk, 2 * chunk)
    try:
        assert pool.blocks_available_from(layer, 0) == 32           # capped by the reservation (64 - 32 blocks)
        with pytest.raises(ValueError):
            pool.blocks_available_from(other, 0)                     # another chunk size
        assert pool.expand_from(layer, 10 * chunk) == 0 and pool.num_blocks == 32   # the twin needs it all
        assert pool.expand_from(layer, 9 * chunk) == 0               # one spare chunk cannot serve K and V
        assert pool.expand_from(layer, 0) == 32 and layer.mapped_bytes() == 6 * chunk
        with pytest.raises(ValueError):
            pool.shrink_to(48, other)
        lib = _capi.lib()
        assert lib.mkv_arena_move_tail(layer.handle, layer.handle, chunk) == _capi.MKV_EINVAL
        assert lib.mkv_arena_move_tail(layer.handle, other.handle, 2 * chunk) == _capi.MKV_EINVAL   # chunk sizes differ
        assert lib.mkv_arena_move_tail(layer.handle, pool._k_arena.handle, chunk) == _capi.MKV_EINVAL  # reservation full
        assert lib.mkv_arena_move_tail(layer.handle, pool._k_arena.handle, chunk // 2) == _capi.MKV_EINVAL
        pool.shrink_into(layer, 32)
        assert layer.mapped_bytes() == 10 * chunk
        with pytest.raises(ValueError):
            pool.shrink_into(layer, 16)                              # the layer's arena is complete already
    finally:
        other.close()
        layer.close()
        pool.close()


def test_layer_replacement_bookkeeping_over_layer_arenas(cuda):
    """``org2quant_and_update_kvcache`` / ``quant2org_and_update_kvcache`` (memory_utils.py:93-116, :617-659)
    with the pool's growth coming out of each replaced layer's own arena and going back into it."""
    from morphserve_amd import LayerArena
    from morphserve_amd.server.memory_utils import (PoolEngine, org2quant_and_update_kvcache,
                                                    quant2org_and_update_kvcache)
    cb = 16
    pool = VmmKVPool(32, 32 + 2 * 48, L, HKV, B, D, max_seqs_in_block_table=4, max_blocks_per_seq=64, chunk_blocks=cb)
    chunk = cb * pool.block_bytes
    arenas = {0: LayerArena(8 * chunk, chunk), 1: LayerArena(8 * chunk, chunk)}
    try:
        eng = PoolEngine(pool, None, num_layers=2, seg_blocks=0, layer_arenas=arenas, quant_layer_bytes=2 * chunk - 7)
        org2quant_and_update_kvcache(eng)                                  # the last layer goes first (model.py:81)
        assert pool.num_blocks == 80 and arenas[1].mapped_bytes() == 2 * chunk and arenas[0].mapped_bytes() == 8 * chunk
        assert eng.model.kv_cache_new_block_size == 48 and eng.model.layer_quant_list == [1]
        org2quant_and_update_kvcache(eng)
        assert pool.num_blocks == 128 and arenas[0].mapped_bytes() == 2 * chunk
        with pytest.raises(RuntimeError):
            org2quant_and_update_kvcache(eng)                              # no layer left
        bm = pool.block_manager
        bm.allocate_blocks_for_seqs(_i32([0, 1], cuda), _i32([16 * 60, 16 * 50], cuda))      # blocks 0..109
        bm.free_blocks_for_seqs(_i32([0], cuda))                                              # 60..109 stay live
        mark = torch.arange(128, dtype=torch.float16, device=cuda).view(128, 1, 1, 1, 1)
        pool.k_cache.copy_(mark.expand_as(pool.k_cache))
        pool.v_cache.copy_((-mark).expand_as(pool.v_cache))
        row_before = bm.block_table[1, :50].cpu().tolist()
        assert quant2org_and_update_kvcache(eng) is True                   # layer 0 comes back: cut at 80
        assert pool.num_blocks == 80 and arenas[0].mapped_bytes() == 8 * chunk and eng.migrated_blocks == 30
        row = bm.block_table[1, :50].cpu().tolist()
        assert row_before == list(range(60, 110)) and row[:20] == list(range(60, 80)) and row[20:] == list(range(30))
        assert pool.k_cache[row, 0, 0, 0, 0].cpu().tolist() == [float(x) for x in range(60, 110)]
        assert pool.v_cache[row, 1, 1, 15, 127].cpu().tolist() == [-float(x) for x in range(60, 110)]
        assert quant2org_and_update_kvcache(eng) is False                  # 50 live blocks do not fit in 32
        assert pool.num_blocks == 80 and arenas[1].mapped_bytes() == 2 * chunk
        bm.free_blocks_for_seqs(_i32([1], cuda))
        assert quant2org_and_update_kvcache(eng) is True
        assert pool.num_blocks == 32 and arenas[1].mapped_bytes() == 8 * chunk and eng.model.layer_quant_list == []
    finally:
        for a in arenas.values():
            a.close()
        pool.close()
