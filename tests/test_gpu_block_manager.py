"""GPU parity of the block manager and the elastic pool against the CPU oracle:
block tables, per-sequence counts, free map and counters bit-exact after every
operation; migrated cache bytes bit-exact."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import make_case
from gpu_helpers import pool_bytes, pool_case, assert_state_equal, bits, load_manager, manager_state
from morphserve_amd import BlockManager, ElasticKVPool, swiftllm_c
from morphserve_amd.worker.kernels import block_mgmt

pytestmark = pytest.mark.gpu


def _i32(x, dev):
    return torch.tensor(np.asarray(x, dtype=np.int32), dtype=torch.int32, device=dev)


def test_hand_scenario(cuda):
    bm = BlockManager("GPU", 10, 4, 12, 16)
    ob = R.BlockManagerOracle("GPU", 10, 4, 12, 16)
    for ids, lens in (([2, 0], [33, 16]), ([0, 2], [17, 48]), ([0], [32])):
        got = bm.allocate_blocks_for_seqs(_i32(ids, cuda), _i32(lens, cuda))
        want = ob.allocate_blocks_for_seqs(ids, lens)
        assert got.dtype == torch.int64 and got.cpu().tolist() == want.tolist()
        assert_state_equal(manager_state(bm), ob.snapshot(), f"alloc {ids}")
    assert bm.num_free_blocks.item() == 5 and bm.num_free_blocks >= 5 and bm.get_num_used_blocks() == 5
    bm.free_blocks_for_seqs(_i32([2], cuda))
    ob.free_blocks_for_seqs([2])
    assert_state_equal(manager_state(bm), ob.snapshot(), "free")
    assert bm.block_table[2, :3].cpu().tolist() == [0, 1, 2], "freed rows keep their stale ids"
    got = bm.allocate_blocks_for_seqs(_i32([1], cuda), _i32([40], cuda))
    assert got.cpu().tolist() == ob.allocate_blocks_for_seqs([1], [40]).tolist() == [0, 1, 2]
    g = bm.gather_allocated_blocks_and_free(_i32([0, 1], cuda))
    assert g.dtype == torch.int32 and g.cpu().tolist() == ob.gather_allocated_blocks_and_free([0, 1]).tolist()
    assert_state_equal(manager_state(bm), ob.snapshot(), "gather")
    before = manager_state(bm)
    with pytest.raises(RuntimeError, match="No enough free blocks"):
        bm.allocate_blocks_for_seqs(_i32([3], cuda), _i32([16 * 11], cuda))
    assert_state_equal(manager_state(bm), before, "failed allocation must not change state")
    bm.allocate_blocks_for_seqs(_i32([3], cuda), _i32([64], cuda))
    ob.allocate_blocks_for_seqs([3], [64])
    with pytest.raises(AssertionError):
        bm.allocate_blocks_for_seqs(_i32([3], cuda), _i32([16], cuda))
    with pytest.raises(ValueError):
        bm.allocate_blocks_for_seqs(_i32([2], cuda), _i32([16 * 13], cuda))      # more than a table row holds
    with pytest.raises(ValueError):
        bm.allocate_blocks_for_seqs(_i32([4], cuda), _i32([16], cuda))           # no such sequence slot
    assert_state_equal(manager_state(bm), ob.snapshot() | {"num_free_blocks": int(bm.num_free_blocks)}, "rejected calls")
    empty = bm.allocate_blocks_for_seqs(_i32([], cuda), _i32([], cuda))
    assert empty.numel() == 0 and empty.dtype == torch.int64


@pytest.mark.parametrize("seed,num_blocks,max_seqs", [(0, 300, 32), (1, 40000, 700)])
def test_random_walk_bit_exact(cuda, seed, num_blocks, max_seqs):
    rng = np.random.default_rng(seed)
    mbs = 48
    bm = BlockManager("GPU", num_blocks, max_seqs, mbs, 16)
    ob = R.BlockManagerOracle("GPU", num_blocks, max_seqs, mbs, 16)
    lens = np.zeros(max_seqs, dtype=np.int64)
    for step in range(60):
        act = rng.integers(0, 4)
        k = int(rng.integers(1, max(2, max_seqs // 4)))
        ids = rng.permutation(max_seqs)[:k]
        if act <= 1:
            tgt = np.minimum(lens[ids] + rng.integers(0, 300, size=k), mbs * 16)
            try:
                want = ob.allocate_blocks_for_seqs(ids, tgt)
            except RuntimeError:
                with pytest.raises(RuntimeError):
                    bm.allocate_blocks_for_seqs(_i32(ids, cuda), _i32(tgt, cuda))
            else:
                got = bm.allocate_blocks_for_seqs(_i32(ids, cuda), _i32(tgt, cuda))
                assert got.cpu().tolist() == want.tolist()
                lens[ids] = np.maximum(lens[ids], tgt)
        elif act == 2:
            bm.free_blocks_for_seqs(_i32(ids, cuda))
            ob.free_blocks_for_seqs(ids)
            lens[ids] = 0
        else:
            got = bm.gather_allocated_blocks_and_free(_i32(ids, cuda))
            want = ob.gather_allocated_blocks_and_free(ids)
            assert got.cpu().tolist() == want.tolist()
            lens[ids] = 0
        assert_state_equal(manager_state(bm), ob.snapshot(), f"step {step} act {act}")
        counts = bm.get_num_allocated_blocks(_i32(ids, cuda)).cpu().numpy()
        assert np.array_equal(counts, ob.get_num_allocated_blocks(ids))


def test_table_kernels_reference_surface(cuda):
    """The three row kernels called the way the reference's BlockManager calls them."""
    bm = BlockManager("GPU", 64, 8, 16, 16)
    ob = R.BlockManagerOracle("GPU", 64, 8, 16, 16)
    ids = [5, 1, 6]
    need = torch.tensor([3, 0, 2], dtype=torch.int32, device=cuda)
    new = bm._allocate_blocks(5)
    assert new.cpu().tolist() == [0, 1, 2, 3, 4]
    block_mgmt.set_block_table_and_num_seq_alloc_blocks(bm.num_seq_allocated_blocks, bm.block_table,
                                                         new, _i32(ids, cuda), need)
    ob.allocate_blocks_for_seqs(ids, [48, 0, 32])
    assert_state_equal(manager_state(bm), ob.snapshot(), "set")
    block_mgmt.unset_block_table_and_num_seq_alloc_blocks(bm.num_seq_allocated_blocks, bm.block_table,
                                                           _i32([6], cuda), bm.is_block_free)
    bm.num_free_blocks += 2
    ob.free_blocks_for_seqs([6])
    assert_state_equal(manager_state(bm), ob.snapshot(), "unset")
    g = block_mgmt.gather_allocated_blocks_and_unset(bm.num_seq_allocated_blocks, bm.block_table,
                                                     _i32([1, 5], cuda), bm.is_block_free)
    assert g.cpu().tolist() == ob.gather_allocated_blocks_and_free([1, 5]).tolist() == [0, 1, 2]
    bm._free_blocks(torch.empty(0, dtype=torch.int64, device=cuda))


def test_carve_segment_and_acquire(cuda):
    swiftllm_c.register_kv_cache_info(2, 2, 4, 8)
    assert swiftllm_c.carve_segment(1000, 4000, 300) == R.acquire_new_kvcache_arith(1000, 4000, 300, 2, 2, 4, 8)
    with pytest.raises(RuntimeError, match="No space"):
        swiftllm_c.carve_segment(0, 1000, 600)
    with pytest.raises(RuntimeError, match="Layer not found"):
        swiftllm_c.acquire_new_kvcache(99)
    # a fake weight layer: first 1 KiB + 5 bytes stay "quantised weights", the rest becomes KV blocks
    weights = torch.full((64 * 1024,), 7, dtype=torch.uint8, device=cuda)
    base = weights.data_ptr()
    swiftllm_c.register_layer_memory_org_gpu(3, base, weights.numel())
    swiftllm_c.register_layer_memory_quant(3, base, 1029)
    k, v = swiftllm_c.acquire_new_kvcache(3, keepalive=weights)
    k0, S, v0 = R.acquire_new_kvcache_arith(base, weights.numel(), 1029, 2, 2, 4, 8)
    assert tuple(k.shape) == (S, 2, 2, 4, 8) and k.dtype == torch.float16
    assert k.data_ptr() == k0 and v.data_ptr() == v0
    torch.cuda.synchronize()
    w = weights.cpu().numpy()
    lo, hi = k0 - base, v0 - base + S * 256
    assert (w[:lo] == 7).all() and (w[lo:hi] == 0).all() and (w[hi:] == 7).all()
    k[1, 0, 1, 2, 3] = 5.0            # the views are writable device tensors
    assert float(k[1, 0, 1, 2, 3]) == 5.0


@pytest.mark.parametrize("seed,org,S,nseg,keep,live_frac", [(0, 16, 8, 4, 1, 0.3), (1, 32, 16, 6, 2, 0.45),
                                                           (2, 8, 4, 5, 0, 0.15)])
def test_shrink_with_migration_bit_exact(cuda, seed, org, S, nseg, keep, live_frac):
    pool, ob, arena, lay = pool_case(cuda, seed, org, S, nseg, live_frac)
    new_n = org + keep * S
    want_src, want_dst = R.apply_migration(arena, lay, ob, new_n)
    src, dst = pool.shrink_to(new_n)
    torch.cuda.synchronize()
    assert src.cpu().tolist() == want_src.tolist() and dst.cpu().tolist() == want_dst.tolist()
    assert_state_equal(manager_state(pool.block_manager), ob.snapshot(), "after shrink")
    assert len(pool.k_cache_new) == keep and pool.num_blocks == new_n
    blk = lay.block_elems
    kept = 2 * org * blk + keep * 2 * S * blk
    assert np.array_equal(pool_bytes(pool), arena[:kept].view(np.uint16))


def test_shrink_refused_when_live_blocks_do_not_fit(cuda):
    pool, ob, arena, lay = pool_case(cuda, 3, 8, 8, 3, 0.6)
    before_state = manager_state(pool.block_manager)
    before_bytes = pool_bytes(pool).copy()
    with pytest.raises(RuntimeError, match="cannot shrink"):
        pool.shrink_to(8)
    assert_state_equal(manager_state(pool.block_manager), before_state, "refused shrink")
    assert np.array_equal(pool_bytes(pool), before_bytes)
    assert len(pool.k_cache_new) == 3


def test_expand_shrink_round_trip(cuda):
    """Grow by two segments then drop them again: all state is restored; a live
    tail segment refuses the reference-style shrink."""
    pool = ElasticKVPool(8, 1, 2, 16, 128, max_seqs_in_block_table=4, max_blocks_per_seq=16)
    ob = R.BlockManagerOracle("GPU", 8, 4, 16, 16)
    bm = pool.block_manager
    bm.allocate_blocks_for_seqs(_i32([0], cuda), _i32([16 * 7], cuda))
    ob.allocate_blocks_for_seqs([0], [16 * 7])
    snap = manager_state(bm)
    pool.expand(4)
    pool.expand(4)
    ob.expand(4)
    ob.expand(4)
    assert_state_equal(manager_state(bm), ob.snapshot(), "expanded")
    assert bm.num_blocks_org == 8 and float(pool.k_cache_new[1].abs().sum()) == 0.0
    assert pool.shrink_tail_if_unused() and pool.shrink_tail_if_unused()
    assert ob.shrink(4, 2) and ob.shrink(4, 1)
    assert_state_equal(manager_state(bm), snap, "round trip")
    assert_state_equal(manager_state(bm), ob.snapshot(), "round trip vs oracle")
    pool.expand(4)
    pool.expand(4)
    ob.expand(4)
    ob.expand(4)
    bm.allocate_blocks_for_seqs(_i32([1], cuda), _i32([16 * 6], cuda))
    ob.allocate_blocks_for_seqs([1], [16 * 6])
    assert not pool.shrink_tail_if_unused() and not ob.shrink(4, 2)
    assert_state_equal(manager_state(bm), ob.snapshot(), "refused")
    bm.free_blocks_for_seqs(_i32([1], cuda))
    assert pool.shrink_tail_if_unused()


def test_step_state_builder_on_the_device(cuda):
    """``StepStateBuilder`` (one pinned staging buffer, one asynchronous copy per step) against the field-by-field
    builder and the block-manager oracle over a run of steps: fields, gathered rotary rows and the allocations
    of ``model.py:364-368``."""
    from oracle import rope_cpu as RO
    from morphserve_amd import BlockManager, StepStateBuilder, build_infer_state
    ct, st_ = RO.rotary_tables(128, 4096)
    cos, sin = torch.from_numpy(ct).to(cuda), torch.from_numpy(st_).to(cuda)
    bm = BlockManager("GPU", 2048, 64, 128, 16, device="cuda")
    ob = R.BlockManagerOracle("GPU", 2048, 64, 128, 16)
    b = StepStateBuilder(64, 8192, 8, 128, cos_cached=cos, sin_cached=sin)
    rng = np.random.default_rng(3)
    lens = {}
    for step in range(10):
        new = [int(x) for x in rng.permutation(64) if int(x) not in lens][:int(rng.integers(0, 4))]
        p = rng.integers(1, 400, size=len(new)).tolist()
        running = sorted(lens)
        d = [lens[s] + 1 for s in running]
        ids = new + running
        if not ids:
            continue
        s = b.build(p, ids, d, block_manager=bm)
        r = build_infer_state(p, ids, d, 8, 128)
        ob.allocate_blocks_for_seqs(np.asarray(ids), np.asarray(p + d))
        for f in ("seq_ids", "prefill_seq_start_locs", "prefill_seq_start_locs_with_end", "prefill_seq_lens",
                  "decoding_seq_lens"):
            assert torch.equal(getattr(s, f), getattr(r, f)), (step, f)
        assert (s.seq_block_size, s.num_seq_blocks, s.num_blocks_org) == (r.seq_block_size, r.num_seq_blocks, 2048)
        pos = np.concatenate([np.arange(x) for x in p] + [np.asarray(d, dtype=np.int64) - 1]).astype(np.int64)
        assert np.array_equal(bits(s.position_cos), ct[pos].view(np.uint16))
        assert np.array_equal(bits(s.position_sin), st_[pos].view(np.uint16))
        assert_state_equal(manager_state(bm), ob.snapshot(), f"step {step}")
        for sid, n in zip(new, p):
            lens[sid] = n
        for sid in running:
            lens[sid] += 1
