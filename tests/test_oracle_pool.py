"""Pins the CPU oracle's block manager, expand/shrink arithmetic, migration and
eviction through invariants and hand-written scenarios."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from helpers import make_case


def check_invariants(bm: R.BlockManagerOracle):
    live_rows = [bm.block_table[s, :bm.num_seq_allocated_blocks[s]] for s in range(bm.block_table.shape[0])]
    owned = np.concatenate(live_rows) if live_rows else np.empty(0, dtype=np.int32)
    assert len(np.unique(owned)) == len(owned), "a block is owned twice"
    assert bm.num_free_blocks + len(owned) == bm.num_blocks, "conservation"
    assert len(bm.is_block_free) == bm.num_blocks
    free = np.ones(bm.num_blocks, dtype=bool)
    free[owned] = False
    assert np.array_equal(free, bm.is_block_free), "free map != complement of live rows"
    assert int(bm.is_block_free.sum()) == bm.num_free_blocks


def test_hand_scenario():
    bm = R.BlockManagerOracle("GPU", 10, 4, 6, 16)
    new = bm.allocate_blocks_for_seqs([2, 0], [33, 16])      # seq 2 needs 3 blocks, seq 0 needs 1
    assert new.dtype == np.int64 and new.tolist() == [0, 1, 2, 3]
    assert bm.block_table[2, :3].tolist() == [0, 1, 2] and bm.block_table[0, 0] == 3
    assert bm.num_seq_allocated_blocks.tolist() == [1, 0, 3, 0]
    assert bm.num_free_blocks == 6 and bm.get_num_used_blocks() == 4
    # growth: seq 0 to 17 tokens needs a second block; seq 2 unchanged
    new = bm.allocate_blocks_for_seqs([0, 2], [17, 48])
    assert new.tolist() == [4] and bm.block_table[0, :2].tolist() == [3, 4]
    assert len(bm.allocate_blocks_for_seqs([0], [32])) == 0
    # free seq 2: its ids become free again, row keeps the stale ids, count is zero
    bm.free_blocks_for_seqs([2])
    assert bm.block_table[2, :3].tolist() == [0, 1, 2] and bm.num_seq_allocated_blocks[2] == 0
    assert bm.is_block_free[:5].tolist() == [True, True, True, False, False]
    # next allocation reuses the lowest ids first
    new = bm.allocate_blocks_for_seqs([1], [40])
    assert new.tolist() == [0, 1, 2]
    g = bm.gather_allocated_blocks_and_free([0, 1])
    assert g.dtype == np.int32 and g.tolist() == [3, 4, 0, 1, 2]
    assert bm.num_free_blocks == 10
    check_invariants(bm)
    with pytest.raises(RuntimeError, match="No enough free blocks"):
        bm.allocate_blocks_for_seqs([3], [16 * 11])
    check_invariants(bm)
    bm.allocate_blocks_for_seqs([3], [64])
    with pytest.raises(AssertionError):
        bm.allocate_blocks_for_seqs([3], [16])            # shrinking a sequence is a logic error


def test_random_walk_invariants():
    rng = np.random.default_rng(0)
    bm = R.BlockManagerOracle("GPU", 300, 32, 40, 16)
    lens = np.zeros(32, dtype=np.int64)
    for step in range(300):
        act = rng.integers(0, 4)
        if act <= 1:
            ids = rng.permutation(32)[:rng.integers(1, 6)]
            grow = rng.integers(0, 50, size=len(ids))
            tgt = np.minimum(lens[ids] + grow, 40 * 16)
            try:
                new = bm.allocate_blocks_for_seqs(ids, tgt)
                assert np.all(np.diff(new) > 0), "ids not ascending"
                lens[ids] = np.maximum(lens[ids], tgt)
            except RuntimeError:
                pass
        elif act == 2:
            ids = rng.permutation(32)[:rng.integers(1, 4)]
            bm.free_blocks_for_seqs(ids)
            lens[ids] = 0
        else:
            ids = rng.permutation(32)[:rng.integers(1, 4)]
            want = np.concatenate([bm.block_table[s, :bm.num_seq_allocated_blocks[s]] for s in ids])
            got = bm.gather_allocated_blocks_and_free(ids)
            assert np.array_equal(got, want)
            lens[ids] = 0
        check_invariants(bm)
        assert np.array_equal(bm.num_seq_allocated_blocks, (lens + 15) // 16)


def test_allocation_takes_lowest_free_ids():
    bm = R.BlockManagerOracle("GPU", 64, 8, 16, 16)
    bm.allocate_blocks_for_seqs(np.arange(8), np.full(8, 16 * 6))
    bm.free_blocks_for_seqs([1, 5])
    free_before = np.nonzero(bm.is_block_free)[0]
    new = bm.allocate_blocks_for_seqs([1], [16 * 9])
    assert np.array_equal(new, free_before[:9])


def test_carve_segment_known_answers():
    # block = 2 * L*Hkv*D*2 * B = 2*2*2*8*2*4 = 512 bytes; quant end 1000+300 -> aligned 1536
    k0, S, v0 = R.acquire_new_kvcache_arith(1000, 4000, 300, 2, 2, 4, 8)
    assert (k0, S, v0) == (1536, (4000 - 536) // 512, 1536 + 6 * 256)
    # already aligned end: no padding
    k0, S, v0 = R.acquire_new_kvcache_arith(4096, 8192, 1024, 2, 2, 4, 8)
    assert (k0, S, v0) == (5120, 14, 5120 + 14 * 256)
    # Llama-3-8B geometry: 2 MiB blocks out of a 436 MiB fp16 layer shrunk to 120 MiB
    MiB = 1 << 20
    k0, S, v0 = R.acquire_new_kvcache_arith(7 * MiB, 436 * MiB, 120 * MiB + 5, 32, 8, 16, 128)
    assert k0 == 127 * MiB + 256 and S == 157 and v0 == k0 + 157 * MiB
    with pytest.raises(RuntimeError, match="No space"):
        R.acquire_new_kvcache_arith(0, 1000, 600, 2, 2, 4, 8)


def test_expand_shrink_round_trip_and_refusal():
    bm = R.BlockManagerOracle("GPU", 8, 4, 8, 16)
    bm.allocate_blocks_for_seqs([0], [16 * 7])
    snap = bm.snapshot()
    bm.expand(4)
    bm.expand(4)
    assert bm.num_blocks == 16 and bm.num_free_blocks == 9 and bm.num_blocks_org == 8
    assert bm.shrink(4, 2) and bm.shrink(4, 1)
    after = bm.snapshot()
    for key in snap:
        assert np.array_equal(snap[key], after[key]), key
    bm.expand(4)
    bm.expand(4)
    bm.allocate_blocks_for_seqs([1], [16 * 6])          # ids 7, 8..12 -> touches both segments
    assert not bm.shrink(4, 2)                           # tail segment (ids 12..15) holds id 12
    assert bm.num_blocks == 16
    bm.free_blocks_for_seqs([1])
    assert bm.shrink(4, 2)
    check_invariants(bm)


# ---------------------------------------------------------------------------
# migration
# ---------------------------------------------------------------------------
def _logical(case, bm):
    out = {}
    for s in range(bm.block_table.shape[0]):
        a = int(bm.num_seq_allocated_blocks[s])
        if a:
            for layer in range(case.L):
                out[(s, layer)] = R.gather_kv(case.arena, case.lay, bm.block_table, s, a * case.B, layer)
    return out


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_migration_preserves_logical_content(seed):
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, 120, size=6)
    case = make_case(seed, 2, 2, 2, lens, num_blocks=96, D=8, fill="all")
    bm = R.BlockManagerOracle("GPU", 96, case.max_seqs, case.max_blocks_per_seq, 16)
    bm.block_table[:] = case.block_table
    bm.num_seq_allocated_blocks[:] = case.n_alloc
    bm.is_block_free[:] = case.is_free
    bm.num_free_blocks = int(case.is_free.sum())
    check_invariants(bm)
    before_logical = _logical(case, bm)
    before_arena = case.arena.copy()
    new_n = 48
    src, dst = R.apply_migration(case.arena, case.lay, bm, new_n)
    assert np.all(np.diff(src) > 0) and np.all(np.diff(dst) > 0)
    assert np.all(src >= new_n) and np.all(dst < new_n)
    assert np.array_equal(src, np.nonzero(~case.is_free[new_n:])[0] + new_n)
    assert np.array_equal(dst, np.nonzero(case.is_free[:new_n])[0][:len(src)])
    check_invariants(bm)
    assert bm.num_blocks == new_n
    for s in range(bm.block_table.shape[0]):
        assert np.all(bm.block_table[s, :bm.num_seq_allocated_blocks[s]] < new_n)
    after_logical = _logical(case, bm)
    for key, (ks, vs) in before_logical.items():
        assert np.array_equal(ks, after_logical[key][0]) and np.array_equal(vs, after_logical[key][1])
    # blocks that are not a destination are byte-identical
    n = case.lay.block_elems
    for which in ("k", "v"):
        for b in range(96):
            if b not in set(dst.tolist()):
                o = case.lay.block_offset(which, b)
                assert np.array_equal(case.arena[o:o + n], before_arena[o:o + n])


def test_migration_refused_when_it_does_not_fit():
    free = np.zeros(20, dtype=bool)
    free[[1, 3]] = True            # two free below the cut
    free[15] = True                # 9 live at or above 10
    with pytest.raises(RuntimeError, match="cannot shrink"):
        R.plan_migration(free, 10)
    src, dst = R.plan_migration(np.ones(20, dtype=bool), 10)
    assert len(src) == 0 and len(dst) == 0


# ---------------------------------------------------------------------------
# eviction
# ---------------------------------------------------------------------------
def test_coalesce_runs():
    assert R.coalesce_runs([4, 5, 6, 9, 10, 2], [0, 1, 2, 3, 4, 5]) == [(4, 0, 3), (9, 3, 2), (2, 5, 1)]
    # consecutive sources but a gap in targets splits the run
    assert R.coalesce_runs([1, 2, 3], [7, 8, 10]) == [(1, 7, 2), (3, 10, 1)]
    # a segment boundary splits the run even when ids are consecutive
    assert R.coalesce_runs([6, 7, 8], [0, 1, 2], src_seg=[-1, -1, 0]) == [(6, 0, 2), (8, 2, 1)]
    assert R.coalesce_runs([], []) == []


def test_swap_round_trip_is_identity():
    rng = np.random.default_rng(9)
    lens = np.array([40, 20])
    case = make_case(9, 2, 2, 2, lens, num_blocks=12, D=8, fill="all")
    n = case.lay.block_elems
    k_swap = np.zeros((6, 2, 2, 16, 8), dtype=np.float16)
    v_swap = np.zeros_like(k_swap)
    s = case.seq_ids[0]
    src = case.block_table[s, :3].astype(np.int64)
    want = R.gather_kv(case.arena, case.lay, case.block_table, s, 40, 1)
    R.swap_blocks(case.arena, case.lay, k_swap, v_swap, src, [2, 3, 4], is_swap_in=False)
    for j, b in enumerate(src):
        assert np.array_equal(k_swap[2 + j].reshape(-1), case.arena[case.lay.block_offset("k", b):][:n])
    # wipe the device copies, bring them back into different blocks
    for b in src:
        case.arena[case.lay.block_offset("k", b):][:n] = 0
        case.arena[case.lay.block_offset("v", b):][:n] = 0
    free = np.nonzero(case.is_free)[0][:3].astype(np.int64)
    R.swap_blocks(case.arena, case.lay, k_swap, v_swap, [2, 3, 4], free, is_swap_in=True)
    case.block_table[s, :3] = free
    got = R.gather_kv(case.arena, case.lay, case.block_table, s, 40, 1)
    assert np.array_equal(want[0], got[0]) and np.array_equal(want[1], got[1])
