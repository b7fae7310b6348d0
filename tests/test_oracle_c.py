"""The C restatement against the independent numpy restatement."""
import numpy as np

from oracle import c_oracle as CO
from oracle import ref_cpu as R
from helpers import make_case, rand_f16


def _i32(x):
    return np.ascontiguousarray(x, dtype=np.int32)


def test_c_append_equals_numpy():
    rng = np.random.default_rng(0)
    p_lens, d_lens = np.array([33, 7, 64]), np.array([5, 17, 100])
    lens = np.concatenate([p_lens, d_lens])
    a = make_case(0, 3, 4, 4, lens, num_blocks=40, D=32, fill="all")
    b_arena = a.arena.copy()
    T = int(p_lens.sum())
    k = rand_f16(rng, T + 3, 4, 32)
    v = rand_f16(rng, T + 3, 4, 32)
    starts = np.cumsum(p_lens) - p_lens
    R.store_kvcache(a.arena, a.lay, k, v, a.block_table, a.seq_ids, 3, T, starts, p_lens, d_lens, 2)
    cl = CO.CLayout(a.lay)
    CO.append_prefill(b_arena, cl, k, v, a.block_table, _i32(a.seq_ids[:3]), _i32(starts), _i32(p_lens), 2)
    CO.append_decode(b_arena, cl, k[T:], v[T:], a.block_table, _i32(a.seq_ids[3:]), _i32(d_lens), 2)
    assert np.array_equal(a.arena.view(np.uint16), b_arena.view(np.uint16))


def test_c_attention_equals_numpy_fp64():
    rng = np.random.default_rng(1)
    lens = np.array([1, 16, 17, 300, 1025])
    case = make_case(1, 2, 8, 2, lens, num_blocks=100, D=128, fill="all")
    q = rand_f16(rng, len(lens), 8, 128)
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                             128 ** -0.5, 1, out_dtype=np.float64, math="np64")
    got = CO.paged_attention(q, case.arena, CO.CLayout(case.lay), case.block_table,
                             _i32(case.seq_ids), _i32(lens), 128 ** -0.5, 1)
    assert np.abs(got.astype(np.float64) - want).max() < 1.5e-3      # fp16 output rounding
    want16 = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                               128 ** -0.5, 1)
    # two fp32 evaluations of the same math: equal up to one fp16 ulp of the output
    assert np.abs(got.astype(np.float64) - want16.astype(np.float64)).max() <= 2 ** -9


def test_c_take_first_free_and_migrate_equal_numpy():
    rng = np.random.default_rng(2)
    free = rng.random(500) < 0.4
    ob = R.BlockManagerOracle("GPU", 500, 2, 2, 16)
    ob.is_block_free[:] = free
    ob.num_free_blocks = int(free.sum())
    u8 = free.astype(np.uint8)
    want = ob._allocate_blocks(77)
    got, found = CO.take_first_free(u8, 77)
    assert found == 77 and np.array_equal(got, want) and np.array_equal(u8.astype(bool), ob.is_block_free)
    _, found = CO.take_first_free(u8, 10_000)
    assert found == int(u8.sum()) and np.array_equal(u8.astype(bool), ob.is_block_free)

    lens = rng.integers(1, 120, size=6)
    case = make_case(3, 2, 2, 2, lens, num_blocks=96, D=8, fill="all")
    c_arena = case.arena.copy()
    bm = R.BlockManagerOracle("GPU", 96, case.max_seqs, case.max_blocks_per_seq, 16)
    bm.block_table[:] = case.block_table
    bm.num_seq_allocated_blocks[:] = case.n_alloc
    bm.is_block_free[:] = case.is_free
    bm.num_free_blocks = int(case.is_free.sum())
    src, dst = R.apply_migration(case.arena, case.lay, bm, 48)
    CO.migrate(c_arena, CO.CLayout(case.lay), src, dst)
    assert np.array_equal(c_arena.view(np.uint16), case.arena.view(np.uint16))
