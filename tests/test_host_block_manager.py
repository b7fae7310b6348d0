"""``HostBlockManager``: the "CPU" block manager of MorphServe/worker/model.py:214-227 with its tables in host
memory, against the oracle's restatement of MorphServe/worker/block_manager.py:64-129 -- same ids in the same
order, same table rows (stale entries after a free included), same counters, same errors.  CPU only."""
import numpy as np
import pytest

from oracle import ref_cpu as R
from morphserve_amd.worker.host_block_manager import HostBlockManager

NB, ROWS, PER_ROW, B = 96, 12, 16, 16


def _equal(m: HostBlockManager, o: R.BlockManagerOracle):
    assert np.array_equal(m.block_table.numpy(), o.block_table)
    assert np.array_equal(m.num_seq_allocated_blocks.numpy(), o.num_seq_allocated_blocks)
    assert np.array_equal(m.is_block_free.numpy(), o.is_block_free)
    assert int(m.num_free_blocks) == int(o.num_free_blocks)
    assert m.get_num_used_blocks() == o.get_num_used_blocks()


def test_hand_scenario():
    m, o = HostBlockManager("CPU", NB, ROWS, PER_ROW, B), R.BlockManagerOracle("CPU", NB, ROWS, PER_ROW, B)
    for mgr in (m, o):
        got = mgr.allocate_blocks_for_seqs([3, 1], [33, 16])           # 3 blocks, then 1: lowest ids, batch order
        assert list(got) == [0, 1, 2, 3]
    _equal(m, o)
    assert list(m.block_table[3, :3]) == [0, 1, 2] and int(m.block_table[1, 0]) == 3
    for mgr in (m, o):
        assert list(mgr.gather_allocated_blocks_and_free([1])) == [3]
        assert list(mgr.allocate_blocks_for_seqs([3, 5], [64, 17])) == [3, 4, 5]     # row 3 grows by one, row 5 takes two
    _equal(m, o)
    assert int(m.block_table[1, 0]) == 3                               # the freed row keeps its stale entry
    assert list(m.get_num_allocated_blocks([3, 5, 1])) == [4, 2, 0] == list(o.get_num_allocated_blocks([3, 5, 1]))
    for mgr in (m, o):
        mgr.free_blocks_for_seqs([3])
        assert list(mgr.allocate_blocks_for_seqs([7], [16 * 5])) == [0, 1, 2, 3, 6]  # holes first, ascending
    _equal(m, o)


def test_errors_leave_the_state_alone():
    m = HostBlockManager("CPU", 8, 4, 8, B)
    m.allocate_blocks_for_seqs([0], [16 * 6])
    before = (m.block_table.clone(), m.num_seq_allocated_blocks.clone(), m.is_block_free.clone(), int(m.num_free_blocks))
    with pytest.raises(RuntimeError, match="No enough free blocks available on CPU"):
        m.allocate_blocks_for_seqs([1], [16 * 3])
    with pytest.raises(ValueError):
        m.allocate_blocks_for_seqs([1], [16 * 9])                      # longer than a table row
    with pytest.raises(ValueError):
        m.allocate_blocks_for_seqs([4], [16])                          # no such row
    with pytest.raises(AssertionError):
        m.allocate_blocks_for_seqs([0], [16])                          # fewer blocks than the row already has
    after = (m.block_table, m.num_seq_allocated_blocks, m.is_block_free, int(m.num_free_blocks))
    for x, y in zip(before[:3], after[:3]):
        assert bool((x == y).all())
    assert before[3] == after[3]


def test_random_walk_equals_the_oracle():
    rng = np.random.default_rng(17)
    m, o = HostBlockManager("CPU", NB, ROWS, PER_ROW, B), R.BlockManagerOracle("CPU", NB, ROWS, PER_ROW, B)
    lens = np.zeros(ROWS, dtype=np.int64)
    for step in range(600):
        rows = rng.permutation(ROWS)[:rng.integers(1, 5)]
        kind = rng.random()
        if kind < 0.55:                                               # grow some rows
            target = np.minimum(lens[rows] + rng.integers(0, 40, size=len(rows)), PER_ROW * B)
            need = int((-(-target // B) - -(-lens[rows] // B)).sum())
            if need > int(o.num_free_blocks):
                with pytest.raises(RuntimeError):
                    m.allocate_blocks_for_seqs(rows.tolist(), target.tolist())
                continue
            a = m.allocate_blocks_for_seqs(rows.tolist(), target.tolist())
            b = o.allocate_blocks_for_seqs(rows, target)
            assert a.tolist() == b.tolist()
            lens[rows] = target
        elif kind < 0.8:
            a = m.gather_allocated_blocks_and_free(rows.tolist())
            b = o.gather_allocated_blocks_and_free(rows)
            assert a.tolist() == b.tolist()
            lens[rows] = 0
        else:
            m.free_blocks_for_seqs(rows.tolist())
            o.free_blocks_for_seqs(rows)
            lens[rows] = 0
        _equal(m, o)
