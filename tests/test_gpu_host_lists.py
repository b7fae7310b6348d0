"""The block manager's calls with host lists: every size and check comes from the host copy of the rows'
counts, nothing is read back -- and the device state, the returned ids and the errors are those of the
plain calls and of the oracle."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from gpu_helpers import assert_state_equal, manager_state
from morphserve_amd import BlockManager, ElasticKVPool, KVSwapper, StepStateBuilder

pytestmark = pytest.mark.gpu


def _dev(x, cuda):
    return torch.tensor(list(x), dtype=torch.int32, device=cuda)


@pytest.mark.parametrize("seed", range(4))
def test_random_walk_with_host_lists_matches_the_oracle(cuda, seed):
    rng = np.random.default_rng(seed)
    N, S, M, B = 700, 24, 40, 16
    bm = BlockManager("GPU", N, S, M, B)
    ob = R.BlockManagerOracle("GPU", N, S, M, B)
    lens = np.zeros(S, dtype=np.int64)
    for step in range(120):
        op = rng.integers(4)
        rows = rng.choice(S, size=int(rng.integers(1, 9)), replace=False)
        with_lists = rng.random() < 0.7                       # the rest goes the plain way: the host copy must recover
        if op <= 1:
            tgt = np.minimum(lens[rows] + rng.integers(0, 90, size=len(rows)), M * B)
            need = int((-(-tgt // B) - -(-lens[rows] // B)).sum())
            kw = dict(seq_ids_host=rows.tolist(), target_lens_host=tgt.tolist()) if with_lists else {}
            if need > ob.num_free_blocks:
                with pytest.raises(RuntimeError, match="No enough free blocks"):
                    bm.allocate_blocks_for_seqs(_dev(rows, cuda), _dev(tgt, cuda), **kw)
                continue
            got = bm.allocate_blocks_for_seqs(_dev(rows, cuda), _dev(tgt, cuda), **kw)
            want = ob.allocate_blocks_for_seqs(rows, tgt)
            assert got.dtype == torch.int64 and got.cpu().tolist() == want.tolist()
            lens[rows] = tgt
        elif op == 2:
            kw = dict(seq_ids_host=rows.tolist()) if with_lists else {}
            bm.free_blocks_for_seqs(_dev(rows, cuda), **kw)
            ob.free_blocks_for_seqs(rows)
            lens[rows] = 0
        else:
            kw = dict(seq_ids_host=rows.tolist()) if with_lists else {}
            got = bm.gather_allocated_blocks_and_free(_dev(rows, cuda), **kw)
            want = ob.gather_allocated_blocks_and_free(rows)
            assert got.dtype == torch.int32 and got.cpu().tolist() == want.tolist()
            lens[rows] = 0
        assert int(bm.num_free_blocks) == ob.num_free_blocks, f"step {step}"
    assert_state_equal(manager_state(bm), ob.snapshot(), "after the walk")
    assert np.array_equal(bm._host_counts(), bm.num_seq_allocated_blocks.cpu().numpy())


def test_errors_come_from_the_host_before_anything_is_launched(cuda):
    bm = BlockManager("GPU", 8, 4, 4, 16)
    before = manager_state(bm)
    with pytest.raises(RuntimeError, match="No enough free blocks"):
        bm.allocate_blocks_for_seqs(_dev([0, 1, 2], cuda), _dev([64, 64, 64], cuda), seq_ids_host=[0, 1, 2],
                                    target_lens_host=[64, 64, 64])
    with pytest.raises(ValueError):
        bm.allocate_blocks_for_seqs(_dev([0], cuda), _dev([65], cuda), seq_ids_host=[0], target_lens_host=[65])
    with pytest.raises(ValueError):
        bm.allocate_blocks_for_seqs(_dev([4], cuda), _dev([1], cuda), seq_ids_host=[4], target_lens_host=[1])
    with pytest.raises(ValueError):
        bm.allocate_blocks_for_seqs(_dev([0], cuda), _dev([1], cuda), seq_ids_host=[0, 1], target_lens_host=[1, 1])
    bm.allocate_blocks_for_seqs(_dev([0], cuda), _dev([40], cuda), seq_ids_host=[0], target_lens_host=[40])
    mid = manager_state(bm)
    with pytest.raises(AssertionError, match="Logic error"):
        bm.allocate_blocks_for_seqs(_dev([0], cuda), _dev([10], cuda), seq_ids_host=[0], target_lens_host=[10])
    assert_state_equal(manager_state(bm), mid, "after a refused call")
    assert before["num_free_blocks"] == 8 and mid["num_free_blocks"] == 5
    assert bm.allocate_blocks_for_seqs(_dev([0], cuda), _dev([40], cuda), seq_ids_host=[0],
                                       target_lens_host=[40]).numel() == 0


def test_step_builder_and_swapper_leave_the_stream_alone(cuda):
    """With host lists at hand neither the step preparation nor an eviction waits for the GPU: a kernel that
    takes a while is queued first, and the calls return while it is still running."""
    pool = ElasticKVPool(256, 1, 2, 16, 128, max_seqs_in_block_table=16, max_blocks_per_seq=16)
    sw = KVSwapper(pool, 128)
    sb = StepStateBuilder(16, 4096, 2, 128)
    ob = R.BlockManagerOracle("GPU", 256, 16, 16, 16)
    st = sb.build([100, 30], [3, 5, 7], [17], block_manager=pool.block_manager)          # warm up every path once
    ob.allocate_blocks_for_seqs(np.array([3, 5, 7]), np.array([100, 30, 17]))
    torch.cuda.synchronize()
    big = torch.empty(1 << 28, dtype=torch.float32, device=cuda)
    marker = torch.cuda.Event()
    for _ in range(40):
        big.mul_(1.0001)                                       # a few tens of milliseconds of queued work
    marker.record()
    st = sb.build([], [3, 5, 7], [101, 31, 18], block_manager=pool.block_manager)
    ob.allocate_blocks_for_seqs(np.array([3, 5, 7]), np.array([101, 31, 18]))
    n_out = sw.swap_out_seqs([5])
    sw.free_seqs_resources([7])
    still_running = not marker.query()
    torch.cuda.synchronize()
    assert still_running, "a call waited for the stream"
    assert n_out == 2 and st.num_decoding_seqs == 3
    moved = ob.gather_allocated_blocks_and_free(np.array([5]))
    ob.free_blocks_for_seqs(np.array([7]))
    assert len(moved) == 2
    assert_state_equal(manager_state(pool.block_manager), ob.snapshot(), "after build + swap-out + free")
