"""Regression tests for the table-row limits and the failure paths: a block-table row that is exactly
full, appends and chunks that would run past a row, a row count that would overflow, and errors that
must leave the device state as it was."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import assert_attn_close, make_case, rand_f16
from gpu_helpers import assert_state_equal, bits, configs, manager_state, to_gpu
from morphserve_amd import (BlockManager, ElasticKVPool, _capi, build_infer_state, chunked_prefill_attention,
                            store_kvcache)
from morphserve_amd.elastic_pool import PoolTooFullError

pytestmark = pytest.mark.gpu


def _i32(x, dev):
    return torch.tensor(np.asarray(x, dtype=np.int32), dtype=torch.int32, device=dev)


def _reseat(case, new_ids):
    """Move the case's sequences to the given table rows."""
    table = np.full_like(case.block_table, -1)
    n_alloc = np.zeros_like(case.n_alloc)
    for old, new in zip(case.seq_ids.tolist(), new_ids):
        table[new] = case.block_table[old]
        n_alloc[new] = case.n_alloc[old]
    case.block_table[:] = table
    case.n_alloc[:] = n_alloc
    case.seq_ids[:] = new_ids


def test_prefill_append_and_chunk_on_a_full_table_row(cuda):
    """Rows of exactly max_blocks_per_seq blocks: the append and the chunked attention use the whole row
    and nothing of the next one (the sequence with the highest slot number has no next row at all)."""
    mbps, Hq, Hkv = 8, 4, 2
    lens = np.array([mbps * 16, mbps * 16 - 5, 40])
    case = make_case(31, 2, Hq, Hkv, lens, num_blocks=32, max_seqs=4, max_blocks_per_seq=mbps, fill="all")
    _reseat(case, [3, 0, 2])                         # the full row is the table's last one
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    rng = np.random.default_rng(31)
    T = int(lens.sum())
    q, k, v = rand_f16(rng, T, Hq, 128), rand_f16(rng, T, Hkv, 128), rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - lens
    st = build_infer_state(lens.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt, model, engine, st, 1)
    R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, 1)
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    prefix = lens // 2
    l2 = lens - prefix
    s2 = np.cumsum(l2) - l2
    q2 = np.concatenate([q[starts[b] + prefix[b]:starts[b] + lens[b]] for b in range(3)])
    want = R.chunked_prefill_attention(q2, case.arena, case.lay, case.block_table, case.seq_ids, s2, l2, prefix,
                                       128 ** -0.5, 1)
    o = torch.full((int(l2.sum()), Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    chunked_prefill_attention(torch.from_numpy(q2).to(cuda), kc, vc, [], [], bt, model, engine,
                              build_infer_state(l2.tolist(), case.seq_ids.tolist(), [], Hkv, 128), 1, o,
                              prefix_lens=_i32(prefix, cuda))
    torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy(), want, "chunk over a full table row")


def test_prefill_append_refuses_lengths_beyond_a_table_row(cuda):
    """A prompt longer than a row can describe is refused on the host; nothing is written."""
    mbps, Hkv = 4, 2
    case = make_case(32, 1, 2, Hkv, [64, 64], num_blocks=16, max_seqs=2, max_blocks_per_seq=mbps, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    lens = [mbps * 16 + 1, 10]                       # the first prompt needs a fifth block
    T = sum(lens)
    rng = np.random.default_rng(32)
    k, v = rand_f16(rng, T, Hkv, 128), rand_f16(rng, T, Hkv, 128)
    st = build_infer_state(lens, case.seq_ids.tolist(), [], Hkv, 128)
    with pytest.raises(_capi.MorphKVError, match="block-table row"):
        store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt, model, engine,
                      st, 0)
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))


def test_chunk_reaching_past_the_table_row_stays_inside_it(cuda):
    """prefix + chunk beyond max_blocks_per_seq * 16 (a caller's mistake the host cannot see: prefix_lens is a
    device array): keys past the row read as zeros instead of the next sequence's blocks, so the rows whose
    keys all lie inside the table row still get their exact result."""
    mbps, Hq, Hkv = 4, 4, 2
    lens = np.array([mbps * 16, mbps * 16])
    case = make_case(33, 1, Hq, Hkv, lens, num_blocks=16, max_seqs=2, max_blocks_per_seq=mbps, fill="all")
    _reseat(case, [0, 1])
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    rng = np.random.default_rng(33)
    chunk = 24                                        # positions 56 .. 79 of sequence 0: the last 16 lie past the row
    q = rand_f16(rng, chunk, Hq, 128)
    o = torch.full((chunk, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    chunked_prefill_attention(torch.from_numpy(q).to(cuda), kc, vc, [], [], bt, model, engine,
                              build_infer_state([chunk], [0], [], Hkv, 128), 0, o, prefix_lens=_i32([56], cuda))
    torch.cuda.synchronize()
    want = R.chunked_prefill_attention(q[:8], case.arena, case.lay, case.block_table, np.array([0]), np.array([0]),
                                       np.array([8]), np.array([56]), 128 ** -0.5, 0)
    assert_attn_close(o[:8].cpu().numpy(), want, "rows inside the table row")
    assert torch.isfinite(o.float()).all()


def test_row_count_never_exceeds_the_row(cuda):
    """set_block_table_and_num_seq_alloc_blocks with more candidates than the row has room for: the count
    stops at the row's capacity, and a later free releases only this row's blocks."""
    from morphserve_amd.worker.kernels import block_mgmt
    bm = BlockManager("GPU", 32, 3, 4, 16)
    bm.allocate_blocks_for_seqs(_i32([0, 1], cuda), _i32([48, 64], cuda))          # 3 + 4 blocks: ids 0..6
    cand = torch.arange(10, 13, dtype=torch.int64, device=cuda)
    bm.is_block_free[10:13] = False
    block_mgmt.set_block_table_and_num_seq_alloc_blocks(bm.num_seq_allocated_blocks, bm.block_table, cand,
                                                        _i32([0], cuda), _i32([3], cuda))
    torch.cuda.synchronize()
    assert bm.num_seq_allocated_blocks.cpu().tolist() == [4, 4, 0], "count clamped to the row"
    assert bm.block_table[0].cpu().tolist() == [0, 1, 2, 10] and bm.block_table[1].cpu().tolist() == [3, 4, 5, 6]
    bm.num_seq_allocated_blocks[0] = 7                                              # a corrupted count
    bm.free_blocks_for_seqs(_i32([0], cuda))
    free = bm.is_block_free.cpu().numpy()
    assert free[[0, 1, 2, 10]].all() and not free[[3, 4, 5, 6]].any(), "the neighbour row's blocks stay allocated"


def test_failed_allocation_leaves_the_device_state_alone(cuda):
    """The host's free counter is lower than the map's (e.g. blocks reserved by the caller): the request is
    refused BEFORE anything is taken from the map or written to the table."""
    bm = BlockManager("GPU", 16, 4, 8, 16)
    bm.allocate_blocks_for_seqs(_i32([0], cuda), _i32([32], cuda))
    bm.num_free_blocks = 3
    before = manager_state(bm)
    with pytest.raises(RuntimeError, match="No enough free blocks"):
        bm.allocate_blocks_for_seqs(_i32([1], cuda), _i32([64], cuda))             # 4 > 3 by the host's count
    assert_state_equal(manager_state(bm), before, "refused allocation")
    got = bm.allocate_blocks_for_seqs(_i32([1], cuda), _i32([48], cuda))
    assert got.cpu().tolist() == [2, 3, 4] and int(bm.num_free_blocks) == 0


def test_shrink_that_does_not_fit_is_a_refusal_and_a_failed_launch_is_not(cuda, monkeypatch):
    from morphserve_amd.server import PoolEngine
    from morphserve_amd.server.memory_utils import org2quant_and_update_kvcache, quant2org_and_update_kvcache
    from helpers import Cfg
    pool = ElasticKVPool(4, 1, 1, 16, 128, max_seqs_in_block_table=4, max_blocks_per_seq=8)
    engine = PoolEngine(pool, Cfg(block_size=16), num_layers=2, seg_blocks=4, migrate=True)
    org2quant_and_update_kvcache(engine)
    pool.block_manager.allocate_blocks_for_seqs(_i32([0], cuda), _i32([16 * 6], cuda))    # 6 live of 8
    before = manager_state(pool.block_manager)
    with pytest.raises(PoolTooFullError):
        pool.shrink_to(4)
    assert quant2org_and_update_kvcache(engine) is False                            # refusal, state untouched
    assert_state_equal(manager_state(pool.block_manager), before, "refused shrink")
    assert pool.num_blocks == 8 and len(pool.k_cache_new) == 1

    def broken(*a, **k):
        raise _capi.MorphKVError(_capi.MKV_EHIP, "injected launch failure")
    monkeypatch.setattr(pool, "_relocate_live_blocks", broken)
    with pytest.raises(_capi.MorphKVError, match="injected"):
        quant2org_and_update_kvcache(engine)


@pytest.mark.parametrize("num_blocks,lo_off", [(98304, 0), (70001, 3), (1000, 13), (37, 5)])
def test_map_scans_with_unaligned_ranges(cuda, num_blocks, lo_off):
    """The free-map scans read 16 bytes per thread; ranges that start or end off a 16-byte boundary, maps
    that are views at odd offsets, and non-bool byte values must give the counts and ids of a plain scan."""
    rng = np.random.default_rng(num_blocks)
    lib = _capi.lib()
    backing = torch.zeros(num_blocks + 32, dtype=torch.uint8, device=cuda)
    free = backing[lo_off:lo_off + num_blocks]                                      # misaligned view
    host = (rng.random(num_blocks) < 0.4)
    free.copy_(torch.from_numpy(host.astype(np.uint8)))
    res = torch.zeros(4, dtype=torch.int64, device=cuda)
    for lo, hi in ((0, num_blocks), (num_blocks // 3 + 1, num_blocks - 2), (7, 9), (num_blocks - 1, num_blocks)):
        _capi.check(lib.mkv_bm_count_live(free.data_ptr(), lo, hi, res.data_ptr(), _capi.current_stream()))
        assert int(res[0].item()) == int((~host[lo:hi]).sum()), f"live count of [{lo}, {hi})"
    want = np.nonzero(host)[0]
    n = min(len(want), 1 + len(want) // 2)
    ids = torch.empty(max(n, 1), dtype=torch.int64, device=cuda)
    _capi.check(lib.mkv_bm_take_first_free(free.data_ptr(), num_blocks, n, ids.data_ptr(), res.data_ptr(),
                                           _capi.current_stream()))
    assert res[:2].cpu().tolist() == [n, 0]
    assert ids[:n].cpu().tolist() == want[:n].tolist()
    host[want[:n]] = False
    assert np.array_equal(free.cpu().numpy() != 0, host)
    assert (backing[:lo_off] == 0).all() and (backing[lo_off + num_blocks:] == 0).all(), "bytes around the map"
