"""Sequence eviction end to end (KVSwapper = MorphServe/worker/model.py:468-534): both block
managers, the swap space and every pool byte against the CPU oracle, through the one-kernel
route (device id lists, pinned swap space) and through the reference's memcpy-run route."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from gpu_helpers import assert_state_equal, bits, manager_state, pool_bytes, pool_case
from morphserve_amd import KVSwapper, _capi

pytestmark = pytest.mark.gpu


def _oracle_swap(arena, lay, src_bm, dst_bm, ks, vs, seq_ids, is_swap_in):
    lens = src_bm.get_num_allocated_blocks(seq_ids) * 16
    src = src_bm.gather_allocated_blocks_and_free(seq_ids)
    dst = dst_bm.allocate_blocks_for_seqs(seq_ids, lens)
    R.swap_blocks(arena, lay, ks, vs, src, dst, is_swap_in)
    return len(src)


@pytest.mark.parametrize("cpu_tables", ["device", "host"])
@pytest.mark.parametrize("use_kernel,pinned", [(True, True), (False, True), (False, False)])
def test_swap_out_and_back_matches_the_oracle(cuda, use_kernel, pinned, cpu_tables):
    org, S, nseg = 16, 8, 3
    pool, ob, arena, lay = pool_case(cuda, 5, org, S, nseg, 0.5)
    n_cpu = 40
    sw = KVSwapper(pool, n_cpu, pinned=pinned, cpu_tables=cpu_tables)
    assert sw.k_swap.is_pinned() == pinned
    ocpu = R.BlockManagerOracle("CPU", n_cpu, 24, org + nseg * S, 16)
    ks = np.zeros(sw.k_swap.shape, dtype=np.float16)
    vs = np.zeros(sw.v_swap.shape, dtype=np.float16)
    live_rows = [s for s in range(24) if ob.num_seq_allocated_blocks[s] > 0]
    out1, out2 = live_rows[1::2][:3], live_rows[0:1]
    full = 2 * (org + nseg * S) * lay.block_elems

    def check(what):
        torch.cuda.synchronize()
        assert_state_equal(manager_state(sw.gpu_block_manager), ob.snapshot(), what + " gpu manager")
        assert_state_equal(manager_state(sw.cpu_block_manager), ocpu.snapshot(), what + " cpu manager")
        assert np.array_equal(bits(sw.k_swap), bits(ks)) and np.array_equal(bits(sw.v_swap), bits(vs)), what
        assert np.array_equal(pool_bytes(pool), arena[:full].view(np.uint16)), what

    n = sw.swap_out_seqs(out1, use_kernel=use_kernel)
    assert n == _oracle_swap(arena, lay, ob, ocpu, ks, vs, out1, False) > 0
    check("first swap-out")
    n = sw.swap_out_seqs(out2, use_kernel=use_kernel)
    assert n == _oracle_swap(arena, lay, ob, ocpu, ks, vs, out2, False)
    check("second swap-out")
    # scribble over the freed device blocks so that a swap-in has to restore them
    freed = np.nonzero(ob.is_block_free)[0]
    for b in freed:
        for which in ("k", "v"):
            o = lay.block_offset(which, int(b))
            arena[o:o + lay.block_elems] = np.float16(7.5)
    for b in freed:
        seg, local = (-1, b) if b < org else ((b - org) // S, (b - org) % S)
        (pool.k_cache if seg < 0 else pool.k_cache_new[seg])[local] = 7.5
        (pool.v_cache if seg < 0 else pool.v_cache_new[seg])[local] = 7.5
    # back in, in another order: blocks land on the lowest free ids, not where they were
    back = [out2[0]] + out1[::-1]
    n = sw.swap_in_seqs(back, use_kernel=use_kernel)
    assert n == _oracle_swap(arena, lay, ocpu, ob, ks, vs, back, True)
    check("swap-in")
    assert sw.block_swap == 2 * n and int(sw.cpu_block_manager.num_free_blocks) == n_cpu
    assert sw.swap_out_seqs([], use_kernel=use_kernel) == 0


def test_device_id_route_rejects_pageable_swap_space(cuda):
    import ctypes as C
    pool, ob, arena, lay = pool_case(cuda, 6, 8, 4, 1, 0.3)
    sw = KVSwapper(pool, 8, pinned=False)
    rows = [s for s in range(24) if ob.num_seq_allocated_blocks[s] > 0][:1]
    before = manager_state(sw.gpu_block_manager)
    with pytest.raises(ValueError, match="pinned"):
        sw.swap_out_seqs(rows, use_kernel=True)
    assert_state_equal(manager_state(sw.gpu_block_manager), before, "refused swap")
    ids = torch.zeros(1, dtype=torch.int64, device=cuda)
    desc = pool.descriptor()
    rc = _capi.lib().mkv_swap_blocks_device_ids(ids.data_ptr(), ids.data_ptr(), 1, 0, C.byref(desc),
                                                sw.k_swap.data_ptr(), sw.v_swap.data_ptr(), 8,
                                                _capi.current_stream())
    assert rc == _capi.MKV_EINVAL and b"pinned" in _capi.lib().mkv_last_error()
    torch.cuda.synchronize()
