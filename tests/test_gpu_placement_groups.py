"""``mkv_arena_pair_grow``: a pool whose K and V memory is chosen by memory group.

What the choice is worth is a measurement (``bench.py``); these tests pin what must hold whatever the
device reports: the pool is an ordinary pool (zeroed, data kept across growth, bit-exact appends and
attention), the report is consistent, every candidate chunk the call did not keep goes back to the
driver, and a second growth measures against the spares the first one kept.
"""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import assert_attn_close, rand_f16
from gpu_helpers import bits
from morphserve_amd import VmmKVPool, build_infer_state, decode_append_and_attend
from helpers import Cfg

pytestmark = pytest.mark.gpu

L, HKV, D, B = 32, 8, 128, 16            # 1 MiB per block and tensor
CHUNK = 512                              # blocks per chunk: 512 MiB, the smallest size measured at full probe length
GIB = 1 << 30


def _free_bytes():
    import gc
    gc.collect()                          # pools of earlier tests that are only garbage by now give their memory back here
    torch.cuda.synchronize()
    return torch.cuda.mem_get_info()[0]


def test_group_placed_pool_is_an_ordinary_pool(cuda):
    if _free_bytes() < 48 * GIB:
        pytest.skip("needs 48 GiB of free device memory")
    before = _free_bytes()
    pool = VmmKVPool(4 * CHUNK, 12 * CHUNK, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=64,
                     chunk_blocks=CHUNK, placement="groups", placement_budget_bytes=24 * GIB)
    try:
        g = pool.kv_placement["growths"]
        assert len(g) == 1
        first = g[0]
        assert first["k_chunks"] == 4 and first["v_chunks"] == 4
        assert 0 <= first["k_in_group"] <= 4 and 0 <= first["v_in_group"] <= 4
        assert first["groups_found"] in (1, 2, 3) and first["candidates"] >= 8 and first["probes"] > 0
        assert first["candidates"] * CHUNK * (1 << 20) <= 24 * GIB + 2 * CHUNK * (1 << 20)
        # the pool, its two spares and nothing else are held: every other candidate went back
        held = before - _free_bytes()
        slack = 512 << 20                 # torch's own allocator takes and returns memory on the side
        assert 8 * CHUNK * (1 << 20) - slack <= held <= (8 + 2) * CHUNK * (1 << 20) + slack
        # zero filled whatever the measurement wrote
        assert not pool.k_cache.any() and not pool.v_cache.any()
        # a decode step on it: cache bytes bit-exact, attention within tolerance
        rng = np.random.default_rng(5)
        n, Hq, layer = 4, 32, 7
        lens = np.array([17, 100, 1, 333])
        ids = torch.arange(n, dtype=torch.int32, device=cuda)
        got = pool.block_manager.allocate_blocks_for_seqs(ids, torch.from_numpy(lens.astype(np.int32)).to(cuda))
        ob = R.BlockManagerOracle("GPU", 4 * CHUNK, 8, 64, B)
        assert got.cpu().tolist() == ob.allocate_blocks_for_seqs(np.arange(n), lens).tolist()
        lay = R.plain_layout(4 * CHUNK, L, HKV, B, D)
        k_elems = 4 * CHUNK * L * HKV * B * D
        arena = np.zeros(2 * k_elems, dtype=np.float16)
        q, k, v = rand_f16(rng, n, Hq, D), rand_f16(rng, n, HKV, D), rand_f16(rng, n, HKV, D)
        # fill the live blocks with data first
        for t in (pool.k_cache, pool.v_cache):
            t[got.long()] = torch.from_numpy(rand_f16(rng, len(got), L, HKV, B, D)).to(cuda)
        torch.cuda.synchronize()
        arena[:k_elems] = pool.k_cache.cpu().numpy().reshape(-1)
        arena[k_elems:] = pool.v_cache.cpu().numpy().reshape(-1)
        R.append_decode(arena, lay, k, v, ob.block_table, np.arange(n), lens, layer)
        want = R.paged_attention(q, arena, lay, ob.block_table, np.arange(n), lens, D ** -0.5, layer)
        model = Cfg(num_layers=L, num_q_heads=Hq, num_kv_heads=HKV, head_dim=D)
        engine = Cfg(block_size=B, max_blocks_per_seq=64)
        st = build_infer_state([], list(range(n)), lens.tolist(), HKV, D)
        o = torch.full((n, Hq * D), float("nan"), dtype=torch.float16, device=cuda)
        decode_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), torch.from_numpy(q).to(cuda),
                                 pool.k_cache, pool.v_cache, [], [], pool.block_manager.block_table, model, engine,
                                 st, layer, o)
        torch.cuda.synchronize()
        assert np.array_equal(bits(pool.k_cache).reshape(-1), arena[:k_elems].view(np.uint16))
        assert np.array_equal(bits(pool.v_cache).reshape(-1), arena[k_elems:].view(np.uint16))
        assert_attn_close(o.cpu().numpy().reshape(n, Hq, D), want, "decode on a group-placed pool")
        # growth: data kept, new blocks zero, the spares of the first call are the references now
        keep_k = pool.k_cache[got.long()].clone()
        pool.expand(2 * CHUNK)
        assert len(pool.kv_placement["growths"]) == 2 and pool.kv_placement["growths"][1]["k_chunks"] == 2
        assert pool.num_blocks == 6 * CHUNK and torch.equal(pool.k_cache[got.long()], keep_k)
        assert not pool.k_cache[4 * CHUNK:].any() and not pool.v_cache[4 * CHUNK:].any()
        assert bool(pool.block_manager.is_block_free[4 * CHUNK:].all())
        # shrink: the tail goes back to the driver
        pool.shrink_to(4 * CHUNK)
        held = before - _free_bytes()
        assert held <= (8 + 2) * CHUNK * (1 << 20) + (512 << 20)
    finally:
        pool.close()
    assert before - _free_bytes() <= (512 << 20)          # spares included: everything returned


def test_plain_placement_and_small_chunks_take_the_drivers_order(cuda):
    pool = VmmKVPool(64, 128, 2, 2, B, D, max_seqs_in_block_table=4, max_blocks_per_seq=8, chunk_blocks=16,
                     placement="groups")
    try:
        assert pool.kv_placement["growths"][0]["groups_found"] == 0      # 256 KiB chunks cannot be measured
        assert not pool.k_cache.any()
    finally:
        pool.close()
    pool = VmmKVPool(64, 128, 2, 2, B, D, max_seqs_in_block_table=4, max_blocks_per_seq=8, chunk_blocks=16,
                     placement="plain")
    try:
        assert pool.kv_placement["growths"] == []
    finally:
        pool.close()
    with pytest.raises(ValueError):
        VmmKVPool(64, 128, 2, 2, B, D, max_seqs_in_block_table=4, max_blocks_per_seq=8, chunk_blocks=16,
                  placement="nearest")


def test_a_pool_that_does_not_fit_is_refused_and_leaves_nothing_behind(cuda):
    """Device nearly full: creation raises MemoryError (MKV_ENOSPC from the library), every candidate chunk
    it had created is back with the driver, and the same pool can be created once there is room."""
    from morphserve_amd.vmm_pool import _Arena
    free = _free_bytes()
    if free < 40 * GIB:
        pytest.skip("needs 40 GiB of free device memory")
    hog_bytes = (free - 12 * GIB) // GIB * GIB              # leave about 12 GiB
    hog = _Arena(hog_bytes, GIB)
    try:
        hog.resize(hog_bytes)
        before = _free_bytes()
        assert before < 14 * GIB
        with pytest.raises(MemoryError):                    # 2 x 8 GiB in 512 MiB chunks: more than what is left
            VmmKVPool(16 * CHUNK, 16 * CHUNK, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=64,
                      chunk_blocks=CHUNK, placement="groups")
        assert abs(before - _free_bytes()) <= (64 << 20)
    finally:
        hog.close()
    pool = VmmKVPool(16 * CHUNK, 16 * CHUNK, L, HKV, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=64,
                     chunk_blocks=CHUNK, placement="groups")
    try:
        assert pool.kv_placement["growths"][0]["k_chunks"] == 16 and not pool.v_cache[-1].any()
    finally:
        pool.close()
