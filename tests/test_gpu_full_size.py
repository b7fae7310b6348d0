"""GPU checks at the full sizes of the benchmark configurations, through
properties that do not need a CPU pass over the whole pool: results must not
depend on where blocks physically live, appended rows must read back, migration
must preserve every sequence's logical KV."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, to_gpu
from morphserve_amd import (ElasticKVPool, build_infer_state, decode_append_and_attend, paged_attention,
                            prefill_attention, store_kvcache)

pytestmark = pytest.mark.gpu


def _mem_gib(dev):
    import gc
    gc.collect()
    torch.cuda.empty_cache()          # memory cached by earlier tests counts as free
    free, _ = torch.cuda.mem_get_info(dev)
    return free / 2 ** 30


def test_config2_full_pool_placement_invariance(cuda):
    """Llama-3-8B decode at the full 65 536-block (128 GiB) pool: the fused step on
    three layers gives bit-identical outputs to the same logical KV held in a
    compact pool, and the appended rows read back from the big pool."""
    if _mem_gib(cuda) < 150:
        pytest.skip("needs ~140 GiB of free HBM")
    L, HQ, HKV, D, B, N, NB = 32, 32, 8, 128, 16, 64, 65536
    rng = np.random.default_rng(22)
    lens = rng.integers(1024, 1537, size=N).astype(np.int32)
    nblk = (lens.astype(np.int64) + B - 1) // B
    total = int(nblk.sum())
    perm = rng.permutation(NB)[:total]
    seq_ids = rng.permutation(256)[:N].astype(np.int32)
    big_table = np.full((256, 128), -1, dtype=np.int32)
    small_table = np.full((256, 128), -1, dtype=np.int32)
    pos = 0
    for i in range(N):
        big_table[seq_ids[i], :nblk[i]] = perm[pos:pos + nblk[i]]
        small_table[seq_ids[i], :nblk[i]] = np.arange(pos, pos + nblk[i])
        pos += nblk[i]
    layers = [0, 17, 31]
    gen = torch.Generator(device=cuda)
    gen.manual_seed(5)
    # compact pool: only the three layers under test, addressed as layers 0..2
    ks = torch.randn((total, 3, HKV, B, D), dtype=torch.float16, device=cuda, generator=gen)
    vs = torch.randn((total, 3, HKV, B, D), dtype=torch.float16, device=cuda, generator=gen)
    kb = torch.zeros((NB, L, HKV, B, D), dtype=torch.float16, device=cuda)
    vb = torch.zeros((NB, L, HKV, B, D), dtype=torch.float16, device=cuda)
    idx = torch.from_numpy(perm).to(cuda)
    for j, layer in enumerate(layers):
        kb[idx, layer] = ks[:, j]
        vb[idx, layer] = vs[:, j]
    q = torch.randn((N, HQ, D), dtype=torch.float16, device=cuda, generator=gen)
    kn = torch.randn((N, HKV, D), dtype=torch.float16, device=cuda, generator=gen)
    vn = torch.randn((N, HKV, D), dtype=torch.float16, device=cuda, generator=gen)
    st = build_infer_state([], seq_ids.tolist(), lens.tolist(), HKV, D)
    engine = Cfg(block_size=B, max_blocks_per_seq=128)
    big_cfg = Cfg(num_layers=L, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    small_cfg = Cfg(num_layers=3, num_q_heads=HQ, num_kv_heads=HKV, head_dim=D)
    bt_big = torch.from_numpy(big_table).to(cuda)
    bt_small = torch.from_numpy(small_table).to(cuda)
    for j, layer in enumerate(layers):
        o_big = torch.empty((N, HQ * D), dtype=torch.float16, device=cuda)
        o_small = torch.empty_like(o_big)
        o_two = torch.empty_like(o_big)
        decode_append_and_attend(kn, vn, q, kb, vb, [], [], bt_big, big_cfg, engine, st, layer, o_big)
        decode_append_and_attend(kn, vn, q, ks, vs, [], [], bt_small, small_cfg, engine, st, j, o_small)
        paged_attention(q, kb, vb, [], [], bt_big, big_cfg, engine, st, layer, o_two)   # cache now holds the token
        torch.cuda.synchronize()
        assert torch.equal(o_big, o_small), f"layer {layer}: output depends on block placement"
        assert torch.equal(o_big, o_two), f"layer {layer}: fused and two-call results differ"
        assert bool(torch.isfinite(o_big).all())
        # the appended rows read back from the big pool
        last_blk = torch.from_numpy(big_table[seq_ids, (lens - 1) // B]).to(cuda).long()
        off = torch.from_numpy((lens - 1) % B).to(cuda).long()
        assert torch.equal(kb[last_blk, layer, :, off, :], kn) and torch.equal(vb[last_blk, layer, :, off, :], vn)
    # a spot check against the CPU oracle on the compact pool (one layer, four sequences)
    sel = np.array([0, 7, 31, 63])
    arena = np.concatenate([ks[:, 0].reshape(-1).cpu().numpy(), vs[:, 0].reshape(-1).cpu().numpy()])
    lay = R.plain_layout(total, 1, HKV, B, D)
    want = R.paged_attention(q[sel].cpu().numpy(), arena, lay, small_table, seq_ids[sel], lens[sel], D ** -0.5, 0)
    o_chk = torch.empty((N, HQ * D), dtype=torch.float16, device=cuda)
    paged_attention(q, ks, vs, [], [], bt_small, small_cfg, engine, st, 0, o_chk)
    torch.cuda.synchronize()
    assert_attn_close(o_chk[torch.from_numpy(sel).to(cuda)].cpu().numpy().reshape(4, HQ, D), want, "config 2 spot check")


def test_config3_full_size_resize_preserves_logical_kv(cuda):
    """2 MiB blocks: 32 768 -> 98 304 blocks, 24 576 live blocks scattered, shrink
    to 40 960: plan equals the CPU plan, every live id ends below the cut, and a
    checksum of every sequence's blocks (in logical order) is unchanged."""
    if _mem_gib(cuda) < 215:
        pytest.skip("needs ~200 GiB of free HBM")
    L, HKV, D, B = 32, 8, 128, 16
    ORG, SEG, NSEG, KEEP = 32768, 8192, 8, 1
    pool = ElasticKVPool(ORG, L, HKV, B, D, max_seqs_in_block_table=512, max_blocks_per_seq=256,
                         zero_init=False)
    for _ in range(NSEG):
        pool.expand(SEG)
    total, new_n = ORG + NSEG * SEG, ORG + KEEP * SEG
    assert float(pool.k_cache_new[3][100, 5, 2].abs().sum()) == 0.0           # expand zero-fills
    rng = np.random.default_rng(33)
    per_seq, n_seq = 192, 128
    live = rng.permutation(total)[:per_seq * n_seq]
    table = np.full((512, 256), -1, dtype=np.int32)
    n_alloc = np.zeros(512, dtype=np.int32)
    rows = rng.permutation(512)[:n_seq]
    for j, s in enumerate(rows):
        table[s, :per_seq] = live[j * per_seq:(j + 1) * per_seq]
        n_alloc[s] = per_seq
    free = np.ones(total, dtype=bool)
    free[live] = False
    bm = pool.block_manager
    bm.block_table.copy_(torch.from_numpy(table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(n_alloc))
    bm.is_block_free.copy_(torch.from_numpy(free))
    bm.num_free_blocks = int(free.sum())

    def block_view(ids):
        """(K, V) int16 views of the given global block ids, gathered segment-wise."""
        ids = torch.as_tensor(ids, device=cuda).long()
        outk = torch.empty((len(ids), L * HKV * B * D), dtype=torch.int16, device=cuda)
        outv = torch.empty_like(outk)
        seg = torch.where(ids < ORG, torch.full_like(ids, -1), (ids - ORG) // SEG)
        for sgi in range(-1, len(pool.k_cache_new)):
            m = seg == sgi
            if not bool(m.any()):
                continue
            kt = pool.k_cache if sgi < 0 else pool.k_cache_new[sgi]
            vt = pool.v_cache if sgi < 0 else pool.v_cache_new[sgi]
            local = ids[m] if sgi < 0 else ids[m] - ORG - sgi * SEG
            outk[m] = kt.view(torch.int16).reshape(kt.shape[0], -1)[local]
            outv[m] = vt.view(torch.int16).reshape(vt.shape[0], -1)[local]
        return outk, outv

    # distinct content per live block: a per-block random 64-bit pattern written into the whole block
    gen = torch.Generator(device=cuda)
    gen.manual_seed(3)
    live_t = torch.from_numpy(live).to(cuda)
    weights = torch.arange(1, 4097, dtype=torch.int64, device=cuda)

    def checksums(ids):
        out = []
        for c0 in range(0, len(ids), 512):
            kk, vv = block_view(ids[c0:c0 + 512])
            sk = (kk.view(len(kk), -1, 4096).to(torch.int64) * weights).sum(dim=(1, 2))
            sv = (vv.view(len(vv), -1, 4096).to(torch.int64) * weights).sum(dim=(1, 2))
            out.append(sk * 31 + sv)
        return torch.cat(out)

    for c0 in range(0, len(live), 512):
        ids = live_t[c0:c0 + 512].long()
        n = len(ids)
        pat = torch.randint(-30000, 30000, (n, L * HKV * B * D), dtype=torch.int16, device=cuda, generator=gen)
        seg = torch.where(ids < ORG, torch.full_like(ids, -1), (ids - ORG) // SEG)
        for sgi in range(-1, NSEG):
            m = seg == sgi
            if not bool(m.any()):
                continue
            kt = pool.k_cache if sgi < 0 else pool.k_cache_new[sgi]
            vt = pool.v_cache if sgi < 0 else pool.v_cache_new[sgi]
            local = ids[m] if sgi < 0 else ids[m] - ORG - sgi * SEG
            kt.view(torch.int16).reshape(kt.shape[0], -1)[local] = pat[m]
            vt.view(torch.int16).reshape(vt.shape[0], -1)[local] = pat[m].flip(1)
    before = checksums(live)                       # logical order: sequence-major, block-minor
    want_src, want_dst = R.plan_migration(free, new_n)
    src, dst = pool.shrink_to(new_n)
    torch.cuda.synchronize()
    assert src.cpu().tolist() == want_src.tolist() and dst.cpu().tolist() == want_dst.tolist()
    assert pool.num_blocks == new_n and len(pool.k_cache_new) == KEEP
    new_table = bm.block_table.cpu().numpy()
    now = np.concatenate([new_table[s, :per_seq] for s in rows])
    assert now.max() < new_n and len(np.unique(now)) == len(now)
    remap = dict(zip(want_src.tolist(), want_dst.tolist()))
    assert np.array_equal(now, np.array([remap.get(int(b), int(b)) for b in live]))
    assert torch.equal(checksums(now), before), "a sequence's KV changed during migration"
    is_free = bm.is_block_free.cpu().numpy()
    assert len(is_free) == new_n and int(is_free.sum()) == bm.num_free_blocks == new_n - len(live)
    assert not is_free[now].any()


def test_config3_full_size_resize_on_the_virtual_memory_pool(cuda):
    """The same resize on the pool the benchmark measures: one tensor per K and V over virtual memory,
    8 GiB chunks placed by memory group, 32 768 -> 98 304 blocks in eight growths, shrink to 40 960 with the
    plan made by the multi-workgroup kernels.  Plan, table, free map and counters equal the CPU plan's, every
    sequence's blocks carry the same bytes afterwards, and the memory above the cut is back with the driver."""
    if _mem_gib(cuda) < 215:
        pytest.skip("needs ~200 GiB of free HBM")
    from morphserve_amd import VmmKVPool
    L, HKV, D, B = 32, 8, 128, 16
    ORG, SEG, NSEG, KEEP = 32768, 8192, 8, 1
    total, new_n = ORG + NSEG * SEG, ORG + KEEP * SEG
    free_at_start = torch.cuda.mem_get_info(cuda)[0]
    pool = VmmKVPool(ORG, total, L, HKV, B, D, max_seqs_in_block_table=512, max_blocks_per_seq=256,
                     chunk_blocks=SEG, placement="groups")
    try:
        for _ in range(NSEG):
            pool.expand(SEG)
        growths = pool.kv_placement["growths"]
        assert len(growths) == 1 + NSEG and growths[0]["k_chunks"] == ORG // SEG
        assert pool.num_blocks == total and pool.k_cache.shape[0] == total
        assert float(pool.k_cache[ORG + 3 * SEG + 100, 5, 2].abs().sum()) == 0.0          # growth zero-fills
        rng = np.random.default_rng(33)
        per_seq, n_seq = 192, 128
        live = rng.permutation(total)[:per_seq * n_seq]
        table = np.full((512, 256), -1, dtype=np.int32)
        n_alloc = np.zeros(512, dtype=np.int32)
        rows = rng.permutation(512)[:n_seq]
        for j, s in enumerate(rows):
            table[s, :per_seq] = live[j * per_seq:(j + 1) * per_seq]
            n_alloc[s] = per_seq
        free = np.ones(total, dtype=bool)
        free[live] = False
        bm = pool.block_manager
        bm.block_table.copy_(torch.from_numpy(table))
        bm.num_seq_allocated_blocks.copy_(torch.from_numpy(n_alloc))
        bm.is_block_free.copy_(torch.from_numpy(free))
        bm.num_free_blocks = int(free.sum())
        bm.invalidate_host_counts()

        gen = torch.Generator(device=cuda)
        gen.manual_seed(3)
        weights = torch.arange(1, 4097, dtype=torch.int64, device=cuda)
        k16 = pool.k_cache.view(torch.int16).reshape(total, -1)
        v16 = pool.v_cache.view(torch.int16).reshape(total, -1)

        def checksums(ids, kk16, vv16):
            out = []
            ids = torch.as_tensor(ids, device=cuda).long()
            for c0 in range(0, len(ids), 512):
                sel = ids[c0:c0 + 512]
                sk = (kk16[sel].view(len(sel), -1, 4096).to(torch.int64) * weights).sum(dim=(1, 2))
                sv = (vv16[sel].view(len(sel), -1, 4096).to(torch.int64) * weights).sum(dim=(1, 2))
                out.append(sk * 31 + sv)
            return torch.cat(out)

        live_t = torch.from_numpy(live).to(cuda).long()
        for c0 in range(0, len(live), 512):
            ids = live_t[c0:c0 + 512]
            pat = torch.randint(-30000, 30000, (len(ids), L * HKV * B * D), dtype=torch.int16, device=cuda, generator=gen)
            k16[ids] = pat
            v16[ids] = pat.flip(1)
        before = checksums(live, k16, v16)
        want_src, want_dst = R.plan_migration(free, new_n)
        del k16, v16                                   # views of memory the shrink unmaps
        src, dst = pool.shrink_to(new_n)
        torch.cuda.synchronize()
        assert src.cpu().tolist() == want_src.tolist() and dst.cpu().tolist() == want_dst.tolist()
        assert pool.num_blocks == new_n and pool.k_cache.shape[0] == new_n
        new_table = bm.block_table.cpu().numpy()
        now = np.concatenate([new_table[s, :per_seq] for s in rows])
        assert now.max() < new_n and len(np.unique(now)) == len(now)
        remap = dict(zip(want_src.tolist(), want_dst.tolist()))
        assert np.array_equal(now, np.array([remap.get(int(b), int(b)) for b in live]))
        k16 = pool.k_cache.view(torch.int16).reshape(new_n, -1)
        v16 = pool.v_cache.view(torch.int16).reshape(new_n, -1)
        assert torch.equal(checksums(now, k16, v16), before), "a sequence's KV changed during migration"
        is_free = bm.is_block_free.cpu().numpy()
        assert len(is_free) == new_n and int(is_free.sum()) == bm.num_free_blocks == new_n - len(live)
        assert not is_free[now].any()
        # the memory above the cut went back to the driver: the pool, its spare chunks and little else are held
        held = free_at_start - torch.cuda.mem_get_info(cuda)[0]
        chunk_bytes = SEG * L * HKV * B * D * 2
        # (torch keeps this test's own temporaries cached: up to a few GiB of gathers and 64-bit sums)
        assert held <= 2 * (new_n // SEG) * chunk_bytes + 2 * chunk_bytes + (24 << 30) < 2 * (total // SEG) * chunk_bytes
        del k16, v16
    finally:
        pool.close()


def test_config5_shapes_one_layer(cuda):
    """CodeLlama-34B decode shapes (GQA 64 q / 8 kv heads, batch 128, contexts in
    [1024, 1536]) on one layer against the CPU oracle."""
    rng = np.random.default_rng(55)
    lens = rng.integers(1024, 1537, size=128)
    nblk = int(((lens + 15) // 16).sum()) + 16
    case = make_case(55, 1, 64, 8, lens, num_blocks=nblk, max_seqs=256, max_blocks_per_seq=128, fill="live")
    kc, vc, bt = to_gpu(case, cuda)
    q = rand_f16(rng, 128, 64, 128)
    k = rand_f16(rng, 128, 8, 128)
    v = rand_f16(rng, 128, 8, 128)
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, 0)
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, case.seq_lens, 128 ** -0.5, 0)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), case.seq_lens.tolist(), 8, 128)
    o = torch.empty((128, 64 * 128), dtype=torch.float16, device=cuda)
    decode_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                             torch.from_numpy(q).to(cuda), kc, vc, [], [], bt, model, engine, st, 0, o)
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    assert_attn_close(o.cpu().numpy().reshape(128, 64, 128), want, "config 5 shapes")


def test_config4_mixed_batch_one_layer(cuda):
    """Llama-2-7B MHA shapes: eight 512-token prefill chunks plus 120 decode
    sequences with lognormal context lengths in one batch: append (both kernels),
    prefill attention over the batch's own k/v, decode attention over the cache."""
    rng = np.random.default_rng(44)
    p_lens = [512] * 8
    d_lens = np.clip(rng.lognormal(6.2, 0.6, size=120), 16, 768).astype(np.int64)
    lens = np.concatenate([p_lens, d_lens])
    nblk = int(((lens + 15) // 16).sum()) + 32
    case = make_case(44, 1, 32, 32, lens, num_blocks=nblk, max_seqs=256, max_blocks_per_seq=64, fill="live")
    kc, vc, bt = to_gpu(case, cuda)
    T = sum(p_lens)
    n_tok = T + len(d_lens)
    q = rand_f16(rng, n_tok, 32, 128)
    k = rand_f16(rng, n_tok, 32, 128)
    v = rand_f16(rng, n_tok, 32, 128)
    starts = np.cumsum(p_lens) - np.asarray(p_lens)
    R.store_kvcache(case.arena, case.lay, k, v, case.block_table, case.seq_ids, 8, T, starts,
                    np.asarray(p_lens), d_lens, 0)
    want_p = R.prefill_attention(q[:T], k[:T], v[:T], starts, np.asarray(p_lens), 128 ** -0.5, math="torch32")
    want_d = R.paged_attention(q[T:], case.arena, case.lay, case.block_table, case.seq_ids[8:], d_lens,
                               128 ** -0.5, 0)
    model, engine = configs(case)
    st = build_infer_state(p_lens, case.seq_ids.tolist(), d_lens.tolist(), 32, 128)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    o = torch.full((n_tok, 32 * 128), float("nan"), dtype=torch.float16, device=cuda)
    store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 0)
    prefill_attention(qg[:T], kg[:T], vg[:T], o[:T].view(T, 32, 128), model, engine, st)
    paged_attention(qg[T:], kc, vc, [], [], bt, model, engine, st, 0, o[T:])
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    got = o.cpu().numpy().reshape(n_tok, 32, 128)
    assert_attn_close(got[:T], want_p, "config 4 prefill")
    assert_attn_close(got[T:], want_d, "config 4 decode")


def test_zero_fill_larger_than_one_launch(cuda):
    """40 GiB + 5 bytes: more 16-byte units than one launch may have threads, plus a tail."""
    from morphserve_amd import _capi
    if _mem_gib(cuda) < 48:
        pytest.skip("needs ~41 GiB of free HBM")
    n = 40 * 2 ** 30 + 5
    buf = torch.empty(n + 16, dtype=torch.uint8, device=cuda)
    probes = [0, 1, 2 ** 35 - 1, 2 ** 35, 2 ** 35 + 16, 39 * 2 ** 30 + 7, n - 6, n - 1, n]
    for p in probes:
        buf[p] = 0xAB
    _capi.check(_capi.lib().mkv_fill_zero(buf.data_ptr(), n, _capi.current_stream()))
    torch.cuda.synchronize()
    got = [int(buf[p]) for p in probes]
    assert got == [0] * (len(probes) - 1) + [0xAB], got         # the byte after the range is untouched
    assert int(buf[:2 ** 31].max()) == 0 and int(buf[n - 2 ** 30:n].max()) == 0
    sample = buf[:n].view(torch.int64)[::4099] if n % 8 == 0 else buf[:n - 5].view(torch.int64)[::4099]
    assert int(sample.abs().max()) == 0
