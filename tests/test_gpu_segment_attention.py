"""GPU parity of every attention entry over a pool that has grown by extension segments
(the reference's segment-aware phase 1, MorphServe/worker/kernels/paged_attn.py:243-437, addressing
:354-360 and :397-403): block tables mix base-pool and segment ids, three segments laid out as the
reference's memory is (segment j one 'weight layer' below segment j-1), one sequence's final block
-- the one a fused append writes to -- sits in the last segment.  Outputs against the CPU oracle on
the matching ``PoolLayout``; after a fused append the WHOLE arena, padding between the segments
included, must be bit-identical to the oracle's."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from oracle import rope_cpu as RO
from helpers import Cfg, assert_attn_close, rand_f16
from gpu_helpers import bits, kernel_variant
from morphserve_amd import (_capi, build_infer_state, chunked_prefill_attention, decode_append_and_attend,
                            decode_rope_append_and_attend, paged_attention, store_kvcache)
from morphserve_amd.worker.kernels import paged_attn as PA
from morphserve_amd.worker.kernels._pool import pool_strided
from test_gpu_append import _segment_setup

pytestmark = pytest.mark.gpu

L, LAYER, ORG, S, NSEG, MAX_SEQS, MBPS = 2, 1, 40, 24, 3, 16, 48
LENS = [600, 333, 16, 17, 1, 250, 129]


class SegCase:
    """Arena + layout + a table whose rows mix base and segment ids."""

    def __init__(self, cuda, seed, Hq, Hkv, lens=LENS):
        self.Hq, self.Hkv, self.D = Hq, Hkv, 128
        (self.arena, self.lay, self.g, self.kc, self.vc, self.k_new, self.v_new,
         self.stride) = _segment_setup(cuda, seed, L, Hkv, ORG, S, NSEG)
        rng = np.random.default_rng(seed + 1)
        total = ORG + NSEG * S
        self.lens = np.asarray(lens, dtype=np.int32)
        need = (self.lens + 15) // 16
        order = rng.permutation(total)
        # the rows straddle the boundaries: ids org-1, org, org+S-1, org+S lead the deal
        edge = [ORG - 1, ORG, ORG + S - 1, ORG + S, ORG + 2 * S - 1, ORG + 2 * S]
        order = np.concatenate([edge, [b for b in order if b not in edge]]).astype(np.int64)
        self.seq_ids = rng.permutation(MAX_SEQS)[:len(lens)].astype(np.int32)
        self.table = np.full((MAX_SEQS, MBPS), -1, dtype=np.int32)
        pos = 0
        for s, nb in zip(self.seq_ids, need):
            self.table[s, :nb] = order[pos:pos + nb]
            pos += nb
        # sequence 0's final block goes to the last segment, sequence 1's to the first, sequence 5's to the base
        used = set(order[:pos].tolist())
        spare_last = [b for b in range(ORG + 2 * S, total) if b not in used]
        spare_first = [b for b in range(ORG, ORG + S) if b not in used]
        spare_base = [b for b in range(ORG) if b not in used]
        self.table[self.seq_ids[0], need[0] - 1] = spare_last[0]
        self.table[self.seq_ids[1], need[1] - 1] = spare_first[0]
        self.table[self.seq_ids[5], need[5] - 1] = spare_base[0]
        live = self.table[self.table >= 0]
        assert len(set(live.tolist())) == len(live), "a block is owned twice"
        assert (live >= ORG + 2 * S).any() and (live < ORG).any()
        self.bt = torch.from_numpy(self.table).to(cuda)
        self.model = Cfg(num_layers=L, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=128)
        self.engine = Cfg(block_size=16, max_blocks_per_seq=MBPS)

    def state(self, p_lens, d_lens, ids=None):
        ids = self.seq_ids.tolist() if ids is None else ids
        return build_infer_state(p_lens, ids, d_lens, self.Hkv, 128, num_blocks_org=ORG,
                                 kv_cache_new_block_size=S, org_layer_param_size=self.stride)

    def oracle(self, q):
        return R.paged_attention(q, self.arena, self.lay, self.table, self.seq_ids, self.lens, 128 ** -0.5, LAYER)


class _Knobs:
    def __init__(self, variant, target_wgs):
        self.variant, self.target_wgs = variant, target_wgs

    def __enter__(self):
        self.old = PA.TARGET_WORKGROUPS
        PA.TARGET_WORKGROUPS = self.target_wgs
        self.pin = kernel_variant(decode=self.variant)
        self.pin.__enter__()

    def __exit__(self, *exc):
        PA.TARGET_WORKGROUPS = self.old
        self.pin.__exit__(*exc)


@pytest.mark.parametrize("Hq,Hkv,variant", [(8, 8, 1), (32, 8, 1), (32, 8, 2), (16, 2, 2), (6, 2, 2)])
@pytest.mark.parametrize("target_wgs", [1, 100000])
def test_paged_attention_over_segments(cuda, Hq, Hkv, variant, target_wgs):
    c = SegCase(cuda, 40 + Hq, Hq, Hkv)
    rng = np.random.default_rng(Hq)
    n = len(c.lens)
    q = rand_f16(rng, n, Hq, 128)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    with _Knobs(variant, target_wgs):
        paged_attention(torch.from_numpy(q).to(cuda), c.kc, c.vc, c.k_new, c.v_new, c.bt, c.model, c.engine,
                        c.state([], c.lens.tolist()), LAYER, o)
        torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), c.oracle(q), f"segments, variant {variant}")
    assert np.array_equal(bits(c.g), bits(c.arena)), "attention must not write to the pool"


@pytest.mark.parametrize("Hq,Hkv,variant", [(8, 8, 1), (32, 8, 1), (32, 8, 2), (64, 8, 2)])
@pytest.mark.parametrize("target_wgs", [1, 100000])
def test_fused_append_and_attend_over_segments(cuda, Hq, Hkv, variant, target_wgs):
    c = SegCase(cuda, 60 + Hq, Hq, Hkv)
    rng = np.random.default_rng(Hq + 1)
    n = len(c.lens)
    q, k, v = rand_f16(rng, n, Hq, 128), rand_f16(rng, n, Hkv, 128), rand_f16(rng, n, Hkv, 128)
    R.append_decode(c.arena, c.lay, k, v, c.table, c.seq_ids, c.lens, LAYER)
    want = c.oracle(q)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    with _Knobs(variant, target_wgs):
        decode_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                                 torch.from_numpy(q).to(cuda), c.kc, c.vc, c.k_new, c.v_new, c.bt, c.model,
                                 c.engine, c.state([], c.lens.tolist()), LAYER, o)
        torch.cuda.synchronize()
    assert np.array_equal(bits(c.g), bits(c.arena)), "whole arena after the fused append"
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), want, f"fused append over segments, variant {variant}")


@pytest.mark.parametrize("Hq,Hkv,variant", [(8, 8, 1), (32, 8, 2)])
@pytest.mark.parametrize("target_wgs", [1, 100000])
def test_rope_fused_append_and_attend_over_segments(cuda, Hq, Hkv, variant, target_wgs):
    c = SegCase(cuda, 80 + Hq, Hq, Hkv)
    rng = np.random.default_rng(Hq + 2)
    n = len(c.lens)
    q, k, v = rand_f16(rng, n, Hq, 128), rand_f16(rng, n, Hkv, 128), rand_f16(rng, n, Hkv, 128)
    ct, st_ = RO.rotary_tables(128, 2048)
    pos = c.lens - 1
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
    state = c.state([], c.lens.tolist())
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    with _Knobs(variant, target_wgs):
        decode_rope_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                                      torch.from_numpy(q).to(cuda), c.kc, c.vc, c.k_new, c.v_new, c.bt, c.model,
                                      c.engine, state, LAYER, o)
        torch.cuda.synchronize()
    q_rot, k_rot = q.copy(), k.copy()
    RO.rotary_embedding_inplace(q_rot, k_rot, cos, sin)
    R.append_decode(c.arena, c.lay, k_rot, v, c.table, c.seq_ids, c.lens, LAYER)
    assert np.array_equal(bits(c.g), bits(c.arena)), "whole arena after rotary + append"
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), c.oracle(q_rot), "rotary + append + attention, segments")


@pytest.mark.parametrize("Hq,Hkv", [(8, 2), (32, 32)])
def test_chunked_prefill_over_segments(cuda, Hq, Hkv):
    """Prompts appended through store_kvcache into base and segment blocks; the last two thirds of each
    prompt attend as a chunk over the cached first third."""
    c = SegCase(cuda, 90 + Hq, Hq, Hkv)
    rng = np.random.default_rng(Hq + 3)
    lens = c.lens.astype(np.int64)
    T = int(lens.sum())
    q, k, v = rand_f16(rng, T, Hq, 128), rand_f16(rng, T, Hkv, 128), rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - lens
    st = c.state(lens.tolist(), [])
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), c.kc, c.vc, c.k_new, c.v_new, c.bt,
                  c.model, c.engine, st, LAYER)
    R.append_prefill(c.arena, c.lay, k, v, c.table, c.seq_ids, starts, lens, LAYER)
    torch.cuda.synchronize()
    assert np.array_equal(bits(c.g), bits(c.arena))
    prefix = lens // 3
    l2 = lens - prefix
    s2 = np.cumsum(l2) - l2
    q2 = np.concatenate([q[starts[b] + prefix[b]:starts[b] + lens[b]] for b in range(len(lens))])
    want = R.chunked_prefill_attention(q2, c.arena, c.lay, c.table, c.seq_ids, s2, l2, prefix, 128 ** -0.5, LAYER)
    o = torch.full((int(l2.sum()), Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    chunked_prefill_attention(torch.from_numpy(q2).to(cuda), c.kc, c.vc, c.k_new, c.v_new, c.bt, c.model, c.engine,
                              c.state(l2.tolist(), []), LAYER, o,
                              prefix_lens=torch.from_numpy(prefix.astype(np.int32)).to(cuda))
    torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy(), want, "chunked prefill over segments")


@pytest.mark.parametrize("Hq,Hkv,variant", [(8, 8, 1), (32, 8, 2)])
@pytest.mark.parametrize("tps", [64, 1024])
def test_attention_through_the_strided_convention(cuda, Hq, Hkv, variant, tps):
    """The reference's calling convention reaches the attention kernels through the C-ABI: only segment 0 is
    passed and mkv_pool_set_strided derives the rest (csrc/src/block_swapping.cpp:156-160)."""
    c = SegCase(cuda, 120 + Hq, Hq, Hkv)
    pool = pool_strided(c.kc, c.vc, c.k_new[0], c.v_new[0], ORG, c.stride, S, 2, NSEG)
    assert [pool.k_seg[j] for j in range(NSEG)] == [t.data_ptr() for t in c.k_new]
    rng = np.random.default_rng(Hq + 4)
    n = len(c.lens)
    q, k, v = rand_f16(rng, n, Hq, 128), rand_f16(rng, n, Hkv, 128), rand_f16(rng, n, Hkv, 128)
    splits = -(-int(c.lens.max()) // tps)
    ids = torch.from_numpy(c.seq_ids).to(cuda)
    lens = torch.from_numpy(c.lens).to(cuda)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    rows = n * Hq * splits
    mid_o = torch.empty(rows * 128, dtype=torch.float32, device=cuda)
    mid_lse = torch.empty(rows, dtype=torch.float32, device=cuda)
    o = torch.full((n, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    with kernel_variant(decode=variant) as lib:
        _capi.check(lib.mkv_paged_attn_decode(
            qg.data_ptr(), o.data_ptr(), C.byref(pool), c.bt.data_ptr(), MBPS, ids.data_ptr(), lens.data_ptr(), n, Hq,
            float(128 ** -0.5), LAYER, tps, splits, mid_o.data_ptr(), mid_lse.data_ptr(), _capi.current_stream()))
        torch.cuda.synchronize()
        assert_attn_close(o.cpu().numpy(), c.oracle(q), f"strided pool, {splits} splits")
        R.append_decode(c.arena, c.lay, k, v, c.table, c.seq_ids, c.lens, LAYER)
        o.fill_(float("nan"))
        _capi.check(lib.mkv_decode_append_attn(
            kg.data_ptr(), vg.data_ptr(), qg.data_ptr(),
            o.data_ptr(), C.byref(pool), c.bt.data_ptr(), MBPS, ids.data_ptr(), lens.data_ptr(), n, Hq,
            float(128 ** -0.5), LAYER, tps, splits, mid_o.data_ptr(), mid_lse.data_ptr(), _capi.current_stream()))
        torch.cuda.synchronize()
    assert np.array_equal(bits(c.g), bits(c.arena)), "whole arena after the fused append (strided pool)"
    assert_attn_close(o.cpu().numpy(), c.oracle(q), f"fused append, strided pool, {splits} splits")


@pytest.mark.parametrize("Hq,Hkv", [(8, 8), (32, 8)])
def test_attention_section_mixed_batch_over_segments(cuda, Hq, Hkv):
    """The layer's whole attention section (rotary + append of every row, prefill attention, decode attention)
    on a mixed batch whose blocks lie in the base pool and in all three segments."""
    from morphserve_amd import attention_section
    c = SegCase(cuda, 120 + Hq, Hq, Hkv)
    rng = np.random.default_rng(Hq + 5)
    pre, dec = [2, 3], [0, 1, 4, 5, 6]                     # the 16- and 17-token sequences arrive as prompts
    p_lens = c.lens[pre].tolist()
    d_lens = c.lens[dec].tolist()
    ids = c.seq_ids[pre + dec]
    P, n = sum(p_lens), len(dec)
    T = P + n
    q, k, v = rand_f16(rng, T, Hq, 128), rand_f16(rng, T, Hkv, 128), rand_f16(rng, T, Hkv, 128)
    ct, st_ = RO.rotary_tables(128, 2048)
    pos = np.concatenate([np.arange(x) for x in p_lens] + [np.asarray(d_lens) - 1])
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
    state = c.state(p_lens, d_lens, ids.tolist())
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    o = torch.full((T, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    attention_section(qg, kg, vg, o, c.kc, c.vc, c.k_new, c.v_new, c.bt, c.model, c.engine, state, LAYER)
    torch.cuda.synchronize()
    RO.rotary_embedding_inplace(q, k, cos, sin)
    starts = np.cumsum(p_lens) - np.asarray(p_lens)
    R.store_kvcache(c.arena, c.lay, k, v, c.table, ids, len(pre), P, starts, np.asarray(p_lens), np.asarray(d_lens),
                    LAYER)
    assert np.array_equal(bits(c.g), bits(c.arena)), "whole arena after rotary + append of the mixed batch"
    assert np.array_equal(bits(qg), bits(q)) and np.array_equal(bits(kg), bits(k))
    got = o.cpu().numpy().reshape(T, Hq, 128)
    want_p = R.prefill_attention(q[:P], k[:P], v[:P], starts, np.asarray(p_lens), 128 ** -0.5, math="np32")
    assert_attn_close(got[:P], np.asarray(want_p), "prefill rows")
    want_d = R.paged_attention(q[P:], c.arena, c.lay, c.table, ids[len(pre):], np.asarray(d_lens), 128 ** -0.5, LAYER)
    assert_attn_close(got[P:], np.asarray(want_d), "decode rows over segments")
