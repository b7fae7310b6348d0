"""Pins the CPU oracle's append and attention functions without retyping them:
brute force on the 5-D cache shape, invariants, closed forms, library routines.
The reference ships no tests or fixtures for this path, so these are the anchors.
"""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import make_case, rand_f16, attn_err


def _views(case):
    return case.k_pool, case.v_pool


# ---------------------------------------------------------------------------
# append
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("seed,Hkv,L,layer", [(0, 2, 1, 0), (1, 4, 3, 2), (2, 8, 2, 1)])
def test_append_decode_brute_force(seed, Hkv, L, layer):
    rng = np.random.default_rng(seed)
    lens = rng.integers(1, 70, size=5)
    case = make_case(seed, L, Hkv, Hkv, lens, num_blocks=40, D=16, fill="all")
    before = case.arena.copy()
    k = rand_f16(rng, len(lens), Hkv, 16)
    v = rand_f16(rng, len(lens), Hkv, 16)
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, layer)

    # expected: written on the 5-D view of a copy, indexed by shape alone
    exp = before.copy()
    nb = case.num_blocks * case.lay.block_elems
    ek = exp[:nb].reshape(case.num_blocks, L, Hkv, 16, 16)
    ev = exp[nb:].reshape(case.num_blocks, L, Hkv, 16, 16)
    for i, (s, n) in enumerate(zip(case.seq_ids, case.seq_lens)):
        blk = case.block_table[s, (n - 1) // 16]
        ek[blk, layer, :, (n - 1) % 16, :] = k[i]
        ev[blk, layer, :, (n - 1) % 16, :] = v[i]
    assert np.array_equal(case.arena.view(np.uint16), exp.view(np.uint16))
    # exactly n * Hkv * D * 2 elements may differ from before (random data: all do)
    changed = np.count_nonzero(case.arena.view(np.uint16) != before.view(np.uint16))
    assert changed <= len(lens) * Hkv * 16 * 2
    # idempotent
    again = case.arena.copy()
    R.append_decode(again, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, layer)
    assert np.array_equal(again.view(np.uint16), case.arena.view(np.uint16))


@pytest.mark.parametrize("seed,Hkv,L,layer", [(3, 2, 2, 1), (4, 4, 1, 0)])
def test_append_prefill_brute_force(seed, Hkv, L, layer):
    rng = np.random.default_rng(seed)
    lens = np.array([1, 16, 17, 40, 5])
    case = make_case(seed, L, Hkv, Hkv, lens, num_blocks=30, D=8, fill="all")
    before = case.arena.copy()
    T = int(lens.sum())
    k = rand_f16(rng, T, Hkv, 8)
    v = rand_f16(rng, T, Hkv, 8)
    starts = np.cumsum(lens) - lens
    R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, layer)
    exp = before.copy()
    nb = case.num_blocks * case.lay.block_elems
    ek = exp[:nb].reshape(case.num_blocks, L, Hkv, 16, 8)
    ev = exp[nb:].reshape(case.num_blocks, L, Hkv, 16, 8)
    for b, s in enumerate(case.seq_ids):
        for t in range(lens[b]):
            blk = case.block_table[s, t // 16]
            ek[blk, layer, :, t % 16, :] = k[starts[b] + t]
            ev[blk, layer, :, t % 16, :] = v[starts[b] + t]
    assert np.array_equal(case.arena.view(np.uint16), exp.view(np.uint16))


def test_prefill_then_gather_is_identity_and_permutation_invariant():
    """Logical content read back through the table equals what was appended,
    whatever physical blocks the table names."""
    rng = np.random.default_rng(5)
    lens = np.array([33, 7, 64])
    T = int(lens.sum())
    k = rand_f16(rng, T, 2, 8)
    v = rand_f16(rng, T, 2, 8)
    starts = np.cumsum(lens) - lens
    got = []
    for permute in (True, False):
        case = make_case(7, 2, 2, 2, lens, num_blocks=20, D=8, permute=permute, fill="live")
        R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, 1)
        per = []
        for b, s in enumerate(case.seq_ids):
            ks, vs = R.gather_kv(case.arena, case.lay, case.block_table, s, lens[b], 1)
            per.append((ks[:, :lens[b]].copy(), vs[:, :lens[b]].copy()))
            assert np.array_equal(ks[:, :lens[b]], k[starts[b]:starts[b] + lens[b]].transpose(1, 0, 2))
            assert np.array_equal(vs[:, :lens[b]], v[starts[b]:starts[b] + lens[b]].transpose(1, 0, 2))
        got.append(per)
    for a, b in zip(*got):
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])


def test_store_kvcache_mixed_batch_order():
    """Prefill rows first, decode rows from k[num_prefill_tokens:] with seq_ids[num_prefill_seqs:]."""
    rng = np.random.default_rng(11)
    p_lens = np.array([20, 3])
    d_lens = np.array([18, 33, 1])
    lens = np.concatenate([p_lens, d_lens])
    case = make_case(11, 1, 2, 2, lens, num_blocks=16, D=8, fill="live")
    T = int(p_lens.sum())
    k = rand_f16(rng, T + 3, 2, 8)
    v = rand_f16(rng, T + 3, 2, 8)
    starts = np.cumsum(p_lens) - p_lens
    R.store_kvcache(case.arena, case.lay, k, v, case.block_table, case.seq_ids, 2, T, starts,
                    p_lens, d_lens, 0)
    kp = case.k_pool
    for i, n in enumerate(d_lens):
        s = case.seq_ids[2 + i]
        blk = case.block_table[s, (n - 1) // 16]
        assert np.array_equal(kp[blk, 0, :, (n - 1) % 16, :], k[T + i])
    s0 = case.seq_ids[0]
    assert np.array_equal(kp[case.block_table[s0, 1], 0, :, 3, :], k[19])


# ---------------------------------------------------------------------------
# segment addressing
# ---------------------------------------------------------------------------
def _segment_arena(rng, L, Hkv, B, D, org, S, nseg, stride_elems):
    """Arena laid out as the reference's memory would be: segments at descending
    addresses (segment j is j * stride below segment 0), base K and V pools after."""
    blk = L * Hkv * B * D
    seg_span = 2 * S * blk                      # K then V of one segment
    assert stride_elems >= seg_span
    seg0 = (nseg - 1) * stride_elems
    base_k = seg0 + seg_span + 64
    base_v = base_k + org * blk
    total = base_v + org * blk
    arena = rng.standard_normal(total, dtype=np.float32).astype(np.float16)
    lay = R.PoolLayout(L, Hkv, B, D, k_base=base_k, v_base=base_v, num_blocks_org=org,
                       seg_blocks=S, k_new0=seg0, v_new0=seg0 + S * blk,
                       org_layer_param_size=stride_elems)
    return arena, lay


def test_segment_offsets_by_hand():
    L, Hkv, B, D = 2, 2, 4, 8
    blk = L * Hkv * B * D                      # 128 elements
    lay = R.PoolLayout(L, Hkv, B, D, k_base=10_000, v_base=20_000, num_blocks_org=5,
                       seg_blocks=3, k_new0=5_000, v_new0=5_000 + 3 * blk,
                       org_layer_param_size=1_000)
    assert lay.block_offset("k", 4) == 10_000 + 4 * 128
    assert lay.block_offset("k", 5) == 5_000                       # first block of segment 0
    assert lay.block_offset("v", 7) == 5_000 + 3 * 128 + 2 * 128   # last block of segment 0
    assert lay.block_offset("k", 8) == 4_000                       # segment 1 = one stride below
    assert lay.block_offset("k", 12) == 3_000 + 128                # segment 2, local 1
    assert lay.slab("v", 12, 1, 1) == 3_000 + 3 * 128 + 128 + (1 * 2 + 1) * 32


def test_segment_vs_plain_equivalence():
    """Appending + attending through segment ids gives the same logical result as
    through base ids when the table is remapped."""
    rng = np.random.default_rng(21)
    L, Hkv, B, D, org, S, nseg = 2, 2, 16, 16, 6, 4, 3
    blk = L * Hkv * B * D
    arena, lay = _segment_arena(rng, L, Hkv, B, D, org, S, nseg, stride_elems=2 * S * blk + 40)
    lens = np.array([30, 50])
    # sequence 0 in base blocks, sequence 1 spread over all three segments
    table = np.full((2, 8), -1, dtype=np.int32)
    table[0, :2] = [3, 1]
    table[1, :4] = [org + 1, org + S + 2, org + 2 * S + 0, org + 3]
    seq_ids = np.array([0, 1], dtype=np.int32)
    T = int(lens.sum())
    k = rand_f16(rng, T, Hkv, D)
    v = rand_f16(rng, T, Hkv, D)
    starts = np.cumsum(lens) - lens
    R.append_prefill(arena, lay, k, v, table, seq_ids, starts, lens, 1)
    q = rand_f16(rng, 2, 4, D)
    o_seg = R.paged_attention(q, arena, lay, table, seq_ids, lens, D ** -0.5, 1, math="np64",
                              out_dtype=np.float64)

    plain = make_case(0, L, 4, Hkv, lens, num_blocks=12, D=D, permute=False, fill="live")
    R.append_prefill(plain.arena, plain.lay, k, v, plain.block_table, plain.seq_ids, starts, lens, 1)
    o_plain = R.paged_attention(q, plain.arena, plain.lay, plain.block_table, plain.seq_ids, lens,
                                D ** -0.5, 1, math="np64", out_dtype=np.float64)
    assert np.array_equal(o_seg, o_plain)
    # explicit segment table = stride rule
    lay2 = R.PoolLayout(L, Hkv, B, D, lay.k_base, lay.v_base, org, S,
                        k_seg=[lay.k_new0 - j * lay.org_layer_param_size for j in range(nseg)],
                        v_seg=[lay.v_new0 - j * lay.org_layer_param_size for j in range(nseg)])
    for bid in range(org + nseg * S):
        assert lay.block_offset("k", bid) == lay2.block_offset("k", bid)
        assert lay.block_offset("v", bid) == lay2.block_offset("v", bid)


# ---------------------------------------------------------------------------
# decode attention
# ---------------------------------------------------------------------------
def _sdpa(q, ks, vs, L, G):
    tq = torch.from_numpy(q.astype(np.float64)).unsqueeze(1)                       # [Hq,1,D]
    tk = torch.from_numpy(ks[:, :L].astype(np.float64)).repeat_interleave(G, 0)    # [Hq,L,D]
    tv = torch.from_numpy(vs[:, :L].astype(np.float64)).repeat_interleave(G, 0)
    return torch.nn.functional.scaled_dot_product_attention(tq, tk, tv).squeeze(1).numpy()


@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2)])
def test_paged_attention_vs_torch_sdpa(Hq, Hkv):
    rng = np.random.default_rng(31)
    lens = np.array([1, 15, 16, 17, 100])
    case = make_case(31, 2, Hq, Hkv, lens, num_blocks=24, D=32, fill="all")
    q = rand_f16(rng, len(lens), Hq, 32)
    for math, tol in (("np64", 1e-12), ("torch32", 2e-6)):
        o = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                              32 ** -0.5, 1, out_dtype=np.float64, math=math)
        for i, n in enumerate(lens):
            ks, vs = R.gather_kv(case.arena, case.lay, case.block_table, case.seq_ids[i], n, 1)
            want = _sdpa(q[i], ks, vs, int(n), Hq // Hkv)
            assert np.abs(o[i] - want).max() < tol, (math, i)


def test_paged_attention_closed_forms():
    rng = np.random.default_rng(32)
    lens = np.array([1, 40])
    case = make_case(32, 1, 4, 2, lens, num_blocks=8, D=16, fill="all")
    q = rand_f16(rng, 2, 4, 16)
    # len == 1: output is V[0] exactly (fp16 in, fp16 out)
    o = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens, 0.25, 0)
    s0 = case.seq_ids[0]
    v0 = case.v_pool[case.block_table[s0, 0], 0, :, 0, :]
    assert np.array_equal(o[0], np.repeat(v0, 2, axis=0))
    # identical keys: uniform weights, output = mean of V over the valid tokens
    s1 = case.seq_ids[1]
    for j in range(3):
        case.k_pool[case.block_table[s1, j], 0] = case.k_pool[case.block_table[s1, 0], 0, :, :1, :]
    o = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens, 0.25, 0,
                          out_dtype=np.float64, math="np64")
    ks, vs = R.gather_kv(case.arena, case.lay, case.block_table, s1, 40, 0)
    mean_v = vs[:, :40].astype(np.float64).mean(axis=1)
    assert np.abs(o[1] - np.repeat(mean_v, 2, axis=0)).max() < 1e-12
    # q heads of one group with equal q give equal o
    q[1, 1] = q[1, 0]
    o = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens, 0.25, 0)
    assert np.array_equal(o[1, 0], o[1, 1])


def test_masked_tail_does_not_leak():
    """Bytes beyond len in the last block must not influence the result."""
    rng = np.random.default_rng(33)
    lens = np.array([21])
    case = make_case(33, 1, 2, 2, lens, num_blocks=4, D=16, fill="all")
    q = rand_f16(rng, 1, 2, 16)
    o1 = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens, 0.25, 0)
    last = case.block_table[case.seq_ids[0], 1]
    case.k_pool[last, 0, :, 5:, :] = 99.0
    case.v_pool[last, 0, :, 5:, :] = -77.0
    o2 = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens, 0.25, 0)
    assert np.array_equal(o1, o2)


@pytest.mark.parametrize("sbs", [16, 64, 512])
def test_split_formulation_matches_unsplit(sbs):
    rng = np.random.default_rng(34)
    lens = np.array([5, 64, 130, 300])
    case = make_case(34, 1, 4, 2, lens, num_blocks=40, D=32, fill="all")
    q = rand_f16(rng, 4, 4, 32)
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                             32 ** -0.5, 0, out_dtype=np.float64, math="np64")
    got = R.paged_attention_split(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                                  32 ** -0.5, 0, sbs)
    ae, _ = attn_err(got, want)
    assert ae < 1.5e-3          # fp16 rounding of outputs of magnitude <~ 2


def test_fp32_vs_fp64_budget():
    """How much of the 2e-3 budget the fp32 math + fp16 rounding already uses."""
    rng = np.random.default_rng(35)
    lens = np.array([700, 1300])
    case = make_case(35, 1, 8, 2, lens, num_blocks=130, D=128, fill="all")
    q = rand_f16(rng, 2, 8, 128)
    o64 = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                            128 ** -0.5, 0, out_dtype=np.float64, math="np64")
    o32 = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                            128 ** -0.5, 0)
    ae, _ = attn_err(o32, o64)
    assert ae < 5e-4


def test_seq_block_size_known_answers():
    # 8 sequences, MHA 32 heads, lengths <= 512: 32*(sum/sbs) stays below 1024 down to 64
    lens = [64, 100, 200, 288, 300, 400, 445, 512]
    assert R.select_seq_block_size(32, lens) == (64, 8)
    # 64 sequences of ~1280 tokens, 8 kv heads: 8 * 81920/512 = 1280 >= 1024 -> stays 512
    assert R.select_seq_block_size(8, [1280] * 64) == (512, 3)
    # one short sequence: halves down to the floor of 64
    assert R.select_seq_block_size(8, [100]) == (64, 2)
    # very long single sequence: max_len / (sbs/2) <= 128 stops the halving at 512
    assert R.select_seq_block_size(1, [40000]) == (512, 79)
    assert R.select_seq_block_size(8, []) == (64, 0)


# ---------------------------------------------------------------------------
# prefill attention
# ---------------------------------------------------------------------------
def test_prefill_attention_vs_dense_and_decode():
    rng = np.random.default_rng(41)
    lens = np.array([1, 9, 16, 40])
    T = int(lens.sum())
    Hq, Hkv, D = 4, 2, 16
    q = rand_f16(rng, T, Hq, D)
    k = rand_f16(rng, T, Hkv, D)
    v = rand_f16(rng, T, Hkv, D)
    starts = np.cumsum(lens) - lens
    o = R.prefill_attention(q, k, v, starts, lens, D ** -0.5, out_dtype=np.float64)
    for b, n in enumerate(lens):
        sl = slice(starts[b], starts[b] + n)
        tq = torch.from_numpy(q[sl].astype(np.float64)).permute(1, 0, 2)
        tk = torch.from_numpy(k[sl].astype(np.float64)).permute(1, 0, 2).repeat_interleave(2, 0)
        tv = torch.from_numpy(v[sl].astype(np.float64)).permute(1, 0, 2).repeat_interleave(2, 0)
        want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)
        assert np.abs(o[sl] - want.permute(1, 0, 2).numpy()).max() < 1e-12
    o32 = R.prefill_attention(q, k, v, starts, lens, D ** -0.5, out_dtype=np.float64, math="torch32")
    assert np.abs(o32 - o).max() < 2e-6
    # last row of each sequence == decode attention over the same tokens in a paged cache
    case = make_case(41, 1, Hq, Hkv, lens, num_blocks=12, D=D, fill="live")
    R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, 0)
    last_q = q[starts + lens - 1]
    od = R.paged_attention(last_q, case.arena, case.lay, case.block_table, case.seq_ids, lens,
                           D ** -0.5, 0, out_dtype=np.float64, math="np64")
    assert np.abs(od - o[starts + lens - 1]).max() < 1e-12
    # chunk-with-prefix over the cache: whole prompt as one chunk == prefill; split in two == same rows
    oc = R.chunked_prefill_attention(q, case.arena, case.lay, case.block_table, case.seq_ids,
                                     starts, lens, np.zeros(4, dtype=np.int64), D ** -0.5, 0,
                                     out_dtype=np.float64)
    assert np.abs(oc - o).max() < 1e-12
    half = lens // 2
    q2 = np.concatenate([q[starts[b] + half[b]:starts[b] + lens[b]] for b in range(4)])
    l2 = lens - half
    s2 = np.cumsum(l2) - l2
    oc2 = R.chunked_prefill_attention(q2, case.arena, case.lay, case.block_table, case.seq_ids,
                                      s2, l2, half, D ** -0.5, 0, out_dtype=np.float64)
    want2 = np.concatenate([o[starts[b] + half[b]:starts[b] + lens[b]] for b in range(4)])
    assert np.abs(oc2 - want2).max() < 1e-12
