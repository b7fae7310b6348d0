"""GPU parity of the rotary embedding (alone and fused with the KV append) against the CPU
oracle: q and k rows bit-exact, the whole cache bit-exact against rotate-then-append."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from oracle import rope_cpu as RO
from helpers import make_case, rand_f16
from gpu_helpers import bits, configs, kernel_variant, to_gpu
from morphserve_amd import (build_infer_state, rotary_embedding_and_store_kvcache, rotary_embedding_inplace,
                            rotary_tables, store_kvcache)

pytestmark = pytest.mark.gpu


def _positions(p_lens, d_lens):
    pos = [np.arange(n) for n in p_lens] + [np.asarray([n - 1]) for n in d_lens]
    return np.concatenate(pos) if pos else np.zeros(0, dtype=np.int64)


@pytest.mark.parametrize("T,Hq,Hkv,D", [(1, 32, 8, 128), (77, 32, 32, 128), (300, 8, 2, 64), (5, 4, 4, 256)])
def test_rotary_inplace_bit_exact(cuda, T, Hq, Hkv, D):
    rng = np.random.default_rng(T)
    q, k = rand_f16(rng, T, Hq, D), rand_f16(rng, T, Hkv, D)
    ct, st = RO.rotary_tables(D, 4096)
    pos = rng.integers(0, 4096, size=T)
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st[pos])
    state = build_infer_state([], list(range(T)), [1] * T, Hkv, D)
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    qg, kg = torch.from_numpy(q).to(cuda), torch.from_numpy(k).to(cuda)
    rotary_embedding_inplace(qg, kg, state)
    RO.rotary_embedding_inplace(q, k, cos, sin)
    assert np.array_equal(bits(qg), bits(q)) and np.array_equal(bits(kg), bits(k))


def test_device_tables_match_the_oracle_tables(cuda):
    cg, sg = rotary_tables(128, 2048, 10000.0, 1.0, device="cuda")
    ct, st = RO.rotary_tables(128, 2048)
    # float32 pow / cos / sin of the two libraries differ in the last bit here and there (the
    # angle itself for large positions); after fp16 rounding under 2 % of the entries move,
    # each by one fp16 step
    dc = np.abs(cg.cpu().numpy().astype(np.float32) - ct.astype(np.float32))
    ds = np.abs(sg.cpu().numpy().astype(np.float32) - st.astype(np.float32))
    assert cg.shape == ct.shape and dc.max() <= 2 ** -10 and ds.max() <= 2 ** -10
    assert (dc > 0).mean() < 2e-2 and (ds > 0).mean() < 2e-2


@pytest.mark.parametrize("seed,L,Hq,Hkv,layer,p_lens,d_lens", [
    (0, 2, 32, 8, 1, [], [1, 16, 17, 300, 1024]),                 # decode only, GQA
    (1, 1, 32, 32, 0, [1, 15, 16, 17, 100], []),                  # prefill only, ragged
    (2, 3, 8, 4, 2, [33, 7, 129], [5, 64, 200, 17]),              # mixed batch
])
def test_fused_rotary_store_equals_rotate_then_append(cuda, seed, L, Hq, Hkv, layer, p_lens, d_lens):
    lens = list(p_lens) + list(d_lens)
    nblk = sum((x + 15) // 16 for x in lens) + 5
    case = make_case(seed, L, Hq, Hkv, lens, num_blocks=nblk, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    rng = np.random.default_rng(seed + 50)
    T = int(sum(p_lens))
    n_tok = T + len(d_lens)
    q, k, v = rand_f16(rng, n_tok, Hq, case.D), rand_f16(rng, n_tok, Hkv, case.D), rand_f16(rng, n_tok, Hkv, case.D)
    ct, st_ = RO.rotary_tables(case.D, 2048)
    pos = _positions(p_lens, d_lens)
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
    model, engine = configs(case)
    state = build_infer_state(p_lens, case.seq_ids.tolist(), d_lens, Hkv, case.D)
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    rotary_embedding_and_store_kvcache(qg, kg, vg, kc, vc, [], [], bt, model, engine, state, layer)
    # oracle: rotate, then the plain append of the rotated rows
    RO.rotary_embedding_inplace(q, k, cos, sin)
    starts = np.cumsum(p_lens) - np.asarray(p_lens) if len(p_lens) else np.zeros(0, dtype=np.int64)
    R.store_kvcache(case.arena, case.lay, k, v, case.block_table, case.seq_ids, len(p_lens), T, starts,
                    np.asarray(p_lens), np.asarray(d_lens), layer)
    torch.cuda.synchronize()
    assert np.array_equal(bits(qg), bits(q)) and np.array_equal(bits(kg), bits(k))
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    # and the two-call route of the package lands on the same bytes
    kc2, vc2, _ = to_gpu(make_case(seed, L, Hq, Hkv, lens, num_blocks=nblk, fill="all"), cuda)
    store_kvcache(kg, vg, kc2, vc2, [], [], bt, model, engine, state, layer)
    assert np.array_equal(bits(kc2), bits(kc)) and np.array_equal(bits(vc2), bits(vc))


@pytest.mark.parametrize("Hq,Hkv,variant", [(32, 32, 1), (8, 4, 1), (32, 8, 2), (64, 8, 2)])
@pytest.mark.parametrize("target_wgs", [1, 100000])
def test_decode_with_rotary_append_and_attention_in_one_launch(cuda, Hq, Hkv, variant, target_wgs):
    """q and k go in unrotated: the cache must receive exactly the rotated k row (and v), the
    output must be the attention of the rotated q over the updated cache, q and k stay as given."""
    from helpers import assert_attn_close
    from morphserve_amd import _capi, decode_rope_append_and_attend
    from morphserve_amd.worker.kernels import paged_attn as PA
    lens = [1, 16, 17, 200, 1024, 1535, 64]
    nblk = sum((x + 15) // 16 for x in lens) + 4
    layer, L = 1, 2
    case = make_case(7, L, Hq, Hkv, lens, num_blocks=nblk, fill="live")
    kc, vc, bt = to_gpu(case, cuda)
    rng = np.random.default_rng(70)
    n = len(lens)
    q, k, v = rand_f16(rng, n, Hq, case.D), rand_f16(rng, n, Hkv, case.D), rand_f16(rng, n, Hkv, case.D)
    ct, st_ = RO.rotary_tables(case.D, 2048)
    pos = np.asarray(lens) - 1
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
    model, engine = configs(case)
    state = build_infer_state([], case.seq_ids.tolist(), lens, Hkv, case.D)
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    o = torch.full((n, Hq * case.D), float("nan"), dtype=torch.float16, device=cuda)
    old = PA.TARGET_WORKGROUPS
    PA.TARGET_WORKGROUPS = target_wgs
    try:
        with kernel_variant(decode=variant):
            decode_rope_append_and_attend(kg, vg, qg, kc, vc, [], [], bt, model, engine, state, layer, o)
            torch.cuda.synchronize()
    finally:
        PA.TARGET_WORKGROUPS = old
    assert np.array_equal(bits(qg), bits(q)) and np.array_equal(bits(kg), bits(k))      # inputs untouched
    q_rot, k_rot = q.copy(), k.copy()
    RO.rotary_embedding_inplace(q_rot, k_rot, cos, sin)
    R.append_decode(case.arena, case.lay, k_rot, v, case.block_table, case.seq_ids, np.asarray(lens), layer)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    want = R.paged_attention(q_rot, case.arena, case.lay, case.block_table, case.seq_ids, np.asarray(lens),
                             case.D ** -0.5, layer)
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, case.D), np.asarray(want), "rotary + append + attention")
