"""``attention_section``: the part of ``LlamaTransformerLayer.forward`` between the QKV and the output projection
(MorphServe/worker/layers/transformer_layer.py:93-191) -- rotary, append, prefill attention, decode attention --
against the same sequence of oracle steps: cache bytes and the in-place rotation bit-exact, ``o`` within tolerance."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from oracle import rope_cpu as RO
from helpers import assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, to_gpu
from morphserve_amd import build_infer_state
from morphserve_amd.worker.layers import attention_section

pytestmark = pytest.mark.gpu


def _positions(p_lens, d_lens):
    pos = [np.arange(n) for n in p_lens] + [np.asarray([n - 1]) for n in d_lens]
    return np.concatenate(pos) if pos else np.zeros(0, dtype=np.int64)


def _run(cuda, seed, L, Hq, Hkv, layer, p_lens, d_lens, rotary=True, keep=False, second_stream=False):
    lens = list(p_lens) + list(d_lens)
    nblk = sum((x + 15) // 16 for x in lens) + 5
    case = make_case(seed, L, Hq, Hkv, lens, num_blocks=nblk, fill="live")
    kc, vc, bt = to_gpu(case, cuda)
    rng = np.random.default_rng(seed + 9)
    P, n = int(sum(p_lens)), len(d_lens)
    T = P + n
    D = case.D
    q, k, v = rand_f16(rng, T, Hq, D), rand_f16(rng, T, Hkv, D), rand_f16(rng, T, Hkv, D)
    ct, st_ = RO.rotary_tables(D, 4096)
    pos = _positions(p_lens, d_lens)
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
    model, engine = configs(case)
    state = build_infer_state(p_lens, case.seq_ids.tolist(), d_lens, Hkv, D)
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    o = torch.full((T, Hq * D), float("nan"), dtype=torch.float16, device=cuda)
    stream = torch.cuda.Stream() if second_stream else None
    attention_section(qg, kg, vg, o, kc, vc, [], [], bt, model, engine, state, layer, rotary=rotary,
                      keep_rotated_inputs=keep, decoding_piggyback_stream=stream)
    torch.cuda.synchronize()

    q_rot, k_rot = q.copy(), k.copy()
    if rotary:
        RO.rotary_embedding_inplace(q_rot, k_rot, cos, sin)
    starts = np.cumsum(p_lens) - np.asarray(p_lens) if len(p_lens) else np.zeros(0, dtype=np.int64)
    R.store_kvcache(case.arena, case.lay, k_rot, v, case.block_table, case.seq_ids, len(p_lens), P, starts,
                    np.asarray(p_lens), np.asarray(d_lens), layer)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    one_launch = not p_lens and not keep
    if rotary and not one_launch:                           # rotated in place, as the reference leaves them
        assert np.array_equal(bits(qg), bits(q_rot)) and np.array_equal(bits(kg), bits(k_rot))
    else:
        assert np.array_equal(bits(qg), bits(q)) and np.array_equal(bits(kg), bits(k))
    got = o.cpu().numpy().reshape(T, Hq, D)
    if P:
        want = R.prefill_attention(q_rot[:P], k_rot[:P], v[:P], starts, np.asarray(p_lens), D ** -0.5, math="np32")
        assert_attn_close(got[:P], np.asarray(want), "prefill rows")
    if n:
        want = R.paged_attention(q_rot[P:], case.arena, case.lay, case.block_table, case.seq_ids[len(p_lens):],
                                 np.asarray(d_lens), D ** -0.5, layer)
        assert_attn_close(got[P:], np.asarray(want), "decode rows")


@pytest.mark.parametrize("second_stream", [False, True])
def test_mixed_batch(cuda, second_stream):
    _run(cuda, 0, 3, 32, 8, 2, [33, 7, 129, 300], [5, 64, 200, 17, 1], second_stream=second_stream)


@pytest.mark.parametrize("keep", [False, True])
def test_decode_only_batch(cuda, keep):
    _run(cuda, 1, 2, 32, 8, 1, [], [1, 16, 17, 300, 1024, 700], keep=keep)


def test_prefill_only_batch(cuda):
    _run(cuda, 2, 1, 32, 32, 0, [1, 15, 16, 17, 100, 257], [])


@pytest.mark.parametrize("p_lens,d_lens", [([40, 90], [33, 500]), ([], [100, 2, 640])])
def test_without_rotary(cuda, p_lens, d_lens):
    _run(cuda, 3, 2, 8, 4, 1, p_lens, d_lens, rotary=False)


def test_prefill_without_a_cache(cuda):
    """``ignore_kvcache`` (the forged batch of ``profile_num_blocks``, model.py:152-158): no cache, no table."""
    rng = np.random.default_rng(4)
    p_lens, Hq, Hkv, D = [64, 200, 31], 8, 8, 128
    P = sum(p_lens)
    q, k, v = rand_f16(rng, P, Hq, D), rand_f16(rng, P, Hkv, D), rand_f16(rng, P, Hkv, D)
    ct, st_ = RO.rotary_tables(D, 4096)
    pos = _positions(p_lens, [])
    cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
    state = build_infer_state(p_lens, [0, 1, 2], [], Hkv, D)
    state.ignore_kvcache = True
    state.position_cos = torch.from_numpy(cos).to(cuda)
    state.position_sin = torch.from_numpy(sin).to(cuda)
    from helpers import Cfg
    model = Cfg(num_layers=1, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=D)
    engine = Cfg(block_size=16, max_blocks_per_seq=32)
    qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
    o = torch.full((P, Hq * D), float("nan"), dtype=torch.float16, device=cuda)
    attention_section(qg, kg, vg, o, None, None, [], [], None, model, engine, state, 0)
    torch.cuda.synchronize()
    RO.rotary_embedding_inplace(q, k, cos, sin)
    starts = np.cumsum(p_lens) - np.asarray(p_lens)
    want = R.prefill_attention(q, k, v, starts, np.asarray(p_lens), D ** -0.5, math="np32")
    assert np.array_equal(bits(qg), bits(q)) and np.array_equal(bits(kg), bits(k))
    assert_attn_close(o.cpu().numpy().reshape(P, Hq, D), np.asarray(want), "prefill without a cache")


def test_serving_steps_with_the_step_builder(cuda):
    """Several engine steps in a row, each prepared by ``StepStateBuilder`` (lists -> state, positions, rotary rows,
    block allocation) and run by ``attention_section`` for every layer: prompts arrive, decode, finish and free
    their blocks.  After every step the pool bytes, the allocator state and ``o`` are checked against the oracle
    run through the same steps."""
    from gpu_helpers import assert_state_equal, manager_state
    from helpers import Cfg
    from morphserve_amd import ElasticKVPool, StepStateBuilder
    L, Hq, Hkv, D, B, NB = 2, 8, 2, 128, 16, 96
    pool = ElasticKVPool(NB, L, Hkv, B, D, max_seqs_in_block_table=8, max_blocks_per_seq=24, device="cuda")
    bm = pool.block_manager
    ob = R.BlockManagerOracle("GPU", NB, 8, 24, B)
    lay = R.plain_layout(NB, L, Hkv, B, D)
    arena = np.zeros(2 * NB * lay.block_elems, dtype=np.float16)
    ct, st_ = RO.rotary_tables(D, 1024)
    builder = StepStateBuilder(8, 1024, Hkv, D, torch.from_numpy(ct).to(cuda), torch.from_numpy(st_).to(cuda))
    model, engine = Cfg(num_layers=L, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=D), Cfg(block_size=B, max_blocks_per_seq=24)
    rng = np.random.default_rng(11)
    arrivals = {0: [(3, 37), (5, 120)], 1: [(0, 16)], 3: [(6, 75), (1, 1)], 5: [(2, 200)]}      # step -> (seq id, prompt)
    finish = {4: [5], 6: [3, 0]}
    lens = {}
    for step in range(8):
        for sid in finish.get(step, []):
            ids_t = torch.tensor([sid], dtype=torch.int32, device=cuda)
            bm.free_blocks_for_seqs(ids_t)
            ob.free_blocks_for_seqs(np.asarray([sid]))
            del lens[sid]
        new = arrivals.get(step, [])
        running = sorted(lens)
        p_lens = [n for _, n in new]
        d_lens = [lens[s] + 1 for s in running]
        ids = [s for s, _ in new] + running
        state = builder.build(p_lens, ids, d_lens, block_manager=bm)
        ob.allocate_blocks_for_seqs(np.asarray(ids), np.asarray(p_lens + d_lens))
        assert_state_equal(manager_state(bm), ob.snapshot(), f"step {step}: allocation")
        P, n = sum(p_lens), len(d_lens)
        T = P + n
        pos = _positions(p_lens, d_lens)
        cos, sin = np.ascontiguousarray(ct[pos]), np.ascontiguousarray(st_[pos])
        starts = np.cumsum(p_lens) - np.asarray(p_lens) if p_lens else np.zeros(0, dtype=np.int64)
        for layer in range(L):
            q, k, v = rand_f16(rng, T, Hq, D), rand_f16(rng, T, Hkv, D), rand_f16(rng, T, Hkv, D)
            qg, kg, vg = (torch.from_numpy(x).to(cuda) for x in (q, k, v))
            o = torch.full((T, Hq * D), float("nan"), dtype=torch.float16, device=cuda)
            attention_section(qg, kg, vg, o, pool.k_cache, pool.v_cache, pool.k_cache_new, pool.v_cache_new,
                              bm.block_table, model, engine, state, layer)
            RO.rotary_embedding_inplace(q, k, cos, sin)
            R.store_kvcache(arena, lay, k, v, ob.block_table, np.asarray(ids), len(p_lens), P, starts,
                            np.asarray(p_lens), np.asarray(d_lens), layer)
            got = o.cpu().numpy().reshape(T, Hq, D)
            if P:
                want = R.prefill_attention(q[:P], k[:P], v[:P], starts, np.asarray(p_lens), D ** -0.5, math="np32")
                assert_attn_close(got[:P], np.asarray(want), f"step {step} layer {layer}: prefill rows")
            if n:
                want = R.paged_attention(q[P:], arena, lay, ob.block_table, np.asarray(running), np.asarray(d_lens),
                                         D ** -0.5, layer)
                assert_attn_close(got[P:], np.asarray(want), f"step {step} layer {layer}: decode rows")
        half = NB * lay.block_elems
        assert np.array_equal(bits(pool.k_cache).reshape(-1), arena[:half].view(np.uint16)), f"step {step}: K pool"
        assert np.array_equal(bits(pool.v_cache).reshape(-1), arena[half:].view(np.uint16)), f"step {step}: V pool"
        for sid, n_tok in new:
            lens[sid] = n_tok
        for sid in running:
            lens[sid] += 1
