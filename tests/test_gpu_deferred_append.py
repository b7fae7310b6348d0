"""The optional deferral of store_kvcache's decode rows into the paged_attention that follows: same cache
bytes and outputs as the two launches, whichever way the pending append ends up being issued."""
import numpy as np
import pytest
import torch

import morphserve_amd as M
from oracle import ref_cpu as R
from helpers import assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, to_gpu
from morphserve_amd.worker.kernels import _deferred

pytestmark = pytest.mark.gpu


@pytest.fixture
def deferral():
    M.enable_deferred_decode_append(True)
    yield
    M.enable_deferred_decode_append(False)
    assert _deferred.pending() is None


def _setup(cuda, seed, Hq, Hkv, p_lens, d_lens, L=3):
    lens = list(p_lens) + list(d_lens)
    nblk = sum((x + 15) // 16 for x in lens) + 4
    case = make_case(seed, L, Hq, Hkv, lens, num_blocks=nblk, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    rng = np.random.default_rng(seed)
    T = int(sum(p_lens))
    k = rand_f16(rng, T + len(d_lens), Hkv, 128)
    v = rand_f16(rng, T + len(d_lens), Hkv, 128)
    q = rand_f16(rng, len(d_lens), Hq, 128)
    model, engine = configs(case)
    st = M.build_infer_state(p_lens, case.seq_ids.tolist(), d_lens, Hkv, 128)
    return case, kc, vc, bt, k, v, q, model, engine, st, T


def _oracle_store(case, k, v, p_lens, d_lens, T, layer):
    starts = np.cumsum(p_lens) - np.asarray(p_lens) if len(p_lens) else np.zeros(0, dtype=np.int64)
    R.store_kvcache(case.arena, case.lay, k, v, case.block_table, case.seq_ids, len(p_lens), T, starts,
                    np.asarray(p_lens), np.asarray(d_lens), layer)


@pytest.mark.parametrize("Hq,Hkv,p_lens,d_lens", [(32, 8, [], [1, 16, 17, 300, 1024]), (8, 8, [33, 7], [5, 64, 200])])
def test_deferred_rows_are_appended_by_the_attention_launch(cuda, deferral, Hq, Hkv, p_lens, d_lens):
    case, kc, vc, bt, k, v, q, model, engine, st, T = _setup(cuda, 41, Hq, Hkv, p_lens, d_lens)
    layer = 1
    kg, vg = torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda)
    before_k = bits(kc).copy()
    M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, layer)
    torch.cuda.synchronize()
    assert _deferred.pending() is not None
    # only the prefill rows have been written so far
    ref = make_case(41, 3, Hq, Hkv, list(p_lens) + list(d_lens), num_blocks=case.num_blocks, fill="all")
    if p_lens:
        starts = np.cumsum(p_lens) - np.asarray(p_lens)
        R.append_prefill(ref.arena, ref.lay, k[:T], v[:T], ref.block_table, ref.seq_ids[:len(p_lens)], starts,
                         np.asarray(p_lens), layer)
        assert np.array_equal(bits(kc), bits(ref.k_pool))
    else:
        assert np.array_equal(bits(kc), before_k)
    n = len(d_lens)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    M.paged_attention(torch.from_numpy(q).to(cuda), kc, vc, [], [], bt, model, engine, st, layer, o)
    torch.cuda.synchronize()
    assert _deferred.pending() is None
    _oracle_store(case, k, v, p_lens, d_lens, T, layer)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids[len(p_lens):],
                             np.asarray(d_lens), 128 ** -0.5, layer)
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), want, "deferred append + attention")


def test_every_other_route_issues_the_pending_append(cuda, deferral):
    d_lens = [40, 129, 16]
    case, kc, vc, bt, k, v, q, model, engine, st, T = _setup(cuda, 43, 8, 2, [], d_lens)
    kg, vg, qg = (torch.from_numpy(x).to(cuda) for x in (k, v, q))
    o = torch.empty((3, 8 * 128), dtype=torch.float16, device=cuda)
    # (1) an explicit flush
    M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 0)
    M.flush_pending_appends()
    # (2) the next store_kvcache (another layer) issues the previous one
    M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 1)
    M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 2)
    # (3) an attention call for a DIFFERENT layer issues it, then attends without appending
    M.paged_attention(qg, kc, vc, [], [], bt, model, engine, st, 0, o)
    torch.cuda.synchronize()
    assert _deferred.pending() is None
    for layer in range(3):
        R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, np.asarray(d_lens), layer)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, np.asarray(d_lens), 128 ** -0.5, 0)
    assert_attn_close(o.cpu().numpy().reshape(3, 8, 128), want, "attention after a flushed append")
    # (4) switching the deferral off issues what is pending
    M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 1)
    M.enable_deferred_decode_append(False)
    assert _deferred.pending() is None
    M.enable_deferred_decode_append(True)


def test_deferred_append_consumed_on_another_stream_and_in_a_graph(cuda, deferral):
    """The reference runs paged_attention on a side stream after an event (transformer_layer.py:177-191); and
    a captured step replays to the same cache bytes and outputs."""
    d_lens = [700, 33, 1024, 5]
    case, kc, vc, bt, k, v, q, model, engine, st, T = _setup(cuda, 47, 32, 8, [], d_lens, L=2)
    kg, vg, qg = (torch.from_numpy(x).to(cuda) for x in (k, v, q))
    o = torch.full((4, 32 * 128), float("nan"), dtype=torch.float16, device=cuda)
    side = torch.cuda.Stream()
    M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 1)
    ev = torch.cuda.Event()
    ev.record()
    with torch.cuda.stream(side):
        side.wait_event(ev)
        M.paged_attention(qg, kc, vc, [], [], bt, model, engine, st, 1, o)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, np.asarray(d_lens), 1)
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, np.asarray(d_lens), 128 ** -0.5, 1)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    assert_attn_close(o.cpu().numpy().reshape(4, 32, 128), want, "side stream")
    eager = o.clone()
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            M.store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 1)
            M.paged_attention(qg, kc, vc, [], [], bt, model, engine, st, 1, o)
    for _ in range(3):
        o.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, eager)
        assert np.array_equal(bits(kc), bits(case.k_pool))
