"""GPU parity of KV append (store_kvcache) against the CPU oracle: the whole
cache must be bit-identical, plain pool and extension segments alike."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, make_case, rand_f16
from gpu_helpers import bits, configs, to_gpu
from morphserve_amd import build_infer_state, store_kvcache

pytestmark = pytest.mark.gpu


def _run_mixed(case, dev, p_lens, d_lens, layer, seed):
    rng = np.random.default_rng(seed)
    T = int(np.sum(p_lens))
    n_dec = len(d_lens)
    k = rand_f16(rng, T + n_dec, case.Hkv, case.D)
    v = rand_f16(rng, T + n_dec, case.Hkv, case.D)
    starts = np.cumsum(p_lens) - p_lens if len(p_lens) else np.zeros(0, dtype=np.int64)
    R.store_kvcache(case.arena, case.lay, k, v, case.block_table, case.seq_ids, len(p_lens), T,
                    starts, np.asarray(p_lens), np.asarray(d_lens), layer)
    return k, v


@pytest.mark.parametrize("seed,L,Hkv,layer,p_lens,d_lens", [
    (0, 1, 32, 0, [], [64, 65, 100, 288, 300, 400, 445, 512]),          # decode only, MHA shapes
    (1, 4, 8, 3, [], [1, 16, 17, 1024, 1535]),                          # GQA kv heads, block edges
    (2, 2, 8, 1, [1, 15, 16, 17, 100, 512], []),                        # prefill only, ragged
    (3, 3, 4, 2, [33, 7, 129], [5, 64, 200, 17]),                       # mixed batch
    (4, 1, 2, 0, [], [7]),                                              # single sequence
])
def test_store_kvcache_bit_exact(cuda, seed, L, Hkv, layer, p_lens, d_lens):
    lens = list(p_lens) + list(d_lens)
    nblk = sum((x + 15) // 16 for x in lens) + 9
    case = make_case(seed, L, Hkv, Hkv, lens, num_blocks=nblk, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    k, v = _run_mixed(case, cuda, p_lens, d_lens, layer, seed)      # oracle mutates case.arena
    model, engine = configs(case)
    st = build_infer_state(p_lens, case.seq_ids.tolist(), d_lens, Hkv, case.D)
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt,
                  model, engine, st, layer)
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool))
    assert np.array_equal(bits(vc), bits(case.v_pool))


def test_store_kvcache_empty_batch(cuda):
    case = make_case(5, 1, 2, 2, [16], num_blocks=4, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state([], [], [], 2, case.D)
    e = torch.empty(0, 2, case.D, dtype=torch.float16, device=cuda)
    store_kvcache(e, e, kc, vc, [], [], bt, model, engine, st, 0)
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool))


def test_store_kvcache_offset_views(cuda):
    """Arguments are routinely offset views; decode rows are the tail slice."""
    case = make_case(6, 2, 4, 4, [40, 3, 70], num_blocks=16, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    rng = np.random.default_rng(6)
    k = rand_f16(rng, 5 + 3, 4, case.D)
    v = rand_f16(rng, 5 + 3, 4, case.D)
    R.append_decode(case.arena, case.lay, k[5:], v[5:], case.block_table, case.seq_ids, case.seq_lens, 1)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), case.seq_lens.tolist(), 4, case.D)
    kg = torch.from_numpy(k).to(cuda)[5:]
    vg = torch.from_numpy(v).to(cuda)[5:]
    store_kvcache(kg, vg, kc, vc, [], [], bt, model, engine, st, 1)
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))


def _segment_setup(cuda, seed, L, Hkv, org, S, nseg, D=128, B=16):
    """One device arena laid out like the reference's memory: extension segments
    at descending addresses one 'weight layer' apart, base pools behind them."""
    rng = np.random.default_rng(seed)
    blk = L * Hkv * B * D
    stride = 2 * S * blk + 4096               # elements between consecutive segments
    seg0 = (nseg - 1) * stride
    base_k = seg0 + 2 * S * blk + 512
    base_v = base_k + org * blk
    total = base_v + org * blk
    arena = rng.standard_normal(total, dtype=np.float32).astype(np.float16)
    lay = R.PoolLayout(L, Hkv, B, D, k_base=base_k, v_base=base_v, num_blocks_org=org,
                       seg_blocks=S, k_new0=seg0, v_new0=seg0 + S * blk, org_layer_param_size=stride)
    g = torch.from_numpy(arena.copy()).to(cuda)
    shape = (L, Hkv, B, D)
    kc = g[base_k:base_k + org * blk].view(org, *shape)
    vc = g[base_v:base_v + org * blk].view(org, *shape)
    k_new, v_new = [], []
    for j in range(nseg):
        o = seg0 - j * stride
        k_new.append(g[o:o + S * blk].view(S, *shape))
        v_new.append(g[o + S * blk:o + 2 * S * blk].view(S, *shape))
    return arena, lay, g, kc, vc, k_new, v_new, stride


def test_store_kvcache_segments_bit_exact(cuda):
    L, Hkv, org, S, nseg = 2, 4, 6, 4, 3
    arena, lay, g, kc, vc, k_new, v_new, stride = _segment_setup(cuda, 7, L, Hkv, org, S, nseg)
    rng = np.random.default_rng(7)
    total = org + nseg * S
    order = rng.permutation(total)
    p_lens, d_lens = [40, 16], [33, 100, 1]
    lens = p_lens + d_lens
    table = np.full((8, 8), -1, dtype=np.int32)
    seq_ids = np.array([5, 2, 7, 0, 3], dtype=np.int32)
    pos = 0
    for s, n in zip(seq_ids, lens):
        nb = (n + 15) // 16
        table[s, :nb] = order[pos:pos + nb]
        pos += nb
    T = sum(p_lens)
    k = rand_f16(rng, T + len(d_lens), Hkv, 128)
    v = rand_f16(rng, T + len(d_lens), Hkv, 128)
    starts = np.cumsum(p_lens) - np.asarray(p_lens)
    R.store_kvcache(arena, lay, k, v, table, seq_ids, 2, T, starts, np.asarray(p_lens),
                    np.asarray(d_lens), 1)
    model = Cfg(num_layers=L, num_q_heads=Hkv, num_kv_heads=Hkv, head_dim=128)
    engine = Cfg(block_size=16, max_blocks_per_seq=8)
    st = build_infer_state(p_lens, seq_ids.tolist(), d_lens, Hkv, 128, num_blocks_org=org,
                           kv_cache_new_block_size=S, org_layer_param_size=stride)
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, k_new, v_new,
                  torch.from_numpy(table).to(cuda), model, engine, st, 1)
    torch.cuda.synchronize()
    # the WHOLE arena, padding between segments included, must match the oracle's
    assert np.array_equal(bits(g), bits(arena))
