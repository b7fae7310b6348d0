"""``allocate_kv_caches``: the V pool may start a few KiB into its allocation (chosen by a timing probe);
whatever it picks, the tensors are the reference's shapes, contiguous, zeroed, and every kernel sees the same
pool as with a plain allocation."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs
from morphserve_amd import ElasticKVPool, build_infer_state, decode_append_and_attend
from morphserve_amd.kv_placement import CANDIDATE_OFFSETS, allocate_kv_caches

pytestmark = pytest.mark.gpu


def test_tuned_allocation_is_a_plain_pool(cuda):
    tail = (2, 8, 16, 128)
    k, v, info = allocate_kv_caches(4096, tail, cuda, zero_init=True, tune=True)
    assert info["tuned"] and info["v_offset_bytes"] in CANDIDATE_OFFSETS
    assert set(info["probe_us_per_launch"]) == {str(x) for x in CANDIDATE_OFFSETS}
    for t in (k, v):
        assert tuple(t.shape) == (4096, *tail) and t.is_contiguous() and t.dtype == torch.float16
        assert t.data_ptr() % 4096 == 0 and not t.any()
    k2, v2, info2 = allocate_kv_caches(64, tail, cuda, tune=True)          # too small to matter: left alone
    assert not info2["tuned"] and info2["v_offset_bytes"] == 0 and v2.storage_offset() == 0
    k3, v3, info3 = allocate_kv_caches(4096, tail, cuda, tune=False)
    assert not info3["tuned"] and v3.storage_offset() == 0


@pytest.mark.parametrize("offset_bytes", [0, 4096, 20480])
def test_kernels_on_an_offset_v_pool(cuda, offset_bytes):
    """Fused append + attention on a pool whose V base sits ``offset_bytes`` into its allocation: cache bytes
    bit-exact, outputs within tolerance, and not a byte of the slack around the pool touched."""
    rng = np.random.default_rng(31 + offset_bytes)
    Hq, Hkv, L, layer = 8, 2, 2, 1
    lens = [1, 16, 17, 100, 333]
    case = make_case(3, L, Hq, Hkv, lens, num_blocks=40, fill="all")
    model, engine = configs(case)
    numel = case.k_pool.size
    kc = torch.from_numpy(case.k_pool.copy()).to(cuda)
    flat = torch.full((numel + 16384,), 7.0, dtype=torch.float16, device=cuda)
    off = offset_bytes // 2
    vc = flat[off:off + numel].view(kc.shape)
    vc.copy_(torch.from_numpy(case.v_pool.copy()).to(cuda))
    bt = torch.from_numpy(case.block_table).to(cuda)
    n = len(lens)
    q = rand_f16(rng, n, Hq, 128)
    k = rand_f16(rng, n, Hkv, 128)
    v = rand_f16(rng, n, Hkv, 128)
    st = build_infer_state([], case.seq_ids.tolist(), case.seq_lens.tolist(), Hkv, 128)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    decode_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), torch.from_numpy(q).to(cuda),
                             kc, vc, [], [], bt, model, engine, st, layer, o)
    torch.cuda.synchronize()
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, layer)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    slack = torch.cat([flat[:off], flat[off + numel:]])
    assert bool((slack == 7.0).all())
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, case.seq_lens, 128 ** -0.5, layer)
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), want, f"V offset {offset_bytes}")


def test_elastic_pool_records_its_placement(cuda):
    pool = ElasticKVPool(4096, 1, 8, 16, 128, max_seqs_in_block_table=8, max_blocks_per_seq=8, device="cuda",
                         tune_placement=True)
    assert pool.kv_placement["tuned"] and pool.v_cache.is_contiguous()
    assert pool.descriptor().v_base == pool.v_cache.data_ptr()
    plain = ElasticKVPool(4096, 1, 8, 16, 128, max_seqs_in_block_table=8, max_blocks_per_seq=8, device="cuda",
                          tune_placement=False)
    assert plain.kv_placement == {"v_offset_bytes": 0, "tuned": False} and plain.v_cache.storage_offset() == 0
    default = ElasticKVPool(4096, 1, 8, 16, 128, max_seqs_in_block_table=8, max_blocks_per_seq=8, device="cuda")
    assert default.kv_placement == {"v_offset_bytes": 0, "tuned": False}    # the probe is opt-in
