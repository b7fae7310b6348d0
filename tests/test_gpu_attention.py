"""GPU parity of paged decode attention against the CPU oracle.

Tolerance of the path (fp16 output, fp32 accumulation): every element within
max-abs 2e-3 and, where the oracle's value is at least 0.2 in magnitude, max-rel 1e-2 of the oracle's fp32
torch-CPU result (``helpers.assert_attn_close``).
"""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, kernel_variant, to_gpu
from morphserve_amd import _capi, build_infer_state, paged_attention, store_kvcache
from morphserve_amd.worker.kernels import paged_attn as PA

pytestmark = pytest.mark.gpu


def _attend(case, dev, q, layer, policy="auto", target_wgs=None, k_new=(), v_new=(), st=None,
            tensors=None, variant=0):
    kc, vc, bt = tensors if tensors is not None else to_gpu(case, dev)
    model, engine = configs(case)
    if st is None:
        st = build_infer_state([], case.seq_ids.tolist(), case.seq_lens.tolist(), case.Hkv, case.D)
    n = len(case.seq_lens)
    # o arrives 2-D [n, Hq*D] in the reference's layer (a row slice of the hidden state)
    o = torch.full((n, case.Hq * case.D), float("nan"), dtype=torch.float16, device=dev)
    old = (PA.SPLIT_POLICY, PA.TARGET_WORKGROUPS)
    PA.SPLIT_POLICY = policy
    if target_wgs is not None:
        PA.TARGET_WORKGROUPS = target_wgs
    try:
        with kernel_variant(decode=variant):                    # 0 auto, 1 vector ALU, 2 matrix cores
            paged_attention(torch.from_numpy(q).to(dev), kc, vc, list(k_new), list(v_new), bt, model,
                            engine, st, layer, o)
    finally:
        PA.SPLIT_POLICY, PA.TARGET_WORKGROUPS = old
    torch.cuda.synchronize()
    return o.cpu().numpy().reshape(n, case.Hq, case.D)


def _oracle(case, q, layer):
    return R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids,
                             case.seq_lens, case.D ** -0.5, layer)


@pytest.mark.parametrize("Hq,Hkv", [(6, 2), (5, 1), (12, 2), (28, 4), (32, 2), (9, 1), (20, 2), (11, 1), (24, 2), (13, 1),
                                    (14, 1), (15, 1)])
@pytest.mark.parametrize("target_wgs", [1, 100000])
def test_decode_attention_other_group_sizes(cuda, Hq, Hkv, target_wgs):
    """Groups of 3, 5, 6, 7 and 9 to 16 query heads per kv head (matrix-core kernel)."""
    rng = np.random.default_rng(Hq)
    lens = [1, 16, 17, 100, 1024, 1300]
    nblk = sum((x + 15) // 16 for x in lens) + 3
    case = make_case(Hq, 2, Hq, Hkv, lens, num_blocks=nblk, fill="live")
    q = rand_f16(rng, len(lens), Hq, 128)
    assert_attn_close(_attend(case, cuda, q, 1, target_wgs=target_wgs), _oracle(case, q, 1), f"G={Hq // Hkv}")
    with pytest.raises(_capi.MorphKVError, match="group size"):
        bad = make_case(1, 1, 17, 1, [16], num_blocks=4, fill="live")
        _attend(bad, cuda, rand_f16(rng, 1, 17, 128), 0)


@pytest.mark.parametrize("Hq,Hkv,variant", [(8, 2, 0), (4, 4, 1)])
def test_decode_attention_many_splits(cuda, Hq, Hkv, variant):
    """Long contexts cut into 47 and 105 splits (more than one 64-split chunk of the merge
    kernel), next to sequences that use one or two of the launched splits."""
    rng = np.random.default_rng(11)
    for lens in ([9000, 300, 5000, 1], [20000, 16, 129]):
        tps, splits = PA.choose_split(len(lens), Hkv, max(lens), 16, target_wgs=100000)
        assert splits > 8 and (max(lens) < 10000 or splits > 64)
        nblk = sum((x + 15) // 16 for x in lens) + 5
        case = make_case(len(lens), 2, Hq, Hkv, lens, num_blocks=nblk, fill="live")
        q = rand_f16(rng, len(lens), Hq, 128)
        assert_attn_close(_attend(case, cuda, q, 1, target_wgs=100000, variant=variant), _oracle(case, q, 1),
                          f"{splits} splits")


@pytest.mark.parametrize("Hq,Hkv", [(32, 32), (8, 4), (32, 8), (64, 8)])
@pytest.mark.parametrize("policy", ["auto", "reference"])
@pytest.mark.parametrize("variant", [1, 2])
def test_decode_attention_group_sizes(cuda, Hq, Hkv, policy, variant):
    rng = np.random.default_rng(Hq * 100 + Hkv)
    lens = [1, 2, 15, 16, 17, 63, 64, 65, 100, 333, 512, 777]
    nblk = sum((x + 15) // 16 for x in lens) + 5
    case = make_case(Hq + Hkv, 2, Hq, Hkv, lens, num_blocks=nblk, fill="all")
    q = rand_f16(rng, len(lens), Hq, case.D)
    got = _attend(case, cuda, q, 1, policy=policy, variant=variant)
    assert_attn_close(got, _oracle(case, q, 1), f"Hq={Hq} Hkv={Hkv} {policy} variant={variant}")


def test_decode_attention_closed_forms(cuda):
    rng = np.random.default_rng(3)
    case = make_case(3, 1, 8, 2, [1, 40, 200], num_blocks=20, fill="all")
    # sequence 1: identical keys -> uniform weights -> mean of V
    s1 = case.seq_ids[1]
    for j in range(3):
        case.k_pool[case.block_table[s1, j], 0] = case.k_pool[case.block_table[s1, 0], 0, :, :1, :]
    q = rand_f16(rng, 3, 8, case.D)
    q[2, 1] = q[2, 0]
    got = _attend(case, cuda, q, 0)
    s0 = case.seq_ids[0]
    v0 = case.v_pool[case.block_table[s0, 0], 0, :, 0, :]
    assert np.array_equal(bits(got[0]), bits(np.repeat(v0, 4, axis=0))), "len 1 must return V[0] exactly"
    _, vs = R.gather_kv(case.arena, case.lay, case.block_table, s1, 40, 0)
    mean_v = np.repeat(vs[:, :40].astype(np.float64).mean(axis=1), 4, axis=0)
    assert np.abs(got[1].astype(np.float64) - mean_v).max() < 1e-3
    assert np.array_equal(bits(got[2, 0]), bits(got[2, 1])), "equal q in one group must give equal o"


def test_decode_attention_tail_garbage_is_masked(cuda):
    """NaN / Inf bytes beyond len in the last block must not reach the output."""
    rng = np.random.default_rng(4)
    case = make_case(4, 1, 8, 2, [21, 130], num_blocks=16, fill="all")
    q = rand_f16(rng, 2, 8, case.D)
    want = _oracle(case, q, 0)
    for i, n in enumerate(case.seq_lens):
        last = case.block_table[case.seq_ids[i], (n - 1) // 16]
        case.k_pool[last, 0, :, n % 16:, :] = np.float16("nan")
        case.v_pool[last, 0, :, n % 16:, :] = np.float16("inf")
    for variant in (1, 2):
        got = _attend(case, cuda, q, 0, variant=variant)
        assert_attn_close(got, want, f"garbage tail variant={variant}")


def test_decode_attention_split_and_permutation_invariance(cuda):
    rng = np.random.default_rng(5)
    lens = [1500, 1024, 1281, 16, 700]
    nblk = sum((x + 15) // 16 for x in lens) + 3
    q = rand_f16(rng, len(lens), 32, 128)
    outs = []
    for permute in (True, False):
        case = make_case(5, 1, 32, 8, lens, num_blocks=nblk, permute=permute, fill="live")
        # same logical content in both layouts
        rr = np.random.default_rng(55)
        T = sum(lens)
        k = rand_f16(rr, T, 8, 128)
        v = rand_f16(rr, T, 8, 128)
        starts = np.cumsum(lens) - np.asarray(lens)
        R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts,
                         np.asarray(lens), 0)
        want = _oracle(case, q, 0)
        for wgs in (1, 64, 1536, 100000):
            for variant in (1, 2):
                got = _attend(case, cuda, q, 0, target_wgs=wgs, variant=variant)
                assert_attn_close(got, want, f"permute={permute} target_wgs={wgs} variant={variant}")
                outs.append(got)
    for o in outs[1:]:
        assert np.abs(o.astype(np.float64) - outs[0].astype(np.float64)).max() <= 2e-3


def test_decode_attention_config1_full_size(cuda):
    """Llama-2-7B-shaped layer: MHA 32 heads, pool of 4096 blocks, batch 8,
    contexts uniform in [64, 512]; append one token per sequence, then attend."""
    rng = np.random.default_rng(1)
    lens = rng.integers(64, 513, size=8)
    case = make_case(1, 1, 32, 32, lens, num_blocks=4096, max_seqs=16, max_blocks_per_seq=64, fill="live")
    kc, vc, bt = to_gpu(case, cuda)
    q = rand_f16(rng, 8, 32, 128)
    k = rand_f16(rng, 8, 32, 128)
    v = rand_f16(rng, 8, 32, 128)
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, 0)
    want = _oracle(case, q, 0)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), case.seq_lens.tolist(), 32, 128)
    assert (st.seq_block_size, st.num_seq_blocks) == R.select_seq_block_size(32, lens.tolist())
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt,
                  model, engine, st, 0)
    got = _attend(case, cuda, q, 0, st=st, tensors=(kc, vc, bt))
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    assert_attn_close(got, want, "config 1")


def test_decode_attention_config2_batch_one_layer(cuda):
    """Llama-3-8B GQA shapes at the full batch (64 sequences, contexts in
    [1024, 1536]), one layer of a 32-layer cache, pool holding the live blocks."""
    rng = np.random.default_rng(2)
    lens = rng.integers(1024, 1537, size=64)
    nblk = int(((lens + 15) // 16).sum()) + 64
    L, layer = 2, 1
    case = make_case(2, L, 32, 8, lens, num_blocks=nblk, max_seqs=128, max_blocks_per_seq=128, fill="live")
    q = rand_f16(rng, 64, 32, 128)
    got = _attend(case, cuda, q, layer)
    assert_attn_close(got, _oracle(case, q, layer), "config 2 batch")


@pytest.mark.parametrize("Hq,Hkv", [(32, 32), (32, 8), (64, 8), (28, 4), (6, 2), (32, 2)])
@pytest.mark.parametrize("variant", [1, 2])
@pytest.mark.parametrize("target_wgs", [1, 100000])
def test_fused_append_and_attend(cuda, Hq, Hkv, variant, target_wgs):
    """One launch per layer doing store_kvcache + paged_attention: the cache must
    end up bit-identical to the oracle's append, the output within tolerance, for
    last-token slots at every position of a block (first, last, middle)."""
    from morphserve_amd import decode_append_and_attend
    rng = np.random.default_rng(Hq + variant)
    lens = [1, 2, 16, 17, 32, 33, 48, 100, 255, 256, 257, 1000]
    nblk = sum((x + 15) // 16 for x in lens) + 4
    case = make_case(Hq * 7 + Hkv, 2, Hq, Hkv, lens, num_blocks=nblk, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    n = len(lens)
    q = rand_f16(rng, n, Hq, case.D)
    k = rand_f16(rng, n, Hkv, case.D)
    v = rand_f16(rng, n, Hkv, case.D)
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, 1)
    want = _oracle(case, q, 1)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), case.seq_lens.tolist(), case.Hkv, case.D)
    o = torch.full((n, Hq * case.D), float("nan"), dtype=torch.float16, device=cuda)
    old = PA.TARGET_WORKGROUPS
    PA.TARGET_WORKGROUPS = target_wgs
    try:
        with kernel_variant(decode=variant):
            decode_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                                     torch.from_numpy(q).to(cuda), kc, vc, [], [], bt, model, engine, st, 1, o)
    finally:
        PA.TARGET_WORKGROUPS = old
    torch.cuda.synchronize()
    assert np.array_equal(bits(kc), bits(case.k_pool)), "K cache after the fused append"
    assert np.array_equal(bits(vc), bits(case.v_pool)), "V cache after the fused append"
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, case.D), want, "fused append + attention")
