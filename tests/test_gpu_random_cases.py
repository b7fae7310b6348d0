"""Seeded random cases of the attention and append operators against the CPU oracle.

Every case draws its own shapes: group size, batch, lengths (with the block-boundary values
15/16/17 and length 1 mixed in), pool size and permutation, layer, split policy, kernel
variant.  Attention within max-abs 2e-3 / max-rel 1e-2 of the oracle; appends bit-exact.
"""
import os

import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, kernel_variant, to_gpu
from morphserve_amd import (_capi, build_infer_state, chunked_prefill_attention, decode_append_and_attend,
                            paged_attention, prefill_attention, store_kvcache)
from morphserve_amd.worker.kernels import paged_attn as PA

pytestmark = pytest.mark.gpu

# MORPHKV_RANDOM_CASES_SCALE=k multiplies the number of seeds per test (a one-off soak; the default run keeps 1)
SCALE = max(1, int(os.environ.get("MORPHKV_RANDOM_CASES_SCALE", "1")))

HEADS = [(1, 1), (4, 4), (4, 2), (8, 2), (6, 2), (8, 1), (16, 2), (5, 1), (7, 1), (16, 1)]


def _lens(rng, n, hi):
    special = np.array([1, 15, 16, 17, 31, 32, 33, 64, 127, 128, 129])
    out = rng.integers(1, hi + 1, size=n)
    pick = rng.random(n) < 0.3
    out[pick] = rng.choice(special[special <= hi], size=int(pick.sum()))
    return out.astype(np.int64)


@pytest.mark.parametrize("seed", range(24 * SCALE))
def test_random_decode_attention(cuda, seed):
    rng = np.random.default_rng(1000 + seed)
    Hq, Hkv = HEADS[int(rng.integers(len(HEADS)))]
    n = int(rng.integers(1, 9))
    lens = _lens(rng, n, int(rng.choice([40, 300, 2500])))
    L = int(rng.integers(1, 4))
    layer = int(rng.integers(L))
    nblk = int(((lens + 15) // 16).sum() + rng.integers(0, 9))
    case = make_case(seed, L, Hq, Hkv, lens.tolist(), num_blocks=nblk, fill="all" if seed % 2 else "live")
    q = rand_f16(rng, n, Hq, 128)
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), Hkv, 128)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    old = (PA.SPLIT_POLICY, PA.TARGET_WORKGROUPS)
    G = Hq // Hkv
    variant = int(rng.choice([0, 1, 2])) if G in (1, 2, 4, 8) else 0      # 0: the product library and its choice
    PA.SPLIT_POLICY = str(rng.choice(["auto", "reference"]))
    PA.TARGET_WORKGROUPS = int(rng.choice([1, 64, 512, 100000]))
    try:
        with kernel_variant(decode=variant):
            paged_attention(torch.from_numpy(q).to(cuda), kc, vc, [], [], bt, model, engine, st, layer, o)
    finally:
        PA.SPLIT_POLICY, PA.TARGET_WORKGROUPS = old
    torch.cuda.synchronize()
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, case.seq_lens, 128 ** -0.5, layer)
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), want,
                      f"seed {seed}: Hq={Hq} Hkv={Hkv} lens={lens.tolist()} layer={layer}/{L} variant={variant}")


@pytest.mark.parametrize("seed", range(12 * SCALE))
def test_random_fused_append_and_attend(cuda, seed):
    """One launch appends token len-1 and attends: cache bytes bit-exact, output within tolerance."""
    rng = np.random.default_rng(2000 + seed)
    Hq, Hkv = HEADS[int(rng.integers(len(HEADS)))]
    n = int(rng.integers(1, 9))
    lens = _lens(rng, n, int(rng.choice([40, 300, 1500])))
    L = int(rng.integers(1, 3))
    layer = int(rng.integers(L))
    nblk = int(((lens + 15) // 16).sum() + rng.integers(0, 5))
    case = make_case(seed, L, Hq, Hkv, lens.tolist(), num_blocks=nblk, fill="all")
    q = rand_f16(rng, n, Hq, 128)
    k = rand_f16(rng, n, Hkv, 128)
    v = rand_f16(rng, n, Hkv, 128)
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), Hkv, 128)
    o = torch.full((n, Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    old = PA.TARGET_WORKGROUPS
    PA.TARGET_WORKGROUPS = int(rng.choice([1, 512, 100000]))
    try:
        decode_append_and_attend(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                                 torch.from_numpy(q).to(cuda), kc, vc, [], [], bt, model, engine, st, layer, o)
    finally:
        PA.TARGET_WORKGROUPS = old
    torch.cuda.synchronize()
    R.append_decode(case.arena, case.lay, k, v, case.block_table, case.seq_ids, case.seq_lens, layer)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    want = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, case.seq_lens, 128 ** -0.5, layer)
    assert_attn_close(o.cpu().numpy().reshape(n, Hq, 128), want, f"seed {seed}: Hq={Hq} Hkv={Hkv} lens={lens.tolist()}")


@pytest.mark.parametrize("seed", range(12 * SCALE))
def test_random_prefill_and_chunked_prefill(cuda, seed):
    rng = np.random.default_rng(3000 + seed)
    Hq, Hkv = HEADS[int(rng.integers(len(HEADS)))]
    n = int(rng.integers(1, 6))
    lens = _lens(rng, n, int(rng.choice([40, 200, 700, 1300])))
    # workgroup shape and tile pairing: the library's choice, or pinned (small grids never pick the paired and the
    # 256-row shapes by themselves): bits 0-7 waves, bits 8-9 pairing forced on (1) / off (2)
    variant = int(rng.choice([0, 4 | (1 << 8), 4 | (2 << 8), 8 | (1 << 8), 8 | (2 << 8)]))
    with kernel_variant(prefill=variant):
        _random_prefill_case(cuda, seed, rng, Hq, Hkv, n, lens, variant)


def _random_prefill_case(cuda, seed, rng, Hq, Hkv, n, lens, variant):
    T = int(lens.sum())
    q = rand_f16(rng, T, Hq, 128)
    k = rand_f16(rng, T, Hkv, 128)
    v = rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - lens
    model = Cfg(num_layers=1, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=128)
    engine = Cfg(block_size=16, max_blocks_per_seq=64)
    st = build_infer_state(lens.tolist(), list(range(n)), [], Hkv, 128)
    o = torch.full((T, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    prefill_attention(torch.from_numpy(q).to(cuda), torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                      o, model, engine, st)
    torch.cuda.synchronize()
    want = R.prefill_attention(q, k, v, starts, lens, 128 ** -0.5, math="np32")
    assert_attn_close(o.cpu().numpy(), want, f"seed {seed}: prefill Hq={Hq} Hkv={Hkv} lens={lens.tolist()} variant={variant}")

    # the same prompts cut at a random point: the tail as a chunk over the cached head
    L = 2
    nblk = int(((lens + 15) // 16).sum() + 3)
    case = make_case(seed, L, Hq, Hkv, lens.tolist(), num_blocks=nblk, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    model2, engine2 = configs(case)
    st_all = build_infer_state(lens.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt, model2, engine2,
                  st_all, 1)
    R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, 1)
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    prefix = np.array([int(rng.integers(0, x)) for x in lens])          # 0 <= prefix < len: chunk never empty
    l2 = lens - prefix
    s2 = np.cumsum(l2) - l2
    q2 = np.concatenate([q[starts[b] + prefix[b]:starts[b] + lens[b]] for b in range(n)])
    st2 = build_infer_state(l2.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    o2 = torch.full((int(l2.sum()), Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    chunked_prefill_attention(torch.from_numpy(q2).to(cuda), kc, vc, [], [], bt, model2, engine2, st2, 1, o2,
                              prefix_lens=torch.from_numpy(prefix.astype(np.int32)).to(cuda))
    torch.cuda.synchronize()
    want2 = np.concatenate([want[starts[b] + prefix[b]:starts[b] + lens[b]] for b in range(n)])
    assert_attn_close(o2.cpu().numpy(), want2, f"seed {seed}: chunk over prefix {prefix.tolist()} of {lens.tolist()}")
