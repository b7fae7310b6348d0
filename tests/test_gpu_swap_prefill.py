"""GPU parity of block eviction (swap_blocks) and of prefill attention."""
import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import Cfg, assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, kernel_variant, to_gpu
from morphserve_amd import (_capi, build_infer_state, chunked_prefill_attention, prefill_attention,
                            store_kvcache, swiftllm_c)
from test_gpu_append import _segment_setup

pytestmark = pytest.mark.gpu


def test_swap_out_in_bit_exact(cuda):
    case = make_case(9, 2, 4, 4, [40, 20, 100], num_blocks=24, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    n_cpu = 12
    k_swap = torch.zeros((n_cpu, 2, 4, 16, 128), dtype=torch.float16)      # pageable host memory
    v_swap = torch.zeros_like(k_swap)
    ks_np = np.zeros(k_swap.shape, dtype=np.float16)
    vs_np = np.zeros_like(ks_np)
    s = case.seq_ids[2]
    src = case.block_table[s, :7].astype(np.int64).tolist()
    dst = [3, 4, 5, 6, 9, 10, 0]
    copies = swiftllm_c.swap_blocks(src, dst, False, kc, vc, k_swap, v_swap)
    torch.cuda.synchronize()
    R.swap_blocks(case.arena, case.lay, ks_np, vs_np, src, dst, False)
    assert np.array_equal(bits(k_swap), bits(ks_np)) and np.array_equal(bits(v_swap), bits(vs_np))
    assert copies == len(R.coalesce_runs(src, dst))
    # bring them back into other blocks (ascending free ids, as the allocator would give)
    free = np.nonzero(case.is_free)[0][:7].astype(np.int64).tolist()
    copies = swiftllm_c.swap_blocks(dst, free, True, kc, vc, k_swap, v_swap)
    torch.cuda.synchronize()
    R.swap_blocks(case.arena, case.lay, ks_np, vs_np, dst, free, True)
    assert copies == len(R.coalesce_runs(dst, free))
    assert np.array_equal(bits(kc), bits(case.k_pool)) and np.array_equal(bits(vc), bits(case.v_pool))
    assert swiftllm_c.swap_blocks([], [], True, kc, vc, k_swap, v_swap) == 0


def test_swap_with_segments_round_trip(cuda):
    """The reference's calling convention: only segment 0 is passed, later segments
    sit one 'weight layer' below each other; swap-in must address the TARGET id."""
    L, Hkv, org, S, nseg = 2, 2, 6, 4, 3
    arena, lay, g, kc, vc, k_new, v_new, stride = _segment_setup(cuda, 12, L, Hkv, org, S, nseg)
    n_cpu = 10
    k_swap = torch.zeros((n_cpu, L, Hkv, 16, 128), dtype=torch.float16)
    v_swap = torch.zeros_like(k_swap)
    ks_np = np.zeros(k_swap.shape, dtype=np.float16)
    vs_np = np.zeros_like(ks_np)
    src = [4, 5, 6, 7, 9, 10, 15, 17]        # base ids, segment 0, crossing into segment 1 and 2
    dst = [0, 1, 2, 3, 4, 5, 6, 7]
    flags = [-1 if b < org else (b - org) // S for b in src]
    copies = swiftllm_c.swap_blocks_new_kv_combined(src, dst, False, org, stride, S, 2, kc, vc,
                                                    k_swap, v_swap, k_new[0], v_new[0])
    torch.cuda.synchronize()
    R.swap_blocks(arena, lay, ks_np, vs_np, src, dst, False)
    assert np.array_equal(bits(k_swap), bits(ks_np)) and np.array_equal(bits(v_swap), bits(vs_np))
    assert copies == len(R.coalesce_runs(src, dst, src_seg=flags))
    back = [16, 2, 3, 12, 13, 14, 0, 8]      # different targets, segments included
    swiftllm_c.swap_blocks_new_kv_combined(dst, back, True, org, stride, S, 2, kc, vc,
                                           k_swap, v_swap, k_new[0], v_new[0])
    torch.cuda.synchronize()
    R.swap_blocks(arena, lay, ks_np, vs_np, dst, back, True)
    assert np.array_equal(bits(g), bits(arena))
    with pytest.raises(RuntimeError):
        swiftllm_c.swap_blocks([org + 5], [0], False, kc, vc, k_swap, v_swap)   # id outside the base pool


@pytest.mark.parametrize("Hq,Hkv,lens", [(4, 4, [1, 9, 16, 17, 63, 64, 65, 200]), (8, 2, [512, 130, 5]),
                                         (32, 32, [512])])
def test_prefill_attention_parity(cuda, Hq, Hkv, lens):
    rng = np.random.default_rng(Hq + len(lens))
    T = sum(lens)
    q = rand_f16(rng, T, Hq, 128)
    k = rand_f16(rng, T, Hkv, 128)
    v = rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - np.asarray(lens)
    want = R.prefill_attention(q, k, v, starts, np.asarray(lens), 128 ** -0.5, math="np32")
    model = Cfg(num_layers=1, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=128)
    engine = Cfg(block_size=16, max_blocks_per_seq=64)
    st = build_infer_state(lens, list(range(len(lens))), [], Hkv, 128)
    o = torch.full((T, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    prefill_attention(torch.from_numpy(q).to(cuda), torch.from_numpy(k).to(cuda),
                      torch.from_numpy(v).to(cuda), o, model, engine, st)
    torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy(), want, f"prefill Hq={Hq} Hkv={Hkv}")


@pytest.mark.parametrize("step_octaves", [0.5, 3.0, 20.0])
def test_prefill_attention_growing_scores(cuda, step_octaves):
    """Scores that climb along the key axis: the row max keeps moving, by less than, about, or far
    more than the distance at which the kernel moves its exponent reference and rescales."""
    rng = np.random.default_rng(5)
    Hq, Hkv, n = 4, 2, 700
    q = np.zeros((n, Hq, 128), np.float32)
    k = np.zeros((n, Hkv, 128), np.float32)
    q[:, :, 0] = 1.0
    q[:, :, 1:] = rng.standard_normal((n, Hq, 127)) * 0.05
    # q.k / sqrt(D) * log2(e) grows by step_octaves every 64 keys, with noise on top
    ramp = (np.arange(n) // 64) * step_octaves / (128 ** -0.5 * 1.4426950408889634)
    k[:, :, 0] = ramp[:, None]
    k[:, :, 1:] = rng.standard_normal((n, Hkv, 127))
    q, k = q.astype(np.float16), k.astype(np.float16)
    v = rand_f16(rng, n, Hkv, 128)
    lens = [n]
    want = R.prefill_attention(q, k, v, np.array([0]), np.asarray(lens), 128 ** -0.5, math="np32")
    model = Cfg(num_layers=1, num_q_heads=Hq, num_kv_heads=Hkv, head_dim=128)
    engine = Cfg(block_size=16, max_blocks_per_seq=64)
    st = build_infer_state(lens, [0], [], Hkv, 128)
    o = torch.full((n, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    prefill_attention(torch.from_numpy(q).to(cuda), torch.from_numpy(k).to(cuda),
                      torch.from_numpy(v).to(cuda), o, model, engine, st)
    torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy(), want, f"prefill with scores growing {step_octaves} octaves per tile")


@pytest.mark.parametrize("waves", [4, 8, 4 | (1 << 8), 4 | (2 << 8), 8 | (1 << 8), 8 | (2 << 8)])
def test_prefill_attention_both_workgroup_shapes(cuda, waves):
    """The 128-row and the 256-row workgroup shapes (the second is picked for long prompts) on ragged
    lengths around their tile edges, contiguous and paged-with-prefix sources; bits 8-9 of the switch force two
    query tiles per workgroup (1) or one (2), which the library otherwise chooses by grid size."""
    rng = np.random.default_rng(21)
    Hq, Hkv = 4, 2
    lens = np.array([1, 127, 128, 129, 255, 256, 257, 300, 513, 700])
    T = int(lens.sum())
    q = rand_f16(rng, T, Hq, 128)
    k = rand_f16(rng, T, Hkv, 128)
    v = rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - lens
    want = R.prefill_attention(q, k, v, starts, lens, 128 ** -0.5, math="np32")
    case = make_case(21, 2, Hq, Hkv, lens, num_blocks=int(((lens + 15) // 16).sum()) + 2, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state(lens.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    with kernel_variant(prefill=waves):
        o = torch.full((T, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
        prefill_attention(torch.from_numpy(q).to(cuda), torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda),
                          o, model, engine, st)
        torch.cuda.synchronize()
        assert_attn_close(o.cpu().numpy(), want, f"prefill, {waves} waves")
        store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt, model, engine,
                      st, 0)
        prefix = lens // 3
        l2 = lens - prefix
        q2 = np.concatenate([q[starts[b] + prefix[b]:starts[b] + lens[b]] for b in range(len(lens))])
        st2 = build_infer_state(l2.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
        o2 = torch.full((int(l2.sum()), Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
        chunked_prefill_attention(torch.from_numpy(q2).to(cuda), kc, vc, [], [], bt, model, engine, st2, 0, o2,
                                  prefix_lens=torch.from_numpy(prefix.astype(np.int32)).to(cuda))
        torch.cuda.synchronize()
    want2 = np.concatenate([want[starts[b] + prefix[b]:starts[b] + lens[b]] for b in range(len(lens))])
    assert_attn_close(o2.cpu().numpy(), want2, f"chunk over prefix, {waves} waves")


def test_chunk_over_long_prefix_with_the_prefix_hint(cuda):
    """Eight chunks over long cached prefixes, a grid wide enough for the library to pick the 256-row workgroup
    shape when it is told how long the prefixes are: the hint must not change a bit, and both match the oracle."""
    rng = np.random.default_rng(505)
    Hq, Hkv = 32, 8
    prefix = np.array([768, 600, 512, 1000, 530, 777, 640, 901])
    chunk = np.array([256, 300, 512, 257, 384, 256, 400, 333])
    lens = prefix + chunk
    T = int(lens.sum())
    k = rand_f16(rng, T, Hkv, 128)
    v = rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - lens
    case = make_case(505, 1, Hq, Hkv, lens, num_blocks=int(((lens + 15) // 16).sum()) + 3, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state(lens.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt, model, engine, st, 0)
    R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, 0)
    s2 = np.cumsum(chunk) - chunk
    q2 = rand_f16(rng, int(chunk.sum()), Hq, 128)
    want = R.chunked_prefill_attention(q2, case.arena, case.lay, case.block_table, case.seq_ids, s2, chunk, prefix,
                                       128 ** -0.5, 0)
    st2 = build_infer_state(chunk.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    outs = []
    for hint in (0, int(prefix.max())):
        o = torch.full((int(chunk.sum()), Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
        chunked_prefill_attention(torch.from_numpy(q2).to(cuda), kc, vc, [], [], bt, model, engine, st2, 0, o,
                                  prefix_lens=torch.from_numpy(prefix.astype(np.int32)).to(cuda), max_prefix_len=hint)
        torch.cuda.synchronize()
        outs.append(o.cpu().numpy())
    assert_attn_close(outs[0], want, "chunk over long prefix, no hint")
    assert np.array_equal(outs[0].view(np.uint16), outs[1].view(np.uint16)), "the prefix hint changed the output"


def test_chunked_prefill_over_paged_cache(cuda):
    """Second half of each prompt as a chunk whose first half is already cached."""
    rng = np.random.default_rng(77)
    lens = np.array([40, 129, 16, 300])
    Hq, Hkv = 8, 2
    T = int(lens.sum())
    q = rand_f16(rng, T, Hq, 128)
    k = rand_f16(rng, T, Hkv, 128)
    v = rand_f16(rng, T, Hkv, 128)
    starts = np.cumsum(lens) - lens
    case = make_case(77, 2, Hq, Hkv, lens, num_blocks=40, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state(lens.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    store_kvcache(torch.from_numpy(k).to(cuda), torch.from_numpy(v).to(cuda), kc, vc, [], [], bt,
                  model, engine, st, 1)
    R.append_prefill(case.arena, case.lay, k, v, case.block_table, case.seq_ids, starts, lens, 1)
    half = lens // 2
    l2 = lens - half
    s2 = np.cumsum(l2) - l2
    q2 = np.concatenate([q[starts[b] + half[b]:starts[b] + lens[b]] for b in range(len(lens))])
    want = R.chunked_prefill_attention(q2, case.arena, case.lay, case.block_table, case.seq_ids, s2,
                                       l2, half, 128 ** -0.5, 1)
    st2 = build_infer_state(l2.tolist(), case.seq_ids.tolist(), [], Hkv, 128)
    o = torch.full((int(l2.sum()), Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
    chunked_prefill_attention(torch.from_numpy(q2).to(cuda), kc, vc, [], [], bt, model, engine, st2,
                              1, o, prefix_lens=torch.from_numpy(half.astype(np.int32)).to(cuda))
    torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy(), want, "chunked prefill")
