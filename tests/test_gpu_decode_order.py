"""The balanced order in which the decode grid takes a batch's rows (``mkv_decode_order``) and the
attention entry that follows it (``mkv_decode_attn_ordered``).

The order is a permutation chosen for balance only: outputs and cache bytes must be the same bits with
and without it, for every decode entry, and an order that has gone stale must still be harmless.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, configs, to_gpu
from morphserve_amd import (_capi, build_infer_state, decode_append_and_attend, decode_rope_append_and_attend,
                            paged_attention, rotary_tables)
from morphserve_amd.worker.kernels import paged_attn as PA

pytestmark = pytest.mark.gpu


def _snake_order(lens: np.ndarray, num_kv_heads: int) -> np.ndarray:
    """Rows by descending length (ties: lower row first), dealt over runs of 256 / Hkv slots with every second
    full run reversed -- written with a stable sort, not with the kernel's rank counting."""
    n = len(lens)
    by_len = np.argsort(-lens.astype(np.int64), kind="stable")
    run = 256 // num_kv_heads if 256 % num_kv_heads == 0 else n
    order = by_len.copy()
    for r in range(n // run):
        if r & 1:
            order[r * run:(r + 1) * run] = by_len[r * run:(r + 1) * run][::-1]
    return order.astype(np.int32)


@pytest.mark.parametrize("n,hkv", [(1, 8), (2, 8), (31, 8), (32, 8), (33, 8), (64, 8), (65, 8), (128, 8), (200, 4),
                                   (64, 32), (7, 3), (300, 3), (1000, 16), (4096, 8)])
def test_order_is_the_balanced_permutation(cuda, n, hkv):
    rng = np.random.default_rng(n * 131 + hkv)
    lens = rng.integers(1, 40, size=n).astype(np.int32) if n % 2 else rng.integers(1, 5000, size=n).astype(np.int32)
    lens_t = torch.from_numpy(lens).to(cuda)
    order = torch.full((n,), -7, dtype=torch.int32, device=cuda)
    _capi.check(_capi.lib().mkv_decode_order(lens_t.data_ptr(), n, hkv, order.data_ptr(), _capi.current_stream()))
    torch.cuda.synchronize()
    got = order.cpu().numpy()
    assert sorted(got.tolist()) == list(range(n)), "not a permutation"
    assert np.array_equal(got, _snake_order(lens, hkv))
    run = 256 // hkv if 256 % hkv == 0 else n
    if n >= 2 * run:        # the two workgroups of a CU: a long and a short row, sums within one step of the sorted lengths
        srt = np.sort(lens.astype(np.int64))[::-1]
        sums = lens[got[:run]].astype(np.int64) + lens[got[run:2 * run]]
        assert sums.max() - sums.min() <= (srt[0] - srt[run - 1]) + (srt[run] - srt[2 * run - 1])


def test_order_refuses_more_rows_than_it_can_rank(cuda):
    lens_t = torch.ones(5000, dtype=torch.int32, device=cuda)
    order = torch.empty(5000, dtype=torch.int32, device=cuda)
    rc = _capi.lib().mkv_decode_order(lens_t.data_ptr(), 5000, 8, order.data_ptr(), _capi.current_stream())
    assert rc != 0 and b"4096" in _capi.lib().mkv_last_error()


@pytest.mark.parametrize("hq,hkv,target_wgs", [(32, 8, None), (8, 8, None), (16, 2, None), (32, 8, 100000)])
def test_outputs_do_not_depend_on_the_order(cuda, hq, hkv, target_wgs):
    """Every decode entry, one and many splits: same bits in o and in the cache with the balanced order,
    with the rows' own order, and with an arbitrary permutation handed to the C entry directly."""
    rng = np.random.default_rng(77 + hq)
    n = 70
    lens = rng.integers(1, 700, size=n)
    lens[:4] = [1, 16, 17, 699]
    L, layer = 2, 1
    case = make_case(5, L, hq, hkv, lens.tolist(), num_blocks=int(((lens + 15) // 16).sum()) + 3, fill="all")
    model, engine = configs(case)
    q = torch.from_numpy(rand_f16(rng, n, hq, 128)).to(cuda)
    k = torch.from_numpy(rand_f16(rng, n, hkv, 128)).to(cuda)
    v = torch.from_numpy(rand_f16(rng, n, hkv, 128)).to(cuda)
    cos_t, sin_t = rotary_tables(128, 1024, device="cuda")
    pos = torch.from_numpy(lens - 1).to(cuda)
    old = (PA.BALANCED_ORDER, PA.TARGET_WORKGROUPS)
    results = {}
    try:
        if target_wgs is not None:
            PA.TARGET_WORKGROUPS = target_wgs
        for balanced in (True, False):
            PA.BALANCED_ORDER = balanced
            outs = []
            for entry in ("attend", "append", "rope"):
                kc, vc, bt = to_gpu(case, cuda)
                st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), hkv, 128)
                st.position_cos, st.position_sin = cos_t[pos].contiguous(), sin_t[pos].contiguous()
                o = torch.full((n, hq * 128), float("nan"), dtype=torch.float16, device=cuda)
                if entry == "attend":
                    paged_attention(q, kc, vc, [], [], bt, model, engine, st, layer, o)
                elif entry == "append":
                    decode_append_and_attend(k, v, q, kc, vc, [], [], bt, model, engine, st, layer, o)
                else:
                    decode_rope_append_and_attend(k, v, q, kc, vc, [], [], bt, model, engine, st, layer, o)
                torch.cuda.synchronize()
                # the order is computed for unsplit batches only: splits carry equal token counts anyway
                one_split = PA._split_for(st, model, engine)[1] == 1
                assert (getattr(st, "_morphkv_decode_order", None) is not None) == (balanced and one_split)
                outs.append((bits(o), bits(kc), bits(vc)))
            results[balanced] = outs
    finally:
        PA.BALANCED_ORDER, PA.TARGET_WORKGROUPS = old
    for a, b in zip(results[True], results[False]):
        for x, y in zip(a, b):
            assert np.array_equal(x, y)
    # an arbitrary permutation through the C entry, one split and several, against the entry without an order
    kc, vc, bt = to_gpu(case, cuda)
    st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), hkv, 128)
    perm = torch.from_numpy(rng.permutation(n).astype(np.int32)).to(cuda)
    pool = _capi.make_pool(kc, vc)
    lib, stream = _capi.lib(), _capi.current_stream()
    for tps, splits in ((1024, 1), (64, 11)):
        mid_o = torch.empty(n * hq * splits * 128, dtype=torch.float32, device=cuda)
        mid_lse = torch.empty(n * hq * splits, dtype=torch.float32, device=cuda)
        o_plain = torch.full((n, hq * 128), float("nan"), dtype=torch.float16, device=cuda)
        o_perm = torch.full((n, hq * 128), float("nan"), dtype=torch.float16, device=cuda)
        _capi.check(lib.mkv_paged_attn_decode(
            q.data_ptr(), o_plain.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], st.seq_ids.data_ptr(),
            st.decoding_seq_lens.data_ptr(), n, hq, 128 ** -0.5, layer, tps, splits, mid_o.data_ptr(),
            mid_lse.data_ptr(), stream))
        _capi.check(lib.mkv_decode_attn_ordered(
            q.data_ptr(), o_perm.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], st.seq_ids.data_ptr(),
            st.decoding_seq_lens.data_ptr(), perm.data_ptr(), n, hq, 128 ** -0.5, layer, tps, splits,
            mid_o.data_ptr(), mid_lse.data_ptr(), None, None, None, None, stream))
        torch.cuda.synchronize()
        assert np.array_equal(bits(o_plain), bits(o_perm))
        want = R.paged_attention(q.cpu().numpy(), case.arena, case.lay, case.block_table, case.seq_ids,
                                 case.seq_lens, 128 ** -0.5, layer)
        assert_attn_close(o_perm.cpu().numpy().reshape(n, hq, 128), want, f"arbitrary order, {splits} splits")


def test_a_stale_order_is_harmless(cuda):
    """The order is kept per infer_state; lengths changed in place afterwards leave a permutation that no
    longer balances anything but still covers every row."""
    rng = np.random.default_rng(9)
    hq, hkv, n = 8, 2, 40
    lens = rng.integers(20, 300, size=n)
    case = make_case(3, 1, hq, hkv, lens.tolist(), num_blocks=int(((lens + 15) // 16).sum()) + 2, fill="all")
    model, engine = configs(case)
    kc, vc, bt = to_gpu(case, cuda)
    st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), hkv, 128)
    q = torch.from_numpy(rand_f16(rng, n, hq, 128)).to(cuda)
    o = torch.full((n, hq * 128), float("nan"), dtype=torch.float16, device=cuda)
    paged_attention(q, kc, vc, [], [], bt, model, engine, st, 0, o)          # the order is computed here
    shorter = np.maximum(1, lens * rng.uniform(0.02, 1.0, size=n)).astype(np.int32)   # another ranking, same tensor
    st.decoding_seq_lens.copy_(torch.from_numpy(shorter))
    o.fill_(float("nan"))
    paged_attention(q, kc, vc, [], [], bt, model, engine, st, 0, o)
    torch.cuda.synchronize()
    want = R.paged_attention(q.cpu().numpy(), case.arena, case.lay, case.block_table, case.seq_ids, shorter.astype(np.int64),
                             128 ** -0.5, 0)
    assert_attn_close(o.cpu().numpy().reshape(n, hq, 128), want, "stale order")


def test_order_entries_outside_the_batch_are_clamped(cuda):
    """The order lives on the device and cannot be checked on the host: the kernels take a slot's own index
    wherever the entry is not a row of the batch.  All entries out of range -> the rows' own order, bit for
    bit; some out of range -> every row is either untouched or equal to the plain result."""
    rng = np.random.default_rng(123)
    hq, hkv, n, layer = 32, 8, 50, 0
    lens = rng.integers(1, 400, size=n)
    case = make_case(11, 1, hq, hkv, lens.tolist(), num_blocks=int(((lens + 15) // 16).sum()) + 2, fill="all")
    kc, vc, bt = to_gpu(case, cuda)
    st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), hkv, 128)
    q = torch.from_numpy(rand_f16(rng, n, hq, 128)).to(cuda)
    pool = _capi.make_pool(kc, vc)
    lib, stream = _capi.lib(), _capi.current_stream()
    garbage = np.array([n, -1, 10 ** 6, 2 ** 31 - 1, -(2 ** 31), n + 7], dtype=np.int64)
    all_bad = garbage[rng.integers(0, len(garbage), size=n)].astype(np.int32)
    some_bad = rng.permutation(n).astype(np.int32)
    hit = rng.choice(n, size=12, replace=False)
    some_bad[hit] = garbage[rng.integers(0, len(garbage), size=12)].astype(np.int32)
    for tps, splits in ((1024, 1), (64, 7)):
        mid_o = torch.empty(n * hq * splits * 128, dtype=torch.float32, device=cuda)
        mid_lse = torch.empty(n * hq * splits, dtype=torch.float32, device=cuda)
        outs = {}
        for name, order in (("plain", None), ("all_bad", all_bad), ("some_bad", some_bad)):
            o = torch.full((n, hq * 128), float("nan"), dtype=torch.float16, device=cuda)
            order_t = torch.from_numpy(order).to(cuda) if order is not None else None
            _capi.check(lib.mkv_decode_attn_ordered(
                q.data_ptr(), o.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], st.seq_ids.data_ptr(),
                st.decoding_seq_lens.data_ptr(), order_t.data_ptr() if order_t is not None else None, n, hq,
                128 ** -0.5, layer, tps, splits, mid_o.data_ptr(), mid_lse.data_ptr(), None, None, None, None, stream))
            torch.cuda.synchronize()
            outs[name] = bits(o)
        assert np.array_equal(outs["plain"], outs["all_bad"])
        for row in hit:         # a slot whose entry is not a row of the batch does its own row
            assert np.array_equal(outs["some_bad"][row], outs["plain"][row]), row
        if splits == 1:         # phase 1 writes o itself: a row is either done or was never touched
            untouched = bits(torch.full((hq * 128,), float("nan"), dtype=torch.float16))
            for row in range(n):
                got = outs["some_bad"][row]
                assert np.array_equal(got, outs["plain"][row]) or np.array_equal(got, untouched), row
