"""``mkv_paged_attn_decode_static``: decode attention whose split partials live in an array built
into the library's device code, so that the call allocates nothing.  Checked through the C-ABI
against ``mkv_paged_attn_decode`` with a caller-provided workspace (same kernels: the outputs must
be bit-identical) and against the CPU oracle, on two calls in a row, the second with a smaller
input, so that whatever the first call left in the shared array is there when the second runs."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ref_cpu as R
from helpers import assert_attn_close, make_case, rand_f16
from gpu_helpers import bits, to_gpu
from morphserve_amd import _capi

pytestmark = pytest.mark.gpu

STATIC_BYTES = 16 << 20


def _both_entries(cuda, case, q, layer, tps, splits):
    """(output of the workspace entry, output of the static entry), each [n, Hq, D] fp16."""
    lib = _capi.lib()
    kc, vc, bt = to_gpu(case, cuda)
    pool = _capi.make_pool(kc, vc)
    n = len(case.seq_lens)
    ids = torch.from_numpy(case.seq_ids).to(cuda)
    lens = torch.from_numpy(case.seq_lens).to(cuda)
    qg = torch.from_numpy(q).to(cuda)
    rows = n * case.Hq * splits
    mid_o = torch.full((rows * case.D,), float("nan"), dtype=torch.float32, device=cuda)
    mid_lse = torch.full((rows,), float("nan"), dtype=torch.float32, device=cuda)
    want = torch.full((n, case.Hq, case.D), float("nan"), dtype=torch.float16, device=cuda)
    got = torch.full_like(want, float("nan"))
    stream = _capi.current_stream()
    scale = float(case.D ** -0.5)
    _capi.check(lib.mkv_paged_attn_decode(
        qg.data_ptr(), want.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], ids.data_ptr(), lens.data_ptr(),
        n, case.Hq, scale, layer, tps, splits, mid_o.data_ptr(), mid_lse.data_ptr(), stream))
    torch.cuda.synchronize()

    def static_call():
        _capi.check(lib.mkv_paged_attn_decode_static(
            qg.data_ptr(), got.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], ids.data_ptr(), lens.data_ptr(),
            n, case.Hq, scale, layer, tps, splits, stream))
        torch.cuda.synchronize()
    static_call()             # warm-up: the kernels' code objects are loaded and the scratch address is taken
    # what the DRIVER reports free (hipMemGetInfo), not torch's own counter: an allocation made inside the
    # library (hipMalloc, a memory pool, a virtual-memory mapping) would show here and nowhere else
    import gc
    gc.collect()              # garbage of earlier tests (pools over virtual memory) gives its memory back now,
    gc.disable()              # not in the middle of the comparison
    try:
        torch.cuda.synchronize()
        free_before, _ = torch.cuda.mem_get_info()
        torch_before = torch.cuda.memory_allocated()
        got.fill_(float("nan"))
        static_call()
        free_after, _ = torch.cuda.mem_get_info()
    finally:
        gc.enable()
    assert free_after == free_before, f"the call changed the device's free memory by {free_before - free_after} bytes"
    assert torch.cuda.memory_allocated() == torch_before
    return want.cpu().numpy(), got.cpu().numpy()


# (Hq, Hkv, first call's lengths, second call's lengths, tokens per split); the second call is smaller
# in sequences, in length and in the number of splits it uses
@pytest.mark.parametrize("Hq,Hkv,lens1,lens2,tps", [
    (32, 8, [1500, 1024, 1281, 16, 700, 1], [300, 129], 128),        # matrix-core kernel, 12 then 3 splits
    (8, 8, [9000, 300, 5000], [2000], 64),                            # vector kernel, 141 splits (wide merge), then 32
    (16, 2, [640, 33], [640], 320),                                   # 2 splits, then the same sequence alone
])
def test_static_scratch_matches_workspace_entry_twice(cuda, Hq, Hkv, lens1, lens2, tps):
    rng = np.random.default_rng(Hq * 31 + Hkv)
    for call, lens in enumerate((lens1, lens2)):
        splits = -(-max(lens) // tps)
        nblk = sum((x + 15) // 16 for x in lens) + 3
        case = make_case(100 + call, 2, Hq, Hkv, lens, num_blocks=nblk, fill="live")
        q = rand_f16(rng, len(lens), Hq, 128)
        want, got = _both_entries(cuda, case, q, 1, tps, splits)
        assert np.array_equal(bits(got), bits(want)), f"call {call}: static entry differs from the workspace entry"
        oracle = R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids, case.seq_lens,
                                   128 ** -0.5, 1)
        assert_attn_close(got, oracle, f"call {call} ({splits} splits)")


def test_static_scratch_single_split_and_limit(cuda):
    """One split needs no scratch at any size; beyond 16 MiB of partials the call refuses with a message
    and launches nothing."""
    lib = _capi.lib()
    rng = np.random.default_rng(5)
    lens = [100, 17, 1]
    case = make_case(7, 1, 8, 2, lens, num_blocks=16, fill="live")
    q = rand_f16(rng, 3, 8, 128)
    want, got = _both_entries(cuda, case, q, 0, 112, 1)
    assert np.array_equal(bits(got), bits(want))
    kc, vc, bt = to_gpu(case, cuda)
    pool = _capi.make_pool(kc, vc)
    o = torch.zeros((3, 8, 128), dtype=torch.float16, device=cuda)
    ids = torch.from_numpy(case.seq_ids).to(cuda)
    ln = torch.from_numpy(case.seq_lens).to(cuda)
    qg = torch.from_numpy(q).to(cuda)
    # 3 sequences x 8 heads x max_splits rows of 129 floats: the largest max_splits that fits, then one more
    fits = STATIC_BYTES // (3 * 8 * 129 * 4)
    args = (qg.data_ptr(), o.data_ptr(), C.byref(pool), bt.data_ptr(), bt.shape[1], ids.data_ptr(), ln.data_ptr(),
            3, 8, float(128 ** -0.5), 0, 16)
    _capi.check(lib.mkv_paged_attn_decode_static(*args, fits, _capi.current_stream()))
    torch.cuda.synchronize()
    assert_attn_close(o.cpu().numpy(), R.paged_attention(q, case.arena, case.lay, case.block_table, case.seq_ids,
                                                         case.seq_lens, 128 ** -0.5, 0), "largest max_splits")
    rc = lib.mkv_paged_attn_decode_static(*args, fits + 1, _capi.current_stream())
    assert rc == _capi.MKV_EINVAL and b"built-in scratch" in lib.mkv_last_error()
