"""The per-workgroup time stamps (``mkv_diag_timeline``): a measurement hook that must not change a result.

The hook lives in the diagnostic twin of the library only (``libmorphkv_diag.so``); the product library's
kernels carry no time-stamp argument.  The reference results below come from the PRODUCT library, the
stamped ones from the twin, so the test also pins that the two libraries compute the same bits.

With a buffer set, the twin's prefill kernel and both decode phase-1 kernels stamp the GPU's constant-rate counter at
fixed points of every workgroup's life; outputs must be the same bits as without it, the stamps of a workgroup
must be in order, and with the buffer taken away nothing may be written.
"""
import numpy as np
import pytest
import torch

from helpers import make_case, rand_f16
from gpu_helpers import bits, configs, kernel_variant, to_gpu
from morphserve_amd import _capi, build_infer_state, paged_attention, prefill_attention
from morphserve_amd.worker.kernels import paged_attn as PA

pytestmark = pytest.mark.gpu
POINTS = 8


def _stamped(cuda, fn, max_wgs):
    """``fn`` through the diagnostic twin while it holds a time-stamp buffer for ``max_wgs`` workgroups."""
    buf = torch.zeros(max_wgs * POINTS, dtype=torch.int64, device=cuda)
    with _capi.use_diag_library() as lib:
        _capi.check(lib.mkv_diag_timeline(buf.data_ptr(), max_wgs))
        try:
            out = fn()
            torch.cuda.synchronize()
        finally:
            _capi.check(lib.mkv_diag_timeline(None, 0))
    return out, buf.cpu().numpy().reshape(max_wgs, POINTS)


def _in_order(stamps):
    live = stamps[stamps[:, 0] > 0]
    assert len(live) > 0
    for row in live:
        seen = row[row > 0]
        assert np.all(np.diff(seen) >= 0), row
    return live


def test_prefill_stamps_leave_the_output_alone(cuda):
    rng = np.random.default_rng(9)
    lens = np.array([300, 129, 700, 64])
    Hq, Hkv = 4, 2
    T = int(lens.sum())
    q, k, v = (torch.from_numpy(rand_f16(rng, T, h, 128)).to(cuda) for h in (Hq, Hkv, Hkv))
    case = make_case(9, 1, Hq, Hkv, lens, num_blocks=int(((lens + 15) // 16).sum()) + 2, fill="all")
    model, engine = configs(case)
    st = build_infer_state(lens.tolist(), case.seq_ids.tolist(), [], Hkv, 128)

    def run():
        o = torch.full((T, Hq, 128), float("nan"), dtype=torch.float16, device=cuda)
        prefill_attention(q, k, v, o, model, engine, st)
        return o
    plain = run()
    torch.cuda.synchronize()
    for variant in (4 | (1 << 8), 4 | (2 << 8), 8 | (1 << 8)):      # two tiles per workgroup, one, the 256-row shape
        with kernel_variant(prefill=variant):
            ref = run()
            got, stamps = _stamped(cuda, run, 4096)
        assert np.array_equal(bits(got), bits(ref)) and np.array_equal(bits(got), bits(plain))
        live = _in_order(stamps)
        ran = live[live[:, 1] > 0]                                  # slots past a short sequence's tiles leave at once
        assert len(ran) > 0 and np.all(ran[:, 3] > 0)               # every workgroup that staged a tile wrote its output
        if variant == 4 | (1 << 8):
            assert np.any(ran[:, 6] > 0)                            # some carried a second tile
    # a buffer too small for the grid is not used at all
    got, stamps = _stamped(cuda, run, 1)
    assert np.array_equal(bits(got), bits(plain)) and not stamps.any()


@pytest.mark.parametrize("Hq,Hkv,target_wgs", [(8, 2, 1), (8, 2, 100000), (4, 4, 1), (4, 4, 100000)])
def test_decode_stamps_leave_the_output_alone(cuda, Hq, Hkv, target_wgs, monkeypatch):
    rng = np.random.default_rng(Hq + target_wgs)
    lens = np.array([1, 17, 250, 1000, 333])
    case = make_case(5, 2, Hq, Hkv, lens, num_blocks=120, fill="live")
    kc, vc, bt = to_gpu(case, cuda)
    model, engine = configs(case)
    st = build_infer_state([], case.seq_ids.tolist(), lens.tolist(), Hkv, 128)
    q = torch.from_numpy(rand_f16(rng, len(lens), Hq, 128)).to(cuda)
    monkeypatch.setattr(PA, "TARGET_WORKGROUPS", target_wgs, raising=False)

    def run():
        o = torch.full((len(lens), Hq * 128), float("nan"), dtype=torch.float16, device=cuda)
        paged_attention(q, kc, vc, [], [], bt, model, engine, st, 1, o)
        return o
    ref = run()
    torch.cuda.synchronize()
    got, stamps = _stamped(cuda, run, 1 << 16)
    assert np.array_equal(bits(got), bits(ref))
    live = _in_order(stamps)
    ran = live[live[:, 1] > 0]                                      # splits past a sequence's end leave at once
    assert len(ran) > 0 and np.all(ran[:, 3] > 0)
    got, stamps = _stamped(cuda, run, 1)
    assert np.array_equal(bits(got), bits(ref)) and not stamps.any()
