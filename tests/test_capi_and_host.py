"""CPU-only checks: the C-ABI library loads and exports every symbol the header
declares (no compute calls here), and the host-side logic of the operator mirror."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import ref_cpu as R

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", "morphkv.h"), os.path.join(ROOT, "include", "morphkv_diag.h")]
DIAG_ONLY = ("mkv_set_decode_variant", "mkv_set_prefill_variant", "mkv_diag_mfma_loop", "mkv_diag_timeline",
             "mkv_diag_slab_gather", "mkv_diag_split_by_rate", "mkv_prof_enable", "mkv_prof_reset", "mkv_prof_collect")


def _declared(headers=HEADERS):
    names = set()
    for header in headers:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(mkv_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_the_reference_facing_header_holds_no_tuning_or_measurement_entries():
    boundary = _declared(HEADERS[:1])
    for name in DIAG_ONLY:
        assert name not in boundary and name in _declared(HEADERS[1:])


def test_header_declares_the_expected_surface():
    names = _declared()
    for must in ("mkv_append_decode", "mkv_append_prefill", "mkv_paged_attn_decode", "mkv_prefill_attn",
                 "mkv_decode_order", "mkv_decode_attn_ordered",
                 "mkv_bm_allocate", "mkv_bt_append", "mkv_bt_release", "mkv_bt_gather_release",
                 "mkv_pool_plan_shrink", "mkv_pool_migrate", "mkv_bt_remap", "mkv_swap_blocks",
                 "mkv_pool_carve_segment", "mkv_fill_zero"):
        assert must in names


def _exported(path):
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
    return sorted(line.split()[-1] for line in out.splitlines() if line.strip())


def test_library_exports_exactly_the_declared_symbols():
    """The product library exports what morphkv.h declares and nothing else (no diagnostics, no C++
    helpers); its diagnostic twin adds exactly what morphkv_diag.h declares."""
    from morphserve_amd import _capi
    lib = _capi.lib()
    boundary = _declared(HEADERS[:1])
    for name in boundary:
        assert hasattr(lib, name), f"{name} is declared in morphkv.h but not exported"
        assert name in _capi.PROTOTYPES, f"{name} has no ctypes prototype"
    assert sorted(_capi.PROTOTYPES) == boundary
    assert _exported(_capi.LIB_PATH) == boundary
    for name in DIAG_ONLY:
        assert not hasattr(lib, name), f"{name} is a diagnostic and must not be in the product library"
    diag = _capi.diag_lib()
    assert sorted(_capi.DIAG_PROTOTYPES) == sorted(DIAG_ONLY) == _declared(HEADERS[1:])
    assert _exported(_capi.DIAG_LIB_PATH) == _declared()
    assert lib.mkv_version() >= 1 and diag.mkv_version() == lib.mkv_version()
    assert ctypes.sizeof(_capi.MkvPool) == lib.mkv_sizeof_pool() == 56 + 2 * 8 * _capi.MKV_MAX_SEGMENTS


def test_host_only_entry_points():
    """Entry points that do no GPU work can be exercised without a GPU."""
    from morphserve_amd import _capi, swiftllm_c
    lib = _capi.lib()
    k0, s, v0 = ctypes.c_uint64(0), ctypes.c_int64(0), ctypes.c_uint64(0)
    rc = lib.mkv_pool_carve_segment(1000, 4000, 300, 2, 2, 4, 8, ctypes.byref(k0), ctypes.byref(s), ctypes.byref(v0))
    assert rc == 0 and (k0.value, s.value, v0.value) == R.acquire_new_kvcache_arith(1000, 4000, 300, 2, 2, 4, 8)
    rc = lib.mkv_pool_carve_segment(0, 1000, 600, 2, 2, 4, 8, ctypes.byref(k0), ctypes.byref(s), ctypes.byref(v0))
    assert rc == _capi.MKV_ENOSPC and b"No space available" in lib.mkv_last_error()
    MiB = 1 << 20
    swiftllm_c.register_kv_cache_info(32, 8, 16, 128)
    assert swiftllm_c.carve_segment(7 * MiB, 436 * MiB, 120 * MiB + 5) == \
        R.acquire_new_kvcache_arith(7 * MiB, 436 * MiB, 120 * MiB + 5, 32, 8, 16, 128)
    # strided segment table: segment j sits j * stride * elem_bytes below segment 0
    pool = _capi.MkvPool()
    _capi.check(lib.mkv_pool_set_strided(ctypes.byref(pool), 1 << 30, (1 << 30) + 4096, 1000, 2, 3))
    assert [pool.k_seg[j] for j in range(3)] == [(1 << 30) - j * 2000 for j in range(3)]
    assert [pool.v_seg[j] for j in range(3)] == [(1 << 30) + 4096 - j * 2000 for j in range(3)]
    assert pool.num_segments == 3 and pool.k_seg[3] is None
    with pytest.raises(_capi.MorphKVError):
        _capi.check(lib.mkv_pool_set_strided(ctypes.byref(pool), 0, 0, 1000, 2, 999))
    # argument validation happens before any launch
    assert lib.mkv_append_decode(None, None, None, None, 0, None, None, 1, 0, None) == _capi.MKV_EINVAL
    # chunk sizes an arena cannot map back to back are refused before the device is touched
    arena = ctypes.c_void_p()
    assert lib.mkv_arena_create(12 << 20, 3 << 20, ctypes.byref(arena)) == _capi.MKV_EINVAL
    assert b"multiple of 2 MiB" in lib.mkv_last_error() and not arena.value
    assert lib.mkv_arena_create(5 << 20, 2 << 20, ctypes.byref(arena)) == _capi.MKV_EINVAL      # not whole chunks
    with pytest.raises(NotImplementedError):
        swiftllm_c.replace_layer_org2quant(0)


def test_plain_c_program_links_and_calls_the_library(tmp_path):
    """morphkv.h is valid C99 and a C program (no Python, no torch) links against the library."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    from morphserve_amd import _capi
    libdir = os.path.dirname(_capi.LIB_PATH)
    exe = str(tmp_path / "abi_consumer")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "c", "abi_consumer.c"), "-o", exe, "-L", libdir, "-lmorphkv",
                    "-Wl,-rpath," + libdir], check=True, capture_output=True, text=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    assert "abi_consumer: ok" in res.stdout


def test_seq_block_size_matches_oracle():
    from morphserve_amd import select_seq_block_size
    rng = np.random.default_rng(0)
    for _ in range(200):
        n = int(rng.integers(0, 200))
        lens = rng.integers(1, 5000, size=n).tolist()
        hkv = int(rng.choice([1, 2, 4, 8, 32]))
        assert select_seq_block_size(hkv, lens) == R.select_seq_block_size(hkv, lens)
    assert select_seq_block_size(32, [64, 100, 200, 288, 300, 400, 445, 512]) == (64, 8)
    assert select_seq_block_size(8, [1280] * 64) == (512, 3)


def test_choose_split_properties():
    from morphserve_amd.worker.kernels.paged_attn import choose_split
    rng = np.random.default_rng(1)
    for _ in range(500):
        n = int(rng.integers(1, 600))
        hkv = int(rng.choice([1, 2, 4, 8, 32]))
        max_len = int(rng.integers(1, 40000))
        tps, splits = choose_split(n, hkv, max_len, 16, target_wgs=int(rng.integers(1, 5000)))
        assert tps % 64 == 0 and tps > 0
        assert splits >= 1 and splits * tps >= max_len and (splits - 1) * tps < max_len
    assert choose_split(64, 8, 1536, 16, target_wgs=1536) == (512, 3)
    assert choose_split(64, 8, 1536, 16) == (1536, 1)
    assert choose_split(8, 32, 512, 16) == (256, 2)
    assert choose_split(1000, 32, 512, 16, target_wgs=1536) == (512, 1)


def test_block_count_behaves_like_the_reference_counter():
    from morphserve_amd.worker.block_manager import BlockCount
    c = BlockCount(10)
    c -= 3
    c += 2
    assert c == 9 and c.item() == 9 and isinstance(c, int) and isinstance(c + 1, BlockCount)
    assert (c >= 9) and (100 - c == 91) and f"{c}" == "9"


def test_product_does_not_import_the_oracle():
    """The shipped package must never reach into the test oracle."""
    pkg = os.path.join(ROOT, "morphserve_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"


def test_bad_arguments_are_refused_before_any_launch():
    """Every entry point validates its arguments on the host: NULL pointers, unsupported shapes and
    out-of-range switches come back as a negative status with a message, without a GPU."""
    from morphserve_amd import _capi
    lib = _capi.lib()
    pool = _capi.MkvPool()                    # all zero: no base pointers, no geometry
    good = _capi.MkvPool()
    good.k_base, good.v_base = 1 << 20, 1 << 21
    good.num_blocks_org, good.num_layers, good.num_kv_heads, good.block_size, good.head_dim = 8, 1, 2, 16, 64
    P, G = ctypes.byref(pool), ctypes.byref(good)
    A = 1 << 20                               # an aligned non-NULL address that is never dereferenced
    calls = {
        "mkv_append_prefill": (None, None, P, None, 0, None, None, None, 1, 16, 0, None),
        "mkv_append_prefill/row too short": (A, A, G, A, 4, A, A, A, 1, 16 * 4 + 1, 0, None),
        "mkv_paged_attn_decode": (A, A, P, A, 4, A, A, 1, 2, 0.1, 0, 64, 1, None, None, None),
        "mkv_paged_attn_decode/head_dim": (A, A, G, A, 4, A, A, 1, 2, 0.1, 0, 64, 1, None, None, None),
        "mkv_paged_attn_decode_static/too large": (A, A, G, A, 4, A, A, 64, 64, 0.1, 0, 64, 64, None),
        "mkv_decode_append_attn": (A, A, A, A, P, A, 4, A, A, 1, 2, 0.1, 0, 64, 1, None, None, None),
        "mkv_decode_rope_append_attn": (A, A, A, A, A, A, P, A, 4, A, A, 1, 2, 0.1, 0, 64, 1, None, None, None),
        "mkv_decode_order": (None, 4, 8, A, None),
        "mkv_decode_order/too many rows": (A, 4097, 8, A, None),
        "mkv_decode_order/heads": (A, 4, 0, A, None),
        "mkv_decode_attn_ordered": (A, A, P, A, 4, A, A, A, 1, 2, 0.1, 0, 64, 1, None, None, None, None, None, None,
                                    None),
        "mkv_decode_attn_ordered/k without v": (A, A, G, A, 4, A, A, None, 1, 2, 0.1, 0, 64, 1, None, None, A, None,
                                                None, None, None),
        "mkv_prefill_attn": (A, A, A, A, A, A, 1, 16, 2, 2, 64, 0.1, None),                  # head_dim 64
        "mkv_prefill_attn/scale": (A, A, A, A, A, A, 1, 16, 2, 2, 128, 0.0, None),
        "mkv_prefill_attn_paged": (A, A, P, A, 4, A, A, A, None, 1, 16, 0, 2, 0.1, 0, None),
        "mkv_pool_migrate": (P, A, A, 1, None),
        "mkv_fill_zero": (A + 4, 64, None),                                                    # unaligned
        "mkv_swap_blocks": (None, None, 1, 0, P, None, None, None, None),
        "mkv_swap_blocks_device_ids": (None, None, 1, 0, P, None, None, 1, None),
        "mkv_rope_store_kvcache": (None, None, None, None, None, P, None, 4, None, None, None, None, 0, 0, 1, 2, 2,
                                   128, 0, 1, None),
        "mkv_bm_allocate": (None, 4, None, 4, None, 8, None, None, 1, 16, None, 0, None, None),
        "mkv_bm_take_first_free": (None, 8, 1, None, None, None),
        "mkv_bt_append": (None, 4, None, 4, None, None, None, 0, 1, None),
        "mkv_bt_release": (None, 4, None, 4, None, 1, None, 8, None, None),
        "mkv_bt_gather_release": (None, 4, None, 4, None, 1, None, 8, None, 0, None, None),
        "mkv_bm_count_live": (None, 0, 8, None, None),
        "mkv_pool_plan_shrink": (None, 8, 4, None, None, 0, None, None, None),
        "mkv_bt_remap": (None, 4, None, 4, None, 8, None),
        "mkv_arena_create": (0, 0, None),
        "mkv_arena_resize": (None, 0),
        "mkv_arena_move_tail": (None, None, 4096),
    }
    diag_calls = {
        "mkv_diag_slab_gather/not a power of two": (A, A, 1000, 8, 8, 4, 2, 0, 0, A, None),
        "mkv_diag_slab_gather/loads in flight": (A, A, 1024, 8, 8, 3, 2, 0, 0, A, None),
        "mkv_diag_slab_gather/unaligned": (A + 64, A, 1024, 8, 8, 4, 2, 0, 0, A, None),
        "mkv_diag_slab_gather/workgroups per CU": (A, A, 1024, 8, 8, 4, 9, 0, 0, A, None),
        "mkv_set_decode_variant": (99,),
        "mkv_set_prefill_variant": (5,),
        "mkv_diag_mfma_loop": (7, 1, None, None, None, None),
        "mkv_prof_collect": (_capi.K_ROPE_STORE + 1, None, None),
    }
    diag = _capi.diag_lib()
    for handle, table in ((lib, calls), (diag, calls), (diag, diag_calls)):      # the twin refuses the same calls
        for name, args in table.items():
            fn = getattr(handle, name.split("/")[0])
            rc = fn(*args)
            assert rc < 0, f"{name} accepted bad arguments (returned {rc})"
            assert handle.mkv_last_error(), f"{name} failed without a message"


def test_model_config_kv_sizes_known_answers(tmp_path):
    """get_kvslot_size (MorphServe/model_config.py:36-40) on the shapes the benchmarks use: bytes of one
    token's K and V over all layers, and of one 16-token block."""
    import json

    import torch

    from morphserve_amd import LlamaModelConfig
    shapes = {   # name: (config.json fields, kv slot bytes, block bytes)
        "llama-3-8b": (dict(num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, hidden_size=4096), 131072, 2 << 20),
        "codellama-34b": (dict(num_hidden_layers=48, num_attention_heads=64, num_key_value_heads=8, hidden_size=8192), 196608, 3 << 20),
        "llama-2-7b": (dict(num_hidden_layers=32, num_attention_heads=32, hidden_size=4096), 524288, 8 << 20),
    }
    for name, (fields, slot, block) in shapes.items():
        cfg = LlamaModelConfig(dict(fields, model_type="llama"))
        assert cfg.head_dim == 128, name
        assert cfg.get_kvslot_size() == slot, name
        assert cfg.get_kvslot_size(torch.float32) == 2 * slot, name
        assert cfg.get_block_bytes(16) == block, name
    # pool sizing (MorphServe/worker/model.py:161-171), worked by hand: a 288 GiB card at 0.9 with 30 GiB in use at
    # the peak leaves 229.2 GiB = 117 350.4 blocks of 2 MiB; 48 GiB of 64 GiB at 0.8 leaves 3.2 GiB = 1638.4 blocks
    gib = 1 << 30
    cfg8 = LlamaModelConfig(dict(shapes["llama-3-8b"][0], model_type="llama"))
    assert cfg8.num_blocks_that_fit(16, 258 * gib, 288 * gib, 0.9) == 117350
    assert cfg8.num_blocks_that_fit(16, 16 * gib, 64 * gib, 0.8) == 1638
    assert cfg8.num_blocks_that_fit(16, 16 * gib, 64 * gib, 0.75) == 0
    with pytest.raises(RuntimeError, match="exceeds usable memory"):
        cfg8.num_blocks_that_fit(16, 16 * gib, 64 * gib, 0.7)
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(dict(shapes["llama-3-8b"][0], model_type="llama", rope_scaling=None)))
    cfg = LlamaModelConfig.load_from_model_path(str(d))
    assert (cfg.num_layers, cfg.num_q_heads, cfg.num_kv_heads, cfg.rope_scaling) == (32, 32, 8, 1.0)
    with pytest.raises(ValueError):
        LlamaModelConfig(dict(shapes["llama-2-7b"][0], model_type="gpt2"))


def test_step_state_builder_matches_the_field_by_field_builder():
    """One staging buffer instead of one tensor per list (model.py:318-436): every field equal to
    ``build_infer_state``'s, positions = 0..len-1 per prefill sequence then len-1 per decoding one, over
    consecutive steps that reuse the buffers."""
    import numpy as np
    import torch

    from morphserve_amd import StepStateBuilder, build_infer_state
    cos = torch.arange(4096, dtype=torch.float32).view(-1, 1).expand(4096, 4).contiguous()
    b = StepStateBuilder(16, 4096, 8, 128, cos_cached=cos, sin_cached=-cos, device="cpu")
    rng = np.random.default_rng(0)
    kept = []
    for step in range(12):
        P, n = int(rng.integers(0, 6)), int(rng.integers(0, 8))
        if P + n == 0:
            n = 1
        p = rng.integers(1, 300, size=P).tolist()
        d = rng.integers(1, 2000, size=n).tolist()
        ids = rng.permutation(64)[:P + n].tolist()
        s = b.build(p, ids, d)
        r = build_infer_state(p, ids, d, 8, 128, device="cpu")
        for f in ("seq_ids", "prefill_seq_start_locs", "prefill_seq_start_locs_with_end", "prefill_seq_lens",
                  "decoding_seq_lens"):
            assert torch.equal(getattr(s, f), getattr(r, f)), (step, f)
            assert getattr(s, f).dtype == torch.int32
        for f in ("batch_size", "num_tokens", "num_prefill_seqs", "num_prefill_tokens", "max_prefill_len",
                  "num_decoding_seqs", "max_decoding_len", "seq_block_size", "num_seq_blocks", "softmax_scale",
                  "num_blocks_org", "ignore_kvcache"):
            assert getattr(s, f) == getattr(r, f), (step, f)
        pos = np.concatenate([np.arange(x) for x in p] + [np.asarray(d, dtype=np.int64) - 1]) if P + n else []
        assert s.position_cos[:, 0].tolist() == [float(x) for x in pos]
        assert s.position_sin[:, 3].tolist() == [-float(x) for x in pos]
        kept.append((s, ids))
        if len(kept) >= 2:                                   # the state before this one is still intact (two slots)
            assert kept[-2][0].seq_ids.tolist() == kept[-2][1]
    with pytest.raises(ValueError):
        b.build([4000, 200], [0, 1], [])
    with pytest.raises(ValueError):
        b.build([], [0, 1], [5])


def test_decode_order_cache_is_tied_to_the_capture_it_was_made_in(monkeypatch):
    """The balanced row order is computed by a launch and kept on the infer state.  A launch that was only
    RECORDED into a graph has written nothing yet, so an entry made during a stream capture must serve that
    capture alone: an eager call (the capture may have been abandoned) and any other capture compute their own.
    Host logic only: the library, the stream and the events are stand-ins."""
    import torch

    from morphserve_amd.worker.kernels import paged_attn as PA
    launches = []

    class Lib:
        def mkv_decode_order(self, lens_ptr, n, hkv, order_ptr, stream):
            launches.append(order_ptr)
            return 0

    class Stream:
        cuda_stream = 7

        def wait_event(self, event):
            pass

    class Event:
        def record(self, stream):
            pass

    capture = {"id": None}
    monkeypatch.setattr(PA._capi, "lib", lambda: Lib())
    monkeypatch.setattr(PA._capi, "capture_id", lambda stream: capture["id"])
    monkeypatch.setattr(PA.torch.cuda, "current_stream", lambda: Stream())
    monkeypatch.setattr(PA.torch.cuda, "Event", Event)
    monkeypatch.setattr(PA, "BALANCED_ORDER", True)

    class State:
        pass
    state, lens = State(), torch.zeros(8, dtype=torch.int32)
    eager = PA._decode_order(state, lens, 8, 2, 1)
    assert len(launches) == 1 and PA._decode_order(state, lens, 8, 2, 1) is eager and len(launches) == 1
    capture["id"] = 5                                   # a capture begins: the eager entry is not carried into it
    in_graph = PA._decode_order(state, lens, 8, 2, 1)
    assert in_graph is not eager and len(launches) == 2
    assert PA._decode_order(state, lens, 8, 2, 1) is in_graph and len(launches) == 2      # the other layers of the capture
    capture["id"] = None                                # eager again (graph not replayed, or abandoned)
    after = PA._decode_order(state, lens, 8, 2, 1)
    assert after is not in_graph and len(launches) == 3 and launches[2] == after.data_ptr()
    capture["id"] = 6                                   # another capture
    assert PA._decode_order(state, lens, 8, 2, 1) is not after and len(launches) == 4
    # nothing to balance: one row, a split batch, or the switch off
    assert PA._decode_order(state, lens[:1], 1, 2, 1) is None and PA._decode_order(state, lens, 8, 2, 3) is None
    monkeypatch.setattr(PA, "BALANCED_ORDER", False)
    assert PA._decode_order(state, lens, 8, 2, 1) is None and len(launches) == 4
