"""Moves seeded scenarios onto the GPU and reads the state back for bit-exact comparison."""
from __future__ import annotations

import contextlib

import numpy as np
import torch

from oracle import ref_cpu as R
from helpers import Case, Cfg
from morphserve_amd import BlockManager, ElasticKVPool, _capi, build_infer_state


@contextlib.contextmanager
def kernel_variant(decode: int = 0, prefill: int = 0):
    """Pin a kernel variant for the block.  0 / 0 is the product library's own choice and runs on the
    product library.  Anything else routes the package through the diagnostic twin for the block: it is
    built from the same sources and also holds the kernels the product never launches (the vector-ALU
    decode kernel for groups of 4 and 8, the matrix-core one for 1 and 2) and the switches that force a
    decode kernel (1 vector ALU, 2 matrix cores) or a prefill workgroup shape (4 / 8 waves, pairing bits)."""
    if not decode and not prefill:
        yield _capi.lib()
        return
    with _capi.use_diag_library() as lib:
        _capi.check(lib.mkv_set_decode_variant(decode))
        _capi.check(lib.mkv_set_prefill_variant(prefill))
        try:
            yield lib
        finally:
            lib.mkv_set_decode_variant(0)
            lib.mkv_set_prefill_variant(0)


def to_gpu(case: Case, dev):
    k = torch.from_numpy(case.k_pool.copy()).to(dev)
    v = torch.from_numpy(case.v_pool.copy()).to(dev)
    bt = torch.from_numpy(case.block_table.copy()).to(dev)
    return k, v, bt


def configs(case: Case, max_blocks_per_seq=None):
    model = Cfg(num_layers=case.L, num_q_heads=case.Hq, num_kv_heads=case.Hkv, head_dim=case.D)
    engine = Cfg(block_size=case.B, max_blocks_per_seq=max_blocks_per_seq or case.max_blocks_per_seq)
    return model, engine


def load_manager(case: Case, dev) -> BlockManager:
    bm = BlockManager("GPU", case.num_blocks, case.max_seqs, case.max_blocks_per_seq, case.B)
    bm.block_table.copy_(torch.from_numpy(case.block_table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(case.n_alloc))
    bm.is_block_free.copy_(torch.from_numpy(case.is_free))
    bm.num_free_blocks = int(case.is_free.sum())
    bm.invalidate_host_counts()                     # the counts were written behind the manager's back
    return bm


def manager_state(bm: BlockManager) -> dict:
    return dict(block_table=bm.block_table.cpu().numpy(),
                num_seq_allocated_blocks=bm.num_seq_allocated_blocks.cpu().numpy(),
                is_block_free=bm.is_block_free.cpu().numpy(),
                num_blocks=int(bm.num_blocks), num_free_blocks=int(bm.num_free_blocks))


def assert_state_equal(got: dict, want: dict, what=""):
    for key in want:
        assert np.array_equal(got[key], want[key]), f"{what}: {key} differs"


def bits(t) -> np.ndarray:
    """fp16 tensor / array -> uint16 bit patterns (NaN-safe, sign-of-zero-exact compare)."""
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().numpy()
    return np.ascontiguousarray(t).view(np.uint16)


def pool_case(cuda, seed, org, S, nseg, live_frac, L=2, Hkv=2, D=128):
    """ElasticKVPool grown to org + nseg*S blocks with a random live set, plus the
    oracle's mirror of it (arena + layout with an explicit segment table)."""
    rng = np.random.default_rng(seed)
    total = org + nseg * S
    pool = ElasticKVPool(org, L, Hkv, 16, D, max_seqs_in_block_table=24, max_blocks_per_seq=total)
    for _ in range(nseg):
        pool.expand(S)
    blk = L * Hkv * 16 * D
    # oracle arena: base K, base V, then per segment K, V
    lay = R.PoolLayout(L, Hkv, 16, D, k_base=0, v_base=org * blk, num_blocks_org=org, seg_blocks=S,
                       k_seg=[2 * org * blk + j * 2 * S * blk for j in range(nseg)],
                       v_seg=[2 * org * blk + j * 2 * S * blk + S * blk for j in range(nseg)])
    arena = rng.standard_normal(2 * total * blk, dtype=np.float32).astype(np.float16)
    pool.k_cache.copy_(torch.from_numpy(arena[:org * blk]).view_as(pool.k_cache))
    pool.v_cache.copy_(torch.from_numpy(arena[org * blk:2 * org * blk]).view_as(pool.v_cache))
    for j in range(nseg):
        pool.k_cache_new[j].copy_(torch.from_numpy(arena[lay.k_seg[j]:lay.k_seg[j] + S * blk]).view_as(pool.k_cache_new[j]))
        pool.v_cache_new[j].copy_(torch.from_numpy(arena[lay.v_seg[j]:lay.v_seg[j] + S * blk]).view_as(pool.v_cache_new[j]))
    # random live set scattered over the whole range, dealt to sequences
    n_live = int(live_frac * total)
    live = np.random.default_rng(seed + 1000).permutation(total)[:n_live]
    ob = R.BlockManagerOracle("GPU", org, 24, total, 16)
    for _ in range(nseg):
        ob.expand(S)
    cuts = np.sort(rng.choice(np.arange(1, n_live), size=min(11, n_live - 1), replace=False))
    for s, ids in enumerate(np.split(live, cuts)):
        ob.block_table[s, :len(ids)] = ids
        ob.num_seq_allocated_blocks[s] = len(ids)
    ob.is_block_free[live] = False
    ob.num_free_blocks = total - n_live
    # a freed row with stale ids that must stay untouched
    ob.block_table[20, :3] = [total - 1, 0, total - 2]
    bm = pool.block_manager
    bm.block_table.copy_(torch.from_numpy(ob.block_table))
    bm.num_seq_allocated_blocks.copy_(torch.from_numpy(ob.num_seq_allocated_blocks))
    bm.is_block_free.copy_(torch.from_numpy(ob.is_block_free))
    bm.num_free_blocks = ob.num_free_blocks
    return pool, ob, arena, lay


def pool_bytes(pool):
    parts = [pool.k_cache.reshape(-1), pool.v_cache.reshape(-1)]
    for k, v in zip(pool.k_cache_new, pool.v_cache_new):
        parts += [k.reshape(-1), v.reshape(-1)]
    return bits(torch.cat(parts))
