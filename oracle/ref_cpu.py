"""CPU restatement of the reference's paged-KV hot path (numpy / torch-CPU).

TEST INFRASTRUCTURE ONLY -- see ``oracle/__init__.py``.

Every function cites the reference lines it follows (paths are relative to the
reference checkout: ``MS/`` = ``MorphServe/``, ``CS/`` = ``csrc/src/``).

How each function is pinned (none of these checks retypes the formula under
test; they are in ``tests/test_oracle_*.py``):

* ``append_decode`` / ``append_prefill`` / ``PoolLayout.slab`` -- brute-force
  per-element loops written from the cache *shape* ``[blocks, L, Hkv, B, D]``
  (numpy fancy indexing on the 5-D view, not flat offsets), untouched-byte
  invariant, idempotence, permutation invariance of the logical content.
* segment addressing -- plain-vs-segment equivalence on an arena where the
  segments are placed by hand, plus hand-computed offsets.
* ``paged_attention`` -- textbook ``softmax(q K^T / sqrt(D)) V`` through
  ``torch.nn.functional.scaled_dot_product_attention`` on gathered KV, fp64
  numpy evaluation, closed forms (``len == 1`` gives ``V[0]``; equal keys give
  ``mean(V)``), split invariance, block-table permutation invariance.
* ``paged_attention_split`` -- equals the unsplit result for every split size.
* ``prefill_attention`` -- per-sequence dense causal softmax in fp64, last row
  equals decode attention over the same tokens.  The live reference call is the
  third-party ``vllm_flash_attn.flash_attn_varlen_func`` (>= 2.5.8, not
  vendored): parity with THAT library's rounding is unpinned; the function is
  pinned against textbook causal attention only.
* ``select_seq_block_size`` -- hand-computed known answers.
* ``BlockManagerOracle`` -- invariants (conservation, disjoint live rows,
  free-map consistency, ascending lowest-id allocation, stale rows after free)
  and hand-written scenarios.
* ``acquire_new_kvcache_arith`` -- hand-computed known answers.
* ``plan_migration`` / ``apply_migration`` -- no counterpart in the reference
  (it refuses to shrink a live segment, MS/server/memory_utils.py:529-544,
  :623-624).  Semantics are defined here; pinned by invariants (logical KV
  content preserved, all live ids below the new size, untouched blocks
  byte-identical, conservation of counters).
* ``coalesce_runs`` / ``swap_blocks`` -- per-block copies give the same bytes;
  swap-out then swap-in is the identity on logical content.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence, Tuple

import numpy as np

LOG2E = 1.442695040888963  # MS/worker/kernels/paged_attn.py:837


# --------------------------------------------------------------------------
# Pool addressing
# --------------------------------------------------------------------------
@dataclasses.dataclass
class PoolLayout:
    """Where K/V blocks live inside one flat fp16 ``arena`` (element offsets).

    Base pool: ``k_cache, v_cache : [num_blocks_org, L, Hkv, B, D]`` contiguous
    (MS/worker/model.py:180-190).  Extension segments of ``seg_blocks`` blocks
    each: block id ``>= num_blocks_org`` belongs to segment
    ``(id - org) // seg_blocks`` at local index ``id - org - seg * seg_blocks``;
    segment ``j`` starts ``j * org_layer_param_size`` ELEMENTS BELOW segment 0
    (MS/worker/kernels/kvcache_mgmt.py:169-183, :240-248;
    MS/worker/kernels/paged_attn.py:354-360).  ``k_seg`` / ``v_seg``, when given,
    replace the stride rule by an explicit per-segment offset table (the
    build's generalisation).
    """
    num_layers: int
    num_kv_heads: int
    block_size: int
    head_dim: int
    k_base: int
    v_base: int
    num_blocks_org: int
    seg_blocks: int = 0
    k_new0: int = 0
    v_new0: int = 0
    org_layer_param_size: int = 0
    k_seg: Optional[Sequence[int]] = None
    v_seg: Optional[Sequence[int]] = None

    @property
    def slab_elems(self) -> int:          # one (block, layer, head): [B, D]
        return self.block_size * self.head_dim

    @property
    def block_elems(self) -> int:         # one block, K only
        return self.num_layers * self.num_kv_heads * self.slab_elems

    def block_offset(self, which: str, block_id: int) -> int:
        """Element offset of block ``block_id`` of the K ('k') or V ('v') pool."""
        block_id = int(block_id)
        if block_id < self.num_blocks_org:
            base = self.k_base if which == "k" else self.v_base
            return base + block_id * self.block_elems
        seg = (block_id - self.num_blocks_org) // self.seg_blocks
        local = block_id - self.num_blocks_org - seg * self.seg_blocks
        if self.k_seg is not None:
            base = (self.k_seg if which == "k" else self.v_seg)[seg]
        else:
            new0 = self.k_new0 if which == "k" else self.v_new0
            base = new0 - seg * self.org_layer_param_size
        return base + local * self.block_elems

    def slab(self, which: str, block_id: int, layer: int, head: int = 0) -> int:
        """Element offset of ``cache[block_id, layer, head, 0, 0]``."""
        return (self.block_offset(which, block_id)
                + (layer * self.num_kv_heads + head) * self.slab_elems)


def plain_layout(num_blocks, num_layers, num_kv_heads, block_size, head_dim) -> PoolLayout:
    """Arena = K pool followed by V pool, no segments."""
    n = num_blocks * num_layers * num_kv_heads * block_size * head_dim
    return PoolLayout(num_layers, num_kv_heads, block_size, head_dim,
                      k_base=0, v_base=n, num_blocks_org=num_blocks)


# --------------------------------------------------------------------------
# KV append
# --------------------------------------------------------------------------
def append_decode(arena: np.ndarray, lay: PoolLayout, k: np.ndarray, v: np.ndarray,
                  block_table: np.ndarray, seq_ids: np.ndarray, seq_lens: np.ndarray,
                  layer: int) -> None:
    """MS/worker/kernels/kvcache_mgmt.py:52-81 (plain), :189-251 (segments).

    ``k, v : [n, Hkv, D]``; row i goes to position ``len_i - 1`` of sequence
    ``seq_ids[i]``: block ``(len-1)//B`` of its table row, slot ``(len-1)%B``.
    """
    B, D, H = lay.block_size, lay.head_dim, lay.num_kv_heads
    for i in range(len(seq_ids)):
        pos = int(seq_lens[i]) - 1
        pid = int(block_table[int(seq_ids[i]), pos // B])
        off = pos % B
        for h in range(H):
            ko = lay.slab("k", pid, layer, h) + off * D
            vo = lay.slab("v", pid, layer, h) + off * D
            arena[ko:ko + D] = k[i, h]
            arena[vo:vo + D] = v[i, h]


def append_prefill(arena: np.ndarray, lay: PoolLayout, k: np.ndarray, v: np.ndarray,
                   block_table: np.ndarray, seq_ids: np.ndarray,
                   start_locs: np.ndarray, seq_lens: np.ndarray, layer: int) -> None:
    """MS/worker/kernels/kvcache_mgmt.py:12-50 (plain), :84-187 (segments).

    ``k, v : [num_prefill_tokens, Hkv, D]``; token t of sequence b (row
    ``start_b + t``) goes to block ``t//B`` of the table row, slot ``t%B``,
    transposed from ``[tok, head]`` to ``[head, tok]`` order.
    """
    B, D, H = lay.block_size, lay.head_dim, lay.num_kv_heads
    for b in range(len(seq_ids)):
        start, n = int(start_locs[b]), int(seq_lens[b])
        row = block_table[int(seq_ids[b])]
        for t in range(n):
            pid = int(row[t // B])
            off = t % B
            for h in range(H):
                ko = lay.slab("k", pid, layer, h) + off * D
                vo = lay.slab("v", pid, layer, h) + off * D
                arena[ko:ko + D] = k[start + t, h]
                arena[vo:vo + D] = v[start + t, h]


def store_kvcache(arena, lay, k, v, block_table, seq_ids, num_prefill_seqs,
                  num_prefill_tokens, prefill_start_locs, prefill_lens,
                  decoding_lens, layer) -> None:
    """MS/worker/kernels/kvcache_mgmt.py:298-414: prefill rows first, decode rows
    are the tail slice ``k[num_prefill_tokens:]`` / ``seq_ids[num_prefill_seqs:]``."""
    if num_prefill_seqs > 0:
        append_prefill(arena, lay, k, v, block_table, seq_ids[:num_prefill_seqs],
                       prefill_start_locs, prefill_lens, layer)
    if len(seq_ids) - num_prefill_seqs > 0:
        append_decode(arena, lay, k[num_prefill_tokens:], v[num_prefill_tokens:],
                      block_table, seq_ids[num_prefill_seqs:], decoding_lens, layer)


# --------------------------------------------------------------------------
# Paged decode attention
# --------------------------------------------------------------------------
def gather_kv(arena: np.ndarray, lay: PoolLayout, block_table: np.ndarray,
              seq_id: int, seq_len: int, layer: int) -> Tuple[np.ndarray, np.ndarray]:
    """Gather one sequence's K and V as ``[Hkv, nblk*B, D]`` (whole blocks, the
    tail beyond ``seq_len`` included) -- MS/worker/kernels/paged_attn.py:1400-1409."""
    B, D, H = lay.block_size, lay.head_dim, lay.num_kv_heads
    nblk = -(-int(seq_len) // B)
    ks = np.empty((H, nblk * B, D), dtype=arena.dtype)
    vs = np.empty_like(ks)
    n = H * B * D
    for j in range(nblk):
        pid = int(block_table[int(seq_id), j])
        ko = lay.slab("k", pid, layer)
        vo = lay.slab("v", pid, layer)
        ks[:, j * B:(j + 1) * B] = arena[ko:ko + n].reshape(H, B, D)
        vs[:, j * B:(j + 1) * B] = arena[vo:vo + n].reshape(H, B, D)
    return ks, vs


def paged_attention(q: np.ndarray, arena: np.ndarray, lay: PoolLayout,
                    block_table: np.ndarray, seq_ids: np.ndarray, seq_lens: np.ndarray,
                    softmax_scale: float, layer: int, out_dtype=np.float16,
                    math: str = "torch32") -> np.ndarray:
    """The reference's own PyTorch statement of decode attention,
    MS/worker/kernels/paged_attn.py:1397-1432: gather blocks, repeat K/V heads
    for GQA, fp32 ``bmm``, scale, mask positions ``>= len`` to -1e20, softmax,
    ``bmm`` with V, cast to fp16.  ``q : [n, Hq, D]``; returns ``[n, Hq, D]``.

    ``math='torch32'`` runs exactly those torch-CPU ops; ``'np64'`` evaluates
    the same expression in float64 numpy (used for tolerance budgeting).
    """
    n, Hq, D = q.shape
    G = Hq // lay.num_kv_heads
    out = np.empty((n, Hq, D), dtype=out_dtype)
    if math == "torch32":
        import torch
    for i in range(n):
        L = int(seq_lens[i])
        ks, vs = gather_kv(arena, lay, block_table, int(seq_ids[i]), L, layer)
        if math == "torch32":
            tk = torch.from_numpy(ks).to(torch.float32).repeat_interleave(G, dim=0)
            tv = torch.from_numpy(vs).to(torch.float32).repeat_interleave(G, dim=0)
            tq = torch.from_numpy(q[i]).to(torch.float32).reshape(Hq, 1, D)
            s = torch.bmm(tq, tk.transpose(1, 2)).reshape(Hq, -1) * softmax_scale
            s = torch.where(torch.arange(s.shape[1]) < L, s, torch.full_like(s, -1e20))
            p = torch.softmax(s, dim=1).unsqueeze(1)
            res = torch.bmm(p, tv).squeeze(1)
            out[i] = res.numpy().astype(out_dtype)
        else:
            fk = np.repeat(ks.astype(np.float64), G, axis=0)
            fv = np.repeat(vs.astype(np.float64), G, axis=0)
            fq = q[i].astype(np.float64)
            s = np.einsum("hd,htd->ht", fq, fk) * softmax_scale
            s[:, L:] = -1e20
            s -= s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            out[i] = np.einsum("ht,htd->hd", p, fv).astype(out_dtype)
    return out


def paged_attention_split(q, arena, lay, block_table, seq_ids, seq_lens,
                          softmax_scale, layer, seq_block_size) -> np.ndarray:
    """Split-KV formulation: phase 1 MS/worker/kernels/paged_attn.py:59-240
    (per ``seq_block_size`` chunk: exp2 online softmax over 16-token blocks,
    emits normalised partial and ``log2(sum)+max``), phase 2 :658-696 (LSE
    merge).  Arithmetic in fp32 throughout -- the reference's fp16 ``q*k``
    product (:174, :207) is a known artefact that is deliberately not kept.
    Returns fp16 ``[n, Hq, D]``.
    """
    n, Hq, D = q.shape
    B = lay.block_size
    G = Hq // lay.num_kv_heads
    scale2 = np.float32(softmax_scale * LOG2E)
    out = np.empty((n, Hq, D), dtype=np.float16)
    for i in range(n):
        L = int(seq_lens[i])
        ks, vs = gather_kv(arena, lay, block_table, int(seq_ids[i]), L, layer)
        ks = ks.astype(np.float32)
        vs = vs.astype(np.float32)
        for hq in range(Hq):
            kvh = hq // G
            qv = q[i, hq].astype(np.float32)
            mids, lses = [], []
            for c0 in range(0, L, seq_block_size):
                c1 = min(c0 + seq_block_size, L)
                m = np.float32(-1e20)
                s_exp = np.float32(0.0)
                acc = np.zeros(D, dtype=np.float32)
                for b0 in range(c0, c1, B):
                    sc = (ks[kvh, b0:b0 + B] @ qv).astype(np.float32) * scale2
                    tok = np.arange(b0, b0 + B)
                    sc = np.where(tok < L, sc, np.float32(-1e20)).astype(np.float32)
                    m_new = np.maximum(m, sc.max())
                    e = np.exp2(sc - m_new).astype(np.float32)
                    old = np.exp2(m - m_new).astype(np.float32)
                    acc = acc * old + e @ vs[kvh, b0:b0 + B]
                    s_exp = s_exp * old + e.sum(dtype=np.float32)
                    m = m_new
                mids.append(acc / s_exp)
                lses.append(np.log2(s_exp) + m)
            m = np.float32(-1e20)
            s_exp = np.float32(0.0)
            acc = np.zeros(D, dtype=np.float32)
            for mid, lse in zip(mids, lses):
                m_new = np.maximum(m, lse)
                old = np.exp2(m - m_new).astype(np.float32)
                e = np.exp2(lse - m_new).astype(np.float32)
                acc = acc * old + e * mid
                s_exp = s_exp * old + e
                m = m_new
            out[i, hq] = (acc / s_exp).astype(np.float16)
    return out


def select_seq_block_size(num_kv_heads: int, decoding_seq_lens: Sequence[int]) -> Tuple[int, int]:
    """MS/worker/model.py:397-402, :426 -- returns ``(seq_block_size, num_seq_blocks)``."""
    sbs = 512
    total = sum(int(x) for x in decoding_seq_lens)
    mx = max((int(x) for x in decoding_seq_lens), default=0)
    while num_kv_heads * (total / sbs) < 1024 and sbs // 2 >= 64 and mx / (sbs // 2) <= 128:
        sbs //= 2
    return sbs, (mx + sbs - 1) // sbs


# --------------------------------------------------------------------------
# Prefill attention (causal, variable length, over the batch's own q/k/v)
# --------------------------------------------------------------------------
def prefill_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray,
                      start_locs: np.ndarray, seq_lens: np.ndarray,
                      softmax_scale: float, out_dtype=np.float16,
                      math: str = "np64") -> np.ndarray:
    """Causal attention per prefill sequence: formula of
    MS/worker/kernels/prefill_attn.py:45-100 (the live call site uses
    ``vllm_flash_attn.flash_attn_varlen_func``, causal,
    MS/worker/layers/transformer_layer.py:154-164).  ``q : [T, Hq, D]``,
    ``k, v : [T, Hkv, D]``; returns ``[T, Hq, D]``.
    """
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = np.zeros((T, Hq, D), dtype=out_dtype)
    if math == "torch32":
        # the same expression through torch-CPU fp32 matmuls (fast enough for 512-token prompts)
        import torch
        for b in range(len(seq_lens)):
            s0, n = int(start_locs[b]), int(seq_lens[b])
            tq = torch.from_numpy(q[s0:s0 + n]).to(torch.float32).permute(1, 0, 2)                      # [Hq,n,D]
            tk = torch.from_numpy(k[s0:s0 + n]).to(torch.float32).permute(1, 0, 2).repeat_interleave(G, 0)
            tv = torch.from_numpy(v[s0:s0 + n]).to(torch.float32).permute(1, 0, 2).repeat_interleave(G, 0)
            sc = torch.bmm(tq, tk.transpose(1, 2)) * softmax_scale
            keep = torch.tril(torch.ones(n, n, dtype=torch.bool))
            sc = torch.where(keep, sc, torch.full_like(sc, -1e20))
            res = torch.bmm(torch.softmax(sc, dim=2), tv).permute(1, 0, 2)
            out[s0:s0 + n] = res.numpy().astype(out_dtype)
        return out
    ft = np.float64 if math == "np64" else np.float32
    for b in range(len(seq_lens)):
        s0, n = int(start_locs[b]), int(seq_lens[b])
        qq = q[s0:s0 + n].astype(ft)                  # [n, Hq, D]
        kk = np.repeat(k[s0:s0 + n].astype(ft), G, axis=1)
        vv = np.repeat(v[s0:s0 + n].astype(ft), G, axis=1)
        s = np.einsum("qhd,khd->hqk", qq, kk) * ft(softmax_scale)
        mask = np.tril(np.ones((n, n), dtype=bool))
        s = np.where(mask[None], s, ft(-1e20))
        s -= s.max(axis=2, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=2, keepdims=True)
        out[s0:s0 + n] = np.einsum("hqk,khd->qhd", p, vv).astype(out_dtype)
    return out


def chunked_prefill_attention(q, arena, lay, block_table, seq_ids, chunk_start_locs,
                              chunk_lens, prefix_lens, softmax_scale, layer,
                              out_dtype=np.float16) -> np.ndarray:
    """Build-defined (the reference prefills whole prompts only,
    MS/server/engine.py:259-262): query chunk b holds tokens at positions
    ``prefix_b .. prefix_b + chunk_b - 1`` of sequence ``seq_ids[b]`` whose K/V
    for positions ``< prefix_b + chunk_b`` are ALREADY in the paged cache; token
    at position p attends to cached positions ``<= p``.  fp64 math.
    """
    T, Hq, D = q.shape
    G = Hq // lay.num_kv_heads
    out = np.zeros((T, Hq, D), dtype=out_dtype)
    for b in range(len(seq_ids)):
        s0, n, pre = int(chunk_start_locs[b]), int(chunk_lens[b]), int(prefix_lens[b])
        ks, vs = gather_kv(arena, lay, block_table, int(seq_ids[b]), pre + n, layer)
        kk = np.repeat(ks[:, :pre + n].astype(np.float64), G, axis=0)   # [Hq, ctx, D]
        vv = np.repeat(vs[:, :pre + n].astype(np.float64), G, axis=0)
        qq = q[s0:s0 + n].astype(np.float64)                             # [n, Hq, D]
        s = np.einsum("qhd,hkd->hqk", qq, kk) * softmax_scale
        pos_q = pre + np.arange(n)[:, None]
        mask = np.arange(pre + n)[None, :] <= pos_q
        s = np.where(mask[None], s, -1e20)
        s -= s.max(axis=2, keepdims=True)
        p = np.exp(s)
        p /= p.sum(axis=2, keepdims=True)
        out[s0:s0 + n] = np.einsum("hqk,hkd->qhd", p, vv).astype(out_dtype)
    return out


# --------------------------------------------------------------------------
# Block manager
# --------------------------------------------------------------------------
class BlockManagerOracle:
    """MS/worker/block_manager.py:18-136 with the three table kernels of
    MS/worker/kernels/block_mgmt.py:5-125 inlined as loops.

    State: ``num_seq_allocated_blocks [max_seqs]`` int32 zeros, ``block_table
    [max_seqs, max_blocks_per_seq]`` int32 filled -1, ``is_block_free
    [num_blocks]`` bool ones, counters.  Allocation hands out the lowest free
    ids in ascending order (``torch.nonzero(is_block_free)[:n]``, :75).  Freed
    rows keep their stale ids (block_mgmt.py:61-64).
    """

    def __init__(self, device_name, num_blocks, max_seqs_in_block_table,
                 max_blocks_per_seq, block_size):
        self.device_name = device_name
        self.num_free_blocks = num_blocks
        self.num_blocks = num_blocks
        self.block_size = block_size
        self.num_free_blocks_org = num_blocks
        self.num_blocks_org = num_blocks
        self.num_seq_allocated_blocks = np.zeros(max_seqs_in_block_table, dtype=np.int32)
        self.block_table = np.full((max_seqs_in_block_table, max_blocks_per_seq), -1, dtype=np.int32)
        self.is_block_free = np.ones(num_blocks, dtype=bool)

    def get_num_used_blocks(self) -> int:
        return self.num_blocks - self.num_free_blocks

    def _allocate_blocks(self, n: int) -> np.ndarray:
        if n > self.num_free_blocks:                      # block_manager.py:69-70
            raise RuntimeError(
                f"No enough free blocks available on {self.device_name} "
                f"({self.num_blocks} in total, {self.num_free_blocks} free, {n} requested)")
        sel = np.nonzero(self.is_block_free)[0][:n].astype(np.int64)
        self.num_free_blocks -= n
        self.is_block_free[sel] = False
        return sel

    def allocate_blocks_for_seqs(self, seq_ids, target_lens) -> np.ndarray:
        seq_ids = np.asarray(seq_ids, dtype=np.int64)
        target = (np.asarray(target_lens, dtype=np.int64) + (self.block_size - 1)) // self.block_size
        have = self.num_seq_allocated_blocks[seq_ids].astype(np.int64)
        assert (have <= target).all(), "Logic error: Some sequences have more blocks already allocated than needed."
        need = target - have
        total = int(need.sum())
        if total == 0:
            return np.empty(0, dtype=np.int64)
        new = self._allocate_blocks(total)
        cum = np.cumsum(need)
        for i, s in enumerate(seq_ids):                   # block_mgmt.py:16-24
            start = cum[i] - need[i]
            a = int(self.num_seq_allocated_blocks[s])
            self.block_table[s, a:a + need[i]] = new[start:start + need[i]]
            self.num_seq_allocated_blocks[s] = a + need[i]
        return new

    def free_blocks_for_seqs(self, seq_ids) -> None:
        seq_ids = np.asarray(seq_ids, dtype=np.int64)
        self.num_free_blocks += int(self.num_seq_allocated_blocks[seq_ids].sum())
        for s in seq_ids:                                 # block_mgmt.py:58-64
            a = int(self.num_seq_allocated_blocks[s])
            self.is_block_free[self.block_table[s, :a]] = True
            self.num_seq_allocated_blocks[s] = 0

    def gather_allocated_blocks_and_free(self, seq_ids) -> np.ndarray:
        seq_ids = np.asarray(seq_ids, dtype=np.int64)
        out: List[int] = []
        for s in seq_ids:                                 # block_mgmt.py:96-104
            a = int(self.num_seq_allocated_blocks[s])
            ids = self.block_table[s, :a]
            out.extend(int(x) for x in ids)
            self.is_block_free[ids] = True
            self.num_seq_allocated_blocks[s] = 0
        self.num_free_blocks += len(out)
        return np.asarray(out, dtype=np.int32)

    def get_num_allocated_blocks(self, seq_ids) -> np.ndarray:
        return self.num_seq_allocated_blocks[np.asarray(seq_ids, dtype=np.int64)].copy()

    # -- elastic pool bookkeeping ------------------------------------------
    def expand(self, seg_blocks: int) -> None:
        """MS/server/memory_utils.py:405-417: one more segment of free blocks."""
        self.num_blocks += seg_blocks
        self.num_free_blocks += seg_blocks
        self.is_block_free = np.concatenate([self.is_block_free, np.ones(seg_blocks, dtype=bool)])

    def tail_segment_unused(self, seg_blocks: int, num_segments: int) -> bool:
        """MS/server/memory_utils.py:529-544."""
        lo = self.num_blocks_org + seg_blocks * (num_segments - 1)
        return bool(self.is_block_free[lo:lo + seg_blocks].all())

    def shrink(self, seg_blocks: int, num_segments: int) -> bool:
        """MS/server/memory_utils.py:623-624, :648-650: drop the last segment,
        refused (returns False, state unchanged) when any of its blocks is live."""
        if not self.tail_segment_unused(seg_blocks, num_segments):
            return False
        self.num_blocks -= seg_blocks
        self.num_free_blocks -= seg_blocks
        self.is_block_free = self.is_block_free[:-seg_blocks]
        return True

    def snapshot(self) -> dict:
        return dict(block_table=self.block_table.copy(),
                    num_seq_allocated_blocks=self.num_seq_allocated_blocks.copy(),
                    is_block_free=self.is_block_free.copy(),
                    num_blocks=int(self.num_blocks), num_free_blocks=int(self.num_free_blocks))


def acquire_new_kvcache_arith(layer_base: int, org_bytes: int, quant_bytes: int,
                              num_layers: int, num_kv_heads: int, block_size: int,
                              head_dim: int) -> Tuple[int, int, int]:
    """CS/memory_manager.cpp:84-97, :145 -- returns ``(k_start_addr, S, v_start_addr)``
    in bytes; raises when no block fits (:99-101)."""
    layer_end = layer_base + quant_bytes
    start = (layer_end + 255) & ~255
    avail = org_bytes - (start - layer_base)
    kv_slot = 2 * num_layers * num_kv_heads * head_dim * 2
    kv_block = kv_slot * block_size
    S = avail // kv_block if avail > 0 else 0
    if S == 0:
        raise RuntimeError("No space available for new KV cache blocks")
    return start, S, start + S * (kv_block // 2)


# --------------------------------------------------------------------------
# Shrink with live-block migration (build-defined; absent from the reference)
# --------------------------------------------------------------------------
def plan_migration(is_block_free: np.ndarray, new_num_blocks: int) -> Tuple[np.ndarray, np.ndarray]:
    """Moves needed so that no live block has id ``>= new_num_blocks``:
    ``src`` = ascending live ids ``>= new_n``; ``dst`` = the first ``len(src)``
    free ids ``< new_n`` ascending (the allocator's own lowest-first policy,
    MS/worker/block_manager.py:75).  Raises when they do not fit."""
    free = np.asarray(is_block_free, dtype=bool)
    src = np.nonzero(~free[new_num_blocks:])[0].astype(np.int64) + new_num_blocks
    cand = np.nonzero(free[:new_num_blocks])[0].astype(np.int64)
    if len(src) > len(cand):
        raise RuntimeError(
            f"cannot shrink to {new_num_blocks} blocks: {len(src)} live blocks to move, "
            f"{len(cand)} free below the cut")
    return src, cand[:len(src)]


def apply_migration(arena: np.ndarray, lay: PoolLayout, bm: BlockManagerOracle,
                    new_num_blocks: int) -> Tuple[np.ndarray, np.ndarray]:
    """Shrink ``bm`` to ``new_num_blocks`` relocating live blocks: copy K and V
    of every move (all layers), rewrite live table entries ``bt[s, j <
    n_alloc[s]]`` through the remap, mark destinations used, truncate the free
    map, update counters.  Stale entries of freed rows are left as they are."""
    src, dst = plan_migration(bm.is_block_free, new_num_blocks)
    n = lay.block_elems
    for s, d in zip(src, dst):
        for which in ("k", "v"):
            so = lay.block_offset(which, s)
            do = lay.block_offset(which, d)
            arena[do:do + n] = arena[so:so + n]
    remap = {int(s): int(d) for s, d in zip(src, dst)}
    for row in range(bm.block_table.shape[0]):
        a = int(bm.num_seq_allocated_blocks[row])
        for j in range(a):
            b = int(bm.block_table[row, j])
            if b in remap:
                bm.block_table[row, j] = remap[b]
    bm.is_block_free[dst] = False
    removed = bm.num_blocks - new_num_blocks
    # every removed id is free after the moves; moved-to ids stop being free
    bm.num_free_blocks = int(bm.num_free_blocks) - removed
    bm.is_block_free = bm.is_block_free[:new_num_blocks].copy()
    bm.num_blocks = new_num_blocks
    return src, dst


# --------------------------------------------------------------------------
# Eviction (device <-> host swap space)
# --------------------------------------------------------------------------
def coalesce_runs(src: Sequence[int], dst: Sequence[int],
                  src_seg: Optional[Sequence[int]] = None,
                  dst_seg: Optional[Sequence[int]] = None) -> List[Tuple[int, int, int]]:
    """CS/block_swapping.cpp:36-44 (plain) and :138-147 (segment flags): greedy
    runs where source AND target ids are consecutive (and stay in one segment).
    Returns ``[(src_start, dst_start, run_len), ...]``."""
    runs = []
    i, n = 0, len(src)
    while i < n:
        j = i + 1
        while (j < n and src[j] == src[j - 1] + 1 and dst[j] == dst[j - 1] + 1
               and (src_seg is None or src_seg[j] == src_seg[j - 1])
               and (dst_seg is None or dst_seg[j] == dst_seg[j - 1])):
            j += 1
        runs.append((int(src[i]), int(dst[i]), j - i))
        i = j
    return runs


def swap_blocks(arena: np.ndarray, lay: PoolLayout, k_swap: np.ndarray, v_swap: np.ndarray,
                src: Sequence[int], dst: Sequence[int], is_swap_in: bool) -> None:
    """CS/block_swapping.cpp:22-85 and the evident intent of :88-202: copy whole
    blocks between the device pool (addressed through ``lay``, segments
    included) and the host swap tensors ``[num_cpu_blocks, L, Hkv, B, D]``.
    Swap-in writes the DEVICE block ``dst[i]`` from host block ``src[i]`` (the
    combined variant of the reference computes that device address from the
    source id, block_swapping.cpp:156-160 -- a defect that is not restated)."""
    n = lay.block_elems
    ks = k_swap.reshape(-1)
    vs = v_swap.reshape(-1)
    for s, d in zip(src, dst):
        s, d = int(s), int(d)
        if is_swap_in:
            ko, vo = lay.block_offset("k", d), lay.block_offset("v", d)
            arena[ko:ko + n] = ks[s * n:(s + 1) * n]
            arena[vo:vo + n] = vs[s * n:(s + 1) * n]
        else:
            ko, vo = lay.block_offset("k", s), lay.block_offset("v", s)
            ks[d * n:(d + 1) * n] = arena[ko:ko + n]
            vs[d * n:(d + 1) * n] = arena[vo:vo + n]
