/*
 * morphkv -- C ABI of the MI355X (gfx950) paged-KV hot path.
 *
 * One shared library, plain pointers and sizes, no torch types.  Every entry
 * point returns 0 on success or a negative MKV_E* code (mkv_last_error() gives
 * the text), never throws, launches on the hipStream_t passed last (as void*),
 * and does not synchronise unless its name ends in _sync.  All pointers are
 * device pointers unless the comment says "host".
 *
 * Citations name the reference interface each entry point replaces
 * (MS/ = MorphServe/, CS/ = csrc/src/ in the reference checkout).
 *
 * Cache layout everywhere: k_cache, v_cache : [num_blocks, L, Hkv, B, D] fp16,
 * contiguous, K and V separate (MS/worker/model.py:180-190).  block_table :
 * [max_seqs, max_blocks_per_seq] int32.
 */
#ifndef MORPHKV_H
#define MORPHKV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MKV_OK            0
#define MKV_EINVAL       -1   /* bad argument / unsupported shape          */
#define MKV_EHIP         -2   /* a HIP runtime call failed                 */
#define MKV_ENOSPC       -3   /* not enough free blocks / does not fit     */
#define MKV_ELOGIC       -4   /* allocator precondition violated           */

#define MKV_MAX_SEGMENTS 128

/*
 * Where blocks live.  Ids < num_blocks_org address the base pool; an id beyond
 * it belongs to extension segment (id - org) / seg_blocks at local index
 * (id - org) % seg_blocks (MS/worker/kernels/kvcache_mgmt.py:169-183,
 * MS/worker/kernels/paged_attn.py:354-360).  The reference passes segment 0
 * only and reaches segment j at "- j * org_layer_param_size" elements; the
 * caller expands that rule into k_seg[j] / v_seg[j] (mkv_pool_set_strided does
 * it), so any placement of segments is expressible.
 */
typedef struct mkv_pool {
    void*   k_base;
    void*   v_base;
    int64_t num_blocks_org;
    int64_t seg_blocks;        /* S; 0 when there are no segments */
    int32_t num_segments;
    int32_t num_layers;        /* L   */
    int32_t num_kv_heads;      /* Hkv */
    int32_t block_size;        /* B   */
    int32_t head_dim;          /* D   */
    int32_t _pad;
    void*   k_seg[MKV_MAX_SEGMENTS];
    void*   v_seg[MKV_MAX_SEGMENTS];
} mkv_pool;

/* ---- library ---------------------------------------------------------- */
const char* mkv_last_error(void);           /* host string, thread-local    */
int  mkv_version(void);
int  mkv_sizeof_pool(void);                 /* sizeof(mkv_pool), for binding checks */
/* Fill k_seg/v_seg from the reference's calling convention: segment j at
 * k_new0 - j * org_layer_param_size * elem_bytes (same for V).
 * CS/block_swapping.cpp:156-160, MS/worker/kernels/kvcache_mgmt.py:177-183. */
int  mkv_pool_set_strided(mkv_pool* pool, void* k_new0, void* v_new0,
                          int64_t org_layer_param_size, int32_t elem_bytes,
                          int32_t num_segments);

/* ---- KV append -------------------------------------------------------- */
/* _fwd_kvcache_mgmt_decoding_kernel{,_new_kv_combined},
 * MS/worker/kernels/kvcache_mgmt.py:52-81, :189-251.
 * k, v : [n, Hkv, D] fp16; row i is written at position seq_lens[i]-1 of
 * sequence seq_ids[i]. */
int mkv_append_decode(const void* k, const void* v, const mkv_pool* pool,
                      const int32_t* block_table, int64_t max_blocks_per_seq,
                      const int32_t* seq_ids, const int32_t* seq_lens,
                      int32_t n, int32_t layer, void* stream);

/* _fwd_kvcache_mgmt_prefill_kernel{,_new_kv_combined},
 * MS/worker/kernels/kvcache_mgmt.py:12-50, :84-187.
 * k, v : [num_prefill_tokens, Hkv, D] fp16. */
int mkv_append_prefill(const void* k, const void* v, const mkv_pool* pool,
                       const int32_t* block_table, int64_t max_blocks_per_seq,
                       const int32_t* seq_ids, const int32_t* start_locs,
                       const int32_t* seq_lens, int32_t num_seqs,
                       int32_t max_len, int32_t layer, void* stream);

/* ---- paged decode attention -------------------------------------------- */
/* Scratch the caller must provide for n sequences, Hq heads and up to
 * max_splits splits: returns bytes for mid_o (fp32 [n,Hq,max_splits,D]) and
 * mid_lse (fp32 [n,Hq,max_splits]).  Replaces the per-call torch.empty of
 * MS/worker/kernels/paged_attn.py:780-793. */
int mkv_paged_attn_scratch_bytes(int32_t n, int32_t num_q_heads, int32_t head_dim,
                                 int32_t max_splits, int64_t* mid_o_bytes,
                                 int64_t* mid_lse_bytes);

/* paged_attention = phase 1 + phase 2, MS/worker/kernels/paged_attn.py:59-240,
 * :243-437, :658-696, :700-1015.  q : [n, Hq, D] fp16, o : [n, Hq, D] fp16.
 * A sequence is cut into splits of tokens_per_split tokens (a multiple of the
 * block size); max_splits >= ceil(max_len / tokens_per_split) sizes the scratch
 * rows.  softmax_scale is 1/sqrt(D); the kernel works in base 2. fp32
 * accumulation throughout.  Limits (MKV_EINVAL otherwise): head_dim 128,
 * block_size 16, num_q_heads / num_kv_heads from 1 to 16, q 16-byte aligned,
 * mid_o 16-byte aligned; mid_o / mid_lse may be NULL when max_splits is 1. */
int mkv_paged_attn_decode(const void* q, void* o, const mkv_pool* pool,
                          const int32_t* block_table, int64_t max_blocks_per_seq,
                          const int32_t* seq_ids, const int32_t* seq_lens,
                          int32_t n, int32_t num_q_heads, float softmax_scale,
                          int32_t layer, int32_t tokens_per_split, int32_t max_splits,
                          void* mid_o, void* mid_lse, void* stream);

/* mkv_paged_attn_decode for callers that cannot allocate device memory and have no
 * workspace to pass: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference (which allocates its
 * partials with torch.empty on every call, MS/worker/kernels/paged_attn.py:780-793).
 * The split partials (mid_o, mid_lse) live in a 16 MiB array built into the library's
 * device code, one copy per GPU, held until the process ends; the call performs no
 * hipMalloc / hipFree and calls no allocating routine.  Same kernels, same results
 * as mkv_paged_attn_decode.  MKV_EINVAL with a message when
 * n * num_q_heads * max_splits * (128 + 1) * 4 bytes exceed 16 MiB (max_splits == 1
 * needs no scratch and always fits).  Every call on a GPU shares that GPU's array:
 * calls that may overlap on one GPU (different streams, different threads) race;
 * nothing in it has to start at zero, so nothing is cleared between calls.  The
 * device current at the call must be the stream's device. */
int mkv_paged_attn_decode_static(const void* q, void* o, const mkv_pool* pool,
                                 const int32_t* block_table, int64_t max_blocks_per_seq,
                                 const int32_t* seq_ids, const int32_t* seq_lens,
                                 int32_t n, int32_t num_q_heads, float softmax_scale,
                                 int32_t layer, int32_t tokens_per_split, int32_t max_splits,
                                 void* stream);

/* store_kvcache (decode rows) + paged_attention of one layer in ONE launch: the
 * call pair of MS/worker/layers/transformer_layer.py:116-126, :181-187 for a
 * decode batch.  k, v : [n, Hkv, D] fp16 is token seq_lens[i]-1 of each
 * sequence; it is written to its cache slot exactly as mkv_append_decode would
 * and takes part in the attention from registers.  Other arguments as
 * mkv_paged_attn_decode. */
int mkv_decode_append_attn(const void* k, const void* v, const void* q, void* o,
                           const mkv_pool* pool, const int32_t* block_table,
                           int64_t max_blocks_per_seq, const int32_t* seq_ids,
                           const int32_t* seq_lens, int32_t n, int32_t num_q_heads,
                           float softmax_scale, int32_t layer, int32_t tokens_per_split,
                           int32_t max_splits, void* mid_o, void* mid_lse, void* stream);

/* rotary_embedding_inplace (decode rows) + store_kvcache + paged_attention of one
 * layer in ONE launch: MS/worker/layers/transformer_layer.py:93-126, :181-187
 * for a decode batch.  q and k arrive UNROTATED; row i of cos_table / sin_table
 * ([n, D/2] fp16) belongs to sequence i's new token.  q and the new k row are
 * rotated on their way in (arithmetic of mkv_rope_store_kvcache), the rotated k
 * row and the v row are written to the cache, attention uses both.  Unlike the
 * separate rotary call, q and k themselves are left as they were. */
int mkv_decode_rope_append_attn(const void* k, const void* v, const void* q,
                                const void* cos_table, const void* sin_table, void* o,
                                const mkv_pool* pool, const int32_t* block_table,
                                int64_t max_blocks_per_seq, const int32_t* seq_ids,
                                const int32_t* seq_lens, int32_t n, int32_t num_q_heads,
                                float softmax_scale, int32_t layer, int32_t tokens_per_split,
                                int32_t max_splits, void* mid_o, void* mid_lse, void* stream);

/* No counterpart in the reference (its kernels take the batch in the caller's order,
 * MS/worker/kernels/paged_attn.py:59-77).  order[slot] = row of the decode batch that the
 * workgroups at grid slot `slot` should take: the rows by descending length, dealt in snake order
 * over runs of 256 / num_kv_heads slots, so that the workgroups sharing a CU stream about the same
 * number of tokens.  It depends on seq_lens only: compute it once per batch and pass it to every
 * layer's mkv_decode_attn_ordered.  n <= 4096. */
int mkv_decode_order(const int32_t* seq_lens, int32_t n, int32_t num_kv_heads,
                     int32_t* order, void* stream);

/* mkv_paged_attn_decode / mkv_decode_append_attn / mkv_decode_rope_append_attn in one entry, with the
 * order in which the grid takes the batch rows: order = NULL keeps the rows' own order (any
 * permutation of 0..n-1 gives the same outputs); k, v = NULL: no append; cos_table, sin_table = NULL:
 * no rotary (they need k, v).  Everything else as in the three entries above. */
int mkv_decode_attn_ordered(const void* q, void* o, const mkv_pool* pool,
                            const int32_t* block_table, int64_t max_blocks_per_seq,
                            const int32_t* seq_ids, const int32_t* seq_lens,
                            const int32_t* order, int32_t n, int32_t num_q_heads,
                            float softmax_scale, int32_t layer, int32_t tokens_per_split,
                            int32_t max_splits, void* mid_o, void* mid_lse,
                            const void* k, const void* v, const void* cos_table,
                            const void* sin_table, void* stream);

/* ---- prefill attention -------------------------------------------------- */
/* prefill_attention, MS/worker/kernels/prefill_attn.py:9-139, and the live
 * flash_attn_varlen_func call, MS/worker/layers/transformer_layer.py:154-164:
 * causal attention of each prefill sequence over its own contiguous q, k, v.
 * q, o : [T, Hq, D] fp16; k, v : [T, Hkv, D] fp16; all four 16-byte aligned. */
int mkv_prefill_attn(const void* q, const void* k, const void* v, void* o,
                     const int32_t* start_locs, const int32_t* seq_lens,
                     int32_t num_seqs, int32_t max_len, int32_t num_q_heads,
                     int32_t num_kv_heads, int32_t head_dim, float softmax_scale,
                     void* stream);

/* Chunked prefill over the paged cache.  No counterpart in the reference, which
 * prefills whole prompts over the batch's own k, v (MS/server/engine.py:259-262,
 * MS/worker/layers/transformer_layer.py:151-164).  Chunk b holds chunk_lens[b]
 * query rows at positions prefix_lens[b] .. of sequence seq_ids[b]; K/V of every
 * position up to the chunk's end are already in the cache (append first); row at
 * position p attends to cached positions <= p.  prefix_lens may be NULL (= 0).
 * max_prefix_len is a host-side upper bound of prefix_lens used only to choose the
 * launch shape (0 = unknown; results do not depend on it).  q and o 16-byte aligned. */
int mkv_prefill_attn_paged(const void* q, void* o, const mkv_pool* pool,
                           const int32_t* block_table, int64_t max_blocks_per_seq,
                           const int32_t* seq_ids, const int32_t* start_locs,
                           const int32_t* chunk_lens, const int32_t* prefix_lens,
                           int32_t num_seqs, int32_t max_chunk_len, int32_t max_prefix_len,
                           int32_t num_q_heads, float softmax_scale, int32_t layer, void* stream);

/* ---- block manager ------------------------------------------------------ */
/* BlockManager.allocate_blocks_for_seqs, MS/worker/block_manager.py:64-112 with
 * set_block_table_and_num_seq_alloc_blocks, MS/worker/kernels/block_mgmt.py:5-46,
 * as ONE launch: need_i = ceil(target_lens[i]/B) - n_alloc[seq_ids[i]]; the
 * sum(need) lowest free ids ascending are marked used, written to new_ids
 * (int64, capacity new_ids_cap) and appended to the table rows in batch order.
 * result (3 x int64, device) receives {total_need, status, free_found}; status
 * 0 ok, MKV_ELOGIC if some need_i < 0, MKV_EINVAL if a seq id is outside
 * [0, max_seqs) or a target needs more than max_blocks_per_seq blocks,
 * MKV_ENOSPC if fewer than total_need
 * blocks are free or total_need > new_ids_cap; on a non-zero status no state
 * is modified. */
int mkv_bm_allocate(int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                    int32_t* block_table, int64_t max_blocks_per_seq,
                    uint8_t* is_block_free, int64_t num_blocks, const int32_t* seq_ids,
                    const int32_t* target_lens, int32_t batch, int32_t block_size,
                    int64_t* new_ids, int64_t new_ids_cap, int64_t* result,
                    void* stream);

/* torch.nonzero(is_block_free)[:n] + mark used, MS/worker/block_manager.py:75-77.
 * result (2 x int64, device) receives {found, status}. */
int mkv_bm_take_first_free(uint8_t* is_block_free, int64_t num_blocks, int64_t n,
                           int64_t* ids_out, int64_t* result, void* stream);

/* set_block_table_and_num_seq_alloc_blocks, MS/worker/kernels/block_mgmt.py:26-46.
 * candidate_blocks int64 [sum(block_needed)], block_needed int32 or int64
 * [batch] (needed_is_i64 selects). */
int mkv_bt_append(int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                  int32_t* block_table, int64_t max_blocks_per_seq,
                  const int64_t* candidate_blocks,
                  const int32_t* seq_ids, const void* block_needed,
                  int32_t needed_is_i64, int32_t batch, void* stream);

/* unset_block_table_and_num_seq_alloc_blocks, MS/worker/kernels/block_mgmt.py:49-80.
 * freed_total (1 x int64, device, may be NULL) receives sum of released counts. */
int mkv_bt_release(int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                   const int32_t* block_table, int64_t max_blocks_per_seq,
                   const int32_t* seq_ids, int32_t batch, uint8_t* is_block_free,
                   int64_t num_blocks, int64_t* freed_total, void* stream);

/* gather_allocated_blocks_and_unset, MS/worker/kernels/block_mgmt.py:83-125.
 * gathered int32 [capacity]; result (2 x int64, device) receives {total, status}
 * (MKV_ENOSPC and nothing modified when total > capacity). */
int mkv_bt_gather_release(int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                          const int32_t* block_table, int64_t max_blocks_per_seq,
                          const int32_t* seq_ids, int32_t batch, uint8_t* is_block_free,
                          int64_t num_blocks, int32_t* gathered, int64_t capacity,
                          int64_t* result, void* stream);

/* ---- elastic pool -------------------------------------------------------- */
/* MemoryManager::acquire_new_kvcache arithmetic, CS/memory_manager.cpp:84-101,
 * :145 (host, no GPU work): from a weight layer region [layer_base, +org_bytes)
 * whose first quant_bytes stay in use, the 256-byte aligned K start, the number
 * of blocks S that fit and the V start.  MKV_ENOSPC when S == 0. */
int mkv_pool_carve_segment(uint64_t layer_base, uint64_t org_bytes, uint64_t quant_bytes,
                           int32_t num_layers, int32_t num_kv_heads, int32_t block_size,
                           int32_t head_dim, uint64_t* k_start, int64_t* seg_blocks,
                           uint64_t* v_start);

/* k_cache.zero_() / v_cache.zero_() of new pool memory,
 * CS/memory_manager.cpp:162-163, MS/worker/model.py:189-190. */
int mkv_fill_zero(void* ptr, uint64_t bytes, void* stream);

/* if_kv_cache_unused, MS/server/memory_utils.py:529-544: result (1 x int64,
 * device) receives the number of live (not free) blocks in [lo, hi). */
int mkv_bm_count_live(const uint8_t* is_block_free, int64_t lo, int64_t hi,
                      int64_t* result, void* stream);

/* Shrink with live-block migration.  No counterpart in the reference, which
 * refuses to shrink a live tail segment (MS/server/memory_utils.py:623-624).
 * Plan: src = ascending live ids >= new_num_blocks, dst = the lowest free ids
 * < new_num_blocks ascending (the allocator's policy,
 * MS/worker/block_manager.py:75).  Writes src/dst (int64, capacity cap),
 * remap (int32 [num_blocks], identity except remap[src_k] = dst_k), marks dst
 * used; result (3 x int64, device) = {moves, status, free_below}.  On
 * MKV_ENOSPC nothing is modified. */
int mkv_pool_plan_shrink(uint8_t* is_block_free, int64_t num_blocks,
                         int64_t new_num_blocks, int64_t* src, int64_t* dst,
                         int64_t cap, int32_t* remap, int64_t* result, void* stream);

/* Copy K and V of block src[k] to block dst[k], all layers, for k < num_moves
 * (num_moves read on the host by the caller from mkv_pool_plan_shrink's
 * result). */
int mkv_pool_migrate(const mkv_pool* pool, const int64_t* src, const int64_t* dst,
                     int64_t num_moves, void* stream);

/* Rewrite live table entries bt[s, j < n_alloc[s]] through remap. */
int mkv_bt_remap(int32_t* block_table, int64_t max_blocks_per_seq,
                 const int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                 const int32_t* remap, int64_t num_blocks, void* stream);

/* ---- pool backing through virtual memory ---------------------------------- */
/* Where the reference grows the pool with tensor views over freed weight memory
 * (acquire_new_kvcache, CS/memory_manager.cpp:69-176) and drops them again
 * (free_kv_cache_tensors, MS/server/memory_utils.py:602-610), an arena reserves
 * reserve_bytes of device ADDRESS space once and maps physical chunks of
 * chunk_bytes at its end: a pool built on it is one contiguous
 * [num_blocks, L, Hkv, B, D] tensor at a fixed address whatever its size, with
 * no extension segments.  mkv_arena_resize maps or unmaps whole chunks at the
 * end (host call; the caller makes sure no kernel still uses memory it gives
 * back); MKV_ENOSPC when the device has no memory left (nothing changed).
 * chunk_bytes: a multiple of the device's allocation granularity, and of 2 MiB when
 * it is larger than that (chunks are mapped back to back, and the driver has refused
 * access rights for a 574.5 MiB chunk mapped off a 2 MiB boundary). */
typedef struct mkv_arena mkv_arena;
int mkv_arena_create(uint64_t reserve_bytes, uint64_t chunk_bytes, mkv_arena** out);
int mkv_arena_info(const mkv_arena* arena, void** base, uint64_t* reserved_bytes,
                   uint64_t* chunk_bytes, uint64_t* mapped_bytes);
int mkv_arena_resize(mkv_arena* arena, uint64_t mapped_bytes);
int mkv_arena_destroy(mkv_arena* arena);
/* The reference's pool grows out of the memory a replaced layer no longer needs
 * (the bytes of org_range beyond the quantized copy, CS/memory_manager.cpp:69-97)
 * and that memory serves the restored layer again afterwards
 * (replace_layer_quant2org after free_kv_cache_tensors, MS/server/memory_utils.py:630-635).
 * With arenas the same hand-over moves physical chunks: the last `bytes` mapped in
 * `from` are unmapped there and mapped at the end of `to` -- no allocation, no
 * free, no copy; the chunks keep their contents (the receiver clears what it
 * needs cleared).  Same chunk size and device for both; host call, the caller
 * makes sure no kernel still uses the moved range.  On a failed mapping the
 * chunk in hand returns to `from`, chunks already moved stay in `to`
 * (mkv_arena_info tells how far it got). */
int mkv_arena_move_tail(mkv_arena* from, mkv_arena* to, uint64_t bytes);
/* Pool creation and growth that choose WHICH physical memory backs K and which backs V.  The
 * reference allocates k_cache and v_cache one after the other (MS/worker/model.py:187-190) and
 * carves K and V of a new segment out of one range (CS/memory_manager.cpp:120-145), so where they
 * lie is the driver's choice.  On an MI355X that choice matters: its memory behaves as three groups
 * of 96 GiB, the migration copy of a shrink runs at 65 % of the HBM peak when the K and the V
 * destinations share a group and at 78 % when they do not, and the decode gather is fastest over a
 * pool that touches at most two groups.  mkv_arena_pair_grow maps k_add_bytes more at the end of
 * `k` and v_add_bytes more at the end of `v` (both arenas of one pool: same chunk size and device)
 * with K chunks from one group and V chunks from another.  The call that creates the pool (both
 * arenas empty) creates candidate chunks until it holds enough of two groups (at most budget_bytes
 * of them at a time, 0 = all free device memory but 4 GiB), tells their groups apart by the rate of
 * a store-only kernel that fills a candidate and a reference side by side (a relative measurement:
 * no absolute rate is assumed, and a device without such groups yields one group and the plain
 * order), keeps what it needs and gives the rest back (info->released_bytes: the driver wipes
 * released memory in the background, about 30 ms per GiB, and kernels run a few per cent slower
 * while it does).  Where an arena can still grow it also keeps one spare chunk of its group as the
 * reference for later calls (held until mkv_arena_destroy); a later call creates exactly the chunks
 * it needs, measures them against those references and gives each arena the ones of its own group
 * first.  Chunks under 256 MiB cannot be measured: plain growth.
 * Host call; it synchronises `stream`, on which the measurement kernels run; the new memory holds
 * whatever the measurement left (the caller clears it, as after mkv_arena_resize).  MKV_ENOSPC when
 * the device has no memory left (nothing changed).  `info` (may be NULL) reports what was found. */
typedef struct mkv_pair_info {
    int32_t groups_found;   /* 0: not measured (plain growth), 1: one group only, 2 or 3 */
    int32_t candidates;     /* physical chunks created by the call */
    int32_t k_chunks, v_chunks;         /* chunks mapped into k / v */
    int32_t k_in_group, v_in_group;     /* ... of which in the arena's own group */
    int32_t probes;         /* measurement launches (x 3) */
    int32_t _pad;
    double probe_ms;        /* GPU time of the measurement */
    double total_ms;        /* host time of the call */
    uint64_t released_bytes;/* candidate memory given back to the driver at the end of the call */
} mkv_pair_info;
int mkv_arena_pair_grow(mkv_arena* k, mkv_arena* v, uint64_t k_add_bytes, uint64_t v_add_bytes,
                        uint64_t budget_bytes, void* stream, mkv_pair_info* info);

/* ---- rotary embedding, optionally fused with the append --------------------- */
/* rotary_embedding_inplace, MS/worker/kernels/rotary_emb.py:7-58: q [T, Hq, D] and
 * k [T, Hkv, D] are rotated in place with row t of cos / sin [T, D/2] (all fp16;
 * pairs are (d, d + D/2)).  With store != 0 the same launch also does what
 * store_kvcache does next (MS/worker/layers/transformer_layer.py:93-126,
 * kvcache_mgmt.py:321-343): the rotated k row and the v row of every token are
 * written to the token's cache slot -- prefill rows t < num_prefill_tokens at
 * position t - start of their sequence, decode rows at position len - 1; row
 * arguments as for mkv_append_prefill / mkv_append_decode, seq_ids holding the
 * prefill sequences first.  With store == 0 pool, v and the row arguments are
 * ignored. */
int mkv_rope_store_kvcache(void* q, void* k, const void* v, const void* cos_table,
                           const void* sin_table, const mkv_pool* pool,
                           const int32_t* block_table, int64_t max_blocks_per_seq,
                           const int32_t* seq_ids, const int32_t* prefill_start_locs,
                           const int32_t* prefill_lens, const int32_t* decoding_seq_lens,
                           int32_t num_prefill_seqs, int32_t num_prefill_tokens,
                           int32_t num_decoding_seqs, int32_t num_q_heads,
                           int32_t num_kv_heads, int32_t head_dim, int32_t layer,
                           int32_t store, void* stream);

/* ---- eviction ------------------------------------------------------------ */
/* swap_blocks / swap_blocks_new_kv_combined, CS/block_swapping.cpp:22-85,
 * :88-202.  src_ids/dst_ids are HOST arrays; k_swap/v_swap are HOST tensors
 * [num_cpu_blocks, L, Hkv, B, D] fp16.  Runs of consecutive ids (same segment
 * on the device side) become one hipMemcpyAsync pair; return codes are
 * checked.  Swap-in writes device block dst_ids[i] from host block src_ids[i].
 * num_copies (host, may be NULL) receives the number of memcpy pairs issued. */
int mkv_swap_blocks(const int64_t* src_ids, const int64_t* dst_ids, int64_t count,
                    int32_t is_swap_in, const mkv_pool* pool, void* k_swap,
                    void* v_swap, int64_t* num_copies, void* stream);

/* The same eviction with the id lists left on the DEVICE (what
 * gather_allocated_blocks_and_free / allocate_blocks_for_seqs return,
 * MS/worker/model.py:476-477, before the reference's .tolist() at :483-484) and
 * the swap space in PINNED host memory: one kernel moves every pair over PCIe,
 * scattered or not, with no host synchronisation.  Pairs naming a block outside
 * the pool or outside [0, num_host_blocks) are skipped.  Replaces the memcpy
 * loops of CS/block_swapping.cpp:40-84, :120-200 for callers that pin their
 * swap space (the reference's is pageable, MS/worker/model.py:203-204). */
int mkv_swap_blocks_device_ids(const int64_t* src_ids, const int64_t* dst_ids, int64_t count,
                               int32_t is_swap_in, const mkv_pool* pool, void* k_swap,
                               void* v_swap, int64_t num_host_blocks, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MORPHKV_H */
