// KV append: scatter new K/V tokens into paged blocks through the block table.
// Pure copies, 16 bytes per lane; bit-exact by construction.
#include <algorithm>

#include "common.h"

namespace mkv {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

// One thread moves one 16-byte unit.  Unit index u over [n][K|V][Hkv][D/8]:
// consecutive lanes read consecutive 16-byte units of k (or v) and write
// 256-byte (D=128) contiguous rows of a head's slab.
__global__ __launch_bounds__(256) void append_decode_kernel(
    const uint4* __restrict__ k, const uint4* __restrict__ v, const mkv_pool pool,
    const int32_t* __restrict__ block_table, int64_t max_blocks_per_seq,
    const int32_t* __restrict__ seq_ids, const int32_t* __restrict__ seq_lens,
    int32_t n, int32_t layer) {
    const int d8 = pool.head_dim >> 3;                  // 16-byte units per head row
    const int per_tensor = pool.num_kv_heads * d8;      // units per sequence per K (or V)
    const int64_t total = (int64_t)n * 2 * per_tensor;
    int64_t u = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (u >= total) return;
    const int i = (int)(u / (2 * per_tensor));
    int r = (int)(u - (int64_t)i * 2 * per_tensor);
    const int is_v = r / per_tensor;
    r -= is_v * per_tensor;
    const int h = r / d8;
    const int c = r - h * d8;

    const int64_t seq = seq_ids[i];
    const int pos = seq_lens[i] - 1;
    const int blk = pos / pool.block_size;
    const int off = pos - blk * pool.block_size;
    if (pos < 0 || blk >= max_blocks_per_seq) return;        // no such position in the table row
    const int64_t pid = block_table[seq * max_blocks_per_seq + blk];
    if (pid < 0 || pid >= pool_total_blocks(pool)) return;   // unallocated row: nothing to write

    const int64_t block_bytes = pool_block_bytes(pool);
    BlockAddr a = block_addr(pool, pid, block_bytes);
    const int64_t slab_bytes = (int64_t)pool.block_size * pool.head_dim * 2;
    const int64_t dst_off = ((int64_t)layer * pool.num_kv_heads + h) * slab_bytes +
                            (int64_t)off * pool.head_dim * 2 + (int64_t)c * 16;
    const int64_t src_idx = (int64_t)i * per_tensor + r;
    if (is_v) {
        *(uint4*)(const_cast<char*>(a.v) + dst_off) = v[src_idx];
    } else {
        *(uint4*)(const_cast<char*>(a.k) + dst_off) = k[src_idx];
    }
}

// One workgroup per (logical block j, prefill sequence b, part z): part z moves K (z even) or
// V (z odd) of the kv heads [h0, h0 + heads_per_part) for up to B tokens.  Source rows
// [tok][Hkv][D] are contiguous per token, so a part reads heads_per_part * D * 2 contiguous
// bytes per token; each destination row [h][tok_local][:] is D * 2 contiguous bytes.  The
// split over parts is there to put enough workgroups on the chip when a batch has few blocks.
__global__ __launch_bounds__(256) void append_prefill_kernel(
    const uint4* __restrict__ k, const uint4* __restrict__ v, const mkv_pool pool,
    const int32_t* __restrict__ block_table, int64_t max_blocks_per_seq,
    const int32_t* __restrict__ seq_ids, const int32_t* __restrict__ start_locs,
    const int32_t* __restrict__ seq_lens, int32_t layer, int32_t heads_per_part) {
    const int b = blockIdx.y;
    const int j = blockIdx.x;
    const bool is_v = (blockIdx.z & 1) != 0;
    const int h0 = (int)(blockIdx.z >> 1) * heads_per_part;
    const int len = seq_lens[b];
    const int t0 = j * pool.block_size;
    if (t0 >= len || h0 >= pool.num_kv_heads) return;
    if (j >= max_blocks_per_seq) return;                     // beyond the table row: never another sequence's block
    const int nh = min(heads_per_part, pool.num_kv_heads - h0);
    const int ntok = min(pool.block_size, len - t0);
    const int64_t seq = seq_ids[b];
    const int64_t start = start_locs[b];
    const int64_t pid = block_table[seq * max_blocks_per_seq + j];
    if (pid < 0 || pid >= pool_total_blocks(pool)) return;   // unallocated row: nothing to write

    const int d8 = pool.head_dim >> 3;
    const int per_tok = pool.num_kv_heads * d8;
    const int per_part = nh * d8;
    const int units = ntok * per_part;
    const int64_t block_bytes = pool_block_bytes(pool);
    BlockAddr a = block_addr(pool, pid, block_bytes);
    const int64_t slab_bytes = (int64_t)pool.block_size * pool.head_dim * 2;
    char* dst_base = const_cast<char*>(is_v ? a.v : a.k) + ((int64_t)layer * pool.num_kv_heads + h0) * slab_bytes;
    const uint4* src = (is_v ? v : k) + (start + t0) * per_tok + (int64_t)h0 * d8;

    auto dst_of = [&](int u) -> uint4* {
        const int tl = u / per_part;
        const int r = u - tl * per_part;
        const int h = r / d8;
        const int c = r - h * d8;
        return (uint4*)(dst_base + (int64_t)h * slab_bytes + (int64_t)tl * pool.head_dim * 2 + (int64_t)c * 16);
    };
    auto src_of = [&](int u) -> const uint4* {
        const int tl = u / per_part;
        return src + (int64_t)tl * per_tok + (u - tl * per_part);
    };
    // four independent 16-byte moves per thread per trip: the loads go out before the stores
    int u = threadIdx.x;
    for (; u + 3 * (int)blockDim.x < units; u += 4 * blockDim.x) {
        v4u x[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) x[e] = __builtin_nontemporal_load((const v4u*)src_of(u + e * blockDim.x));
#pragma unroll
        for (int e = 0; e < 4; ++e) *(v4u*)dst_of(u + e * blockDim.x) = x[e];
    }
    for (; u < units; u += blockDim.x) *dst_of(u) = *src_of(u);
}

}  // namespace mkv

extern "C" {

int mkv_append_decode(const void* k, const void* v, const mkv_pool* pool,
                      const int32_t* block_table, int64_t max_blocks_per_seq,
                      const int32_t* seq_ids, const int32_t* seq_lens, int32_t n,
                      int32_t layer, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(n >= 0, "n must be >= 0");
    if (n == 0) return MKV_OK;
    MKV_REQUIRE(k && v && block_table && seq_ids && seq_lens, "NULL argument");
    MKV_REQUIRE(layer >= 0 && layer < pool->num_layers, "layer %d outside [0, %d)", layer, pool->num_layers);
    MKV_REQUIRE(((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0, "k/v must be 16-byte aligned");
    const int64_t total = (int64_t)n * 2 * pool->num_kv_heads * (pool->head_dim / 8);
    const int threads = 256;
    const int64_t blocks = (total + threads - 1) / threads;
    hipStream_t s = (hipStream_t)stream;
    {
        MKV_PROF(MKV_K_APPEND_DECODE, s);
        hipLaunchKernelGGL(mkv::append_decode_kernel, dim3((unsigned)blocks), dim3(threads), 0, s,
                           (const uint4*)k, (const uint4*)v, *pool, block_table, max_blocks_per_seq,
                           seq_ids, seq_lens, n, layer);
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_append_prefill(const void* k, const void* v, const mkv_pool* pool,
                       const int32_t* block_table, int64_t max_blocks_per_seq,
                       const int32_t* seq_ids, const int32_t* start_locs,
                       const int32_t* seq_lens, int32_t num_seqs, int32_t max_len,
                       int32_t layer, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(num_seqs >= 0 && max_len >= 0, "num_seqs/max_len must be >= 0");
    if (num_seqs == 0 || max_len == 0) return MKV_OK;
    MKV_REQUIRE(k && v && block_table && seq_ids && start_locs && seq_lens, "NULL argument");
    MKV_REQUIRE(layer >= 0 && layer < pool->num_layers, "layer %d outside [0, %d)", layer, pool->num_layers);
    MKV_REQUIRE(((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0, "k/v must be 16-byte aligned");
    MKV_REQUIRE(num_seqs <= 65535, "at most 65535 prefill sequences per call");
    MKV_REQUIRE(mkv::cdiv(max_len, pool->block_size) <= max_blocks_per_seq,
                "max_len %d needs %d blocks per sequence, a block-table row holds %lld", max_len,
                mkv::cdiv(max_len, pool->block_size), (long long)max_blocks_per_seq);
    // K and V go to separate workgroups, and the kv heads are cut into parts until the grid
    // has about eight workgroups per compute unit (a part keeps at least one head)
    const int64_t cells = (int64_t)mkv::cdiv(max_len, pool->block_size) * num_seqs * 2;
    const int parts = (int)std::min<int64_t>(pool->num_kv_heads, std::max<int64_t>(1, mkv::cdiv(2048, cells)));
    const int heads_per_part = (int)mkv::cdiv(pool->num_kv_heads, parts);
    dim3 grid((unsigned)mkv::cdiv(max_len, pool->block_size), (unsigned)num_seqs,
              2u * (unsigned)mkv::cdiv(pool->num_kv_heads, heads_per_part));
    hipStream_t s = (hipStream_t)stream;
    {
        MKV_PROF(MKV_K_APPEND_PREFILL, s);
        hipLaunchKernelGGL(mkv::append_prefill_kernel, grid, dim3(256), 0, s, (const uint4*)k,
                           (const uint4*)v, *pool, block_table, max_blocks_per_seq, seq_ids,
                           start_locs, seq_lens, layer, heads_per_part);
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

}  // extern "C"
