// Bulk HBM movers of the elastic pool: live-block migration (batched block copy),
// zero fill of new pool memory, and host<->device block eviction.
#include "common.h"

#include <vector>

namespace mkv {

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

static constexpr int kCopyThreads = 256;
static constexpr int kCopyUnroll = 4;                                   // 16-byte units per thread per chunk
static constexpr int64_t kChunkBytes = (int64_t)kCopyThreads * kCopyUnroll * 16;   // 16 KiB

// Work item w = (move, K|V, chunk) in that order of significance; a persistent
// grid strides over the items.  Within a chunk every wave instruction moves
// 1 KiB of contiguous bytes (16 bytes per lane), loads first, then stores.
__global__ __launch_bounds__(kCopyThreads) void pool_migrate_kernel(
    const mkv_pool pool, const int64_t* __restrict__ src, const int64_t* __restrict__ dst,
    int64_t num_moves, int64_t block_bytes, int32_t chunks_per_block) {
    const int64_t total_blocks = pool_total_blocks(pool);
    const int64_t items = num_moves * 2 * chunks_per_block;
    for (int64_t w = blockIdx.x; w < items; w += gridDim.x) {
        const int64_t mv = w / (2 * chunks_per_block);
        const int rem = (int)(w - mv * 2 * chunks_per_block);
        const int is_v = rem / chunks_per_block;
        const int chunk = rem - is_v * chunks_per_block;
        const int64_t s = src[mv];
        const int64_t d = dst[mv];
        if (s < 0 || s >= total_blocks || d < 0 || d >= total_blocks) continue;
        BlockAddr sa = block_addr(pool, s, block_bytes);
        BlockAddr da = block_addr(pool, d, block_bytes);
        const int64_t off = (int64_t)chunk * kChunkBytes;
        const uint4* sp = (const uint4*)((is_v ? sa.v : sa.k) + off) + threadIdx.x;
        uint4* dp = (uint4*)(const_cast<char*>(is_v ? da.v : da.k) + off) + threadIdx.x;
        const int64_t left = block_bytes - off;                         // bytes left in this block
        if (left >= kChunkBytes) {
            v4u r[kCopyUnroll];
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) r[u] = __builtin_nontemporal_load((const v4u*)sp + u * kCopyThreads);
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) __builtin_nontemporal_store(r[u], (v4u*)dp + u * kCopyThreads);
        } else {
            const int64_t units = left >> 4;                            // block_bytes is a multiple of 16
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) {
                const int64_t idx = (int64_t)u * kCopyThreads + threadIdx.x;
                if (idx < units) dp[u * kCopyThreads] = sp[u * kCopyThreads];
            }
        }
    }
}

// Eviction without the host in the loop: the (device block, host block) pairs are
// read from DEVICE arrays and one launch moves every pair between the pool and a
// pinned host swap space that the GPU addresses directly over PCIe.  Same item
// decomposition as the migration kernel; scattered pairs cost nothing extra.
template <bool SWAP_IN>
__global__ __launch_bounds__(kCopyThreads) void pool_swap_kernel(
    const mkv_pool pool, const int64_t* __restrict__ src, const int64_t* __restrict__ dst,
    int64_t count, char* __restrict__ k_swap, char* __restrict__ v_swap, int64_t num_host_blocks,
    int64_t block_bytes, int32_t chunks_per_block) {
    const int64_t total_blocks = pool_total_blocks(pool);
    const int64_t items = count * 2 * chunks_per_block;
    for (int64_t w = blockIdx.x; w < items; w += gridDim.x) {
        const int64_t mv = w / (2 * chunks_per_block);
        const int rem = (int)(w - mv * 2 * chunks_per_block);
        const int is_v = rem / chunks_per_block;
        const int chunk = rem - is_v * chunks_per_block;
        const int64_t dev_id = SWAP_IN ? dst[mv] : src[mv];
        const int64_t host_id = SWAP_IN ? src[mv] : dst[mv];
        if (dev_id < 0 || dev_id >= total_blocks || host_id < 0 || host_id >= num_host_blocks) continue;
        BlockAddr da = block_addr(pool, dev_id, block_bytes);
        const int64_t off = (int64_t)chunk * kChunkBytes;
        char* dev_p = const_cast<char*>(is_v ? da.v : da.k) + off;
        char* host_p = (is_v ? v_swap : k_swap) + host_id * block_bytes + off;
        const uint4* sp = (const uint4*)(SWAP_IN ? host_p : dev_p) + threadIdx.x;
        uint4* dp = (uint4*)(SWAP_IN ? dev_p : host_p) + threadIdx.x;
        const int64_t left = block_bytes - off;
        if (left >= kChunkBytes) {
            v4u r[kCopyUnroll];
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) r[u] = __builtin_nontemporal_load((const v4u*)sp + u * kCopyThreads);
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) __builtin_nontemporal_store(r[u], (v4u*)dp + u * kCopyThreads);
        } else {
            const int64_t units = left >> 4;
#pragma unroll
            for (int u = 0; u < kCopyUnroll; ++u) {
                const int64_t idx = (int64_t)u * kCopyThreads + threadIdx.x;
                if (idx < units) dp[u * kCopyThreads] = sp[u * kCopyThreads];
            }
        }
    }
}

// One 16-byte store per thread, one 4 KiB run per workgroup, plain (cached) stores:
// on this part that shape writes fastest (a persistent grid-stride loop or
// non-temporal stores are 15-25 % slower).
__global__ __launch_bounds__(256) void fill_zero_kernel(uint4* __restrict__ p, int64_t units,
                                                        uint8_t* __restrict__ tail, int tail_bytes) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < units) p[i] = make_uint4(0u, 0u, 0u, 0u);
    if (blockIdx.x == 0 && (int)threadIdx.x < tail_bytes) tail[threadIdx.x] = 0;
}

}  // namespace mkv

extern "C" {

int mkv_pool_migrate(const mkv_pool* pool, const int64_t* src, const int64_t* dst,
                     int64_t num_moves, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(num_moves >= 0, "num_moves must be >= 0");
    if (num_moves == 0) return MKV_OK;
    MKV_REQUIRE(src && dst, "src/dst are NULL");
    const int64_t block_bytes = mkv::pool_block_bytes(*pool);
    const int chunks = mkv::cdiv(block_bytes, mkv::kChunkBytes);
    const int64_t items = num_moves * 2 * chunks;
    const int64_t want = (int64_t)mkv::num_cus() * 16;
    const unsigned grid = (unsigned)(items < want ? items : want);
    hipStream_t s = (hipStream_t)stream;
    {
        MKV_PROF(MKV_K_MIGRATE, s);
        hipLaunchKernelGGL(mkv::pool_migrate_kernel, dim3(grid), dim3(mkv::kCopyThreads), 0, s,
                           *pool, src, dst, num_moves, block_bytes, chunks);
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_fill_zero(void* ptr, uint64_t bytes, void* stream) {
    if (bytes == 0) return MKV_OK;
    MKV_REQUIRE(ptr != nullptr, "ptr is NULL");
    MKV_REQUIRE(((uintptr_t)ptr & 15) == 0, "ptr must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    // a launch may not have 2^32 or more threads: at most 2^31 16-byte units (32 GiB) each
    const uint64_t max_bytes = (uint64_t)1 << 35;
    char* cur = (char*)ptr;
    while (bytes > 0) {
        const uint64_t now = bytes < max_bytes ? bytes : max_bytes;
        const int64_t units = (int64_t)(now >> 4);
        const int tail = (int)(now & 15);
        const int64_t grid = units > 0 ? (units + 255) / 256 : 1;
        {
            MKV_PROF(MKV_K_FILL_ZERO, s);
            hipLaunchKernelGGL(mkv::fill_zero_kernel, dim3((unsigned)grid), dim3(256), 0, s, (uint4*)cur,
                               units, (uint8_t*)cur + (units << 4), tail);
        }
        MKV_HIP(hipGetLastError());
        cur += now;
        bytes -= now;
    }
    return MKV_OK;
}

int mkv_swap_blocks(const int64_t* src_ids, const int64_t* dst_ids, int64_t count,
                    int32_t is_swap_in, const mkv_pool* pool, void* k_swap, void* v_swap,
                    int64_t* num_copies, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(count >= 0, "count must be >= 0");
    if (num_copies) *num_copies = 0;
    if (count == 0) return MKV_OK;
    MKV_REQUIRE(src_ids && dst_ids && k_swap && v_swap, "NULL argument");
    const int64_t block_bytes = mkv::pool_block_bytes(*pool);
    const int64_t total_blocks = mkv::pool_total_blocks(*pool);
    // the device side of the pair: target on swap-in, source on swap-out
    const int64_t* dev_ids = is_swap_in ? dst_ids : src_ids;
    const int64_t* host_ids = is_swap_in ? src_ids : dst_ids;
    auto seg_of = [&](int64_t id) -> int64_t {
        return id < pool->num_blocks_org ? -1 : (id - pool->num_blocks_org) / pool->seg_blocks;
    };
    for (int64_t i = 0; i < count; ++i) {
        MKV_REQUIRE(dev_ids[i] >= 0 && dev_ids[i] < total_blocks,
                    "device block id %lld outside the pool (%lld blocks)", (long long)dev_ids[i],
                    (long long)total_blocks);
        MKV_REQUIRE(host_ids[i] >= 0, "host block id %lld is negative", (long long)host_ids[i]);
    }
    hipStream_t s = (hipStream_t)stream;
    int64_t copies = 0;
    int64_t i = 0;
    while (i < count) {
        int64_t j = i + 1;
        const int64_t seg = seg_of(dev_ids[i]);
        while (j < count && src_ids[j] == src_ids[j - 1] + 1 && dst_ids[j] == dst_ids[j - 1] + 1 &&
               seg_of(dev_ids[j]) == seg)
            ++j;
        const int64_t bytes = (j - i) * block_bytes;
        const int64_t id = dev_ids[i];
        char *kd, *vd;
        if (seg < 0) {
            kd = (char*)pool->k_base + id * block_bytes;
            vd = (char*)pool->v_base + id * block_bytes;
        } else {
            const int64_t local = id - pool->num_blocks_org - seg * pool->seg_blocks;
            kd = (char*)pool->k_seg[seg] + local * block_bytes;
            vd = (char*)pool->v_seg[seg] + local * block_bytes;
        }
        char* kh = (char*)k_swap + host_ids[i] * block_bytes;
        char* vh = (char*)v_swap + host_ids[i] * block_bytes;
        if (is_swap_in) {
            MKV_HIP(hipMemcpyAsync(kd, kh, bytes, hipMemcpyHostToDevice, s));
            MKV_HIP(hipMemcpyAsync(vd, vh, bytes, hipMemcpyHostToDevice, s));
        } else {
            MKV_HIP(hipMemcpyAsync(kh, kd, bytes, hipMemcpyDeviceToHost, s));
            MKV_HIP(hipMemcpyAsync(vh, vd, bytes, hipMemcpyDeviceToHost, s));
        }
        ++copies;
        i = j;
    }
    if (num_copies) *num_copies = copies;
    return MKV_OK;
}

int mkv_swap_blocks_device_ids(const int64_t* src_ids, const int64_t* dst_ids, int64_t count,
                               int32_t is_swap_in, const mkv_pool* pool, void* k_swap, void* v_swap,
                               int64_t num_host_blocks, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(count >= 0 && num_host_blocks >= 0, "count/num_host_blocks must be >= 0");
    if (count == 0) return MKV_OK;
    MKV_REQUIRE(src_ids && dst_ids && k_swap && v_swap, "NULL argument");
    // the swap space must be memory the GPU can address: pinned host (or device) memory
    void* dev_ptr[2] = {nullptr, nullptr};
    void* host_ptr[2] = {k_swap, v_swap};
    for (int t = 0; t < 2; ++t) {
        hipPointerAttribute_t attr;
        hipError_t e = hipPointerGetAttributes(&attr, host_ptr[t]);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            MKV_REQUIRE(false, "swap space is not pinned host memory (allocate it with hipHostMalloc / pin_memory=True)");
        }
        MKV_REQUIRE(attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeDevice ||
                        attr.type == hipMemoryTypeManaged,
                    "swap space is not pinned host memory (allocate it with hipHostMalloc / pin_memory=True)");
        dev_ptr[t] = attr.devicePointer ? attr.devicePointer : host_ptr[t];
    }
    const int64_t block_bytes = mkv::pool_block_bytes(*pool);
    const int chunks = mkv::cdiv(block_bytes, mkv::kChunkBytes);
    const int64_t items = count * 2 * chunks;
    const int64_t want = (int64_t)mkv::num_cus() * 4;
    const unsigned grid = (unsigned)(items < want ? items : want);
    hipStream_t s = (hipStream_t)stream;
    {
        MKV_PROF(MKV_K_SWAP, s);
        if (is_swap_in) {
            hipLaunchKernelGGL(mkv::pool_swap_kernel<true>, dim3(grid), dim3(mkv::kCopyThreads), 0, s, *pool,
                               src_ids, dst_ids, count, (char*)dev_ptr[0], (char*)dev_ptr[1], num_host_blocks,
                               block_bytes, chunks);
        } else {
            hipLaunchKernelGGL(mkv::pool_swap_kernel<false>, dim3(grid), dim3(mkv::kCopyThreads), 0, s, *pool,
                               src_ids, dst_ids, count, (char*)dev_ptr[0], (char*)dev_ptr[1], num_host_blocks,
                               block_bytes, chunks);
        }
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

}  // extern "C"
