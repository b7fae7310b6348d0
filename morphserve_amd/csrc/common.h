// Shared host/device helpers for the morphkv HIP library (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "morphkv.h"
#include "morphkv_diag.h"

namespace mkv {

// ---- host-side error plumbing ---------------------------------------------
void set_error(const char* fmt, ...);
int  hip_fail(hipError_t e, const char* what);

#define MKV_HIP(call)                                             \
    do {                                                          \
        hipError_t _e = (call);                                   \
        if (_e != hipSuccess) return ::mkv::hip_fail(_e, #call);  \
    } while (0)

#define MKV_REQUIRE(cond, ...)                                    \
    do {                                                          \
        if (!(cond)) {                                            \
            ::mkv::set_error(__VA_ARGS__);                        \
            return MKV_EINVAL;                                    \
        }                                                         \
    } while (0)

int  check_pool(const mkv_pool* p);

// Brackets one launch with an event pair when profiling is on.
struct ProfScope {
    int kernel_id;
    hipStream_t stream;
    void* rec;
    ProfScope(int kernel_id, hipStream_t s);
    ~ProfScope();
};

// ---- device-side pool addressing ---------------------------------------------
// Byte offset of a block inside its pool/segment and the K/V bases it is
// relative to.  Block ids below num_blocks_org live in the base pool; others in
// segment (id-org)/S at local index (id-org)%S.
struct BlockAddr {
    const char* k;
    const char* v;
};

__device__ __forceinline__ BlockAddr block_addr(const mkv_pool& p, int64_t id, int64_t block_bytes) {
    BlockAddr a;
    if (id < p.num_blocks_org) {
        a.k = (const char*)p.k_base + id * block_bytes;
        a.v = (const char*)p.v_base + id * block_bytes;
    } else {
        // ids are below 2^31 (checked with the pool): a 32-bit division, not the 64-bit routine
        const uint32_t rel = (uint32_t)(id - p.num_blocks_org);
        const uint32_t seg = rel / (uint32_t)p.seg_blocks;
        const int64_t local = rel - seg * (uint32_t)p.seg_blocks;
        a.k = (const char*)p.k_seg[seg] + local * block_bytes;
        a.v = (const char*)p.v_seg[seg] + local * block_bytes;
    }
    return a;
}

__host__ __device__ __forceinline__ int64_t pool_block_bytes(const mkv_pool& p) {
    return (int64_t)p.num_layers * p.num_kv_heads * p.block_size * p.head_dim * 2;
}

// Ids outside [0, total) would address memory outside the pool; kernels skip them.
__host__ __device__ __forceinline__ int64_t pool_total_blocks(const mkv_pool& p) {
    return p.num_blocks_org + (int64_t)p.num_segments * p.seg_blocks;
}

static inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// ---- per-workgroup time stamps (diagnostic, mkv_diag_timeline) -----------------
// The attention launchers hand their kernels the buffer set by mkv_diag_timeline when it holds the
// launch's workgroups, NULL otherwise.  With a buffer, thread 0 of workgroup w stores the constant-rate
// 100 MHz counter at point k of its life into buf[w * MKV_TIMELINE_POINTS + k]; without one a mark is
// a scalar test and a branch.
long long* timeline_buffer(int64_t workgroups);

__device__ __forceinline__ void timeline_mark(long long* tl, int64_t wg, int k) {
    if (tl != nullptr && threadIdx.x == 0) {
        unsigned long long t;
        asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t));
        tl[wg * MKV_TIMELINE_POINTS + k] = (long long)t;
    }
}

}  // namespace mkv
