// Shared host/device helpers for the morphkv HIP library (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>

#include "morphkv.h"

// MKV_DIAG = 1 builds the diagnostic twin of the library (libmorphkv_diag.so): the same entry points plus
// the switches and measurement hooks of morphkv_diag.h.  The product library is built with MKV_DIAG = 0 and
// carries none of them: no time-stamp argument in any kernel, no event pairs around launches, no process-wide
// variant switches.
#ifndef MKV_DIAG
#define MKV_DIAG 0
#endif
#if MKV_DIAG
#include "morphkv_diag.h"
#endif

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

// Number of compute units of the current device (cached per process; 256 when the query fails).
int num_cus();

#if MKV_DIAG
// Brackets one launch with an event pair when profiling is on (diagnostic build only).
struct ProfScope {
    int kernel_id;
    hipStream_t stream;
    void* rec;
    ProfScope(int kernel_id, hipStream_t s);
    ~ProfScope();
};
#define MKV_PROF(id, s) ::mkv::ProfScope mkv_prof_scope_((id), (s))
#else
#define MKV_PROF(id, s) do { } while (0)
#endif

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

// ---- per-workgroup time stamps (diagnostic build only, mkv_diag_timeline) --------
// The attention kernels take a TimelineArg<TL> as their last argument.  TL = false, the only instance the
// product library contains, is an empty struct whose mark() is nothing.  In the diagnostic build the
// launchers pick the TL = true instance while mkv_diag_timeline holds a buffer large enough for the
// launch's workgroups: thread 0 of workgroup w then stores the constant-rate 100 MHz counter at point k
// of its life into buf[w * MKV_TIMELINE_POINTS + k].
template <bool TL>
struct TimelineArg {
    __device__ __forceinline__ void mark(int64_t, int) const {}
};

#if MKV_DIAG
long long* timeline_buffer(int64_t workgroups);

template <>
struct TimelineArg<true> {
    long long* buf;
    __device__ __forceinline__ void mark(int64_t wg, int k) const {
        if (threadIdx.x == 0) {
            unsigned long long t;
            asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t));
            buf[wg * MKV_TIMELINE_POINTS + k] = (long long)t;
        }
    }
};
#endif

}  // namespace mkv
