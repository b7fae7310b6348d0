// Calibration loops for the matrix pipe: what v_mfma_f32_16x16x32_f16 sustains on this part
// with nothing else in the way, so that a kernel's matrix-core utilisation can be read against
// a measured ceiling as well as the published peak.  Not on any product path.
#include "common.h"

namespace mkv {

typedef _Float16 d_v8h __attribute__((ext_vector_type(8)));
typedef float d_v4f __attribute__((ext_vector_type(4)));
typedef short d_v4s __attribute__((ext_vector_type(4)));

static constexpr int kDiagRowK = 272, kDiagRowV = 288;      // the prefill kernel's LDS row strides
static constexpr int kDiagWorkgroups = 512;                 // two per CU: two waves per SIMD
static constexpr int kDiagMfmaPerIter = 64;

// MODE 0: operands in registers, every element of an operand equal (little switching activity)
// MODE 1: operands in registers, taken from `data`
// MODE 2: operands from LDS in the prefill kernel's fragment pattern (b128 row reads feeding the
//         first product, transposing reads feeding the second), LDS filled from `data`
template <int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void diag_mfma_kernel(
    const uint4* __restrict__ data, float* __restrict__ sink, int iters) {
    __shared__ __attribute__((aligned(16))) char kl[64 * kDiagRowK];
    __shared__ __attribute__((aligned(16))) char vl[64 * kDiagRowV];
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 15, c = lane >> 4;
    for (int u = 0; u < 4; ++u) {
        *(uint4*)(kl + ((tid >> 4) + 16 * u) * kDiagRowK + (tid & 15) * 16) = data[tid + 256 * u];
        *(uint4*)(vl + ((tid >> 4) + 16 * u) * kDiagRowV + (tid & 15) * 16) = data[1024 + tid + 256 * u];
    }
    __syncthreads();
    d_v8h qb[2][4];
    for (int u = 0; u < 2; ++u)
        for (int x = 0; x < 4; ++x) {
            qb[u][x] = __builtin_bit_cast(d_v8h, data[2048 + lane * 8 + u * 4 + x]);
            if (MODE == 0) {       // one value per operand register set: distinct products, little switching
                const _Float16 f = (_Float16)(1 + u + 2 * x);
                qb[u][x] = (d_v8h){f, f, f, f, f, f, f, f};
            }
        }
    d_v4f acc[2][8], st[2][4];
    for (int u = 0; u < 2; ++u)
        for (int t = 0; t < 8; ++t) acc[u][t] = (d_v4f){0.f, 0.f, 0.f, 0.f};
    const char* k_rd = kl + m * kDiagRowK + c * 64;
    const char* v_rd = vl + (4 * c + (m >> 2)) * kDiagRowV + (m & 3) * 8;
    float keep = 0.f;
    for (int it = 0; it < iters; ++it) {
        // first product: four 16-key sub-tiles, each 4 fragments x 2 column tiles
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            uint4 kf[4];
#pragma unroll
            for (int x = 0; x < 4; ++x)
                kf[x] = (MODE == 2) ? *(const uint4*)(k_rd + 16 * n * kDiagRowK + 16 * x)
                                    : __builtin_bit_cast(uint4, qb[0][(x + n) & 3]);
#pragma unroll
            for (int u = 0; u < 2; ++u) st[u][n] = (d_v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int x = 0; x < 4; ++x)
#pragma unroll
                for (int u = 0; u < 2; ++u)
                    st[u][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(d_v8h, kf[x]), qb[u][x], st[u][n], 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int n = 0; n < 4; ++n) keep += st[u][n][0];
        // second product: eight 16-dim output tiles x two 32-key halves x 2 column tiles
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const char* vp = v_rd + 32 * h * kDiagRowV;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                d_v8h va;
                if (MODE == 2) {
                    const d_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((d_v4s __attribute__((address_space(3)))*)(vp + 32 * t));
                    const d_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((d_v4s __attribute__((address_space(3)))*)(vp + 16 * kDiagRowV + 32 * t));
                    va = __builtin_bit_cast(d_v8h, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                } else {
                    va = qb[1][(t + h) & 3];
                }
#pragma unroll
                for (int u = 0; u < 2; ++u) acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, qb[u][h * 2], acc[u][t], 0, 0, 0);
            }
        }
    }
    for (int u = 0; u < 2; ++u)
        for (int t = 0; t < 8; ++t) keep += acc[u][t][0] + acc[u][t][3];
    sink[blockIdx.x * blockDim.x + tid] = keep;
}

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Random 4 KiB slab reads and nothing else: what the memory system gives the decode gather.  Workgroup w reads
// slabs_per_wg slabs, U at a time; the slab comes from a multiplicative hash of (w, i), its buffer from one hash bit
// or, with by_xcd, from bit (w % 8) of xcd_mask (the XCD a workgroup of a 1-D grid runs on).
template <int U>
__global__ __launch_bounds__(256) void diag_slab_gather_kernel(const char* __restrict__ a, const char* __restrict__ b,
                                                               uint64_t slabs_in_buf, int32_t slabs_per_wg,
                                                               int32_t by_xcd, uint32_t xcd_mask,
                                                               uint32_t* __restrict__ sink) {
    extern __shared__ char occupancy_pad[];                 // sized by the launcher to limit the workgroups per CU
    const uint32_t w = blockIdx.x;
    v4u acc = (v4u){0u, 0u, 0u, 0u};
    for (int i = 0; i < slabs_per_wg; i += U) {
        v4u v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t h = ((uint64_t)w * (uint64_t)slabs_per_wg + (uint64_t)(i + u)) * 0x9E3779B97F4A7C15ull;
            const uint64_t slab = (h >> 20) & (slabs_in_buf - 1);
            const bool second = by_xcd ? ((xcd_mask >> (w & 7u)) & 1u) != 0 : ((h >> 50) & 1u) != 0;
            v[u] = __builtin_nontemporal_load((const v4u*)((second ? b : a) + slab * 4096) + threadIdx.x);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) acc ^= v[u];
        asm volatile("" : "+v"(acc.x));                     // the next group's loads wait for this one
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345677u) {   // keeps the loads; practically never true
        sink[0] = 1;
        occupancy_pad[0] = 1;
    }
}

}  // namespace mkv

extern "C" {

int mkv_diag_slab_gather(const void* a, const void* b, uint64_t slabs_in_buf, int32_t workgroups,
                         int32_t slabs_per_wg, int32_t loads_in_flight, int32_t workgroups_per_cu, int32_t by_xcd,
                         uint32_t xcd_mask, void* sink, void* stream) {
    MKV_REQUIRE(a && b && sink, "NULL argument");
    MKV_REQUIRE(slabs_in_buf > 0 && (slabs_in_buf & (slabs_in_buf - 1)) == 0, "slabs_in_buf must be a power of two");
    MKV_REQUIRE(workgroups > 0 && slabs_per_wg > 0, "bad grid");
    MKV_REQUIRE(loads_in_flight == 1 || loads_in_flight == 2 || loads_in_flight == 4 || loads_in_flight == 8,
                "loads_in_flight must be 1, 2, 4 or 8");
    MKV_REQUIRE(slabs_per_wg % loads_in_flight == 0, "slabs_per_wg must be a multiple of loads_in_flight");
    MKV_REQUIRE(workgroups_per_cu >= 1 && workgroups_per_cu <= 8, "workgroups_per_cu must be 1 ... 8");
    MKV_REQUIRE((((uintptr_t)a | (uintptr_t)b) & 4095) == 0, "buffers must be 4 KiB aligned");
    hipStream_t s = (hipStream_t)stream;
    const int lds = 160 * 1024 / workgroups_per_cu - 1024;  // that many workgroups fit the CU's 160 KiB
    const dim3 grid((unsigned)workgroups), block(256);
#define MKV_SLAB_GATHER(U)                                                                                          \
    do {                                                                                                            \
        MKV_HIP(hipFuncSetAttribute((const void*)mkv::diag_slab_gather_kernel<U>,                                    \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, lds));                               \
        hipLaunchKernelGGL(mkv::diag_slab_gather_kernel<U>, grid, block, lds, s, (const char*)a, (const char*)b,     \
                           slabs_in_buf, slabs_per_wg, by_xcd, xcd_mask, (uint32_t*)sink);                           \
    } while (0)
    if (loads_in_flight == 1) MKV_SLAB_GATHER(1);
    if (loads_in_flight == 2) MKV_SLAB_GATHER(2);
    if (loads_in_flight == 4) MKV_SLAB_GATHER(4);
    if (loads_in_flight == 8) MKV_SLAB_GATHER(8);
#undef MKV_SLAB_GATHER
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_diag_mfma_loop(int32_t mode, int32_t iters, const void* data, void* sink, double* flops,
                       void* stream) {
    MKV_REQUIRE(mode >= 0 && mode <= 2, "mode must be 0, 1 or 2");
    MKV_REQUIRE(iters > 0 && data && sink, "bad arguments");
    MKV_REQUIRE(((uintptr_t)data & 15) == 0, "data must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(mkv::kDiagWorkgroups), block(256);
    if (mode == 0) hipLaunchKernelGGL(mkv::diag_mfma_kernel<0>, grid, block, 0, s, (const uint4*)data, (float*)sink, iters);
    if (mode == 1) hipLaunchKernelGGL(mkv::diag_mfma_kernel<1>, grid, block, 0, s, (const uint4*)data, (float*)sink, iters);
    if (mode == 2) hipLaunchKernelGGL(mkv::diag_mfma_kernel<2>, grid, block, 0, s, (const uint4*)data, (float*)sink, iters);
    MKV_HIP(hipGetLastError());
    if (flops) *flops = (double)mkv::kDiagWorkgroups * 4 * iters * mkv::kDiagMfmaPerIter * 16384.0;
    return MKV_OK;
}

}  // extern "C"
