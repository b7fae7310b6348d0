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

}  // namespace mkv

extern "C" {

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
