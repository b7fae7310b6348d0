// fp16 rotary arithmetic shared by the rotary kernel and the fused decode launch: one
// rounded product under one fused multiply-add per output,
//     out[d]       = fma(x[d], cos[d], -(x[d + D/2] * sin[d]))
//     out[d + D/2] = fma(x[d], sin[d],   x[d + D/2] * cos[d])          d < D/2.
#pragma once
#include <hip/hip_runtime.h>

namespace mkv {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ void rotate8(const h8 x0, const h8 x1, const h8 c, const h8 s, h8& o0, h8& o1) {
#pragma clang fp contract(off)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const _Float16 p0 = x1[e] * s[e];          // rounded to fp16 on its own
        const _Float16 p1 = x1[e] * c[e];
        o0[e] = __builtin_fmaf16(x0[e], c[e], -p0);
        o1[e] = __builtin_fmaf16(x0[e], s[e], p1);
    }
}

// Eight values of one half of a head and the eight of the other half they pair with ->
// the rotated eight in the caller's own half (`upper`: the caller holds dims >= D/2).
__device__ __forceinline__ uint4 rotate_own_half(uint4 own, uint4 partner, uint4 c, uint4 s, bool upper) {
    h8 o0, o1;
    const h8 a = __builtin_bit_cast(h8, upper ? partner : own);     // dims < D/2
    const h8 b = __builtin_bit_cast(h8, upper ? own : partner);     // dims >= D/2
    rotate8(a, b, __builtin_bit_cast(h8, c), __builtin_bit_cast(h8, s), o0, o1);
    return __builtin_bit_cast(uint4, upper ? o1 : o0);
}

}  // namespace mkv
