// Paged decode attention for gfx950 (wave64).
//
// Phase 1: one workgroup (4 waves) per (split, kv head, sequence).  All G = Hq/Hkv
// query heads of the kv head are handled by the same waves, so every K/V slab
// is read from HBM exactly once.  A 16-token block of one head is a contiguous
// 4 KiB slab; a wave reads it with four fully coalesced 16-byte-per-lane loads
// (1 KiB per instruction).  Lane = (r, c): row r = lane / 16 selects a token
// within each group of four, c = lane % 16 selects eight head dims.  Dot
// products are reduced over the 16 lanes of a DPP row; every row keeps its own
// online-softmax state (fp32, base 2), merged across rows and waves at the end.
// Phase 2 merges the per-split partials by log-sum-exp.
#include "common.h"

namespace mkv {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

static constexpr float kNegBig = -1.0e30f;   // finite "minus infinity": never produces NaN in m - m
static constexpr float kLog2e = 1.442695040888963f;
static constexpr int kD = 128;               // head dim handled by these kernels
static constexpr int kB = 16;                // tokens per block handled by these kernels

// v_exp_f32: arguments here are <= 0 and a result that underflows may flush to 0.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int N>
__device__ __forceinline__ float dpp_row_ror(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + N, 0xf, 0xf, false));
}

// Sum over the 16 lanes of a row; every lane of the row gets the total.
__device__ __forceinline__ float row_sum16(float x) {
    x += dpp_row_ror<8>(x);
    x += dpp_row_ror<4>(x);
    x += dpp_row_ror<2>(x);
    x += dpp_row_ror<1>(x);
    return x;
}

__device__ __forceinline__ h2 as_h2(uint32_t u) { return __builtin_bit_cast(h2, u); }

__device__ __forceinline__ float dot8(const uint4& a, const uint4& b, float acc) {
    acc = __builtin_amdgcn_fdot2(as_h2(a.x), as_h2(b.x), acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(a.y), as_h2(b.y), acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(a.z), as_h2(b.z), acc, false);
    acc = __builtin_amdgcn_fdot2(as_h2(a.w), as_h2(b.w), acc, false);
    return acc;
}

struct Slab {
    const uint4* k;
    const uint4* v;
    bool ok;
};

template <int G>
struct RowState {
    float m[G];
    float l[G];
    float acc[G][8];
};

// Consume one 16-token block held in registers.  first_tok is the sequence
// position of the block's token 0; tokens at positions >= len are masked.
template <int G, bool MASK>
__device__ __forceinline__ void consume_block(RowState<G>& st, const uint4 (&q)[G],
                                              const uint4 (&kc)[4], uint4 (&vc)[4],
                                              float scale2, int first_tok, int len, int r) {
    bool valid[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        valid[i] = !MASK || (first_tok + 4 * i + r) < len;
        if (MASK && !valid[i]) vc[i] = make_uint4(0u, 0u, 0u, 0u);   // stale bytes past len never reach the sum
    }
    float vf[4][8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w[4] = {vc[i].x, vc[i].y, vc[i].z, vc[i].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            h2 p = as_h2(w[j]);
            vf[i][2 * j] = (float)p.x;
            vf[i][2 * j + 1] = (float)p.y;
        }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float s[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float d = row_sum16(dot8(kc[i], q[g], 0.f)) * scale2;
            s[i] = valid[i] ? d : kNegBig;
        }
        const float m_new = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), st.m[g]);
        const float alpha = fast_exp2(st.m[g] - m_new);
        float p[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) p[i] = valid[i] ? fast_exp2(s[i] - m_new) : 0.f;
        st.l[g] = st.l[g] * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
        st.m[g] = m_new;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float a = st.acc[g][j] * alpha;
            a = fmaf(p[0], vf[0][j], a);
            a = fmaf(p[1], vf[1][j], a);
            a = fmaf(p[2], vf[2][j], a);
            a = fmaf(p[3], vf[3][j], a);
            st.acc[g][j] = a;
        }
    }
}

template <int G>
__global__ __launch_bounds__(256) void attn_decode_phase1(
    const uint4* __restrict__ q,        // [n, Hq, D] fp16
    __half* __restrict__ o,             // [n, Hq, D] fp16 (written only when gridDim.x == 1)
    float* __restrict__ mid_o,          // [n, Hq, max_splits, D]
    float* __restrict__ mid_lse,        // [n, Hq, max_splits]
    const mkv_pool pool, const int32_t* __restrict__ block_table, int64_t max_blocks_per_seq,
    const int32_t* __restrict__ seq_ids, const int32_t* __restrict__ seq_lens, float scale2,
    int32_t layer, int32_t blocks_per_split, int32_t max_splits) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r = lane >> 4;       // token row within a group of four
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    const int i = blockIdx.z;
    const int Hq = pool.num_kv_heads * G;

    const int len = seq_lens[i];
    const int nblk = (int)min((int64_t)((len + kB - 1) / kB), max_blocks_per_seq);   // never read past the table row
    const int blk_begin = split * blocks_per_split;
    if (blk_begin >= nblk) return;                      // uniform over the workgroup
    // the last launched split also takes whatever lies beyond it, so an
    // under-estimated max_splits costs balance, never tokens
    const int blk_end = (split == (int)gridDim.x - 1) ? nblk : min(blk_begin + blocks_per_split, nblk);
    const int64_t seq = seq_ids[i];
    const int32_t* row = block_table + seq * max_blocks_per_seq;

    const int64_t block_bytes = pool_block_bytes(pool);
    const int64_t total_blocks = pool_total_blocks(pool);
    const int64_t head_off = ((int64_t)layer * pool.num_kv_heads + kvh) * (kB * kD * 2);

    // q for the G heads of this kv head: lane holds dims [c*8, c*8+8)
    uint4 qreg[G];
#pragma unroll
    for (int g = 0; g < G; ++g)
        qreg[g] = q[((int64_t)i * Hq + kvh * G + g) * (kD / 8) + (lane & 15)];

    RowState<G> st;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        st.m[g] = kNegBig;
        st.l[g] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) st.acc[g][j] = 0.f;
    }

    // This wave's blocks: blk_begin + wave + 4 * it.  Table entries are fetched
    // 64 iterations at a time (one per lane) and handed out with readlane.
    const int my_first = blk_begin + wave;
    const int n_it = (blk_end - my_first + 3) >> 2;      // may be <= 0
    auto slab_of = [&](int32_t pid) {
        Slab s;
        s.ok = pid >= 0 && pid < total_blocks;
        BlockAddr a = block_addr(pool, s.ok ? pid : 0, block_bytes);
        s.k = (const uint4*)(a.k + head_off) + lane;
        s.v = (const uint4*)(a.v + head_off) + lane;
        return s;
    };

    for (int it0 = 0; it0 < n_it; it0 += 64) {
        const int b_lane = my_first + 4 * (it0 + lane);
        const int32_t tbl = (b_lane < blk_end) ? row[b_lane] : -1;
        const int cnt = min(64, n_it - it0);

        uint4 kc[4], vc[4];
        Slab cur = slab_of(__builtin_amdgcn_readlane(tbl, 0));
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            kc[x] = cur.ok ? cur.k[x * 64] : make_uint4(0u, 0u, 0u, 0u);
            vc[x] = cur.ok ? cur.v[x * 64] : make_uint4(0u, 0u, 0u, 0u);
        }
        for (int t = 0; t < cnt; ++t) {
            const int b = my_first + 4 * (it0 + t);
            uint4 kn[4], vn[4];
            const bool has_next = (t + 1) < cnt;
            if (has_next) {
                Slab nx = slab_of(__builtin_amdgcn_readlane(tbl, t + 1));
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    kn[x] = nx.ok ? nx.k[x * 64] : make_uint4(0u, 0u, 0u, 0u);
                    vn[x] = nx.ok ? nx.v[x * 64] : make_uint4(0u, 0u, 0u, 0u);
                }
            }
            if (b == nblk - 1) {
                consume_block<G, true>(st, qreg, kc, vc, scale2, b * kB, len, r);
            } else {
                consume_block<G, false>(st, qreg, kc, vc, scale2, b * kB, len, r);
            }
            if (has_next) {
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    kc[x] = kn[x];
                    vc[x] = vn[x];
                }
            }
        }
    }

    // ---- merge the four token rows of this wave --------------------------------
#pragma unroll
    for (int g = 0; g < G; ++g) {
        float m_all = fmaxf(st.m[g], __shfl_xor(st.m[g], 16));
        m_all = fmaxf(m_all, __shfl_xor(m_all, 32));
        const float f = fast_exp2(st.m[g] - m_all);
        float l = st.l[g] * f;
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        st.l[g] = l;
        st.m[g] = m_all;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float a = st.acc[g][j] * f;
            a += __shfl_xor(a, 16);
            a += __shfl_xor(a, 32);
            st.acc[g][j] = a;
        }
    }

    // ---- merge the four waves through LDS ------------------------------------------
    __shared__ float sm_acc[4][G][kD];
    __shared__ float sm_m[4][G];
    __shared__ float sm_l[4][G];
    if (lane < 16) {
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int j = 0; j < 8; ++j) sm_acc[wave][g][lane * 8 + j] = st.acc[g][j];
            if (lane == 0) {
                sm_m[wave][g] = st.m[g];
                sm_l[wave][g] = st.l[g];
            }
        }
    }
    __syncthreads();

    const bool direct = gridDim.x == 1;
    for (int idx = tid; idx < G * kD; idx += 256) {
        const int g = idx / kD;
        const int d = idx - g * kD;
        float m_tot = fmaxf(fmaxf(sm_m[0][g], sm_m[1][g]), fmaxf(sm_m[2][g], sm_m[3][g]));
        float l_tot = 0.f, a_tot = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = fast_exp2(sm_m[w][g] - m_tot);
            l_tot += sm_l[w][g] * f;
            a_tot += sm_acc[w][g][d] * f;
        }
        const float val = a_tot / l_tot;
        const int64_t hq = (int64_t)i * Hq + kvh * G + g;
        if (direct) {
            o[hq * kD + d] = __float2half(val);
        } else {
            mid_o[(hq * max_splits + split) * kD + d] = val;
            if (d == 0) mid_lse[hq * max_splits + split] = log2f(l_tot) + m_tot;
        }
    }
}

// Phase 2: one workgroup of 128 threads per (sequence, q head): log-sum-exp merge
// of the per-split partials, cast to fp16.
__global__ __launch_bounds__(128) void attn_decode_phase2(
    const float* __restrict__ mid_o, const float* __restrict__ mid_lse, __half* __restrict__ o,
    const int32_t* __restrict__ seq_lens, int32_t num_q_heads, int32_t tokens_per_split,
    int32_t max_splits) {
    const int i = blockIdx.y;
    const int hq = blockIdx.x;
    const int d = threadIdx.x;
    const int len = seq_lens[i];
    const int ns = min((len + tokens_per_split - 1) / tokens_per_split, max_splits);
    const int64_t base = ((int64_t)i * num_q_heads + hq) * max_splits;
    float m = kNegBig, l = 0.f, acc = 0.f;
    for (int s = 0; s < ns; ++s) {
        const float lse = mid_lse[base + s];
        const float v = mid_o[(base + s) * kD + d];
        const float m_new = fmaxf(m, lse);
        const float old = fast_exp2(m - m_new);
        const float e = fast_exp2(lse - m_new);
        acc = acc * old + e * v;
        l = l * old + e;
        m = m_new;
    }
    o[((int64_t)i * num_q_heads + hq) * kD + d] = __float2half(ns > 0 ? acc / l : 0.f);
}

template <int G>
static void launch_phase1(dim3 grid, hipStream_t s, const void* q, void* o, void* mid_o,
                          void* mid_lse, const mkv_pool* pool, const int32_t* block_table,
                          int64_t max_blocks_per_seq, const int32_t* seq_ids,
                          const int32_t* seq_lens, float scale2, int32_t layer,
                          int32_t blocks_per_split, int32_t max_splits) {
    hipLaunchKernelGGL(attn_decode_phase1<G>, grid, dim3(256), 0, s, (const uint4*)q, (__half*)o,
                       (float*)mid_o, (float*)mid_lse, *pool, block_table, max_blocks_per_seq,
                       seq_ids, seq_lens, scale2, layer, blocks_per_split, max_splits);
}

}  // namespace mkv

extern "C" {

int mkv_paged_attn_scratch_bytes(int32_t n, int32_t num_q_heads, int32_t head_dim,
                                 int32_t max_splits, int64_t* mid_o_bytes,
                                 int64_t* mid_lse_bytes) {
    MKV_REQUIRE(n >= 0 && num_q_heads > 0 && head_dim > 0 && max_splits > 0, "bad sizes");
    MKV_REQUIRE(mid_o_bytes && mid_lse_bytes, "output pointers are NULL");
    *mid_lse_bytes = (int64_t)n * num_q_heads * max_splits * 4;
    *mid_o_bytes = *mid_lse_bytes * head_dim;
    return MKV_OK;
}

int mkv_paged_attn_decode(const void* q, void* o, const mkv_pool* pool,
                          const int32_t* block_table, int64_t max_blocks_per_seq,
                          const int32_t* seq_ids, const int32_t* seq_lens, int32_t n,
                          int32_t num_q_heads, float softmax_scale, int32_t layer,
                          int32_t tokens_per_split, int32_t max_splits, void* mid_o,
                          void* mid_lse, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(n >= 0, "n must be >= 0");
    if (n == 0) return MKV_OK;
    MKV_REQUIRE(q && o && block_table && seq_ids && seq_lens, "NULL argument");
    MKV_REQUIRE(pool->head_dim == mkv::kD, "decode attention supports head_dim 128 only (got %d)", pool->head_dim);
    MKV_REQUIRE(pool->block_size == mkv::kB, "decode attention supports block_size 16 only (got %d)", pool->block_size);
    MKV_REQUIRE(layer >= 0 && layer < pool->num_layers, "layer %d outside [0, %d)", layer, pool->num_layers);
    MKV_REQUIRE(num_q_heads > 0 && num_q_heads % pool->num_kv_heads == 0,
                "num_q_heads %d must be a multiple of num_kv_heads %d", num_q_heads, pool->num_kv_heads);
    MKV_REQUIRE(tokens_per_split > 0 && tokens_per_split % pool->block_size == 0,
                "tokens_per_split %d must be a positive multiple of block_size %d", tokens_per_split, pool->block_size);
    MKV_REQUIRE(max_splits >= 1, "max_splits must be >= 1");
    MKV_REQUIRE(max_splits == 1 || (mid_o && mid_lse), "scratch buffers are NULL");
    MKV_REQUIRE(n <= 65535 && pool->num_kv_heads <= 65535, "grid dimension limit: n, Hkv <= 65535");
    MKV_REQUIRE(((uintptr_t)q & 15) == 0, "q must be 16-byte aligned");
    const int G = num_q_heads / pool->num_kv_heads;
    const float scale2 = softmax_scale * mkv::kLog2e;
    const int bps = tokens_per_split / pool->block_size;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)max_splits, (unsigned)pool->num_kv_heads, (unsigned)n);
    {
        mkv::ProfScope prof(MKV_K_ATTN_PHASE1, s);
        switch (G) {
#define MKV_CASE(GG)                                                                               \
    case GG:                                                                                       \
        mkv::launch_phase1<GG>(grid, s, q, o, mid_o, mid_lse, pool, block_table,                   \
                               max_blocks_per_seq, seq_ids, seq_lens, scale2, layer, bps,          \
                               max_splits);                                                        \
        break;
            MKV_CASE(1)
            MKV_CASE(2)
            MKV_CASE(4)
            MKV_CASE(8)
#undef MKV_CASE
            default:
                mkv::set_error("unsupported GQA group size %d (supported: 1, 2, 4, 8)", G);
                return MKV_EINVAL;
        }
    }
    MKV_HIP(hipGetLastError());
    if (max_splits > 1) {
        mkv::ProfScope prof(MKV_K_ATTN_PHASE2, s);
        hipLaunchKernelGGL(mkv::attn_decode_phase2, dim3((unsigned)num_q_heads, (unsigned)n),
                           dim3(128), 0, s, (const float*)mid_o, (const float*)mid_lse, (__half*)o,
                           seq_lens, num_q_heads, tokens_per_split, max_splits);
        MKV_HIP(hipGetLastError());
    }
    return MKV_OK;
}

}  // extern "C"
