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
#include "rope_math.h"

#include <mutex>

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

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

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

// Final step of a phase-1 workgroup: merge the four waves' (max, sum, accumulator)
// states held in LDS and store either the finished output (one split launched) or
// this split's normalised partial and its log2-sum-exp.
template <int G>
__device__ __forceinline__ void merge_waves_and_store(const float (&sm_acc)[4][G][kD],
                                                      const float (&sm_m)[4][G],
                                                      const float (&sm_l)[4][G], __half* o,
                                                      float* mid_o, float* mid_lse, int64_t hq0,
                                                      int split, int max_splits) {
    const bool direct = gridDim.x == 1;
    for (int idx = threadIdx.x; idx < G * kD; idx += 256) {
        const int g = idx / kD;
        const int d = idx - g * kD;
        const float m_tot = fmaxf(fmaxf(sm_m[0][g], sm_m[1][g]), fmaxf(sm_m[2][g], sm_m[3][g]));
        float l_tot = 0.f, a_tot = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = fast_exp2(sm_m[w][g] - m_tot);
            l_tot += sm_l[w][g] * f;
            a_tot += sm_acc[w][g][d] * f;
        }
        const float val = a_tot / l_tot;
        const int64_t hq = hq0 + g;
        if (direct) {
            o[hq * kD + d] = __float2half(val);
        } else {
            mid_o[(hq * max_splits + split) * kD + d] = val;
            if (d == 0) mid_lse[hq * max_splits + split] = log2f(l_tot) + m_tot;
        }
    }
}


// Which sequence should the workgroup at batch slot w take?  With one split per sequence a launch holds
// one workgroup per (kv head, sequence), and the CUs receive consecutive workgroups in turn: slots w
// and w + 256 / Hkv end up on the same CU.  Dealing the sequences to the slots by length in snake
// order (longest first over one run of 256 / Hkv slots, the next run reversed, ...) gives every CU
// about the same number of tokens to stream, so a launch does not end on the CUs that happened to
// draw two long sequences.  The order depends on the lengths only, so it is computed once per batch
// (this kernel: one workgroup, rank by (length, row) with n compares per row) and handed to every
// layer's launch.  order[slot] = row of the batch; any permutation is valid, this one is balanced.
__global__ __launch_bounds__(1024) void decode_order_kernel(const int32_t* __restrict__ seq_lens, int32_t n,
                                                            int32_t run, int32_t* __restrict__ order) {
    __shared__ int32_t s_len[4096];
    for (int j = threadIdx.x; j < n; j += blockDim.x) s_len[j] = seq_lens[j];
    __syncthreads();
    for (int j = threadIdx.x; j < n; j += blockDim.x) {
        const int mine = s_len[j];
        int rank = 0;                                   // rows that come before row j: longer, or as long and earlier
        for (int k = 0; k < n; ++k) {
            const int other = s_len[k];
            rank += (other > mine) || (other == mine && k < j);
        }
        const int r = rank / run, c = rank - r * run;
        const int slot = (r < n / run && (r & 1)) ? r * run + (run - 1 - c) : rank;    // a trailing partial run stays in order
        order[slot] = j;
    }
}

template <int G, bool TL>
__global__ __launch_bounds__(256) void attn_decode_phase1(
    const uint4* __restrict__ q,        // [n, Hq, D] fp16
    __half* __restrict__ o,             // [n, Hq, D] fp16 (written only when gridDim.x == 1)
    float* __restrict__ mid_o,          // [n, Hq, max_splits, D]
    float* __restrict__ mid_lse,        // [n, Hq, max_splits]
    const mkv_pool pool, const int32_t* __restrict__ block_table, int64_t max_blocks_per_seq,
    const int32_t* __restrict__ seq_ids, const int32_t* __restrict__ seq_lens, float scale2,
    int32_t layer, int32_t blocks_per_split, int32_t max_splits,
    const uint4* __restrict__ k_new,    // [n, Hkv, D] fp16 or NULL: token len-1 to append first
    const uint4* __restrict__ v_new,
    const uint4* __restrict__ cos_t,    // [n, D/2] fp16 or NULL: rotate q and the new k row on the way in
    const uint4* __restrict__ sin_t,
    const int32_t* __restrict__ order,     // [n] or NULL: batch row taken by each slot of the grid
    const TimelineArg<TL> timeline) {      // per-workgroup time stamps (an empty struct unless TL)
    const int64_t wg_id = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
    timeline.mark(wg_id, 0);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int r = lane >> 4;       // token row within a group of four
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    // a slot's row comes from the caller's order; an entry outside the batch (a buffer that was never
    // written) falls back to the slot's own row instead of indexing past the batch's arrays
    int i = order ? order[blockIdx.z] : (int)blockIdx.z;
    if ((unsigned)i >= gridDim.z) i = (int)blockIdx.z;
    const int Hq = pool.num_kv_heads * G;

    const int len = seq_lens[i];
    const int nblk = (int)min((int64_t)((len + kB - 1) / kB), max_blocks_per_seq);   // never read past the table row
    const int blk_begin = split * blocks_per_split;
    if (blk_begin >= nblk) {
        // nothing of the sequence lies in this split: the merge must see an empty slot, not stale scratch
        if (gridDim.x > 1 && threadIdx.x < G)
            mid_lse[((int64_t)i * Hq + kvh * G + threadIdx.x) * max_splits + split] = kNegBig;
        return;                                         // uniform over the workgroup
    }
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
    // rotary on the way in: chunk c pairs with chunk c ^ 8 (dims d and d + 64)
    const bool rope = cos_t != nullptr;
    uint4 cosc = make_uint4(0u, 0u, 0u, 0u), sinc = cosc;
    if (rope) {
        cosc = cos_t[(int64_t)i * (kD / 16) + (lane & 7)];
        sinc = sin_t[(int64_t)i * (kD / 16) + (lane & 7)];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const uint4 partner = q[((int64_t)i * Hq + kvh * G + g) * (kD / 8) + ((lane & 15) ^ 8)];
            qreg[g] = rotate_own_half(qreg[g], partner, cosc, sinc, (lane & 8) != 0);
        }
    }

    RowState<G> st;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        st.m[g] = kNegBig;
        st.l[g] = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) st.acc[g][j] = 0.f;
    }

    // This wave's blocks: blk_begin + wave + 4 * t.  Table entries are fetched 64
    // iterations at a time (one per lane) and handed out with readlane.  Only the
    // sequence's final block can be partial; it is the last of its wave's list and
    // is handled apart, so the main loop carries no masking and no branches around
    // its loads: the loads of block t+1 are issued before block t is consumed and
    // stay in flight behind it.
    timeline.mark(wg_id, 1);
    const int my_first = blk_begin + __builtin_amdgcn_readfirstlane(wave);
    const int n_it = max(0, (blk_end - my_first + 3) >> 2);
    // blocks [0, nblk_full) hold 16 valid tokens and need no special care; with a
    // fused append the final block always does (it receives the new token)
    const bool fused = k_new != nullptr;
    const int nblk_full = fused ? nblk - 1 : len / kB;
    auto load_block = [&](int32_t pid, uint4 (&kk)[4], uint4 (&vv)[4]) {
        BlockAddr a = block_addr(pool, pid, block_bytes);
        const v4u* kp = (const v4u*)(a.k + head_off) + lane;
        const v4u* vp = (const v4u*)(a.v + head_off) + lane;
#pragma unroll
        for (int x = 0; x < 4; ++x) kk[x] = __builtin_bit_cast(uint4, __builtin_nontemporal_load(kp + x * 64));
#pragma unroll
        for (int x = 0; x < 4; ++x) vv[x] = __builtin_bit_cast(uint4, __builtin_nontemporal_load(vp + x * 64));
    };

    for (int it0 = 0; it0 < n_it; it0 += 64) {
        const int b_lane = my_first + 4 * (it0 + lane);
        const bool in_range = b_lane < blk_end;
        const int32_t tbl = in_range ? row[b_lane] : 0;
        const bool bad = in_range && (tbl < 0 || tbl >= total_blocks);
        const bool any_bad = __ballot(bad) != 0;          // wave-uniform
        const int cnt = min(64, n_it - it0);
        const int b_last = my_first + 4 * (it0 + cnt - 1);
        const int cnt_full = (b_last >= nblk_full) ? cnt - 1 : cnt;
        auto pid_of = [&](int t) { return __builtin_amdgcn_readlane(tbl, t); };
        auto tok_of = [&](int t) { return (my_first + 4 * (it0 + t)) * kB; };

        if (!any_bad) {
            if (cnt_full > 0) {
                uint4 k0[4], v0[4], k1[4], v1[4];
                load_block(pid_of(0), k0, v0);
                int t = 0;
                while (t + 2 < cnt_full) {
                    load_block(pid_of(t + 1), k1, v1);
                    consume_block<G, false>(st, qreg, k0, v0, scale2, tok_of(t), len, r);
                    load_block(pid_of(t + 2), k0, v0);
                    consume_block<G, false>(st, qreg, k1, v1, scale2, tok_of(t + 1), len, r);
                    t += 2;
                }
                if (t + 1 < cnt_full) {
                    load_block(pid_of(t + 1), k1, v1);
                    consume_block<G, false>(st, qreg, k0, v0, scale2, tok_of(t), len, r);
                    consume_block<G, false>(st, qreg, k1, v1, scale2, tok_of(t + 1), len, r);
                } else {
                    consume_block<G, false>(st, qreg, k0, v0, scale2, tok_of(t), len, r);
                }
            }
        } else {
            // a table entry names no block of the pool: skip such blocks
            for (int t = 0; t < cnt_full; ++t) {
                const int32_t pid = pid_of(t);
                if (pid < 0 || pid >= total_blocks) continue;
                uint4 k0[4], v0[4];
                load_block(pid, k0, v0);
                consume_block<G, false>(st, qreg, k0, v0, scale2, tok_of(t), len, r);
            }
        }
        if (cnt_full < cnt) {                              // the partial final block
            const int32_t pid = pid_of(cnt - 1);
            if (pid >= 0 && pid < total_blocks) {
                uint4 k0[4], v0[4];
                load_block(pid, k0, v0);
                if (fused) {
                    // token len-1: write it into its slot of the cache and use it from
                    // registers, whatever the slot held before
                    const int off = (len - 1) & (kB - 1);
                    uint4 kn = k_new[((int64_t)i * pool.num_kv_heads + kvh) * (kD / 8) + (lane & 15)];
                    const uint4 vn = v_new[((int64_t)i * pool.num_kv_heads + kvh) * (kD / 8) + (lane & 15)];
                    if (rope) {
                        const uint4 partner = k_new[((int64_t)i * pool.num_kv_heads + kvh) * (kD / 8) + ((lane & 15) ^ 8)];
                        kn = rotate_own_half(kn, partner, cosc, sinc, (lane & 8) != 0);
                    }
                    if (r == (off & 3)) {
                        BlockAddr a = block_addr(pool, pid, block_bytes);
                        const int64_t slot = head_off + (int64_t)off * (kD * 2) + (lane & 15) * 16;
                        *(uint4*)(const_cast<char*>(a.k) + slot) = kn;
                        *(uint4*)(const_cast<char*>(a.v) + slot) = vn;
#pragma unroll
                        for (int x = 0; x < 4; ++x) {
                            if (x == (off >> 2)) {
                                k0[x] = kn;
                                v0[x] = vn;
                            }
                        }
                    }
                }
                consume_block<G, true>(st, qreg, k0, v0, scale2, tok_of(cnt - 1), len, r);
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
    timeline.mark(wg_id, 2);
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
    merge_waves_and_store<G>(sm_acc, sm_m, sm_l, o, mid_o, mid_lse, (int64_t)i * Hq + kvh * G, split,
                             max_splits);
    timeline.mark(wg_id, 3);
}

// ---- matrix-core variant for GQA groups (G >= 4) -----------------------------------
// Same workgroup / wave decomposition.  A wave stages each 16-token K and V tile
// in its private LDS area (row-major, rows padded to 272 bytes) and reads it back
// in matrix-core operand order:
//   S^T[token, head] = K[token, :] . Q^T      one v_mfma_f32_16x16x32_f16 per 32 dims,
//                                             the G heads padded to 16 columns
//   O^T[dim, head]  += V^T[dim, token] . P^T  one v_mfma_f32_16x16x16_f16 per 16 dims
// The accumulator layout of S^T (lane = head, registers = four consecutive
// tokens) is the B-operand layout of the second product, so the probabilities
// never cross lanes.  Which 8 dims a lane contributes to a product is free as
// long as K and Q agree, so a lane takes 64 contiguous bytes of its K row.
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((ext_vector_type(4)));

static constexpr int kLdsRow = 272;                 // K rows: 256 data bytes + 16 pad: conflict-free b128 row reads
static constexpr int kLdsRowV = 288;                // V rows 8 banks apart: conflict-free transposing reads
static constexpr int kLdsTile = kB * kLdsRowV;      // room for either tile

struct FullTag { static constexpr bool value = false; };    // a block of 16 valid tokens
struct FinalTag { static constexpr bool value = true; };    // the sequence's last block: masked

__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

template <int G, bool TL>
__global__ __launch_bounds__(256) void attn_decode_phase1_mfma(
    const uint4* __restrict__ q, __half* __restrict__ o, float* __restrict__ mid_o,
    float* __restrict__ mid_lse, const mkv_pool pool, const int32_t* __restrict__ block_table,
    int64_t max_blocks_per_seq, const int32_t* __restrict__ seq_ids,
    const int32_t* __restrict__ seq_lens, float scale2, int32_t layer, int32_t blocks_per_split,
    int32_t max_splits, const uint4* __restrict__ k_new, const uint4* __restrict__ v_new,
    const uint4* __restrict__ cos_t, const uint4* __restrict__ sin_t, const int32_t* __restrict__ order,
    const TimelineArg<TL> timeline) {
    const int64_t wg_id = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
    timeline.mark(wg_id, 0);
    __shared__ __attribute__((aligned(16))) char stage[4][2][kLdsTile];
    __shared__ float sm_acc[4][G][kD];
    __shared__ float sm_m[4][G];
    __shared__ float sm_l[4][G];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n = lane & 15;       // head column (B / C operands), token or dim row (A operands)
    const int c = lane >> 4;       // lane group
    const int split = blockIdx.x;
    const int kvh = blockIdx.y;
    // a slot's row comes from the caller's order; an entry outside the batch (a buffer that was never
    // written) falls back to the slot's own row instead of indexing past the batch's arrays
    int i = order ? order[blockIdx.z] : (int)blockIdx.z;
    if ((unsigned)i >= gridDim.z) i = (int)blockIdx.z;
    const int Hq = pool.num_kv_heads * G;

    const int len = seq_lens[i];
    const int nblk = (int)min((int64_t)((len + kB - 1) / kB), max_blocks_per_seq);
    const int blk_begin = split * blocks_per_split;
    if (blk_begin >= nblk) {
        // nothing of the sequence lies in this split: the merge must see an empty slot, not stale scratch
        if (gridDim.x > 1 && threadIdx.x < G)
            mid_lse[((int64_t)i * Hq + kvh * G + threadIdx.x) * max_splits + split] = kNegBig;
        return;                                         // uniform over the workgroup
    }
    const int blk_end = (split == (int)gridDim.x - 1) ? nblk : min(blk_begin + blocks_per_split, nblk);
    const int64_t seq = seq_ids[i];
    const int32_t* row = block_table + seq * max_blocks_per_seq;
    const int64_t block_bytes = pool_block_bytes(pool);
    const int64_t total_blocks = pool_total_blocks(pool);
    const int64_t head_off = ((int64_t)layer * pool.num_kv_heads + kvh) * (kB * kD * 2);

    // Q^T as B operand: lane (head n, group c) holds dims c*32 + 8x .. +8 for product x
    v8h qb[4];
    if (n < G) {
        const uint4* qp = q + ((int64_t)i * Hq + kvh * G + n) * (kD / 8) + c * 4;
#pragma unroll
        for (int x = 0; x < 4; ++x) qb[x] = __builtin_bit_cast(v8h, qp[x]);
        if (cos_t != nullptr) {       // rotary on the way in: dims c*32.. pair with dims (c^2)*32..
            const uint4* pp = q + ((int64_t)i * Hq + kvh * G + n) * (kD / 8) + (c ^ 2) * 4;
            const uint4* cp = cos_t + (int64_t)i * (kD / 16) + (c & 1) * 4;
            const uint4* sp = sin_t + (int64_t)i * (kD / 16) + (c & 1) * 4;
#pragma unroll
            for (int x = 0; x < 4; ++x)
                qb[x] = __builtin_bit_cast(v8h, rotate_own_half(__builtin_bit_cast(uint4, qb[x]), pp[x], cp[x], sp[x], c >= 2));
        }
    } else {
#pragma unroll
        for (int x = 0; x < 4; ++x) qb[x] = (v8h){0, 0, 0, 0, 0, 0, 0, 0};
    }

    v4f oacc[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) oacc[t] = (v4f){0.f, 0.f, 0.f, 0.f};
    float m_run = kNegBig;         // running max of head n (same in the four lane groups)
    float l_run = 0.f;             // this lane's share of the running sum

    char* kl = stage[wave][0];
    char* vl = stage[wave][1];
    const int wr_off = c * kLdsRow + n * 16;                     // load x of lane (c, n): token 4x + c, bytes 16n..
    const int wr_off_v = c * kLdsRowV + n * 16;
    const char* k_rd = kl + n * kLdsRow + c * 64;                // token row n, 64 bytes of it
    // V^T operand through the transposing LDS read (ds_read_b64_tr_b16): within a
    // 16-lane group lane r supplies the address of four consecutive halves and
    // lane 4a+b receives element b of the rows supplied by lanes a, a+4, a+8, a+12.
    // Lane r therefore points at token 4c + r/4, dims 4*(r%4).. of the tile, and
    // lane n ends up with tokens 4c..4c+3 of dim n -- the A-operand order.
    const char* v_rd = vl + (4 * c + (n >> 2)) * kLdsRowV + (n & 3) * 8;

    auto issue_loads = [&](int32_t pid, v4u (&kg)[4], v4u (&vg)[4]) {
        BlockAddr a = block_addr(pool, pid, block_bytes);
        const v4u* kp = (const v4u*)(a.k + head_off) + lane;
        const v4u* vp = (const v4u*)(a.v + head_off) + lane;
#pragma unroll
        for (int x = 0; x < 4; ++x) kg[x] = __builtin_nontemporal_load(kp + x * 64);
#pragma unroll
        for (int x = 0; x < 4; ++x) vg[x] = __builtin_nontemporal_load(vp + x * 64);
    };
    // registers -> LDS
    auto stage_tile = [&](const v4u (&kg)[4], const v4u (&vg)[4]) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            *(v4u*)(kl + wr_off + x * 4 * kLdsRow) = kg[x];
            *(v4u*)(vl + wr_off_v + x * 4 * kLdsRowV) = vg[x];
        }
        wave_lds_fence();
    };
    // The sequence's final block: rows of tokens at or beyond len are zeroed so that
    // stale bytes (NaN included) cannot reach either product.
    auto mask_final_tile = [&](v4u (&kg)[4], v4u (&vg)[4], int tok0) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            if (tok0 + 4 * x + c >= len) {
                kg[x] = (v4u){0u, 0u, 0u, 0u};
                vg[x] = (v4u){0u, 0u, 0u, 0u};
            }
        }
    };
    // Fused append: token len-1 goes into its cache slot and, whatever the slot
    // held, into the staged tile (one 256-byte row of K and of V, 16 lanes each).
    auto append_into_tile = [&](int32_t pid) {
        const int off = (len - 1) & (kB - 1);
        if (lane < 32) {
            const bool is_v = lane >= 16;
            const int64_t src = ((int64_t)i * pool.num_kv_heads + kvh) * (kD / 8) + n;
            v4u val = __builtin_bit_cast(v4u, is_v ? v_new[src] : k_new[src]);
            if (cos_t != nullptr && !is_v) {    // the new k row is rotated before it is stored and used
                const uint4 partner = k_new[src - n + (n ^ 8)];
                const uint4 cc = cos_t[(int64_t)i * (kD / 16) + (n & 7)];
                const uint4 ss = sin_t[(int64_t)i * (kD / 16) + (n & 7)];
                val = __builtin_bit_cast(v4u, rotate_own_half(__builtin_bit_cast(uint4, val), partner, cc, ss, n >= 8));
            }
            BlockAddr a = block_addr(pool, pid, block_bytes);
            const int64_t slot = head_off + (int64_t)off * (kD * 2) + n * 16;
            *(v4u*)(const_cast<char*>(is_v ? a.v : a.k) + slot) = val;
            *(v4u*)((is_v ? vl + off * kLdsRowV : kl + off * kLdsRow) + n * 16) = val;
        }
        wave_lds_fence();
    };
    auto compute_tile = [&](int tok0, auto partial_tag) {
        constexpr bool partial = decltype(partial_tag)::value;
        v4f s = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const v8h a = *(const v8h*)(k_rd + x * 16);
            s = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qb[x], s, 0, 0, 0);
        }
        float sc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            sc[j] = s[j] * scale2;
            if (partial && tok0 + 4 * c + j >= len) sc[j] = kNegBig;
        }
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        if (__ballot(m_new > m_run) != 0) {          // some head's max moved: rescale (wave-uniform branch)
            const float alpha = fast_exp2(m_run - m_new);
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < 8; ++t) oacc[t] *= alpha;
            m_run = m_new;
        }
        float p[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) p[j] = fast_exp2(sc[j] - m_run);
        l_run += (p[0] + p[1]) + (p[2] + p[3]);
        const v4h pb = (v4h){(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3]};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const v4h va = __builtin_bit_cast(v4h, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (v4s __attribute__((address_space(3)))*)(v_rd + 32 * t)));
            oacc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(va, pb, oacc[t], 0, 0, 0);
        }
        wave_lds_fence();                            // reads done before the next tile is staged
    };

    timeline.mark(wg_id, 1);
    const int my_first = blk_begin + __builtin_amdgcn_readfirstlane(wave);
    const int n_it = max(0, (blk_end - my_first + 3) >> 2);
    // blocks [0, nblk_full) hold 16 valid tokens; the final block takes the careful
    // path when it is partial or, with a fused append, always
    const int nblk_full = (k_new != nullptr) ? nblk - 1 : len / kB;
    for (int it0 = 0; it0 < n_it; it0 += 64) {
        const int b_lane = my_first + 4 * (it0 + lane);
        const bool in_range = b_lane < blk_end;
        const int32_t tbl = in_range ? row[b_lane] : 0;
        const bool bad = in_range && (tbl < 0 || tbl >= total_blocks);
        const bool any_bad = __ballot(bad) != 0;
        const int cnt = min(64, n_it - it0);
        const int b_last = my_first + 4 * (it0 + cnt - 1);
        const int cnt_full = (b_last >= nblk_full) ? cnt - 1 : cnt;
        auto pid_of = [&](int t) { return __builtin_amdgcn_readlane(tbl, t); };
        auto tok_of = [&](int t) { return (my_first + 4 * (it0 + t)) * kB; };
        v4u kg[4], vg[4];
        if (!any_bad) {
            // block t is staged from registers, block t+1's loads go out, block t is consumed
            issue_loads(pid_of(0), kg, vg);
            for (int t = 0; t < cnt_full; ++t) {
                stage_tile(kg, vg);
                if (t + 1 < cnt) issue_loads(pid_of(t + 1), kg, vg);
                compute_tile(tok_of(t), FullTag{});
            }
            if (cnt_full < cnt) {
                mask_final_tile(kg, vg, tok_of(cnt - 1));
                stage_tile(kg, vg);
                if (k_new != nullptr && tok_of(cnt - 1) + kB >= len) append_into_tile(pid_of(cnt - 1));
                compute_tile(tok_of(cnt - 1), FinalTag{});
            }
        } else {
            for (int t = 0; t < cnt; ++t) {
                const int32_t pid = pid_of(t);
                if (pid < 0 || pid >= total_blocks) continue;      // names no block of the pool
                issue_loads(pid, kg, vg);
                if (t >= cnt_full) mask_final_tile(kg, vg, tok_of(t));
                stage_tile(kg, vg);
                if (t >= cnt_full && k_new != nullptr && tok_of(t) + kB >= len) append_into_tile(pid);
                compute_tile(tok_of(t), FinalTag{});
            }
        }
    }

    timeline.mark(wg_id, 2);
    float l_tot = l_run + __shfl_xor(l_run, 16);
    l_tot += __shfl_xor(l_tot, 32);
    if (n < G) {
#pragma unroll
        for (int t = 0; t < 8; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) sm_acc[wave][n][16 * t + 4 * c + j] = oacc[t][j];
        if (c == 0) {
            sm_m[wave][n] = m_run;
            sm_l[wave][n] = l_tot;
        }
    }
    __syncthreads();
    merge_waves_and_store<G>(sm_acc, sm_m, sm_l, o, mid_o, mid_lse, (int64_t)i * Hq + kvh * G, split,
                             max_splits);
    timeline.mark(wg_id, 3);
}

// Phase 2: log-sum-exp merge of the per-split partials, cast to fp16.  Both kernels read
// ALL max_splits slots of their (sequence, q head) -- phase 1 marks the slots of splits beyond a
// sequence's end with kNegBig -- so nothing here waits for the sequence's length: the partials and
// their log-sum-exps are requested together, one trip to memory between launch and store.
__device__ __forceinline__ bool slot_live(float lse) { return lse > 0.5f * kNegBig; }

// Up to 8 splits: one workgroup of 128 threads per (sequence, q head), thread = output dim.
__global__ __launch_bounds__(128) void attn_decode_phase2(
    const float* __restrict__ mid_o, const float* __restrict__ mid_lse, __half* __restrict__ o,
    int32_t num_q_heads, int32_t max_splits) {
    const int i = blockIdx.y;
    const int hq = blockIdx.x;
    const int d = threadIdx.x;
    const int64_t base = ((int64_t)i * num_q_heads + hq) * max_splits;
    float lse[8], v[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const int sc = min(s, max_splits - 1);                  // slots past the last re-read it (and are ignored)
        lse[s] = mid_lse[base + sc];
        v[s] = mid_o[(base + sc) * kD + d];
    }
    float m = kNegBig;
#pragma unroll
    for (int s = 0; s < 8; ++s)
        if (s < max_splits) m = fmaxf(m, lse[s]);
    float l = 0.f, acc = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        if (s < max_splits && slot_live(lse[s])) {              // an empty slot's partial is never touched
            const float e = fast_exp2(lse[s] - m);
            l += e;
            acc = fmaf(e, v[s], acc);
        }
    }
    o[((int64_t)i * num_q_heads + hq) * kD + d] = __float2half(l > 0.f ? acc / l : 0.f);
}

// More than 8 splits (long contexts at small batch): a workgroup of four waves takes one
// (sequence, q head); slots are consumed 64 at a time.  Wave w requests the partials of slots
// w, w+4, ... with SIXTEEN independent 8-byte loads per lane (lane l owns dims 2l, 2l+1) and, behind
// them, the chunk's 64 log-sum-exps (one per lane); the loads return while the chunk max and the
// weights w_s = exp2(lse_s - max) -- the same values in all four waves -- are formed with wave
// reductions.  The four waves' sums meet in LDS.
__global__ __launch_bounds__(256) void attn_decode_phase2_wide(
    const float* __restrict__ mid_o, const float* __restrict__ mid_lse, __half* __restrict__ o,
    int32_t num_q_heads, int32_t max_splits) {
    __shared__ float part[4][kD];
    const int i = blockIdx.y;
    const int hq = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t base = ((int64_t)i * num_q_heads + hq) * max_splits;
    float m = kNegBig, l = 0.f, a0 = 0.f, a1 = 0.f;
    for (int s0 = 0; s0 < max_splits; s0 += 64) {
        const int cnt = min(64, max_splits - s0);
        float2 v[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int jc = min(wave + 4 * e, cnt - 1);                 // wave-uniform
            v[e] = *(const float2*)(mid_o + (base + s0 + jc) * kD + 2 * lane);
        }
        const float lse = mid_lse[base + s0 + min(lane, cnt - 1)];
        const bool live = lane < cnt && slot_live(lse);
        float mc = live ? lse : kNegBig;
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1) mc = fmaxf(mc, __shfl_xor(mc, sh));
        const float m_new = fmaxf(m, mc);
        const float old = fast_exp2(m - m_new);
        const float wgt = live ? fast_exp2(lse - m_new) : 0.f;
        float wsum = wgt;
#pragma unroll
        for (int sh = 32; sh >= 1; sh >>= 1) wsum += __shfl_xor(wsum, sh);
        l = l * old + wsum;
        a0 *= old;
        a1 *= old;
        m = m_new;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int j = wave + 4 * e;                                // wave-uniform
            const float w = j < cnt ? __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wgt), min(j, cnt - 1))) : 0.f;
            if (w != 0.f) {                                            // wave-uniform: an empty slot's partial is never touched
                a0 = fmaf(w, v[e].x, a0);
                a1 = fmaf(w, v[e].y, a1);
            }
        }
    }
    part[wave][2 * lane] = a0;
    part[wave][2 * lane + 1] = a1;
    __syncthreads();
    if (threadIdx.x < kD) {
        const int d = threadIdx.x;
        const float acc = (part[0][d] + part[1][d]) + (part[2][d] + part[3][d]);
        o[((int64_t)i * num_q_heads + hq) * kD + d] = __float2half(l > 0.f ? acc / l : 0.f);
    }
}

#if MKV_DIAG
// 0: by group size (matrix cores for G >= 3), 1: vector ALU kernel, 2: matrix-core kernel
static int g_decode_variant = 0;
#endif

template <int G, bool TL>
static void launch_phase1_as(bool mfma, dim3 grid, hipStream_t s, const void* q, void* o, void* mid_o,
                             void* mid_lse, const mkv_pool* pool, const int32_t* block_table,
                             int64_t max_blocks_per_seq, const int32_t* seq_ids, const int32_t* seq_lens,
                             float scale2, int32_t layer, int32_t blocks_per_split, int32_t max_splits,
                             const void* k_new, const void* v_new, const void* cos_t, const void* sin_t,
                             const int32_t* order, const TimelineArg<TL> timeline) {
    // The vector-ALU kernel serves one or two q heads per kv head, the matrix-core kernel every larger
    // group (up to the 16 columns of a matrix tile).  The diagnostic build also holds the vector kernel
    // for groups of 4 and 8 and the matrix kernel for 1 and 2, for A/B runs.
    constexpr bool valu_built = MKV_DIAG ? (G == 1 || G == 2 || G == 4 || G == 8) : (G <= 2);
    constexpr bool mfma_built = MKV_DIAG ? true : (G >= 3);
    if constexpr (mfma_built) {
        if (mfma || !valu_built) {
            hipLaunchKernelGGL((attn_decode_phase1_mfma<G, TL>), grid, dim3(256), 0, s, (const uint4*)q,
                               (__half*)o, (float*)mid_o, (float*)mid_lse, *pool, block_table,
                               max_blocks_per_seq, seq_ids, seq_lens, scale2, layer, blocks_per_split,
                               max_splits, (const uint4*)k_new, (const uint4*)v_new, (const uint4*)cos_t,
                               (const uint4*)sin_t, order, timeline);
            return;
        }
    }
    if constexpr (valu_built) {
        hipLaunchKernelGGL((attn_decode_phase1<G, TL>), grid, dim3(256), 0, s, (const uint4*)q, (__half*)o,
                           (float*)mid_o, (float*)mid_lse, *pool, block_table, max_blocks_per_seq,
                           seq_ids, seq_lens, scale2, layer, blocks_per_split, max_splits,
                           (const uint4*)k_new, (const uint4*)v_new, (const uint4*)cos_t, (const uint4*)sin_t,
                           order, timeline);
    }
}

template <int G>
static void launch_phase1(dim3 grid, hipStream_t s, const void* q, void* o, void* mid_o,
                          void* mid_lse, const mkv_pool* pool, const int32_t* block_table,
                          int64_t max_blocks_per_seq, const int32_t* seq_ids,
                          const int32_t* seq_lens, float scale2, int32_t layer,
                          int32_t blocks_per_split, int32_t max_splits, const void* k_new,
                          const void* v_new, const void* cos_t, const void* sin_t, const int32_t* order) {
    bool mfma = G >= 3;
#if MKV_DIAG
    if (g_decode_variant == 1) mfma = false;
    if (g_decode_variant == 2) mfma = true;
    // time stamps: the groups the timeline workloads use
    if constexpr (G == 1 || G == 2 || G == 4 || G == 8) {
        if (long long* buf = timeline_buffer((int64_t)grid.x * grid.y * grid.z)) {
            launch_phase1_as<G, true>(mfma, grid, s, q, o, mid_o, mid_lse, pool, block_table, max_blocks_per_seq,
                                      seq_ids, seq_lens, scale2, layer, blocks_per_split, max_splits, k_new, v_new,
                                      cos_t, sin_t, order, TimelineArg<true>{buf});
            return;
        }
    }
#endif
    launch_phase1_as<G, false>(mfma, grid, s, q, o, mid_o, mid_lse, pool, block_table, max_blocks_per_seq,
                               seq_ids, seq_lens, scale2, layer, blocks_per_split, max_splits, k_new, v_new,
                               cos_t, sin_t, order, TimelineArg<false>{});
}

}  // namespace mkv

extern "C" {

#if MKV_DIAG
int mkv_set_decode_variant(int32_t variant) {
    MKV_REQUIRE(variant >= 0 && variant <= 2, "variant must be 0 (auto), 1 (vector ALU) or 2 (matrix core)");
    mkv::g_decode_variant = variant;
    return MKV_OK;
}
#endif

int mkv_paged_attn_scratch_bytes(int32_t n, int32_t num_q_heads, int32_t head_dim,
                                 int32_t max_splits, int64_t* mid_o_bytes,
                                 int64_t* mid_lse_bytes) {
    MKV_REQUIRE(n >= 0 && num_q_heads > 0 && head_dim > 0 && max_splits > 0, "bad sizes");
    MKV_REQUIRE(mid_o_bytes && mid_lse_bytes, "output pointers are NULL");
    *mid_lse_bytes = (int64_t)n * num_q_heads * max_splits * 4;
    *mid_o_bytes = *mid_lse_bytes * head_dim;
    return MKV_OK;
}

static int decode_impl(const void* q, void* o, const mkv_pool* pool, const int32_t* block_table,
                       int64_t max_blocks_per_seq, const int32_t* seq_ids, const int32_t* seq_lens,
                       int32_t n, int32_t num_q_heads, float softmax_scale, int32_t layer,
                       int32_t tokens_per_split, int32_t max_splits, void* mid_o, void* mid_lse,
                       const void* k_new, const void* v_new, const void* cos_t, const void* sin_t,
                       void* stream, const int32_t* order = nullptr) {
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
    MKV_REQUIRE(((uintptr_t)mid_o & 15) == 0 && ((uintptr_t)mid_lse & 3) == 0, "mid_o must be 16-byte aligned, mid_lse 4-byte aligned");
    MKV_REQUIRE(n <= 65535 && pool->num_kv_heads <= 65535, "grid dimension limit: n, Hkv <= 65535");
    MKV_REQUIRE(((uintptr_t)q & 15) == 0, "q must be 16-byte aligned");
    const int G = num_q_heads / pool->num_kv_heads;
    const float scale2 = softmax_scale * mkv::kLog2e;
    const int bps = tokens_per_split / pool->block_size;
    hipStream_t s = (hipStream_t)stream;
    dim3 grid((unsigned)max_splits, (unsigned)pool->num_kv_heads, (unsigned)n);
    {
        MKV_PROF(MKV_K_ATTN_PHASE1, s);
        switch (G) {
#define MKV_CASE(GG)                                                                               \
    case GG:                                                                                       \
        mkv::launch_phase1<GG>(grid, s, q, o, mid_o, mid_lse, pool, block_table,                   \
                               max_blocks_per_seq, seq_ids, seq_lens, scale2, layer, bps,          \
                               max_splits, k_new, v_new, cos_t, sin_t, order);                     \
        break;
            MKV_CASE(1)
            MKV_CASE(2)
            MKV_CASE(3)
            MKV_CASE(4)
            MKV_CASE(5)
            MKV_CASE(6)
            MKV_CASE(7)
            MKV_CASE(8)
            MKV_CASE(9)
            MKV_CASE(10)
            MKV_CASE(11)
            MKV_CASE(12)
            MKV_CASE(13)
            MKV_CASE(14)
            MKV_CASE(15)
            MKV_CASE(16)
#undef MKV_CASE
            default:
                mkv::set_error("unsupported GQA group size %d (supported: 1 to 16)", G);
                return MKV_EINVAL;
        }
    }
    MKV_HIP(hipGetLastError());
    if (max_splits > 1) {
        MKV_PROF(MKV_K_ATTN_PHASE2, s);
        if (max_splits > 8) {       // a long chain of partials per head: the gather-in-parallel merge
            hipLaunchKernelGGL(mkv::attn_decode_phase2_wide, dim3((unsigned)num_q_heads, (unsigned)n),
                               dim3(256), 0, s, (const float*)mid_o, (const float*)mid_lse, (__half*)o,
                               num_q_heads, max_splits);
        } else {
            hipLaunchKernelGGL(mkv::attn_decode_phase2, dim3((unsigned)num_q_heads, (unsigned)n),
                               dim3(128), 0, s, (const float*)mid_o, (const float*)mid_lse, (__half*)o,
                               num_q_heads, max_splits);
        }
        MKV_HIP(hipGetLastError());
    }
    return MKV_OK;
}

int mkv_paged_attn_decode(const void* q, void* o, const mkv_pool* pool,
                          const int32_t* block_table, int64_t max_blocks_per_seq,
                          const int32_t* seq_ids, const int32_t* seq_lens, int32_t n,
                          int32_t num_q_heads, float softmax_scale, int32_t layer,
                          int32_t tokens_per_split, int32_t max_splits, void* mid_o,
                          void* mid_lse, void* stream) {
    return decode_impl(q, o, pool, block_table, max_blocks_per_seq, seq_ids, seq_lens, n,
                       num_q_heads, softmax_scale, layer, tokens_per_split, max_splits, mid_o,
                       mid_lse, nullptr, nullptr, nullptr, nullptr, stream);
}

// ---- the entry point that allocates nothing ----------------------------------------------
// Split partials of mkv_paged_attn_decode_static live here instead of in a caller-provided
// workspace: one array per GPU, held from library load until the process ends.  On the host the
// array's name is only a handle for hipGetSymbolAddress; kernels receive the device address kept
// in g_static_scratch[device].
static constexpr size_t kStaticScratchBytes = 16u << 20;
static constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::mutex g_static_scratch_mu;
static void* g_static_scratch[kMaxDevices] = {};

int mkv_paged_attn_decode_static(const void* q, void* o, const mkv_pool* pool,
                                 const int32_t* block_table, int64_t max_blocks_per_seq,
                                 const int32_t* seq_ids, const int32_t* seq_lens, int32_t n,
                                 int32_t num_q_heads, float softmax_scale, int32_t layer,
                                 int32_t tokens_per_split, int32_t max_splits, void* stream) {
    MKV_REQUIRE(n >= 0 && num_q_heads > 0 && max_splits >= 1, "bad sizes (n=%d, Hq=%d, max_splits=%d)", n,
                num_q_heads, max_splits);
    // mid_o [n, Hq, max_splits, 128] fp32 followed by mid_lse [n, Hq, max_splits] fp32
    const uint64_t rows = (uint64_t)n * (uint64_t)num_q_heads * (uint64_t)max_splits;
    const uint64_t mid_o_bytes = rows * mkv::kD * 4;
    const uint64_t need = max_splits > 1 ? mid_o_bytes + rows * 4 : 0;
    MKV_REQUIRE(need <= kStaticScratchBytes,
                "mkv_paged_attn_decode_static: n * num_q_heads * max_splits = %llu rows of split partials need "
                "%llu bytes, the built-in scratch holds %llu (use mkv_paged_attn_decode with a workspace)",
                (unsigned long long)rows, (unsigned long long)need, (unsigned long long)kStaticScratchBytes);
    int dev = 0;
    MKV_HIP(hipGetDevice(&dev));
    MKV_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index %d outside [0, %d)", dev, kMaxDevices);
    void* base = nullptr;
    {
        std::lock_guard<std::mutex> lk(g_static_scratch_mu);
        if (g_static_scratch[dev] == nullptr) {       // once per device, with that device current
            void* p = nullptr;
            MKV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            MKV_REQUIRE(p != nullptr, "hipGetSymbolAddress returned a NULL address for the scratch array");
            g_static_scratch[dev] = p;
        }
        base = g_static_scratch[dev];
    }
    void* mid_o = max_splits > 1 ? base : nullptr;
    void* mid_lse = max_splits > 1 ? (void*)((char*)base + mid_o_bytes) : nullptr;
    return decode_impl(q, o, pool, block_table, max_blocks_per_seq, seq_ids, seq_lens, n, num_q_heads,
                       softmax_scale, layer, tokens_per_split, max_splits, mid_o, mid_lse, nullptr, nullptr,
                       nullptr, nullptr, stream);
}

int mkv_decode_append_attn(const void* k, const void* v, const void* q, void* o,
                           const mkv_pool* pool, const int32_t* block_table,
                           int64_t max_blocks_per_seq, const int32_t* seq_ids,
                           const int32_t* seq_lens, int32_t n, int32_t num_q_heads,
                           float softmax_scale, int32_t layer, int32_t tokens_per_split,
                           int32_t max_splits, void* mid_o, void* mid_lse, void* stream) {
    MKV_REQUIRE(n == 0 || (k && v), "k/v are NULL");
    MKV_REQUIRE(((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0, "k/v must be 16-byte aligned");
    return decode_impl(q, o, pool, block_table, max_blocks_per_seq, seq_ids, seq_lens, n,
                       num_q_heads, softmax_scale, layer, tokens_per_split, max_splits, mid_o,
                       mid_lse, k, v, nullptr, nullptr, stream);
}

int mkv_decode_rope_append_attn(const void* k, const void* v, const void* q, const void* cos_table,
                                const void* sin_table, void* o, const mkv_pool* pool,
                                const int32_t* block_table, int64_t max_blocks_per_seq,
                                const int32_t* seq_ids, const int32_t* seq_lens, int32_t n,
                                int32_t num_q_heads, float softmax_scale, int32_t layer,
                                int32_t tokens_per_split, int32_t max_splits, void* mid_o, void* mid_lse,
                                void* stream) {
    MKV_REQUIRE(n == 0 || (k && v && cos_table && sin_table), "k/v/cos/sin are NULL");
    MKV_REQUIRE(((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0 && ((uintptr_t)cos_table & 15) == 0 &&
                    ((uintptr_t)sin_table & 15) == 0,
                "k/v/cos/sin must be 16-byte aligned");
    return decode_impl(q, o, pool, block_table, max_blocks_per_seq, seq_ids, seq_lens, n,
                       num_q_heads, softmax_scale, layer, tokens_per_split, max_splits, mid_o,
                       mid_lse, k, v, cos_table, sin_table, stream);
}

int mkv_decode_order(const int32_t* seq_lens, int32_t n, int32_t num_kv_heads, int32_t* order, void* stream) {
    MKV_REQUIRE(n >= 0, "n must be >= 0");
    if (n == 0) return MKV_OK;
    MKV_REQUIRE(seq_lens && order, "NULL argument");
    MKV_REQUIRE(n <= 4096, "at most 4096 sequences (got %d)", n);
    MKV_REQUIRE(num_kv_heads > 0, "num_kv_heads must be positive");
    // slots one run apart share a CU (one workgroup per kv head and slot, handed to the CUs in turn); when
    // the kv heads do not divide the CU count there is no such pairing and the order is plain longest-first
    const int cus = mkv::num_cus();
    const int run = (cus % num_kv_heads == 0 && cus / num_kv_heads >= 1) ? cus / num_kv_heads : n;
    hipLaunchKernelGGL(mkv::decode_order_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, seq_lens, n, run, order);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_decode_attn_ordered(const void* q, void* o, const mkv_pool* pool, const int32_t* block_table,
                            int64_t max_blocks_per_seq, const int32_t* seq_ids, const int32_t* seq_lens,
                            const int32_t* order, int32_t n, int32_t num_q_heads, float softmax_scale,
                            int32_t layer, int32_t tokens_per_split, int32_t max_splits, void* mid_o,
                            void* mid_lse, const void* k, const void* v, const void* cos_table,
                            const void* sin_table, void* stream) {
    MKV_REQUIRE((k == nullptr) == (v == nullptr), "k and v go together");
    MKV_REQUIRE((cos_table == nullptr) == (sin_table == nullptr), "cos and sin tables go together");
    MKV_REQUIRE(!cos_table || k, "the rotary tables need the new k and v rows");
    MKV_REQUIRE(((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0 && ((uintptr_t)cos_table & 15) == 0 &&
                    ((uintptr_t)sin_table & 15) == 0 && ((uintptr_t)order & 3) == 0,
                "k/v/cos/sin must be 16-byte aligned, order 4-byte aligned");
    return decode_impl(q, o, pool, block_table, max_blocks_per_seq, seq_ids, seq_lens, n, num_q_heads,
                       softmax_scale, layer, tokens_per_split, max_splits, mid_o, mid_lse, k, v, cos_table,
                       sin_table, stream, order);
}

}  // extern "C"
