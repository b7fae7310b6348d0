// Causal (chunked-)prefill attention on the gfx950 matrix cores.
//
// One workgroup (4 waves) per (64-row query tile, q head, sequence); a wave owns
// 16 query rows.  K/V tiles of 64 keys are staged once per workgroup in LDS.
// Scores are produced TRANSPOSED, S^T = K Q^T (mfma 16x16x16 f16, fp32
// accumulate), so the accumulator layout of S^T (lane = query row, registers =
// four consecutive keys) is exactly the B-operand layout of the second product
// O^T = V^T P^T: probabilities go from the softmax straight back into the
// matrix core without any cross-lane movement.  Online softmax in fp32, base 2;
// a query row's running max is reduced over the four lane groups that share it.
//
// Two K/V sources: the batch's own contiguous k, v ([T, Hkv, D]) -- the
// reference's whole-prompt prefill -- or the paged cache through the block
// table, where a chunk of queries at positions prefix .. prefix+len-1 attends to
// everything cached up to its own position.
#include "common.h"

namespace mkv {

typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

static constexpr int kPD = 128;             // head dim
static constexpr int kQTile = 64;           // query rows per workgroup
static constexpr int kKTile = 64;           // keys staged per iteration
static constexpr int kRowBytes = 272;       // LDS row stride: 256 data + 16 pad (bank spread)
static constexpr float kPNegBig = -1.0e30f;
static constexpr float kPLog2e = 1.442695040888963f;

struct PrefillArgs {
    const __half* q;          // [T, Hq, D]
    __half* o;                // [T, Hq, D]
    const __half* k;          // contiguous source: [T, Hkv, D]
    const __half* v;
    const int32_t* start_locs;    // [num_seqs] first row of each sequence in q / k / v
    const int32_t* seq_lens;      // [num_seqs] query rows per sequence
    const int32_t* prefix_lens;   // paged source: cached tokens before the chunk (NULL = 0)
    const int32_t* seq_ids;       // paged source
    const int32_t* block_table;   // paged source
    int64_t max_blocks_per_seq;
    int32_t num_q_heads;
    int32_t num_kv_heads;
    int32_t layer;
    float scale2;
};

__device__ __forceinline__ float pf_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <bool PAGED>
__global__ __launch_bounds__(256) void prefill_attn_kernel(const PrefillArgs a, const mkv_pool pool) {
    __shared__ __attribute__((aligned(16))) char k_lds[kKTile * kRowBytes];
    __shared__ __attribute__((aligned(16))) char v_lds[kKTile * kRowBytes];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int m = lane & 15;          // query row (B / C column) or key / dim row (A)
    const int c = lane >> 4;          // lane group
    const int qt = blockIdx.x;
    const int hq = blockIdx.y;
    const int b = blockIdx.z;
    const int Hq = a.num_q_heads;
    const int Hkv = a.num_kv_heads;
    const int kvh = hq / (Hq / Hkv);

    const int len = a.seq_lens[b];
    const int q0 = qt * kQTile;
    if (q0 >= len) return;
    const int64_t start = a.start_locs[b];
    const int prefix = (PAGED && a.prefix_lens) ? a.prefix_lens[b] : 0;
    const int kv_len = prefix + min(len, q0 + kQTile);       // keys this tile can see
    const int my_row = q0 + wave * 16 + m;                   // chunk-local query row of this lane
    const int my_pos = prefix + my_row;                      // its position in the sequence
    const int wave_max_pos = prefix + min(len - 1, q0 + wave * 16 + 15);

    // Q^T as B operand: lane (row m, group c) holds dims c*32 + kk*4 .. +3, kk = 0..7
    // (the contraction order over dims is free; K uses the same permutation).
    v4h qb[8];
    {
        uint4 raw[4];
        if (my_row < len) {
            const uint4* qp = (const uint4*)(a.q + ((start + my_row) * Hq + hq) * kPD + c * 32);
#pragma unroll
            for (int x = 0; x < 4; ++x) raw[x] = qp[x];
        } else {
#pragma unroll
            for (int x = 0; x < 4; ++x) raw[x] = make_uint4(0u, 0u, 0u, 0u);
        }
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const uint2 lo = make_uint2(raw[x].x, raw[x].y);
            const uint2 hi = make_uint2(raw[x].z, raw[x].w);
            qb[2 * x] = __builtin_bit_cast(v4h, lo);
            qb[2 * x + 1] = __builtin_bit_cast(v4h, hi);
        }
    }

    v4f acc[8];                       // O^T tiles: dims 16t + 4c + j, query row m
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[t] = (v4f){0.f, 0.f, 0.f, 0.f};
    float m_run = kPNegBig;
    float l_run = 0.f;                // per-lane partial of the row sum (reduced over c at the end)

    const int64_t block_bytes = PAGED ? pool_block_bytes(pool) : 0;
    const int64_t total_blocks = PAGED ? pool_total_blocks(pool) : 0;
    const int32_t* bt_row = PAGED ? a.block_table + (int64_t)a.seq_ids[b] * a.max_blocks_per_seq : nullptr;

    for (int key0 = 0; key0 < kv_len; key0 += kKTile) {
        __syncthreads();              // previous tile fully consumed
        // ---- stage 64 keys of K and V in LDS (16 bytes per thread per step) ----
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int idx = tid + 256 * u;
            const int key = idx >> 4;
            const int ch = idx & 15;
            const int pos = key0 + key;
            uint4 kk4 = make_uint4(0u, 0u, 0u, 0u), vv4 = kk4;
            if (pos < kv_len) {
                if (PAGED) {
                    const int64_t pid = bt_row[pos / pool.block_size];
                    if (pid >= 0 && pid < total_blocks) {
                        BlockAddr ba = block_addr(pool, pid, block_bytes);
                        const int64_t off = ((int64_t)a.layer * Hkv + kvh) * ((int64_t)pool.block_size * kPD * 2) +
                                            (int64_t)(pos % pool.block_size) * (kPD * 2) + ch * 16;
                        kk4 = *(const uint4*)(ba.k + off);
                        vv4 = *(const uint4*)(ba.v + off);
                    }
                } else {
                    const int64_t off = ((start + pos) * Hkv + kvh) * kPD + ch * 8;
                    kk4 = *(const uint4*)(a.k + off);
                    vv4 = *(const uint4*)(a.v + off);
                }
            }
            *(uint4*)(k_lds + key * kRowBytes + ch * 16) = kk4;
            *(uint4*)(v_lds + key * kRowBytes + ch * 16) = vv4;
        }
        __syncthreads();

        // ---- four 16-key sub-tiles ------------------------------------------------
        float s[4][4];
        bool live[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            live[n] = (key0 + 16 * n) <= wave_max_pos && (key0 + 16 * n) < kv_len;   // wave-uniform
            v4f st = (v4f){0.f, 0.f, 0.f, 0.f};
            if (live[n]) {
                const uint4* kr = (const uint4*)(k_lds + (16 * n + m) * kRowBytes + c * 64);
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const uint4 w = kr[x];
                    const v4h a0 = __builtin_bit_cast(v4h, make_uint2(w.x, w.y));
                    const v4h a1 = __builtin_bit_cast(v4h, make_uint2(w.z, w.w));
                    st = __builtin_amdgcn_mfma_f32_16x16x16f16(a0, qb[2 * x], st, 0, 0, 0);
                    st = __builtin_amdgcn_mfma_f32_16x16x16f16(a1, qb[2 * x + 1], st, 0, 0, 0);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int key_pos = key0 + 16 * n + 4 * c + j;
                const bool ok = live[n] && key_pos <= my_pos && key_pos < kv_len;
                s[n][j] = ok ? st[j] * a.scale2 : kPNegBig;
            }
        }
        float mx = m_run;
#pragma unroll
        for (int n = 0; n < 4; ++n)
#pragma unroll
            for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[n][j]);
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float alpha = pf_exp2(m_run - mx);
        m_run = mx;
        l_run *= alpha;
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[t] *= alpha;

#pragma unroll
        for (int n = 0; n < 4; ++n) {
            if (!live[n]) continue;
            float p[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                p[j] = (s[n][j] > 0.5f * kPNegBig) ? pf_exp2(s[n][j] - mx) : 0.f;
                l_run += p[j];
            }
            const v4h pb = (v4h){(_Float16)p[0], (_Float16)p[1], (_Float16)p[2], (_Float16)p[3]};
            // A operand = V^T: lane (dim row m of tile t, group c) holds keys 4c .. 4c+3
            const _Float16* vbase = (const _Float16*)(v_lds + (16 * n + 4 * c) * kRowBytes) + m;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                v4h va;
                va[0] = vbase[0 * (kRowBytes / 2) + 16 * t];
                va[1] = vbase[1 * (kRowBytes / 2) + 16 * t];
                va[2] = vbase[2 * (kRowBytes / 2) + 16 * t];
                va[3] = vbase[3 * (kRowBytes / 2) + 16 * t];
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(va, pb, acc[t], 0, 0, 0);
            }
        }
    }

    float l_tot = l_run + __shfl_xor(l_run, 16);
    l_tot += __shfl_xor(l_tot, 32);
    if (my_row < len) {
        const float inv = 1.f / l_tot;
        __half* op = a.o + ((start + my_row) * Hq + hq) * kPD;
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            const v4h out = (v4h){(_Float16)(acc[t][0] * inv), (_Float16)(acc[t][1] * inv),
                                  (_Float16)(acc[t][2] * inv), (_Float16)(acc[t][3] * inv)};
            *(uint2*)(op + 16 * t + 4 * c) = __builtin_bit_cast(uint2, out);
        }
    }
}

static int launch_prefill(bool paged, const PrefillArgs& a, const mkv_pool* pool, int num_seqs,
                          int max_len, hipStream_t s) {
    dim3 grid((unsigned)cdiv(max_len, kQTile), (unsigned)a.num_q_heads, (unsigned)num_seqs);
    static const mkv_pool empty = {};
    {
        ProfScope prof(MKV_K_PREFILL_ATTN, s);
        if (paged) {
            hipLaunchKernelGGL(prefill_attn_kernel<true>, grid, dim3(256), 0, s, a, *pool);
        } else {
            hipLaunchKernelGGL(prefill_attn_kernel<false>, grid, dim3(256), 0, s, a, empty);
        }
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

}  // namespace mkv

extern "C" {

int mkv_prefill_attn(const void* q, const void* k, const void* v, void* o,
                     const int32_t* start_locs, const int32_t* seq_lens, int32_t num_seqs,
                     int32_t max_len, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                     float softmax_scale, void* stream) {
    MKV_REQUIRE(num_seqs >= 0 && max_len >= 0, "num_seqs/max_len must be >= 0");
    if (num_seqs == 0 || max_len == 0) return MKV_OK;
    MKV_REQUIRE(q && k && v && o && start_locs && seq_lens, "NULL argument");
    MKV_REQUIRE(head_dim == mkv::kPD, "prefill attention supports head_dim 128 only (got %d)", head_dim);
    MKV_REQUIRE(num_kv_heads > 0 && num_q_heads > 0 && num_q_heads % num_kv_heads == 0,
                "num_q_heads %d must be a multiple of num_kv_heads %d", num_q_heads, num_kv_heads);
    MKV_REQUIRE(num_seqs <= 65535 && num_q_heads <= 65535, "grid dimension limit");
    MKV_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0 &&
                    ((uintptr_t)o & 7) == 0,
                "q/k/v must be 16-byte aligned, o 8-byte aligned");
    mkv::PrefillArgs a = {};
    a.q = (const __half*)q;
    a.o = (__half*)o;
    a.k = (const __half*)k;
    a.v = (const __half*)v;
    a.start_locs = start_locs;
    a.seq_lens = seq_lens;
    a.num_q_heads = num_q_heads;
    a.num_kv_heads = num_kv_heads;
    a.scale2 = softmax_scale * mkv::kPLog2e;
    return mkv::launch_prefill(false, a, nullptr, num_seqs, max_len, (hipStream_t)stream);
}

int mkv_prefill_attn_paged(const void* q, void* o, const mkv_pool* pool,
                           const int32_t* block_table, int64_t max_blocks_per_seq,
                           const int32_t* seq_ids, const int32_t* start_locs,
                           const int32_t* chunk_lens, const int32_t* prefix_lens,
                           int32_t num_seqs, int32_t max_chunk_len, int32_t num_q_heads,
                           float softmax_scale, int32_t layer, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(num_seqs >= 0 && max_chunk_len >= 0, "num_seqs/max_chunk_len must be >= 0");
    if (num_seqs == 0 || max_chunk_len == 0) return MKV_OK;
    MKV_REQUIRE(q && o && block_table && seq_ids && start_locs && chunk_lens, "NULL argument");
    MKV_REQUIRE(pool->head_dim == mkv::kPD, "prefill attention supports head_dim 128 only (got %d)", pool->head_dim);
    MKV_REQUIRE(layer >= 0 && layer < pool->num_layers, "layer %d outside [0, %d)", layer, pool->num_layers);
    MKV_REQUIRE(num_q_heads > 0 && num_q_heads % pool->num_kv_heads == 0,
                "num_q_heads %d must be a multiple of num_kv_heads %d", num_q_heads, pool->num_kv_heads);
    MKV_REQUIRE(num_seqs <= 65535 && num_q_heads <= 65535, "grid dimension limit");
    MKV_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)o & 7) == 0,
                "q must be 16-byte aligned, o 8-byte aligned");
    mkv::PrefillArgs a = {};
    a.q = (const __half*)q;
    a.o = (__half*)o;
    a.start_locs = start_locs;
    a.seq_lens = chunk_lens;
    a.prefix_lens = prefix_lens;
    a.seq_ids = seq_ids;
    a.block_table = block_table;
    a.max_blocks_per_seq = max_blocks_per_seq;
    a.num_q_heads = num_q_heads;
    a.num_kv_heads = pool->num_kv_heads;
    a.layer = layer;
    a.scale2 = softmax_scale * mkv::kPLog2e;
    return mkv::launch_prefill(true, a, pool, num_seqs, max_chunk_len, (hipStream_t)stream);
}

}  // extern "C"
