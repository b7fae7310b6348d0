// Rotary position embedding of q and k, optionally fused with the KV append: the
// rotated k row and the v row of every token go straight to their cache slot, so one
// launch replaces the rotary kernel and both append kernels of a mixed batch.
//
// Arithmetic is fp16 throughout, as in the reference kernel whose operands are all
// fp16 (q, k and the cos / sin tables): each output is one fused multiply-add on top
// of one rounded product,
//     out[d]        = fma(x[d], cos[d], -(x[d + D/2] * sin[d]))
//     out[d + D/2]  = fma(x[d], sin[d],   x[d + D/2] * cos[d])        d < D/2
// (the contraction a compiler applies to "a*b - c*d" / "a*b + c*d" with fp16 operands).
#include "common.h"
#include "rope_math.h"

namespace mkv {

struct RopeArgs {
    __half* q;                    // [T, Hq, D], rotated in place
    __half* k;                    // [T, Hkv, D], rotated in place
    const __half* v;              // [T, Hkv, D] (STORE only)
    const __half* cos_t;          // [T, D/2]
    const __half* sin_t;          // [T, D/2]
    const int32_t* block_table;   // STORE only, as for the append kernels
    int64_t max_blocks_per_seq;
    const int32_t* seq_ids;       // [num_prefill_seqs + num_decoding_seqs]
    const int32_t* prefill_start_locs;
    const int32_t* prefill_lens;
    const int32_t* decoding_seq_lens;
    int32_t num_prefill_seqs;
    int32_t num_prefill_tokens;
    int32_t num_tokens;
    int32_t num_q_heads;
    int32_t num_kv_heads;
    int32_t head_dim;
    int32_t layer;
};

// One workgroup per token.  Units of eight rotation pairs: q heads first, then k heads,
// then (STORE) the 16-byte units of the v row.
template <bool STORE>
__global__ __launch_bounds__(256) void rope_store_kernel(const RopeArgs a, const mkv_pool pool) {
    const int t = blockIdx.x;
    const int D = a.head_dim;
    const int half_units = D >> 4;                 // 8-pair units per head
    const int Hq = a.num_q_heads, Hkv = a.num_kv_heads;

    // cache slot of this token's row (workgroup-uniform)
    char* k_slot = nullptr;
    char* v_slot = nullptr;
    if (STORE) {
        int64_t seq;
        int pos;
        if (t < a.num_prefill_tokens) {
            int lo = 0, hi = a.num_prefill_seqs - 1;        // last sequence that starts at or before t
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (a.prefill_start_locs[mid] <= t) lo = mid; else hi = mid - 1;
            }
            seq = a.seq_ids[lo];
            pos = t - a.prefill_start_locs[lo];
            if (pos >= a.prefill_lens[lo]) pos = -1;        // a gap between sequences: nothing to store
        } else {
            const int i = t - a.num_prefill_tokens;
            seq = a.seq_ids[a.num_prefill_seqs + i];
            pos = a.decoding_seq_lens[i] - 1;
        }
        const int blk = pos >= 0 ? pos / pool.block_size : 0;
        if (pos >= 0 && blk < a.max_blocks_per_seq) {
            const int64_t pid = a.block_table[seq * a.max_blocks_per_seq + blk];
            if (pid >= 0 && pid < pool_total_blocks(pool)) {
                BlockAddr ba = block_addr(pool, pid, pool_block_bytes(pool));
                const int64_t off = (int64_t)a.layer * Hkv * pool.block_size * D * 2 +
                                    (int64_t)(pos - blk * pool.block_size) * D * 2;
                k_slot = const_cast<char*>(ba.k) + off;     // + h * block_size * D * 2
                v_slot = const_cast<char*>(ba.v) + off;
            }
        }
    }
    const int64_t slab_bytes = STORE ? (int64_t)pool.block_size * D * 2 : 0;

    const h8* cp = (const h8*)(a.cos_t + (int64_t)t * (D >> 1));
    const h8* sp = (const h8*)(a.sin_t + (int64_t)t * (D >> 1));
    const int rot_units = (Hq + Hkv) * half_units;
    const int v_units = STORE ? Hkv * (D >> 3) : 0;
    for (int u = threadIdx.x; u < rot_units + v_units; u += blockDim.x) {
        if (u < rot_units) {
            const int head = u / half_units;
            const int c = u - head * half_units;
            const bool is_k = head >= Hq;
            __half* row = is_k ? a.k + ((int64_t)t * Hkv + (head - Hq)) * D : a.q + ((int64_t)t * Hq + head) * D;
            h8* lo = (h8*)row + c;
            h8* hi = (h8*)(row + (D >> 1)) + c;
            h8 o0, o1;
            rotate8(*lo, *hi, cp[c], sp[c], o0, o1);
            *lo = o0;
            *hi = o1;
            if (STORE && is_k && k_slot) {
                char* dst = k_slot + (int64_t)(head - Hq) * slab_bytes;
                *((h8*)dst + c) = o0;
                *((h8*)(dst + D) + c) = o1;              // D bytes = D/2 halves further
            }
        } else if (STORE) {
            const int r = u - rot_units;
            const int h = r / (D >> 3);
            const int c = r - h * (D >> 3);
            if (v_slot)
                *((uint4*)(v_slot + (int64_t)h * slab_bytes) + c) =
                    *((const uint4*)(a.v + ((int64_t)t * Hkv + h) * D) + c);
        }
    }
}

}  // namespace mkv

extern "C" {

int mkv_rope_store_kvcache(void* q, void* k, const void* v, const void* cos_table, const void* sin_table,
                           const mkv_pool* pool, const int32_t* block_table, int64_t max_blocks_per_seq,
                           const int32_t* seq_ids, const int32_t* prefill_start_locs,
                           const int32_t* prefill_lens, const int32_t* decoding_seq_lens,
                           int32_t num_prefill_seqs, int32_t num_prefill_tokens, int32_t num_decoding_seqs,
                           int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t layer,
                           int32_t store, void* stream) {
    MKV_REQUIRE(num_prefill_seqs >= 0 && num_prefill_tokens >= 0 && num_decoding_seqs >= 0, "negative count");
    const int64_t T = (int64_t)num_prefill_tokens + num_decoding_seqs;
    if (T == 0) return MKV_OK;
    MKV_REQUIRE(T <= 0x7fffffff, "too many tokens");
    MKV_REQUIRE(q && k && cos_table && sin_table, "NULL argument");
    MKV_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0 && head_dim % 16 == 0,
                "head counts must be positive and head_dim a multiple of 16 (got %d)", head_dim);
    MKV_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)k & 15) == 0 && ((uintptr_t)cos_table & 15) == 0 &&
                    ((uintptr_t)sin_table & 15) == 0,
                "q/k/cos/sin must be 16-byte aligned");
    mkv::RopeArgs a = {};
    a.q = (__half*)q;
    a.k = (__half*)k;
    a.v = (const __half*)v;
    a.cos_t = (const __half*)cos_table;
    a.sin_t = (const __half*)sin_table;
    a.num_prefill_seqs = num_prefill_seqs;
    a.num_prefill_tokens = num_prefill_tokens;
    a.num_tokens = (int32_t)T;
    a.num_q_heads = num_q_heads;
    a.num_kv_heads = num_kv_heads;
    a.head_dim = head_dim;
    hipStream_t s = (hipStream_t)stream;
    if (!store) {
        static const mkv_pool empty = {};
        hipLaunchKernelGGL(mkv::rope_store_kernel<false>, dim3((unsigned)T), dim3(256), 0, s, a, empty);
        MKV_HIP(hipGetLastError());
        return MKV_OK;
    }
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(v && block_table && seq_ids, "NULL argument");
    MKV_REQUIRE(num_prefill_seqs == 0 || (prefill_start_locs && prefill_lens), "prefill rows without their tables");
    MKV_REQUIRE(num_decoding_seqs == 0 || decoding_seq_lens, "decode rows without their lengths");
    MKV_REQUIRE(num_prefill_tokens == 0 || num_prefill_seqs > 0, "prefill tokens without prefill sequences");
    MKV_REQUIRE(pool->num_kv_heads == num_kv_heads && pool->head_dim == head_dim,
                "k has %d heads x %d, the pool %d x %d", num_kv_heads, head_dim, pool->num_kv_heads, pool->head_dim);
    MKV_REQUIRE(layer >= 0 && layer < pool->num_layers, "layer %d outside [0, %d)", layer, pool->num_layers);
    MKV_REQUIRE(((uintptr_t)v & 15) == 0, "v must be 16-byte aligned");
    a.block_table = block_table;
    a.max_blocks_per_seq = max_blocks_per_seq;
    a.seq_ids = seq_ids;
    a.prefill_start_locs = prefill_start_locs;
    a.prefill_lens = prefill_lens;
    a.decoding_seq_lens = decoding_seq_lens;
    a.layer = layer;
    {
        MKV_PROF(MKV_K_ROPE_STORE, s);
        hipLaunchKernelGGL(mkv::rope_store_kernel<true>, dim3((unsigned)T), dim3(256), 0, s, a, *pool);
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

}  // extern "C"
