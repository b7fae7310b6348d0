/*
 * C restatement of the paged-KV hot path (CPU).  TEST INFRASTRUCTURE ONLY: it is
 * compiled by oracle/build.py, loaded by tests/ and by the cpu_baseline leg of
 * bench.py, and never linked into or called by the shipped library.
 *
 * Reference lines followed (MS/ = MorphServe/, CS/ = csrc/src/):
 *   ora_append_decode    MS/worker/kernels/kvcache_mgmt.py:52-81, :189-251
 *   ora_append_prefill   MS/worker/kernels/kvcache_mgmt.py:12-50, :84-187
 *   ora_block_offset     MS/worker/kernels/kvcache_mgmt.py:169-183 (segment rule)
 *   ora_paged_attention  MS/worker/kernels/paged_attn.py:1397-1432 (fp32 math)
 *   ora_take_first_free  MS/worker/block_manager.py:75-77
 *   ora_migrate          no counterpart in the reference (it refuses to shrink a
 *                        live segment, MS/server/memory_utils.py:623-624)
 *
 * Pinned by tests/test_oracle_c.py: bit-exact agreement with the independent
 * numpy restatement (oracle/ref_cpu.py, itself pinned by brute force and closed
 * forms) for the copies, and agreement to 1e-5 with its float64 evaluation for
 * attention.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef uint16_t f16;

typedef struct {
    int64_t num_layers, num_kv_heads, block_size, head_dim;
    int64_t k_base, v_base;            /* element offsets into the arena */
    int64_t num_blocks_org, seg_blocks;
    int64_t num_segments;
    const int64_t* k_seg;              /* per-segment element offsets */
    const int64_t* v_seg;
} ora_layout;

static float f16_to_f32(f16 h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static f16 f32_to_f16(float f) {            /* round to nearest even */
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    int32_t exp = (int32_t)((x >> 23) & 0xff) - 127 + 15;
    uint32_t man = x & 0x7fffffu;
    if (((x >> 23) & 0xff) == 0xff) return (f16)(sign | 0x7c00u | (man ? 0x200u : 0));
    if (exp >= 31) return (f16)(sign | 0x7c00u);
    if (exp <= 0) {
        if (exp < -10) return (f16)sign;
        man |= 0x800000u;
        int shift = 14 - exp;
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) ++half;
        return (f16)(sign | half);
    }
    uint32_t half = ((uint32_t)exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) ++half;
    return (f16)(sign | half);
}

int64_t ora_block_elems(const ora_layout* l) {
    return l->num_layers * l->num_kv_heads * l->block_size * l->head_dim;
}

int64_t ora_block_offset(const ora_layout* l, int is_v, int64_t id) {
    int64_t be = ora_block_elems(l);
    if (id < l->num_blocks_org) return (is_v ? l->v_base : l->k_base) + id * be;
    int64_t seg = (id - l->num_blocks_org) / l->seg_blocks;
    int64_t local = id - l->num_blocks_org - seg * l->seg_blocks;
    return (is_v ? l->v_seg : l->k_seg)[seg] + local * be;
}

static int64_t slab(const ora_layout* l, int is_v, int64_t id, int64_t layer, int64_t head) {
    return ora_block_offset(l, is_v, id) + (layer * l->num_kv_heads + head) * l->block_size * l->head_dim;
}

void ora_append_decode(f16* arena, const ora_layout* l, const f16* k, const f16* v,
                       const int32_t* block_table, int64_t max_blocks_per_seq,
                       const int32_t* seq_ids, const int32_t* seq_lens, int64_t n, int64_t layer) {
    const int64_t H = l->num_kv_heads, D = l->head_dim, B = l->block_size;
    for (int64_t i = 0; i < n; ++i) {
        int64_t pos = (int64_t)seq_lens[i] - 1;
        int64_t pid = block_table[(int64_t)seq_ids[i] * max_blocks_per_seq + pos / B];
        int64_t off = pos % B;
        for (int64_t h = 0; h < H; ++h) {
            memcpy(arena + slab(l, 0, pid, layer, h) + off * D, k + (i * H + h) * D, (size_t)D * 2);
            memcpy(arena + slab(l, 1, pid, layer, h) + off * D, v + (i * H + h) * D, (size_t)D * 2);
        }
    }
}

void ora_append_prefill(f16* arena, const ora_layout* l, const f16* k, const f16* v,
                        const int32_t* block_table, int64_t max_blocks_per_seq,
                        const int32_t* seq_ids, const int32_t* start_locs,
                        const int32_t* seq_lens, int64_t num_seqs, int64_t layer) {
    const int64_t H = l->num_kv_heads, D = l->head_dim, B = l->block_size;
    for (int64_t b = 0; b < num_seqs; ++b) {
        const int32_t* row = block_table + (int64_t)seq_ids[b] * max_blocks_per_seq;
        for (int64_t t = 0; t < seq_lens[b]; ++t) {
            int64_t pid = row[t / B], off = t % B, src = (int64_t)start_locs[b] + t;
            for (int64_t h = 0; h < H; ++h) {
                memcpy(arena + slab(l, 0, pid, layer, h) + off * D, k + (src * H + h) * D, (size_t)D * 2);
                memcpy(arena + slab(l, 1, pid, layer, h) + off * D, v + (src * H + h) * D, (size_t)D * 2);
            }
        }
    }
}

/* q, o : [n, Hq, D] fp16.  Scores, softmax and the weighted sum in fp32. */
void ora_paged_attention(const f16* q, f16* o, const f16* arena, const ora_layout* l,
                         const int32_t* block_table, int64_t max_blocks_per_seq,
                         const int32_t* seq_ids, const int32_t* seq_lens, int64_t n, int64_t Hq,
                         float softmax_scale, int64_t layer) {
    const int64_t H = l->num_kv_heads, D = l->head_dim, B = l->block_size, G = Hq / H;
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int64_t i = 0; i < n; ++i) {
        for (int64_t hq = 0; hq < Hq; ++hq) {
            const int64_t len = seq_lens[i], kvh = hq / G;
            const int32_t* row = block_table + (int64_t)seq_ids[i] * max_blocks_per_seq;
            float* s = (float*)malloc((size_t)len * sizeof(float));
            float* qf = (float*)malloc((size_t)D * sizeof(float));
            float* acc = (float*)calloc((size_t)D, sizeof(float));
            for (int64_t d = 0; d < D; ++d) qf[d] = f16_to_f32(q[(i * Hq + hq) * D + d]);
            float mx = -INFINITY;
            for (int64_t t = 0; t < len; ++t) {
                const f16* kr = arena + slab(l, 0, row[t / B], layer, kvh) + (t % B) * D;
                float dot = 0.f;
                for (int64_t d = 0; d < D; ++d) dot += qf[d] * f16_to_f32(kr[d]);
                s[t] = dot * softmax_scale;
                if (s[t] > mx) mx = s[t];
            }
            float sum = 0.f;
            for (int64_t t = 0; t < len; ++t) { s[t] = expf(s[t] - mx); sum += s[t]; }
            for (int64_t t = 0; t < len; ++t) {
                const f16* vr = arena + slab(l, 1, row[t / B], layer, kvh) + (t % B) * D;
                const float p = s[t] / sum;
                for (int64_t d = 0; d < D; ++d) acc[d] += p * f16_to_f32(vr[d]);
            }
            for (int64_t d = 0; d < D; ++d) o[(i * Hq + hq) * D + d] = f32_to_f16(acc[d]);
            free(s); free(qf); free(acc);
        }
    }
}

/* The n lowest free ids ascending; marks them used.  Returns how many were found. */
int64_t ora_take_first_free(uint8_t* is_free, int64_t num_blocks, int64_t n, int64_t* out) {
    int64_t found = 0;
    for (int64_t b = 0; b < num_blocks && found < n; ++b)
        if (is_free[b]) out[found++] = b;
    if (found < n) return found;
    for (int64_t x = 0; x < n; ++x) is_free[out[x]] = 0;
    return found;
}

/* Block copies of a migration: K and V of src[k] -> dst[k], all layers. */
void ora_migrate(f16* arena, const ora_layout* l, const int64_t* src, const int64_t* dst, int64_t moves) {
    const int64_t be = ora_block_elems(l);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < moves; ++m) {
        memcpy(arena + ora_block_offset(l, 0, dst[m]), arena + ora_block_offset(l, 0, src[m]), (size_t)be * 2);
        memcpy(arena + ora_block_offset(l, 1, dst[m]), arena + ora_block_offset(l, 1, src[m]), (size_t)be * 2);
    }
}
