// Causal (chunked-)prefill attention on the gfx950 matrix cores.
//
// One workgroup of four waves per (128-row query tile, q head, sequence); a wave
// owns two 16-row column tiles (32 query rows).  K/V tiles of 64 keys are staged
// per workgroup in LDS, row-major, double buffered: while one buffer is consumed
// the next tile's global loads are in flight in registers and are written to the
// other buffer at the end of the iteration -- one barrier per tile.
//   S^T[key, row] = K[key, :] . Q^T        v_mfma_f32_16x16x32_f16, 4 per 16x16 tile
//   O^T[dim, row] += V^T[dim, key] . P^T   v_mfma_f32_16x16x32_f16 over 32 keys
// Scores are produced TRANSPOSED so that the accumulator layout of S^T (lane =
// query row, registers = four consecutive keys) is the B-operand layout of the
// second product: two 16-key score tiles side by side are its eight k-slots.
// V^T comes out of the row-major V tile through the transposing LDS read
// (ds_read_b64_tr_b16).  Every A operand (K rows, V^T) is read from LDS once
// and used for both of the wave's column tiles.  Online softmax in fp32, base 2,
// on the raw scores (the scale is folded into the exponent's fma); a query row's
// running max is reduced over the four lane groups that share it with the
// lane-swap instructions.  Tiles entirely below a wave's diagonal take a body
// without any masking; only the one or two diagonal tiles pay for the compares.
// The output leaves through LDS: each wave transposes its column tiles in a corner
// of the idle V buffer and writes whole 256-byte rows, 16 bytes per lane.  In the
// four-wave shape a workgroup that carries two query tiles requests the second
// tile's q and first K/V tile while the first tile's last key tile is consumed.
//
// Two K/V sources: the batch's own contiguous k, v ([T, Hkv, D]) -- the
// reference's whole-prompt prefill -- or the paged cache through the block
// table, where a chunk of queries at positions prefix .. prefix+len-1 attends to
// everything cached up to its own position.
#include <type_traits>

#include "common.h"

namespace mkv {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

static constexpr int kPD = 128;             // head dim
static constexpr int kKTile = 64;           // keys staged per iteration
static constexpr int kU = 2;                // 16-row column tiles per wave
static constexpr int kVPre = 4;             // V^T fragments requested ahead of the softmax arithmetic
// Waves per workgroup is a kernel parameter: 4 (128 query rows, two workgroups per CU) for short
// prompts, 8 (256 query rows, one workgroup per CU) for long ones, where a K/V tile staged once
// serves twice the rows and the next-but-one tile is already on its way in a second register set.
static constexpr int kRowBytes = 272;       // K tile row stride: 256 data + 16 pad -> conflict-free b128 row reads
static constexpr int kRowBytesV = 288;      // V tile row stride: rows 8 banks apart -> conflict-free transposing reads
static constexpr int kKBuf = kKTile * kRowBytes;
static constexpr int kVBuf = kKTile * kRowBytesV;
static constexpr float kPNegBig = -1.0e30f;
static constexpr float kPLog2e = 1.442695040888963f;
static constexpr float kLazyLog2 = 8.0f;    // growth of a row max (in octaves) that forces a rescale

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
    float scale2;                 // softmax scale * log2(e), > 0
    int32_t num_seqs;
    int32_t num_q_tiles;          // ceil(max_len / query rows per workgroup)
    int32_t pair_tiles;           // 1: a workgroup takes two query tiles (i-th from the end, i-th from the start); 0: one
};

__device__ __forceinline__ float pf_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// three-input max in one instruction (the two-input form first canonicalises both operands)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// max over the four lanes {l, l^16, l^32, l^48}: swap 16-lane rows, then 32-lane halves
__device__ __forceinline__ float max_over_groups(float x) {
    const unsigned xi = __builtin_bit_cast(unsigned, x);
    auto a = __builtin_amdgcn_permlane16_swap(xi, xi, false, false);
    x = fmaxf(__builtin_bit_cast(float, (unsigned)a[0]), __builtin_bit_cast(float, (unsigned)a[1]));
    const unsigned yi = __builtin_bit_cast(unsigned, x);
    auto b = __builtin_amdgcn_permlane32_swap(yi, yi, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)b[0]), __builtin_bit_cast(float, (unsigned)b[1]));
}
// TL: the instance that takes per-workgroup time stamps (diagnostic build only, launched while mkv_diag_timeline
// holds a buffer); the product library holds the TL = false instances alone
template <bool PAGED, int WAVES, bool TL>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void prefill_attn_kernel(const PrefillArgs a, const mkv_pool pool,
                                                                                                    const TimelineArg<TL> timeline) {
    constexpr int kThreads = 64 * WAVES;
    constexpr int kQTile = 16 * kU * WAVES;                    // query rows per workgroup
    constexpr int kFetchSteps = (kKTile * 16) / kThreads;      // 16-byte units per thread per K (or V) tile
    constexpr int kStepRows = kThreads / 16;                   // tile rows covered by one fetch step
    constexpr int kSets = WAVES == 8 ? 2 : 1;                  // staging register sets = tiles in flight
    __shared__ __attribute__((aligned(16))) char k_lds[2 * kKBuf];
    __shared__ __attribute__((aligned(16))) char v_lds[2 * kVBuf];

    const int tid = threadIdx.x;
    timeline.mark(blockIdx.x, 0);
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int m = lane & 15;          // query row of a column tile (B / C), key or dim row (A)
    const int c = lane >> 4;          // lane group
    // Workgroup id -> (query tile, q head, sequence).  Consecutive ids go to the
    // eight XCDs in turn and every XCD has its own L2, so the id's low three bits
    // pick the (sequence, head) pair's residue and ALL query tiles of a pair land
    // on one XCD: the pair's K/V is fetched into that L2 once and shared by its
    // tiles.  A workgroup takes TWO query tiles of its sequence, the i-th from the
    // end and the i-th from the start: under the causal mask their key counts add
    // up to the same total for every i, so all workgroups of a sequence carry equal
    // work.
    const int Hq = a.num_q_heads;
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    // When pairing would leave CUs short of workgroups the launcher turns it off: one tile per
    // workgroup.  An XCD hands consecutive workgroups to its 32 CUs in turn, so slots s and s + 32
    // share a CU: the XCD's (tile rank, pair) jobs, longest tiles first, are dealt to the slots in
    // snake order (every second run of 32 reversed), which puts a long and a short tile on each CU.
    int ti, pair;
    if (a.pair_tiles) {
        const int half_tiles = (a.num_q_tiles + 1) >> 1;
        ti = slot % half_tiles;
        pair = (slot / half_tiles) * 8 + xcd;
    } else {
        const int pairs_x = (Hq * a.num_seqs + 7) >> 3;
        const int run = slot >> 5, c32 = slot & 31;
        const int job = (run << 5) + ((run & 1) ? 31 - c32 : c32);
        ti = job / pairs_x;
        pair = (job - ti * pairs_x) * 8 + xcd;
        if (ti >= a.num_q_tiles) return;
    }
    if (pair >= Hq * a.num_seqs) return;
    const int hq = pair % Hq;
    const int b = pair / Hq;
    const int Hkv = a.num_kv_heads;
    const int kvh = hq / (Hq / Hkv);

    const int len = a.seq_lens[b];
    const int n_qt = (len + kQTile - 1) / kQTile;            // query tiles of THIS sequence
    if ((a.pair_tiles ? 2 * ti : ti) >= n_qt) return;
    const int64_t start = a.start_locs[b];
    const int prefix = (PAGED && a.prefix_lens) ? a.prefix_lens[b] : 0;

  // State that outlives a part: while the last key tile of part 0 is consumed, q and the first K/V
  // tile(s) of part 1 are already requested, so the second part starts without a trip to memory.
  v8h qb[kU][4];
  v4u kreg[kSets][kFetchSteps], vreg[kSets][kFetchSteps];     // staging registers: one set per tile in flight
  int32_t tile_ids = 0;
  int f_kv_len = 0;                   // the fetch side's view: keys of the part whose tiles are being requested
  uint32_t last_off = 0, next_off = 0;
  bool carried = false;               // this part's q and first tile(s) were requested by the previous part
  for (int part = 0; part < 2; ++part) {
    const int qt = part == 0 ? n_qt - 1 - ti : ti;
    if (part == 1 && (!a.pair_tiles || 2 * ti == n_qt - 1)) break;   // unpaired, or odd count: the middle tile was part 0
    const int q0 = qt * kQTile;
    const int kv_len = prefix + min(len, q0 + kQTile);       // keys this workgroup can see
    const bool more = WAVES == 4 && part == 0 && a.pair_tiles && 2 * ti != n_qt - 1;   // a second part follows (short-prompt shape only)
    const int nx_q0 = ti * kQTile;
    int nx_kv_len = more ? prefix + min(len, nx_q0 + kQTile) : 0;

    // this wave's 32 rows: chunk-local rows r0w .. r0w+31, column tile u = rows r0w+16u ..
    const int r0w = q0 + wave * (16 * kU);
    const int wave_min_pos = prefix + r0w;
    const int wave_max_pos = prefix + min(len - 1, r0w + 16 * kU - 1);   // < wave_min_pos: no row at all
    int my_row[kU], my_last_key[kU];   // a row sees keys 0 .. its own position (and < kv_len)
#pragma unroll
    for (int u = 0; u < kU; ++u) {
        my_row[u] = r0w + u * 16 + m;
        my_last_key[u] = min(prefix + my_row[u], kv_len - 1);
    }

    // Q^T as B operand: lane (row m, group c) holds dims c*32 + 8x .. +8 for product x
    // (the contraction order over dims is free; K uses the same order).
    auto load_q = [&](int tile_q0) {
        if (WAVES == 4) asm volatile("" : "+s"(tile_q0));      // the addresses are formed here, not ahead of the tile loop
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int row = tile_q0 + wave * (16 * kU) + u * 16 + m;
            if (row < len) {
                const uint4* qp = (const uint4*)(a.q + ((start + row) * Hq + hq) * kPD + c * 32);
#pragma unroll
                for (int x = 0; x < 4; ++x) qb[u][x] = __builtin_bit_cast(v8h, qp[x]);
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x) qb[u][x] = (v8h){0, 0, 0, 0, 0, 0, 0, 0};
            }
        }
    };
    if (!carried) load_q(q0);

    v4f acc[kU][8];                    // O^T tiles: dims 16t + 4c + j, query row m of column tile u
#pragma unroll
    for (int u = 0; u < kU; ++u)
#pragma unroll
        for (int t = 0; t < 8; ++t) acc[u][t] = (v4f){0.f, 0.f, 0.f, 0.f};
    // Row sums come out of the matrix cores as well: a V^T row of ones turns the second
    // product into sum_k P^T[k, row], so every register of lsum[u] holds the row's sum of the
    // fp16-rounded probabilities -- the same values the numerator is built from.
    float m_run[kU];                   // running max of the RAW scores
    v4f lsum[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
        m_run[u] = kPNegBig;
        lsum[u] = (v4f){0.f, 0.f, 0.f, 0.f};
    }
    const v8h ones = (v8h){1, 1, 1, 1, 1, 1, 1, 1};

    const int64_t block_bytes = PAGED ? pool_block_bytes(pool) : 0;
    const int64_t total_blocks = PAGED ? pool_total_blocks(pool) : 0;
    const int32_t* bt_row = PAGED ? a.block_table + (int64_t)a.seq_ids[b] * a.max_blocks_per_seq : nullptr;

    // global -> registers for one 64-key tile: 16 bytes per thread per step.  Keys at or past
    // kv_len re-read the last visible key (finite values; their scores are masked and their
    // probabilities are zero); unmapped table entries read as zeros.
    // Contiguous source: one uniform base per (sequence, kv head) plus a 32-bit byte offset
    // per lane that advances by a constant per tile (the launcher bounds len * Hkv * 256).
    const uint32_t row_stride = (uint32_t)Hkv * (kPD * 2);
    const char* k_src = PAGED ? nullptr : (const char*)a.k + (start * Hkv + kvh) * (int64_t)(kPD * 2);
    const char* v_src = PAGED ? nullptr : (const char*)a.v + (start * Hkv + kvh) * (int64_t)(kPD * 2);
    auto begin_fetch = [&](int kvl) {
        f_kv_len = kvl;
        last_off = (uint32_t)(kvl - 1) * row_stride + (tid & 15) * 16;
        next_off = (uint32_t)(tid >> 4) * row_stride + (tid & 15) * 16;          // key (tid >> 4) of the next tile
    };
    // Paged source: fetch step u covers keys key0 + 16u .. +15 = ONE block (block_size is 16
    // here), so its id and address are workgroup-uniform and only the row inside it differs
    // per thread.  The four ids of a tile are loaded one tile ahead (lane u keeps step u's),
    // so no fetch ever waits on a table lookup.
    auto load_tile_ids = [&](int key0, int kvl) {
        if (PAGED) {      // entries past the table row name no block: they read as zeros, never as a neighbour's row
            const int idx = min((key0 >> 4) + (lane & 3), (kvl - 1) >> 4);
            tile_ids = idx < a.max_blocks_per_seq ? bt_row[idx] : -1;
        }
    };
    if (!carried) {
        begin_fetch(kv_len);
        load_tile_ids(0, kv_len);
    }
    auto fetch_tile = [&](int key0, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
#pragma unroll
        for (int u = 0; u < kFetchSteps; ++u) {
            if (PAGED) {
                // a step covers kStepRows keys = kStepRows / 16 blocks; a wave's rows lie in one of them
                const int blk_in_tile = (kStepRows / 16) * u + ((tid >> 4) >> 4);      // wave-uniform
                const int blk = min((key0 >> 4) + blk_in_tile, (f_kv_len - 1) >> 4);
                const int pos = min(key0 + kStepRows * u + (tid >> 4), f_kv_len - 1);
                const int64_t pid = __builtin_amdgcn_readlane(tile_ids, __builtin_amdgcn_readfirstlane(blk_in_tile));
                kreg[SET][u] = (v4u){0u, 0u, 0u, 0u};
                vreg[SET][u] = kreg[SET][u];
                if (pid >= 0 && pid < total_blocks) {
                    BlockAddr ba = block_addr(pool, pid, block_bytes);
                    const int64_t head_off = ((int64_t)a.layer * Hkv + kvh) * (int64_t)(16 * kPD * 2);
                    const uint32_t off = (uint32_t)(pos - (blk << 4)) * (kPD * 2) + (tid & 15) * 16;
                    kreg[SET][u] = *(const v4u*)(ba.k + head_off + off);
                    vreg[SET][u] = *(const v4u*)(ba.v + head_off + off);
                }
            } else {
                const uint32_t off = min(next_off + (uint32_t)u * (uint32_t)kStepRows * row_stride, last_off);
                kreg[SET][u] = *(const v4u*)(k_src + off);
                vreg[SET][u] = *(const v4u*)(v_src + off);
            }
        }
        next_off += kKTile * row_stride;
        // the ids of the tile after this one; after a part's last tile, those of the next part's first
        if (nx_kv_len != 0 && key0 + kKTile >= f_kv_len) {
            load_tile_ids(0, nx_kv_len);
        } else {
            load_tile_ids(key0 + kKTile, f_kv_len);
        }
    };
    const int k_wr_off = (tid >> 4) * kRowBytes + (tid & 15) * 16;           // + 16u rows
    const int v_wr_off = (tid >> 4) * kRowBytesV + (tid & 15) * 16;
    auto stage_tile = [&](int buf, auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
        char* kw = k_lds + buf * kKBuf + k_wr_off;
        char* vw = v_lds + buf * kVBuf + v_wr_off;
#pragma unroll
        for (int u = 0; u < kFetchSteps; ++u) {
            *(v4u*)(kw + u * kStepRows * kRowBytes) = kreg[SET][u];
            *(v4u*)(vw + u * kStepRows * kRowBytesV) = vreg[SET][u];
        }
    };

    const int k_rd_off = m * kRowBytes + c * 64;                            // + 16n rows, + 16x bytes
    const int v_rd_off = (4 * c + (m >> 2)) * kRowBytesV + (m & 3) * 8;     // + 16n rows, + 32t bytes

    // one 64-key tile against this wave's 32 rows
    auto tile_body = [&](auto masked_tag, int buf, int key0, const uint4 (&kf_first)[4], int reload_q0) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const char* k_rd = k_lds + buf * kKBuf + k_rd_off;
        const char* v_rd = v_lds + buf * kVBuf + v_rd_off;
        // ---- raw scores of the four 16-key sub-tiles, both column tiles ------------------
        // (matrix phases run at raised wave priority: the SIMD's other wave fills the gaps with
        // its softmax arithmetic instead of competing for the matrix pipe in lockstep)
        __builtin_amdgcn_s_setprio(2);
        // K fragments of sub-tile n+1 are requested before the products of sub-tile n, so
        // the LDS latency is covered by eight matrix instructions
        v4f st[kU][4];
        uint4 kf[2][4];
#pragma unroll
        for (int x = 0; x < 4; ++x) kf[0][x] = kf_first[x];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
            if (n < 3) {
                const uint4* kr = (const uint4*)(k_rd + 16 * (n + 1) * kRowBytes);
#pragma unroll
                for (int x = 0; x < 4; ++x) kf[(n + 1) & 1][x] = kr[x];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kU; ++u) st[u][n] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const v8h ka = __builtin_bit_cast(v8h, kf[n & 1][x]);
#pragma unroll
                for (int u = 0; u < kU; ++u)
                    st[u][n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qb[u][x], st[u][n], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (MASKED) {
#pragma unroll
                for (int u = 0; u < kU; ++u)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int key_pos = key0 + 16 * n + 4 * c + j;
                        if (key_pos > my_last_key[u]) st[u][n][j] = kPNegBig;
                    }
            }
        }
        // V^T fragments of the first kVPre products are requested now: their LDS latency passes
        // under the softmax arithmetic instead of in front of the second matrix phase
        v8h va_pre[kVPre];
#pragma unroll
        for (int t = 0; t < kVPre; ++t) {
            const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (v4s __attribute__((address_space(3)))*)(v_rd + 32 * t));
            const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (v4s __attribute__((address_space(3)))*)(v_rd + 16 * kRowBytesV + 32 * t));
            va_pre[t] = __builtin_bit_cast(v8h, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
        __builtin_amdgcn_sched_barrier(0);
        // the scores were q's last use in this part: the next part's q is requested here
        if (reload_q0 >= 0) load_q(reload_q0);
        // ---- online softmax per column tile -----------------------------------------------
        __builtin_amdgcn_s_setprio(0);
        v8h pb[kU][2];                 // P^T as B operand: [pair of sub-tiles] = 8 k-slots
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            float mx = m_run[u];
#pragma unroll
            for (int n = 0; n < 4; ++n) mx = max3(max3(mx, st[u][n][0], st[u][n][1]), st[u][n][2], st[u][n][3]);
            // m_run is the exponent's reference point, not necessarily the exact running max:
            // it is moved (and the accumulators rescaled) only when some row's max has grown
            // by more than kLazyLog2 octaves, so probabilities stay below 2^kLazyLog2 -- well
            // inside fp16 -- and the final acc / lsum is the same quotient either way.
            // Some row has outgrown the reference iff some LANE's own scores have, so the test
            // runs on the lane-local max and the row max is completed across the four lane
            // groups only when the reference does move.
            if (__ballot((mx - m_run[u]) * a.scale2 > kLazyLog2) != 0) {      // wave-uniform branch
                mx = max_over_groups(mx);
                const float alpha = pf_exp2((m_run[u] - mx) * a.scale2);
                lsum[u] *= alpha;
#pragma unroll
                for (int t = 0; t < 8; ++t) acc[u][t] *= alpha;
                m_run[u] = mx;
            }
            const float ms = -m_run[u] * a.scale2;
            float p[4][4];
#pragma unroll
            for (int n = 0; n < 4; ++n)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    p[n][j] = pf_exp2(__builtin_fmaf(st[u][n][j], a.scale2, ms));   // masked: exp2(-huge) = 0
#pragma unroll
            for (int h = 0; h < 2; ++h)
                pb[u][h] = (v8h){(_Float16)p[2 * h][0],     (_Float16)p[2 * h][1],     (_Float16)p[2 * h][2],
                                 (_Float16)p[2 * h][3],     (_Float16)p[2 * h + 1][0], (_Float16)p[2 * h + 1][1],
                                 (_Float16)p[2 * h + 1][2], (_Float16)p[2 * h + 1][3]};
        }
        // ---- O^T += V^T . P^T, 32 keys per product ----------------------------------------
        __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const char* vp = v_rd + 32 * h * kRowBytesV;
#pragma unroll
            for (int u = 0; u < kU; ++u)
                lsum[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, pb[u][h], lsum[u], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                v8h va;
                if (h == 0 && t < kVPre) {
                    va = va_pre[t];
                } else {
                    const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (v4s __attribute__((address_space(3)))*)(vp + 32 * t));
                    const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (v4s __attribute__((address_space(3)))*)(vp + 16 * kRowBytesV + 32 * t));
                    va = __builtin_bit_cast(v8h, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
#pragma unroll
                for (int u = 0; u < kU; ++u)
                    acc[u][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va, pb[u][h], acc[u][t], 0, 0, 0);
            }
        }
        __builtin_amdgcn_s_setprio(0);
    };

    const int num_tiles = (kv_len + kKTile - 1) / kKTile;
    const bool wave_has_rows = r0w < len;
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, kSets - 1>;       // the same set when there is only one
    // tile j travels through register set j % kSets; with two sets tile it+2 is requested while tile
    // it is consumed and tile it+1, requested one iteration earlier, goes to LDS at the end
    auto first_frags = [&](int buf, uint4 (&out)[4]) {
#pragma unroll
        for (int x = 0; x < 4; ++x) out[x] = ((const uint4*)(k_lds + buf * kKBuf + k_rd_off))[x];
    };
    auto iteration = [&](int it, auto cur_set, auto nxt_set) {
        const int buf = it & 1;
        const int key0 = it * kKTile;
        const bool active = wave_has_rows && key0 <= wave_max_pos;    // wave-uniform: some row of this wave sees the tile
        // the first K fragments are requested before the address arithmetic of the global fetch,
        // which then covers their LDS latency
        uint4 kf_first[4];
        if (active) first_frags(buf, kf_first);
        __builtin_amdgcn_sched_barrier(0);
        if (kSets == 1) {
            fetch_tile(key0 + kKTile, nxt_set);       // in flight during the math below
        } else if (it + 2 < num_tiles) {
            fetch_tile(key0 + 2 * kKTile, cur_set);   // cur_set's tile went to LDS one iteration ago
        }
        if (active) {
            if (key0 + kKTile - 1 <= wave_min_pos) {  // every row sees every key (and all keys < kv_len)
                tile_body(std::false_type{}, buf, key0, kf_first, -1);
            } else {
                tile_body(std::true_type{}, buf, key0, kf_first, -1);
            }
        }
        stage_tile(buf ^ 1, nxt_set);                 // the other buffer: last read one iteration ago
        __syncthreads();
    };
    if (!carried) {
        fetch_tile(0, Set0{});
        if (kSets == 2 && num_tiles > 1) fetch_tile(kKTile, Set1{});
        stage_tile(0, Set0{});
        __syncthreads();
    }
    carried = false;
    timeline.mark(blockIdx.x, 1 + 3 * part);
    for (int it = 0; it + 1 < num_tiles; it += 2) {
        iteration(it, Set0{}, Set1{});
        if (it + 2 < num_tiles) iteration(it + 1, Set1{}, Set0{});
    }
    {   // the last tile holds the workgroup's diagonal: never fully visible to a wave
        const int it = num_tiles - 1;
        const int key0 = it * kKTile;
        const bool active = wave_has_rows && key0 <= wave_max_pos;
        uint4 kf_first[4];
        auto request_next_part = [&]() {              // both staging sets are idle: the next part's first tile(s)
            int kvl = nx_kv_len;
            asm volatile("" : "+s"(kvl));             // keeps the next part's addresses out of the tile loop's registers
            const int nx_tiles = (kvl + kKTile - 1) / kKTile;
            begin_fetch(kvl);
            nx_kv_len = 0;
            fetch_tile(0, Set0{});
            if (kSets == 2 && nx_tiles > 1) fetch_tile(kKTile, Set1{});
        };
        // Contiguous source: the request's address arithmetic covers the latency of the first K fragments, and
        // the next part's q is asked for inside the tile, once the scores have released its registers.  The
        // paged source's arithmetic needs those registers itself (fragments held across it would spill, and
        // their reload would wait for the very loads just issued): request first, q after the tile.
        if (PAGED) {
            if (more) request_next_part();
            if (active) {
                first_frags(it & 1, kf_first);
                tile_body(std::true_type{}, it & 1, key0, kf_first, -1);
            }
            if (more) load_q(nx_q0);
        } else {
            if (active) first_frags(it & 1, kf_first);
            __builtin_amdgcn_sched_barrier(0);
            if (more) request_next_part();
            if (active) tile_body(std::true_type{}, it & 1, key0, kf_first, more ? nx_q0 : -1);
            else if (more) load_q(nx_q0);
        }
        __syncthreads();                              // every read of the staged tiles is done
    }
    timeline.mark(blockIdx.x, 2 + 3 * part);

    // Output: a lane holds four dims of sixteen rows' worth of 8-byte pieces; the column tile goes
    // through this wave's corner of the idle V buffer (rows 288 bytes apart: conflict-free 8-byte
    // writes) and comes back as whole rows, so that o is written 256 contiguous bytes per row,
    // 16 bytes per lane.  The four-wave shape keeps V buffer 0 for the next part's first tile.
    {
        constexpr int kORow = 288;
        char* o_lds = v_lds + (WAVES == 4 ? kVBuf : 0) + wave * (16 * kORow);
        const bool follows = part == 0 && a.pair_tiles && 2 * ti != n_qt - 1;
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const float inv = 1.f / lsum[u][0];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const v4h out = (v4h){(_Float16)(acc[u][t][0] * inv), (_Float16)(acc[u][t][1] * inv),
                                      (_Float16)(acc[u][t][2] * inv), (_Float16)(acc[u][t][3] * inv)};
                *(uint2*)(o_lds + m * kORow + 32 * t + 8 * c) = __builtin_bit_cast(uint2, out);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 orow = *(const uint4*)(o_lds + (4 * i + c) * kORow + 16 * m);
                const int row = r0w + u * 16 + 4 * i + c;
                if (row < len) *(uint4*)(a.o + ((start + row) * Hq + hq) * kPD + 8 * m) = orow;
            }
        }
        if (more) stage_tile(0, Set0{});
        if (follows) __syncthreads();                 // the next part's staging may reuse every buffer
        if (more) carried = true;
        timeline.mark(blockIdx.x, 3 + 3 * part);
    }
  }   // part
}

static constexpr int kLongPrompt = 2048;    // shortest prompt (or chunk) from which the eight-wave kernel is used
static constexpr int kChunkRows = 256;      // ... or a chunk of at least this many rows (one eight-wave query tile)
static constexpr int kLongPrefix = 512;     //     over a cached prefix of at least this many tokens
#if MKV_DIAG
static int g_prefill_waves = 0;             // 0: by length; 4 or 8: forced (experiments and tests)
static int g_prefill_pairing = 0;           // 0: by grid size; 1: always two tiles per workgroup; 2: never
#else
static constexpr int g_prefill_waves = 0;   // the product library always chooses by the call
static constexpr int g_prefill_pairing = 0;
#endif

static int launch_prefill(bool paged, const PrefillArgs& a, const mkv_pool* pool, int num_seqs,
                          int max_len, int max_prefix, hipStream_t s) {
    PrefillArgs args = a;
    args.num_seqs = num_seqs;
    const int64_t pairs8 = ((int64_t)a.num_q_heads * num_seqs + 7) / 8 * 8;     // pairs padded to the XCD count
    // eight waves only where their workgroups (one per CU) still cover the chip; a chunk over a long cached
    // prefix streams as many key tiles as a long prompt does, so it takes the eight-wave shape from a
    // shorter chunk on (8 x 512 over 2048 cached tokens: 217 -> 207 us, 4 x 1024 over 4096: 388 -> 349 us)
    const bool many_keys = max_len >= kLongPrompt ||
                           (max_len >= kChunkRows && max_prefix >= kLongPrefix && max_len + max_prefix >= 1024);
    // (over the batch's own k, v a grid of exactly one eight-wave workgroup per CU loses to two four-wave ones:
    // 2 x 2048 tokens 86 against 79 us, 1 x 4096 158 against 142 us; from one and a half per CU on it wins)
    const int cus = num_cus();
    const bool long_and_wide = many_keys && pairs8 * ((cdiv(max_len, 16 * kU * 8) + 1) / 2) >= (paged ? cus : cus + cus / 4);
    const int waves = (g_prefill_waves == 4 || g_prefill_waves == 8) ? g_prefill_waves : (long_and_wide ? 8 : 4);
    const int q_tile = 16 * kU * waves;
    args.num_q_tiles = cdiv(max_len, q_tile);
    // two tiles per workgroup balance the causal triangle inside a workgroup; a grid that then has fewer
    // workgroups than the chip holds at once (two per CU), or sequences of at most three tiles, are better off
    // with one tile per workgroup and the balance made across the two workgroups of a CU
    // (4 x 512: 25.7 -> 22.4 us, 3 x 700: 39.0 -> 26.1 us, 1 x 1024: 32.5 -> 27.2 us, 8 x 256: 22.0 -> 18.9 us)
    const int64_t paired = pairs8 * ((args.num_q_tiles + 1) / 2);
    const bool unpair = paired < 2 * cus || args.num_q_tiles <= 3;
    args.pair_tiles = (g_prefill_pairing == 1 || (g_prefill_pairing == 0 && !unpair)) ? 1 : 0;
    const int64_t unpaired = ((pairs8 / 8 * args.num_q_tiles + 31) / 32 * 32) * 8;      // whole runs of 32 slots per XCD
    dim3 grid((unsigned)(args.pair_tiles ? paired : unpaired));
    static const mkv_pool empty = {};
    {
        MKV_PROF(MKV_K_PREFILL_ATTN, s);
#define MKV_LAUNCH(P, W, T, TH, PL, TA) \
    hipLaunchKernelGGL((prefill_attn_kernel<P, W, T>), grid, dim3(TH), 0, s, args, PL, TA)
#if MKV_DIAG
        if (long long* buf = timeline_buffer(grid.x)) {
            const TimelineArg<true> ta{buf};
            if (paged && waves == 8) MKV_LAUNCH(true, 8, true, 512, *pool, ta);
            else if (paged) MKV_LAUNCH(true, 4, true, 256, *pool, ta);
            else if (waves == 8) MKV_LAUNCH(false, 8, true, 512, empty, ta);
            else MKV_LAUNCH(false, 4, true, 256, empty, ta);
            MKV_HIP(hipGetLastError());
            return MKV_OK;
        }
#endif
        const TimelineArg<false> none{};
        if (paged && waves == 8) MKV_LAUNCH(true, 8, false, 512, *pool, none);
        else if (paged) MKV_LAUNCH(true, 4, false, 256, *pool, none);
        else if (waves == 8) MKV_LAUNCH(false, 8, false, 512, empty, none);
        else MKV_LAUNCH(false, 4, false, 256, empty, none);
#undef MKV_LAUNCH
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

}  // namespace mkv

extern "C" {

#if MKV_DIAG
int mkv_set_prefill_variant(int32_t waves) {
    const int pairing = (waves >> 8) & 3;       // bits 8-9: 0 tiles paired by grid size, 1 always, 2 never
    waves &= 0xFF;
    MKV_REQUIRE(waves == 0 || waves == 4 || waves == 8, "waves must be 0 (by length), 4 or 8");
    mkv::g_prefill_waves = waves;
    mkv::g_prefill_pairing = pairing;
    return MKV_OK;
}
#endif

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
    MKV_REQUIRE(softmax_scale > 0.f, "softmax_scale must be positive");
    MKV_REQUIRE((int64_t)max_len * num_kv_heads < (1 << 23), "max_len * num_kv_heads must be below 2^23");
    MKV_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)k & 15) == 0 && ((uintptr_t)v & 15) == 0 &&
                    ((uintptr_t)o & 15) == 0,
                "q/k/v/o must be 16-byte aligned");
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
    return mkv::launch_prefill(false, a, nullptr, num_seqs, max_len, 0, (hipStream_t)stream);
}

int mkv_prefill_attn_paged(const void* q, void* o, const mkv_pool* pool,
                           const int32_t* block_table, int64_t max_blocks_per_seq,
                           const int32_t* seq_ids, const int32_t* start_locs,
                           const int32_t* chunk_lens, const int32_t* prefix_lens,
                           int32_t num_seqs, int32_t max_chunk_len, int32_t max_prefix_len,
                           int32_t num_q_heads, float softmax_scale, int32_t layer, void* stream) {
    int rc = mkv::check_pool(pool);
    if (rc) return rc;
    MKV_REQUIRE(num_seqs >= 0 && max_chunk_len >= 0, "num_seqs/max_chunk_len must be >= 0");
    MKV_REQUIRE(max_prefix_len >= 0, "max_prefix_len must be >= 0 (0 = unknown)");
    if (num_seqs == 0 || max_chunk_len == 0) return MKV_OK;
    MKV_REQUIRE(q && o && block_table && seq_ids && start_locs && chunk_lens, "NULL argument");
    MKV_REQUIRE(pool->head_dim == mkv::kPD, "prefill attention supports head_dim 128 only (got %d)", pool->head_dim);
    MKV_REQUIRE(pool->block_size == 16, "chunked prefill supports block_size 16 only (got %d)", pool->block_size);
    MKV_REQUIRE(layer >= 0 && layer < pool->num_layers, "layer %d outside [0, %d)", layer, pool->num_layers);
    MKV_REQUIRE(num_q_heads > 0 && num_q_heads % pool->num_kv_heads == 0,
                "num_q_heads %d must be a multiple of num_kv_heads %d", num_q_heads, pool->num_kv_heads);
    MKV_REQUIRE(num_seqs <= 65535 && num_q_heads <= 65535, "grid dimension limit");
    MKV_REQUIRE(softmax_scale > 0.f, "softmax_scale must be positive");
    MKV_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)o & 15) == 0,
                "q and o must be 16-byte aligned");
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
    return mkv::launch_prefill(true, a, pool, num_seqs, max_chunk_len, max_prefix_len, (hipStream_t)stream);
}

}  // extern "C"
