// Block manager on the device: first-free allocation (ascending lowest ids, the
// order torch.nonzero would give), block-table append / release / gather, live
// counts.  Every operation is ONE single-workgroup launch: the state is small
// (one byte per block, a few ints per sequence), the work is ordered scans, and
// a single workgroup keeps them deterministic without atomics or host round
// trips between the steps.
#include "common.h"

#include <algorithm>

namespace mkv {

static constexpr int kScanThreads = 1024;
static constexpr int kScanWaves = kScanThreads / 64;
static constexpr int kBytesPerThread = 64;                 // four 16-byte loads in flight per thread
static constexpr int64_t kTileBytes = (int64_t)kScanThreads * kBytesPerThread;      // 64 Ki map bytes per round
static constexpr int kIdCache = 4096;                      // ids kept in LDS between the taking and the handing out

// Exclusive prefix sum over the workgroup (1024 threads); total returned in *total.
// All threads must call it.
template <typename T>
__device__ __forceinline__ T block_excl_scan(T v, T* total, T* sm /* [kScanWaves + 1] */) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    T inc = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        T t = __shfl_up(inc, d);
        if (lane >= d) inc += t;
    }
    __syncthreads();                       // sm reuse across calls
    if (lane == 63) sm[wave] = inc;
    __syncthreads();
    if (wave == 0) {
        T w = lane < kScanWaves ? sm[lane] : 0;
        T winc = w;
#pragma unroll
        for (int d = 1; d < kScanWaves; d <<= 1) {
            T t = __shfl_up(winc, d);
            if (lane >= d) winc += t;
        }
        if (lane < kScanWaves) sm[lane] = winc - w;       // exclusive wave offsets
        if (lane == kScanWaves - 1) sm[kScanWaves] = winc;
    }
    __syncthreads();
    *total = sm[kScanWaves];
    return sm[wave] + inc - v;
}

// 16 map bytes as a 16-bit mask of the non-zero ones.
__device__ __forceinline__ uint32_t nonzero_mask16(const uint4 w) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
    uint32_t nz = 0u;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t t = words[q];
        t |= t >> 4;
        t |= t >> 2;
        t |= t >> 1;
        t &= 0x01010101u;                                   // one flag per non-zero byte
        nz |= (((t * 0x01020408u) >> 24) & 0xfu) << (4 * q);
    }
    return nz;
}

// One thread's 64 map bytes starting at b0 (16-byte aligned as an address) as a bit mask: bit k is
// set when byte b0 + k lies in [lo, hi) and is non-zero (want != 0) or zero (want == 0).  A thread
// whose bytes lie wholly inside the range issues four independent 16-byte loads.
__device__ __forceinline__ uint64_t match_mask64(const uint8_t* map, int64_t b0, int64_t lo, int64_t hi,
                                                 uint8_t want) {
    if (b0 + kBytesPerThread <= lo || b0 >= hi) return 0ull;
    uint64_t nz = 0ull, in = ~0ull;
    if (b0 >= lo && b0 + kBytesPerThread <= hi) {
        const uint4* p = (const uint4*)(map + b0);
        const uint4 w0 = p[0], w1 = p[1], w2 = p[2], w3 = p[3];
        nz = (uint64_t)nonzero_mask16(w0) | ((uint64_t)nonzero_mask16(w1) << 16) |
             ((uint64_t)nonzero_mask16(w2) << 32) | ((uint64_t)nonzero_mask16(w3) << 48);
    } else {
        in = 0ull;
        for (int k = 0; k < kBytesPerThread; ++k) {
            const int64_t b = b0 + k;
            if (b >= lo && b < hi) {
                in |= 1ull << k;
                if (map[b] != 0) nz |= 1ull << k;
            }
        }
    }
    return (want != 0 ? nz : ~nz) & in;
}

// The scans below walk [lo, hi) in tiles of kTileBytes that start at an address multiple of 16, so
// that every thread's bytes can be aligned 16-byte loads whatever lo and the map's own alignment.
__device__ __forceinline__ int64_t aligned_start(const uint8_t* map, int64_t lo) {
    return lo - (int64_t)(((uintptr_t)map + (uint64_t)lo) & 15u);
}

// Counts bytes equal to `want` in map[lo, hi) until at least `limit` are seen
// (early exit at tile granularity).  All threads must call it.
__device__ int64_t count_bytes(const uint8_t* map, int64_t lo, int64_t hi, uint8_t want,
                               int64_t limit, int32_t* sm) {
    int64_t seen = 0;
    for (int64_t t0 = aligned_start(map, lo); t0 < hi && seen < limit; t0 += kTileBytes) {
        const int64_t b0 = t0 + (int64_t)threadIdx.x * kBytesPerThread;
        const int32_t c = __popcll(match_mask64(map, b0, lo, hi, want));
        int32_t tot;
        block_excl_scan<int32_t>(c, &tot, sm);
        seen += tot;
    }
    return seen;
}

// Position (0 .. 63) of the r-th set bit of `bits` (r counted from 0, r < popcount).
__device__ __forceinline__ int select64(uint64_t bits, int r) {
    uint32_t w = (uint32_t)bits;
    int off = 0;
    int c = __popc(w);
    if (r >= c) {
        r -= c;
        w = (uint32_t)(bits >> 32);
        off = 32;
    }
#pragma unroll
    for (int shift = 16; shift >= 1; shift >>= 1) {
        c = __popc(w & ((1u << shift) - 1u));
        if (r >= c) {
            r -= c;
            w >>= shift;
            off += shift;
        }
    }
    return off;
}

// Writes the first `n` positions of map[lo, hi) whose byte equals `want`, ascending, to out[0..n)
// (and the first kIdCache of them to `cache`, when given) WITHOUT touching the map; returns how many
// were found, which is below n only when the range holds fewer.  `first_bits` / `have_first`: the
// mask of the first tile when the caller has requested it early.  All threads must call it.
//
// Two ways to turn a tile's masks into positions.  When a tile contributes many positions every thread
// walks its own mask (64 bytes, up to 64 stores).  When it contributes few -- the usual allocation: a
// handful of blocks out of a map that is mostly free -- those few would all sit in the first threads'
// masks and one lane would walk them alone; then thread p finds the p-th position itself, by a binary
// search over the threads' running counts and a select inside the mask it lands in, and the stores are
// coalesced.
__device__ int64_t collect_bytes(const uint8_t* map, int64_t lo, int64_t hi, uint8_t want, int64_t n,
                                 int64_t* out, int32_t* cache, int32_t* sm, uint64_t first_bits, bool have_first) {
    __shared__ int32_t s_pref[kScanThreads];
    __shared__ uint64_t s_mask[kScanThreads];
    int64_t base = 0;
    bool first = true;
    for (int64_t t0 = aligned_start(map, lo); t0 < hi && base < n; t0 += kTileBytes) {
        const int64_t b0 = t0 + (int64_t)threadIdx.x * kBytesPerThread;
        uint64_t bits = (first && have_first) ? first_bits : match_mask64(map, b0, lo, hi, want);
        first = false;
        const int32_t c = __popcll(bits);
        int32_t tot;
        const int32_t excl = block_excl_scan<int32_t>(c, &tot, sm);
        const int64_t take = min((int64_t)tot, n - base);           // positions this tile contributes
        if (take <= 2 * kScanThreads) {
            s_pref[threadIdx.x] = excl;
            s_mask[threadIdx.x] = bits;
            __syncthreads();
            for (int64_t p = threadIdx.x; p < take; p += kScanThreads) {
                int lo_t = 0, hi_t = kScanThreads - 1;               // last thread whose running count is <= p
                while (lo_t < hi_t) {
                    const int mid = (lo_t + hi_t + 1) >> 1;
                    if (s_pref[mid] <= (int32_t)p) lo_t = mid; else hi_t = mid - 1;
                }
                const int k = select64(s_mask[lo_t], (int)p - s_pref[lo_t]);
                const int64_t id = t0 + (int64_t)lo_t * kBytesPerThread + k;
                out[base + p] = id;
                if (cache != nullptr && base + p < kIdCache) cache[base + p] = (int32_t)id;
            }
            __syncthreads();                                         // the arrays are reused by the next tile
        } else {
            int64_t pos = base + excl;
            while (bits != 0ull && pos < n) {
                const int k = __builtin_ctzll(bits);
                bits &= bits - 1;
                out[pos] = b0 + k;
                if (cache != nullptr && pos < kIdCache) cache[pos] = (int32_t)(b0 + k);
                ++pos;
            }
        }
        base += tot;
    }
    return base < n ? base : n;
}

// ---- allocate_blocks_for_seqs, fused ---------------------------------------------
// One launch: needs -> do they fit -> the lowest free ids -> the table rows.  The first 64 Ki map
// bytes are requested before anything else, so that their trip to memory overlaps the trip for the
// rows' counts; ids are collected first and the map is only marked once the request is known to fit,
// so a refused call changes nothing but the scratch in new_ids.
__global__ __launch_bounds__(kScanThreads) void bm_allocate_kernel(
    int32_t* __restrict__ n_alloc, int32_t* __restrict__ block_table, int64_t max_blocks_per_seq,
    uint8_t* __restrict__ is_free, int64_t num_blocks, const int32_t* __restrict__ seq_ids,
    const int32_t* __restrict__ target_lens, int32_t batch, int32_t block_size,
    int64_t* __restrict__ new_ids, int64_t new_ids_cap, int64_t* __restrict__ result,
    int64_t max_seqs) {
    __shared__ int64_t sm[kScanWaves + 1];
    __shared__ int32_t s_ids[kIdCache];
    __shared__ int s_bad;
    int32_t* sm32 = (int32_t*)sm;
    const int tid = threadIdx.x;
    if (tid == 0) s_bad = 0;
    const uint64_t first_bits = match_mask64(is_free, aligned_start(is_free, 0) + (int64_t)tid * kBytesPerThread, 0,
                                             num_blocks, 1);
    __syncthreads();

    // pass 1: total need, precondition need_i >= 0 and room in the table row.  A thread keeps the row it
    // reads first (row tid: the whole batch when it has at most 1024 rows), so that handing the ids out
    // does not have to fetch the row's sequence id and count a second time.
    int64_t my_need = 0, r_seq = 0, r_have = 0, r_need = 0;
    for (int i = tid; i < batch; i += kScanThreads) {
        const int64_t target = ((int64_t)target_lens[i] + block_size - 1) / block_size;
        const int64_t seq = seq_ids[i];
        if (seq < 0 || seq >= max_seqs) { atomicMax(&s_bad, 2); continue; }
        const int64_t have = n_alloc[seq];
        const int64_t need = target - have;
        if (target > max_blocks_per_seq) atomicMax(&s_bad, 2);   // would not fit the table row
        else if (need < 0) atomicMax(&s_bad, 1);
        my_need += need;
        if (i == tid) { r_seq = seq; r_have = have; r_need = need; }
    }
    int64_t total;
    // with at most one row per thread this is also every row's first position in the list of new ids
    const int64_t r_start = block_excl_scan<int64_t>(my_need, &total, sm);
    __syncthreads();
    if (s_bad) {
        if (tid == 0) { result[0] = total; result[1] = (s_bad == 2) ? MKV_EINVAL : MKV_ELOGIC; result[2] = 0; }
        return;
    }
    if (total == 0) {
        if (tid == 0) { result[0] = 0; result[1] = MKV_OK; result[2] = 0; }
        return;
    }
    if (total > new_ids_cap) {
        if (tid == 0) { result[0] = total; result[1] = MKV_ENOSPC; result[2] = 0; }
        return;
    }
    // pass 2: the lowest `total` free ids (the map is not touched yet)
    const int64_t found = collect_bytes(is_free, 0, num_blocks, 1, total, new_ids, s_ids, sm32, first_bits, true);
    if (found < total) {
        if (tid == 0) { result[0] = total; result[1] = MKV_ENOSPC; result[2] = found; }
        return;
    }
    __threadfence_block();
    __syncthreads();
    // pass 3: they are used from now on
    for (int64_t p = tid; p < total; p += kScanThreads)
        is_free[p < kIdCache ? (int64_t)s_ids[p] : new_ids[p]] = 0;
    // pass 4: hand them to the rows in batch order
    int64_t base = 0;
    for (int i0 = 0; i0 < batch; i0 += kScanThreads) {
        const int i = i0 + tid;
        int64_t need = 0, have = 0, seq = 0;
        if (i0 == 0) {                                       // the rows remembered from pass 1
            if (i < batch) { seq = r_seq; have = r_have; need = r_need; }
        } else if (i < batch) {
            seq = seq_ids[i];
            have = n_alloc[seq];
            need = ((int64_t)target_lens[i] + block_size - 1) / block_size - have;
        }
        int64_t tot = total, start = r_start;
        if (batch > kScanThreads) start = base + block_excl_scan<int64_t>(need, &tot, sm);
        if (i < batch && need > 0) {
            int32_t* dst = block_table + seq * max_blocks_per_seq + have;
            for (int64_t x = 0; x < need; ++x) {
                const int64_t p = start + x;
                dst[x] = p < kIdCache ? s_ids[p] : (int32_t)new_ids[p];
            }
            n_alloc[seq] = (int32_t)(have + need);
        }
        base += tot;
    }
    if (tid == 0) { result[0] = total; result[1] = MKV_OK; result[2] = found; }
}

__global__ __launch_bounds__(kScanThreads) void bm_take_first_free_kernel(
    uint8_t* __restrict__ is_free, int64_t num_blocks, int64_t n, int64_t* __restrict__ ids_out,
    int64_t* __restrict__ result) {
    __shared__ int64_t sm[kScanWaves + 1];
    const int64_t found = collect_bytes(is_free, 0, num_blocks, 1, n, ids_out, nullptr, (int32_t*)sm, 0ull, false);
    if (found < n) {
        if (threadIdx.x == 0) { result[0] = found; result[1] = MKV_ENOSPC; }
        return;
    }
    __threadfence_block();
    __syncthreads();
    for (int64_t p = threadIdx.x; p < n; p += kScanThreads) is_free[ids_out[p]] = 0;
    if (threadIdx.x == 0) { result[0] = n; result[1] = MKV_OK; }
}

template <typename NeedT>
__global__ __launch_bounds__(kScanThreads) void bt_append_kernel(
    int32_t* __restrict__ n_alloc, int32_t* __restrict__ block_table, int64_t max_blocks_per_seq,
    const int64_t* __restrict__ cand, const int32_t* __restrict__ seq_ids,
    const NeedT* __restrict__ needed, int32_t batch, int64_t max_seqs) {
    __shared__ int64_t sm[kScanWaves + 1];
    const int tid = threadIdx.x;
    int64_t base = 0;
    for (int i0 = 0; i0 < batch; i0 += kScanThreads) {
        const int i = i0 + tid;
        int64_t need = 0, have = 0, seq = 0;
        bool ok = false;
        if (i < batch) {
            seq = seq_ids[i];
            ok = seq >= 0 && seq < max_seqs;                   // rows naming no sequence are skipped
            if (ok) have = n_alloc[seq];
            need = (int64_t)needed[i];
            if (need < 0) need = 0;
        }
        int64_t tot;
        const int64_t start = base + block_excl_scan<int64_t>(need, &tot, sm);
        if (ok && need > 0) {
            // never write past the row, and never count more entries than the row holds
            const int64_t fit = max((int64_t)0, min(need, max_blocks_per_seq - have));
            int32_t* dst = block_table + seq * max_blocks_per_seq + have;
            for (int64_t x = 0; x < fit; ++x) dst[x] = (int32_t)cand[start + x];
            n_alloc[seq] = (int32_t)(have + fit);
        }
        base += tot;
    }
}

// One wave per row at a time; lanes stride over the row's live entries.
__global__ __launch_bounds__(kScanThreads) void bt_release_kernel(
    int32_t* __restrict__ n_alloc, const int32_t* __restrict__ block_table,
    int64_t max_blocks_per_seq, const int32_t* __restrict__ seq_ids, int32_t batch,
    uint8_t* __restrict__ is_free, int64_t* __restrict__ freed_total, int64_t max_seqs,
    int64_t num_blocks) {
    __shared__ int64_t sm[kScanWaves + 1];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int64_t mine = 0;
    for (int i = wave; i < batch; i += kScanWaves) {
        const int64_t seq = seq_ids[i];
        if (seq < 0 || seq >= max_seqs) continue;
        const int32_t cnt = (int32_t)min((int64_t)n_alloc[seq], max_blocks_per_seq);   // a row holds no more
        const int32_t* row = block_table + seq * max_blocks_per_seq;
        for (int j = lane; j < cnt; j += 64) {
            const int64_t id = row[j];
            if (id >= 0 && id < num_blocks) is_free[id] = 1;
        }
        if (lane == 0) mine += cnt;
    }
    __syncthreads();                      // every wave has read the counts it needs
    for (int i = wave; i < batch; i += kScanWaves) {
        const int64_t seq = seq_ids[i];
        if (lane == 0 && seq >= 0 && seq < max_seqs) n_alloc[seq] = 0;
    }
    int64_t tot;
    block_excl_scan<int64_t>(mine, &tot, sm);
    if (threadIdx.x == 0 && freed_total) *freed_total = tot;
}

__global__ __launch_bounds__(kScanThreads) void bt_gather_release_kernel(
    int32_t* __restrict__ n_alloc, const int32_t* __restrict__ block_table,
    int64_t max_blocks_per_seq, const int32_t* __restrict__ seq_ids, int32_t batch,
    uint8_t* __restrict__ is_free, int32_t* __restrict__ gathered, int64_t capacity,
    int64_t* __restrict__ result, int64_t max_seqs, int64_t num_blocks) {
    __shared__ int64_t sm[kScanWaves + 1];
    const int tid = threadIdx.x;
    auto count_of = [&](int i) -> int64_t {
        const int64_t seq = seq_ids[i];
        return (seq >= 0 && seq < max_seqs) ? min((int64_t)n_alloc[seq], max_blocks_per_seq) : 0;
    };
    // total first: nothing is modified when it does not fit
    int64_t mine = 0;
    for (int i = tid; i < batch; i += kScanThreads) mine += count_of(i);
    int64_t total;
    block_excl_scan<int64_t>(mine, &total, sm);
    __syncthreads();
    if (total > capacity) {
        if (tid == 0) { result[0] = total; result[1] = MKV_ENOSPC; }
        return;
    }
    // Rows are copied one wave at a time; the start offset of row i is the sum of
    // the counts of the rows before it (seq-major, logical block order).
    int64_t base = 0;
    for (int i0 = 0; i0 < batch; i0 += kScanThreads) {
        const int i = i0 + tid;
        const int64_t cnt = (i < batch) ? count_of(i) : 0;
        int64_t tot;
        const int64_t start = base + block_excl_scan<int64_t>(cnt, &tot, sm);
        // the thread that owns row i copies it (rows are short: ceil(len/B) entries)
        if (i < batch && cnt > 0) {
            const int64_t seq = seq_ids[i];
            const int32_t* row = block_table + seq * max_blocks_per_seq;
            for (int64_t x = 0; x < cnt; ++x) {
                const int32_t id = row[x];
                gathered[start + x] = id;
                if (id >= 0 && id < num_blocks) is_free[id] = 1;
            }
        }
        base += tot;
    }
    __syncthreads();
    for (int i = tid; i < batch; i += kScanThreads) {
        const int64_t seq = seq_ids[i];
        if (seq >= 0 && seq < max_seqs) n_alloc[seq] = 0;
    }
    if (tid == 0) { result[0] = total; result[1] = MKV_OK; }
}

__global__ __launch_bounds__(kScanThreads) void bm_count_live_kernel(
    const uint8_t* __restrict__ is_free, int64_t lo, int64_t hi, int64_t* __restrict__ result) {
    __shared__ int64_t sm[kScanWaves + 1];
    const int64_t live = count_bytes(is_free, lo, hi, 0, INT64_MAX, (int32_t*)sm);
    if (threadIdx.x == 0) *result = live;
}

// ---- shrink planning ---------------------------------------------------------------
// Live ids >= new_n, ascending, move to the lowest free ids < new_n.  Both lists are collected without
// touching the map; only a plan that fits is applied (sources become free, destinations used, remap
// holds the new id of every moved block and the identity elsewhere).
__global__ __launch_bounds__(kScanThreads) void pool_plan_shrink_kernel(
    uint8_t* __restrict__ is_free, int64_t num_blocks, int64_t new_n, int64_t* __restrict__ src,
    int64_t* __restrict__ dst, int64_t cap, int32_t* __restrict__ remap,
    int64_t* __restrict__ result) {
    __shared__ int64_t sm[kScanWaves + 1];
    int32_t* sm32 = (int32_t*)sm;
    const int tid = threadIdx.x;
    // identity first: independent stores that drain while the map is read (four ids per store where the
    // array's alignment allows)
    if ((((uintptr_t)remap) & 15u) == 0) {
        int4* r4 = (int4*)remap;
        for (int64_t q = tid; q < num_blocks / 4; q += kScanThreads) {
            const int32_t b = (int32_t)(4 * q);
            r4[q] = make_int4(b, b + 1, b + 2, b + 3);
        }
        for (int64_t b = (num_blocks / 4) * 4 + tid; b < num_blocks; b += kScanThreads) remap[b] = (int32_t)b;
    } else {
        for (int64_t b = tid; b < num_blocks; b += kScanThreads) remap[b] = (int32_t)b;
    }
    // live blocks above the cut: all of them, as many as the lists hold (one more than `cap` says "too many")
    const int64_t moves = collect_bytes(is_free, new_n, num_blocks, 0, cap, src, nullptr, sm32, 0ull, false);
    const int64_t live_above = moves < cap ? moves : count_bytes(is_free, new_n, num_blocks, 0, INT64_MAX, sm32);
    const int64_t free_below = collect_bytes(is_free, 0, new_n, 1, live_above <= cap ? live_above : 0, dst, nullptr,
                                             sm32, 0ull, false);
    if (live_above > cap || free_below < live_above) {
        const int64_t fb = live_above > cap ? count_bytes(is_free, 0, new_n, 1, live_above, sm32) : free_below;
        if (tid == 0) { result[0] = live_above; result[1] = MKV_ENOSPC; result[2] = fb; }
        return;
    }
    __threadfence_block();
    __syncthreads();
    // four moves per thread and round, every load ahead of the stores (the lists were written by other
    // threads: each round is a trip to the L2)
    for (int64_t k0 = tid; k0 < moves; k0 += 4 * kScanThreads) {
        int64_t s_id[4], d_id[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int64_t k = k0 + (int64_t)u * kScanThreads;
            s_id[u] = k < moves ? src[k] : -1;
            d_id[u] = k < moves ? dst[k] : -1;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (s_id[u] >= 0) {
                is_free[s_id[u]] = 1;
                is_free[d_id[u]] = 0;
                remap[s_id[u]] = (int32_t)d_id[u];
            }
    }
    if (tid == 0) { result[0] = moves; result[1] = MKV_OK; result[2] = free_below; }
}

// ---- shrink planning over many workgroups (large maps) -----------------------------------
// One workgroup cannot enumerate ten thousand positions of a 100 k map in much under 30 us: the
// enumeration and its scattered stores are one CU's work.  For large maps the plan is three launches
// of one workgroup per 4096 map bytes:
//   count  every tile counts its free bytes below the cut and its live bytes above it, and writes
//          the identity into its part of remap (the counts travel in remap[0 .. 2T), which no move
//          ever writes: moved ids are >= new_n >= 2T, the host checks);
//   place  every workgroup sums the counts of the tiles before it (T is small), decides whether the
//          plan fits (all workgroups see the same totals) and, if it does, writes its tile's live ids
//          above the cut into src and its free ids below the cut, up to the number needed, into dst;
//   apply  restores the identity in remap[0 .. 2T) and applies the moves to the map and to remap.
// Nothing but scratch (src, dst, remap) is written unless the plan fits.
static constexpr int kPlanThreads = 256;
static constexpr int kPlanTileBytes = kPlanThreads * 16;

__device__ __forceinline__ uint32_t plan_mask16(const uint8_t* map, int64_t b0, int64_t lo, int64_t hi, uint8_t want) {
    if (b0 + 16 <= lo || b0 >= hi) return 0u;
    uint32_t nz = 0u, in = 0xffffu;
    if (b0 >= lo && b0 + 16 <= hi && (((uintptr_t)(map + b0)) & 15u) == 0) {
        nz = nonzero_mask16(*(const uint4*)(map + b0));
    } else {
        in = 0u;
        for (int k = 0; k < 16; ++k) {
            const int64_t b = b0 + k;
            if (b >= lo && b < hi) {
                in |= 1u << k;
                if (map[b] != 0) nz |= 1u << k;
            }
        }
    }
    return (want != 0 ? nz : ~nz) & in;
}

// sum over the 256 threads of a plan workgroup; all threads call it
__device__ __forceinline__ int32_t plan_block_sum(int32_t v, int32_t* sm /* [4] */) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    return sm[0] + sm[1] + sm[2] + sm[3];
}

__global__ __launch_bounds__(kPlanThreads) void plan_count_kernel(const uint8_t* __restrict__ is_free, int64_t num_blocks,
                                                                  int64_t new_n, int32_t* __restrict__ remap, int32_t tiles) {
    __shared__ int32_t sm[4];
    const int64_t b0 = (int64_t)blockIdx.x * kPlanTileBytes + (int64_t)threadIdx.x * 16;
    const int32_t free_below = __popc(plan_mask16(is_free, b0, 0, new_n, 1));
    const int32_t live_above = __popc(plan_mask16(is_free, b0, new_n, num_blocks, 0));
    for (int k = 0; k < 16; ++k) {
        const int64_t b = b0 + k;
        if (b < num_blocks && b >= 2 * (int64_t)tiles) remap[b] = (int32_t)b;
    }
    const int32_t f = plan_block_sum(free_below, sm);
    const int32_t l = plan_block_sum(live_above, sm);
    if (threadIdx.x == 0) {
        remap[2 * blockIdx.x] = f;
        remap[2 * blockIdx.x + 1] = l;
    }
}

__global__ __launch_bounds__(kPlanThreads) void plan_place_kernel(const uint8_t* __restrict__ is_free, int64_t num_blocks,
                                                                  int64_t new_n, int64_t* __restrict__ src,
                                                                  int64_t* __restrict__ dst, int64_t cap,
                                                                  const int32_t* __restrict__ remap, int32_t tiles,
                                                                  int64_t* __restrict__ result) {
    __shared__ int32_t sm[4];
    __shared__ int32_t s_scan[kPlanThreads / 64 + 1];
    const int tid = threadIdx.x;
    // totals and this tile's offsets from the per-tile counts
    int32_t f_before = 0, l_before = 0, f_all = 0, l_all = 0;
    for (int t = tid; t < tiles; t += kPlanThreads) {
        const int32_t f = remap[2 * t], l = remap[2 * t + 1];
        f_all += f;
        l_all += l;
        if (t < (int)blockIdx.x) { f_before += f; l_before += l; }
    }
    f_before = plan_block_sum(f_before, sm);
    l_before = plan_block_sum(l_before, sm);
    f_all = plan_block_sum(f_all, sm);
    l_all = plan_block_sum(l_all, sm);
    const int64_t moves = l_all;
    const bool fits = moves <= cap && (int64_t)f_all >= moves;
    if (blockIdx.x == 0 && tid == 0) {
        result[0] = moves;
        result[1] = fits ? MKV_OK : MKV_ENOSPC;
        result[2] = f_all < moves ? f_all : (fits ? moves : f_all);
    }
    if (!fits) return;
    const int64_t b0 = (int64_t)blockIdx.x * kPlanTileBytes + (int64_t)tid * 16;
    const int lane = tid & 63, wave = tid >> 6;
    // two ordered compactions of this tile: live above the cut -> src, free below the cut -> dst
    for (int which = 0; which < 2; ++which) {
        const uint32_t bits = which == 0 ? plan_mask16(is_free, b0, new_n, num_blocks, 0)
                                         : plan_mask16(is_free, b0, 0, new_n, 1);
        const int32_t c = __popc(bits);
        int32_t inc = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int32_t t = __shfl_up(inc, d);
            if (lane >= d) inc += t;
        }
        __syncthreads();
        if (lane == 63) s_scan[wave] = inc;
        __syncthreads();
        int32_t wave_off = 0;
        for (int w = 0; w < wave; ++w) wave_off += s_scan[w];
        int64_t pos = (int64_t)(which == 0 ? l_before : f_before) + wave_off + inc - c;
        int64_t* out = which == 0 ? src : dst;
        if (c != 0 && pos < moves) {
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                if ((bits >> k) & 1u) {
                    if (pos < moves) out[pos] = b0 + k;
                    ++pos;
                }
            }
        }
    }
}

__global__ __launch_bounds__(kPlanThreads) void plan_apply_kernel(uint8_t* __restrict__ is_free, const int64_t* __restrict__ src,
                                                                  const int64_t* __restrict__ dst, int32_t* __restrict__ remap,
                                                                  int32_t tiles, const int64_t* __restrict__ result) {
    if (blockIdx.x == 0)                              // the counts have been read: their slots become identity again
        for (int b = threadIdx.x; b < 2 * tiles; b += kPlanThreads) remap[b] = b;
    if (result[1] != MKV_OK) return;
    const int64_t moves = result[0];
    for (int64_t k = (int64_t)blockIdx.x * kPlanThreads + threadIdx.x; k < moves; k += (int64_t)gridDim.x * kPlanThreads) {
        const int64_t s_id = src[k], d_id = dst[k];
        is_free[s_id] = 1;
        is_free[d_id] = 0;
        remap[s_id] = (int32_t)d_id;
    }
}

__global__ __launch_bounds__(256) void bt_remap_kernel(int32_t* __restrict__ block_table,
                                                       int64_t max_blocks_per_seq,
                                                       const int32_t* __restrict__ n_alloc,
                                                       int64_t max_seqs,
                                                       const int32_t* __restrict__ remap,
                                                       int64_t num_blocks) {
    for (int64_t row = blockIdx.x; row < max_seqs; row += gridDim.x) {
        const int32_t cnt = (int32_t)min((int64_t)n_alloc[row], max_blocks_per_seq);
        int32_t* r = block_table + row * max_blocks_per_seq;
        for (int j = threadIdx.x; j < cnt; j += blockDim.x) {
            const int32_t id = r[j];
            if (id >= 0 && id < num_blocks) {
                const int32_t to = remap[id];
                if (to != id) r[j] = to;
            }
        }
    }
}

}  // namespace mkv

extern "C" {

int mkv_bm_allocate(int32_t* num_seq_allocated_blocks, int64_t max_seqs, int32_t* block_table,
                    int64_t max_blocks_per_seq, uint8_t* is_block_free, int64_t num_blocks,
                    const int32_t* seq_ids, const int32_t* target_lens, int32_t batch,
                    int32_t block_size, int64_t* new_ids, int64_t new_ids_cap, int64_t* result,
                    void* stream) {
    MKV_REQUIRE(num_seq_allocated_blocks && block_table && is_block_free && result, "NULL argument");
    MKV_REQUIRE(batch >= 0 && block_size > 0 && num_blocks >= 0 && max_blocks_per_seq > 0, "bad sizes");
    MKV_REQUIRE(batch == 0 || (seq_ids && target_lens), "NULL seq_ids/target_lens");
    MKV_REQUIRE(new_ids || new_ids_cap == 0, "new_ids is NULL");
    hipLaunchKernelGGL(mkv::bm_allocate_kernel, dim3(1), dim3(mkv::kScanThreads), 0,
                       (hipStream_t)stream, num_seq_allocated_blocks, block_table,
                       max_blocks_per_seq, is_block_free, num_blocks, seq_ids, target_lens, batch,
                       block_size, new_ids, new_ids_cap, result, max_seqs);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_bm_take_first_free(uint8_t* is_block_free, int64_t num_blocks, int64_t n,
                           int64_t* ids_out, int64_t* result, void* stream) {
    MKV_REQUIRE(is_block_free && result, "NULL argument");
    MKV_REQUIRE(n >= 0 && num_blocks >= 0, "bad sizes");
    MKV_REQUIRE(ids_out || n == 0, "ids_out is NULL");
    hipLaunchKernelGGL(mkv::bm_take_first_free_kernel, dim3(1), dim3(mkv::kScanThreads), 0,
                       (hipStream_t)stream, is_block_free, num_blocks, n, ids_out, result);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_bt_append(int32_t* num_seq_allocated_blocks, int64_t max_seqs, int32_t* block_table,
                  int64_t max_blocks_per_seq, const int64_t* candidate_blocks,
                  const int32_t* seq_ids, const void* block_needed, int32_t needed_is_i64,
                  int32_t batch, void* stream) {
    MKV_REQUIRE(batch >= 0, "batch must be >= 0");
    if (batch == 0) return MKV_OK;
    MKV_REQUIRE(num_seq_allocated_blocks && block_table && seq_ids && block_needed, "NULL argument");
    if (needed_is_i64) {
        hipLaunchKernelGGL(mkv::bt_append_kernel<int64_t>, dim3(1), dim3(mkv::kScanThreads), 0,
                           (hipStream_t)stream, num_seq_allocated_blocks, block_table,
                           max_blocks_per_seq, candidate_blocks, seq_ids,
                           (const int64_t*)block_needed, batch, max_seqs);
    } else {
        hipLaunchKernelGGL(mkv::bt_append_kernel<int32_t>, dim3(1), dim3(mkv::kScanThreads), 0,
                           (hipStream_t)stream, num_seq_allocated_blocks, block_table,
                           max_blocks_per_seq, candidate_blocks, seq_ids,
                           (const int32_t*)block_needed, batch, max_seqs);
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_bt_release(int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                   const int32_t* block_table, int64_t max_blocks_per_seq,
                   const int32_t* seq_ids, int32_t batch, uint8_t* is_block_free,
                   int64_t num_blocks, int64_t* freed_total, void* stream) {
    MKV_REQUIRE(batch >= 0, "batch must be >= 0");
    MKV_REQUIRE(num_seq_allocated_blocks && block_table && is_block_free, "NULL argument");
    MKV_REQUIRE(batch == 0 || seq_ids, "seq_ids is NULL");
    hipLaunchKernelGGL(mkv::bt_release_kernel, dim3(1), dim3(mkv::kScanThreads), 0,
                       (hipStream_t)stream, num_seq_allocated_blocks, block_table,
                       max_blocks_per_seq, seq_ids, batch, is_block_free, freed_total, max_seqs,
                       num_blocks);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_bt_gather_release(int32_t* num_seq_allocated_blocks, int64_t max_seqs,
                          const int32_t* block_table, int64_t max_blocks_per_seq,
                          const int32_t* seq_ids, int32_t batch, uint8_t* is_block_free,
                          int64_t num_blocks, int32_t* gathered, int64_t capacity,
                          int64_t* result, void* stream) {
    MKV_REQUIRE(batch >= 0 && capacity >= 0, "bad sizes");
    MKV_REQUIRE(num_seq_allocated_blocks && block_table && is_block_free && result, "NULL argument");
    MKV_REQUIRE(batch == 0 || seq_ids, "seq_ids is NULL");
    MKV_REQUIRE(gathered || capacity == 0, "gathered is NULL");
    hipLaunchKernelGGL(mkv::bt_gather_release_kernel, dim3(1), dim3(mkv::kScanThreads), 0,
                       (hipStream_t)stream, num_seq_allocated_blocks, block_table,
                       max_blocks_per_seq, seq_ids, batch, is_block_free, gathered, capacity,
                       result, max_seqs, num_blocks);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_bm_count_live(const uint8_t* is_block_free, int64_t lo, int64_t hi, int64_t* result,
                      void* stream) {
    MKV_REQUIRE(is_block_free && result, "NULL argument");
    MKV_REQUIRE(0 <= lo && lo <= hi, "need 0 <= lo <= hi");
    hipLaunchKernelGGL(mkv::bm_count_live_kernel, dim3(1), dim3(mkv::kScanThreads), 0,
                       (hipStream_t)stream, is_block_free, lo, hi, result);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_pool_plan_shrink(uint8_t* is_block_free, int64_t num_blocks, int64_t new_num_blocks,
                         int64_t* src, int64_t* dst, int64_t cap, int32_t* remap,
                         int64_t* result, void* stream) {
    MKV_REQUIRE(is_block_free && remap && result, "NULL argument");
    MKV_REQUIRE(0 <= new_num_blocks && new_num_blocks <= num_blocks,
                "need 0 <= new_num_blocks (%lld) <= num_blocks (%lld)", (long long)new_num_blocks,
                (long long)num_blocks);
    MKV_REQUIRE(num_blocks <= INT32_MAX, "block ids must fit int32");
    MKV_REQUIRE((src && dst) || cap == 0, "src/dst are NULL");
    // large maps: one workgroup per 4096 bytes in three launches (the per-tile counts travel in the first
    // 2 * tiles entries of remap, which must lie below the cut); small ones: one workgroup does it all
    const int64_t tiles = (num_blocks + mkv::kPlanTileBytes - 1) / mkv::kPlanTileBytes;
    hipStream_t s = (hipStream_t)stream;
    if (num_blocks >= 32768 && 2 * tiles <= new_num_blocks && tiles <= 65535 && cap > 0) {
        hipLaunchKernelGGL(mkv::plan_count_kernel, dim3((unsigned)tiles), dim3(mkv::kPlanThreads), 0, s, is_block_free,
                           num_blocks, new_num_blocks, remap, (int32_t)tiles);
        hipLaunchKernelGGL(mkv::plan_place_kernel, dim3((unsigned)tiles), dim3(mkv::kPlanThreads), 0, s, is_block_free,
                           num_blocks, new_num_blocks, src, dst, cap, remap, (int32_t)tiles, result);
        const unsigned apply_grid = (unsigned)std::min<int64_t>(tiles, 2 * (int64_t)mkv::num_cus());
        hipLaunchKernelGGL(mkv::plan_apply_kernel, dim3(apply_grid), dim3(mkv::kPlanThreads), 0, s, is_block_free, src, dst,
                           remap, (int32_t)tiles, result);
    } else {
        hipLaunchKernelGGL(mkv::pool_plan_shrink_kernel, dim3(1), dim3(mkv::kScanThreads), 0, s, is_block_free, num_blocks,
                           new_num_blocks, src, dst, cap, remap, result);
    }
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_bt_remap(int32_t* block_table, int64_t max_blocks_per_seq,
                 const int32_t* num_seq_allocated_blocks, int64_t max_seqs, const int32_t* remap,
                 int64_t num_blocks, void* stream) {
    MKV_REQUIRE(block_table && num_seq_allocated_blocks && remap, "NULL argument");
    MKV_REQUIRE(max_seqs >= 0 && max_blocks_per_seq > 0, "bad sizes");
    if (max_seqs == 0) return MKV_OK;
    const unsigned grid = (unsigned)(max_seqs < 65535 ? max_seqs : 65535);
    hipLaunchKernelGGL(mkv::bt_remap_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream,
                       block_table, max_blocks_per_seq, num_seq_allocated_blocks, max_seqs, remap,
                       num_blocks);
    MKV_HIP(hipGetLastError());
    return MKV_OK;
}

int mkv_pool_carve_segment(uint64_t layer_base, uint64_t org_bytes, uint64_t quant_bytes,
                           int32_t num_layers, int32_t num_kv_heads, int32_t block_size,
                           int32_t head_dim, uint64_t* k_start, int64_t* seg_blocks,
                           uint64_t* v_start) {
    MKV_REQUIRE(k_start && seg_blocks && v_start, "output pointers are NULL");
    MKV_REQUIRE(num_layers > 0 && num_kv_heads > 0 && block_size > 0 && head_dim > 0, "bad dims");
    const uint64_t layer_end = layer_base + quant_bytes;
    const uint64_t start = (layer_end + 255) & ~(uint64_t)255;
    const uint64_t used = start - layer_base;
    const uint64_t kv_slot = 2ull * num_layers * num_kv_heads * head_dim * 2ull;
    const uint64_t kv_block = kv_slot * block_size;
    const uint64_t avail = org_bytes > used ? org_bytes - used : 0;
    const uint64_t S = avail / kv_block;
    if (S == 0) {
        mkv::set_error("No space available for new KV cache blocks");
        return MKV_ENOSPC;
    }
    *k_start = start;
    *seg_blocks = (int64_t)S;
    *v_start = start + S * (kv_block / 2);
    return MKV_OK;
}

}  // extern "C"
