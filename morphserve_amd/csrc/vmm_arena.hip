// Pool backing through HIP virtual memory: one address range reserved once, physical
// chunks mapped at its end when the pool grows and unmapped when it shrinks.  The pool
// stays ONE contiguous [num_blocks, L, Hkv, B, D] tensor at a fixed address, so block ids
// never need the segment arithmetic and growing never copies.
//
// Memory groups.  On an MI355X the 288 GiB of HBM behave as three groups of 96 GiB of physical
// addresses: two streams of stores run about a fifth faster when they go to different groups than
// when they share one, a copy kernel whose K and V destinations share a group runs at 65 % of peak
// against 78 % when they do not, and a gather over a pool runs fastest when the pool touches at most
// two groups.  Which group a chunk lies in cannot be asked for, but it can be measured: the rate of a
// store-only kernel that fills the chunk and a reference chunk side by side.  mkv_arena_pair_grow uses
// that to give the K arena of a pool chunks of one group and the V arena chunks of another.  The
// measurement is relative (a candidate against two references, or against the candidates' own spread),
// never an absolute rate, so a device without such groups simply yields one group and the plain order.
#include "common.h"

#include <algorithm>
#include <chrono>
#include <vector>

struct mkv_arena {
    char* base = nullptr;
    uint64_t reserved = 0;
    uint64_t chunk = 0;
    int device = 0;
    std::vector<hipMemGenericAllocationHandle_t> chunks;     // chunk i backs [i * chunk, (i + 1) * chunk)
    // one spare chunk of this arena's memory group, mapped at ref_va and never part of the pool: what
    // later growth measures its candidates against (mkv_arena_pair_grow); none until a pair call made one
    hipMemGenericAllocationHandle_t ref = {};
    char* ref_va = nullptr;
    bool has_ref = false;
};

namespace mkv {

static int arena_map_one(mkv_arena* a) {
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = a->device;
    hipMemGenericAllocationHandle_t h;
    MKV_HIP(hipMemCreate(&h, a->chunk, &prop, 0));
    char* at = a->base + a->chunks.size() * a->chunk;
    hipError_t e = hipMemMap(at, a->chunk, 0, h, 0);
    if (e == hipSuccess) {
        hipMemAccessDesc acc = {};
        acc.location = prop.location;
        acc.flags = hipMemAccessFlagsProtReadWrite;
        e = hipMemSetAccess(at, a->chunk, &acc, 1);
        if (e != hipSuccess) (void)hipMemUnmap(at, a->chunk);
    }
    if (e != hipSuccess) {
        (void)hipMemRelease(h);
        return ::mkv::hip_fail(e, "hipMemMap / hipMemSetAccess of a fresh chunk at the end of the arena");
    }
    a->chunks.push_back(h);
    return MKV_OK;
}

static int arena_map_handle(mkv_arena* a, hipMemGenericAllocationHandle_t h) {
    char* at = a->base + a->chunks.size() * a->chunk;
    MKV_HIP(hipMemMap(at, a->chunk, 0, h, 0));
    hipMemAccessDesc acc = {};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = a->device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    hipError_t e = hipMemSetAccess(at, a->chunk, &acc, 1);
    if (e != hipSuccess) {
        (void)hipMemUnmap(at, a->chunk);
        return ::mkv::hip_fail(e, "hipMemMap / hipMemSetAccess of a handed-over chunk at the end of the arena");
    }
    a->chunks.push_back(h);
    return MKV_OK;
}

static int arena_unmap_one(mkv_arena* a) {
    char* at = a->base + (a->chunks.size() - 1) * a->chunk;
    MKV_HIP(hipMemUnmap(at, a->chunk));
    MKV_HIP(hipMemRelease(a->chunks.back()));
    a->chunks.pop_back();
    return MKV_OK;
}

}  // namespace mkv

extern "C" {

int mkv_arena_create(uint64_t reserve_bytes, uint64_t chunk_bytes, mkv_arena** out) {
    MKV_REQUIRE(out != nullptr, "out is NULL");
    *out = nullptr;
    MKV_REQUIRE(chunk_bytes > 0 && reserve_bytes >= chunk_bytes && reserve_bytes % chunk_bytes == 0,
                "reserve_bytes must be a positive multiple of chunk_bytes");
    // Chunks are mapped back to back.  A 574.5 MiB chunk mapped at an odd multiple of its size has been
    // refused by hipMemSetAccess ("invalid argument", the 174th chunk of a range, where the physical
    // memory crosses from one 96 GiB group of the device into the next); multiples of 2 MiB never were.
    MKV_REQUIRE(chunk_bytes <= (2ull << 20) || chunk_bytes % (2ull << 20) == 0,
                "chunk_bytes above 2 MiB must be a multiple of 2 MiB (got %llu)", (unsigned long long)chunk_bytes);
    int dev = 0;
    MKV_HIP(hipGetDevice(&dev));
    int vmm = 0;
    MKV_HIP(hipDeviceGetAttribute(&vmm, hipDeviceAttributeVirtualMemoryManagementSupported, dev));
    MKV_REQUIRE(vmm != 0, "this device does not support virtual memory management");
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = dev;
    size_t gran = 0;
    MKV_HIP(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended));
    MKV_REQUIRE(gran > 0 && chunk_bytes % gran == 0, "chunk_bytes must be a multiple of the allocation granularity (%zu)", gran);
    void* base = nullptr;
    MKV_HIP(hipMemAddressReserve(&base, reserve_bytes, 0, nullptr, 0));
    mkv_arena* a = new mkv_arena();
    a->base = (char*)base;
    a->reserved = reserve_bytes;
    a->chunk = chunk_bytes;
    a->device = dev;
    *out = a;
    return MKV_OK;
}

int mkv_arena_info(const mkv_arena* arena, void** base, uint64_t* reserved_bytes, uint64_t* chunk_bytes,
                   uint64_t* mapped_bytes) {
    MKV_REQUIRE(arena != nullptr, "arena is NULL");
    if (base) *base = arena->base;
    if (reserved_bytes) *reserved_bytes = arena->reserved;
    if (chunk_bytes) *chunk_bytes = arena->chunk;
    if (mapped_bytes) *mapped_bytes = arena->chunks.size() * arena->chunk;
    return MKV_OK;
}

int mkv_arena_resize(mkv_arena* arena, uint64_t mapped_bytes) {
    MKV_REQUIRE(arena != nullptr, "arena is NULL");
    MKV_REQUIRE(mapped_bytes % arena->chunk == 0 && mapped_bytes <= arena->reserved,
                "mapped_bytes must be a multiple of the chunk size and at most the reservation");
    const size_t want = mapped_bytes / arena->chunk;
    const size_t had = arena->chunks.size();
    while (arena->chunks.size() < want) {
        int rc = mkv::arena_map_one(arena);
        if (rc) {                                  // out of memory: give back what this call mapped
            while (arena->chunks.size() > had) (void)mkv::arena_unmap_one(arena);
            return rc == MKV_EHIP ? MKV_ENOSPC : rc;
        }
    }
    while (arena->chunks.size() > want) {
        int rc = mkv::arena_unmap_one(arena);
        if (rc) return rc;
    }
    return MKV_OK;
}

int mkv_arena_move_tail(mkv_arena* from, mkv_arena* to, uint64_t bytes) {
    MKV_REQUIRE(from != nullptr && to != nullptr && from != to, "two different arenas are needed");
    MKV_REQUIRE(from->chunk == to->chunk && from->device == to->device,
                "both arenas must have the same chunk size and device");
    MKV_REQUIRE(bytes % from->chunk == 0, "bytes must be a multiple of the chunk size");
    const size_t n = bytes / from->chunk;
    MKV_REQUIRE(n <= from->chunks.size(), "the source arena has fewer mapped bytes than that");
    MKV_REQUIRE((to->chunks.size() + n) * to->chunk <= to->reserved, "the destination's reservation is too small");
    for (size_t i = 0; i < n; ++i) {
        hipMemGenericAllocationHandle_t h = from->chunks.back();
        char* at = from->base + (from->chunks.size() - 1) * from->chunk;
        MKV_HIP(hipMemUnmap(at, from->chunk));
        from->chunks.pop_back();
        int rc = mkv::arena_map_handle(to, h);
        if (rc) {                                  // put the chunk back where it was; earlier chunks stay moved
            if (mkv::arena_map_handle(from, h) != MKV_OK) (void)hipMemRelease(h);
            return rc;
        }
    }
    return MKV_OK;
}

int mkv_arena_destroy(mkv_arena* arena) {
    if (arena == nullptr) return MKV_OK;
    int rc = MKV_OK;
    if (arena->has_ref) {
        (void)hipMemUnmap(arena->ref_va, arena->chunk);
        (void)hipMemRelease(arena->ref);
        arena->has_ref = false;
    }
    if (arena->ref_va) {
        (void)hipMemAddressFree(arena->ref_va, arena->chunk);
        arena->ref_va = nullptr;
    }
    while (!arena->chunks.empty()) {
        int r = mkv::arena_unmap_one(arena);
        if (r) {
            rc = r;
            break;
        }
    }
    if (rc == MKV_OK) {
        hipError_t e = hipMemAddressFree(arena->base, arena->reserved);
        if (e != hipSuccess) rc = MKV_EHIP;
    }
    delete arena;
    return rc;
}

}  // extern "C"

// ---- memory-group aware growth of a K / V arena pair ---------------------------------------------
namespace mkv {

typedef unsigned int pv4u __attribute__((ext_vector_type(4)));

// Two store streams side by side: 16 KiB items alternate between the two destinations, a persistent
// grid strides over them, four 16-byte non-temporal stores per thread and item.  Writes zeros.
__global__ __launch_bounds__(256) void group_probe_kernel(pv4u* __restrict__ a, pv4u* __restrict__ b, int64_t items_each) {
    const pv4u z = {0u, 0u, 0u, 0u};
    for (int64_t w = blockIdx.x; w < 2 * items_each; w += gridDim.x) {
        pv4u* dp = ((w & 1) ? b : a) + (w >> 1) * 1024 + threadIdx.x;
#pragma unroll
        for (int u = 0; u < 4; ++u) __builtin_nontemporal_store(z, dp + u * 256);
    }
}

struct Candidate {
    hipMemGenericAllocationHandle_t h;
    char* va;
    int group;        // 0 = the K reference's group, 1 = the V reference's, 2 = neither, -1 = not measured
    bool taken;
};

struct PairGrow {
    mkv_arena *k, *v;
    uint64_t chunk, probe_bytes;
    hipStream_t stream;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    std::vector<Candidate> cand;
    std::vector<std::pair<char*, uint64_t>> windows;      // staging address ranges
    int probes = 0;
    double probe_ms = 0.0;

    // GB/s of the two-stream fill into [a, a + probe_bytes) and [b, b + probe_bytes): best of two after a warm-up
    int rate(char* a, char* b, double* out) {
        const int64_t items = (int64_t)(probe_bytes / 16384);
        const unsigned grid = (unsigned)std::min<int64_t>(2 * items, (int64_t)num_cus() * 16);
        float best = 1e30f;
        for (int rep = 0; rep < 3; ++rep) {
            MKV_HIP(hipEventRecord(e0, stream));
            hipLaunchKernelGGL(group_probe_kernel, dim3(grid), dim3(256), 0, stream, (pv4u*)a, (pv4u*)b, items);
            MKV_HIP(hipEventRecord(e1, stream));
            MKV_HIP(hipEventSynchronize(e1));
            float ms = 0.f;
            MKV_HIP(hipEventElapsedTime(&ms, e0, e1));
            if (rep > 0) best = std::min(best, ms);
            probe_ms += ms;
        }
        MKV_HIP(hipGetLastError());
        ++probes;
        *out = 2.0 * (double)probe_bytes / (double)best / 1e6;
        return MKV_OK;
    }

    // create `n` more chunks and map them into a staging window; stops quietly when the device is full
    int more(size_t n, size_t* got) {
        *got = 0;
        if (n == 0) return MKV_OK;
        hipMemAllocationProp prop = {};
        prop.type = hipMemAllocationTypePinned;
        prop.location.type = hipMemLocationTypeDevice;
        prop.location.id = k->device;
        void* win = nullptr;
        MKV_HIP(hipMemAddressReserve(&win, n * chunk, 0, nullptr, 0));
        windows.push_back({(char*)win, n * chunk});
        hipMemAccessDesc acc = {};
        acc.location = prop.location;
        acc.flags = hipMemAccessFlagsProtReadWrite;
        for (size_t i = 0; i < n; ++i) {
            hipMemGenericAllocationHandle_t h;
            if (hipMemCreate(&h, chunk, &prop, 0) != hipSuccess) {
                (void)hipGetLastError();
                break;                                      // out of device memory: work with what there is
            }
            char* at = (char*)win + i * chunk;
            const char* what = "hipMemMap";
            hipError_t e = hipMemMap(at, chunk, 0, h, 0);
            if (e == hipSuccess) {
                what = "hipMemSetAccess";
                e = hipMemSetAccess(at, chunk, &acc, 1);
                if (e != hipSuccess) (void)hipMemUnmap(at, chunk);
            }
            if (e != hipSuccess) {
                (void)hipMemRelease(h);
                set_error("HIP error %d (%s) in %s of candidate %zu of %zu in the staging window (chunks of %llu bytes)",
                          (int)e, hipGetErrorString(e), what, i, n, (unsigned long long)chunk);
                return MKV_EHIP;
            }
            cand.push_back({h, at, -1, false});
            ++*got;
        }
        return MKV_OK;
    }

    int unstage(Candidate& c) { MKV_HIP(hipMemUnmap(c.va, chunk)); c.va = nullptr; return MKV_OK; }

    void drop_everything() {
        for (auto& c : cand) {
            if (c.va) (void)hipMemUnmap(c.va, chunk);
            if (!c.taken) (void)hipMemRelease(c.h);
        }
        cand.clear();
        for (auto& w : windows) (void)hipMemAddressFree(w.first, w.second);
        windows.clear();
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        e0 = e1 = nullptr;
    }
};

// Split rates measured against one anchor into "same group as the anchor" (slow) and "another group"
// (fast).  On an MI355X a pair of chunks of one group fills at 4.7-5.8 TB/s and a pair of two groups at
// 6.0-7.1 TB/s: the two kinds do not overlap, but with a few hundred chunks the gap between them can be as
// narrow as 6 %, no wider than steps inside a kind are with few chunks.  So the cut is the two-class split
// of the sorted rates with the largest variance between the classes, and it counts only when the class
// means lie at least 15 % apart (two kinds: 28 %; one kind cut in two: 10 %); otherwise all rates are of one
// kind, and the anchor's own rate (its two halves filled side by side: one group by construction) says which.
static void split_by_rate(const std::vector<double>& rate, double self_rate, std::vector<char>* same) {
    const size_t n = rate.size();
    same->assign(n, 1);
    if (n == 0) return;
    std::vector<double> sorted(rate);
    std::sort(sorted.begin(), sorted.end());
    double total = 0.0;
    for (double r : sorted) total += r;
    double best = -1.0, cut = 0.0, lo_sum = 0.0, ratio = 1.0;
    for (size_t i = 0; i + 1 < n; ++i) {
        lo_sum += sorted[i];
        const double n_lo = (double)(i + 1), n_hi = (double)(n - i - 1);
        const double m_lo = lo_sum / n_lo, m_hi = (total - lo_sum) / n_hi;
        const double between = n_lo * n_hi * (m_hi - m_lo) * (m_hi - m_lo);
        if (between > best) {
            best = between;
            cut = 0.5 * (sorted[i] + sorted[i + 1]);
            ratio = m_hi / m_lo;
        }
    }
    if (ratio < 1.15) cut = sorted[n / 2] > 1.14 * self_rate ? 0.0 : 1e30;      // all different : all the same
    for (size_t i = 0; i < n; ++i) (*same)[i] = rate[i] < cut;
}

static int map_ref(mkv_arena* a, hipMemGenericAllocationHandle_t h) {
    if (!a->ref_va) {
        void* va = nullptr;
        MKV_HIP(hipMemAddressReserve(&va, a->chunk, 0, nullptr, 0));
        a->ref_va = (char*)va;
    }
    MKV_HIP(hipMemMap(a->ref_va, a->chunk, 0, h, 0));
    hipMemAccessDesc acc = {};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = a->device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    hipError_t e = hipMemSetAccess(a->ref_va, a->chunk, &acc, 1);
    if (e != hipSuccess) {
        (void)hipMemUnmap(a->ref_va, a->chunk);
        return ::mkv::hip_fail(e, "hipMemMap / hipMemSetAccess of the reference chunk");
    }
    a->ref = h;
    a->has_ref = true;
    return MKV_OK;
}

// The purest of a few candidates: a chunk whose own two halves fill slowest lies in ONE group (a chunk
// pieced together from two groups fills as fast as two chunks of different groups do, and would make
// every other chunk look "different" if it were the reference).
static int purest(PairGrow& g, const std::vector<size_t>& among, size_t* best, double* best_rate) {
    *best = among[0];
    *best_rate = 1e30;
    for (size_t j = 0; j < among.size() && j < 6; ++j) {
        double r = 0.0;
        int rc = g.rate(g.cand[among[j]].va, g.cand[among[j]].va + g.probe_bytes, &r);
        if (rc) return rc;
        if (r < *best_rate) {
            *best_rate = r;
            *best = among[j];
        }
    }
    return MKV_OK;
}

static int pair_grow(PairGrow& g, size_t need_k, size_t need_v, uint64_t budget_bytes, mkv_pair_info* info) {
    mkv_arena *k = g.k, *v = g.v;
    MKV_HIP(hipEventCreate(&g.e0));
    MKV_HIP(hipEventCreate(&g.e1));
    const size_t need = need_k + need_v;
    // Only the call that creates the pool searches for chunks of two groups, and keeps one spare of each as
    // the references of later calls (where the arenas can still grow).  A later call measures the chunks the
    // driver hands it against those references and deals them out as well as they allow, no more: looking
    // further would mean creating and giving back memory the rest of the process may be waiting for.
    const bool first = !k->has_ref && !v->has_ref && k->chunks.empty() && v->chunks.empty();
    const bool k_wants_ref = first && (k->chunks.size() + need_k) * k->chunk < k->reserved;
    const bool v_wants_ref = first && (v->chunks.size() + need_v) * v->chunk < v->reserved;
    const size_t spare = (k_wants_ref ? 1 : 0) + (v_wants_ref ? 1 : 0);
    size_t budget_chunks = first ? (size_t)(budget_bytes / g.chunk) : 0;
    if (budget_chunks < need + spare) budget_chunks = need + spare;

    size_t got = 0;
    int rc = g.more(need + spare, &got);
    if (rc) return rc;
    if (got < need) {
        set_error("the device has no memory left for %zu chunks of %llu bytes", need, (unsigned long long)g.chunk);
        return MKV_ENOSPC;
    }
    // references: the arenas' spares, or (first call) candidates that turn out to lie in different groups
    char *ref_k = k->has_ref ? k->ref_va : nullptr, *ref_v = v->has_ref ? v->ref_va : nullptr;
    size_t first_unmeasured = 0;
    double self_k = 0.0;
    int groups_found = 1;
    for (;;) {
        // measure what has not been measured yet
        const size_t lo = first_unmeasured, hi = g.cand.size();
        if (!ref_k && !ref_v) {
            std::vector<size_t> all;
            for (size_t i = lo; i < hi; ++i) all.push_back(i);
            size_t anchor = 0;
            if ((rc = purest(g, all, &anchor, &self_k))) return rc;
            ref_k = g.cand[anchor].va;
            g.cand[anchor].group = 0;
        }
        if (ref_k && ref_v) {
            // two references in different groups: a candidate's own two rates decide (same group ~ 3/4 of the other)
            for (size_t i = lo; i < hi; ++i) {
                if (g.cand[i].group >= 0) continue;
                double rk = 0, rv = 0;
                if ((rc = g.rate(ref_k, g.cand[i].va, &rk)) || (rc = g.rate(ref_v, g.cand[i].va, &rv))) return rc;
                g.cand[i].group = rk < 0.9 * rv ? 0 : (rv < 0.9 * rk ? 1 : 2);
            }
        } else {
            // one reference so far: split by the step in the rates against it
            char* ref = ref_k ? ref_k : ref_v;
            const int own = ref_k ? 0 : 1;
            if (self_k == 0.0 && (rc = g.rate(ref, ref + g.probe_bytes, &self_k))) return rc;
            std::vector<size_t> idx;
            for (size_t i = lo; i < hi; ++i) if (g.cand[i].group < 0) idx.push_back(i);
            std::vector<double> r(idx.size());
            for (size_t j = 0; j < idx.size(); ++j)
                if ((rc = g.rate(ref, g.cand[idx[j]].va, &r[j]))) return rc;
            std::vector<char> same;
            split_by_rate(r, self_k, &same);
            std::vector<size_t> others;
            for (size_t j = 0; j < idx.size(); ++j) {
                if (same[j]) g.cand[idx[j]].group = own;
                else others.push_back(idx[j]);
            }
            if (!others.empty()) {
                // the purest chunk of another group becomes the second reference; the rest of "another
                // group" is measured against it
                size_t second = 0;
                double self2 = 0.0;
                if ((rc = purest(g, others, &second, &self2))) return rc;
                char* ref2 = g.cand[second].va;
                (ref_k ? ref_v : ref_k) = ref2;
                g.cand[second].group = 1 - own;
                std::vector<size_t> rest;
                for (size_t i : others) if (i != second) rest.push_back(i);
                std::vector<double> r2(rest.size());
                for (size_t j = 0; j < rest.size(); ++j)
                    if ((rc = g.rate(ref2, g.cand[rest[j]].va, &r2[j]))) return rc;
                std::vector<char> same2;
                split_by_rate(r2, self2, &same2);
                for (size_t j = 0; j < rest.size(); ++j) g.cand[rest[j]].group = same2[j] ? 1 - own : 2;
            }
        }
        first_unmeasured = hi;
        size_t n0 = 0, n1 = 0, n2 = 0;
        for (auto& c : g.cand) { n0 += c.group == 0; n1 += c.group == 1; n2 += c.group == 2; }
        groups_found = 1 + (n1 > 0 || (ref_k && ref_v)) + (n2 > 0);
        // enough chunks of two different groups?  (the references are candidates like any other)
        const size_t want_k = need_k + (k_wants_ref ? 1 : 0), want_v = need_v + (v_wants_ref ? 1 : 0);
        const bool fits = (n0 >= want_k && n1 >= want_v) || (first && n1 >= want_k && n0 >= want_v);
        if (fits || g.cand.size() >= budget_chunks) break;
        // small steps: every candidate beyond the ones kept goes back to the driver, which wipes it in the background
        size_t batch = std::min(budget_chunks - g.cand.size(), std::max<size_t>(need / 8, 4));
        if ((rc = g.more(batch, &got))) return rc;
        if (got == 0) break;                                    // the device is full
    }
    // On a first call the two groups are interchangeable: K takes the one with more chunks.
    size_t n0 = 0, n1 = 0;
    for (auto& c : g.cand) { n0 += c.group == 0; n1 += c.group == 1; }
    if (first && n1 > n0) {
        for (auto& c : g.cand) if (c.group == 0 || c.group == 1) c.group = 1 - c.group;
        std::swap(n0, n1);
    }
    // hand out in creation order: each arena from its own group first, then what is missing from the
    // chunks of neither group, then from whatever is left (the other arena's group, unmeasured chunks)
    std::vector<size_t> for_k, for_v;
    auto take = [&](std::vector<size_t>* out, size_t n, int group, bool any) {
        for (size_t i = 0; i < g.cand.size() && out->size() < n; ++i)
            if (!g.cand[i].taken && (any || g.cand[i].group == group)) {
                g.cand[i].taken = true;
                out->push_back(i);
            }
    };
    take(&for_k, need_k, 0, false);
    take(&for_v, need_v, 1, false);
    take(&for_k, need_k, 2, false);
    take(&for_v, need_v, 2, false);
    take(&for_k, need_k, 0, true);
    take(&for_v, need_v, 0, true);
    if (for_k.size() < need_k || for_v.size() < need_v) {
        for (auto& c : g.cand) c.taken = false;
        set_error("the device has no memory left for %zu chunks of %llu bytes", need, (unsigned long long)g.chunk);
        return MKV_ENOSPC;
    }
    int in_k = 0, in_v = 0;
    for (size_t i : for_k) in_k += g.cand[i].group == 0;
    for (size_t i : for_v) in_v += g.cand[i].group == 1;
    // spares for later growth: one more chunk of each arena's own group, if there is one
    int spare_k = -1, spare_v = -1;
    if (groups_found >= 2) {
        for (size_t i = 0; i < g.cand.size(); ++i) {
            if (g.cand[i].taken) continue;
            if (k_wants_ref && spare_k < 0 && g.cand[i].group == 0) { spare_k = (int)i; g.cand[i].taken = true; }
            else if (v_wants_ref && spare_v < 0 && g.cand[i].group == 1) { spare_v = (int)i; g.cand[i].taken = true; }
        }
    }
    // move the chosen chunks from the staging window to the ends of the arenas
    const size_t k_had = k->chunks.size(), v_had = v->chunks.size();
    auto undo = [&]() {
        while (k->chunks.size() > k_had) { (void)hipMemUnmap(k->base + (k->chunks.size() - 1) * k->chunk, k->chunk); k->chunks.pop_back(); }
        while (v->chunks.size() > v_had) { (void)hipMemUnmap(v->base + (v->chunks.size() - 1) * v->chunk, v->chunk); v->chunks.pop_back(); }
        for (auto& c : g.cand) c.taken = false;                 // drop_everything releases every handle
    };
    for (size_t i : for_k) {
        if ((rc = g.unstage(g.cand[i])) || (rc = arena_map_handle(k, g.cand[i].h))) { undo(); return rc; }
    }
    for (size_t i : for_v) {
        if ((rc = g.unstage(g.cand[i])) || (rc = arena_map_handle(v, g.cand[i].h))) { undo(); return rc; }
    }
    if (spare_k >= 0 && ((rc = g.unstage(g.cand[spare_k])) || (rc = map_ref(k, g.cand[spare_k].h)))) g.cand[spare_k].taken = false;
    if (spare_v >= 0 && ((rc = g.unstage(g.cand[spare_v])) || (rc = map_ref(v, g.cand[spare_v].h)))) g.cand[spare_v].taken = false;
    if (info) {
        size_t kept = need_k + need_v + (spare_k >= 0 ? 1 : 0) + (spare_v >= 0 ? 1 : 0);
        info->released_bytes = (uint64_t)(g.cand.size() - kept) * g.chunk;
        info->groups_found = groups_found;
        info->candidates = (int32_t)g.cand.size();
        info->k_chunks = (int32_t)need_k;
        info->v_chunks = (int32_t)need_v;
        info->k_in_group = in_k;
        info->v_in_group = in_v;
        info->probes = g.probes;
        info->probe_ms = g.probe_ms;
    }
    return MKV_OK;
}

}  // namespace mkv

extern "C" {

int mkv_arena_pair_grow(mkv_arena* k, mkv_arena* v, uint64_t k_add_bytes, uint64_t v_add_bytes,
                        uint64_t budget_bytes, void* stream, mkv_pair_info* info) {
    MKV_REQUIRE(k != nullptr && v != nullptr && k != v, "two different arenas are needed");
    MKV_REQUIRE(k->chunk == v->chunk && k->device == v->device, "both arenas must have the same chunk size and device");
    MKV_REQUIRE(k_add_bytes % k->chunk == 0 && v_add_bytes % k->chunk == 0, "sizes must be multiples of the chunk size");
    MKV_REQUIRE(k->chunks.size() * k->chunk + k_add_bytes <= k->reserved && v->chunks.size() * v->chunk + v_add_bytes <= v->reserved,
                "the reservation is too small for that growth");
    if (info) *info = mkv_pair_info{};
    const size_t need_k = k_add_bytes / k->chunk, need_v = v_add_bytes / k->chunk;
    if (need_k + need_v == 0) return MKV_OK;
    const auto t0 = std::chrono::steady_clock::now();
    int rc;
    // the measurement fills two ranges of probe_bytes side by side; under 128 MiB each it no longer tells the
    // groups apart, and a one-sided growth has nothing to separate: plain growth then
    const uint64_t probe_bytes = std::min<uint64_t>(256ull << 20, k->chunk / 2) / 16384 * 16384;
    if (probe_bytes < (128ull << 20) || need_k == 0 || need_v == 0) {
        rc = mkv_arena_resize(k, k->chunks.size() * k->chunk + k_add_bytes);
        if (rc == MKV_OK) {
            rc = mkv_arena_resize(v, v->chunks.size() * v->chunk + v_add_bytes);
            if (rc != MKV_OK) (void)mkv_arena_resize(k, k->chunks.size() * k->chunk - k_add_bytes);
        }
        if (info) { info->k_chunks = (int32_t)need_k; info->v_chunks = (int32_t)need_v; }
        return rc;
    }
    int dev = 0;
    MKV_HIP(hipGetDevice(&dev));
    MKV_REQUIRE(dev == k->device, "the arenas' device must be current");
    if (budget_bytes == 0) {
        size_t free_b = 0, total_b = 0;
        MKV_HIP(hipMemGetInfo(&free_b, &total_b));
        budget_bytes = free_b > (4ull << 30) ? free_b - (4ull << 30) : 0;
    }
    mkv::PairGrow g;
    g.k = k;
    g.v = v;
    g.chunk = k->chunk;
    g.probe_bytes = probe_bytes;
    g.stream = (hipStream_t)stream;
    rc = mkv::pair_grow(g, need_k, need_v, budget_bytes, info);
    const hipError_t se = hipStreamSynchronize(g.stream);
    g.drop_everything();
    if (rc == MKV_OK && se != hipSuccess) rc = mkv::hip_fail(se, "hipStreamSynchronize");
    if (info) info->total_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    return rc;
}

#if MKV_DIAG
int mkv_diag_split_by_rate(const double* rates, int64_t n, double self_rate, uint8_t* same) {
    MKV_REQUIRE(rates != nullptr && same != nullptr && n >= 0, "rates and same must not be NULL");
    std::vector<double> r(rates, rates + n);
    std::vector<char> out;
    mkv::split_by_rate(r, self_rate, &out);
    for (int64_t i = 0; i < n; ++i) same[i] = out[(size_t)i] ? 1 : 0;
    return MKV_OK;
}
#endif

}  // extern "C"
