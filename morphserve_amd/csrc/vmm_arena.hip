// Pool backing through HIP virtual memory: one address range reserved once, physical
// chunks mapped at its end when the pool grows and unmapped when it shrinks.  The pool
// stays ONE contiguous [num_blocks, L, Hkv, B, D] tensor at a fixed address, so block ids
// never need the segment arithmetic and growing never copies.
#include "common.h"

#include <vector>

struct mkv_arena {
    char* base = nullptr;
    uint64_t reserved = 0;
    uint64_t chunk = 0;
    int device = 0;
    std::vector<hipMemGenericAllocationHandle_t> chunks;     // chunk i backs [i * chunk, (i + 1) * chunk)
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
        MKV_HIP(e);
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
        MKV_HIP(e);
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
