// Library plumbing: error text, argument checks, per-kernel event timing.
#include "common.h"

#include <stdarg.h>
#include <string.h>
#include <mutex>
#include <vector>

namespace mkv {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
    set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return MKV_EHIP;
}

int check_pool(const mkv_pool* p) {
    MKV_REQUIRE(p != nullptr, "pool is NULL");
    MKV_REQUIRE(p->k_base && p->v_base, "pool base pointers are NULL");
    MKV_REQUIRE(p->num_layers > 0 && p->num_kv_heads > 0 && p->block_size > 0 && p->head_dim > 0,
                "pool dims must be positive (L=%d Hkv=%d B=%d D=%d)", p->num_layers,
                p->num_kv_heads, p->block_size, p->head_dim);
    MKV_REQUIRE(p->head_dim % 8 == 0, "head_dim %d must be a multiple of 8 (16-byte units)", p->head_dim);
    MKV_REQUIRE(p->num_blocks_org >= 0, "num_blocks_org must be >= 0");
    MKV_REQUIRE(p->num_segments >= 0 && p->num_segments <= MKV_MAX_SEGMENTS,
                "num_segments %d outside [0, %d]", p->num_segments, MKV_MAX_SEGMENTS);
    if (p->num_segments > 0) {
        MKV_REQUIRE(p->seg_blocks > 0, "seg_blocks must be positive when segments exist");
        for (int j = 0; j < p->num_segments; ++j)
            MKV_REQUIRE(p->k_seg[j] && p->v_seg[j], "segment %d has a NULL base", j);
    }
    MKV_REQUIRE(p->num_blocks_org + (int64_t)p->num_segments * p->seg_blocks <= 0x7fffffff &&
                    p->seg_blocks <= 0x7fffffff,
                "block ids are 32-bit: the pool may hold at most 2^31 - 1 blocks");
    MKV_REQUIRE(((uintptr_t)p->k_base & 15) == 0 && ((uintptr_t)p->v_base & 15) == 0,
                "pool bases must be 16-byte aligned");
    for (int j = 0; j < p->num_segments; ++j)
        MKV_REQUIRE(((uintptr_t)p->k_seg[j] & 15) == 0 && ((uintptr_t)p->v_seg[j] & 15) == 0,
                    "segment %d base must be 16-byte aligned", j);
    return MKV_OK;
}

int num_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

#if MKV_DIAG
// ---- per-workgroup time stamps -----------------------------------------------------
static long long* g_timeline = nullptr;
static int64_t g_timeline_wgs = 0;

long long* timeline_buffer(int64_t workgroups) {
    return (g_timeline != nullptr && workgroups <= g_timeline_wgs) ? g_timeline : nullptr;
}

// ---- profiling ---------------------------------------------------------------
struct ProfRec {
    hipEvent_t start, stop;
};
static std::mutex g_prof_mu;
static bool g_prof_on = false;
static std::vector<ProfRec> g_prof[MKV_K_COUNT];

ProfScope::ProfScope(int id, hipStream_t s) : kernel_id(id), stream(s), rec(nullptr) {
    if (!g_prof_on) return;
    ProfRec* r = new ProfRec;
    if (hipEventCreate(&r->start) != hipSuccess || hipEventCreate(&r->stop) != hipSuccess) {
        delete r;
        return;
    }
    (void)hipEventRecord(r->start, stream);
    rec = r;
}

ProfScope::~ProfScope() {
    if (!rec) return;
    ProfRec* r = (ProfRec*)rec;
    (void)hipEventRecord(r->stop, stream);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof[kernel_id].push_back(*r);
    delete r;
}
#endif  // MKV_DIAG

}  // namespace mkv

extern "C" {

const char* mkv_last_error(void) { return mkv::g_err; }

int mkv_version(void) { return 1; }

int mkv_sizeof_pool(void) { return (int)sizeof(mkv_pool); }

int mkv_pool_set_strided(mkv_pool* pool, void* k_new0, void* v_new0,
                         int64_t org_layer_param_size, int32_t elem_bytes,
                         int32_t num_segments) {
    MKV_REQUIRE(pool != nullptr, "pool is NULL");
    MKV_REQUIRE(num_segments >= 0 && num_segments <= MKV_MAX_SEGMENTS,
                "num_segments %d outside [0, %d]", num_segments, MKV_MAX_SEGMENTS);
    MKV_REQUIRE(num_segments == 0 || (k_new0 && v_new0), "segment 0 bases are NULL");
    pool->num_segments = num_segments;
    for (int j = 0; j < num_segments; ++j) {
        int64_t back = (int64_t)j * org_layer_param_size * elem_bytes;
        pool->k_seg[j] = (char*)k_new0 - back;
        pool->v_seg[j] = (char*)v_new0 - back;
    }
    for (int j = num_segments; j < MKV_MAX_SEGMENTS; ++j) pool->k_seg[j] = pool->v_seg[j] = nullptr;
    return MKV_OK;
}

#if MKV_DIAG
int mkv_diag_timeline(void* buf, int64_t max_workgroups) {
    MKV_REQUIRE(buf == nullptr || max_workgroups > 0, "max_workgroups must be positive with a buffer");
    MKV_REQUIRE(((uintptr_t)buf & 7) == 0, "the time stamp buffer must be 8-byte aligned");
    mkv::g_timeline = (long long*)buf;
    mkv::g_timeline_wgs = buf ? max_workgroups : 0;
    return MKV_OK;
}

int mkv_prof_enable(int32_t on) {
    std::lock_guard<std::mutex> lk(mkv::g_prof_mu);
    mkv::g_prof_on = on != 0;
    return MKV_OK;
}

int mkv_prof_reset(void) {
    std::lock_guard<std::mutex> lk(mkv::g_prof_mu);
    for (auto& v : mkv::g_prof) {
        for (auto& r : v) {
            (void)hipEventDestroy(r.start);
            (void)hipEventDestroy(r.stop);
        }
        v.clear();
    }
    return MKV_OK;
}

int mkv_prof_collect(int32_t kernel_id, int64_t* launches, double* total_ms) {
    MKV_REQUIRE(kernel_id >= 0 && kernel_id < MKV_K_COUNT, "kernel_id %d out of range", kernel_id);
    MKV_REQUIRE(launches && total_ms, "output pointers are NULL");
    std::lock_guard<std::mutex> lk(mkv::g_prof_mu);
    double sum = 0.0;
    for (auto& r : mkv::g_prof[kernel_id]) {
        MKV_HIP(hipEventSynchronize(r.stop));
        float ms = 0.f;
        MKV_HIP(hipEventElapsedTime(&ms, r.start, r.stop));
        sum += ms;
    }
    *launches = (int64_t)mkv::g_prof[kernel_id].size();
    *total_ms = sum;
    return MKV_OK;
}
#endif  // MKV_DIAG

}  // extern "C"
