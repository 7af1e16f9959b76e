// Library plumbing: version, error strings, device query, event-based profiling.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>
#include <vector>

#include "f8mi_common.h"

namespace f8mi {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return F8MI_OK;
    set_error("%s: %s", what, hipGetErrorString(e));
    return F8MI_ERR_HIP;
}

// ------------------------------------------------------------- profiling

struct ProfRec {
    int kernel;
    double work;
    hipEvent_t start, stop;
};

static std::mutex g_prof_mu;
static std::atomic<bool> g_prof_on{false};  // read by every launch, on any thread, without the lock
static std::vector<ProfRec*> g_prof_recs;
static uint64_t g_prof_launches[F8MI_K_COUNT];
static double g_prof_ms[F8MI_K_COUNT];
static double g_prof_work[F8MI_K_COUNT];

ProfScope::ProfScope(int kernel_, double work_, hipStream_t stream_) : kernel(kernel_), work(work_), stream(stream_), rec(nullptr) {
    if (!g_prof_on.load(std::memory_order_relaxed)) return;
    ProfRec* r = new ProfRec{kernel, work, nullptr, nullptr};
    if (hipEventCreate(&r->start) != hipSuccess || hipEventCreate(&r->stop) != hipSuccess) { delete r; return; }
    (void)hipEventRecord(r->start, stream);
    rec = r;
}

ProfScope::~ProfScope() {
    if (!rec) return;
    ProfRec* r = (ProfRec*)rec;
    (void)hipEventRecord(r->stop, stream);
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_recs.push_back(r);
}

static void prof_drain_locked() {
    for (ProfRec* r : g_prof_recs) {
        float ms = 0.f;
        if (hipEventSynchronize(r->stop) == hipSuccess && hipEventElapsedTime(&ms, r->start, r->stop) == hipSuccess) {
            g_prof_launches[r->kernel] += 1;
            g_prof_ms[r->kernel] += ms;
            g_prof_work[r->kernel] += r->work;
        }
        (void)hipEventDestroy(r->start);
        (void)hipEventDestroy(r->stop);
        delete r;
    }
    g_prof_recs.clear();
}

}  // namespace f8mi

using namespace f8mi;

extern "C" int f8mi_version(void) { return F8MI_VERSION; }

extern "C" const char* f8mi_last_error(void) { return g_err; }

extern "C" int64_t f8mi_padded_k(int64_t k) { return k <= 0 ? 0 : (k + 127) / 128 * 128; }

// Names every measurement knob (f8mi_knobs.h) this build was compiled with a non-default value of; "" for the
// shipped configuration.
extern "C" const char* f8mi_build_knobs(void) {
    static char knobs[256];
    static std::once_flag once;
    std::call_once(once, [] {
        size_t n = 0;
        auto add = [&](const char* name, long long value, long long dflt) {
            if (value != dflt && n < sizeof(knobs)) n += (size_t)snprintf(knobs + n, sizeof(knobs) - n, "%s%s=%lld", n ? " " : "", name, value);
        };
        add("F8MI_WALK_GROUP", F8MI_WALK_GROUP, 4);
        add("F8MI_WALK_XCD_CHUNK", F8MI_WALK_XCD_CHUNK, 0);
        add("F8MI_WALK_SHORT_SIDE", F8MI_WALK_SHORT_SIDE, 0);
        add("F8MI_DMA_CACHE_POLICY_SET", !F8MI_DMA_CACHE_POLICY_IS_DEFAULT, 0);
        add("F8MI_CAST_REVERSE_WALK", F8MI_CAST_REVERSE_WALK, 0);
        add("F8MI_CAST_NT_STORES", F8MI_CAST_NT_STORES, 0);
        add("F8MI_AMAX_PLAIN_LOADS_MAX_BYTES", F8MI_AMAX_PLAIN_LOADS_MAX_BYTES, 0);
    });
    return knobs;
}

extern "C" size_t f8mi_workspace_bytes(void) { return WS_WORDS * sizeof(uint32_t); }

extern "C" int f8mi_device_info(int device, int* cu_count, int* lds_bytes, char* arch, int arch_len) {
    hipDeviceProp_t p;
    int rc = check_hip(hipGetDeviceProperties(&p, device), "hipGetDeviceProperties");
    if (rc) return rc;
    if (cu_count) *cu_count = p.multiProcessorCount;
    if (lds_bytes) *lds_bytes = (int)p.sharedMemPerBlock;
    if (arch && arch_len > 0) {
        strncpy(arch, p.gcnArchName, (size_t)arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0) {
        set_error("device %d is %s; this library is built for gfx950 only", device, p.gcnArchName);
        return F8MI_ERR_ARCH;
    }
    return F8MI_OK;
}

extern "C" int f8mi_prof_enable(int on) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    g_prof_on.store(on != 0, std::memory_order_relaxed);
    return F8MI_OK;
}

extern "C" int f8mi_prof_reset(void) {
    std::lock_guard<std::mutex> lk(g_prof_mu);
    prof_drain_locked();
    for (int i = 0; i < F8MI_K_COUNT; i++) { g_prof_launches[i] = 0; g_prof_ms[i] = 0; g_prof_work[i] = 0; }
    return F8MI_OK;
}

extern "C" int f8mi_prof_read(int kernel, uint64_t* launches, double* total_ms, double* total_work) {
    if (kernel < 0 || kernel >= F8MI_K_COUNT) { set_error("f8mi_prof_read: unknown kernel id %d", kernel); return F8MI_ERR_INVALID_ARG; }
    std::lock_guard<std::mutex> lk(g_prof_mu);
    prof_drain_locked();
    if (launches) *launches = g_prof_launches[kernel];
    if (total_ms) *total_ms = g_prof_ms[kernel];
    if (total_work) *total_work = g_prof_work[kernel];
    return F8MI_OK;
}
