// Error plumbing and device queries shared by the C-ABI entry points.
#include "st_common.h"

#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <unordered_set>
#include <vector>

namespace st {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what)
{
    set_error("HIP error %d (%s) in %s", (int)e, hipGetErrorString(e), what);
    return ST_ERR_HIP;
}

int device_cu_count()
{
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev] = cus;
    }
    return cached[dev];
}

// hipFuncAttributeMaxDynamicSharedMemorySize, set once per kernel symbol (keyed by the kernel's address: the
// instantiations of one kernel template share a function-pointer type, so a flag per call site is not enough).
int allow_dynamic_lds(const void *kernel, int bytes)
{
    static std::mutex mu;
    static std::unordered_set<const void *> done;
    std::lock_guard<std::mutex> lock(mu);
    if (done.count(kernel)) return ST_OK;
    ST_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    done.insert(kernel);
    return ST_OK;
}

// ---- per-kernel event timing ------------------------------------------------
struct ProfState {
    bool on = false;
    int cap = 0, used = 0;
    std::vector<hipEvent_t> start, stop;
    std::vector<int> kind;
};
static ProfState g_prof;

ProfScope::ProfScope(int kind, hipStream_t) : slot(-1), start(nullptr), stop(nullptr)
{
    if (!g_prof.on || g_prof.used >= g_prof.cap) return;
    slot = g_prof.used++;
    g_prof.kind[slot] = kind;
    start = g_prof.start[slot];
    stop = g_prof.stop[slot];
}

}  // namespace st

extern "C" int st_profile_enable(int max_samples)
{
    using namespace st;
    ST_REQUIRE(max_samples > 0 && max_samples <= (1 << 20), "st_profile_enable: max_samples out of range");
    while ((int)g_prof.start.size() < max_samples) {
        hipEvent_t a, b;
        ST_HIP(hipEventCreate(&a));
        ST_HIP(hipEventCreate(&b));
        g_prof.start.push_back(a);
        g_prof.stop.push_back(b);
    }
    g_prof.kind.assign(max_samples, 0);
    g_prof.cap = max_samples;
    g_prof.used = 0;
    g_prof.on = true;
    return ST_OK;
}

extern "C" int st_profile_disable(void)
{
    st::g_prof.on = false;
    return ST_OK;
}

extern "C" int st_profile_collect(int *kinds, float *ms, int cap)
{
    using namespace st;
    ST_REQUIRE(kinds && ms && cap >= 0, "st_profile_collect: bad arguments");
    int nout = 0;
    for (int i = 0; i < g_prof.used && nout < cap; ++i) {
        ST_HIP(hipEventSynchronize(g_prof.stop[i]));
        float t = 0.f;
        ST_HIP(hipEventElapsedTime(&t, g_prof.start[i], g_prof.stop[i]));
        kinds[nout] = g_prof.kind[i];
        ms[nout] = t;
        ++nout;
    }
    return nout;
}

extern "C" int st_version(void) { return 1; }
extern "C" const char *st_last_error(void) { return st::g_err; }
