// Library-wide plumbing of the C ABI: error string, version, and optional per-kernel timing.
//
// Timing: when enabled, every instrumented kernel launch carries a start and a stop event of its own
// (entry points that launch several kernels under one id are bracketed by two events recorded on the
// stream instead); mole_kernel_timing_read() synchronises those events and returns, per kernel id, the
// number of launches and their summed duration.  Disabled (the default) it costs
// one predictable branch per launch.
#include "common.h"

#include <mutex>
#include <vector>

namespace mole {
static thread_local char g_err[512] = "";
void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

struct TimedLaunch { int id; hipEvent_t a, b; };
static bool g_timing = false;
static std::mutex g_tmu;
static std::vector<TimedLaunch> g_launches;
// Events are created for every timed launch and destroyed when their times have been read: an event that is used again
// keeps its old time stamp when a launch does not record it, and the launch is then charged with whatever ran since.

bool timing_enabled() { return g_timing; }

static hipEvent_t get_event() {
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}

void timing_begin(int id, hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_tmu);
    TimedLaunch t{id, get_event(), get_event()};
    (void)hipEventRecord(t.a, st);
    g_launches.push_back(t);
}
void timing_events(int id, hipEvent_t *start, hipEvent_t *stop) {
    std::lock_guard<std::mutex> lk(g_tmu);
    TimedLaunch t{id, get_event(), get_event()};
    *start = t.a;
    *stop = t.b;
    g_launches.push_back(t);
}
void timing_end(hipStream_t st) {
    std::lock_guard<std::mutex> lk(g_tmu);
    if (!g_launches.empty()) (void)hipEventRecord(g_launches.back().b, st);
}
}  // namespace mole

using namespace mole;

extern "C" int mole_version(void) { return 100; }
extern "C" const char *mole_last_error_string(void) { return g_err; }

extern "C" int mole_kernel_timing_enable(int on) {
    std::lock_guard<std::mutex> lk(g_tmu);
    g_timing = on != 0;
    return 0;
}

extern "C" int mole_kernel_timing_read(int n_ids, int *counts, float *ms_total) {
    MOLE_REQUIRE(n_ids >= 0 && counts && ms_total, "mole_kernel_timing_read: null pointer");
    std::lock_guard<std::mutex> lk(g_tmu);
    for (int i = 0; i < n_ids; ++i) { counts[i] = 0; ms_total[i] = 0.f; }
    for (auto &t : g_launches) {
        float ms = 0.f;
        // a launch whose events were not both recorded is left out of the count rather than guessed at
        const bool ok = hipEventSynchronize(t.b) == hipSuccess && hipEventElapsedTime(&ms, t.a, t.b) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        if (ok && t.id >= 0 && t.id < n_ids) { counts[t.id] += 1; ms_total[t.id] += ms; }
        (void)hipEventDestroy(t.a);
        (void)hipEventDestroy(t.b);
    }
    g_launches.clear();
    return 0;
}
