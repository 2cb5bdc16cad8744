#include "common.h"

#include <algorithm>
#include <mutex>
#include <string>
#include <vector>

namespace forge {

char* error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), 512, fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace forge

namespace forge {
namespace {
struct TimedLaunch { std::string name; double work; WorkKind kind; hipEvent_t t0, t1; };
struct TimingSummary { std::string name; int64_t launches; double ms, work; int kind; };
std::mutex g_mu;
bool g_enabled = false;
std::vector<TimedLaunch> g_launches;
std::vector<TimingSummary> g_summary;

void drop_events() {
    for (auto& l : g_launches) {
        (void)hipEventDestroy(l.t0);
        (void)hipEventDestroy(l.t1);
    }
    g_launches.clear();
}

// Wait for every bracketed launch and fold the pairs into one line per kernel name.
int summarise() {
    g_summary.clear();
    for (auto& l : g_launches) {
        if (hipEventSynchronize(l.t1) != hipSuccess) return -1;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, l.t0, l.t1) != hipSuccess) return -1;
        auto it = std::find_if(g_summary.begin(), g_summary.end(),
                               [&](const TimingSummary& s) { return s.name == l.name; });
        if (it == g_summary.end()) {
            g_summary.push_back({l.name, 0, 0.0, 0.0, (int)l.kind});
            it = g_summary.end() - 1;
        }
        it->launches += 1;
        it->ms += ms;
        it->work += l.work;
    }
    drop_events();
    return (int)g_summary.size();
}
}  // namespace

KernelTiming::KernelTiming(const char* name, hipStream_t st, double work, WorkKind kind)
    : slot_(-1), st_(st) {
    if (!name) return;                       // a caller that must not create events
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_enabled) return;
    TimedLaunch l{name, work, kind, nullptr, nullptr};
    if (hipEventCreate(&l.t0) != hipSuccess || hipEventCreate(&l.t1) != hipSuccess) return;
    (void)hipEventRecord(l.t0, st);
    g_launches.push_back(l);
    slot_ = (int)g_launches.size() - 1;
}

KernelTiming::~KernelTiming() {
    if (slot_ < 0) return;
    std::lock_guard<std::mutex> lock(g_mu);
    if (slot_ < (int)g_launches.size()) (void)hipEventRecord(g_launches[slot_].t1, st_);
}
}  // namespace forge

extern "C" int forge_kernel_timing_enable(int on) {
    std::lock_guard<std::mutex> lock(forge::g_mu);
    forge::drop_events();
    forge::g_summary.clear();
    forge::g_enabled = on != 0;
    return FORGE_OK;
}

extern "C" int forge_kernel_timing_collect(void) {
    std::lock_guard<std::mutex> lock(forge::g_mu);
    const int n = forge::summarise();
    if (n < 0) return -forge::fail(FORGE_ERR_HIP, "reading timing events failed");
    return n;
}

extern "C" int forge_kernel_timing_get(int index, char* name, int name_cap, int64_t* launches,
                                       double* total_ms, double* work, int* work_kind) {
    std::lock_guard<std::mutex> lock(forge::g_mu);
    if (index < 0 || index >= (int)forge::g_summary.size() || !name || name_cap < 1)
        return forge::fail(FORGE_ERR_INVALID, "timing index %d out of range", index);
    const auto& s = forge::g_summary[index];
    snprintf(name, (size_t)name_cap, "%s", s.name.c_str());
    if (launches) *launches = s.launches;
    if (total_ms) *total_ms = s.ms;
    if (work) *work = s.work;
    if (work_kind) *work_kind = s.kind;
    return FORGE_OK;
}

extern "C" int forge_hip_abi_version(void) { return 1; }
extern "C" const char* forge_last_error(void) { return forge::error_buffer(); }
