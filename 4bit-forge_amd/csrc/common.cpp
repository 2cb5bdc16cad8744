#include "common.h"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <cstring>
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

namespace forge {
namespace {
struct OptionInfo { const char* name; const char* env; int64_t lo, hi, dflt; };
const OptionInfo kOptions[OPT_COUNT] = {
    {"sweep_schedule", "FORGE_SWEEP_SCHEDULE", 0, 2, 0},
    {"fp32_blocked_sum", "FORGE_FP32_BLOCKED_SUM", 0, 1, 0},
    {"sweep_update_products", "FORGE_SWEEP_UPDATE_PRODUCTS", 0, 6, 0},
    {"factor_pieces", "FORGE_FACTOR_PIECES", 0, 1, 0},
    {"mse_reference_quantiser", "FORGE_MSE_REFERENCE_QUANTISER", 0, 1, 0},
};
std::atomic<int64_t> g_options[OPT_COUNT];

bool valid_option(int o, int64_t v) {
    if (v < kOptions[o].lo || v > kOptions[o].hi) return false;
    return o != OPT_SWEEP_PRODUCTS || v == 0 || v == 1 || v == 2 || v == 3 || v == 4 || v == 6;
}

// Runs when the library is loaded: the environment is looked at here and nowhere else.
struct OptionInit {
    OptionInit() {
        for (int o = 0; o < OPT_COUNT; ++o) {
            int64_t v = kOptions[o].dflt;
            if (const char* e = getenv(kOptions[o].env)) {
                int64_t x = v;
                if (o == OPT_SWEEP_SCHEDULE && (e[0] == 'l' || e[0] == 'r')) x = e[0] == 'l' ? 1 : 2;
                else if (e[0] >= '0' && e[0] <= '9') x = strtoll(e, nullptr, 10);
                if (valid_option(o, x)) v = x;
            }
            g_options[o].store(v, std::memory_order_relaxed);
        }
    }
} g_option_init;
}  // namespace

int64_t option(Option o) { return g_options[o].load(std::memory_order_relaxed); }
}  // namespace forge

extern "C" int forge_set_option(const char* name, int64_t value) {
    if (!name) return forge::fail(FORGE_ERR_INVALID, "option name is null");
    for (int o = 0; o < forge::OPT_COUNT; ++o)
        if (strcmp(name, forge::kOptions[o].name) == 0) {
            if (!forge::valid_option(o, value))
                return forge::fail(FORGE_ERR_INVALID, "option %s: value %lld not allowed", name,
                                   (long long)value);
            forge::g_options[o].store(value, std::memory_order_relaxed);
            return FORGE_OK;
        }
    return forge::fail(FORGE_ERR_INVALID, "unknown option %s", name);
}

extern "C" int64_t forge_get_option(const char* name) {
    if (name)
        for (int o = 0; o < forge::OPT_COUNT; ++o)
            if (strcmp(name, forge::kOptions[o].name) == 0) return forge::option((forge::Option)o);
    forge::fail(FORGE_ERR_INVALID, "unknown option %s", name ? name : "(null)");
    return -1;
}

extern "C" int forge_hip_abi_version(void) { return 1; }
extern "C" const char* forge_last_error(void) { return forge::error_buffer(); }
