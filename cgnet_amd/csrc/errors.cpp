// Thread-local error message of the C ABI, trivial queries and the per-kernel timing hooks.
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"

namespace cgnet {
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
void clear_error() { g_err[0] = 0; }

int raise_dynamic_lds(const void* func, size_t bytes) {
    static std::mutex mu;
    static std::map<std::pair<const void*, int>, size_t> granted;
    if (bytes <= 64 * 1024) return CGNET_OK;          // the default limit covers it
    int device = 0;
    CGNET_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(mu);
    size_t& have = granted[std::make_pair(func, device)];
    if (bytes <= have) return CGNET_OK;
    CGNET_HIP(hipFuncSetAttribute(func, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
    have = bytes;
    return CGNET_OK;
}
}  // namespace cgnet

extern "C" const char* cgnet_last_error(void) { return cgnet::g_err; }
extern "C" int cgnet_abi_version(void) { return 1; }
extern "C" int cgnet_sparse_maxL(void) { return cgnet::kMaxL; }

// --------------------------------------------------------------------------- kernel timing
namespace cgnet {
namespace {
struct Pending { const char* name; hipEvent_t start, stop; };
struct Total { double ms = 0.; int launches = 0; };
std::mutex g_mu;
bool g_enabled = false;
std::string g_only;              // when set, only launches of this kernel are timed
std::vector<Pending> g_pending;
std::vector<hipEvent_t> g_pool;
std::map<std::string, Total> g_totals;

hipEvent_t take_event() {
    if (!g_pool.empty()) {
        hipEvent_t e = g_pool.back();
        g_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}
}  // namespace

KernelTimer::KernelTimer(const char* name, hipStream_t stream) : name_(name), stream_(stream) {
    std::lock_guard<std::mutex> lock(g_mu);
    if (!g_enabled) return;
    if (!g_only.empty() && std::strncmp(name, g_only.c_str(), g_only.size()) != 0) return;
    start_ = take_event();
    stop_ = take_event();
    if (start_ && stop_) {
        (void)hipEventRecord(start_, stream_);
    } else {
        if (start_) g_pool.push_back(start_);
        if (stop_) g_pool.push_back(stop_);
        start_ = stop_ = nullptr;
    }
}

KernelTimer::~KernelTimer() {
    if (!start_) return;
    (void)hipEventRecord(stop_, stream_);
    std::lock_guard<std::mutex> lock(g_mu);
    g_pending.push_back(Pending{name_, start_, stop_});
}
}  // namespace cgnet

extern "C" int cgnet_profile_enable(int on) {
    std::lock_guard<std::mutex> lock(cgnet::g_mu);
    const int prev = cgnet::g_enabled ? 1 : 0;
    cgnet::g_enabled = on != 0;
    return prev;
}

extern "C" int cgnet_profile_select(const char* kernel_name) {
    std::lock_guard<std::mutex> lock(cgnet::g_mu);
    cgnet::g_only = kernel_name ? kernel_name : "";
    return CGNET_OK;
}

extern "C" int cgnet_profile_reset(void) {
    std::lock_guard<std::mutex> lock(cgnet::g_mu);
    for (const cgnet::Pending& p : cgnet::g_pending) {
        cgnet::g_pool.push_back(p.start);
        cgnet::g_pool.push_back(p.stop);
    }
    cgnet::g_pending.clear();
    cgnet::g_totals.clear();
    return CGNET_OK;
}

extern "C" int cgnet_profile_collect(void) {
    std::lock_guard<std::mutex> lock(cgnet::g_mu);
    for (const cgnet::Pending& p : cgnet::g_pending) {
        float ms = 0.f;
        // the caller has synchronised the streams; an event that is not ready is skipped
        if (hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
            cgnet::Total& t = cgnet::g_totals[p.name];
            t.ms += ms;
            t.launches += 1;
        }
        cgnet::g_pool.push_back(p.start);
        cgnet::g_pool.push_back(p.stop);
    }
    cgnet::g_pending.clear();
    (void)hipGetLastError();
    return (int)cgnet::g_totals.size();
}

extern "C" int cgnet_profile_get(int index, char* name, int name_capacity, double* total_ms, int* launches) {
    std::lock_guard<std::mutex> lock(cgnet::g_mu);
    if (index < 0 || index >= (int)cgnet::g_totals.size() || !name || name_capacity <= 0) return CGNET_ERR_ARG;
    auto it = cgnet::g_totals.begin();
    std::advance(it, index);
    std::strncpy(name, it->first.c_str(), (size_t)name_capacity - 1);
    name[name_capacity - 1] = 0;
    if (total_ms) *total_ms = it->second.ms;
    if (launches) *launches = it->second.launches;
    return CGNET_OK;
}
