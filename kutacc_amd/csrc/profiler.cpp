#include "profiler.h"

#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "kutacc_hip.h"

namespace {
struct Pending {
    const char *name;
    double flops;
    hipEvent_t start, stop;
};
struct Total {
    std::string name;
    double ms = 0.0;
    double flops = 0.0;
    int64_t launches = 0;
};
std::mutex g_mu;
bool g_enabled = false;
std::vector<Pending> g_pending;
std::vector<Total> g_totals;

void resolve_locked()
{
    for (auto &p : g_pending) {
        float ms = 0.f;
        if (hipEventSynchronize(p.stop) == hipSuccess && hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
            Total *t = nullptr;
            for (auto &c : g_totals) {
                if (c.name == p.name) {
                    t = &c;
                }
            }
            if (!t) {
                g_totals.emplace_back();
                t = &g_totals.back();
                t->name = p.name;
            }
            t->ms += ms;
            t->flops = p.flops;
            t->launches += 1;
        }
        (void)hipEventDestroy(p.start);
        (void)hipEventDestroy(p.stop);
    }
    g_pending.clear();
}
} // namespace

namespace kutacc_prof {
bool enabled() { return g_enabled; }

static thread_local int t_suppressed = 0;
Suppress::Suppress() { ++t_suppressed; }
Suppress::~Suppress() { --t_suppressed; }

KernelTimer::KernelTimer(const char *name, double flops, hipStream_t stream) : name_(name), flops_(flops), stream_(stream)
{
    if (g_enabled && t_suppressed == 0 && hipEventCreate(&start_) == hipSuccess) {
        (void)hipEventRecord(start_, stream_);
    }
}

KernelTimer::~KernelTimer()
{
    if (!start_) {
        return;
    }
    hipEvent_t stop = nullptr;
    if (hipEventCreate(&stop) != hipSuccess) {
        (void)hipEventDestroy(start_);
        return;
    }
    (void)hipEventRecord(stop, stream_);
    std::lock_guard<std::mutex> lk(g_mu);
    g_pending.push_back({name_, flops_, start_, stop});
}
} // namespace kutacc_prof

void kutacc_hip_profile_enable(int on)
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (on && !g_enabled) {
        resolve_locked();
        g_totals.clear();
    }
    g_enabled = on != 0;
}

int kutacc_hip_profile_read(int index, char *name, int name_len, double *total_ms, int64_t *launches,
                            double *flops_per_launch)
{
    std::lock_guard<std::mutex> lk(g_mu);
    resolve_locked();
    if (index < 0 || (size_t)index >= g_totals.size()) {
        return -1;
    }
    const Total &t = g_totals[(size_t)index];
    if (name && name_len > 0) {
        std::strncpy(name, t.name.c_str(), (size_t)name_len - 1);
        name[name_len - 1] = '\0';
    }
    if (total_ms) {
        *total_ms = t.ms;
    }
    if (launches) {
        *launches = t.launches;
    }
    if (flops_per_launch) {
        *flops_per_launch = t.flops;
    }
    return 0;
}
