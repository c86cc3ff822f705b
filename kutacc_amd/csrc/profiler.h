// Optional per-kernel timing for the benchmark: when enabled, every launch made through
// KernelTimer is bracketed by a pair of hipEvents on the launch stream.  Totals per kernel name are
// resolved lazily (at read time) so that recording never blocks the host.
#pragma once
#include <hip/hip_runtime.h>

namespace kutacc_prof {
bool enabled();

// While one of these lives on a thread, KernelTimer records nothing there (event creation allocates, which the entry
// points that promise not to allocate must not do even when a benchmark has switched timing on).
class Suppress {
public:
    Suppress();
    ~Suppress();
    Suppress(const Suppress &) = delete;
    Suppress &operator=(const Suppress &) = delete;
};

// Brackets the launches issued during its lifetime.  `flops` is the algorithmic work of one launch,
// reported back next to the measured time.
class KernelTimer {
public:
    KernelTimer(const char *name, double flops, hipStream_t stream);
    ~KernelTimer();
    KernelTimer(const KernelTimer &) = delete;
    KernelTimer &operator=(const KernelTimer &) = delete;

private:
    const char *name_;
    double flops_;
    hipStream_t stream_;
    hipEvent_t start_ = nullptr;
};
} // namespace kutacc_prof
