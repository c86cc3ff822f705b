// Staged (host-pointer) calls: device mirrors of host ranges, taken from a pool that the library keeps between calls.
// Shared by the translation units that implement the handle-based entry points; the pool itself is defined in api.cpp.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <mutex>
#include <vector>

namespace kutacc_api {
// Device mirror of a host range, for the staged (host-pointer) path.
struct Mirror {
    void *dev = nullptr;
    void *host = nullptr;
    size_t bytes = 0;
    bool copy_back = false;
};

// Device buffers of the staged path are kept between calls: a call takes what it needs from the pool (smallest buffer
// that is large enough, else a new allocation) and gives everything back when it is done, so a caller that repeats a
// shape pays hipMalloc once.  kutacc_hip_release_staging() frees the pool.
struct StagingPool {
    struct Block {
        void *dev;
        size_t bytes;
        int device; // the device the memory lives on: a block is only handed out again there
    };
    std::mutex mu;
    std::vector<Block> free_blocks;
    static int current_device()
    {
        int d = 0;
        (void)hipGetDevice(&d);
        return d;
    }
    hipError_t take(size_t bytes, void **out, size_t *got)
    {
        {
            const int here = current_device();
            std::lock_guard<std::mutex> lk(mu);
            int best = -1;
            for (int i = 0; i < (int)free_blocks.size(); ++i) {
                if (free_blocks[i].device == here && free_blocks[i].bytes >= bytes &&
                    (best < 0 || free_blocks[i].bytes < free_blocks[best].bytes)) {
                    best = i;
                }
            }
            if (best >= 0) {
                *out = free_blocks[best].dev, *got = free_blocks[best].bytes;
                free_blocks.erase(free_blocks.begin() + best);
                return hipSuccess;
            }
        }
        *got = bytes;
        return hipMalloc(out, bytes);
    }
    void give(void *dev, size_t bytes)
    {
        const int here = current_device(); // a call takes and gives on the same current device
        std::lock_guard<std::mutex> lk(mu);
        free_blocks.push_back({dev, bytes, here});
    }
    size_t release()
    {
        std::lock_guard<std::mutex> lk(mu);
        size_t total = 0;
        for (auto &b : free_blocks) {
            total += b.bytes;
            (void)hipFree(b.dev);
        }
        free_blocks.clear();
        return total;
    }
};
extern StagingPool g_staging;

struct Stager {
    std::vector<Mirror> items;
    std::vector<size_t> capacity; // what the pool gave for each item
    hipStream_t stream;
    int rc = 0;
    explicit Stager(hipStream_t s) : stream(s) {}
    void *in(const void *host, size_t bytes) { return add(const_cast<void *>(host), bytes, true, false); }
    void *scratch(size_t bytes) { return add(nullptr, bytes, false, false); }
    void *out(void *host, size_t bytes, bool preload) { return add(host, bytes, preload, true); }
    void *add(void *host, size_t bytes, bool upload, bool back)
    {
        if (rc != 0 || bytes == 0) {
            return nullptr;
        }
        Mirror m;
        m.host = host, m.bytes = bytes, m.copy_back = back;
        size_t got = 0;
        hipError_t e = g_staging.take(bytes, &m.dev, &got);
        if (e == hipSuccess && upload && host) {
            e = hipMemcpyAsync(m.dev, host, bytes, hipMemcpyHostToDevice, stream);
        }
        if (e != hipSuccess) {
            rc = (int)e;
            if (m.dev) {
                g_staging.give(m.dev, got);
            }
            return nullptr;
        }
        items.push_back(m);
        capacity.push_back(got);
        return m.dev;
    }
    int finish()
    {
        for (auto &m : items) {
            if (rc == 0 && m.copy_back) {
                const hipError_t e = hipMemcpyAsync(m.host, m.dev, m.bytes, hipMemcpyDeviceToHost, stream);
                if (e != hipSuccess) {
                    rc = (int)e;
                }
            }
        }
        const hipError_t e = hipStreamSynchronize(stream);
        if (rc == 0 && e != hipSuccess) {
            rc = (int)e;
        }
        for (size_t i = 0; i < items.size(); ++i) {
            g_staging.give(items[i].dev, capacity[i]);
        }
        items.clear();
        capacity.clear();
        return rc;
    }
};
} // namespace kutacc_api
