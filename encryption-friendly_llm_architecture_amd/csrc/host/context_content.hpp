// Internal: the object behind HEaaN::Context (parameters, per-level scales, encoding tables and the
// device-buffer pool).  Not part of the public surface.
#pragma once
#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <vector>

#include "../../../include/hemm.h"
#include "HEaaN/HEaaN.hpp"

namespace HEaaN {

struct ContextContent {
    hemm_context *dev = nullptr;
    u64 logN = 0, N = 0, nQ = 0, nP = 0, dnum = 0, alpha = 0, log_scale = 42;
    std::vector<u64> q, p;
    std::vector<Real> delta;             // fixed scale of each level
    std::vector<u64> rot_group;          // 5^j mod 2N
    std::vector<double> ksi_re, ksi_im;  // exp(2 pi i k / 2N)
    // Freed buffers are kept by size and handed out again: every kernel runs on the one default
    // stream, so reuse is ordered after the last use without any synchronisation.
    std::multimap<size_t, u64 *> pool;
    std::mutex mu;
    size_t pool_bytes = 0;

    u64 prime(size_t i) const { return i < nQ ? q[i] : p[i - nQ]; }
    u64 *alloc(size_t words) {
        {
            std::lock_guard<std::mutex> lk(mu);
            auto it = pool.find(words);
            if (it != pool.end()) {
                u64 *r = it->second;
                pool.erase(it);
                return r;
            }
        }
        u64 *d = nullptr;
        hipError_t e = hipMalloc((void **)&d, words * sizeof(u64));
        if (e != hipSuccess) throw RuntimeException(std::string("hipMalloc: ") + hipGetErrorString(e));
        pool_bytes += words * 8;
        return d;
    }
    void release(u64 *ptr, size_t words) {
        std::lock_guard<std::mutex> lk(mu);
        pool.emplace(words, ptr);
    }
    ~ContextContent() {
        (void)hipDeviceSynchronize();
        for (auto &kv : pool) (void)hipFree(kv.second);
        if (dev) hemm_context_destroy(dev);
    }
};

}  // namespace HEaaN
