// Internal: the object behind HEaaN::Context (parameters, per-level scales, encoding tables and the
// device-buffer pool).  Not part of the public surface.
#pragma once
#include <hip/hip_runtime.h>

#include <map>
#include <mutex>
#include <string>
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
    // Freed buffers are kept by size and handed out again: kernels run on the default stream, so reuse is
    // ordered after the last use without any synchronisation.  The one exception is a side chain (forkSide /
    // joinSide below): while it is open, freed buffers are parked and only return to the pool at the join.
    std::multimap<size_t, u64 *> pool;
    std::vector<std::pair<size_t, u64 *>> parked;
    std::mutex mu;
    size_t pool_bytes = 0;
    hipStream_t side = nullptr;
    hipEvent_t ev_fork = nullptr, ev_join = nullptr, ev_main = nullptr, ev_side = nullptr;
    bool side_open = false;
    // the stream the host layer queues on: the device context's (hemm_context_set_stream), by default the legacy
    // default stream; on(s) resolves a stream argument whose null value means that stream
    hipStream_t stream() const { return (hipStream_t)hemm_context_stream(dev); }
    hipStream_t on(hipStream_t s) const { return s != nullptr ? s : stream(); }

    // Opens a side chain: work given to the returned stream starts after everything queued on the default stream
    // so far and runs beside what the default stream is given next.  The stream does not synchronise implicitly
    // with the default stream; joinSide() makes the default stream wait for it.  Default priority.
    hipStream_t forkSide() {
        if (side_open) throw RuntimeException("side chain already open");
        auto ok = [](hipError_t e, const char *what) {
            if (e != hipSuccess) throw RuntimeException(std::string(what) + ": " + hipGetErrorString(e));
        };
        if (!side) {
            ok(hipStreamCreateWithFlags(&side, hipStreamNonBlocking), "hipStreamCreateWithFlags");
            ok(hipEventCreateWithFlags(&ev_fork, hipEventDisableTiming), "hipEventCreateWithFlags");
            ok(hipEventCreateWithFlags(&ev_join, hipEventDisableTiming), "hipEventCreateWithFlags");
            ok(hipEventCreateWithFlags(&ev_main, hipEventDisableTiming), "hipEventCreateWithFlags");
            ok(hipEventCreateWithFlags(&ev_side, hipEventDisableTiming), "hipEventCreateWithFlags");
        }
        ok(hipEventRecord(ev_fork, stream()), "hipEventRecord");
        ok(hipStreamWaitEvent(side, ev_fork, 0), "hipStreamWaitEvent");
        std::lock_guard<std::mutex> lk(mu);
        side_open = true;
        return side;
    }
    // While a side chain is open, the two streams can also wait for each other half way without closing it:
    // sideWaitsForMain() orders what the side stream is given next after everything queued on the default stream so
    // far; markSide() notes the side stream's position and waitSideMark() makes the default stream wait for the last
    // such note (work queued on the side stream after the note is not waited for).
    void sideWaitsForMain() {
        if (!side_open) throw RuntimeException("no side chain open");
        (void)hipEventRecord(ev_main, stream());
        (void)hipStreamWaitEvent(side, ev_main, 0);
    }
    void markSide() {
        if (!side_open) throw RuntimeException("no side chain open");
        (void)hipEventRecord(ev_side, side);
    }
    void waitSideMark() {
        if (!side_open) throw RuntimeException("no side chain open");
        (void)hipStreamWaitEvent(stream(), ev_side, 0);
    }
    void joinSide() {
        if (!side_open) return;
        (void)hipEventRecord(ev_join, side);
        (void)hipStreamWaitEvent(stream(), ev_join, 0);
        std::lock_guard<std::mutex> lk(mu);
        side_open = false;
        for (auto &kv : parked) pool.emplace(kv.first, kv.second);
        parked.clear();
    }

    // Optional phase trace of the batched products: while it is on, mark() records an event on the default stream at
    // a named point of the schedule; the report gives the time between consecutive marks.
    bool trace_on = false;
    std::vector<std::pair<std::string, hipEvent_t>> trace_marks;
    void mark(const char *name) {
        if (!trace_on) return;
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return;
        (void)hipEventRecord(e, stream());
        trace_marks.emplace_back(name, e);
    }
    void traceClear() {
        for (auto &m : trace_marks) (void)hipEventDestroy(m.second);
        trace_marks.clear();
    }

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
    // Stream capture of a sequence of calls (hellm_graph_begin / _end): a buffer released while the capture is open
    // stays with the graph being recorded -- its replays write that memory -- and returns to the pool when the graph
    // is destroyed.
    bool capture_open = false;
    std::vector<std::pair<size_t, u64 *>> captured;
    void release(u64 *ptr, size_t words) {
        std::lock_guard<std::mutex> lk(mu);
        if (capture_open)
            captured.emplace_back(words, ptr);
        else if (side_open)
            parked.emplace_back(words, ptr);
        else
            pool.emplace(words, ptr);
    }
    ~ContextContent() {
        (void)hipDeviceSynchronize();
        traceClear();
        for (auto &kv : pool) (void)hipFree(kv.second);
        for (auto &kv : parked) (void)hipFree(kv.second);
        for (auto &kv : captured) (void)hipFree(kv.second);
        if (side) (void)hipStreamDestroy(side);
        if (ev_fork) (void)hipEventDestroy(ev_fork);
        if (ev_join) (void)hipEventDestroy(ev_join);
        if (ev_main) (void)hipEventDestroy(ev_main);
        if (ev_side) (void)hipEventDestroy(ev_side);
        if (dev) hemm_context_destroy(dev);
    }
};

}  // namespace HEaaN
