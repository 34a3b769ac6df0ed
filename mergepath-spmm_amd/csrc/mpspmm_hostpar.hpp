// Host-side parallel-for shared by the host translation units (not installed).
#ifndef MPSPMM_HOSTPAR_HPP
#define MPSPMM_HOSTPAR_HPP

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <exception>
#include <mutex>
#include <system_error>
#include <thread>
#include <vector>

namespace mps_host {

// ---------------------------------------------------------------------------
// Threads: a tiny parallel-for.  The pool is capped at 16 workers unless
// MPS_HOST_THREADS says otherwise; results never depend on the count.
// ---------------------------------------------------------------------------
inline int host_threads()
{
    static int n = [] {
        const char *e = std::getenv("MPS_HOST_THREADS");
        int v = e ? std::atoi(e) : 0;
        if (v <= 0) {
            v = (int)std::thread::hardware_concurrency();
            if (v <= 0) v = 1;
            if (v > 16) v = 16;
        }
        return v;
    }();
    return n;
}

template <typename F>
void parallel_for(int64_t n, int64_t grain, F &&fn)
{
    if (n <= 0) return;
    int nt = host_threads();
    int64_t chunks = (n + grain - 1) / grain;
    if (nt > chunks) nt = (int)chunks;
    if (nt <= 1) {
        fn((int64_t)0, n);
        return;
    }
    std::atomic<int64_t> next(0);
    // an exception in a chunk (out of memory, in practice) stops the hand-out of
    // further chunks and is thrown again on the calling thread after the join
    std::exception_ptr failure;
    std::mutex failure_lock;
    auto worker = [&] {
        try {
            for (;;) {
                int64_t c = next.fetch_add(1, std::memory_order_relaxed);
                if (c >= chunks) break;
                int64_t lo = c * grain, hi = std::min(n, lo + grain);
                fn(lo, hi);
            }
        } catch (...) {
            next.store(chunks, std::memory_order_relaxed);
            std::lock_guard<std::mutex> hold(failure_lock);
            if (!failure) failure = std::current_exception();
        }
    };
    std::vector<std::thread> th;
    th.reserve(nt - 1);
    try {
        for (int t = 1; t < nt; ++t) th.emplace_back(worker);
    } catch (const std::system_error &) {
        // fewer threads than asked for: the ones that started and this one share the chunks
    }
    worker();
    for (auto &t : th) t.join();
    if (failure) std::rethrow_exception(failure);
}

}  // namespace mps_host

#endif
