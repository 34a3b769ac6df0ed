// Host-side parallel-for shared by the host translation units (not installed).
#ifndef MPSPMM_HOSTPAR_HPP
#define MPSPMM_HOSTPAR_HPP

#include <algorithm>
#include <atomic>
#include <condition_variable>
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

// The workers: started at the first parallel_for that wants them and kept until the process ends (a builder makes
// ten to twenty parallel_for calls per plan, and starting 15 threads costs 0.3-0.6 ms each time).  One job at a
// time: a call that finds the pool busy - another thread's call, or a call from inside a chunk - runs its chunks on
// the calling thread alone.
class Pool {
public:
    static Pool &get()
    {
        static Pool pool;
        return pool;
    }
    // job() on up to `helpers` workers and on the calling thread; returns when all of them have returned
    template <typename Job>
    void run(int helpers, Job &job)
    {
        if (inside() || helpers < 1 || !busy_.try_lock()) {
            job();
            return;
        }
        std::lock_guard<std::mutex> release(busy_, std::adopt_lock);
        inside() = true;
        struct Leave {
            ~Leave() { inside() = false; }
        } leave;
        {
            std::lock_guard<std::mutex> hold(lock_);
            grow(helpers);
            call_ = [](void *j) { (*static_cast<Job *>(j))(); };
            job_ = &job;
            wanted_ = std::min<int>(helpers, (int)threads_.size());
            started_ = 0;
            ++generation_;
        }
        wake_.notify_all();
        job();
        std::unique_lock<std::mutex> hold(lock_);
        wanted_ = started_;  // workers that have not woken up yet find nothing to do
        done_.wait(hold, [&] { return running_ == 0; });
        job_ = nullptr;
    }

private:
    Pool() = default;
    ~Pool()
    {
        {
            std::lock_guard<std::mutex> hold(lock_);
            stop_ = true;
        }
        wake_.notify_all();
        for (auto &t : threads_) t.join();
    }
    static bool &inside()
    {
        static thread_local bool in = false;
        return in;
    }
    void grow(int helpers)  // lock_ held
    {
        try {
            while ((int)threads_.size() < helpers) threads_.emplace_back([this] { work(); });
        } catch (const std::system_error &) {
            // fewer threads than asked for: the ones that started and the caller share the chunks
        }
    }
    void work()
    {
        inside() = true;  // a parallel_for inside a chunk runs on the worker alone
        unsigned long long seen = 0;
        std::unique_lock<std::mutex> hold(lock_);
        for (;;) {
            wake_.wait(hold, [&] { return stop_ || generation_ != seen; });
            if (stop_) return;
            seen = generation_;
            if (started_ >= wanted_) continue;
            ++started_;
            ++running_;
            void (*call)(void *) = call_;
            void *job = job_;
            hold.unlock();
            call(job);  // (the job catches what its chunks throw)
            hold.lock();
            if (--running_ == 0) done_.notify_all();
        }
    }
    std::mutex busy_, lock_;
    std::condition_variable wake_, done_;
    std::vector<std::thread> threads_;
    void (*call_)(void *) = nullptr;
    void *job_ = nullptr;
    unsigned long long generation_ = 0;
    int wanted_ = 0, started_ = 0, running_ = 0;
    bool stop_ = false;
};

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
    Pool::get().run(nt - 1, worker);
    if (failure) std::rethrow_exception(failure);
}

}  // namespace mps_host

#endif
