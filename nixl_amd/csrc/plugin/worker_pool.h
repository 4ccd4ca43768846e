// A few helper threads that share one loop over slices with the thread that calls run().
// Made for host passes of a hundred microseconds (a request's 65 536 descriptor pairs read
// once): the caller starts on the slices at once and the helpers join in as they wake, so a
// helper that wakes late costs nothing but its share.  Helpers poll for the next job for a
// short while after each one and then sleep on a condition variable.
#ifndef NIXL_AMD_WORKER_POOL_H
#define NIXL_AMD_WORKER_POOL_H

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdint>
#include <mutex>
#include <thread>
#include <vector>

namespace nixl_amd_hip {

class WorkerPool {
public:
    explicit WorkerPool(unsigned helpers) {
        threads_.reserve(helpers);
        for (unsigned i = 0; i < helpers; ++i)
            threads_.emplace_back([this] { helperLoop(); });
    }

    ~WorkerPool() {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            stop_ = true;
        }
        wake_.notify_all();
        for (std::thread &t : threads_)
            t.join();
    }

    WorkerPool(const WorkerPool &) = delete;
    WorkerPool &
    operator=(const WorkerPool &) = delete;

    // Calls fn(slice) once for every slice in [0, slices), on this thread and on the helpers,
    // and returns true when all calls have returned.  Returns false without calling fn when
    // another thread's job occupies the pool: the caller then does its work alone.
    template<class F>
    bool
    run(unsigned slices, F &&fn) {
        bool expected = false;
        if (!busy_.compare_exchange_strong(expected, true, std::memory_order_acquire)) return false;
        uint64_t ticket;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            call_ = [](void *ctx, unsigned slice) { (*static_cast<std::remove_reference_t<F> *>(ctx))(slice); };
            ctx_ = &fn;
            slices_ = slices;
            done_.store(0, std::memory_order_relaxed);
            ticket = (generation_.load(std::memory_order_relaxed) + 1) & 0xffffffffu;
            next_.store(ticket << 32, std::memory_order_relaxed);
            generation_.store(ticket, std::memory_order_release);
        }
        wake_.notify_all();
        work(ticket, call_, ctx_, slices);
        while (done_.load(std::memory_order_acquire) < slices)
            relax();
        busy_.store(false, std::memory_order_release);
        return true;
    }

private:
    using call_t = void (*)(void *, unsigned);

    static void
    relax() {
#if defined(__x86_64__)
        __builtin_ia32_pause();
#else
        std::this_thread::yield();
#endif
    }

    // Claims slices of job `ticket` until none is left.  The counter carries the ticket in its
    // upper half, so a thread that still holds an older job's ticket claims nothing of this one.
    void
    work(uint64_t ticket, call_t call, void *ctx, unsigned slices) {
        for (;;) {
            uint64_t v = next_.load(std::memory_order_relaxed);
            for (;;) {
                if ((v >> 32) != ticket || static_cast<unsigned>(v) >= slices) return;
                if (next_.compare_exchange_weak(v, v + 1, std::memory_order_acq_rel, std::memory_order_relaxed)) break;
            }
            call(ctx, static_cast<unsigned>(v));
            done_.fetch_add(1, std::memory_order_release);
        }
    }

    void
    helperLoop() {
        uint64_t seen = 0;
        for (;;) {
            // a short poll first: the next request of a pair follows within a few hundred microseconds
            const auto until = std::chrono::steady_clock::now() + std::chrono::microseconds(300);
            bool fresh = false;
            while (!(fresh = generation_.load(std::memory_order_acquire) != seen) && std::chrono::steady_clock::now() < until)
                relax();
            call_t call;
            void *ctx;
            unsigned slices;
            {
                std::unique_lock<std::mutex> lock(mutex_);
                if (!fresh) wake_.wait(lock, [&] { return stop_ || generation_.load(std::memory_order_relaxed) != seen; });
                if (stop_) return;
                seen = generation_.load(std::memory_order_relaxed);
                call = call_;
                ctx = ctx_;
                slices = slices_;
            }
            work(seen, call, ctx, slices);
        }
    }

    std::mutex mutex_;
    std::condition_variable wake_;
    std::vector<std::thread> threads_;
    bool stop_ = false;
    std::atomic<bool> busy_{false};
    std::atomic<uint64_t> generation_{0}; // ticket of the newest job (32 bits in use)
    std::atomic<uint64_t> next_{0}; // ticket << 32 | next unclaimed slice
    std::atomic<unsigned> done_{0};
    call_t call_ = nullptr;
    void *ctx_ = nullptr;
    unsigned slices_ = 0;
};

} // namespace nixl_amd_hip

#endif
