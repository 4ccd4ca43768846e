// The helper-thread pool of the HIP backend's prepXfer, on the CPU: every slice of every job
// runs exactly once, jobs of different sizes follow each other without a helper of an earlier
// job touching a later one, a second caller is turned away while the pool is busy, and the
// pool shuts down with helpers asleep or polling.  make SANITIZE="-fsanitize=thread -g"
// builds it with the thread sanitizer.
//
// usage: worker_pool_check; prints "OK".
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>
#include "worker_pool.h"
#define REQUIRE(c) do { if (!(c)) { std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #c); std::exit(1);} } while (0)
using nixl_amd_hip::WorkerPool;
int main() {
    {
        WorkerPool pool(3);
        // many jobs back to back, slice counts that change: each slice once, sums right
        for (int job = 0; job < 2000; ++job) {
            const unsigned slices = 1 + static_cast<unsigned>(job % 37);
            std::vector<std::atomic<int>> hits(slices);
            std::vector<long> partial(slices, 0);
            REQUIRE(pool.run(slices, [&](unsigned s) {
                hits[s].fetch_add(1);
                long sum = 0;
                for (int i = 0; i < 1000; ++i) sum += (job + 1) * static_cast<long>(s + 1) + i;
                partial[s] = sum; // plain store: the pool's completion must publish it
            }));
            for (unsigned s = 0; s < slices; ++s) {
                REQUIRE(hits[s].load() == 1);
                REQUIRE(partial[s] == 1000L * (job + 1) * (s + 1) + 499500L);
            }
            if (job % 500 == 499) std::this_thread::sleep_for(std::chrono::milliseconds(2)); // let the helpers fall asleep
        }
        // a second caller while a job runs is turned away and does its work alone
        std::atomic<bool> inside{false}, release{false};
        std::atomic<int> refused{0};
        std::thread other([&] {
            while (!inside.load()) std::this_thread::yield();
            if (!pool.run(4, [&](unsigned) {})) refused.fetch_add(1);
            release.store(true);
        });
        REQUIRE(pool.run(8, [&](unsigned s) {
            if (s == 0) {
                inside.store(true);
                while (!release.load()) std::this_thread::yield();
            }
        }));
        other.join();
        REQUIRE(refused.load() == 1);
        // several callers competing: every job that was accepted ran all of its slices
        std::atomic<long> ran{0}, expected{0};
        std::vector<std::thread> callers;
        for (int t = 0; t < 4; ++t)
            callers.emplace_back([&] {
                for (int job = 0; job < 300; ++job) {
                    const bool taken = pool.run(16, [&](unsigned) { ran.fetch_add(1); });
                    if (taken) expected.fetch_add(16);
                }
            });
        for (auto &c : callers) c.join();
        REQUIRE(ran.load() == expected.load() && expected.load() > 0);
    } // destructor with helpers polling
    {
        WorkerPool pool(2);
        std::this_thread::sleep_for(std::chrono::milliseconds(3)); // destructor with helpers asleep
    }
    {
        WorkerPool none(0); // no helpers: the caller does everything
        int count = 0;
        REQUIRE(none.run(5, [&](unsigned) { ++count; }));
        REQUIRE(count == 5);
    }
    std::puts("OK");
}
