// Host-only check of the worker pool behind the box stage: every index runs exactly once, exceptions reach the caller, the pool
// survives many short jobs, and idle workers sleep (no CPU time is spent between jobs).
#include "Msnhnet/utils/MsnhTaskPool.h"
#include <atomic>
#include <chrono>
#include <cstdio>
#include <ctime>
#include <stdexcept>
#include <thread>
#include <vector>

static double cpuSeconds()
{
    timespec ts;
    clock_gettime(CLOCK_PROCESS_CPUTIME_ID, &ts);
    return ts.tv_sec + ts.tv_nsec * 1e-9;
}

int main()
{
    Msnhnet::TaskPool &pool = Msnhnet::TaskPool::instance();
    if (pool.threads() < 1) { std::printf("no threads\n"); return 1; }
    for (int n : {0, 1, 2, 7, 64, 1000})
    {
        std::vector<std::atomic<int>> hits(static_cast<size_t>(n));
        for (auto &h : hits) h = 0;
        pool.parallelFor(n, [&](int i) { ++hits[static_cast<size_t>(i)]; });
        for (int i = 0; i < n; ++i)
            if (hits[static_cast<size_t>(i)] != 1) { std::printf("n=%d: index %d ran %d times\n", n, i, hits[static_cast<size_t>(i)].load()); return 1; }
    }
    // many short jobs back to back, as the box stage issues them
    std::atomic<long long> sum{0};
    for (int rep = 0; rep < 2000; ++rep) pool.parallelFor(8, [&](int i) { sum += i; });
    if (sum != 2000LL * 28) { std::printf("sum %lld\n", sum.load()); return 1; }
    // an exception in one task reaches the caller, the other tasks still run, and the pool works afterwards
    std::atomic<int> ran{0};
    bool caught = false;
    try { pool.parallelFor(32, [&](int i) { ++ran; if (i == 5) throw std::runtime_error("task 5"); }); }
    catch (const std::runtime_error &e) { caught = std::string(e.what()) == "task 5"; }
    if (!caught || ran != 32) { std::printf("exception: caught %d ran %d\n", int(caught), ran.load()); return 1; }
    ran = 0;
    pool.parallelFor(16, [&](int) { ++ran; });
    if (ran != 16) { std::printf("after exception: %d\n", ran.load()); return 1; }
    // several callers at once (the instances of a group): every job completes with every index once
    {
        std::vector<std::thread> callers;
        std::atomic<int> wrong{0};
        for (int c = 0; c < 4; ++c)
            callers.emplace_back([&, c] {
                for (int rep = 0; rep < 300; ++rep)
                {
                    const int n = 5 + (rep + c) % 40;
                    std::vector<std::atomic<int>> hits(static_cast<size_t>(n));
                    for (auto &h : hits) h = 0;
                    pool.parallelFor(n, [&](int i) { ++hits[static_cast<size_t>(i)]; });
                    for (int i = 0; i < n; ++i)
                        if (hits[static_cast<size_t>(i)] != 1) ++wrong;
                }
            });
        for (std::thread &t : callers) t.join();
        if (wrong != 0) { std::printf("concurrent callers: %d wrong counts\n", wrong.load()); return 1; }
    }
    // idle workers sleep
    const double c0 = cpuSeconds();
    std::this_thread::sleep_for(std::chrono::milliseconds(300));
    const double idle = cpuSeconds() - c0;
    if (idle > 0.03) { std::printf("idle pool used %.3f s of CPU in 0.3 s\n", idle); return 1; }
    std::printf("threads %d, idle cpu %.4f s\nok\n", pool.threads(), idle);
    return 0;
}
