#include "Msnhnet/utils/MsnhTaskPool.h"
#include <algorithm>
#include <cstdlib>

namespace Msnhnet
{
TaskPool &TaskPool::instance()
{
    static TaskPool pool;
    return pool;
}

// Thread count: MSNH_HOST_THREADS, else OMP_NUM_THREADS (what a deployment that sizes its CPU share already sets), else the
// hardware's, capped at 16 -- a batch has a few dozen tasks worth a thread each.
TaskPool::TaskPool()
{
    int want = 0;
    for (const char *name : {"MSNH_HOST_THREADS", "OMP_NUM_THREADS"})
        if (const char *v = std::getenv(name))
        {
            want = std::atoi(v);
            if (want > 0) break;
        }
    if (want <= 0) want = static_cast<int>(std::thread::hardware_concurrency());
    want = std::max(1, std::min(want, 16));
    for (int i = 1; i < want; ++i) _threads.emplace_back([this] { worker(); });
}

TaskPool::~TaskPool()
{
    {
        std::lock_guard<std::mutex> lk(_m);
        _stop = true;
    }
    _cvWork.notify_all();
    for (std::thread &t : _threads) t.join();
}

void TaskPool::drain(Job &job)
{
    for (;;)
    {
        const int i = job.next.fetch_add(1, std::memory_order_relaxed);
        if (i >= job.n) return;
        try { (*job.fn)(i); }
        catch (...)
        {
            std::lock_guard<std::mutex> lk(_m);
            if (!job.error) job.error = std::current_exception();
        }
        if (job.done.fetch_add(1, std::memory_order_acq_rel) + 1 == job.n)
        {
            std::lock_guard<std::mutex> lk(_m);
            _cvDone.notify_all();
        }
    }
}

void TaskPool::worker()
{
    std::unique_lock<std::mutex> lk(_m);
    for (;;)
    {
        std::shared_ptr<Job> job;
        _cvWork.wait(lk, [&] {
            if (_stop) return true;
            for (const std::shared_ptr<Job> &j : _jobs)
                if (j->next.load(std::memory_order_relaxed) < j->n) { job = j; return true; }
            return false;
        });
        if (_stop) return;
        lk.unlock();
        drain(*job);
        job.reset();
        lk.lock();
    }
}

void TaskPool::parallelFor(int n, const std::function<void(int)> &fn)
{
    if (n <= 0) return;
    if (n == 1 || _threads.empty())
    {
        for (int i = 0; i < n; ++i) fn(i);
        return;
    }
    std::shared_ptr<Job> job = std::make_shared<Job>();
    job->fn = &fn;
    job->n = n;
    {
        std::lock_guard<std::mutex> lk(_m);
        _jobs.push_back(job);
    }
    // as many workers as there are tasks beside the caller's
    const int wake = std::min(n - 1, static_cast<int>(_threads.size()));
    if (wake == static_cast<int>(_threads.size())) _cvWork.notify_all();
    else for (int i = 0; i < wake; ++i) _cvWork.notify_one();
    drain(*job);
    std::unique_lock<std::mutex> lk(_m);
    _cvDone.wait(lk, [&] { return job->done.load(std::memory_order_acquire) == n; });
    for (size_t i = 0; i < _jobs.size(); ++i)
        if (_jobs[i] == job) { _jobs.erase(_jobs.begin() + static_cast<long>(i)); break; }
    if (job->error) std::rethrow_exception(job->error);
}
}
