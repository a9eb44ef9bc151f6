#ifndef MSNH_TASK_POOL_H
#define MSNH_TASK_POOL_H
#include <atomic>
#include <condition_variable>
#include <cstdint>
#include <exception>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace Msnhnet
{
// Host worker threads for the short parallel phases between two forwards (box decoding, per-class suppression).  Idle workers
// sleep on a condition variable: an OpenMP team that spins between parallel regions keeps every core of the process's CPU
// allowance busy, and a container that enforces the allowance per 100 ms period then stops the whole process -- the thread that
// feeds the GPU included -- for several milliseconds of every period.
class TaskPool
{
public:
    static TaskPool &instance();
    // fn(i) for every i in [0, n), indices handed out one at a time in ascending order (big tasks first: sort before calling);
    // the caller works along and returns when every index is done -- it waits for tasks, not for workers: a worker that wakes up
    // late finds nothing left and goes back to sleep.  The first exception thrown by fn is rethrown here.  Calls from several
    // threads run side by side (the instances of a NetGroup each have a host stage): a worker takes indices of whichever job has
    // some left.
    void parallelFor(int n, const std::function<void(int)> &fn);
    int threads() const { return static_cast<int>(_threads.size()) + 1; }
    ~TaskPool();

private:
    TaskPool();
    struct Job
    {
        const std::function<void(int)> *fn;
        int n;
        std::atomic<int> next{0}, done{0};
        std::exception_ptr error;
    };
    void worker();
    void drain(Job &job);
    std::vector<std::thread> _threads;
    std::mutex _m;
    std::condition_variable _cvWork, _cvDone;
    std::vector<std::shared_ptr<Job>> _jobs;        // jobs that may still have indices to hand out
    bool _stop = false;
};
}
#endif
