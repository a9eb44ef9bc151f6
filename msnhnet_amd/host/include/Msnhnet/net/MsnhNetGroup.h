#ifndef MSNH_NET_GROUP_H
#define MSNH_NET_GROUP_H
#include <condition_variable>
#include <deque>
#include <exception>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>
#include "Msnhnet/net/MsnhNetBuilder.h"

namespace Msnhnet
{
// Several instances of one network on one GPU, fed round-robin: the throughput arrangement for serving.
//
// A forward is a chain of dependent launches; the launch gaps, prologues and write bursts of its kernels leave much of the device idle
// and nothing in the same stream can fill them.  Another forward on another stream can.  Each instance is a NetBuilder of its own (stream,
// activation arena, captured graph; the per-layer tile choices and the packed weights of the first are used by the others, so all instances run
// the same kernels), driven by its own host thread, which enqueues a batch and fetches the result of an earlier one so that `depth`
// batches per instance are in flight.  Results come back in submission order.  No counterpart in the reference, whose callers would
// create several NetBuilder objects and threads themselves.
class NetGroup
{
public:
    // depth: batches in flight per instance (detectors: 1 or 2; a classifier's result is read from its output tensor, one at a time)
    NetGroup(const std::string &msnhnetPath, const std::string &msnhbinPath, int instances, int depth);
    ~NetGroup();
    NetGroup(const NetGroup &) = delete;
    NetGroup &operator=(const NetGroup &) = delete;

    int instances() const { return static_cast<int>(_lanes.size()); }
    int depth() const { return _depth; }
    bool isDetector() const { return _detect; }
    NetBuilder &instance(int i) { return *_lanes.at(static_cast<size_t>(i))->net; }

    // One forward of the float32 NCHW batch at deviceInput on every instance, one after the other on the calling thread: every
    // instance's input buffer then holds that batch (submit(nullptr) runs on it), its graph is captured and its buffers exist.
    void prime(const float *deviceInput);
    // Hands the next batch to the next instance.  deviceInput: device pointer to the batch (copied into the instance's input buffer on
    // its stream; must stay valid until the result has been fetched) or nullptr to run on what that buffer holds.
    void submit(const float *deviceInput);
    // Makes every instance fetch what it still holds in flight now (an instance otherwise keeps depth - 1 results back until more work
    // comes or one of them is asked for).
    void flush();
    // The oldest outstanding result; blocks until it is there.  An exception thrown inside an instance's thread is rethrown here.
    // prime, submit, flush and the fetches are for one calling thread (or callers that serialise them).
    std::vector<std::vector<YoloBox>> fetchYolo();
    std::vector<float> fetchClassify();
    long long outstanding() const { return _submitted - _fetched; }

private:
    struct Result
    {
        std::vector<std::vector<YoloBox>> boxes;
        std::vector<float> logits;
        std::exception_ptr error;
    };
    struct Job { int kind; const float *input; bool fail; };          // kind 0 = forward, 1 = flush, 2 = stop; fail: see submit()
    struct Lane
    {
        std::unique_ptr<NetBuilder> net;
        std::thread thread;
        std::mutex m;
        std::condition_variable cvIn, cvOut;
        std::deque<Job> in;
        std::deque<Result> out;
        long long submitted = 0, taken = 0;                // by the caller's thread only
    };
    void drive(Lane &lane);
    void stop();
    Result take();
    std::vector<std::unique_ptr<Lane>> _lanes;
    int _depth = 1;
    bool _detect = false;
    long long _submitted = 0, _fetched = 0;
};
}
#endif
