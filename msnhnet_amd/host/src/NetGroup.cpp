#include "Msnhnet/net/MsnhNetGroup.h"
#include "Msnhnet/layers/MsnhLayers.h"
#include "Msnhnet/core/MsnhPlan.h"
#include <cstdlib>

namespace Msnhnet
{
NetGroup::NetGroup(const std::string &msnhnetPath, const std::string &msnhbinPath, int instances, int depth)
{
    if (instances < 1 || instances > 16) MSNH_THROW("NetGroup: 1 to 16 instances");
    for (int i = 0; i < instances; ++i)
    {
        std::unique_ptr<Lane> lane(new Lane());
        lane->net.reset(new NetBuilder());
        lane->net->buildNetFromMsnhNet(msnhnetPath);
        lane->net->loadWeightsFromMsnhBin(msnhbinPath);
        if (instances > 1)
        {
            // one stream per instance: see YoloOutLayer::copyOnForwardStream
            Network *net = lane->net->getNet();
            if (!net->layers.empty() && net->layers.back()->type() == LayerType::YOLO_OUT)
                static_cast<YoloOutLayer *>(net->layers.back())->copyOnForwardStream = true;
        }
        _lanes.push_back(std::move(lane));
    }
    // One packed copy of the convolution and connected weights for all instances: the others drop their own and read the first
    // instance's (identical bytes: same weights file, same plan, same tile choices).  A third of the weight footprint against the
    // memory-side cache, +0.7 % images/s for YOLOv3-608 with three instances.  The lane threads are joined before any instance
    // is destroyed, and a view frees nothing.
    {
        Plan &p0 = *_lanes[0]->net->getNet()->plan;
        for (size_t i = 1; i < _lanes.size(); ++i)
        {
            Plan &pi = *_lanes[i]->net->getNet()->plan;
            if (pi.ops.size() != p0.ops.size()) continue;
            for (size_t j = 0; j < pi.ops.size(); ++j)
            {
                PlanOp &mine = pi.ops[j];
                const PlanOp &first = p0.ops[j];
                if (mine.dead || first.dead || mine.kind != first.kind || mine.algo != first.algo || mine.wDev.ptr() == nullptr ||
                    mine.wDev.bytes() != first.wDev.bytes() || mine.wDev2.bytes() != first.wDev2.bytes())
                    continue;
                mine.wDev.aliasOf(first.wDev);
                if (first.wDev2.ptr()) mine.wDev2.aliasOf(first.wDev2);
            }
        }
    }
    Network *n = _lanes[0]->net->getNet();
    _detect = !n->layers.empty() && n->layers.back()->type() == LayerType::YOLO_OUT;
    _depth = _detect ? std::max(1, std::min(depth, 2)) : 1;
    try
    {
        for (std::unique_ptr<Lane> &lane : _lanes)
        {
            Lane *l = lane.get();
            l->thread = std::thread([this, l] { drive(*l); });
        }
    }
    catch (...)
    {
        stop();                                             // a thread that could not be started: end the ones that were
        throw;
    }
}

NetGroup::~NetGroup() { stop(); }

void NetGroup::stop()
{
    for (std::unique_ptr<Lane> &lane : _lanes)
    {
        {
            std::lock_guard<std::mutex> lk(lane->m);
            lane->in.push_back({2, nullptr, false});
        }
        lane->cvIn.notify_one();
    }
    for (std::unique_ptr<Lane> &lane : _lanes)
        if (lane->thread.joinable()) lane->thread.join();
}

// The instance's thread: enqueue the next batch, and once `depth` are in flight fetch the oldest.
void NetGroup::drive(Lane &lane)
{
    int inFlight = 0;
    const auto fetchOne = [&] {
        Result r;
        try
        {
            if (_detect) r.boxes = lane.net->fetchYolo();
            else r.logits = lane.net->fetchClassify();
        }
        catch (...) { r.error = std::current_exception(); }
        --inFlight;
        {
            std::lock_guard<std::mutex> lk(lane.m);
            lane.out.push_back(std::move(r));
        }
        lane.cvOut.notify_one();
    };
    for (;;)
    {
        Job job;
        {
            std::unique_lock<std::mutex> lk(lane.m);
            lane.cvIn.wait(lk, [&] { return !lane.in.empty(); });
            job = lane.in.front();
            lane.in.pop_front();
        }
        if (job.kind != 0)
        {
            while (inFlight > 0) fetchOne();
            if (job.kind == 2) return;
            continue;
        }
        try
        {
            if (job.fail) MSNH_THROW("NetGroup: enqueue failure requested by MSNH_GROUP_FAIL_ENQUEUE");
            lane.net->enqueueForward(job.input);
            ++inFlight;
        }
        catch (...)
        {
            // the batch has no result of its own: its place in the order carries the error.  The results of the batches
            // enqueued before it come first, so that every fetch still returns what belongs to its own submission.
            Result r;
            r.error = std::current_exception();
            while (inFlight > 0) fetchOne();
            {
                std::lock_guard<std::mutex> lk(lane.m);
                lane.out.push_back(std::move(r));
            }
            lane.cvOut.notify_one();
            continue;
        }
        if (inFlight == _depth) fetchOne();
    }
}

void NetGroup::prime(const float *deviceInput)
{
    if (outstanding() != 0) MSNH_THROW("NetGroup: fetch the outstanding results before prime()");
    for (std::unique_ptr<Lane> &lane : _lanes)
    {
        lane->net->enqueueForward(deviceInput);
        if (_detect) lane->net->fetchYolo();
        else lane->net->fetchClassify();
    }
}

void NetGroup::submit(const float *deviceInput)
{
    Lane &lane = *_lanes[static_cast<size_t>(_submitted % static_cast<long long>(_lanes.size()))];
    {
        std::lock_guard<std::mutex> lk(lane.m);
        // (tests) MSNH_GROUP_FAIL_ENQUEUE = n: the n-th submission of the group fails when its instance tries to enqueue it
        const char *failAt = std::getenv("MSNH_GROUP_FAIL_ENQUEUE");
        lane.in.push_back({0, deviceInput, failAt != nullptr && std::atoll(failAt) == _submitted});
    }
    lane.cvIn.notify_one();
    ++lane.submitted;
    ++_submitted;
}

void NetGroup::flush()
{
    for (std::unique_ptr<Lane> &lane : _lanes)
    {
        {
            std::lock_guard<std::mutex> lk(lane->m);
            lane->in.push_back({1, nullptr, false});
        }
        lane->cvIn.notify_one();
    }
}

NetGroup::Result NetGroup::take()
{
    if (outstanding() <= 0) MSNH_THROW("NetGroup: nothing outstanding");
    Lane &lane = *_lanes[static_cast<size_t>(_fetched % static_cast<long long>(_lanes.size()))];
    Result r;
    {
        std::unique_lock<std::mutex> lk(lane.m);
        // The instance hands out its j-th result when batch j + depth - 1 arrives.  If that batch has not been submitted, the result
        // asked for would wait for it for ever: make the instance fetch what it holds.
        if (lane.submitted < lane.taken + _depth)
        {
            lane.in.push_back({1, nullptr, false});
            lane.cvIn.notify_one();
        }
        lane.cvOut.wait(lk, [&] { return !lane.out.empty(); });
        r = std::move(lane.out.front());
        lane.out.pop_front();
    }
    ++lane.taken;
    ++_fetched;
    if (r.error) std::rethrow_exception(r.error);
    return r;
}

std::vector<std::vector<YoloBox>> NetGroup::fetchYolo()
{
    if (!_detect) MSNH_THROW("not a yolo net");
    return take().boxes;
}

std::vector<float> NetGroup::fetchClassify()
{
    if (_detect) MSNH_THROW("NetGroup: a detector's results are fetched with fetchYolo");
    return take().logits;
}
}
