// Host-only check of the box stage's parallel structure, meant to be built with a sanitizer (-fsanitize=thread or
// -fsanitize=address,undefined) together with the host library's sources: candidates of several images are grouped by class, the
// (image, class) groups are suppressed as tasks of the worker pool, largest first, exactly as YoloOutLayer::finish() issues them, and the
// result must equal the reference-shaped greedy loop (YoloOutLayer::nms, src/layers/MsnhYoloOutLayer.cpp:381-461) box for box.  Several
// caller threads do this at once, as the instances of a group do.
#include "Msnhnet/layers/MsnhLayers.h"
#include "Msnhnet/utils/MsnhTaskPool.h"
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

using namespace Msnhnet;

static std::vector<YoloBox> candidates(unsigned seed, int n, int classes)
{
    std::mt19937 rng(seed);
    std::uniform_real_distribution<float> pos(0.f, 608.f), ext(8.f, 180.f), score(0.5f, 1.f);
    std::vector<YoloBox> b(static_cast<size_t>(n));
    for (YoloBox &q : b)
    {
        q.xywhBox = Box::XYWHBox(pos(rng), pos(rng), ext(rng), ext(rng));
        q.conf = (rng() % 4 == 0) ? 1.f : score(rng);              // ties, as saturated objectness values give them
        q.bestClsConf = score(rng);
        q.bestClsIdx = static_cast<int>(rng() % static_cast<unsigned>(classes));
    }
    // a box of infinite extent (its IoU is NaN and never suppresses) and a class with a single member
    b[0].xywhBox.w = INFINITY;
    b[1].bestClsIdx = classes;
    // the layer passes them sorted by objectness * class score, descending
    std::stable_sort(b.begin(), b.end(), [](const YoloBox &x, const YoloBox &y) { return x.conf * x.bestClsConf > y.conf * y.bestClsConf; });
    return b;
}

static bool sameBox(const YoloBox &a, const YoloBox &b)
{
    return std::memcmp(&a.xywhBox, &b.xywhBox, sizeof(a.xywhBox)) == 0 && a.conf == b.conf && a.bestClsConf == b.bestClsConf && a.bestClsIdx == b.bestClsIdx;
}

static int oneBatch(unsigned seed, int images, int perImage)
{
    TaskPool &pool = TaskPool::instance();
    std::vector<std::vector<YoloBox>> cand(static_cast<size_t>(images)), out(static_cast<size_t>(images));
    std::vector<std::vector<std::vector<int>>> groups(static_cast<size_t>(images));
    pool.parallelFor(images, [&](int b) {
        cand[static_cast<size_t>(b)] = candidates(seed * 131u + static_cast<unsigned>(b), perImage, 6);
        groups[static_cast<size_t>(b)] = YoloOutLayer::groupByClass(cand[static_cast<size_t>(b)]);
    });
    std::vector<std::pair<int, int>> tasks;
    for (int b = 0; b < images; ++b)
        for (size_t g = 0; g < groups[static_cast<size_t>(b)].size(); ++g) tasks.emplace_back(b, static_cast<int>(g));
    std::stable_sort(tasks.begin(), tasks.end(), [&groups](const std::pair<int, int> &x, const std::pair<int, int> &y) {
        return groups[static_cast<size_t>(x.first)][static_cast<size_t>(x.second)].size() > groups[static_cast<size_t>(y.first)][static_cast<size_t>(y.second)].size();
    });
    pool.parallelFor(static_cast<int>(tasks.size()), [&](int t) {
        const size_t b = static_cast<size_t>(tasks[static_cast<size_t>(t)].first);
        YoloOutLayer::nmsClass(cand[b], groups[b][static_cast<size_t>(tasks[static_cast<size_t>(t)].second)], 0.45f);
    });
    pool.parallelFor(images, [&](int b) {
        for (const std::vector<int> &m : groups[static_cast<size_t>(b)])
            for (int j : m) out[static_cast<size_t>(b)].push_back(cand[static_cast<size_t>(b)][static_cast<size_t>(j)]);
    });
    int wrong = 0;
    for (int b = 0; b < images; ++b)
    {
        const std::vector<YoloBox> want = YoloOutLayer::nms(cand[static_cast<size_t>(b)], 0.45f, false);
        const std::vector<YoloBox> &got = out[static_cast<size_t>(b)];
        if (want.size() != got.size() || want.size() == cand[static_cast<size_t>(b)].size()) { ++wrong; continue; }     // (something must be suppressed)
        for (size_t i = 0; i < want.size(); ++i)
            if (!sameBox(want[i], got[i])) { ++wrong; break; }
        const std::vector<YoloBox> sorted = YoloOutLayer::nmsSorted(cand[static_cast<size_t>(b)], 0.45f);
        if (sorted.size() != want.size()) ++wrong;
    }
    return wrong;
}

int main()
{
    int wrong = oneBatch(1, 8, 400);
    std::atomic<int> wrongConcurrent{0};
    std::vector<std::thread> callers;
    for (unsigned c = 0; c < 3; ++c)
        callers.emplace_back([&wrongConcurrent, c] {
            for (unsigned rep = 0; rep < 4; ++rep) wrongConcurrent += oneBatch(10 + 7 * c + rep, 4, 300);
        });
    for (std::thread &t : callers) t.join();
    wrong += wrongConcurrent;
    if (wrong != 0) { std::printf("%d images differ from the reference-shaped loop\n", wrong); return 1; }
    std::printf("ok\n");
    return 0;
}
