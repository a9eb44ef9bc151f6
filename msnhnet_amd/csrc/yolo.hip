// YOLO v3/v4/v5 head decode fused with the [anchor][channel][pixel] -> [anchor][pixel][channel] reordering and
// the objectness threshold.  The NHWC head tensor already stores the (5+classes) values of one anchor of
// one pixel contiguously, so both the read and the write of a wavefront are contiguous runs.
#include "common.hpp"
#include <mutex>

namespace msnh {

struct Anchors { float v[6]; };

// A workgroup decodes CHUNK consecutive values of one image.  Entries whose objectness passes the threshold are
// first collected in LDS; one global atomic per workgroup then reserves their slots in the image's candidate list
// (one atomic per candidate on a single counter would serialise half of all cells with the benchmark weights).
constexpr int YOLO_CHUNK = 256 * 8;

// The 5 + classes logistics per cell are what the kernel computes most of (logisticF: hardware exp2 and
// reciprocal); box width and height keep expf.
// One decoded value: m = index inside the cell's 5 + classes values, (px, py) = cell, a = anchor.
template <bool V5>
__device__ __forceinline__ float yoloDecodeOne(float v, int m, int px, int py, int a, const Anchors &an, float ratio)
{
    if (V5)
    {
        // yolov5: centre (2s - 0.5 + cell) * ratio, size anchor * (2s)^2, s = logistic (src/layers/MsnhYoloLayer.cpp:250-296)
        const float s2 = 2.f * logisticF(v);
        if (m == 0) return (s2 - 0.5f + static_cast<float>(px)) * ratio;
        if (m == 1) return (s2 - 0.5f + static_cast<float>(py)) * ratio;
        if (m == 2) return an.v[(2 * a) % 6] * (s2 * s2);
        if (m == 3) return an.v[(2 * a + 1) % 6] * (s2 * s2);
        return 0.5f * s2;
    }
    if (m == 0) return (logisticF(v) + static_cast<float>(px)) * ratio;
    if (m == 1) return (logisticF(v) + static_cast<float>(py)) * ratio;
    if (m == 2) return an.v[(2 * a) % 6] * expf(v);
    if (m == 3) return an.v[(2 * a + 1) % 6] * expf(v);
    return logisticF(v);
}

template <typename T, bool V5>
__global__ __launch_bounds__(256) void yoloDecodeKernel(const T *__restrict__ x, int xLd, float xMul, Anchors an, float ratio,
                                                        float *__restrict__ decoded, long long decStride, float confThresh, int *__restrict__ candIdx,
                                                        int candCap, int candBase, int *__restrict__ candCnt, int W, int HW, int per,
                                                        int perImage)
{
    __shared__ int found[YOLO_CHUNK / 6 + 8];
    __shared__ int nFound, base;
    const int b = blockIdx.y;
    if (threadIdx.x == 0) nFound = 0;
    __syncthreads();
    const int start = blockIdx.x * YOLO_CHUNK;
    // idx = (a*HW + p)*per + m inside the image; a thread's idx advances by 256 per step, so (m, p, a) are carried
    // along with adds and compares instead of being recovered by three divisions per element
    int idx = start + threadIdx.x;
    int m = idx % per;
    int cell = idx / per;
    int p = cell % HW;
    int a = cell / HW;
    int px = p % W, py = p / W;
    const int stepCell = 256 / per, stepM = 256 % per;
    const int stepY = stepCell / W, stepX = stepCell % W;
    const T *xb = x + static_cast<size_t>(b) * HW * xLd;
    float *db = decoded + static_cast<size_t>(b) * decStride;
#pragma unroll 4
    for (int k = 0; k < YOLO_CHUNK / 256; ++k)
    {
        const bool live = idx < perImage;          // predicate, not an exit: the unrolled loads can then be issued together
        const float v = live ? xMul * toF(xb[static_cast<size_t>(p) * xLd + a * per + m]) : 0.f;
        const float r = yoloDecodeOne<V5>(v, m, px, py, a, an, ratio);
        if (live) db[idx] = r;
        if (live && m == 4 && candIdx != nullptr && r > confThresh) found[atomicAdd(&nFound, 1)] = candBase + a * HW + p;
        idx += 256;
        m += stepM;
        int dc = stepCell;
        if (m >= per) { m -= per; ++dc; }
        // advance the pixel by dc cells: dc = stepCell or stepCell + 1
        px += stepX + (dc - stepCell);
        py += stepY;
        p += dc;
        if (px >= W) { px -= W; ++py; }
        if (px >= W) { px -= W; ++py; }
        if (p >= HW)
        {
            do { p -= HW; ++a; } while (p >= HW);
            py = p / W;
            px = p - py * W;
        }
    }
    __syncthreads();
    if (candIdx == nullptr || nFound == 0) return;
    if (threadIdx.x == 0) base = atomicAdd(candCnt + b, nFound);
    __syncthreads();
    for (int i = threadIdx.x; i < nFound; i += 256)
        if (base + i < candCap) candIdx[static_cast<size_t>(b) * candCap + base + i] = found[i];
}

// Objectness only: the candidate list of a head without materialising its decoded tensor.  One lane per cell
// (anchor, pixel); same logistic and same threshold test as the full decode, so the list is identical.
template <typename T>
__global__ __launch_bounds__(256) void yoloScanKernel(const T *__restrict__ x, int xLd, float xMul, float confThresh, int *__restrict__ candIdx,
                                                      int candCap, int candBase, int *__restrict__ candCnt, int HW, int per)
{
    __shared__ int found[256];
    __shared__ int nFound, base;
    const int b = blockIdx.y;
    if (threadIdx.x == 0) nFound = 0;
    __syncthreads();
    const int cell = blockIdx.x * 256 + threadIdx.x;             // a * HW + p
    if (cell < 3 * HW)
    {
        const int a = cell / HW, p = cell - a * HW;
        const float v = xMul * toF(x[(static_cast<size_t>(b) * HW + p) * xLd + a * per + 4]);
        if (logisticF(v) > confThresh) found[atomicAdd(&nFound, 1)] = candBase + cell;
    }
    __syncthreads();
    if (nFound == 0) return;
    if (threadIdx.x == 0) base = atomicAdd(candCnt + b, nFound);
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < nFound && base + static_cast<int>(threadIdx.x) < candCap)
        candIdx[static_cast<size_t>(b) * candCap + base + threadIdx.x] = found[threadIdx.x];
}

// Decodes the rows of the listed candidates that belong to this head into their places of the decoded buffer and, when
// `rows` is given, writes the candidate's compact row { x, y, w, h, objectness, best class score, best class index, cell }
// (what yoloGatherKernel derives from the decoded row).  Sixteen lanes per candidate, four candidates per wavefront (the
// kernel lives on the latency of its dependent loads, so candidates in flight count, not lanes per candidate): lane s of a
// group decodes values s, s + 16, ...; the best class is the first maximum in channel order, found with a reduction on
// (score, index) over the group's lanes.
template <typename T, bool V5>
__global__ __launch_bounds__(256) void yoloRowsKernel(const T *__restrict__ x, int xLd, float xMul, Anchors an, float ratio,
                                                      float *__restrict__ decoded, long long decStride, const int *__restrict__ candIdx, int candCap,
                                                      int candBase, const int *__restrict__ candCnt, float *__restrict__ rows, int W, int HW, int per)
{
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int sub = lane & 15;                                   // lane inside the candidate's group
    const int groupLane0 = lane & 48;                            // first lane of the group
    const int group = threadIdx.x >> 4;                          // 16 groups per workgroup
    int n = candCnt[b];
    n = n < candCap ? n : candCap;
    for (int k = blockIdx.x * 16 + group; k < n; k += gridDim.x * 16)
    {
        const int cellG = candIdx[static_cast<size_t>(b) * candCap + k];
        const int cell = cellG - candBase;
        if (cell < 0 || cell >= 3 * HW) continue;                // another head's candidate
        const int a = cell / HW, p = cell - a * HW;
        const int py = p / W, px = p - py * W;
        const T *xr = x + (static_cast<size_t>(b) * HW + p) * xLd + a * per;
        float *dr = decoded + static_cast<size_t>(b) * decStride + static_cast<size_t>(cell) * per;
        float first = 0.f;                                       // this lane's value of m = sub (box and objectness live in lanes 0..4 of the group)
        float bv = -3.402823466e38f * 2.f;                       // -inf: NaN scores are never selected
        int bi = 0x7fffffff;
        for (int m = sub; m < per; m += 16)
        {
            const float v = yoloDecodeOne<V5>(xMul * toF(xr[m]), m, px, py, a, an, ratio);
            if (decoded != nullptr) dr[m] = v;
            if (m == sub) first = v;
            if (m >= 5 && v > bv) { bv = v; bi = m - 5; }
        }
        if (rows == nullptr) continue;
#pragma unroll
        for (int off = 8; off > 0; off >>= 1)
        {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        // a NaN score of class 0 absorbs the sequential scan of the reference (nothing compares greater than it)
        const float c0v = __shfl(first, groupLane0 + 5, 64);
        if (c0v != c0v) { bv = c0v; bi = 0; }
        if (bi == 0x7fffffff) bi = 0;
        float *o = rows + (static_cast<size_t>(b) * candCap + k) * 8;
        if (sub < 5) o[sub] = first;
        else if (sub == 5) o[5] = bv;
        else if (sub == 6) o[6] = static_cast<float>(bi);
        else if (sub == 7) o[7] = static_cast<float>(cellG);
    }
}

// ---- per-class greedy NMS on the device (src/layers/MsnhYoloOutLayer.cpp:175-194 sort, :381-461 nms) -------------------
// One workgroup per (class, image).  The reference sorts all candidates of an image by objectness * best class score
// (descending; here ties keep cell order), visits the classes in the order of their first appearance in that list and,
// inside a class, repeatedly picks the highest objectness (first of the list on ties) and erases what overlaps it by more
// than the threshold.  Per class that is: order the members by (objectness, score, cell) and keep a member unless one kept
// before it overlaps it.  The workgroup collects the members of its class, ranks them by counting, runs the greedy pass in
// its first wavefront (lanes test the later members against the pick in parallel) and appends one record per kept box:
// the compact row, the (score, cell) of the class's first member in the global list -- the host orders classes by it --,
// the pick order inside the class and the image index.
constexpr int NMS_CAP = 1024;           // members of one class in one image; more -> the image is flagged for the caller

__device__ __forceinline__ unsigned orderedBits(float f)
{
    const unsigned u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Box::iou(candidate, pick) > thr (include/Msnhnet/utils/MsnhTypes.h:123-140: corners from centre and size, "+ 1" extents,
// min / max spelled out so that NaN behaves alike), decided without the division wherever the product form is clear of
// rounding: inter / uni > thr is certain when inter > (thr * uni)(1 + 1e-5) and impossible when inter < (thr * uni)(1 - 1e-5)
// for positive finite operands; everything else (and every NaN / infinity / zero-union case) takes the division itself.
__device__ __forceinline__ bool iouAbove(float kx1, float ky1, float kx2, float ky2, float karea, float jx1, float jy1, float jx2, float jy2,
                                         float jarea, float thr)
{
#pragma clang fp contract(off)
    const float ix2 = (kx2 < jx2) ? kx2 : jx2;
    const float ix1 = (jx1 < kx1) ? kx1 : jx1;
    const float iy2 = (ky2 < jy2) ? ky2 : jy2;
    const float iy1 = (jy1 < ky1) ? ky1 : jy1;
    const float iw = ix2 - ix1 + 1;
    const float ih = iy2 - iy1 + 1;
    const float inter = (iw < 0 ? 0 : iw) * (ih < 0 ? 0 : ih);
    const float uni = jarea + karea - inter;
    if (thr >= 0.f && thr <= 1e3f && uni > 1e-20f && uni < 1e30f && inter < 1e30f)
    {
        if (inter == 0.f) return false;
        const float p = thr * uni;
        if (p > 1e-20f)
        {
            if (inter > p * 1.00001f) return true;
            if (inter < p * 0.99999f) return false;
        }
    }
    return 1.f * inter / uni > thr;
}

__global__ __launch_bounds__(256) void yoloNmsKernel(const float *__restrict__ rows, int candCap, const int *__restrict__ candCnt, float thr,
                                                     float *__restrict__ kept, int keptCap, int *__restrict__ keptCnt, int *__restrict__ bigCnt,
                                                     int *__restrict__ wsUsed)
{
#pragma clang fp contract(off)
    __shared__ unsigned long long keyA[NMS_CAP];
    __shared__ unsigned keyB[NMS_CAP];
    __shared__ int member[NMS_CAP], sorted[NMS_CAP];
    __shared__ float x1[NMS_CAP], y1[NMS_CAP], x2[NMS_CAP], y2[NMS_CAP], area[NMS_CAP];
    __shared__ unsigned short pickOf[NMS_CAP];
    __shared__ unsigned char gone[NMS_CAP];
    __shared__ unsigned long long top;
    __shared__ int nMem, bad, base;
    const int cls = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    int n = candCnt[b];
    n = n < candCap ? n : candCap;
    const float *r = rows + static_cast<size_t>(b) * candCap * 8;
    if (tid == 0) { nMem = 0; bad = 0; top = 0ull; }
    if (wsUsed != nullptr && cls == 0 && tid == 0) wsUsed[b] = 0;       // yoloNmsBigKernel's cursor into the image's workspace
    __syncthreads();
    for (int k = tid; k < n; k += 256)
        if (static_cast<int>(r[static_cast<size_t>(k) * 8 + 6]) == cls)
        {
            const int slot = atomicAdd(&nMem, 1);
            if (slot < NMS_CAP) member[slot] = k;
        }
    __syncthreads();
    const int m = nMem;
    if (bigCnt != nullptr && tid == 0) bigCnt[b * gridDim.x + cls] = m;
    if (m == 0) return;
    if (m > NMS_CAP)
    {
        if (bigCnt == nullptr && tid == 0) atomicOr(&keptCnt[1 + b], 1);    // (else yoloNmsBigKernel takes the class)
        return;
    }
    for (int i = tid; i < m; i += 256)
    {
        const float *q = r + static_cast<size_t>(member[i]) * 8;
        const float conf = q[4];
        const float score = conf * q[5];
        if (!(score == score) || !(conf == conf)) bad = 1;
        const unsigned sb = orderedBits(score), cell = ~static_cast<unsigned>(q[7]);
        keyA[i] = (static_cast<unsigned long long>(orderedBits(conf)) << 32) | sb;
        keyB[i] = cell;
        atomicMax(&top, (static_cast<unsigned long long>(sb) << 32) | cell);
    }
    __syncthreads();
    if (bad)
    {
        if (tid == 0) atomicOr(&keptCnt[1 + b], 2);    // the order of NaN scores is whatever the caller's sort makes of them
        return;
    }
    for (int i = tid; i < m; i += 256)
    {
        const unsigned long long a = keyA[i];
        const unsigned bk = keyB[i];
        int rank = 0;
        for (int j = 0; j < m; ++j)
        {
            const unsigned long long oa = keyA[j];
            rank += (oa > a || (oa == a && keyB[j] > bk)) ? 1 : 0;
        }
        const float *q = r + static_cast<size_t>(member[i]) * 8;
        const float bx = q[0], by = q[1], bw = q[2], bh = q[3];
        const float ax1 = bx - bw / 2.f, ax2 = bx + bw / 2.f, ay1 = by - bh / 2.f, ay2 = by + bh / 2.f;
        sorted[rank] = member[i];
        x1[rank] = ax1; x2[rank] = ax2; y1[rank] = ay1; y2[rank] = ay2;
        area[rank] = (ax2 - ax1 + 1) * (ay2 - ay1 + 1);
        gone[rank] = 0;
    }
    __syncthreads();
    {
        volatile unsigned char *g = gone;           // written by other threads between two reads; the barrier orders them
        int picks = 0;
        for (int i = 0; i < m; ++i)
        {
            if (g[i]) continue;                          // same answer in every thread
            const float kx1 = x1[i], ky1 = y1[i], kx2 = x2[i], ky2 = y2[i], karea = area[i];
            for (int j = i + 1 + tid; j < m; j += 256)
                if (!g[j] && iouAbove(kx1, ky1, kx2, ky2, karea, x1[j], y1[j], x2[j], y2[j], area[j], thr)) g[j] = 1;
            if (tid == 0) pickOf[i] = static_cast<unsigned short>(picks);
            ++picks;
            __syncthreads();
        }
        if (tid == 0) base = atomicAdd(&keptCnt[0], picks);
    }
    __syncthreads();
    const unsigned long long t = top;
    const float topScore = __uint_as_float((static_cast<unsigned>(t >> 32) & 0x80000000u) ? (static_cast<unsigned>(t >> 32) & 0x7fffffffu) : ~static_cast<unsigned>(t >> 32));
    const float topCell = static_cast<float>(~static_cast<unsigned>(t & 0xffffffffull));
    for (int i = tid; i < m; i += 256)
    {
        if (gone[i]) continue;
        const int pos = base + pickOf[i];
        if (pos >= keptCap) continue;                    // (cannot happen with keptCap >= batch * candCap)
        const float4 *q = reinterpret_cast<const float4 *>(r + static_cast<size_t>(sorted[i]) * 8);
        float4 *o = reinterpret_cast<float4 *>(kept + static_cast<size_t>(pos) * 12);
        o[0] = q[0]; o[1] = q[1];
        o[2] = make_float4(topScore, topCell, static_cast<float>(pickOf[i]), static_cast<float>(b));
    }
}

// The same procedure for a class with more than NMS_CAP members in an image (up to NMS_BIG): the members are sorted by a
// bitonic network in LDS (keys and row indices, 128 KiB), the sorted row indices go to the workspace, then the corner
// coordinates of all members take the keys' place in LDS and the whole workgroup runs the greedy pass (one barrier per pick).
// state[i]: 0xffff = erased, 0xfffe = not visited yet, else the pick order.
constexpr int NMS_BIG = 6144, NMS_SORT = 8192, NMS_SLOTS = NMS_BIG / 256;
constexpr int NMS_BIG_LDS = NMS_SORT * 16 + NMS_BIG * 2;        // max(sort: 8+4+4 bytes per slot, boxes: 20 bytes per member) + state

__global__ __launch_bounds__(256) void yoloNmsBigKernel(const float *__restrict__ rows, int candCap, const int *__restrict__ candCnt, float thr,
                                                        float *__restrict__ kept, int keptCap, int *__restrict__ keptCnt,
                                                        const int *__restrict__ bigCnt, int *__restrict__ wsSorted, int *__restrict__ wsUsed)
{
#pragma clang fp contract(off)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ unsigned long long top;
    __shared__ int nMem, bad, base, off;
    const int cls = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int m = bigCnt[b * gridDim.x + cls];
    if (m <= NMS_CAP) return;
    if (m > NMS_BIG)
    {
        if (tid == 0) atomicOr(&keptCnt[1 + b], 1);
        return;
    }
    unsigned long long *kA = reinterpret_cast<unsigned long long *>(smem);
    unsigned *kB = reinterpret_cast<unsigned *>(smem + NMS_SORT * 8);
    int *ix = reinterpret_cast<int *>(smem + NMS_SORT * 12);
    int n = candCnt[b];
    n = n < candCap ? n : candCap;
    const float *r = rows + static_cast<size_t>(b) * candCap * 8;
    if (tid == 0) { nMem = 0; bad = 0; top = 0ull; off = atomicAdd(&wsUsed[b], m); }
    __syncthreads();
    for (int k = tid; k < n; k += 256)
    {
        const float *q = r + static_cast<size_t>(k) * 8;
        if (static_cast<int>(q[6]) != cls) continue;
        const int slot = atomicAdd(&nMem, 1);
        if (slot >= NMS_SORT) continue;
        const float conf = q[4];
        const float score = conf * q[5];
        if (!(score == score) || !(conf == conf)) bad = 1;
        const unsigned sb = orderedBits(score), cell = ~static_cast<unsigned>(q[7]);
        kA[slot] = (static_cast<unsigned long long>(orderedBits(conf)) << 32) | sb;
        kB[slot] = cell;
        ix[slot] = k;
        atomicMax(&top, (static_cast<unsigned long long>(sb) << 32) | cell);
    }
    __syncthreads();
    if (bad || nMem != m || off + m > candCap)
    {
        if (tid == 0) atomicOr(&keptCnt[1 + b], bad ? 2 : 4);
        return;
    }
    int S = 2048;
    while (S < m) S <<= 1;
    for (int i = m + tid; i < S; i += 256) { kA[i] = 0ull; kB[i] = 0u; ix[i] = -1; }       // below every real key (objectness > 0)
    for (int k2 = 2; k2 <= S; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1)
        {
            __syncthreads();
            for (int t = tid; t < S / 2; t += 256)
            {
                const int lo = ((t / j) * 2 * j) + (t % j), hi = lo + j;
                const unsigned long long a0 = kA[lo], a1 = kA[hi];
                const unsigned b0 = kB[lo], b1 = kB[hi];
                const bool loLess = a0 < a1 || (a0 == a1 && b0 < b1);
                const bool descending = (lo & k2) == 0;
                if (loLess == descending)
                {
                    kA[lo] = a1; kA[hi] = a0; kB[lo] = b1; kB[hi] = b0;
                    const int t0 = ix[lo]; ix[lo] = ix[hi]; ix[hi] = t0;
                }
            }
        }
    __syncthreads();
    int *sortedRow = wsSorted + static_cast<size_t>(b) * candCap + off;
    for (int i = tid; i < m; i += 256) sortedRow[i] = ix[i];
    __syncthreads();                                             // the keys are dead from here on
    float *x1 = reinterpret_cast<float *>(smem), *y1 = x1 + NMS_BIG, *x2 = y1 + NMS_BIG, *y2 = x2 + NMS_BIG, *area = y2 + NMS_BIG;
    volatile unsigned short *state = reinterpret_cast<unsigned short *>(smem + NMS_SORT * 16);
    // Every thread keeps its members (sorted positions tid, tid + 256, ...) in registers, so that the test against a pick is
    // arithmetic only; LDS holds the same coordinates for the broadcast of the pick and the erased / picked state.
    float rx1[NMS_SLOTS], ry1[NMS_SLOTS], rx2[NMS_SLOTS], ry2[NMS_SLOTS], rar[NMS_SLOTS];
    unsigned alive = 0u;
#pragma unroll
    for (int t = 0; t < NMS_SLOTS; ++t)
    {
        const int i = t * 256 + tid;
        rx1[t] = ry1[t] = rx2[t] = ry2[t] = rar[t] = 0.f;
        if (i >= m) continue;
        const float *q = r + static_cast<size_t>(sortedRow[i]) * 8;
        const float bx = q[0], by = q[1], bw = q[2], bh = q[3];
        const float ax1 = bx - bw / 2.f, ax2 = bx + bw / 2.f, ay1 = by - bh / 2.f, ay2 = by + bh / 2.f;
        const float ar = (ax2 - ax1 + 1) * (ay2 - ay1 + 1);
        x1[i] = ax1; x2[i] = ax2; y1[i] = ay1; y2[i] = ay2; area[i] = ar;
        rx1[t] = ax1; rx2[t] = ax2; ry1[t] = ay1; ry2[t] = ay2; rar[t] = ar;
        state[i] = 0xfffe;
        alive |= 1u << t;
    }
    __syncthreads();
    int picks = 0;
    for (int i = 0;; ++i)
    {
        while (i < m && state[i] == 0xffff) ++i;                 // same answer in every thread: writes end at the barrier below
        if (i >= m) break;
        const float kx1 = x1[i], ky1 = y1[i], kx2 = x2[i], ky2 = y2[i], karea = area[i];
#pragma unroll
        for (int t = 0; t < NMS_SLOTS; ++t)
        {
            if (t * 256 + 255 <= i || t * 256 >= m) continue;    // (uniform) nothing of this slot lies behind the pick
            const int j = t * 256 + tid;
            if (j <= i || !((alive >> t) & 1u)) continue;
            if (iouAbove(kx1, ky1, kx2, ky2, karea, rx1[t], ry1[t], rx2[t], ry2[t], rar[t], thr)) { alive &= ~(1u << t); state[j] = 0xffff; }
        }
        __syncthreads();
        if (tid == 0) state[i] = static_cast<unsigned short>(picks);
        ++picks;
    }
    if (tid == 0) base = atomicAdd(&keptCnt[0], picks);
    __syncthreads();
    const unsigned long long t = top;
    const float topScore = __uint_as_float((static_cast<unsigned>(t >> 32) & 0x80000000u) ? (static_cast<unsigned>(t >> 32) & 0x7fffffffu) : ~static_cast<unsigned>(t >> 32));
    const float topCell = static_cast<float>(~static_cast<unsigned>(t & 0xffffffffull));
    for (int i = tid; i < m; i += 256)
    {
        const unsigned short st = state[i];
        if (st == 0xffff) continue;
        const int pos = base + st;
        if (pos >= keptCap) continue;
        const float4 *q = reinterpret_cast<const float4 *>(r + static_cast<size_t>(sortedRow[i]) * 8);
        float4 *o = reinterpret_cast<float4 *>(kept + static_cast<size_t>(pos) * 12);
        o[0] = q[0]; o[1] = q[1];
        o[2] = make_float4(topScore, topCell, static_cast<float>(st), static_cast<float>(b));
    }
}

__global__ __launch_bounds__(256) void yoloGatherKernel(const float *__restrict__ decoded, long long decStride, const int *__restrict__ candIdx,
                                                        int candCap, const int *__restrict__ candCnt, float *__restrict__ rows, int per,
                                                        int batch)
{
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    const int b = blockIdx.y;
    if (b >= batch) return;
    int n = candCnt[b];
    n = n < candCap ? n : candCap;
    if (k >= n) return;
    const int cell = candIdx[static_cast<size_t>(b) * candCap + k];
    const float *r = decoded + static_cast<size_t>(b) * decStride + static_cast<size_t>(cell) * per;
    int best = 0;
    float bv = r[5];
    for (int m = 1; m < per - 5; ++m)
    {
        const float v = r[5 + m];
        if (bv < v) { bv = v; best = m; }
    }
    float *o = rows + (static_cast<size_t>(b) * candCap + k) * 8;
    o[0] = r[0]; o[1] = r[1]; o[2] = r[2]; o[3] = r[3]; o[4] = r[4];
    o[5] = bv; o[6] = static_cast<float>(best); o[7] = static_cast<float>(cell);
}

template <typename T>
__global__ __launch_bounds__(256) void absMaxKernel(const T *__restrict__ x, int xLd, int c, long long total, float *__restrict__ result)
{
    float m = 0.f;
    for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<long long>(gridDim.x) * blockDim.x)
    {
        const long long p = idx / c;
        const int ch = static_cast<int>(idx - p * c);
        const float v = fabsf(toF(x[p * xLd + ch]));
        if (v <= FLT_MAX && v > m) m = v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
    {
        const float o = __shfl_xor(m, off, 64);
        m = o > m ? o : m;
    }
    if ((threadIdx.x & 63) == 0 && m > 0.f) atomicMax(reinterpret_cast<int *>(result), __float_as_int(m));
}

template <typename T>
__global__ __launch_bounds__(256) void countNonFiniteKernel(const T *__restrict__ x, int xLd, int c, long long total, unsigned *__restrict__ result)
{
    unsigned n = 0;
    for (long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<long long>(gridDim.x) * blockDim.x)
    {
        const long long p = idx / c;
        const int ch = static_cast<int>(idx - p * c);
        const float v = fabsf(toF(x[p * xLd + ch]));
        n += (v <= FLT_MAX) ? 0u : 1u;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) n += __shfl_xor(n, off, 64);
    if ((threadIdx.x & 63) == 0 && n > 0) atomicAdd(result, n);
}

} // namespace msnh

using namespace msnh;

extern "C" int msnh_hip_yolo_decode(int dtype, int batch, int h, int w, int classes, const void *x, int x_ld, float x_mul,
                                    const float *anchors6, float ratio, int yolo_version, float *decoded, long long decoded_batch_stride,
                                    float conf_thresh, int *cand_idx, int cand_cap, int cand_base, int *cand_cnt, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "yolo_decode: bad dtype");
    MSNH_REQUIRE(batch > 0 && h > 0 && w > 0 && classes > 0, "yolo_decode: bad geometry");
    MSNH_REQUIRE(yolo_version == 3 || yolo_version == 4 || yolo_version == 5, "yolo_decode: yolo_version must be 3, 4 or 5");
    const int per = 5 + classes;
    MSNH_REQUIRE(x && decoded && anchors6 && x_ld >= 3 * per, "yolo_decode: bad argument");
    MSNH_REQUIRE(decoded_batch_stride >= static_cast<long long>(3) * h * w * per, "yolo_decode: decoded_batch_stride too small");
    MSNH_REQUIRE(cand_idx == nullptr || (cand_cnt != nullptr && cand_cap > 0), "yolo_decode: candidate list without counter");
    Anchors an;
    for (int i = 0; i < 6; ++i) an.v[i] = anchors6[i];
    MSNH_REQUIRE(per >= 6 && batch <= 65535, "yolo_decode: unsupported geometry");
    const int perImage = 3 * h * w * per;
    dim3 grid((perImage + YOLO_CHUNK - 1) / YOLO_CHUNK, batch);
    hipStream_t st = resolveStream(s);
#define MSNH_YOLO(T, V5)                                                                                                \
    hipLaunchKernelGGL((yoloDecodeKernel<T, V5>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, x_mul, an, ratio, decoded, \
                       decoded_batch_stride, conf_thresh, cand_idx, cand_cap, cand_base, cand_cnt, w, h * w, per, perImage)
    if (dtype == MSNH_F16) { if (yolo_version == 5) MSNH_YOLO(f16, true); else MSNH_YOLO(f16, false); }
    else { if (yolo_version == 5) MSNH_YOLO(float, true); else MSNH_YOLO(float, false); }
#undef MSNH_YOLO
    MSNH_LAUNCH_CHECK();
    return 0;
}

extern "C" int msnh_hip_yolo_decode_candidates(int dtype, int batch, int h, int w, int classes, const void *x, int x_ld, float x_mul,
                                               const float *anchors6, float ratio, int yolo_version, float *decoded,
                                               long long decoded_batch_stride, float conf_thresh, int *cand_idx, int cand_cap, int cand_base,
                                               int *cand_cnt, float *rows, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "yolo_decode_candidates: bad dtype");
    MSNH_REQUIRE(batch > 0 && batch <= 65535 && h > 0 && w > 0 && classes > 0, "yolo_decode_candidates: bad geometry");
    MSNH_REQUIRE(yolo_version == 3 || yolo_version == 4 || yolo_version == 5, "yolo_decode_candidates: yolo_version must be 3, 4 or 5");
    const int per = 5 + classes;
    MSNH_REQUIRE(x && (decoded || rows) && anchors6 && cand_idx && cand_cnt && cand_cap > 0 && x_ld >= 3 * per, "yolo_decode_candidates: bad argument");
    MSNH_REQUIRE(decoded_batch_stride >= static_cast<long long>(3) * h * w * per, "yolo_decode_candidates: decoded_batch_stride too small");
    Anchors an;
    for (int i = 0; i < 6; ++i) an.v[i] = anchors6[i];
    hipStream_t st = resolveStream(s);
    const int HW = h * w;
    dim3 sgrid((3 * HW + 255) / 256, batch), rgrid(256, batch);
#define MSNH_YC(T)                                                                                                      \
    do {                                                                                                                \
        hipLaunchKernelGGL((yoloScanKernel<T>), sgrid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, x_mul, conf_thresh, cand_idx, cand_cap,  \
                           cand_base, cand_cnt, HW, per);                                                               \
        if (yolo_version == 5)                                                                                          \
            hipLaunchKernelGGL((yoloRowsKernel<T, true>), rgrid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, x_mul, an, ratio, decoded,  \
                               decoded_batch_stride, cand_idx, cand_cap, cand_base, cand_cnt, rows, w, HW, per);        \
        else                                                                                                            \
            hipLaunchKernelGGL((yoloRowsKernel<T, false>), rgrid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, x_mul, an, ratio, decoded, \
                               decoded_batch_stride, cand_idx, cand_cap, cand_base, cand_cnt, rows, w, HW, per);        \
    } while (0)
    if (dtype == MSNH_F16) MSNH_YC(f16); else MSNH_YC(float);
#undef MSNH_YC
    MSNH_LAUNCH_CHECK();
    return 0;
}

extern "C" int msnh_hip_yolo_gather(int batch, int classes, const float *decoded, long long decoded_batch_stride, const int *cand_idx,
                                    int cand_cap, const int *cand_cnt, float *rows, msnh_stream_t s)
{
    MSNH_REQUIRE(batch > 0 && batch <= 65535 && classes > 0 && cand_cap > 0, "yolo_gather: bad geometry");
    MSNH_REQUIRE(decoded && cand_idx && cand_cnt && rows, "yolo_gather: NULL pointer");
    dim3 grid(gridFor(cand_cap, 256), batch);
    hipLaunchKernelGGL(yoloGatherKernel, grid, dim3(256), 0, resolveStream(s), decoded, decoded_batch_stride, cand_idx, cand_cap, cand_cnt,
                       rows, 5 + classes, batch);
    MSNH_LAUNCH_CHECK();
    return 0;
}

extern "C" size_t msnh_hip_yolo_nms_workspace_bytes(int batch, int classes, int cand_cap)
{
    if (batch <= 0 || classes <= 0 || cand_cap <= 0) return 0;
    return sizeof(int) * (static_cast<size_t>(batch) * classes + static_cast<size_t>(batch) * cand_cap + static_cast<size_t>(batch));
}

// The two launches of the device NMS; ws = [batch*classes] class sizes | [batch*cand_cap] sorted rows | [batch] cursors, or NULL
// (small classes only).
static int launchYoloNms(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept, int kept_cap,
                         int *kept_cnt, int *ws, bool bigKernelReady, hipStream_t st)
{
    int *bigCnt = ws;
    int *wsSorted = bigCnt ? bigCnt + static_cast<size_t>(batch) * classes : nullptr;
    int *wsUsed = bigCnt ? wsSorted + static_cast<size_t>(batch) * cand_cap : nullptr;
    hipLaunchKernelGGL(yoloNmsKernel, dim3(classes, batch), dim3(256), 0, st, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt, bigCnt, wsUsed);
    MSNH_LAUNCH_CHECK();
    if (ws == nullptr) return 0;
    if (!bigKernelReady)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(yoloNmsBigKernel), hipFuncAttributeMaxDynamicSharedMemorySize, NMS_BIG_LDS);
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(yoloNmsBigKernel, dim3(classes, batch), dim3(256), NMS_BIG_LDS, st, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt,
                       bigCnt, wsSorted, wsUsed);
    MSNH_LAUNCH_CHECK();
    return 0;
}

static int checkYoloNmsArgs(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, const float *kept, int kept_cap, const int *kept_cnt)
{
    MSNH_REQUIRE(batch > 0 && batch <= 65535 && classes > 0 && cand_cap > 0 && cand_cap <= (1 << 24) && kept_cap > 0, "yolo_nms: bad geometry");
    MSNH_REQUIRE(rows && cand_cnt && kept && kept_cnt, "yolo_nms: NULL pointer");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(rows) % 16 == 0 && reinterpret_cast<uintptr_t>(kept) % 16 == 0, "yolo_nms: rows and kept must be 16-byte aligned");
    return 0;
}

extern "C" int msnh_hip_yolo_nms(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept,
                                 int kept_cap, int *kept_cnt, void *workspace, size_t workspace_bytes, msnh_stream_t s)
{
    if (int rc = checkYoloNmsArgs(batch, classes, rows, cand_cap, cand_cnt, kept, kept_cap, kept_cnt)) return rc;
    MSNH_REQUIRE(workspace == nullptr || (workspace_bytes >= msnh_hip_yolo_nms_workspace_bytes(batch, classes, cand_cap) && reinterpret_cast<uintptr_t>(workspace) % 4 == 0),
                 "yolo_nms: workspace too small (msnh_hip_yolo_nms_workspace_bytes)");
    return launchYoloNms(batch, classes, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt, static_cast<int *>(workspace), false, resolveStream(s));
}

// ---- the same call for callers that cannot allocate ------------------------------------------------------------------------------
// The workspace lives in a device array of this module: 4 MiB per GPU the library runs on, held until the process ends.  The
// array's name is only a host-side stand-in; its device address is asked for once per device and kept.
namespace {
constexpr size_t kNmsScratchInts = static_cast<size_t>(1) << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) int scratch[kNmsScratchInts];
int *g_scratchPtr[kMaxDevices] = {};
std::mutex g_scratchMutex;
}

namespace msnh {
// One-time set-up on the current device: the scratch array's address there, and the large-class kernel's LDS limit.
int yoloNmsSetupDevice()
{
    int dev = -1;
    MSNH_HIP_CHECK(hipGetDevice(&dev));
    MSNH_REQUIRE(dev >= 0 && dev < kMaxDevices, "yolo_nms_static: device index %d is beyond the %d this library keeps state for", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratchMutex);
    if (g_scratchPtr[dev] != nullptr) return 0;
    void *p = nullptr;
    MSNH_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    MSNH_REQUIRE(p != nullptr, "yolo_nms_static: the scratch array has no address on device %d", dev);
    MSNH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(yoloNmsBigKernel), hipFuncAttributeMaxDynamicSharedMemorySize, NMS_BIG_LDS));
    g_scratchPtr[dev] = static_cast<int *>(p);
    return 0;
}
}

extern "C" size_t msnh_hip_yolo_nms_static_max_bytes(void) { return kNmsScratchInts * sizeof(int); }

extern "C" int msnh_hip_yolo_nms_static(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept,
                                        int kept_cap, int *kept_cnt, msnh_stream_t s)
{
    if (int rc = checkYoloNmsArgs(batch, classes, rows, cand_cap, cand_cnt, kept, kept_cap, kept_cnt)) return rc;
    const size_t need = msnh_hip_yolo_nms_workspace_bytes(batch, classes, cand_cap);
    MSNH_REQUIRE(need <= kNmsScratchInts * sizeof(int),
                 "yolo_nms_static: batch %d x (%d classes + %d candidate slots + 1) needs %zu bytes of workspace, the built-in one holds %zu; "
                 "use msnh_hip_yolo_nms with a workspace of the caller", batch, classes, cand_cap, need, kNmsScratchInts * sizeof(int));
    int dev = -1;
    MSNH_HIP_CHECK(hipGetDevice(&dev));
    MSNH_REQUIRE(dev >= 0 && dev < kMaxDevices, "yolo_nms_static: device index %d is beyond the %d this library keeps state for", dev, kMaxDevices);
    if (g_scratchPtr[dev] == nullptr)
        if (int rc = yoloNmsSetupDevice()) return rc;        // (msnh_hip_init does this for the device it selects)
    // Nothing in the workspace has to start at zero: the first kernel writes every class size and resets every image's cursor,
    // and the sorted rows are written before they are read.
    return launchYoloNms(batch, classes, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt, g_scratchPtr[dev], true, resolveStream(s));
}

extern "C" int msnh_hip_absmax(int dtype, long long pixels, int c, const void *x, int x_ld, float *result, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "absmax: bad dtype");
    MSNH_REQUIRE(pixels > 0 && c > 0 && x && result && x_ld >= c, "absmax: bad argument");
    const long long total = pixels * c;
    long long blocks = (total + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    dim3 grid(static_cast<unsigned>(blocks));
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((absMaxKernel<f16>), grid, dim3(256), 0, resolveStream(s), static_cast<const f16 *>(x), x_ld, c, total, result);
    else
        hipLaunchKernelGGL((absMaxKernel<float>), grid, dim3(256), 0, resolveStream(s), static_cast<const float *>(x), x_ld, c, total, result);
    MSNH_LAUNCH_CHECK();
    return 0;
}

extern "C" int msnh_hip_count_nonfinite(int dtype, long long pixels, int c, const void *x, int x_ld, unsigned *result, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype) && pixels >= 0 && c > 0 && x_ld >= c && x && result, "count_nonfinite: bad argument");
    if (pixels == 0) return 0;
    const long long total = pixels * c;
    long long blocks = (total + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    dim3 grid(static_cast<unsigned>(blocks));
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((countNonFiniteKernel<f16>), grid, dim3(256), 0, resolveStream(s), static_cast<const f16 *>(x), x_ld, c, total, result);
    else
        hipLaunchKernelGGL((countNonFiniteKernel<float>), grid, dim3(256), 0, resolveStream(s), static_cast<const float *>(x), x_ld, c, total, result);
    MSNH_LAUNCH_CHECK();
    return 0;
}
