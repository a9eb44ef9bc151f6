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

// All heads of a network in two launches instead of two per head: an objectness scan over the cells of an image numbered over
// the heads in list order (which is the numbering of the candidate list), then the rows of the listed candidates, each decoded
// from the head its cell number falls into.  Same logistic, same threshold test and same per-value decode as the per-head
// kernels, so list (as a set) and rows are identical.  (Decoding a workgroup's own candidates right after its scan, in one
// launch, was slower: where objectness is dense a few workgroups hold most of the candidates.)
constexpr int YOLO_MAX_HEADS = 4;
struct YoloHeads
{
    const void *x[YOLO_MAX_HEADS];
    int xLd[YOLO_MAX_HEADS], W[YOLO_MAX_HEADS], HW[YOLO_MAX_HEADS], base[YOLO_MAX_HEADS];
    float xMul[YOLO_MAX_HEADS], ratio[YOLO_MAX_HEADS];
    Anchors an[YOLO_MAX_HEADS];
    int n, cells;
};

__device__ __forceinline__ int yoloHeadOf(const YoloHeads &hd, int cellG)
{
    int k = 0;
#pragma unroll
    for (int i = 1; i < YOLO_MAX_HEADS; ++i)
        if (i < hd.n && cellG >= hd.base[i]) k = i;
    return k;
}

template <typename T>
__global__ __launch_bounds__(256) void yoloHeadsScanKernel(YoloHeads hd, float confThresh, int *__restrict__ candIdx, int candCap, int *__restrict__ candCnt, int per)
{
    __shared__ int found[256];
    __shared__ int nFound, base;
    const int b = blockIdx.y;
    if (threadIdx.x == 0) nFound = 0;
    __syncthreads();
    const int cellG = blockIdx.x * 256 + threadIdx.x;
    if (cellG < hd.cells)
    {
        const int k = yoloHeadOf(hd, cellG);
        const int cell = cellG - hd.base[k];
        const int HW = hd.HW[k];
        const int a = cell / HW, p = cell - a * HW;
        const float v = hd.xMul[k] * toF(static_cast<const T *>(hd.x[k])[(static_cast<size_t>(b) * HW + p) * hd.xLd[k] + a * per + 4]);
        if (logisticF(v) > confThresh) found[atomicAdd(&nFound, 1)] = cellG;
    }
    __syncthreads();
    if (nFound == 0) return;
    if (threadIdx.x == 0) base = atomicAdd(candCnt + b, nFound);
    __syncthreads();
    if (static_cast<int>(threadIdx.x) < nFound && base + static_cast<int>(threadIdx.x) < candCap)
        candIdx[static_cast<size_t>(b) * candCap + base + threadIdx.x] = found[threadIdx.x];
}

template <typename T, bool V5>
__global__ __launch_bounds__(256) void yoloHeadsRowsKernel(YoloHeads hd, float *__restrict__ decoded, long long decStride, const int *__restrict__ candIdx,
                                                           int candCap, const int *__restrict__ candCnt, float *__restrict__ rows, int per)
{
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int sub = lane & 15;
    const int groupLane0 = lane & 48;
    const int group = threadIdx.x >> 4;
    int n = candCnt[b];
    n = n < candCap ? n : candCap;
    for (int slot = blockIdx.x * 16 + group; slot < n; slot += gridDim.x * 16)
    {
        const int cellG = candIdx[static_cast<size_t>(b) * candCap + slot];
        if (cellG < 0 || cellG >= hd.cells) continue;
        const int k = yoloHeadOf(hd, cellG);
        const int cell = cellG - hd.base[k];
        const int HW = hd.HW[k], W = hd.W[k];
        const int a = cell / HW, p = cell - a * HW;
        const int py = p / W, px = p - py * W;
        const T *xr = static_cast<const T *>(hd.x[k]) + (static_cast<size_t>(b) * HW + p) * hd.xLd[k] + a * per;
        float *dr = decoded + static_cast<size_t>(b) * decStride + static_cast<size_t>(cellG) * per;
        const float xMul = hd.xMul[k], ratio = hd.ratio[k];
        const Anchors an = hd.an[k];
        float first = 0.f;
        float bv = -3.402823466e38f * 2.f;
        int bi = 0x7fffffff;
        // all loads of the row first (the stores into `decoded` below may alias the head tensor as far as the compiler knows, and
        // a load per round trip would make the row cost one memory latency per sixteen values)
        constexpr int ROUNDS = 8;
        float raw[ROUNDS];
#pragma unroll
        for (int it = 0; it < ROUNDS; ++it)
        {
            const int m = sub + 16 * it;
            raw[it] = m < per ? toF(xr[m]) : 0.f;
        }
#pragma unroll
        for (int it = 0; it < ROUNDS; ++it)
        {
            const int m = sub + 16 * it;
            if (m >= per) break;
            const float v = yoloDecodeOne<V5>(xMul * raw[it], m, px, py, a, an, ratio);
            if (decoded != nullptr) dr[m] = v;
            if (it == 0) first = v;
            if (m >= 5 && v > bv) { bv = v; bi = m - 5; }
        }
        for (int m = sub + 16 * ROUNDS; m < per; m += 16)        // more than 123 classes
        {
            const float v = yoloDecodeOne<V5>(xMul * toF(xr[m]), m, px, py, a, an, ratio);
            if (decoded != nullptr) dr[m] = v;
            if (v > bv) { bv = v; bi = m - 5; }
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1)
        {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        const float c0v = __shfl(first, groupLane0 + 5, 64);
        if (c0v != c0v) { bv = c0v; bi = 0; }
        if (bi == 0x7fffffff) bi = 0;
        float *o = rows + (static_cast<size_t>(b) * candCap + slot) * 8;
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
constexpr int NMS_PAIR_MIN = 256;       // with the pair workspace, classes with more members than this go through the bit matrix

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

// One LDS atomic per wavefront instead of one per lane: the lanes with `pred` get consecutive slots from *counter (-1 for the others).
// Every lane of the wavefront must make the call.
__device__ __forceinline__ int waveSlot(bool pred, int *counter)
{
    const unsigned long long mask = __ballot(pred);
    if (mask == 0ull) return -1;
    const int lane = threadIdx.x & 63;
    const int leader = __ffsll(static_cast<long long>(mask)) - 1;
    int first = 0;
    if (lane == leader) first = atomicAdd(counter, __popcll(mask));
    first = __shfl(first, leader, 64);
    return pred ? first + __popcll(mask & ((1ull << lane) - 1ull)) : -1;
}

__device__ __forceinline__ unsigned long long waveMax64(unsigned long long v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1)
    {
        const unsigned lo = __shfl_xor(static_cast<unsigned>(v), o, 64), hi = __shfl_xor(static_cast<unsigned>(v >> 32), o, 64);
        const unsigned long long other = (static_cast<unsigned long long>(hi) << 32) | lo;
        v = other > v ? other : v;
    }
    return v;
}

__global__ __launch_bounds__(256) void yoloNmsKernel(const float *__restrict__ rows, int candCap, const int *__restrict__ candCnt, float thr,
                                                     float *__restrict__ kept, int keptCap, int *__restrict__ keptCnt, int *__restrict__ bigCnt,
                                                     int *__restrict__ wsUsed, unsigned long long *__restrict__ pairHdr, int deferAbove)
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
    if (pairHdr != nullptr && cls == 0 && b == 0 && tid == 0) { pairHdr[0] = 0ull; pairHdr[1] = 0ull; }    // pool cursor, list length
    __syncthreads();
    for (int k0 = 0; k0 < n; k0 += 256)
    {
        const int k = k0 + tid;
        const int slot = waveSlot(k < n && static_cast<int>(r[static_cast<size_t>(k < n ? k : 0) * 8 + 6]) == cls, &nMem);
        if (slot >= 0 && slot < NMS_CAP) member[slot] = k;
    }
    __syncthreads();
    const int m = nMem;
    if (bigCnt != nullptr && tid == 0) bigCnt[b * gridDim.x + cls] = m;
    if (m == 0) return;
    if (m > deferAbove)                                  // (<= NMS_CAP)
    {
        if (bigCnt == nullptr && tid == 0) atomicOr(&keptCnt[1 + b], 1);    // (else yoloNmsBigKernel takes the class)
        return;
    }
    unsigned long long best = 0ull;
    for (int i = tid; i < m; i += 256)
    {
        const float *q = r + static_cast<size_t>(member[i]) * 8;
        const float conf = q[4];
        const float score = conf * q[5];
        if (!(score == score) || !(conf == conf)) bad = 1;
        const unsigned sb = orderedBits(score), cell = ~static_cast<unsigned>(q[7]);
        keyA[i] = (static_cast<unsigned long long>(orderedBits(conf)) << 32) | sb;
        keyB[i] = cell;
        const unsigned long long key = (static_cast<unsigned long long>(sb) << 32) | cell;
        best = key > best ? key : best;
    }
    best = waveMax64(best);
    if ((tid & 63) == 0 && best != 0ull) atomicMax(&top, best);
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

// The same procedure for a class with more than NMS_CAP members in an image (up to NMS_BIG), one workgroup of 16 wavefronts per class:
//   1. the members are sorted by a bitonic network in LDS (keys and row indices, 128 KiB); the sorted row indices go to the workspace;
//   2. the corner coordinates of the sorted members take the keys' place in LDS;
//   3. the greedy pass runs over chunks of 64 members in sorted order.  A member survives iff no box kept before it overlaps it, so a
//      chunk is first tested against everything kept so far (lane = member, the kept boxes dealt over the wavefronts, LDS broadcast
//      reads) and against its own earlier members (a 64 x 64 bit block, 4 columns per wavefront); the first wavefront then resolves the
//      block with bit operations only (ascending, an alive member erases the later members of its column) and appends the survivors to
//      the kept list, which grows in place over the coordinates of members already visited (kept <= visited).
// Two barriers per chunk instead of one per pick, and the pair tests of a chunk use the whole workgroup.
constexpr int NMS_BIG = 6144, NMS_SORT = 8192, NMS_BIG_THREADS = 1024;
constexpr int NMS_BIG_LDS = NMS_SORT * 16 + NMS_BIG * 2;        // max(sort: 8+4+4 bytes per slot, boxes: 20 bytes per member) + kept positions

// With the larger workspace (msnh_hip_yolo_nms_pair_workspace_bytes) step 3 of a large class leaves its workgroup: the sorted members'
// corners go to the workspace, the class is entered in a list, yoloNmsPairKernel fills a bit matrix (row = a member, bit = a later
// member it would erase) with the whole chip, and yoloNmsScanKernel walks it (bit operations only).  A class whose matrix does not fit
// into what is left of the pool keeps to its own workgroup.
struct NmsPairWs
{
    unsigned long long *hdr;            // [0] words of the pool handed out, [1] classes in the list (both zeroed by yoloNmsKernel)
    int *list;                          // [maxList][8]: image, class, members, offset of the class in the image's sorted rows, matrix offset lo / hi,
                                        //               score bits and cell of the class's best-scoring member (the record's fields 8, 9)
    float *boxes;                       // [batch * candCap][8]: x1, y1, x2, y2, area of the sorted members, at the place of their sorted row
    unsigned long long *pool;
    unsigned long long poolWords;
    int maxList;
};

__global__ __launch_bounds__(NMS_BIG_THREADS) void yoloNmsBigKernel(const float *__restrict__ rows, int candCap, const int *__restrict__ candCnt, float thr,
                                                                    float *__restrict__ kept, int keptCap, int *__restrict__ keptCnt,
                                                                    const int *__restrict__ bigCnt, int *__restrict__ wsSorted, int *__restrict__ wsUsed,
                                                                    NmsPairWs pw, int deferAbove)
{
#pragma clang fp contract(off)
    constexpr int NT = NMS_BIG_THREADS, NW = NT / 64, COLS = 64 / NW;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ unsigned long long top, erasedBits, blockBits[64], matOff;
    __shared__ int nMem, bad, base, off, nKept, usePair;
    const int cls = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int m = bigCnt[b * gridDim.x + cls];
    if (m <= deferAbove) return;
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
    if (tid == 0) { nMem = 0; bad = 0; top = 0ull; erasedBits = 0ull; nKept = 0; off = atomicAdd(&wsUsed[b], m); }
    if (tid < 64) blockBits[tid] = 0ull;
    __syncthreads();
    unsigned long long best = 0ull;
    for (int k0 = 0; k0 < n; k0 += NT)
    {
        const int k = k0 + tid;
        const float *q = r + static_cast<size_t>(k < n ? k : 0) * 8;
        const int slot = waveSlot(k < n && static_cast<int>(q[6]) == cls, &nMem);
        if (slot < 0 || slot >= NMS_SORT) continue;
        const float conf = q[4];
        const float score = conf * q[5];
        if (!(score == score) || !(conf == conf)) bad = 1;
        const unsigned sb = orderedBits(score), cell = ~static_cast<unsigned>(q[7]);
        kA[slot] = (static_cast<unsigned long long>(orderedBits(conf)) << 32) | sb;
        kB[slot] = cell;
        ix[slot] = k;
        const unsigned long long key = (static_cast<unsigned long long>(sb) << 32) | cell;
        best = key > best ? key : best;
    }
    best = waveMax64(best);
    if ((tid & 63) == 0 && best != 0ull) atomicMax(&top, best);
    __syncthreads();
    if (bad || nMem != m || off + m > candCap)
    {
        if (tid == 0) atomicOr(&keptCnt[1 + b], bad ? 2 : 4);
        return;
    }
    int S = 512;
    while (S < m) S <<= 1;
    for (int i = m + tid; i < S; i += NT) { kA[i] = 0ull; kB[i] = 0u; ix[i] = -1; }       // below every real key (objectness > 0)
    for (int k2 = 2; k2 <= S; k2 <<= 1)
        for (int j = k2 >> 1; j > 0; j >>= 1)
        {
            __syncthreads();
            for (int t = tid; t < S / 2; t += NT)
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
    for (int i = tid; i < m; i += NT) sortedRow[i] = ix[i];
    if (tid == 0)
    {
        usePair = 0;
        if (pw.pool != nullptr)
        {
            const unsigned long long W64 = static_cast<unsigned long long>((m + 63) / 64);
            const unsigned long long need = (static_cast<unsigned long long>(m) + 64ull) * W64;      // rows, then the transposed diagonal blocks
            const unsigned long long at = atomicAdd(&pw.hdr[0], need);
            if (at + need <= pw.poolWords)
            {
                const int e = atomicAdd(reinterpret_cast<int *>(&pw.hdr[1]), 1);
                if (e < pw.maxList)
                {
                    int *ent = pw.list + static_cast<size_t>(e) * 8;
                    ent[0] = b; ent[1] = cls; ent[2] = m; ent[3] = off;
                    ent[4] = static_cast<int>(at & 0xffffffffull); ent[5] = static_cast<int>(at >> 32);
                    ent[6] = static_cast<int>(top >> 32); ent[7] = static_cast<int>(top & 0xffffffffull);
                    usePair = 1;
                }
            }
        }
    }
    __syncthreads();                                             // the keys are dead from here on
    if (usePair)
    {
        float *bx8 = pw.boxes + (static_cast<size_t>(b) * candCap + off) * 8;
        for (int i = tid; i < m; i += NT)
        {
            const float *q = r + static_cast<size_t>(ix[i]) * 8;
            const float bx = q[0], by = q[1], bw = q[2], bh = q[3];
            const float ax1 = bx - bw / 2.f, ax2 = bx + bw / 2.f, ay1 = by - bh / 2.f, ay2 = by + bh / 2.f;
            *reinterpret_cast<float4 *>(bx8 + static_cast<size_t>(i) * 8) = make_float4(ax1, ay1, ax2, ay2);
            bx8[static_cast<size_t>(i) * 8 + 4] = (ax2 - ax1 + 1) * (ay2 - ay1 + 1);
        }
        return;
    }
    float *x1 = reinterpret_cast<float *>(smem), *y1 = x1 + NMS_BIG, *x2 = y1 + NMS_BIG, *y2 = x2 + NMS_BIG, *area = y2 + NMS_BIG;
    unsigned short *keptPos = reinterpret_cast<unsigned short *>(smem + NMS_SORT * 16);
    __syncthreads();
    for (int i = tid; i < m; i += NT)
    {
        const float *q = r + static_cast<size_t>(sortedRow[i]) * 8;
        const float bx = q[0], by = q[1], bw = q[2], bh = q[3];
        const float ax1 = bx - bw / 2.f, ax2 = bx + bw / 2.f, ay1 = by - bh / 2.f, ay2 = by + bh / 2.f;
        x1[i] = ax1; x2[i] = ax2; y1[i] = ay1; y2[i] = ay2;
        area[i] = (ax2 - ax1 + 1) * (ay2 - ay1 + 1);
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    for (int c0 = 0; c0 < m; c0 += 64)
    {
        const int j = c0 + lane;
        const bool valid = j < m;
        const int K = nKept;                                     // <= c0: the kept list never reaches the members still to visit
        float jx1 = 0.f, jy1 = 0.f, jx2 = 0.f, jy2 = 0.f, jar = 0.f;
        if (valid) { jx1 = x1[j]; jy1 = y1[j]; jx2 = x2[j]; jy2 = y2[j]; jar = area[j]; }
        bool erased = false;
        if (valid)
            for (int k = wave; k < K; k += NW)
                if (iouAbove(x1[k], y1[k], x2[k], y2[k], area[k], jx1, jy1, jx2, jy2, jar, thr)) { erased = true; break; }
        unsigned long long word = 0ull;
        if (valid && !erased)
#pragma unroll
            for (int t = 0; t < COLS; ++t)
            {
                const int i = wave * COLS + t;
                if (i < lane && iouAbove(x1[c0 + i], y1[c0 + i], x2[c0 + i], y2[c0 + i], area[c0 + i], jx1, jy1, jx2, jy2, jar, thr)) word |= 1ull << i;
            }
        const unsigned long long eb = __ballot(erased);
        if (lane == 0 && eb != 0ull) atomicOr(&erasedBits, eb);
        if (word != 0ull) atomicOr(&blockBits[lane], word);
        __syncthreads();
        if (wave == 0)
        {
            unsigned long long alive = __ballot(valid) & ~erasedBits;
            const unsigned long long mine = blockBits[lane];     // bit i: member i of this chunk, if kept, erases this lane's member
            unsigned long long rest = alive;
            while (rest != 0ull)
            {
                const int i = __ffsll(static_cast<long long>(rest)) - 1;
                alive &= ~__ballot(((mine >> i) & 1ull) != 0ull);
                rest = alive & ~((2ull << i) - 1ull);            // (2 << 63 wraps to 0: nothing is left behind the last member)
            }
            if ((alive >> lane) & 1ull)
            {
                const int p = K + __popcll(alive & ((1ull << lane) - 1ull));
                x1[p] = jx1; y1[p] = jy1; x2[p] = jx2; y2[p] = jy2; area[p] = jar;
                keptPos[p] = static_cast<unsigned short>(j);
            }
            blockBits[lane] = 0ull;
            if (lane == 0) { nKept = K + __popcll(alive); erasedBits = 0ull; }
        }
        __syncthreads();
    }
    const int picks = nKept;
    if (tid == 0) base = atomicAdd(&keptCnt[0], picks);
    __syncthreads();
    const unsigned long long t = top;
    const float topScore = __uint_as_float((static_cast<unsigned>(t >> 32) & 0x80000000u) ? (static_cast<unsigned>(t >> 32) & 0x7fffffffu) : ~static_cast<unsigned>(t >> 32));
    const float topCell = static_cast<float>(~static_cast<unsigned>(t & 0xffffffffull));
    for (int k = tid; k < picks; k += NT)
    {
        const int pos = base + k;
        if (pos >= keptCap) continue;
        const float4 *q = reinterpret_cast<const float4 *>(r + static_cast<size_t>(sortedRow[keptPos[k]]) * 8);
        float4 *o = reinterpret_cast<float4 *>(kept + static_cast<size_t>(pos) * 12);
        o[0] = q[0]; o[1] = q[1];
        o[2] = make_float4(topScore, topCell, static_cast<float>(k), static_cast<float>(b));
    }
}

// Bit matrix of the listed classes: bit v - 64 w of M[i][w] says that member i, if kept, erases the later member v (64 w <= v < 64 w + 64).
// Work item = one wavefront: the 64 rows of chunk rc (lane = row) against up to NMS_PAIR_GROUP words w >= rc (a lone wavefront needs
// some 400 cycles per victim, so a longer item would be the kernel's critical path); the victims' corners are the same for
// every lane: lane l loads victim l and the loop reads lane j's registers, so the item needs neither LDS nor a barrier.  The item holding a diagonal word (w = rc)
// also writes that block transposed (lane = victim j, bit i = member 64 rc + i erases it) behind the rows: the scan resolves a chunk
// from it.  The items of all classes form one sequence that the wavefronts of the grid stride through.
constexpr int NMS_PAIR_GRID = 1024, NMS_PAIR_GROUP = 2;

__device__ __forceinline__ long long nmsPairItems(int W)        // sum over rc < W of ceil((W - rc) / GROUP)
{
    const long long q = W / NMS_PAIR_GROUP, r = W % NMS_PAIR_GROUP;
    return NMS_PAIR_GROUP * q * (q + 1) / 2 + r * (q + 1);
}

__global__ __launch_bounds__(256) void yoloNmsPairKernel(const unsigned long long *__restrict__ hdr, const int *__restrict__ list, int maxList,
                                                         const float *__restrict__ boxes, unsigned long long *__restrict__ pool, int candCap, float thr)
{
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const long long nWaves = static_cast<long long>(gridDim.x) * 4;
    int nList = static_cast<int>(hdr[1]);
    nList = nList < maxList ? nList : maxList;
    for (long long t = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x * 4 + (threadIdx.x >> 6)));; t += nWaves)
    {
        long long left = t;
        int e = 0;
        for (; e < nList; ++e)
        {
            const long long items = nmsPairItems((list[e * 8 + 2] + 63) / 64);
            if (left < items) break;
            left -= items;
        }
        if (e >= nList) break;                                  // past the last item: every wavefront gets here
        const int b = list[e * 8], m = list[e * 8 + 2], off = list[e * 8 + 3];
        const int W = (m + 63) / 64;
        int rc = 0;
        for (;; ++rc)
        {
            const int groups = (W - rc + NMS_PAIR_GROUP - 1) / NMS_PAIR_GROUP;
            if (left < groups) break;
            left -= groups;
        }
        const int w0 = rc + static_cast<int>(left) * NMS_PAIR_GROUP;
        const int w1 = w0 + NMS_PAIR_GROUP < W ? w0 + NMS_PAIR_GROUP : W;
        const unsigned long long at = (static_cast<unsigned long long>(static_cast<unsigned>(list[e * 8 + 5])) << 32) | static_cast<unsigned>(list[e * 8 + 4]);
        const float *bx8 = boxes + (static_cast<size_t>(b) * candCap + off) * 8;
        const int i = rc * 64 + lane;
        const int iSafe = i < m ? i : m - 1;
        const float4 k4 = *reinterpret_cast<const float4 *>(bx8 + static_cast<size_t>(iSafe) * 8);
        const float ka = bx8[static_cast<size_t>(iSafe) * 8 + 4];
        // the 64 victims of a word: lane l loads victim l (one coalesced read, the next word's under way while this one is worked on);
        // the loop takes victim j out of lane j's registers
        const auto victim = [&](int w, float4 &c, float &a) {
            const int v = w * 64 + lane;
            const float *q = bx8 + static_cast<size_t>(v < m ? v : m - 1) * 8;
            c = *reinterpret_cast<const float4 *>(q);
            a = q[4];
        };
        // A pair whose boxes are more than a unit apart in x or y has no intersection (inter = 0, never above a threshold >= 0): most
        // pairs of a real image, decided with four comparisons.  The margin of 2 instead of the "+ 1" of the extents keeps the skip
        // on the safe side of any rounding; NaN or infinite corners never skip (every comparison with them is false).
        const float kx2p = k4.z + 2.f, ky2p = k4.w + 2.f;
        const bool skipOk = thr >= 0.f;
        float4 vcNext;
        float vaNext;
        victim(w0, vcNext, vaNext);
        for (int w = w0; w < w1; ++w)
        {
            const float4 vc = vcNext;
            const float va = vaNext;
            if (w + 1 < w1) victim(w + 1, vcNext, vaNext);
            const float vx2p = vc.z + 2.f, vy2p = vc.w + 2.f;
            unsigned long long word = 0ull, col = 0ull;
            const int jEnd = m - w * 64 < 64 ? m - w * 64 : 64;
            for (int j = 0; j < jEnd; ++j)
            {
                const float c0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(vc.x), j));
                const float c1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(vc.y), j));
                const float c2p = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(vx2p), j));
                const float c3p = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(vy2p), j));
                const bool apart = skipOk && (c0 > kx2p || k4.x > c2p || c1 > ky2p || k4.y > c3p);
                const bool later = w * 64 + j > i, earlier = w == rc && j < lane;
                if (!__any(!apart && (later || earlier))) continue;
                const float c2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(vc.z), j));
                const float c3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(vc.w), j));
                const float c4 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(va), j));
                if (later && !apart && iouAbove(k4.x, k4.y, k4.z, k4.w, ka, c0, c1, c2, c3, c4, thr)) word |= 1ull << j;
                if (earlier && !apart && iouAbove(c0, c1, c2, c3, c4, k4.x, k4.y, k4.z, k4.w, ka, thr)) col |= 1ull << j;
            }
            if (i < m) pool[at + static_cast<unsigned long long>(i) * W + w] = word;
            if (w == rc) pool[at + static_cast<unsigned long long>(m) * W + static_cast<unsigned long long>(i)] = i < m ? col : 0ull;
        }
    }
}

// The greedy pass of one listed class over its bit matrix, 64 members (one word column) at a time, by a workgroup of four wavefronts.
// Every wavefront keeps erased bits for all members in two registers per lane (lane l: words l and l + 64): the OR of the rows it has
// folded in so far.  Per chunk: (1) the first wavefront ORs the four partial words of the chunk, and resolves the chunk from the
// transposed diagonal block: alive' = candidates & ~{ j : an alive earlier member of the chunk erases j }, repeated until nothing
// changes (the first t members are final after t rounds; the greedy result is the only fixed point); meanwhile the other three copy
// the next chunk's rows from the pool to LDS; (2) the kept rows of the chunk are dealt over the four wavefronts and folded into their
// erased bits, and each publishes its word of the next chunk.
constexpr int NMS_SCAN_W = (NMS_BIG + 63) / 64;                 // 96 words per row at most
constexpr int NMS_SCAN_LDS = 2 * 64 * NMS_SCAN_W * 8 + NMS_BIG * 2;

__device__ __forceinline__ unsigned long long readLane64(unsigned long long v, int lane)
{
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<int>(static_cast<unsigned>(v)), lane);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<int>(static_cast<unsigned>(v >> 32)), lane);
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}

__global__ __launch_bounds__(256) void yoloNmsScanKernel(const unsigned long long *__restrict__ hdr, const int *__restrict__ list, int maxList,
                                                         const unsigned long long *__restrict__ pool, const float *__restrict__ rows, int candCap,
                                                         const int *__restrict__ wsSorted, float *__restrict__ kept, int keptCap, int *__restrict__ keptCnt)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ unsigned long long partial[2][4], aliveSh;
    __shared__ int nKept, base;
    int nList = static_cast<int>(hdr[1]);
    nList = nList < maxList ? nList : maxList;
    const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (e >= nList) return;
    const int *ent = list + e * 8;
    const int b = ent[0], m = ent[2], off = ent[3];
    const int W = (m + 63) / 64;
    const unsigned long long *M = pool + ((static_cast<unsigned long long>(static_cast<unsigned>(ent[5])) << 32) | static_cast<unsigned>(ent[4]));
    const unsigned long long *diagT = M + static_cast<unsigned long long>(m) * W;
    unsigned long long *buf0 = reinterpret_cast<unsigned long long *>(smem), *buf1 = buf0 + 64 * NMS_SCAN_W;
    unsigned short *keptPos = reinterpret_cast<unsigned short *>(smem + 2 * 64 * NMS_SCAN_W * 8);
    // rows of chunk c, words c + 1 .. W - 1 (what the later chunks need); wavefront q of nq takes rows q, q + nq, ...; all its loads are
    // in flight before the first is stored.  Rows past the last member are never folded in and are skipped.
    const auto fetch = [&](int c, unsigned long long *dst, int q, int nq) {
        constexpr int R = 22;                                   // ceil(64 / 3)
        unsigned long long v0[R], v1[R];
        const int wa = c + 1 + lane, wb = c + 65 + lane;
#pragma unroll
        for (int t = 0; t < R; ++t)
        {
            const int row = q + t * nq, i = c * 64 + row;
            const bool ok = row < 64 && i < m;
            v0[t] = ok && wa < W ? M[static_cast<unsigned long long>(i) * W + wa] : 0ull;
            v1[t] = ok && wb < W ? M[static_cast<unsigned long long>(i) * W + wb] : 0ull;
        }
#pragma unroll
        for (int t = 0; t < R; ++t)
        {
            const int row = q + t * nq;
            if (row < 64 && wa < W) dst[row * W + wa] = v0[t];
            if (row < 64 && wb < W) dst[row * W + wb] = v1[t];
        }
    };
    if (wave != 0) fetch(0, buf0, wave - 1, 3);
    if (tid < 8) partial[tid >> 2][tid & 3] = 0ull;
    unsigned long long r0 = 0ull, r1 = 0ull;
    int K = 0;
    unsigned long long colNext = diagT[lane];                   // (rows past the end hold 0)
    for (int c = 0; c < W; ++c)
    {
        __syncthreads();                                        // the partial words of chunk c are out; (c > 0) its rows are in LDS
        unsigned long long *cur = (c & 1) ? buf1 : buf0, *nxt = (c & 1) ? buf0 : buf1;
        if (wave == 0)
        {
            const unsigned long long col = colNext;
            if (c + 1 < W) colNext = diagT[(c + 1) * 64 + lane];
            const unsigned long long erased = (partial[c & 1][0] | partial[c & 1][1]) | (partial[c & 1][2] | partial[c & 1][3]);
            const unsigned long long cand = __ballot(c * 64 + lane < m) & ~erased;
            unsigned long long alive = cand;
            for (;;)
            {
                const unsigned long long next = cand & ~__ballot((col & alive) != 0ull);
                if (next == alive) break;
                alive = next;
            }
            if ((alive >> lane) & 1ull) keptPos[K + __popcll(alive & ((1ull << lane) - 1ull))] = static_cast<unsigned short>(c * 64 + lane);
            K += __popcll(alive);
            if (lane == 0) aliveSh = alive;
        }
        else if (c + 1 < W && c > 0) fetch(c, cur, wave - 1, 3);     // (chunk 0 was fetched before the loop)
        __syncthreads();                                        // the kept members of chunk c are known, its rows are in LDS
        if (c + 1 >= W) break;
        unsigned long long it = aliveSh;
        const bool mine0 = lane > c && lane < W, mine1 = 64 + lane > c && 64 + lane < W;
        // this wavefront's share: the kept members among rows 16 wave .. 16 wave + 15 of the chunk, four rows per round so that their
        // LDS reads are in flight together
        it = (it >> (16 * wave)) & 0xffffull;
        while (it != 0ull)
        {
            int idx[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                idx[u] = it != 0ull ? __builtin_amdgcn_readfirstlane(__ffsll(static_cast<long long>(it)) - 1) + 16 * wave : -1;
                it &= it - 1ull;
            }
            unsigned long long a0[4], a1[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                a0[u] = (idx[u] >= 0 && mine0) ? cur[idx[u] * W + lane] : 0ull;
                a1[u] = (idx[u] >= 0 && mine1) ? cur[idx[u] * W + 64 + lane] : 0ull;
            }
            r0 |= (a0[0] | a0[1]) | (a0[2] | a0[3]);
            r1 |= (a1[0] | a1[1]) | (a1[2] | a1[3]);
        }
        const unsigned long long mineNext = c + 1 < 64 ? readLane64(r0, c + 1) : readLane64(r1, c + 1 - 64);
        if (lane == 0) partial[(c + 1) & 1][wave] = mineNext;
        (void)nxt;
    }
    if (tid == 0) { nKept = K; base = atomicAdd(&keptCnt[0], K); }
    __syncthreads();
    const int picks = nKept;
    const unsigned sbTop = static_cast<unsigned>(ent[6]), cellTop = static_cast<unsigned>(ent[7]);
    const float topScore = __uint_as_float((sbTop & 0x80000000u) ? (sbTop & 0x7fffffffu) : ~sbTop);
    const float topCell = static_cast<float>(~cellTop);
    const float *r = rows + static_cast<size_t>(b) * candCap * 8;
    const int *sortedRow = wsSorted + static_cast<size_t>(b) * candCap + off;
    for (int k = tid; k < picks; k += 256)
    {
        const int pos = base + k;
        if (pos >= keptCap) continue;
        const float4 *q = reinterpret_cast<const float4 *>(r + static_cast<size_t>(sortedRow[keptPos[k]]) * 8);
        float4 *o = reinterpret_cast<float4 *>(kept + static_cast<size_t>(pos) * 12);
        o[0] = q[0]; o[1] = q[1];
        o[2] = make_float4(topScore, topCell, static_cast<float>(k), static_cast<float>(b));
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

extern "C" int msnh_hip_yolo_decode_candidates_heads(int dtype, int batch, int classes, int n_heads, const msnh_yolo_head *heads, int yolo_version,
                                                     float *decoded, long long decoded_batch_stride, float conf_thresh, int *cand_idx, int cand_cap,
                                                     int *cand_cnt, float *rows, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "yolo_decode_candidates_heads: bad dtype");
    MSNH_REQUIRE(batch > 0 && batch <= 65535 && classes > 0, "yolo_decode_candidates_heads: bad geometry");
    MSNH_REQUIRE(n_heads >= 1 && n_heads <= YOLO_MAX_HEADS && heads, "yolo_decode_candidates_heads: 1 to 4 heads");
    MSNH_REQUIRE(yolo_version == 3 || yolo_version == 4 || yolo_version == 5, "yolo_decode_candidates_heads: yolo_version must be 3, 4 or 5");
    MSNH_REQUIRE(rows && cand_idx && cand_cnt && cand_cap > 0, "yolo_decode_candidates_heads: bad argument");
    const int per = 5 + classes;
    YoloHeads hd;
    std::memset(&hd, 0, sizeof(hd));
    hd.n = n_heads;
    int cells = 0;
    for (int k = 0; k < n_heads; ++k)
    {
        const msnh_yolo_head &h = heads[k];
        MSNH_REQUIRE(h.x && h.h > 0 && h.w > 0 && h.x_ld >= 3 * per, "yolo_decode_candidates_heads: bad head");
        MSNH_REQUIRE(h.cand_base == cells, "yolo_decode_candidates_heads: the heads' cell numbers must follow one another from 0");
        hd.x[k] = h.x; hd.xLd[k] = h.x_ld; hd.xMul[k] = h.x_mul; hd.W[k] = h.w; hd.HW[k] = h.h * h.w; hd.base[k] = cells; hd.ratio[k] = h.ratio;
        for (int i = 0; i < 6; ++i) hd.an[k].v[i] = h.anchors[i];
        cells += 3 * h.h * h.w;
    }
    hd.cells = cells;
    MSNH_REQUIRE(decoded == nullptr || decoded_batch_stride >= static_cast<long long>(cells) * per, "yolo_decode_candidates_heads: decoded_batch_stride too small");
    hipStream_t st = resolveStream(s);
    dim3 sgrid((cells + 255) / 256, batch), rgrid(256, batch);
#define MSNH_YH(T)                                                                                                                                   \
    do {                                                                                                                                             \
        hipLaunchKernelGGL((yoloHeadsScanKernel<T>), sgrid, dim3(256), 0, st, hd, conf_thresh, cand_idx, cand_cap, cand_cnt, per);                   \
        if (yolo_version == 5)                                                                                                                       \
            hipLaunchKernelGGL((yoloHeadsRowsKernel<T, true>), rgrid, dim3(256), 0, st, hd, decoded, decoded_batch_stride, cand_idx, cand_cap,       \
                               cand_cnt, rows, per);                                                                                                 \
        else                                                                                                                                         \
            hipLaunchKernelGGL((yoloHeadsRowsKernel<T, false>), rgrid, dim3(256), 0, st, hd, decoded, decoded_batch_stride, cand_idx, cand_cap,      \
                               cand_cnt, rows, per);                                                                                                 \
    } while (0)
    if (dtype == MSNH_F16) MSNH_YH(f16); else MSNH_YH(float);
#undef MSNH_YH
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

// What follows the plain workspace in the larger one: header (2 x 8 bytes), class list, boxes, pool.
namespace {
constexpr size_t kPairPoolMax = static_cast<size_t>(64) << 20;
size_t pairBase(int batch, int classes, int cand_cap) { return (msnh_hip_yolo_nms_workspace_bytes(batch, classes, cand_cap) + 15) & ~static_cast<size_t>(15); }
int pairMaxList(int batch, int classes, int cand_cap)
{
    const long long perImage = std::min<long long>(classes, cand_cap / (NMS_PAIR_MIN + 1));
    return static_cast<int>(std::min<long long>(perImage * batch, 4096));
}
size_t pairFixed(int batch, int classes, int cand_cap)
{
    return pairBase(batch, classes, cand_cap) + 16 + static_cast<size_t>(pairMaxList(batch, classes, cand_cap)) * 32 + static_cast<size_t>(batch) * cand_cap * 32;
}
}

extern "C" size_t msnh_hip_yolo_nms_pair_workspace_bytes(int batch, int classes, int cand_cap)
{
    if (batch <= 0 || classes <= 0 || cand_cap <= 0) return 0;
    if (cand_cap <= NMS_PAIR_MIN) return msnh_hip_yolo_nms_workspace_bytes(batch, classes, cand_cap);      // no class can be large
    // all large classes of an image together have at most cand_cap members, each row at most NMS_BIG / 64 words
    const size_t rowWords = (static_cast<size_t>(std::min(cand_cap, NMS_BIG)) + 63) / 64;
    const size_t worst = static_cast<size_t>(batch) * cand_cap * (rowWords + 2) * 8;       // (+ the transposed diagonal blocks, 64 words per chunk)
    return pairFixed(batch, classes, cand_cap) + std::min(worst, kPairPoolMax);
}

// The launches of the device NMS; ws = [batch*classes] class sizes | [batch*cand_cap] sorted rows | [batch] cursors, or NULL (small
// classes only); with wsBytes beyond that part (16-byte aligned): | header | class list | boxes | matrix pool.
static int launchYoloNms(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept, int kept_cap,
                         int *kept_cnt, int *ws, size_t wsBytes, hipStream_t st)
{
    int *bigCnt = ws;
    int *wsSorted = bigCnt ? bigCnt + static_cast<size_t>(batch) * classes : nullptr;
    int *wsUsed = bigCnt ? wsSorted + static_cast<size_t>(batch) * cand_cap : nullptr;
    NmsPairWs pw = {nullptr, nullptr, nullptr, nullptr, 0ull, 0};
    if (ws != nullptr && cand_cap > NMS_PAIR_MIN && wsBytes >= pairFixed(batch, classes, cand_cap) + (static_cast<size_t>(1) << 20) &&
        reinterpret_cast<uintptr_t>(ws) % 16 == 0)
    {
        unsigned char *p = reinterpret_cast<unsigned char *>(ws) + pairBase(batch, classes, cand_cap);
        pw.hdr = reinterpret_cast<unsigned long long *>(p);
        pw.maxList = pairMaxList(batch, classes, cand_cap);
        pw.list = reinterpret_cast<int *>(p + 16);
        pw.boxes = reinterpret_cast<float *>(p + 16 + static_cast<size_t>(pw.maxList) * 32);
        pw.pool = reinterpret_cast<unsigned long long *>(reinterpret_cast<unsigned char *>(ws) + pairFixed(batch, classes, cand_cap));
        pw.poolWords = (wsBytes - pairFixed(batch, classes, cand_cap)) / 8;
    }
    hipLaunchKernelGGL(yoloNmsKernel, dim3(classes, batch), dim3(256), 0, st, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt, bigCnt, wsUsed, pw.hdr,
                       pw.pool ? NMS_PAIR_MIN : NMS_CAP);
    MSNH_LAUNCH_CHECK();
    if (ws == nullptr) return 0;
    hipLaunchKernelGGL(yoloNmsBigKernel, dim3(classes, batch), dim3(NMS_BIG_THREADS), NMS_BIG_LDS, st, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt,
                       bigCnt, wsSorted, wsUsed, pw, pw.pool ? NMS_PAIR_MIN : NMS_CAP);
    MSNH_LAUNCH_CHECK();
    if (pw.pool == nullptr) return 0;
    hipLaunchKernelGGL(yoloNmsPairKernel, dim3(NMS_PAIR_GRID), dim3(256), 0, st, pw.hdr, pw.list, pw.maxList, pw.boxes, pw.pool, cand_cap, nms_thresh);
    MSNH_LAUNCH_CHECK();
    hipLaunchKernelGGL(yoloNmsScanKernel, dim3(pw.maxList), dim3(256), NMS_SCAN_LDS, st, pw.hdr, pw.list, pw.maxList, pw.pool, rows, cand_cap, wsSorted, kept, kept_cap,
                       kept_cnt);
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

// ---- the same call for callers that cannot allocate ------------------------------------------------------------------------------
// The workspace lives in a device array of this module: 4 MiB per GPU the library runs on, held until the process ends.  The
// array's name is only a host-side stand-in; its device address is asked for once per device and kept.
namespace {
constexpr size_t kNmsScratchInts = static_cast<size_t>(1) << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) int scratch[kNmsScratchInts];
struct NmsDeviceState
{
    bool attrsTried = false, attrsOk = false;       // the large-class kernels' LDS limits (both entry points need them)
    bool scratchTried = false;
    int *scratchPtr = nullptr;                      // device address of `scratch` on this device
    hipEvent_t done = nullptr;                      // end of the last msnh_hip_yolo_nms_static call on this device
    bool haveDone = false;
    hipStream_t lastStream = nullptr;
    char error[256] = {0};                          // why the set-up failed, reported by the calls that need it
};
NmsDeviceState g_nms[kMaxDevices];
std::mutex g_nmsMutex;                              // guards g_nms and orders the static entry point's calls

int currentDevice(int *dev)
{
    MSNH_HIP_CHECK(hipGetDevice(dev));
    MSNH_REQUIRE(*dev >= 0 && *dev < kMaxDevices, "yolo_nms: device index %d is beyond the %d this library keeps state for", *dev, kMaxDevices);
    return 0;
}

// (g_nmsMutex held) once per device: the LDS limits of the large-class kernels
bool ensureNmsAttributes(NmsDeviceState &st)
{
    if (st.attrsTried) return st.attrsOk;
    st.attrsTried = true;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(yoloNmsBigKernel), hipFuncAttributeMaxDynamicSharedMemorySize, NMS_BIG_LDS);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void *>(yoloNmsScanKernel), hipFuncAttributeMaxDynamicSharedMemorySize, NMS_SCAN_LDS);
    if (e != hipSuccess)
    {
        std::snprintf(st.error, sizeof(st.error), "yolo_nms: hipFuncSetAttribute for the large-class kernels: %s", hipGetErrorString(e));
        (void)hipGetLastError();
    }
    st.attrsOk = e == hipSuccess;
    return st.attrsOk;
}

// (g_nmsMutex held) once per device: the scratch array's address there and the event that orders the calls
bool ensureNmsScratch(NmsDeviceState &st)
{
    if (st.scratchTried) return st.scratchPtr != nullptr;
    st.scratchTried = true;
    void *p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e == hipSuccess && p == nullptr) e = hipErrorInvalidSymbol;
    if (e == hipSuccess) e = hipEventCreateWithFlags(&st.done, hipEventDisableTiming);
    if (e != hipSuccess)
    {
        std::snprintf(st.error, sizeof(st.error), "yolo_nms_static: set-up of the built-in workspace: %s", hipGetErrorString(e));
        (void)hipGetLastError();
        return false;
    }
    st.scratchPtr = static_cast<int *>(p);
    return true;
}
}

namespace msnh {
// One-time set-up on the current device, called by msnh_hip_init.  A failure here does not fail the library's initialisation: it is
// kept and reported by the calls that need what could not be set up (msnh_hip_yolo_nms_static, the large-class path).
void yoloNmsSetupDevice()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) { (void)hipGetLastError(); return; }
    std::lock_guard<std::mutex> lock(g_nmsMutex);
    ensureNmsAttributes(g_nms[dev]);
    ensureNmsScratch(g_nms[dev]);
}
}

extern "C" int msnh_hip_yolo_nms(int batch, int classes, const float *rows, int cand_cap, const int *cand_cnt, float nms_thresh, float *kept,
                                 int kept_cap, int *kept_cnt, void *workspace, size_t workspace_bytes, msnh_stream_t s)
{
    if (int rc = checkYoloNmsArgs(batch, classes, rows, cand_cap, cand_cnt, kept, kept_cap, kept_cnt)) return rc;
    MSNH_REQUIRE(workspace == nullptr || (workspace_bytes >= msnh_hip_yolo_nms_workspace_bytes(batch, classes, cand_cap) && reinterpret_cast<uintptr_t>(workspace) % 4 == 0),
                 "yolo_nms: workspace too small (msnh_hip_yolo_nms_workspace_bytes)");
    if (workspace != nullptr)
    {
        int dev = -1;
        if (int rc = currentDevice(&dev)) return rc;
        std::lock_guard<std::mutex> lock(g_nmsMutex);
        MSNH_REQUIRE(ensureNmsAttributes(g_nms[dev]), "%s", g_nms[dev].error);
    }
    return launchYoloNms(batch, classes, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt, static_cast<int *>(workspace), workspace ? workspace_bytes : 0,
                         resolveStream(s));
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
    if (int rc = currentDevice(&dev)) return rc;
    // Every call on a device works in that device's one array.  The calls are put in order here: enqueued one at a time (the lock),
    // and a call on another stream than the call before it first makes its stream wait for that call's end (an event recorded behind
    // its launches) -- on the device, the host does not block.  A stream under graph capture cannot wait for an event recorded
    // outside the capture nor record one for later calls: captured calls are ordered by the graph's own edges, and keeping them
    // apart from other users of the array is left to the caller.
    std::lock_guard<std::mutex> lock(g_nmsMutex);
    NmsDeviceState &st = g_nms[dev];
    MSNH_REQUIRE(ensureNmsScratch(st) && ensureNmsAttributes(st), "%s", st.error);
    const hipStream_t stream = resolveStream(s);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) { capture = hipStreamCaptureStatusNone; (void)hipGetLastError(); }
    const bool ordered = capture == hipStreamCaptureStatusNone;
    if (ordered && st.haveDone && st.lastStream != stream) MSNH_HIP_CHECK(hipStreamWaitEvent(stream, st.done, 0));
    // Nothing in the workspace has to start at zero: the first kernel writes every class size and resets every image's cursor,
    // and the sorted rows are written before they are read.
    const int rc = launchYoloNms(batch, classes, rows, cand_cap, cand_cnt, nms_thresh, kept, kept_cap, kept_cnt, st.scratchPtr, need, stream);
    if (ordered)
    {
        MSNH_HIP_CHECK(hipEventRecord(st.done, stream));
        st.haveDone = true;
        st.lastStream = stream;
    }
    return rc;
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
