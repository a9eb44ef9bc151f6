// YOLO v3/v4/v5 head decode fused with the [anchor][channel][pixel] -> [anchor][pixel][channel] reordering and
// the objectness threshold.  The NHWC head tensor already stores the (5+classes) values of one anchor of
// one pixel contiguously, so both the read and the write of a wavefront are contiguous runs.
#include "common.hpp"

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
// (what yoloGatherKernel derives from the decoded row).  One wavefront per candidate: lane l decodes values l, l + 64, ...;
// the best class is the first maximum in channel order, found with a wavefront reduction on (score, index).
template <typename T, bool V5>
__global__ __launch_bounds__(256) void yoloRowsKernel(const T *__restrict__ x, int xLd, float xMul, Anchors an, float ratio,
                                                      float *__restrict__ decoded, long long decStride, const int *__restrict__ candIdx, int candCap,
                                                      int candBase, const int *__restrict__ candCnt, float *__restrict__ rows, int W, int HW, int per)
{
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int n = candCnt[b];
    n = n < candCap ? n : candCap;
    for (int k = blockIdx.x * 4 + wave; k < n; k += gridDim.x * 4)
    {
        const int cellG = candIdx[static_cast<size_t>(b) * candCap + k];
        const int cell = cellG - candBase;
        if (cell < 0 || cell >= 3 * HW) continue;                // another head's candidate
        const int a = cell / HW, p = cell - a * HW;
        const int py = p / W, px = p - py * W;
        const T *xr = x + (static_cast<size_t>(b) * HW + p) * xLd + a * per;
        float *dr = decoded + static_cast<size_t>(b) * decStride + static_cast<size_t>(cell) * per;
        float first = 0.f;                                       // this lane's value of m = lane (box and objectness live in lanes 0..4)
        float bv = -3.402823466e38f * 2.f;                       // -inf: NaN scores are never selected
        int bi = 0x7fffffff;
        for (int m = lane; m < per; m += 64)
        {
            const float v = yoloDecodeOne<V5>(xMul * toF(xr[m]), m, px, py, a, an, ratio);
            dr[m] = v;
            if (m == lane) first = v;
            if (m >= 5 && v > bv) { bv = v; bi = m - 5; }
        }
        if (rows == nullptr) continue;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
        {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        // a NaN score of class 0 absorbs the sequential scan of the reference (nothing compares greater than it)
        const float c0v = __shfl(first, 5, 64);
        if (c0v != c0v) { bv = c0v; bi = 0; }
        if (bi == 0x7fffffff) bi = 0;
        float *o = rows + (static_cast<size_t>(b) * candCap + k) * 8;
        if (lane < 5) o[lane] = first;
        else if (lane == 5) o[5] = bv;
        else if (lane == 6) o[6] = static_cast<float>(bi);
        else if (lane == 7) o[7] = static_cast<float>(cellG);
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
    MSNH_REQUIRE(x && decoded && anchors6 && cand_idx && cand_cnt && cand_cap > 0 && x_ld >= 3 * per, "yolo_decode_candidates: bad argument");
    MSNH_REQUIRE(decoded_batch_stride >= static_cast<long long>(3) * h * w * per, "yolo_decode_candidates: decoded_batch_stride too small");
    Anchors an;
    for (int i = 0; i < 6; ++i) an.v[i] = anchors6[i];
    hipStream_t st = resolveStream(s);
    const int HW = h * w;
    dim3 sgrid((3 * HW + 255) / 256, batch), rgrid(128, batch);
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
