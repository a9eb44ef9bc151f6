// Bandwidth-bound NHWC layers: stand-alone batch-norm affine, residual add, channel copy (concat),
// max/avg pooling, nearest upsample, fully-connected, and the NCHW<->NHWC boundary conversions.
// Every kernel maps consecutive lanes to consecutive channel vectors of a pixel (16-byte accesses when
// the channel count, pixel strides and base addresses allow it, scalar otherwise), so global accesses
// are coalesced along the contiguous NHWC channel axis.
#include "common.hpp"

namespace msnh {

int convIgemm(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
              const void *residual, void *y, hipStream_t st, bool dryRun);


template <typename T, int VEC> struct VecOf { typedef T type __attribute__((ext_vector_type(VEC))); };
template <typename T> struct VecOf<T, 1> { typedef T type; };

template <typename T, int VEC> __device__ __forceinline__ void loadVec(const T *p, float (&v)[VEC])
{
    if constexpr (VEC == 1) { v[0] = toF(p[0]); }
    else
    {
        typedef typename VecOf<T, VEC>::type V;
        const V t = *reinterpret_cast<const V *>(p);
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = toF(t[i]);
    }
}

template <typename T, int VEC> __device__ __forceinline__ void storeVec(T *p, const float (&v)[VEC])
{
    if constexpr (VEC == 1) { p[0] = fromF<T>(v[0]); }
    else
    {
        typedef typename VecOf<T, VEC>::type V;
        V t;
#pragma unroll
        for (int i = 0; i < VEC; ++i) t[i] = fromF<T>(v[i]);
        *reinterpret_cast<V *>(p) = t;
    }
}

// ---- y = out_mul * act(x*scale[c] + shift[c]) ------------------------------------------------------
template <typename T, typename TOut, int VEC>
__global__ __launch_bounds__(256) void affineActKernel(const T *__restrict__ x, int xLd, const float *__restrict__ scale,
                                                       const float *__restrict__ shift, int act, float actParam, float outMul,
                                                       TOut *__restrict__ y, int yLd, int c, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    float v[VEC];
    loadVec<T, VEC>(x + p * xLd + c0, v);
#pragma unroll
    for (int i = 0; i < VEC; ++i)
    {
        const float sc = scale ? scale[c0 + i] : 1.f;
        const float sh = shift ? shift[c0 + i] : 0.f;
        v[i] = v[i] * sc + sh;
    }
    activateArray<VEC>(v, act, actParam);
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] *= outMul;
    storeVec<TOut, VEC>(y + p * yLd + c0, v);
}

// ---- y = out_mul * act(a_mul*a + b_mul*b) ----------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void addActKernel(const T *__restrict__ a, int aLd, float aMul, const T *__restrict__ b, int bLd,
                                                    float bMul, int act, float actParam, float outMul, T *__restrict__ y, int yLd,
                                                    int c, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    float va[VEC], vb[VEC];
    loadVec<T, VEC>(a + p * aLd + c0, va);
    loadVec<T, VEC>(b + p * bLd + c0, vb);
#pragma unroll
    for (int i = 0; i < VEC; ++i) va[i] = aMul * va[i] + bMul * vb[i];
    activateArray<VEC>(va, act, actParam);
#pragma unroll
    for (int i = 0; i < VEC; ++i) va[i] *= outMul;
    storeVec<T, VEC>(y + p * yLd + c0, va);
}

// ---- max pooling -----------------------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void maxPoolKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int ksize, int stride,
                                                     int pad, int OH, int OW, T *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    float m[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) m[i] = -FLT_MAX;
    const int y0 = oy * stride - pad, x0 = ox * stride - pad;
    const int ya = y0 < 0 ? 0 : y0, yb = (y0 + ksize > H) ? H : y0 + ksize;
    const int xa = x0 < 0 ? 0 : x0, xb = (x0 + ksize > W) ? W : x0 + ksize;
    for (int iy = ya; iy < yb; ++iy)
        for (int ix = xa; ix < xb; ++ix)
        {
            float v[VEC];
            loadVec<T, VEC>(x + ((b * H + iy) * W + ix) * xLd + c0, v);
#pragma unroll
            for (int i = 0; i < VEC; ++i) m[i] = (v[i] > m[i]) ? v[i] : m[i];
        }
    if constexpr (sizeof(T) == 2)
    {
        // a window lying entirely in the padding yields -FLT_MAX in the reference; clamp to the half range
#pragma unroll
        for (int i = 0; i < VEC; ++i) m[i] = m[i] < -65504.f ? -65504.f : m[i];
    }
    storeVec<T, VEC>(y + p * yLd + c0, m);
}

// The same for the window sizes the shipped graphs use (2, 3, 5), with the window unrolled: every load of the window is issued
// before the first comparison (a window position outside the image loads a clamped position and is ignored), where the loop
// above waits for each load in turn -- 25 dependent round trips for a 5 x 5 window.  Workgroups are dealt to the 8 XCDs in
// contiguous runs, so the rows that neighbouring output rows share are found in one L2.
template <typename T, int VEC, int K>
__global__ __launch_bounds__(256) void maxPoolUnrolledKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int stride, int pad, int OH,
                                                             int OW, T *__restrict__ y, int yLd, long long total, int blocks)
{
    const int perXcd = (blocks + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    if (logical >= blocks) return;
    const long long idx = static_cast<long long>(logical) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    const int y0 = oy * stride - pad, x0 = ox * stride - pad;
    float m[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) m[i] = -FLT_MAX;
    // one window row at a time: its K loads are in flight together, and the next row's are issued while this one is compared
#pragma unroll
    for (int ky = 0; ky < K; ++ky)
    {
        const int iy = y0 + ky;
        const bool rowOk = iy >= 0 && iy < H;
        const int cy = iy < 0 ? 0 : (iy >= H ? H - 1 : iy);
        const T *row = x + (b * H + cy) * W * xLd + c0;
        float v[K][VEC];
        bool ok[K];
#pragma unroll
        for (int kx = 0; kx < K; ++kx)
        {
            const int ix = x0 + kx;
            ok[kx] = rowOk && ix >= 0 && ix < W;
            const int cx = ix < 0 ? 0 : (ix >= W ? W - 1 : ix);
            loadVec<T, VEC>(row + static_cast<long long>(cx) * xLd, v[kx]);
        }
#pragma unroll
        for (int kx = 0; kx < K; ++kx)
#pragma unroll
            for (int i = 0; i < VEC; ++i) m[i] = (ok[kx] && v[kx][i] > m[i]) ? v[kx][i] : m[i];
    }
    if constexpr (sizeof(T) == 2)
    {
#pragma unroll
        for (int i = 0; i < VEC; ++i) m[i] = m[i] < -65504.f ? -65504.f : m[i];
    }
    storeVec<T, VEC>(y + p * yLd + c0, m);
}

// A chain of stride-1 "same" max-pools of one window size, each reading the result of the one before it (the SPP block of the YOLOv4 /
// YOLOv5 graphs: windows 5, 9 and 13 over one tensor are 5 over 5 over 5), in ONE launch: a workgroup holds the H x W tile of one
// image for CG channels in LDS, runs every pool of the chain as a row pass and a column pass over it (the maximum over a window is
// the maximum over its rows of the row maxima) and writes each result straight to its own destination.  The input crosses memory
// once instead of once per pool, and one launch replaces three whose 25-tap windows were bound by load latency on 6 MB tensors.
// Results are those of the separate launches bit for bit: a value replaces the running maximum only if it compares greater (a NaN
// never does), positions outside the image are ignored, a window without any usable value gives -FLT_MAX, float16 stores clamp that
// to the most negative finite half -- and each pool of the chain sees its predecessor's stored values.
template <typename T, int VEC, int K>
__global__ __launch_bounds__(1024) void maxPoolChainKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int cg, int steps, int blocks, T *__restrict__ y0, int y0Ld,
                                                           T *__restrict__ y1, int y1Ld, T *__restrict__ y2, int y2Ld)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char poolSmem[];
    T *bufA = reinterpret_cast<T *>(poolSmem);
    T *bufB = bufA + static_cast<size_t>(H) * W * cg;
    const int groups = (c + cg - 1) / cg;
    // workgroups are dealt to the 8 XCDs in contiguous runs: the channel groups of one image, which share every 128-byte line of
    // the tensor between two of them, meet in one L2
    const int perXcd = (blocks + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    if (logical >= blocks) return;
    const int b = logical / groups;
    const int c0 = (logical % groups) * cg;
    const int cw = ((c - c0 < cg) ? c - c0 : cg) / VEC;           // channel vectors of a pixel in this group
    const int pixels = H * W;
    const int items = pixels * cw;                                // at most 4 per thread (host)
    const long long img = static_cast<long long>(b) * pixels;
    constexpr int R = K / 2;
    constexpr int MAXI = 4;
    typedef typename VecOf<T, VEC>::type V;
    // a thread keeps the same (pixel, channel vector) items through every pass: where they sit in LDS, which neighbours of their row
    // and column exist (bit d + R of a mask), where they go in memory -- the divisions are paid once
    int ldsOff[MAXI], chan[MAXI], pix[MAXI];
    unsigned rowMask[MAXI], colMask[MAXI];
#pragma unroll
    for (int k = 0; k < MAXI; ++k)
    {
        const int i = threadIdx.x + k * 1024;
        ldsOff[k] = -1;
        chan[k] = pix[k] = 0;
        rowMask[k] = colMask[k] = 0u;
        if (i < items)
        {
            const int p = i / cw, v = i - p * cw;
            const int py = p / W, px = p - py * W;
            ldsOff[k] = p * cg + v * VEC;
            pix[k] = p;
            chan[k] = v * VEC;
#pragma unroll
            for (int d = -R; d <= R; ++d)
            {
                if (px + d >= 0 && px + d < W) rowMask[k] |= 1u << (d + R);
                if (py + d >= 0 && py + d < H) colMask[k] |= 1u << (d + R);
            }
            *reinterpret_cast<V *>(bufA + ldsOff[k]) = *reinterpret_cast<const V *>(x + (img + p) * xLd + c0 + v * VEC);
        }
    }
    __syncthreads();
    const int rowStep = cg, colStep = W * cg;
    auto pass = [&](const T *src, int step, unsigned mask, int off, float (&m)[VEC]) {
        float t[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[e] = -FLT_MAX;
#pragma unroll
        for (int d = -R; d <= R; ++d)
        {
            if (!(mask & (1u << (d + R)))) continue;
            loadVec<T, VEC>(src + off + d * step, t);
#pragma unroll
            for (int e = 0; e < VEC; ++e) m[e] = t[e] > m[e] ? t[e] : m[e];
        }
        if constexpr (sizeof(T) == 2)
        {
#pragma unroll
            for (int e = 0; e < VEC; ++e) m[e] = m[e] < -65504.f ? -65504.f : m[e];
        }
    };
    for (int s = 0; s < steps; ++s)
    {
        float m[VEC];
        // rows: A -> B
#pragma unroll
        for (int k = 0; k < MAXI; ++k)
            if (ldsOff[k] >= 0)
            {
                pass(bufA, rowStep, rowMask[k], ldsOff[k], m);
                storeVec<T, VEC>(bufB + ldsOff[k], m);
            }
        __syncthreads();
        // columns: B -> this pool's destination, and back into A for the next pool
        T *y = s == 0 ? y0 : (s == 1 ? y1 : y2);
        const int yLd = s == 0 ? y0Ld : (s == 1 ? y1Ld : y2Ld);
#pragma unroll
        for (int k = 0; k < MAXI; ++k)
            if (ldsOff[k] >= 0)
            {
                pass(bufB, colStep, colMask[k], ldsOff[k], m);
                storeVec<T, VEC>(y + (img + pix[k]) * yLd + c0 + chan[k], m);
                if (s + 1 < steps) storeVec<T, VEC>(bufA + ldsOff[k], m);
            }
        __syncthreads();
    }
}

// ---- average pooling over valid elements -------------------------------------------------------------
template <typename T, typename TOut, int VEC>
__global__ __launch_bounds__(256) void avgPoolKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int ksize, int stride,
                                                     int pad, int OH, int OW, float outMul, TOut *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    float sum[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) sum[i] = 0.f;
    int count = 0;
    for (int n = 0; n < ksize; ++n)
        for (int m = 0; m < ksize; ++m)
        {
            const int iy = oy * stride - pad + n, ix = ox * stride - pad + m;
            if (iy < 0 || iy >= H || ix < 0 || ix >= W) continue;
            float v[VEC];
            loadVec<T, VEC>(x + ((b * H + iy) * W + ix) * xLd + c0, v);
            ++count;
#pragma unroll
            for (int i = 0; i < VEC; ++i) sum[i] += v[i];
        }
#pragma unroll
    for (int i = 0; i < VEC; ++i) sum[i] = outMul * (sum[i] / static_cast<float>(count));
    storeVec<TOut, VEC>(y + p * yLd + c0, sum);
}

// One window that covers the whole image (the classifier heads: 7x7 -> 1x1): a thread per output would walk all H*W
// pixels alone, with only batch * c / VEC threads on the device.  Here a workgroup takes 16 channel vectors of one image,
// 16 threads share the pixels of each (pixel p, p + 16, ...) and their partial sums are added in a fixed order through LDS.
template <typename T, typename TOut, int VEC>
__global__ __launch_bounds__(256) void avgPoolGlobalKernel(const T *__restrict__ x, int xLd, int HW, int c, float outMul, TOut *__restrict__ y, int yLd)
{
    __shared__ float part[16][16][VEC];
    const int cl = threadIdx.x & 15, pl = threadIdx.x >> 4;
    const int cv = blockIdx.x * 16 + cl;
    const long long b = blockIdx.y;
    const bool live = cv * VEC < c;
    float sum[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) sum[i] = 0.f;
    if (live)
        for (int p = pl; p < HW; p += 16)
        {
            float v[VEC];
            loadVec<T, VEC>(x + (b * HW + p) * xLd + cv * VEC, v);
#pragma unroll
            for (int i = 0; i < VEC; ++i) sum[i] += v[i];
        }
#pragma unroll
    for (int i = 0; i < VEC; ++i) part[pl][cl][i] = sum[i];
    __syncthreads();
    if (pl != 0 || !live) return;
#pragma unroll
    for (int q = 1; q < 16; ++q)
#pragma unroll
        for (int i = 0; i < VEC; ++i) sum[i] += part[q][cl][i];
#pragma unroll
    for (int i = 0; i < VEC; ++i) sum[i] = outMul * (sum[i] / static_cast<float>(HW));
    storeVec<TOut, VEC>(y + b * yLd + cv * VEC, sum);
}

// ---- nearest upsample / channel copy -------------------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void upsampleKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int stride, float scale,
                                                      T *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int OW = W * stride, OH = H * stride;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    float v[VEC];
    loadVec<T, VEC>(x + ((b * H + oy / stride) * W + ox / stride) * xLd + c0, v);
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = scale * v[i];
    storeVec<T, VEC>(y + p * yLd + c0, v);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void copyChannelsKernel(const T *__restrict__ x, int xLd, float mul, T *__restrict__ y, int yLd, int c,
                                                          long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    float v[VEC];
    loadVec<T, VEC>(x + p * xLd + c0, v);
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = mul * v[i];
    storeVec<T, VEC>(y + p * yLd + c0, v);
}

// ---- constant padding / strided slice / bilinear resize ---------------------------------------------------------
template <typename T, int VEC>
__global__ __launch_bounds__(256) void padKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int top, int left, int OH, int OW,
                                                 float mul, float value, T *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    const int iy = oy - top, ix = ox - left;
    float v[VEC];
    if (iy >= 0 && iy < H && ix >= 0 && ix < W)
    {
        loadVec<T, VEC>(x + ((b * H + iy) * W + ix) * xLd + c0, v);
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = mul * v[i];
    }
    else
    {
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = value;
    }
    storeVec<T, VEC>(y + p * yLd + c0, v);
}

template <typename T>
__global__ __launch_bounds__(256) void sliceKernel(const T *__restrict__ x, int xLd, int H, int W, int c0, int cs, int h0, int hs, int w0, int ws,
                                                   int OC, int OH, int OW, float mul, T *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int oc = static_cast<int>(idx % OC);
    const long long p = idx / OC;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    const float v = toF(x[((b * H + h0 + oy * hs) * W + w0 + ox * ws) * xLd + c0 + oc * cs]);
    y[p * yLd + oc] = fromF<T>(mul * v);
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void bilinearKernel(const T *__restrict__ x, int xLd, int H, int W, int c, int OH, int OW, int alignCorners,
                                                      float rH, float rW, float mul, T *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    float h1r, w1r;
    if (alignCorners == 0)
    {
        const float ih = rH * (oy + 0.5f) - 0.5f;
        const float iw = rW * (ox + 0.5f) - 0.5f;
        h1r = ih < 0 ? 0 : ih;
        w1r = iw < 0 ? 0 : iw;
    }
    else
    {
        h1r = rH * oy;
        w1r = rW * ox;
    }
    const int h1 = static_cast<int>(h1r), w1 = static_cast<int>(w1r);
    const int h1p = h1 < H - 1 ? 1 : 0, w1p = w1 < W - 1 ? 1 : 0;
    const float h1L = h1r - h1, h0L = 1.f - h1L, w1L = w1r - w1, w0L = 1.f - w1L;
    const T *base = x + ((b * H + h1) * W + w1) * xLd + c0;
    float v00[VEC], v01[VEC], v10[VEC], v11[VEC], o[VEC];
    loadVec<T, VEC>(base, v00);
    loadVec<T, VEC>(base + static_cast<long long>(w1p) * xLd, v01);
    loadVec<T, VEC>(base + static_cast<long long>(h1p) * W * xLd, v10);
    loadVec<T, VEC>(base + (static_cast<long long>(h1p) * W + w1p) * xLd, v11);
#pragma unroll
    for (int i = 0; i < VEC; ++i)
        o[i] = mul * (h0L * (w0L * v00[i] + w1L * v01[i]) + h1L * (w0L * v10[i] + w1L * v11[i]));
    storeVec<T, VEC>(y + p * yLd + c0, o);
}

// ---- softmax over all values of one image --------------------------------------------------------------------
// One workgroup per image: maximum, sum of exp((x - max) / T), quotient (Blas::softmax, src/core/MsnhBlas.cpp:1970-2110).
template <typename T>
__global__ __launch_bounds__(256) void softmaxKernel(const T *__restrict__ x, int xLd, float xMul, int pixels, int c, float temperature,
                                                     T *__restrict__ y, int yLd, float yMul)
{
    __shared__ float red[256];
    const int b = blockIdx.x;
    const long long n = static_cast<long long>(pixels) * c;
    const T *xb = x + static_cast<size_t>(b) * pixels * xLd;
    T *yb = y + static_cast<size_t>(b) * pixels * yLd;
    float m = -3.402823466e38f;
    for (long long i = threadIdx.x; i < n; i += 256)
    {
        const float v = xMul * toF(xb[(i / c) * xLd + (i % c)]);
        m = v > m ? v : m;
    }
    red[threadIdx.x] = m;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1)
    {
        if (threadIdx.x < s) red[threadIdx.x] = red[threadIdx.x + s] > red[threadIdx.x] ? red[threadIdx.x + s] : red[threadIdx.x];
        __syncthreads();
    }
    const float largest = red[0];
    __syncthreads();
    float sum = 0.f;
    for (long long i = threadIdx.x; i < n; i += 256)
        sum += expf(xMul * toF(xb[(i / c) * xLd + (i % c)]) / temperature - largest / temperature);
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1)
    {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    const float total = red[0];
    for (long long i = threadIdx.x; i < n; i += 256)
    {
        const float e = expf(xMul * toF(xb[(i / c) * xLd + (i % c)]) / temperature - largest / temperature);
        yb[(i / c) * yLd + (i % c)] = fromF<T>(yMul * (e / total));
    }
}

// ---- transposed convolution, second half: gather of the per-tap products ------------------------------------------
// cols[b][y][x][(ky*k + kx)*C + c] holds, for input pixel (y, x), the product of the input vector with the weights of tap
// (ky, kx) (a 1x1 convolution with k*k*C outputs).  Output pixel (oy, ox) sums the taps whose source pixel
// ((oy + pad - ky) / stride, (ox + pad - kx) / stride) exists, in (ky, kx) order -- the order in which
// Gemm::cpuCol2Im accumulates them (src/core/MsnhGemm.cpp:115-154) -- then bias and activation
// (DeConvolutionalLayer::forward, src/layers/MsnhDeConvolutionalLayer.cpp:140-200).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void col2imKernel(const T *__restrict__ cols, int colsLd, float colsMul, int H, int W, int c, int ksize, int stride,
                                                    int pad, int OH, int OW, const float *__restrict__ bias, int act, float actParam, float outMul,
                                                    T *__restrict__ y, int yLd, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = c / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    const long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const long long b = t / OH;
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    for (int ky = 0; ky < ksize; ++ky)
    {
        const int ny = oy + pad - ky;
        if (ny < 0 || ny % stride != 0 || ny / stride >= H) continue;
        for (int kx = 0; kx < ksize; ++kx)
        {
            const int nx = ox + pad - kx;
            if (nx < 0 || nx % stride != 0 || nx / stride >= W) continue;
            float v[VEC];
            loadVec<T, VEC>(cols + ((b * H + ny / stride) * W + nx / stride) * colsLd + (ky * ksize + kx) * c + c0, v);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += v[i];
        }
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = colsMul * acc[i] + (bias ? bias[c0 + i] : 0.f);
    activateArray<VEC>(acc, act, actParam);
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] *= outMul;
    storeVec<T, VEC>(y + p * yLd + c0, acc);
}

// ---- fully connected: one wavefront per (batch row, output), wave-level reduction -------------------------
template <typename T>
__global__ __launch_bounds__(256) void connectedKernel(const T *__restrict__ x, float xMul, const T *__restrict__ w,
                                                       const float *__restrict__ bias, int act, float actParam, float *__restrict__ y,
                                                       int batch, int inputs, int outputs)
{
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (wave >= batch * outputs) return;
    const int b = wave / outputs, o = wave - b * outputs;
    const T *xp = x + static_cast<size_t>(b) * inputs;
    const T *wp = w + static_cast<size_t>(o) * inputs;
    float sum = 0.f;
    for (int i = lane; i < inputs; i += 64) sum += toF(xp[i]) * toF(wp[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0)
    {
        float v = sum * xMul + (bias ? bias[o] : 0.f);
        y[static_cast<size_t>(b) * outputs + o] = activate(v, act, actParam);
    }
}

// ---- boundary layout conversions (tiled transposes through LDS) --------------------------------------------
// NCHW float32 -> NHWC T.  Block handles 32 pixels x 32 channels of one image.
template <typename T>
__global__ __launch_bounds__(256) void nchwToNhwcKernel(const float *__restrict__ x, float mul, T *__restrict__ y, int yLd, int C, int HW)
{
    __shared__ float tile[32][33];
    const int b = blockIdx.z;
    const int p0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;          // 32 x 8
    for (int i = ty; i < 32; i += 8)
    {
        const int c = c0 + i, p = p0 + tx;
        tile[i][tx] = (c < C && p < HW) ? x[(static_cast<size_t>(b) * C + c) * HW + p] : 0.f;
    }
    __syncthreads();
    for (int i = ty; i < 32; i += 8)
    {
        const int p = p0 + i, c = c0 + tx;
        if (p < HW && c < C) y[(static_cast<size_t>(b) * HW + p) * yLd + c] = fromF<T>(mul * tile[tx][i]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void nhwcToNchwKernel(const T *__restrict__ x, int xLd, float mul, float *__restrict__ y, int C, int HW)
{
    __shared__ float tile[32][33];
    const int b = blockIdx.z;
    const int p0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int i = ty; i < 32; i += 8)
    {
        const int p = p0 + i, c = c0 + tx;
        tile[i][tx] = (p < HW && c < C) ? toF(x[(static_cast<size_t>(b) * HW + p) * xLd + c]) : 0.f;
    }
    __syncthreads();
    for (int i = ty; i < 32; i += 8)
    {
        const int c = c0 + i, p = p0 + tx;
        if (c < C && p < HW) y[(static_cast<size_t>(b) * C + c) * HW + p] = mul * tile[tx][i];
    }
}

// Picks the widest vector every participating tensor supports.
static int pickVec(int dtype, int c, std::initializer_list<int> lds, std::initializer_list<const void *> ptrs)
{
    const int vec = dtype == MSNH_F16 ? 8 : 4;
    if (c % vec) return 1;
    for (int ld : lds) if (ld % vec) return 1;
    for (const void *p : ptrs) if (p && reinterpret_cast<uintptr_t>(p) % 16) return 1;
    return vec;
}

} // namespace msnh

using namespace msnh;

#define MSNH_CHECK_COMMON(name, pixels, c)                                                           \
    MSNH_REQUIRE((pixels) > 0 && (c) > 0, name ": non-positive size");                              \
    MSNH_REQUIRE(static_cast<long long>(pixels) * (c) < (1LL << 40), name ": tensor too large")

extern "C" {

int msnh_hip_affine_act(int dtype, int out_dtype, long long pixels, int c, const void *x, int x_ld, const float *scale,
                        const float *shift, int act, float act_param, float out_mul, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype) && dtypeOk(out_dtype), "affine_act: bad dtype");
    MSNH_CHECK_COMMON("affine_act", pixels, c);
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c && actOk(act), "affine_act: bad argument");
    hipStream_t st = resolveStream(s);
    int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    if (dtype != out_dtype) vec = (vec > 1 && c % 8 == 0 && x_ld % 8 == 0 && y_ld % 8 == 0) ? 4 : 1;
    const long long total = pixels * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_AFF(T, TO, V)                                                                                                     \
    hipLaunchKernelGGL((affineActKernel<T, TO, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, scale, shift, act, \
                       act_param, out_mul, static_cast<TO *>(y), y_ld, c, total)
    if (dtype == MSNH_F16 && out_dtype == MSNH_F16) { if (vec == 8) MSNH_AFF(f16, f16, 8); else MSNH_AFF(f16, f16, 1); }
    else if (dtype == MSNH_F32 && out_dtype == MSNH_F32) { if (vec == 4) MSNH_AFF(float, float, 4); else MSNH_AFF(float, float, 1); }
    else if (dtype == MSNH_F16) { if (vec == 4) MSNH_AFF(f16, float, 4); else MSNH_AFF(f16, float, 1); }
    else { if (vec == 4) MSNH_AFF(float, f16, 4); else MSNH_AFF(float, f16, 1); }
#undef MSNH_AFF
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_add_act(int dtype, long long pixels, int c, const void *a, int a_ld, float a_mul, const void *b, int b_ld,
                     float b_mul, int act, float act_param, float out_mul, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "add_act: bad dtype");
    MSNH_CHECK_COMMON("add_act", pixels, c);
    MSNH_REQUIRE(a && b && y && a_ld >= c && b_ld >= c && y_ld >= c && actOk(act), "add_act: bad argument");
    hipStream_t st = resolveStream(s);
    const int vec = pickVec(dtype, c, {a_ld, b_ld, y_ld}, {a, b, y});
    const long long total = pixels * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_ADD(T, V)                                                                                                          \
    hipLaunchKernelGGL((addActKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(a), a_ld, a_mul, static_cast<const T *>(b), \
                       b_ld, b_mul, act, act_param, out_mul, static_cast<T *>(y), y_ld, c, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_ADD(f16, 8); else MSNH_ADD(f16, 1); }
    else { if (vec == 4) MSNH_ADD(float, 4); else MSNH_ADD(float, 1); }
#undef MSNH_ADD
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_copy_channels(int dtype, long long pixels, int c, const void *x, int x_ld, float mul, void *y, int y_ld,
                           msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "copy_channels: bad dtype");
    MSNH_CHECK_COMMON("copy_channels", pixels, c);
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c, "copy_channels: bad argument");
    hipStream_t st = resolveStream(s);
    const int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    const long long total = pixels * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_CPY(T, V)                                                                                                   \
    hipLaunchKernelGGL((copyChannelsKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, mul, static_cast<T *>(y), \
                       y_ld, c, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_CPY(f16, 8); else MSNH_CPY(f16, 1); }
    else { if (vec == 4) MSNH_CPY(float, 4); else MSNH_CPY(float, 1); }
#undef MSNH_CPY
    MSNH_LAUNCH_CHECK();
    return 0;
}

static int checkPool(const char *name, int batch, int in_h, int in_w, int c, int ksize, int stride, int pad, int out_h, int out_w)
{
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && c > 0 && ksize > 0 && stride > 0 && pad >= 0, "%s: bad geometry", name);
    // (a single window that covers the whole plane may overhang the shorter axis: the global mean of a non-square plane)
    MSNH_REQUIRE((in_h + 2 * pad >= ksize && in_w + 2 * pad >= ksize) || (out_h == 1 && out_w == 1 && pad == 0),
                 "%s: window larger than padded input", name);
    MSNH_REQUIRE(out_h > 0 && out_w > 0, "%s: non-positive output size", name);
    // every window must start inside the padded input (covers floor and ceil output sizes)
    MSNH_REQUIRE((out_h - 1) * stride - pad < in_h && (out_w - 1) * stride - pad < in_w, "%s: output size too large", name);
    return 0;
}

int msnh_hip_maxpool(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int ksize, int stride,
                     int pad, int out_h, int out_w, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "maxpool: bad dtype");
    if (checkPool("maxpool", batch, in_h, in_w, c, ksize, stride, pad, out_h, out_w)) return 2;
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c, "maxpool: bad argument");
    hipStream_t st = resolveStream(s);
    const int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    const long long total = static_cast<long long>(batch) * out_h * out_w * (c / vec);
    dim3 grid(gridFor(total, 256));
    if ((ksize == 2 || ksize == 3 || ksize == 5) && vec > 1)
    {
        const int blocks = static_cast<int>(grid.x);
        const dim3 xgrid((blocks + 7) / 8 * 8);
#define MSNH_MPU(T, V, K)                                                                                               \
        hipLaunchKernelGGL((maxPoolUnrolledKernel<T, V, K>), xgrid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, stride, \
                           pad, out_h, out_w, static_cast<T *>(y), y_ld, total, blocks)
#define MSNH_MPUK(T, V) do { if (ksize == 2) MSNH_MPU(T, V, 2); else if (ksize == 3) MSNH_MPU(T, V, 3); else MSNH_MPU(T, V, 5); } while (0)
        if (dtype == MSNH_F16) MSNH_MPUK(f16, 8); else MSNH_MPUK(float, 4);
#undef MSNH_MPUK
#undef MSNH_MPU
        MSNH_LAUNCH_CHECK();
        return 0;
    }
#define MSNH_MP(T, V)                                                                                                  \
    hipLaunchKernelGGL((maxPoolKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, ksize, stride, \
                       pad, out_h, out_w, static_cast<T *>(y), y_ld, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_MP(f16, 8); else MSNH_MP(f16, 1); }
    else { if (vec == 4) MSNH_MP(float, 4); else MSNH_MP(float, 1); }
#undef MSNH_MP
    MSNH_LAUNCH_CHECK();
    return 0;
}

// channels per workgroup of the chained max-pool for this geometry (two H x W tiles of them must fit 48 KiB of LDS); 0 = not taken
static int poolChainGroup(int dtype, int in_h, int in_w, int c, int ksize, int steps)
{
    const int vec = dtype == MSNH_F16 ? 8 : 4;
    const size_t es = dtype == MSNH_F16 ? 2 : 4;
    if (!(ksize == 3 || ksize == 5) || steps < 2 || steps > 3 || c % vec != 0) return 0;
    // two tiles in at most 48 KiB of LDS, and at most 4 (pixel, channel vector) items for each of the 1024 threads
    for (int cg = 64; cg >= vec; cg /= 2)
        if (2 * static_cast<size_t>(in_h) * in_w * cg * es <= 48 * 1024 && static_cast<long long>(in_h) * in_w * (cg / vec) <= 4096) return cg;
    return 0;
}

int msnh_hip_maxpool_chain_supported(int dtype, int in_h, int in_w, int c, int ksize, int steps)
{
    return dtypeOk(dtype) && in_h > 0 && in_w > 0 && c > 0 && poolChainGroup(dtype, in_h, in_w, c, ksize, steps) > 0 ? 1 : 0;
}

int msnh_hip_maxpool_chain(int dtype, int batch, int in_h, int in_w, int c, int ksize, int steps, const void *x, int x_ld, void *const *y,
                           const int *y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "maxpool_chain: bad dtype");
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && c > 0 && x && y && y_ld && x_ld >= c, "maxpool_chain: bad argument");
    const int cg = poolChainGroup(dtype, in_h, in_w, c, ksize, steps);
    MSNH_REQUIRE(cg > 0, "maxpool_chain: windows of 3 or 5, 2 or 3 pools, channels a multiple of the 16-byte vector, and an H x W tile that fits LDS "
                         "(msnh_hip_maxpool_chain_supported)");
    const int vec = dtype == MSNH_F16 ? 8 : 4;
    MSNH_REQUIRE(x_ld % vec == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0, "maxpool_chain: input must be 16-byte aligned with a row stride of whole vectors");
    for (int i = 0; i < steps; ++i)
        MSNH_REQUIRE(y[i] && y_ld[i] >= c && y_ld[i] % vec == 0 && reinterpret_cast<uintptr_t>(y[i]) % 16 == 0,
                     "maxpool_chain: every destination must be 16-byte aligned with a row stride of whole vectors");
    const long long blocks = static_cast<long long>(batch) * ((c + cg - 1) / cg);
    MSNH_REQUIRE(blocks < (1LL << 31), "maxpool_chain: too many tiles");
    hipStream_t st = resolveStream(s);
    const size_t smem = 2 * static_cast<size_t>(in_h) * in_w * cg * (dtype == MSNH_F16 ? 2 : 4);
    void *y2 = steps > 2 ? y[2] : y[1];
    const int y2Ld = steps > 2 ? y_ld[2] : y_ld[1];
#define MSNH_MPC(T, V, K)                                                                                              \
    hipLaunchKernelGGL((maxPoolChainKernel<T, V, K>), dim3(static_cast<unsigned>((blocks + 7) / 8 * 8)), dim3(1024), smem, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, cg, \
                       steps, static_cast<int>(blocks), static_cast<T *>(y[0]), y_ld[0], static_cast<T *>(y[1]), y_ld[1], static_cast<T *>(y2), y2Ld)
    if (dtype == MSNH_F16) { if (ksize == 3) MSNH_MPC(f16, 8, 3); else MSNH_MPC(f16, 8, 5); }
    else { if (ksize == 3) MSNH_MPC(float, 4, 3); else MSNH_MPC(float, 4, 5); }
#undef MSNH_MPC
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_avgpool(int dtype, int out_dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int ksize,
                     int stride, int pad, int out_h, int out_w, float out_mul, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype) && dtypeOk(out_dtype), "avgpool: bad dtype");
    MSNH_REQUIRE(!(dtype == MSNH_F32 && out_dtype == MSNH_F16), "avgpool: float32 -> float16 not supported");
    if (checkPool("avgpool", batch, in_h, in_w, c, ksize, stride, pad, out_h, out_w)) return 2;
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c, "avgpool: bad argument");
    hipStream_t st = resolveStream(s);
    int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    if (dtype != out_dtype) vec = (vec > 1 && y_ld % 8 == 0) ? 4 : 1;
    if (out_h == 1 && out_w == 1 && pad == 0 && ksize >= in_h && ksize >= in_w && batch <= 65535)
    {
        dim3 ggrid((c / vec + 15) / 16, batch);
#define MSNH_APG(T, TO, V)                                                                                             \
        hipLaunchKernelGGL((avgPoolGlobalKernel<T, TO, V>), ggrid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h * in_w, c, out_mul,  \
                           static_cast<TO *>(y), y_ld)
        if (dtype == MSNH_F16 && out_dtype == MSNH_F16) { if (vec == 8) MSNH_APG(f16, f16, 8); else MSNH_APG(f16, f16, 1); }
        else if (dtype == MSNH_F16) { if (vec == 4) MSNH_APG(f16, float, 4); else MSNH_APG(f16, float, 1); }
        else { if (vec == 4) MSNH_APG(float, float, 4); else MSNH_APG(float, float, 1); }
#undef MSNH_APG
        MSNH_LAUNCH_CHECK();
        return 0;
    }
    const long long total = static_cast<long long>(batch) * out_h * out_w * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_AP(T, TO, V)                                                                                              \
    hipLaunchKernelGGL((avgPoolKernel<T, TO, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, ksize,  \
                       stride, pad, out_h, out_w, out_mul, static_cast<TO *>(y), y_ld, total)
    if (dtype == MSNH_F16 && out_dtype == MSNH_F16) { if (vec == 8) MSNH_AP(f16, f16, 8); else MSNH_AP(f16, f16, 1); }
    else if (dtype == MSNH_F16) { if (vec == 4) MSNH_AP(f16, float, 4); else MSNH_AP(f16, float, 1); }
    else { if (vec == 4) MSNH_AP(float, float, 4); else MSNH_AP(float, float, 1); }
#undef MSNH_AP
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_upsample_nearest(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int stride,
                              float scale, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "upsample: bad dtype");
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && c > 0 && stride > 0, "upsample: bad geometry");
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c, "upsample: bad argument");
    hipStream_t st = resolveStream(s);
    const int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    const long long total = static_cast<long long>(batch) * in_h * stride * in_w * stride * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_UP(T, V)                                                                                                  \
    hipLaunchKernelGGL((upsampleKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, stride, scale, \
                       static_cast<T *>(y), y_ld, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_UP(f16, 8); else MSNH_UP(f16, 1); }
    else { if (vec == 4) MSNH_UP(float, 4); else MSNH_UP(float, 1); }
#undef MSNH_UP
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_pad(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int top, int left, int out_h,
                 int out_w, float mul, float value, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "pad: bad dtype");
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && c > 0 && top >= 0 && left >= 0 && out_h >= in_h + top && out_w >= in_w + left, "pad: bad geometry");
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c, "pad: bad argument");
    hipStream_t st = resolveStream(s);
    const int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    const long long total = static_cast<long long>(batch) * out_h * out_w * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_PAD(T, V)                                                                                                 \
    hipLaunchKernelGGL((padKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, top, left, out_h, out_w, \
                       mul, value, static_cast<T *>(y), y_ld, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_PAD(f16, 8); else MSNH_PAD(f16, 1); }
    else { if (vec == 4) MSNH_PAD(float, 4); else MSNH_PAD(float, 1); }
#undef MSNH_PAD
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_slice(int dtype, int batch, int in_h, int in_w, const void *x, int x_ld, int c0, int cs, int h0, int hs, int w0,
                   int ws, int out_c, int out_h, int out_w, float mul, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "slice: bad dtype");
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && out_c > 0 && out_h > 0 && out_w > 0 && c0 >= 0 && h0 >= 0 && w0 >= 0 && cs > 0 && hs > 0 && ws > 0,
                 "slice: bad geometry");
    MSNH_REQUIRE(h0 + (out_h - 1) * hs < in_h && w0 + (out_w - 1) * ws < in_w && c0 + (out_c - 1) * cs < x_ld, "slice: window leaves the tensor");
    MSNH_REQUIRE(x && y && y_ld >= out_c, "slice: bad argument");
    hipStream_t st = resolveStream(s);
    const long long total = static_cast<long long>(batch) * out_h * out_w * out_c;
    dim3 grid(gridFor(total, 256));
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((sliceKernel<f16>), grid, dim3(256), 0, st, static_cast<const f16 *>(x), x_ld, in_h, in_w, c0, cs, h0, hs, w0, ws, out_c, out_h,
                           out_w, mul, static_cast<f16 *>(y), y_ld, total);
    else
        hipLaunchKernelGGL((sliceKernel<float>), grid, dim3(256), 0, st, static_cast<const float *>(x), x_ld, in_h, in_w, c0, cs, h0, hs, w0, ws, out_c,
                           out_h, out_w, mul, static_cast<float *>(y), y_ld, total);
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_upsample_bilinear(int dtype, int batch, int in_h, int in_w, int c, const void *x, int x_ld, int out_h, int out_w,
                               int align_corners, float mul, void *y, int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "bilinear: bad dtype");
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && c > 0 && out_h > 0 && out_w > 0, "bilinear: w*x and outw*outx must > 1");
    MSNH_REQUIRE(x && y && x_ld >= c && y_ld >= c, "bilinear: bad argument");
    hipStream_t st = resolveStream(s);
    const float rH = align_corners == 0 ? 1.0f * in_h / out_h : 1.0f * (in_h - 1) / (out_h - 1);
    const float rW = align_corners == 0 ? 1.0f * in_w / out_w : 1.0f * (in_w - 1) / (out_w - 1);
    const int vec = pickVec(dtype, c, {x_ld, y_ld}, {x, y});
    const long long total = static_cast<long long>(batch) * out_h * out_w * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_BIL(T, V)                                                                                                 \
    hipLaunchKernelGGL((bilinearKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), x_ld, in_h, in_w, c, out_h, out_w, align_corners, \
                       rH, rW, mul, static_cast<T *>(y), y_ld, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_BIL(f16, 8); else MSNH_BIL(f16, 1); }
    else { if (vec == 4) MSNH_BIL(float, 4); else MSNH_BIL(float, 1); }
#undef MSNH_BIL
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_softmax(int dtype, int batch, int pixels, int c, const void *x, int x_ld, float x_mul, float temperature, void *y,
                     int y_ld, float y_mul, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "softmax: bad dtype");
    MSNH_REQUIRE(batch > 0 && pixels > 0 && c > 0 && x && y && x_ld >= c && y_ld >= c && temperature != 0.f, "softmax: bad argument");
    hipStream_t st = resolveStream(s);
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((softmaxKernel<f16>), dim3(batch), dim3(256), 0, st, static_cast<const f16 *>(x), x_ld, x_mul, pixels, c, temperature,
                           static_cast<f16 *>(y), y_ld, y_mul);
    else
        hipLaunchKernelGGL((softmaxKernel<float>), dim3(batch), dim3(256), 0, st, static_cast<const float *>(x), x_ld, x_mul, pixels, c, temperature,
                           static_cast<float *>(y), y_ld, y_mul);
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_deconv_col2im(int dtype, int batch, int in_h, int in_w, int c, int ksize, int stride, int pad, const void *cols, int cols_ld,
                           float cols_mul, const float *bias, int act, float act_param, int out_h, int out_w, float out_mul, void *y,
                           int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "deconv_col2im: bad dtype");
    MSNH_REQUIRE(batch > 0 && in_h > 0 && in_w > 0 && c > 0 && ksize > 0 && stride > 0 && pad >= 0 && actOk(act), "deconv_col2im: bad geometry");
    MSNH_REQUIRE(out_h == (in_h - 1) * stride - 2 * pad + ksize && out_w == (in_w - 1) * stride - 2 * pad + ksize && out_h > 0 && out_w > 0,
                 "deconv_col2im: out size does not match geometry");
    MSNH_REQUIRE(cols && y && cols_ld >= ksize * ksize * c && y_ld >= c, "deconv_col2im: bad argument");
    hipStream_t st = resolveStream(s);
    const int vec = pickVec(dtype, c, {cols_ld, y_ld}, {cols, y});
    const long long total = static_cast<long long>(batch) * out_h * out_w * (c / vec);
    dim3 grid(gridFor(total, 256));
#define MSNH_C2I(T, V)                                                                                                 \
    hipLaunchKernelGGL((col2imKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(cols), cols_ld, cols_mul, in_h, in_w, c, ksize, stride, \
                       pad, out_h, out_w, bias, act, act_param, out_mul, static_cast<T *>(y), y_ld, total)
    if (dtype == MSNH_F16) { if (vec == 8) MSNH_C2I(f16, 8); else MSNH_C2I(f16, 1); }
    else { if (vec == 4) MSNH_C2I(float, 4); else MSNH_C2I(float, 1); }
#undef MSNH_C2I
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_connected(int dtype, int batch, int inputs, int outputs, const void *x, float x_mul, const void *w,
                       const float *bias, int act, float act_param, float *y, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "connected: bad dtype");
    MSNH_REQUIRE(batch > 0 && inputs > 0 && outputs > 0 && x && w && y && actOk(act), "connected: bad argument");
    hipStream_t st = resolveStream(s);
    // With a real batch this is a GEMM [outputs x inputs] x [inputs x batch]: the 1x1 case of the implicit-GEMM
    // convolution (batch "pixels"), which reads the weights once instead of once per image.
    const int vec = dtype == MSNH_F16 ? 8 : 4;
    if (batch >= 8 && x_mul == 1.f && inputs % vec == 0 && outputs % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 32 == 0)
    {
        msnh_conv_desc d;
        std::memset(&d, 0, sizeof(d));
        d.dtype = dtype; d.out_dtype = MSNH_F32;
        d.batch = batch; d.in_h = 1; d.in_w = 1; d.in_c = inputs; d.in_ld = inputs;
        d.out_c = outputs; d.out_h = 1; d.out_w = 1; d.out_ld = outputs;
        d.ksize = 1; d.stride = 1; d.pad = 0; d.dilation = 1; d.groups = 1;
        d.act = act; d.act_param = act_param; d.has_residual = 0; d.res_ld = outputs; d.act2 = MSNH_ACT_NONE; d.act2_param = 0.f;
        d.res_mul = 1.f; d.out_mul = 1.f; d.algo = MSNH_CONV_IGEMM;
        d.tile = batch <= 64 ? 12 : 0;           // 64 x 64 tile for small batches, else the default by output count
        return convIgemm(&d, x, w, nullptr, bias, nullptr, y, st, false);
    }
    const long long waves = static_cast<long long>(batch) * outputs;
    dim3 grid(gridFor(waves * 64, 256));
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((connectedKernel<f16>), grid, dim3(256), 0, st, static_cast<const f16 *>(x), x_mul, static_cast<const f16 *>(w),
                           bias, act, act_param, y, batch, inputs, outputs);
    else
        hipLaunchKernelGGL((connectedKernel<float>), grid, dim3(256), 0, st, static_cast<const float *>(x), x_mul,
                           static_cast<const float *>(w), bias, act, act_param, y, batch, inputs, outputs);
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_nchw_to_nhwc(int out_dtype, int batch, int c, int h, int w, const float *x_nchw, float mul, void *y,
                          int y_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(out_dtype), "nchw_to_nhwc: bad dtype");
    MSNH_REQUIRE(batch > 0 && c > 0 && h > 0 && w > 0 && x_nchw && y && y_ld >= c, "nchw_to_nhwc: bad argument");
    MSNH_REQUIRE(batch <= 65535 && (c + 31) / 32 <= 65535, "nchw_to_nhwc: grid too large");
    hipStream_t st = resolveStream(s);
    const int hw = h * w;
    dim3 grid((hw + 31) / 32, (c + 31) / 32, batch);
    if (out_dtype == MSNH_F16)
        hipLaunchKernelGGL((nchwToNhwcKernel<f16>), grid, dim3(256), 0, st, x_nchw, mul, static_cast<f16 *>(y), y_ld, c, hw);
    else
        hipLaunchKernelGGL((nchwToNhwcKernel<float>), grid, dim3(256), 0, st, x_nchw, mul, static_cast<float *>(y), y_ld, c, hw);
    MSNH_LAUNCH_CHECK();
    return 0;
}

int msnh_hip_nhwc_to_nchw(int dtype, int batch, int c, int h, int w, const void *x, int x_ld, float mul, float *y_nchw,
                          msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "nhwc_to_nchw: bad dtype");
    MSNH_REQUIRE(batch > 0 && c > 0 && h > 0 && w > 0 && x && y_nchw && x_ld >= c, "nhwc_to_nchw: bad argument");
    MSNH_REQUIRE(batch <= 65535 && (c + 31) / 32 <= 65535, "nhwc_to_nchw: grid too large");
    hipStream_t st = resolveStream(s);
    const int hw = h * w;
    dim3 grid((hw + 31) / 32, (c + 31) / 32, batch);
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((nhwcToNchwKernel<f16>), grid, dim3(256), 0, st, static_cast<const f16 *>(x), x_ld, mul, y_nchw, c, hw);
    else
        hipLaunchKernelGGL((nhwcToNchwKernel<float>), grid, dim3(256), 0, st, static_cast<const float *>(x), x_ld, mul, y_nchw, c, hw);
    MSNH_LAUNCH_CHECK();
    return 0;
}

}
