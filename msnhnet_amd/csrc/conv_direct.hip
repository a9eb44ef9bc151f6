// Convolution entry point of the C ABI plus the non-GEMM algorithms:
//   DIRECT    : one thread per output element, any geometry -- the fallback every shape can use;
//   DEPTHWISE : groups == channels; bandwidth-bound, one thread per (pixel, channel vector);
//   STEM      : first layer with <= 4 input channels, reads the NCHW float32 network input directly
//               (layout conversion and dtype cast fused) and writes NHWC.
// Host-side weight packing and algorithm selection live here too.
#include "common.hpp"
#include <vector>

namespace msnh {

int convIgemm(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
              const void *residual, void *y, hipStream_t st, bool dryRun);
int convIgemmTail(const msnh_conv_desc *d, const msnh_conv_tail_desc *tail, const void *x, const void *w, const float *scale, const float *shift,
                  const void *residual, void *y, const void *w2, const float *scale2, const float *shift2, void *z, hipStream_t st, bool dryRun);
int igemmTailTileFirst();
int convIgemmWs(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
                const void *residual, void *y, hipStream_t st, bool dryRun, void *splitWs, size_t splitWsBytes);
size_t igemmSplitKWorkspaceBytes(const msnh_conv_desc *d);
bool pointwiseOk(const msnh_conv_desc *d);
int convPointwise(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, const void *residual,
                  void *y, hipStream_t st);
int igemmTileCount();
int convWinograd(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
                 const void *residual, void *y, void *ws, size_t wsBytes, hipStream_t st);
size_t winogradWorkspaceBytes(const msnh_conv_desc *d);
void   winogradPackWeights(const msnh_conv_desc *d, const float *oihw, void *packed);
void   winogradGemmDesc(const msnh_conv_desc *d, msnh_conv_desc *gd);
bool   winogradFusedOk(const msnh_conv_desc *d);
int convWinogradFused(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, const void *residual, void *y,
                      hipStream_t st);
bool   depthwise3x3Ok(const msnh_conv_desc *d, const void *x, const void *w, const void *y);
int    convDepthwise3x3(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, void *y, hipStream_t st);
bool   stemMfmaOk(const msnh_conv_desc *d);
size_t stemMfmaElems(const msnh_conv_desc *d);
void   stemMfmaPack(const msnh_conv_desc *d, const float *oihw, _Float16 *packed);
int    convStemMfma(const msnh_conv_desc *d, const float *x, const _Float16 *wA, const float *scale, const float *shift, void *y, hipStream_t st);

struct EpiArgs
{
    const float *scale;
    const float *shift;
    int   act, act2, hasRes;
    float actParam, act2Param, resMul, outMul;
};

__device__ __forceinline__ float epilogue(const EpiArgs &e, float acc, int ch, float res)
{
    const float sc = e.scale ? e.scale[ch] : 1.f;
    const float sh = e.shift ? e.shift[ch] : 0.f;
    float v = activate(acc * sc + sh, e.act, e.actParam);
    if (e.hasRes) v = activate(v + e.resMul * res, e.act2, e.act2Param);
    return e.outMul * v;
}

// ---- DIRECT ---------------------------------------------------------------------------------------
template <typename T, typename TOut>
__global__ __launch_bounds__(256) void convDirectKernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ res,
                                                        TOut *__restrict__ y, EpiArgs e, int H, int W, int inLd, int OH, int OW,
                                                        int outLd, int resLd, int cinG, int coutG, int outC, int ksize, int stride,
                                                        int pad, int dil, long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int oc = static_cast<int>(idx % outC);
    long long p = idx / outC;
    const int ox = static_cast<int>(p % OW);
    long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const int b  = static_cast<int>(t / OH);
    const int g  = oc / coutG;
    const T *wp = w + static_cast<size_t>(oc) * ksize * ksize * cinG;
    float acc = 0.f;
    for (int ki = 0; ki < ksize; ++ki)
    {
        const int iy = oy * stride - pad + ki * dil;
        if (iy < 0 || iy >= H) continue;
        for (int kj = 0; kj < ksize; ++kj)
        {
            const int ix = ox * stride - pad + kj * dil;
            if (ix < 0 || ix >= W) continue;
            const T *xp = x + ((static_cast<size_t>(b) * H + iy) * W + ix) * inLd + g * cinG;
            const T *wt = wp + (ki * ksize + kj) * cinG;
            for (int c = 0; c < cinG; ++c) acc += toF(xp[c]) * toF(wt[c]);
        }
    }
    const float r = e.hasRes ? toF(res[static_cast<size_t>(p) * resLd + oc]) : 0.f;
    y[static_cast<size_t>(p) * outLd + oc] = fromF<TOut>(epilogue(e, acc, oc, r));
}

// Register-blocked variant for out_c/groups % 8 == 0: a lane owns one output pixel and 8 consecutive output channels
// (blockIdx.y picks the channel block, so the weight addresses are uniform over a wavefront and every input value
// fetched feeds 8 multiply-adds); one 8-channel NHWC store per lane.
template <typename T, typename TOut>
__global__ __launch_bounds__(256) void convDirectBlockedKernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ res,
                                                               TOut *__restrict__ y, EpiArgs e, int H, int W, int inLd, int OH, int OW,
                                                               int outLd, int resLd, int cinG, int coutG, int ksize, int stride,
                                                               int pad, int dil, long long pixels)
{
    constexpr int OCB = 8;
    const long long p = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= pixels) return;
    const int oc0 = blockIdx.y * OCB;
    const int g = oc0 / coutG;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const int b  = static_cast<int>(t / OH);
    const int K = ksize * ksize * cinG;
    const T *wp = w + static_cast<size_t>(oc0) * K;
    float acc[OCB];
#pragma unroll
    for (int j = 0; j < OCB; ++j) acc[j] = 0.f;
    for (int ki = 0; ki < ksize; ++ki)
    {
        const int iy = oy * stride - pad + ki * dil;
        for (int kj = 0; kj < ksize; ++kj)
        {
            const int ix = ox * stride - pad + kj * dil;
            const bool in = iy >= 0 && iy < H && ix >= 0 && ix < W;
            const T *xp = x + ((static_cast<size_t>(b) * H + (in ? iy : 0)) * W + (in ? ix : 0)) * inLd + g * cinG;
            const T *wt = wp + (ki * ksize + kj) * cinG;
            for (int c = 0; c < cinG; ++c)
            {
                const float xv = in ? toF(xp[c]) : 0.f;
#pragma unroll
                for (int j = 0; j < OCB; ++j) acc[j] += xv * toF(wt[static_cast<size_t>(j) * K + c]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < OCB; ++j)
    {
        const float r = e.hasRes ? toF(res[static_cast<size_t>(p) * resLd + oc0 + j]) : 0.f;
        y[static_cast<size_t>(p) * outLd + oc0 + j] = fromF<TOut>(epilogue(e, acc[j], oc0 + j, r));
    }
}

// Wider variant for small K = ksize^2 * (in_c/groups): the OCB x K weight block of the workgroup sits in LDS as float32,
// [k][OCB], so that the inner loop is one input load, OCB/4 broadcast 16-byte LDS reads and OCB multiply-adds.
template <typename T, typename TOut, int OCB>
__global__ __launch_bounds__(256) void convDirectLdsKernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ res,
                                                           TOut *__restrict__ y, EpiArgs e, int H, int W, int inLd, int OH, int OW,
                                                           int outLd, int resLd, int cinG, int coutG, int ksize, int stride,
                                                           int pad, int dil, long long pixels)
{
    extern __shared__ __attribute__((aligned(16))) float wl[];
    const int oc0 = blockIdx.y * OCB;
    const int g = oc0 / coutG;
    const int K = ksize * ksize * cinG;
    for (int i = threadIdx.x; i < K * OCB; i += 256)
    {
        const int k = i / OCB, j = i - k * OCB;
        wl[i] = toF(w[static_cast<size_t>(oc0 + j) * K + k]);
    }
    __syncthreads();
    const long long p = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= pixels) return;
    const int ox = static_cast<int>(p % OW);
    const long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const int b  = static_cast<int>(t / OH);
    float acc[OCB];
#pragma unroll
    for (int j = 0; j < OCB; ++j) acc[j] = 0.f;
    for (int ki = 0; ki < ksize; ++ki)
    {
        const int iy = oy * stride - pad + ki * dil;
        for (int kj = 0; kj < ksize; ++kj)
        {
            const int ix = ox * stride - pad + kj * dil;
            const bool in = iy >= 0 && iy < H && ix >= 0 && ix < W;
            const T *xp = x + ((static_cast<size_t>(b) * H + (in ? iy : 0)) * W + (in ? ix : 0)) * inLd + g * cinG;
            const f32x4 *wr = reinterpret_cast<const f32x4 *>(wl + static_cast<size_t>(ki * ksize + kj) * cinG * OCB);
            for (int c = 0; c < cinG; ++c)
            {
                const float xv = in ? toF(xp[c]) : 0.f;
#pragma unroll
                for (int j4 = 0; j4 < OCB / 4; ++j4)
                {
                    const f32x4 w4 = wr[c * (OCB / 4) + j4];
                    acc[4 * j4 + 0] += xv * w4[0];
                    acc[4 * j4 + 1] += xv * w4[1];
                    acc[4 * j4 + 2] += xv * w4[2];
                    acc[4 * j4 + 3] += xv * w4[3];
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < OCB; ++j)
    {
        const float r = e.hasRes ? toF(res[static_cast<size_t>(p) * resLd + oc0 + j]) : 0.f;
        y[static_cast<size_t>(p) * outLd + oc0 + j] = fromF<TOut>(epilogue(e, acc[j], oc0 + j, r));
    }
}

// ---- DEPTHWISE ------------------------------------------------------------------------------------
// weights [tap][C]; thread = (pixel, VEC channels).  VEC = 1 is the unaligned fallback.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void convDepthwiseKernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ res,
                                                           T *__restrict__ y, EpiArgs e, int H, int W, int inLd, int OH, int OW, int outLd,
                                                           int resLd, int C, int ksize, int stride, int pad, int dil, long long total)
{
    typedef T V __attribute__((ext_vector_type(VEC)));
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int cv = C / VEC;
    const int c0 = static_cast<int>(idx % cv) * VEC;
    long long p = idx / cv;
    const int ox = static_cast<int>(p % OW);
    long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const int b  = static_cast<int>(t / OH);
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
    for (int ki = 0; ki < ksize; ++ki)
    {
        const int iy = oy * stride - pad + ki * dil;
        if (iy < 0 || iy >= H) continue;
        for (int kj = 0; kj < ksize; ++kj)
        {
            const int ix = ox * stride - pad + kj * dil;
            if (ix < 0 || ix >= W) continue;
            const V xv = *reinterpret_cast<const V *>(x + ((static_cast<size_t>(b) * H + iy) * W + ix) * inLd + c0);
            const V wv = *reinterpret_cast<const V *>(w + static_cast<size_t>(ki * ksize + kj) * C + c0);
#pragma unroll
            for (int i = 0; i < VEC; ++i) acc[i] += toF(xv[i]) * toF(wv[i]);
        }
    }
    V rv;
#pragma unroll
    for (int i = 0; i < VEC; ++i) rv[i] = fromF<T>(0.f);
    if (e.hasRes) rv = *reinterpret_cast<const V *>(res + static_cast<size_t>(p) * resLd + c0);
    V o;
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = fromF<T>(epilogue(e, acc[i], c0 + i, toF(rv[i])));
    *reinterpret_cast<V *>(y + static_cast<size_t>(p) * outLd + c0) = o;
}

// ---- STEM -----------------------------------------------------------------------------------------
// x: NCHW float32 [B][Cin][H][W], Cin <= 4.  weights [tap*Cin + ci][outC] float32, staged in LDS.
// thread = one output pixel x OCT consecutive output channels (blockIdx.y selects the channel chunk);
// consecutive lanes take consecutive ox, so input reads are coalesced along W and every lane stores
// OCT contiguous channels.
template <typename TOut, int OCT>
__global__ __launch_bounds__(256) void convStemKernel(const float *__restrict__ x, const float *__restrict__ w, TOut *__restrict__ y,
                                                      EpiArgs e, int Cin, int H, int W, int OH, int OW, int outLd, int outC, int ksize,
                                                      int stride, int pad, long long P)
{
    extern __shared__ float wl[];                         // [taps*Cin][OCT]
    const int oc0 = blockIdx.y * OCT;
    const int kTot = ksize * ksize * Cin;
    for (int i = threadIdx.x; i < kTot * OCT; i += blockDim.x)
        wl[i] = w[static_cast<size_t>(i / OCT) * outC + oc0 + (i % OCT)];
    __syncthreads();
    long long p = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (p >= P) return;
    const int ox = static_cast<int>(p % OW);
    long long t = p / OW;
    const int oy = static_cast<int>(t % OH);
    const int b  = static_cast<int>(t / OH);
    float acc[OCT];
#pragma unroll
    for (int i = 0; i < OCT; ++i) acc[i] = 0.f;
    for (int ki = 0; ki < ksize; ++ki)
    {
        const int iy = oy * stride - pad + ki;
        if (iy < 0 || iy >= H) continue;
        for (int kj = 0; kj < ksize; ++kj)
        {
            const int ix = ox * stride - pad + kj;
            if (ix < 0 || ix >= W) continue;
            for (int ci = 0; ci < Cin; ++ci)
            {
                const float xv = x[((static_cast<size_t>(b) * Cin + ci) * H + iy) * W + ix];
                const float *wr = wl + ((ki * ksize + kj) * Cin + ci) * OCT;
#pragma unroll
                for (int i = 0; i < OCT; ++i) acc[i] += xv * wr[i];
            }
        }
    }
    TOut *yp = y + static_cast<size_t>(p) * outLd + oc0;
    typedef TOut OutV __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int i = 0; i < OCT; i += 4)
    {
        OutV o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = fromF<TOut>(epilogue(e, acc[i + j], oc0 + i + j, 0.f));
        *reinterpret_cast<OutV *>(yp + i) = o;
    }
}

// ---- host side ------------------------------------------------------------------------------------
static int validate(const msnh_conv_desc *d)
{
    MSNH_REQUIRE(d != nullptr, "conv desc is NULL");
    MSNH_REQUIRE(dtypeOk(d->dtype) && dtypeOk(d->out_dtype), "conv: bad dtype");
    MSNH_REQUIRE(d->batch > 0 && d->in_h > 0 && d->in_w > 0 && d->in_c > 0 && d->out_c > 0, "conv: non-positive size");
    MSNH_REQUIRE(d->ksize > 0 && d->stride > 0 && d->pad >= 0 && d->dilation > 0 && d->groups > 0, "conv: bad geometry");
    MSNH_REQUIRE(d->in_c % d->groups == 0 && d->out_c % d->groups == 0, "conv: channels not divisible by groups");
    const int ext = d->dilation * (d->ksize - 1) + 1;
    MSNH_REQUIRE(d->in_h + 2 * d->pad >= ext && d->in_w + 2 * d->pad >= ext, "conv: kernel larger than padded input");
    const int oh = (d->in_h + 2 * d->pad - ext) / d->stride + 1;
    const int ow = (d->in_w + 2 * d->pad - ext) / d->stride + 1;
    MSNH_REQUIRE(oh == d->out_h && ow == d->out_w, "conv: out size %dx%d does not match geometry (%dx%d)", d->out_h, d->out_w, oh, ow);
    MSNH_REQUIRE(d->out_ld >= d->out_c, "conv: out_ld < out_c");
    MSNH_REQUIRE(d->out_upsample >= 0 && d->out_upsample <= 2, "conv: out_upsample is 0, 1 or 2");
    MSNH_REQUIRE(d->xcd_blocks == 0 || d->xcd_blocks == 1 || d->xcd_blocks == 2 || d->xcd_blocks == 4 || d->xcd_blocks == 8, "conv: xcd_blocks is 0, 1, 2, 4 or 8");
    MSNH_REQUIRE(d->out_upsample != 2 || ((d->algo == MSNH_CONV_IGEMM || d->algo == MSNH_CONV_AUTO) && !d->has_residual && d->out_c % 8 == 0 && d->out_ld % 8 == 0 &&
                                         d->groups == 1 && static_cast<long long>(d->batch) * d->out_h * d->out_w * 4 * d->out_ld * 4 < 0x7fffffffLL),
                 "conv: the upsampling epilogue belongs to the IGEMM algorithm, without residual, channel counts multiples of 8");
    MSNH_REQUIRE(!d->has_residual || d->res_ld >= d->out_c, "conv: res_ld < out_c");
    MSNH_REQUIRE(actOk(d->act) && (!d->has_residual || actOk(d->act2)), "conv: unsupported activation");
    MSNH_REQUIRE(static_cast<long long>(d->batch) * d->out_h * d->out_w < (1LL << 31), "conv: too many output pixels");
    return 0;
}

static bool igemmOk(const msnh_conv_desc *d)
{
    const int vec = d->dtype == MSNH_F16 ? 8 : 4;
    if (d->dtype == MSNH_F32 && d->out_dtype != MSNH_F32) return false;
    return (d->in_c / d->groups) % vec == 0 && d->in_ld % vec == 0;
}

static bool depthwiseOk(const msnh_conv_desc *d)
{
    return d->groups == d->in_c && d->out_c == d->in_c && d->groups > 1 && d->dtype == d->out_dtype;
}

static bool stemOk(const msnh_conv_desc *d)
{
    return d->in_c <= 4 && d->groups == 1 && d->dilation == 1 && d->out_c % 32 == 0 && d->out_ld % 4 == 0 &&
           !d->has_residual && static_cast<size_t>(d->ksize) * d->ksize * d->in_c * 32 * 4 <= 60 * 1024;
}

static bool winogradOk(const msnh_conv_desc *d)
{
    return d->ksize == 3 && d->stride == 1 && d->dilation == 1 && d->groups == 1 && d->pad == 1 && d->dtype == MSNH_F16 &&
           d->in_c % 8 == 0 && d->in_ld % 8 == 0 && d->out_c % 8 == 0 && d->out_ld % 8 == 0;
}

} // namespace msnh

using namespace msnh;

extern "C" {

int msnh_hip_conv2d_tile_count(void) { return igemmTileCount(); }

// Bumped whenever msnh_hip_conv2d_pack_weights changes what it writes for some (descriptor, algorithm).
int msnh_hip_conv2d_pack_layout_version(void) { return 1; }

int msnh_hip_conv2d_tile_supported(const msnh_conv_desc *d, int tile)
{
    if (!d || validate(d) || tile < 0 || tile > igemmTileCount()) return 0;
    msnh_conv_desc t = *d;
    if (d->algo == MSNH_CONV_POINTWISE) return tile == 0 && pointwiseOk(d) ? 1 : 0;
    if (d->algo == MSNH_CONV_WINOGRAD_FUSED) return tile == 0 && winogradFusedOk(d) ? 1 : 0;
    if (d->algo == MSNH_CONV_WINOGRAD)
    {
        // the tile applies to the 16 transformed-domain GEMMs
        if (!winogradOk(d) || static_cast<long long>(d->batch) * ((d->out_h + 1) / 2) * ((d->out_w + 1) / 2) * 16 * d->in_c * 2 >= (1LL << 31)) return 0;
        winogradGemmDesc(d, &t);
    }
    else if (!igemmOk(d)) return 0;
    if (tile == 0 && d->algo != MSNH_CONV_IGEMM_SPLITK) return 1;
    t.tile = tile;
    return convIgemm(&t, d, d, nullptr, nullptr, nullptr, &t, nullptr, true) == 0 ? 1 : 0;      // pointers unused in a dry run
}

int msnh_hip_conv2d_tail_tile_first(void) { return igemmTailTileFirst(); }

static bool tailDescOk(const msnh_conv_desc *d, const msnh_conv_tail_desc *t)
{
    return d && t && !validate(d) && igemmOk(d) && d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16 && d->groups == 1 &&
           (d->algo == MSNH_CONV_IGEMM || d->algo == MSNH_CONV_AUTO) && d->out_c % 8 == 0 && d->out_ld % 8 == 0 && (!d->has_residual || d->res_ld % 8 == 0) &&
           t->out_c > 0 && t->out_c % 8 == 0 && t->out_ld >= t->out_c && t->out_ld % 8 == 0 && actOk(t->act);
}

int msnh_hip_conv2d_tail_supported(const msnh_conv_desc *d, const msnh_conv_tail_desc *t, int tile)
{
    if (!tailDescOk(d, t) || tile < 0 || tile > igemmTileCount() || (tile != 0 && tile < igemmTailTileFirst())) return 0;
    msnh_conv_desc c = *d;
    c.algo = MSNH_CONV_IGEMM;
    c.tile = tile;
    return convIgemmTail(&c, t, d, d, nullptr, nullptr, d, &c, d, nullptr, nullptr, &c, nullptr, true) == 0 ? 1 : 0;      // pointers unused in a dry run
}

int msnh_hip_conv2d_tail(const msnh_conv_desc *d, const msnh_conv_tail_desc *t, const void *x, const void *w, const float *scale, const float *shift,
                         const void *residual, void *y, const void *w2, const float *scale2, const float *shift2, void *z, msnh_stream_t s)
{
    MSNH_REQUIRE(tailDescOk(d, t), "conv2d_tail: a float16 ungrouped IGEMM convolution followed by a 1x1 convolution, channel counts and pixel strides multiples of 8");
    MSNH_REQUIRE(x && w && y && w2 && z, "conv2d_tail: NULL tensor pointer");
    MSNH_REQUIRE(!d->has_residual || residual, "conv2d_tail: has_residual without a residual tensor");
    MSNH_REQUIRE(d->in_ld >= d->in_c, "conv2d_tail: in_ld < in_c");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                 (!d->has_residual || reinterpret_cast<uintptr_t>(residual) % 16 == 0), "conv2d_tail: 16-byte aligned tensors");
    msnh_conv_desc c = *d;
    c.algo = MSNH_CONV_IGEMM;
    return convIgemmTail(&c, t, x, w, scale, shift, residual, y, w2, scale2, shift2, z, resolveStream(s), false);
}

int msnh_hip_conv2d_select_algo(const msnh_conv_desc *d)
{
    if (!d) return MSNH_CONV_DIRECT;
    if (d->algo != MSNH_CONV_AUTO) return d->algo;
    if (d->out_upsample == 2) return MSNH_CONV_IGEMM;
    if (stemOk(d)) return MSNH_CONV_STEM;
    if (depthwiseOk(d)) return MSNH_CONV_DEPTHWISE;
    if (igemmOk(d)) return MSNH_CONV_IGEMM;
    return MSNH_CONV_DIRECT;
}

size_t msnh_hip_conv2d_packed_weight_elems(const msnh_conv_desc *d, int algo)
{
    if (!d) return 0;
    const size_t kk = static_cast<size_t>(d->ksize) * d->ksize;
    const size_t cinG = static_cast<size_t>(d->in_c / d->groups);
    if (algo == MSNH_CONV_WINOGRAD || algo == MSNH_CONV_WINOGRAD_FUSED) return static_cast<size_t>(16) * d->out_c * d->in_c;
    // float32 payload for the scalar kernel, followed (float16 plans) by the MFMA operand fragments
    if (algo == MSNH_CONV_STEM) return kk * d->in_c * d->out_c * (d->dtype == MSNH_F16 ? 2 : 1) + (stemMfmaOk(d) ? stemMfmaElems(d) : 0);
    return static_cast<size_t>(d->out_c) * kk * cinG;
}

int msnh_hip_conv2d_pack_weights(const msnh_conv_desc *d, int algo, const float *oihw, void *packed)
{
    if (validate(d)) return 2;
    MSNH_REQUIRE(oihw && packed, "pack_weights: NULL pointer");
    const int kk = d->ksize * d->ksize;
    const int cinG = d->in_c / d->groups;
    auto put = [&](size_t i, float v) {
        if (d->dtype == MSNH_F16) static_cast<_Float16 *>(packed)[i] = static_cast<_Float16>(v);
        else static_cast<float *>(packed)[i] = v;
    };
    switch (algo)
    {
    case MSNH_CONV_DIRECT:
    case MSNH_CONV_IGEMM:
    case MSNH_CONV_IGEMM_SPLITK:
    case MSNH_CONV_POINTWISE:
        for (int oc = 0; oc < d->out_c; ++oc)
            for (int ci = 0; ci < cinG; ++ci)
                for (int t = 0; t < kk; ++t)
                    put((static_cast<size_t>(oc) * kk + t) * cinG + ci, oihw[(static_cast<size_t>(oc) * cinG + ci) * kk + t]);
        return 0;
    case MSNH_CONV_DEPTHWISE:
        MSNH_REQUIRE(depthwiseOk(d), "pack_weights: not a depthwise convolution");
        for (int c = 0; c < d->out_c; ++c)
            for (int t = 0; t < kk; ++t) put(static_cast<size_t>(t) * d->out_c + c, oihw[static_cast<size_t>(c) * kk + t]);
        return 0;
    case MSNH_CONV_STEM:
    {
        MSNH_REQUIRE(stemOk(d), "pack_weights: shape not supported by the stem kernel");
        float *o = static_cast<float *>(packed);
        for (int oc = 0; oc < d->out_c; ++oc)
            for (int ci = 0; ci < d->in_c; ++ci)
                for (int t = 0; t < kk; ++t)
                    o[(static_cast<size_t>(t) * d->in_c + ci) * d->out_c + oc] = oihw[(static_cast<size_t>(oc) * d->in_c + ci) * kk + t];
        if (stemMfmaOk(d)) stemMfmaPack(d, oihw, static_cast<_Float16 *>(packed) + static_cast<size_t>(kk) * d->in_c * d->out_c * 2);
        return 0;
    }
    case MSNH_CONV_WINOGRAD:
    case MSNH_CONV_WINOGRAD_FUSED:
        MSNH_REQUIRE(winogradOk(d), "pack_weights: shape not supported by the Winograd kernel");
        winogradPackWeights(d, oihw, packed);
        return 0;
    default:
        setError("pack_weights: unknown algo %d", algo);
        return 2;
    }
}

size_t msnh_hip_conv2d_workspace_bytes(const msnh_conv_desc *d, int algo)
{
    if (!d) return 0;
    if (algo == MSNH_CONV_IGEMM_SPLITK) return igemmSplitKWorkspaceBytes(d);
    return algo == MSNH_CONV_WINOGRAD ? winogradWorkspaceBytes(d) : 0;
}

int msnh_hip_conv2d(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
                    const void *residual, void *y, void *workspace, size_t workspace_bytes, msnh_stream_t s)
{
    if (validate(d)) return 2;
    MSNH_REQUIRE(x && w && y, "conv2d: NULL tensor pointer");
    MSNH_REQUIRE(!d->has_residual || residual, "conv2d: has_residual without a residual tensor");
    hipStream_t st = resolveStream(s);
    const int algo = msnh_hip_conv2d_select_algo(d);
    EpiArgs e;
    e.scale = scale; e.shift = shift; e.act = d->act; e.act2 = d->act2; e.hasRes = d->has_residual ? 1 : 0;
    e.actParam = d->act_param; e.act2Param = d->act2_param; e.resMul = d->res_mul; e.outMul = d->out_mul;
    const int cinG = d->in_c / d->groups, coutG = d->out_c / d->groups;
    const long long P = static_cast<long long>(d->batch) * d->out_h * d->out_w;
    if (algo != MSNH_CONV_STEM) MSNH_REQUIRE(d->in_ld >= d->in_c, "conv2d: in_ld < in_c");

    switch (algo)
    {
    case MSNH_CONV_IGEMM:
        MSNH_REQUIRE(igemmOk(d), "conv2d: IGEMM needs (in_c/groups) and in_ld to be multiples of %d", d->dtype == MSNH_F16 ? 8 : 4);
        MSNH_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0, "conv2d: IGEMM needs 16-byte aligned x and w");
        MSNH_REQUIRE(d->out_upsample != 2 || reinterpret_cast<uintptr_t>(y) % 16 == 0, "conv2d: the upsampling epilogue needs a 16-byte aligned y");
        return convIgemm(d, x, w, scale, shift, residual, y, st, false);
    case MSNH_CONV_IGEMM_SPLITK:
        MSNH_REQUIRE(igemmOk(d), "conv2d: IGEMM needs (in_c/groups) and in_ld to be multiples of %d", d->dtype == MSNH_F16 ? 8 : 4);
        MSNH_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0, "conv2d: IGEMM needs 16-byte aligned x and w");
        return convIgemmWs(d, x, w, scale, shift, residual, y, st, false, workspace, workspace_bytes);
    case MSNH_CONV_POINTWISE:
        return convPointwise(d, x, w, scale, shift, residual, y, st);
    case MSNH_CONV_WINOGRAD_FUSED:
        return convWinogradFused(d, x, w, scale, shift, residual, y, st);
    case MSNH_CONV_WINOGRAD:
        MSNH_REQUIRE(winogradOk(d), "conv2d: shape not supported by the Winograd kernel");
        return convWinograd(d, x, w, scale, shift, residual, y, workspace, workspace_bytes, st);
    case MSNH_CONV_DEPTHWISE:
    {
        MSNH_REQUIRE(depthwiseOk(d), "conv2d: not a depthwise convolution");
        if (depthwise3x3Ok(d, x, w, y)) return convDepthwise3x3(d, x, w, scale, shift, y, st);
        const int C = d->in_c;
        const int vec = d->dtype == MSNH_F16 ? 8 : 4;
        const size_t el = dtypeSize(d->dtype);
        const bool aligned = C % vec == 0 && d->in_ld % vec == 0 && d->out_ld % vec == 0 && (!d->has_residual || d->res_ld % vec == 0) &&
                             reinterpret_cast<uintptr_t>(x) % (vec * el) == 0 && reinterpret_cast<uintptr_t>(y) % (vec * el) == 0 &&
                             reinterpret_cast<uintptr_t>(w) % (vec * el) == 0 &&
                             (!d->has_residual || reinterpret_cast<uintptr_t>(residual) % (vec * el) == 0);
        const long long total = P * (aligned ? C / vec : C);
        dim3 grid(gridFor(total, 256));
#define MSNH_DW(T, V)                                                                                                   \
    hipLaunchKernelGGL((convDepthwiseKernel<T, V>), grid, dim3(256), 0, st, static_cast<const T *>(x), static_cast<const T *>(w), \
                       static_cast<const T *>(residual), static_cast<T *>(y), e, d->in_h, d->in_w, d->in_ld, d->out_h, d->out_w,    \
                       d->out_ld, d->res_ld, C, d->ksize, d->stride, d->pad, d->dilation, total)
        if (d->dtype == MSNH_F16) { if (aligned) MSNH_DW(f16, 8); else MSNH_DW(f16, 1); }
        else                      { if (aligned) MSNH_DW(float, 4); else MSNH_DW(float, 1); }
#undef MSNH_DW
        MSNH_LAUNCH_CHECK();
        return 0;
    }
    case MSNH_CONV_STEM:
    {
        MSNH_REQUIRE(stemOk(d), "conv2d: shape not supported by the stem kernel");
        const size_t outEl = dtypeSize(d->out_dtype);
        MSNH_REQUIRE(reinterpret_cast<uintptr_t>(y) % (4 * outEl) == 0, "conv2d: stem needs aligned output");
        if (stemMfmaOk(d))
            return convStemMfma(d, static_cast<const float *>(x), static_cast<const _Float16 *>(w) + static_cast<size_t>(d->ksize) * d->ksize * d->in_c * d->out_c * 2,
                                scale, shift, y, st);
        // a lane owns one pixel and OCT output channels: 32 when there are pixels enough to fill the chip, 8 for small images
        // (a single 224 x 224 image gives 98 workgroups at 32 channels per lane, 392 at 8)
#define MSNH_STEM(TO, OCT)                                                                                              \
    do {                                                                                                                \
        dim3 grid(gridFor(P, 256), d->out_c / OCT);                                                                     \
        const size_t smem = static_cast<size_t>(d->ksize) * d->ksize * d->in_c * OCT * sizeof(float);                  \
        hipLaunchKernelGGL((convStemKernel<TO, OCT>), grid, dim3(256), smem, st, static_cast<const float *>(x), static_cast<const float *>(w), \
                           static_cast<TO *>(y), e, d->in_c, d->in_h, d->in_w, d->out_h, d->out_w, d->out_ld, d->out_c, d->ksize, d->stride, d->pad, P); \
    } while (0)
        const bool few = P * (d->out_c / 32) < 256LL * 512;
        if (d->out_dtype == MSNH_F16) { if (few) MSNH_STEM(f16, 8); else MSNH_STEM(f16, 32); }
        else                          { if (few) MSNH_STEM(float, 8); else MSNH_STEM(float, 32); }
#undef MSNH_STEM
        MSNH_LAUNCH_CHECK();
        return 0;
    }
    case MSNH_CONV_DIRECT:
    {
        const int Kdir = d->ksize * d->ksize * cinG;
        const int ocb = coutG % 32 == 0 ? 32 : (coutG % 16 == 0 ? 16 : 0);
        if (ocb && static_cast<size_t>(Kdir) * ocb * sizeof(float) <= 48 * 1024 && d->out_c / ocb <= 65535)
        {
            dim3 lgrid(gridFor(P, 256), d->out_c / ocb);
            const size_t lds = static_cast<size_t>(Kdir) * ocb * sizeof(float);
#define MSNH_DIRECTL(T, TO, B)                                                                                          \
    hipLaunchKernelGGL((convDirectLdsKernel<T, TO, B>), lgrid, dim3(256), lds, st, static_cast<const T *>(x), static_cast<const T *>(w),  \
                       static_cast<const T *>(residual), static_cast<TO *>(y), e, d->in_h, d->in_w, d->in_ld, d->out_h, d->out_w,  \
                       d->out_ld, d->res_ld, cinG, coutG, d->ksize, d->stride, d->pad, d->dilation, P)
#define MSNH_DIRECTL2(T, TO) do { if (ocb == 32) MSNH_DIRECTL(T, TO, 32); else MSNH_DIRECTL(T, TO, 16); } while (0)
            if (d->dtype == MSNH_F16) { if (d->out_dtype == MSNH_F16) MSNH_DIRECTL2(f16, f16); else MSNH_DIRECTL2(f16, float); }
            else
            {
                MSNH_REQUIRE(d->out_dtype == MSNH_F32, "conv2d: float32 input needs float32 output");
                MSNH_DIRECTL2(float, float);
            }
#undef MSNH_DIRECTL2
#undef MSNH_DIRECTL
            MSNH_LAUNCH_CHECK();
            return 0;
        }
        if (coutG % 8 == 0 && d->out_c / 8 <= 65535)
        {
            dim3 bgrid(gridFor(P, 256), d->out_c / 8);
#define MSNH_DIRECTB(T, TO)                                                                                             \
    hipLaunchKernelGGL((convDirectBlockedKernel<T, TO>), bgrid, dim3(256), 0, st, static_cast<const T *>(x), static_cast<const T *>(w),  \
                       static_cast<const T *>(residual), static_cast<TO *>(y), e, d->in_h, d->in_w, d->in_ld, d->out_h, d->out_w,  \
                       d->out_ld, d->res_ld, cinG, coutG, d->ksize, d->stride, d->pad, d->dilation, P)
            if (d->dtype == MSNH_F16) { if (d->out_dtype == MSNH_F16) MSNH_DIRECTB(f16, f16); else MSNH_DIRECTB(f16, float); }
            else
            {
                MSNH_REQUIRE(d->out_dtype == MSNH_F32, "conv2d: float32 input needs float32 output");
                MSNH_DIRECTB(float, float);
            }
#undef MSNH_DIRECTB
            MSNH_LAUNCH_CHECK();
            return 0;
        }
        const long long total = P * d->out_c;
        dim3 grid(gridFor(total, 256));
#define MSNH_DIRECT(T, TO)                                                                                              \
    hipLaunchKernelGGL((convDirectKernel<T, TO>), grid, dim3(256), 0, st, static_cast<const T *>(x), static_cast<const T *>(w),  \
                       static_cast<const T *>(residual), static_cast<TO *>(y), e, d->in_h, d->in_w, d->in_ld, d->out_h, d->out_w,  \
                       d->out_ld, d->res_ld, cinG, coutG, d->out_c, d->ksize, d->stride, d->pad, d->dilation, total)
        if (d->dtype == MSNH_F16) { if (d->out_dtype == MSNH_F16) MSNH_DIRECT(f16, f16); else MSNH_DIRECT(f16, float); }
        else
        {
            MSNH_REQUIRE(d->out_dtype == MSNH_F32, "conv2d: float32 input needs float32 output");
            MSNH_DIRECT(float, float);
        }
#undef MSNH_DIRECT
        MSNH_LAUNCH_CHECK();
        return 0;
    }
    default:
        setError("conv2d: unknown algo %d", algo);
        return 2;
    }
}

}
