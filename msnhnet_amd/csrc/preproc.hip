// Letterbox of one 8-bit RGB image (HWC) straight into the network's NCHW float32 input: pad to a square with 127,
// bilinear resize, optional R<->B swap, scale to [0,1] or [-1,1] -- the reference's CVUtil::getPaddingZeroF32C3
// (src/utils/MsnhCVUtil.cpp:203-261) as one pass.  The padded square is never materialised: a sample outside the
// image reads as 127.  The float expressions are the reference's (MatOp::resize, src/cv/MsnhCVMatOp.cpp:404-437),
// evaluated without fused multiply-add, so the truncated 8-bit result is reproduced exactly; that includes its
// behaviour when enlarging, where the last rows / columns get weights that sum to zero.
// msnh_hip_image_u8_to_input is the same pass for the reference's plain-resize pre-processing variants (getImgDataF32C3,
// getGoogLenetF32C3, getTransformedF32C3, getCaffeModeF32C3, src/utils/MsnhCVUtil.cpp:91-375): no padding, separate
// horizontal and vertical scale factors, and the per-channel normalisation each of them writes.
// Bandwidth: one byte image read per source sample (L2 resident), 12 bytes written per output pixel.
#include "common.hpp"

namespace msnh {

namespace {

struct LetterboxArgs
{
    const unsigned char *img;
    float *out;
    int w, h, netW, netH, S, top, left, halfInit, shuffle;
    // plain resize (S == 0): source extent w x h, normalisation `kind` with mean / std
    int kind;
    float mean[3], stdv[3];
};

__device__ __forceinline__ float sampleU8(const LetterboxArgs &a, int y, int x, int k)
{
    const int iy = y - a.top, ix = x - a.left;
    if (iy < 0 || iy >= a.h || ix < 0 || ix >= a.w) return 127.f;
    return static_cast<float>(a.img[(static_cast<size_t>(iy) * a.w + ix) * 3 + k]);
}

__global__ __launch_bounds__(256) void letterboxKernel(LetterboxArgs a)
{
#pragma clang fp contract(off)
    const int j = blockIdx.x * 64 + (threadIdx.x & 63);       // output column
    const int i = blockIdx.y * 4 + (threadIdx.x >> 6);        // output row
    if (i >= a.netH || j >= a.netW) return;
    float v[3];
    if (a.netW == a.S && a.netH == a.S)
    {
#pragma unroll
        for (int k = 0; k < 3; ++k) v[k] = sampleU8(a, i, j, k);
    }
    else
    {
        const float fx = 1.f * a.S / a.netW;
        const float fy = 1.f * a.S / a.netH;
        float sh = (i + 0.5f) * fy - 0.5f;
        sh = sh < 0 ? 0 : sh;
        const int h0 = static_cast<int>(sh);
        const int h1 = h0 + 1 < a.S - 1 ? h0 + 1 : a.S - 1;
        float sw = (j + 0.5f) * fx - 0.5f;
        sw = sw < 0 ? 0 : sw;
        const int w0 = static_cast<int>(sw);
        const int w1 = w0 + 1 < a.S - 1 ? w0 + 1 : a.S - 1;
#pragma unroll
        for (int k = 0; k < 3; ++k)
        {
            const float r = (h1 - sh) * ((w1 - sw) * sampleU8(a, h0, w0, k) + (sw - w0) * sampleU8(a, h0, w1, k)) +
                            (sh - h0) * ((w1 - sw) * sampleU8(a, h1, w0, k) + (sw - w0) * sampleU8(a, h1, w1, k));
            const unsigned short q = static_cast<unsigned short>(static_cast<int>(r));
            v[k] = static_cast<float>(q > 255 ? 255 : q);
        }
    }
    const size_t plane = static_cast<size_t>(a.netW) * a.netH;
#pragma unroll
    for (int k = 0; k < 3; ++k)
    {
        const float u = v[a.shuffle ? 2 - k : k];
        a.out[k * plane + static_cast<size_t>(i) * a.netW + j] = a.halfInit ? (u - 127.5f) / 127.5f : u / 255.0f;
    }
}

// Plain bilinear resize + normalisation.  Same float expressions as letterboxKernel with the source extent (w, h) in place
// of the padded square.
__global__ __launch_bounds__(256) void resizeNormKernel(LetterboxArgs a)
{
#pragma clang fp contract(off)
    const int j = blockIdx.x * 64 + (threadIdx.x & 63);
    const int i = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (i >= a.netH || j >= a.netW) return;
    float v[3];
    if (a.netW == a.w && a.netH == a.h)
    {
#pragma unroll
        for (int k = 0; k < 3; ++k) v[k] = static_cast<float>(a.img[(static_cast<size_t>(i) * a.w + j) * 3 + k]);
    }
    else
    {
        const float fx = 1.f * a.w / a.netW;
        const float fy = 1.f * a.h / a.netH;
        float sh = (i + 0.5f) * fy - 0.5f;
        sh = sh < 0 ? 0 : sh;
        const int h0 = static_cast<int>(sh);
        const int h1 = h0 + 1 < a.h - 1 ? h0 + 1 : a.h - 1;
        float sw = (j + 0.5f) * fx - 0.5f;
        sw = sw < 0 ? 0 : sw;
        const int w0 = static_cast<int>(sw);
        const int w1 = w0 + 1 < a.w - 1 ? w0 + 1 : a.w - 1;
        const unsigned char *r0 = a.img + static_cast<size_t>(h0) * a.w * 3, *r1 = a.img + static_cast<size_t>(h1) * a.w * 3;
#pragma unroll
        for (int k = 0; k < 3; ++k)
        {
            const float r = (h1 - sh) * ((w1 - sw) * r0[w0 * 3 + k] + (sw - w0) * r0[w1 * 3 + k]) +
                            (sh - h0) * ((w1 - sw) * r1[w0 * 3 + k] + (sw - w0) * r1[w1 * 3 + k]);
            const unsigned short q = static_cast<unsigned short>(static_cast<int>(r));
            v[k] = static_cast<float>(q > 255 ? 255 : q);
        }
    }
    const size_t plane = static_cast<size_t>(a.netW) * a.netH;
    const float gStd[3] = {0.229f, 0.224f, 0.225f}, gMean[3] = {0.485f, 0.456f, 0.406f};
    const float caffe[3] = {123.68f, 116.779f, 103.939f};
#pragma unroll
    for (int k = 0; k < 3; ++k)
    {
        const float u = v[a.shuffle ? 2 - k : k];
        float o;
        switch (a.kind)
        {
        case MSNH_PRE_F32C3_HALF:  o = (u - 127.5f) / 127.5f; break;
        case MSNH_PRE_GOOGLENET:   o = u / 255.0f * (gStd[k] / 0.5f) + (gMean[k] - 0.5f) / 0.5f; break;
        case MSNH_PRE_TRANSFORMED: o = ((u / 255.0f) - a.mean[k]) / a.stdv[k]; break;
        case MSNH_PRE_CAFFE:       o = u - caffe[k]; break;
        default:                   o = u / 255.0f; break;
        }
        a.out[k * plane + static_cast<size_t>(i) * a.netW + j] = o;
    }
}

} // namespace

} // namespace msnh

using namespace msnh;

extern "C" int msnh_hip_letterbox_u8(const unsigned char *rgb_hwc, int width, int height, int net_w, int net_h, int half_init,
                                     int shuffle_rgb, float *out_chw, msnh_stream_t s)
{
    MSNH_REQUIRE(rgb_hwc && out_chw, "letterbox: NULL pointer");
    MSNH_REQUIRE(width > 0 && height > 0 && net_w > 0 && net_h > 0, "letterbox: bad geometry");
    LetterboxArgs a;
    a.img = rgb_hwc; a.out = out_chw; a.w = width; a.h = height; a.netW = net_w; a.netH = net_h;
    const int diff = width > height ? width - height : height - width;
    a.S = width > height ? width : height;
    a.top = width > height ? diff / 2 : 0;
    a.left = width < height ? diff / 2 : 0;
    a.halfInit = half_init; a.shuffle = shuffle_rgb; a.kind = 0;
    for (int k = 0; k < 3; ++k) { a.mean[k] = 0.f; a.stdv[k] = 1.f; }
    const dim3 grid((net_w + 63) / 64, (net_h + 3) / 4);
    hipLaunchKernelGGL(letterboxKernel, grid, dim3(256), 0, resolveStream(s), a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

extern "C" int msnh_hip_image_u8_to_input(const unsigned char *rgb_hwc, int width, int height, int net_w, int net_h, int kind,
                                          const float *mean3, const float *std3, int shuffle_rgb, float *out_chw, msnh_stream_t s)
{
    MSNH_REQUIRE(rgb_hwc && out_chw, "image_u8_to_input: NULL pointer");
    MSNH_REQUIRE(width > 0 && height > 0 && net_w > 0 && net_h > 0, "image_u8_to_input: bad geometry");
    MSNH_REQUIRE(kind >= MSNH_PRE_F32C3 && kind <= MSNH_PRE_PADDING_ZERO_HALF, "image_u8_to_input: unknown kind");
    if (kind == MSNH_PRE_PADDING_ZERO || kind == MSNH_PRE_PADDING_ZERO_HALF)
        return msnh_hip_letterbox_u8(rgb_hwc, width, height, net_w, net_h, kind == MSNH_PRE_PADDING_ZERO_HALF, shuffle_rgb, out_chw, s);
    MSNH_REQUIRE(kind != MSNH_PRE_TRANSFORMED || (mean3 && std3), "image_u8_to_input: mean or std can't be null");
    LetterboxArgs a;
    a.img = rgb_hwc; a.out = out_chw; a.w = width; a.h = height; a.netW = net_w; a.netH = net_h;
    a.S = 0; a.top = 0; a.left = 0; a.halfInit = 0; a.shuffle = shuffle_rgb; a.kind = kind;
    for (int k = 0; k < 3; ++k) { a.mean[k] = mean3 ? mean3[k] : 0.f; a.stdv[k] = std3 ? std3[k] : 1.f; }
    const dim3 grid((net_w + 63) / 64, (net_h + 3) / 4);
    hipLaunchKernelGGL(resizeNormKernel, grid, dim3(256), 0, resolveStream(s), a);
    MSNH_LAUNCH_CHECK();
    return 0;
}
