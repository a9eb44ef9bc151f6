// First-layer convolution on the matrix cores: 3x3 filter over <= 3 input channels, read straight from the NCHW
// float32 network input (layout conversion and cast to float16 fused), NHWC float16 out.
//
// GEMM view: 32 output channels x 32 consecutive output pixels of one row per wavefront, K = 9 * Cin <= 27
// padded to 32, i.e. two 32x32x16 MFMAs.  The kernel is bound by the write of the output (64 bytes per pixel
// and 32 channels) and by the 16 scalar gathers per lane that assemble the B operand; the weights (operand A,
// 2 KiB per 32 channels) stay in registers for the wavefront's whole life.
//
// The rows of the MFMA are a permutation of the channels: MFMA row 8q + 4h + e computes channel 16h + 4q + e.
// The 32x32 accumulator layout gives lane l, register r the row 8(r/4) + 4(l/32) + r%4, so with that permutation
// the 16 registers of a lane are 16 CONSECUTIVE channels of its pixel: two 16-byte stores, no transposition.
#include "common.hpp"

namespace msnh {

namespace {

struct StemArgs
{
    const float *x;
    const f16   *wA;        // [mBlocks][2][64 lanes][8]
    const float *scale;
    const float *shift;
    f16         *y;
    int B, H, W, OH, OW, outLd, outC, stride, pad;
    int groupsPerRow;       // ceil(OW / 32)
    int nGroups;            // B * OH * groupsPerRow
    int act;
    float actParam, outMul;
};

template <int CIN>
__global__ __launch_bounds__(256) void convStemMfmaKernel(StemArgs a)
{
    constexpr int K = 9 * CIN;
    const int lane = threadIdx.x & 63;
    const int n = lane & 31, h = lane >> 5;
    const int wavesTotal = gridDim.x * 4;
    const int wave0 = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int mBlocks = a.outC / 32;

    // this lane's 16 K indices: k = kb*16 + 8h + e  ->  (tap, ci), offset inside the image stack of one batch item
    int koff[16], kky[16], kkx[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
    {
        const int k = (i / 8) * 16 + 8 * h + (i % 8);
        const int tap = k / CIN, ci = k - tap * CIN;
        const int ky = tap / 3, kx = tap - 3 * ky;
        kky[i] = k < K ? ky : -100000;              // never inside the image: reads as zero
        kkx[i] = kx;
        koff[i] = (ci * a.H + ky) * a.W + kx;
    }

    float slope;
    const bool lin = (a.act == MSNH_ACT_LEAKY || a.act == MSNH_ACT_RELU || a.act == MSNH_ACT_NONE);
    slope = a.act == MSNH_ACT_LEAKY ? a.actParam : (a.act == MSNH_ACT_RELU ? 0.f : 1.f);

    for (int mb = 0; mb < mBlocks; ++mb)
    {
        const f16x8 wa0 = *reinterpret_cast<const f16x8 *>(a.wA + (static_cast<size_t>(mb * 2 + 0) * 64 + lane) * 8);
        const f16x8 wa1 = *reinterpret_cast<const f16x8 *>(a.wA + (static_cast<size_t>(mb * 2 + 1) * 64 + lane) * 8);
        float sc[16], sh[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
        {
            const int ch = mb * 32 + 16 * h + r;
            sc[r] = a.scale ? a.scale[ch] : 1.f;
            sh[r] = a.shift ? a.shift[ch] : 0.f;
        }
        for (int g = wave0; g < a.nGroups; g += wavesTotal)
        {
            const int gx = g % a.groupsPerRow;
            const int row = g / a.groupsPerRow;
            const int oy = row % a.OH;
            const int b = row / a.OH;
            const int ox = gx * 32 + n;
            const int iy0 = oy * a.stride - a.pad;
            const int ix0 = ox * a.stride - a.pad;
            const float *xb = a.x + (static_cast<size_t>(b) * CIN * a.H + iy0) * a.W + ix0;   // may point outside: only
                                                                                           // dereferenced when valid
            const bool interior = iy0 >= 0 && iy0 + 2 < a.H && gx * 32 * a.stride - a.pad >= 0 &&
                                  (gx * 32 + 31) * a.stride - a.pad + 2 < a.W;
            float v[16];
            if (interior)
            {
#pragma unroll
                for (int i = 0; i < 16; ++i) v[i] = kky[i] >= 0 ? xb[koff[i]] : 0.f;
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 16; ++i)
                {
                    const int iy = iy0 + kky[i], ix = ix0 + kkx[i];
                    v[i] = (iy >= 0 && iy < a.H && ix >= 0 && ix < a.W && ox < a.OW) ? xb[koff[i]] : 0.f;
                }
            }
            f16x8 b0, b1;
#pragma unroll
            for (int e = 0; e < 8; ++e) { b0[e] = static_cast<f16>(v[e]); b1[e] = static_cast<f16>(v[8 + e]); }
            f32x16 acc;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = 0.f;
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa0, b0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa1, b1, acc, 0, 0, 0);
            if (ox < a.OW)
            {
                f16x8 o0, o1;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    float t = acc[r] * sc[r] + sh[r];
                    t = lin ? (t > 0.f ? t : slope * t) : activate(t, a.act, a.actParam);
                    t *= a.outMul;
                    if (r < 8) o0[r] = static_cast<f16>(t); else o1[r - 8] = static_cast<f16>(t);
                }
                f16 *yp = a.y + (static_cast<size_t>(row) * a.OW + ox) * a.outLd + mb * 32 + 16 * h;
                *reinterpret_cast<f16x8 *>(yp) = o0;
                *reinterpret_cast<f16x8 *>(yp + 8) = o1;
            }
        }
    }
}

} // namespace

bool stemMfmaOk(const msnh_conv_desc *d)
{
    return d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16 && d->ksize == 3 && (d->in_c == 3 || d->in_c == 1) && d->groups == 1 &&
           d->dilation == 1 && d->out_c % 32 == 0 && d->out_ld % 8 == 0 && !d->has_residual;
}

size_t stemMfmaElems(const msnh_conv_desc *d) { return static_cast<size_t>(d->out_c / 32) * 2 * 64 * 8; }

// packed[mb][kb][lane][e] = W[channel(mb, lane % 32)][k = kb*16 + 8*(lane/32) + e], k = tap*Cin + ci
void stemMfmaPack(const msnh_conv_desc *d, const float *oihw, _Float16 *packed)
{
    const int cin = d->in_c, K = 9 * cin;
    for (int mb = 0; mb < d->out_c / 32; ++mb)
        for (int kb = 0; kb < 2; ++kb)
            for (int lane = 0; lane < 64; ++lane)
                for (int e = 0; e < 8; ++e)
                {
                    const int m = lane % 32;
                    const int oc = mb * 32 + 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
                    const int k = kb * 16 + 8 * (lane / 32) + e;
                    float v = 0.f;
                    if (k < K)
                    {
                        const int tap = k / cin, ci = k % cin;
                        v = oihw[(static_cast<size_t>(oc) * cin + ci) * 9 + tap];
                    }
                    packed[((static_cast<size_t>(mb) * 2 + kb) * 64 + lane) * 8 + e] = static_cast<_Float16>(v);
                }
}

int convStemMfma(const msnh_conv_desc *d, const float *x, const _Float16 *wA, const float *scale, const float *shift, void *y, hipStream_t st)
{
    MSNH_REQUIRE(stemMfmaOk(d), "conv2d: shape not supported by the matrix-core stem kernel");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(y) % 16 == 0 && reinterpret_cast<uintptr_t>(wA) % 16 == 0, "conv2d: stem needs 16-byte aligned output and weights");
    StemArgs a;
    a.x = x; a.wA = wA; a.scale = scale; a.shift = shift; a.y = static_cast<f16 *>(y);
    a.B = d->batch; a.H = d->in_h; a.W = d->in_w; a.OH = d->out_h; a.OW = d->out_w; a.outLd = d->out_ld; a.outC = d->out_c;
    a.stride = d->stride; a.pad = d->pad;
    a.groupsPerRow = (d->out_w + 31) / 32;
    const long long groups = static_cast<long long>(d->batch) * d->out_h * a.groupsPerRow;
    MSNH_REQUIRE(groups < (1LL << 31), "conv2d: stem output too large");
    a.nGroups = static_cast<int>(groups);
    a.act = d->act; a.actParam = d->act_param; a.outMul = d->out_mul;
    // 8 wavefronts per SIMD hide the gather latency; every wavefront then walks the pixel groups with a grid stride
    const long long want = (groups + 3) / 4;
    const unsigned blocks = static_cast<unsigned>(want < 256 * 8 ? (want < 1 ? 1 : want) : 256 * 8);
    if (d->in_c == 3) hipLaunchKernelGGL(convStemMfmaKernel<3>, dim3(blocks), dim3(256), 0, st, a);
    else              hipLaunchKernelGGL(convStemMfmaKernel<1>, dim3(blocks), dim3(256), 0, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
