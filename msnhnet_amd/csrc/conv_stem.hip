// First-layer convolution on the matrix cores: 3x3 / 5x5 / 7x7 filter over <= 4 input channels, read straight from
// the NCHW float32 network input (layout conversion and cast to float16 fused), NHWC float16 out.
//
// GEMM view: all output channels (32, 64 or 128) x 32 consecutive output pixels of one row per wavefront,
// K = ksize^2 * Cin padded to a multiple of 32, two 32x32x16 MFMAs per 32 of K and 32 channels.  The kernel is
// bound by the write of the output and by the scalar gathers (16 per lane and 32 of K) that assemble the B
// operand; where each K index points inside the image is a table in the kernel-argument segment, read with scalar
// loads.  The weights (operand A, already in MFMA lane order) and the channel affine sit in LDS.
//
// The rows of the MFMA are a permutation of the channels: MFMA row 8q + 4h + e computes channel 16h + 4q + e.
// The 32x32 accumulator layout gives lane l, register r the row 8(r/4) + 4(l/32) + r%4, so with that permutation
// the 16 registers of a lane are 16 CONSECUTIVE channels of its pixel: two 16-byte stores, no transposition.
#include "common.hpp"
#include <type_traits>

namespace msnh {

namespace {

template <int I, int N, typename F> __device__ __forceinline__ void staticFor(F &&f)
{
    if constexpr (I < N)
    {
        f(std::integral_constant<int, I>());
        staticFor<I + 1, N>(f);
    }
}

constexpr int kStemMaxK = 160;          // 7x7x3 = 147 padded to five 32-wide K blocks

struct StemArgs
{
    const float *x;
    const f16   *wA;        // [mBlocks][KB*2][64 lanes][8]
    const float *scale;
    const float *shift;
    f16         *y;
    int B, H, W, OH, OW, outLd, outC, stride, pad, cin, ksize;
    int groupsPerRow;       // ceil(OW / 32)
    int nGroups;            // B * OH * groupsPerRow
    int act;
    float actParam, outMul;
    // per K index: offset of the tap inside one batch item's NCHW planes (ci*H*W + ky*W + kx), and ky << 8 | kx.
    // Lives in the kernel-argument segment: the kernel indexes it with compile-time constants, i.e. scalar loads.
    int koff[kStemMaxK];
    int kyx[kStemMaxK];     // ky << 8 | kx; K padding: ky = 32767 (never inside the image)
};

// KB: 32-wide K blocks; MBLK: 32-channel output blocks
template <int KB, int MBLK>
__global__ __launch_bounds__(256) void convStemMfmaKernel(StemArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    f16 *wl = reinterpret_cast<f16 *>(smem);                                  // [MBLK][KB*2][64][8]
    float *ssl = reinterpret_cast<float *>(smem + MBLK * KB * 2 * 1024);       // [2][MBLK*32]
    for (int i = threadIdx.x; i < MBLK * KB * 2 * 64; i += 256)
        reinterpret_cast<f16x8 *>(wl)[i] = reinterpret_cast<const f16x8 *>(a.wA)[i];
    for (int i = threadIdx.x; i < MBLK * 32; i += 256)
    {
        ssl[i] = a.scale ? a.scale[i] : 1.f;
        ssl[MBLK * 32 + i] = a.shift ? a.shift[i] : 0.f;
    }
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int n = lane & 31;
    const bool hi = lane >= 32;
    const int wavesTotal = gridDim.x * 4;
    const int wave0 = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int planes = a.cin * a.H * a.W;

    const bool lin = (a.act == MSNH_ACT_LEAKY || a.act == MSNH_ACT_RELU || a.act == MSNH_ACT_NONE);
    const float slope = a.act == MSNH_ACT_LEAKY ? a.actParam : (a.act == MSNH_ACT_RELU ? 0.f : 1.f);

    for (int g = wave0; g < a.nGroups; g += wavesTotal)
    {
        const int gx = g % a.groupsPerRow;
        const int row = g / a.groupsPerRow;
        const int oy = row % a.OH;
        const int b = row / a.OH;
        const int ox = gx * 32 + n;
        const int iy0 = oy * a.stride - a.pad;
        const int ix0 = ox * a.stride - a.pad;
        // valid taps are dereferenced only; the base may lie outside the tensor
        const float *xb = a.x + static_cast<long long>(b) * planes + static_cast<long long>(iy0) * a.W + ix0;
        f32x16 acc[MBLK];
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][r] = 0.f;

        // wave-uniform: every tap of every pixel of the group lies inside the image (no bounds tests then)
        const int ixFirst = gx * 32 * a.stride - a.pad;
        const int ixLast  = (gx * 32 + 31) * a.stride - a.pad;
        const bool interior = iy0 >= 0 && iy0 + a.ksize <= a.H && ixFirst >= 0 && ixLast + a.ksize <= a.W && gx * 32 + 31 < a.OW;
        staticFor<0, KB>([&](auto kbTag) {
            constexpr int kb = decltype(kbTag)::value;
            float v[16];
            if (interior)
            {
#pragma unroll
                for (int i = 0; i < 16; ++i)
                {
                    // lanes 0-31 hold K index kLo, lanes 32-63 kLo + 8; K padding has offset 0 and a zero weight
                    const int kLo = kb * 32 + (i / 8) * 16 + (i % 8);
                    v[i] = xb[hi ? a.koff[kLo + 8] : a.koff[kLo]];
                }
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 16; ++i)
                {
                    const int kLo = kb * 32 + (i / 8) * 16 + (i % 8);
                    const int off = hi ? a.koff[kLo + 8] : a.koff[kLo];
                    const int yx  = hi ? a.kyx[kLo + 8] : a.kyx[kLo];
                    const unsigned iy = static_cast<unsigned>(iy0 + (yx >> 8)), ix = static_cast<unsigned>(ix0 + (yx & 255));
                    v[i] = (iy < static_cast<unsigned>(a.H) && ix < static_cast<unsigned>(a.W)) ? xb[off] : 0.f;
                }
            }
            f16x8 b0, b1;
#pragma unroll
            for (int e = 0; e < 8; ++e) { b0[e] = static_cast<f16>(v[e]); b1[e] = static_cast<f16>(v[8 + e]); }
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb)
            {
                const f16x8 wa0 = *reinterpret_cast<const f16x8 *>(wl + ((static_cast<size_t>(mb) * KB * 2 + kb * 2 + 0) * 64 + lane) * 8);
                const f16x8 wa1 = *reinterpret_cast<const f16x8 *>(wl + ((static_cast<size_t>(mb) * KB * 2 + kb * 2 + 1) * 64 + lane) * 8);
                acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa0, b0, acc[mb], 0, 0, 0);
                acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa1, b1, acc[mb], 0, 0, 0);
            }
        });
        if (ox < a.OW)
        {
            f16 *yp = a.y + (static_cast<size_t>(row) * a.OW + ox) * a.outLd + (hi ? 16 : 0);
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb)
            {
                const float *scp = ssl + mb * 32 + (hi ? 16 : 0);
                const float *shp = scp + MBLK * 32;
                f16x8 o0, o1;
                float t[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) t[r] = acc[mb][r] * scp[r] + shp[r];
                if (lin)
                {
#pragma unroll
                    for (int r = 0; r < 16; ++r) t[r] = t[r] > 0.f ? t[r] : slope * t[r];
                }
                else activateArray<16>(t, a.act, a.actParam);       // one choice of the activation for the 16 values
#pragma unroll
                for (int r = 0; r < 16; ++r)
                {
                    const float u = t[r] * a.outMul;
                    if (r < 8) o0[r] = static_cast<f16>(u); else o1[r - 8] = static_cast<f16>(u);
                }
                *reinterpret_cast<f16x8 *>(yp + mb * 32) = o0;
                *reinterpret_cast<f16x8 *>(yp + mb * 32 + 8) = o1;
            }
        }
    }
}

template <int KB, int MBLK>
int launchStem(const StemArgs &a, unsigned blocks, hipStream_t st)
{
    const size_t smem = static_cast<size_t>(MBLK) * KB * 2 * 1024 + 2 * MBLK * 32 * sizeof(float);
    auto kern = convStemMfmaKernel<KB, MBLK>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), smem, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

inline int stemKBlocks(const msnh_conv_desc *d) { return (d->ksize * d->ksize * d->in_c + 31) / 32; }

} // namespace

bool stemMfmaOk(const msnh_conv_desc *d)
{
    const int mb = d->out_c / 32;
    return d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16 && (d->ksize == 3 || d->ksize == 5 || d->ksize == 7) && d->in_c >= 1 && d->in_c <= 4 &&
           d->ksize * d->ksize * d->in_c <= kStemMaxK && d->groups == 1 && d->dilation == 1 && d->out_c % 32 == 0 && (mb == 1 || mb == 2 || mb == 4) &&
           d->out_ld % 8 == 0 && !d->has_residual && d->in_h < 30000;
}

size_t stemMfmaElems(const msnh_conv_desc *d) { return static_cast<size_t>(d->out_c / 32) * stemKBlocks(d) * 2 * 64 * 8; }

// packed[mb][kb16][lane][e] = W[channel(mb, lane % 32)][k = kb16*16 + 8*(lane/32) + e], k = tap*Cin + ci
void stemMfmaPack(const msnh_conv_desc *d, const float *oihw, _Float16 *packed)
{
    const int cin = d->in_c, kk = d->ksize * d->ksize, K = kk * cin, KB2 = stemKBlocks(d) * 2;
    for (int mb = 0; mb < d->out_c / 32; ++mb)
        for (int kb = 0; kb < KB2; ++kb)
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
                        v = oihw[(static_cast<size_t>(oc) * cin + ci) * kk + tap];
                    }
                    packed[((static_cast<size_t>(mb) * KB2 + kb) * 64 + lane) * 8 + e] = static_cast<_Float16>(v);
                }
}

int convStemMfma(const msnh_conv_desc *d, const float *x, const _Float16 *wA, const float *scale, const float *shift, void *y, hipStream_t st)
{
    MSNH_REQUIRE(stemMfmaOk(d), "conv2d: shape not supported by the matrix-core stem kernel");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(y) % 16 == 0 && reinterpret_cast<uintptr_t>(wA) % 16 == 0, "conv2d: stem needs 16-byte aligned output and weights");
    StemArgs a;
    a.x = x; a.wA = wA; a.scale = scale; a.shift = shift; a.y = static_cast<f16 *>(y);
    a.B = d->batch; a.H = d->in_h; a.W = d->in_w; a.OH = d->out_h; a.OW = d->out_w; a.outLd = d->out_ld; a.outC = d->out_c;
    a.stride = d->stride; a.pad = d->pad; a.cin = d->in_c; a.ksize = d->ksize;
    a.groupsPerRow = (d->out_w + 31) / 32;
    const long long groups = static_cast<long long>(d->batch) * d->out_h * a.groupsPerRow;
    MSNH_REQUIRE(groups < (1LL << 31) && static_cast<long long>(d->in_c) * d->in_h * d->in_w < (1LL << 31), "conv2d: stem tensor too large");
    a.nGroups = static_cast<int>(groups);
    a.act = d->act; a.actParam = d->act_param; a.outMul = d->out_mul;
    const int K = d->ksize * d->ksize * d->in_c;
    for (int k = 0; k < kStemMaxK; ++k)
    {
        if (k < K)
        {
            const int tap = k / d->in_c, ci = k % d->in_c;
            const int ky = tap / d->ksize, kx = tap % d->ksize;
            a.koff[k] = (ci * d->in_h + ky) * d->in_w + kx;
            a.kyx[k] = ky << 8 | kx;
        }
        else { a.koff[k] = 0; a.kyx[k] = 32767 << 8; }
    }
    // several wavefronts per SIMD hide the gather latency; every wavefront walks the pixel groups with a grid stride
    const long long want = (groups + 3) / 4;
    const int kb = stemKBlocks(d), mb = d->out_c / 32;
    const long long cap = 256 * (kb <= 2 ? 8 : 4);             // measured: short K wants more wavefronts in flight
    const unsigned blocks = static_cast<unsigned>(want < cap ? (want < 1 ? 1 : want) : cap);
#define MSNH_STEM(KBV, MBV) if (kb == KBV && mb == MBV) return launchStem<KBV, MBV>(a, blocks, st)
    MSNH_STEM(1, 1); MSNH_STEM(1, 2); MSNH_STEM(1, 4);
    MSNH_STEM(2, 1); MSNH_STEM(2, 2); MSNH_STEM(2, 4);
    MSNH_STEM(3, 1); MSNH_STEM(3, 2); MSNH_STEM(3, 4);
    MSNH_STEM(4, 1); MSNH_STEM(4, 2); MSNH_STEM(4, 4);
    MSNH_STEM(5, 1); MSNH_STEM(5, 2); MSNH_STEM(5, 4);
#undef MSNH_STEM
    setError("conv2d: stem shape not instantiated");
    return 2;
}

} // namespace msnh
