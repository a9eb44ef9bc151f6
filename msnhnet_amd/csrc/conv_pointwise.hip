// 1x1 stride-1 convolution with few channels (in_c <= 128, out_c <= 128, float16): the bandwidth-bound pointwise
// layers of MobileNetV2, of the high-resolution stages of the YOLO graphs and of ResNet bottlenecks.
//
// Such a layer is a GEMM with a K of 16..128: in the tiled implicit GEMM a workgroup spends its life in the
// prologue and the epilogue of a two- or four-step loop.  Here nothing but the weights goes through LDS and there
// is no barrier after the first one:
//   * the whole weight matrix sits in LDS in matrix-core fragment order (rows permuted so that the 16 accumulators
//     of a lane are 16 consecutive output channels), with the channel affine beside it;
//   * a wavefront owns strips of 64 (32 for more than 64 output channels) consecutive pixels (of the batch-flattened image) and walks over them
//     persistently; the pixel operand is loaded from global memory straight into fragment registers -- for the
//     32x32x16 MFMA a lane's 8 K values are 16 contiguous bytes of one pixel's channel vector -- through a buffer
//     resource, so pixels past the end and channels past in_c read zeros;
//   * once the MFMAs of a strip have consumed the fragment registers, the loads of the wave's next strip are
//     issued into them and stay in flight during the strip's epilogue (affine, activation, residual, second
//     activation, scale; two 16-byte stores per lane and 32-channel block, straight from the accumulators).
#include "conv_igemm.hpp"

namespace msnh {

struct PwArgs
{
    const f16   *x;
    const f16   *w;         // [out_c][in_c]
    const float *scale;
    const float *shift;
    const f16   *res;
    f16         *y;
    int P, cin, cout, inLd, outLd, resLd, strips;
    unsigned xBytes;
    int act, act2, hasRes;
    float actParam, act2Param, resMul, outMul;
};

// MFMA row r of a 32-row block carries output channel pwChannelOfRow(r): the accumulator registers i = 0..15 of a
// lane in half h then hold channels 16h + i.
__device__ __forceinline__ int pwChannelOfRow(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

// Register budget: at least three wavefronts per SIMD (four for a single channel block, one fewer for in_c > 64) -- the only
// latency hiding this kernel has is other wavefronts; strips narrow to 32 pixels for three and four channel blocks to make room.
constexpr int pwStripBlocks(int mb) { return mb <= 2 ? 2 : 1; }

template <int MB, int KS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu((MB == 1 ? 4 : 3) - (KS >= 6 ? 1 : 0))))
void convPointwiseKernel(PwArgs a)
{
    constexpr int NB  = pwStripBlocks(MB);            // 32-pixel column blocks per strip
    constexpr int NCH = KS * 2;                       // 16-byte chunks per weight row
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    f16x8 *wl = reinterpret_cast<f16x8 *>(smem);
    float *sc = reinterpret_cast<float *>(smem + MB * 32 * NCH * 16);
    float *sh = sc + MB * 32;
    const int tid = threadIdx.x;

    // ---- weights and affine into LDS (once) -------------------------------------------------------------------
    for (int idx = tid; idx < MB * 32 * NCH; idx += 256)
    {
        const int r = idx / NCH, ch = idx - r * NCH;
        const int rr = r & 31;
        const int c = (r & ~31) + pwChannelOfRow(rr);
        f16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (c < a.cout && ch * 8 < a.cin) v = *reinterpret_cast<const f16x8 *>(a.w + static_cast<size_t>(c) * a.cin + ch * 8);
        wl[r * NCH + (ch + rr * NCH / 16) % NCH] = v;  // rotated so that 16 lanes reading one chunk index hit 16 different banks groups
    }
    for (int c = tid; c < MB * 32; c += 256)
    {
        sc[c] = c < a.cout ? (a.scale ? a.scale[c] : 1.f) : 0.f;
        sh[c] = c < a.cout ? (a.shift ? a.shift[c] : 0.f) : 0.f;
    }
    __syncthreads();

    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5, n = lane & 31;
    const __amdgpu_buffer_rsrc_t rx = makeRsrc(a.x, a.xBytes);
    const int totalWaves = gridDim.x * 4;

    f16x8 b[NB][KS];
    auto loadB = [&](int strip) {
#pragma unroll
        for (int j = 0; j < NB; ++j)
        {
            const int p = strip * (32 * NB) + 32 * j + n;
#pragma unroll
            for (int s = 0; s < KS; ++s)
            {
                const int koff = 16 * s + 8 * h;
                const unsigned voff = (p < a.P && koff < a.cin) ? (static_cast<unsigned>(p) * a.inLd + koff) * 2u : kOobOffset;
                b[j][s] = bufferLoad16<f16x8>(rx, voff, 0);
            }
        }
    };

    int strip = blockIdx.x * 4 + wave;
    if (strip < a.strips) loadB(strip);
    for (; strip < a.strips; strip += totalWaves)
    {
        f32x16 acc[MB][NB];
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
#pragma unroll
        for (int s = 0; s < KS; ++s)
#pragma unroll
            for (int i = 0; i < MB; ++i)
            {
                const f16x8 af = wl[(32 * i + n) * NCH + (2 * s + h + n * NCH / 16) % NCH];
#pragma unroll
                for (int j = 0; j < NB; ++j) mfmaBlock(af, b[j][s], acc[i][j]);
            }
        // the fragment registers are free: the next strip's pixels travel while this strip's results are written
        const int next = strip + totalWaves;
        if (next < a.strips) loadB(next);

#pragma unroll
        for (int j = 0; j < NB; ++j)
        {
            const int p = strip * (32 * NB) + 32 * j + n;
            if (p >= a.P) continue;
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int g = 0; g < 2; ++g)
                {
                    const int c0 = 32 * i + 16 * h + 8 * g;
                    if (c0 >= a.cout) continue;
                    float v[8];
                    const f32x4 s0 = *reinterpret_cast<const f32x4 *>(sc + c0), s1 = *reinterpret_cast<const f32x4 *>(sc + c0 + 4);
                    const f32x4 h0 = *reinterpret_cast<const f32x4 *>(sh + c0), h1 = *reinterpret_cast<const f32x4 *>(sh + c0 + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                    {
                        v[e]     = acc[i][j][8 * g + e] * s0[e] + h0[e];
                        v[4 + e] = acc[i][j][8 * g + 4 + e] * s1[e] + h1[e];
                    }
                    activateArray<8>(v, a.act, a.actParam);
                    if (a.hasRes)
                    {
                        const f16x8 r = *reinterpret_cast<const f16x8 *>(a.res + static_cast<size_t>(p) * a.resLd + c0);
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[e] += a.resMul * static_cast<float>(r[e]);
                        activateArray<8>(v, a.act2, a.act2Param);
                    }
                    f16x8 o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) o[e] = static_cast<f16>(a.outMul * v[e]);
                    *reinterpret_cast<f16x8 *>(a.y + static_cast<size_t>(p) * a.outLd + c0) = o;
                }
        }
    }
}

template <int MB, int KS>
static int launchPointwise(PwArgs a, hipStream_t st)
{
    a.strips = (a.P + 32 * pwStripBlocks(MB) - 1) / (32 * pwStripBlocks(MB));
    const size_t lds = static_cast<size_t>(MB) * 32 * KS * 2 * 16 + static_cast<size_t>(MB) * 32 * 2 * sizeof(float);
    int blocks = (a.strips + 3) / 4;
    if (blocks > 256 * 3) blocks = 256 * 3;
    hipLaunchKernelGGL((convPointwiseKernel<MB, KS>), dim3(blocks), dim3(256), lds, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

template <int MB>
static int dispatchKs(const PwArgs &a, int ks, hipStream_t st)
{
    switch (ks)
    {
    case 1: return launchPointwise<MB, 1>(a, st);
    case 2: return launchPointwise<MB, 2>(a, st);
    case 3: return launchPointwise<MB, 3>(a, st);
    case 4: return launchPointwise<MB, 4>(a, st);
    case 5: case 6: return launchPointwise<MB, 6>(a, st);
    default: return launchPointwise<MB, 8>(a, st);
    }
}

bool pointwiseOk(const msnh_conv_desc *d)
{
    return d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16 && d->ksize == 1 && d->stride == 1 && d->pad == 0 && d->groups == 1 &&
           d->in_c % 8 == 0 && d->in_c <= 128 && d->out_c % 8 == 0 && d->out_c <= 128 && d->in_ld % 8 == 0 && d->out_ld % 8 == 0 &&
           (!d->has_residual || d->res_ld % 8 == 0) && d->in_h == d->out_h && d->in_w == d->out_w;
}

int convPointwise(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, const void *residual,
                  void *y, hipStream_t st)
{
    MSNH_REQUIRE(pointwiseOk(d), "conv2d: shape not supported by the pointwise kernel");
    const long long P = static_cast<long long>(d->batch) * d->out_h * d->out_w;
    const unsigned long long xb = (static_cast<unsigned long long>(P - 1) * d->in_ld + d->in_c) * 2ull;
    MSNH_REQUIRE(xb < 0x7fffffffull, "conv2d: the pointwise kernel needs an input below 2 GiB");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                 (!d->has_residual || reinterpret_cast<uintptr_t>(residual) % 16 == 0), "conv2d: the pointwise kernel needs 16-byte aligned tensors");
    PwArgs a;
    a.x = static_cast<const f16 *>(x); a.w = static_cast<const f16 *>(w); a.scale = scale; a.shift = shift;
    a.res = static_cast<const f16 *>(residual); a.y = static_cast<f16 *>(y);
    a.P = static_cast<int>(P); a.cin = d->in_c; a.cout = d->out_c; a.inLd = d->in_ld; a.outLd = d->out_ld; a.resLd = d->res_ld;
    a.strips = static_cast<int>((P + 63) / 64);
    a.xBytes = static_cast<unsigned>(xb);
    a.act = d->act; a.act2 = d->act2; a.hasRes = (d->has_residual && residual) ? 1 : 0;
    a.actParam = d->act_param; a.act2Param = d->act2_param; a.resMul = d->res_mul; a.outMul = d->out_mul;
    const int ks = (d->in_c + 15) / 16;
    switch ((d->out_c + 31) / 32)
    {
    case 1: return dispatchKs<1>(a, ks, st);
    case 2: return dispatchKs<2>(a, ks, st);
    case 3: return dispatchKs<3>(a, ks, st);
    default: return dispatchKs<4>(a, ks, st);
    }
}

} // namespace msnh
