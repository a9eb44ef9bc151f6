// First-layer convolution on the matrix cores: 3x3 / 5x5 / 7x7 filter over <= 4 input channels (7x7 over 3 channels has a
// kernel of its own further down), read straight from
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
    // A workgroup takes one contiguous run of pixel groups (its four wavefronts interleaved), and the hardware's round-robin of
    // workgroup ids over the 8 XCDs is undone so that an XCD works on one contiguous run of image rows: the input rows that
    // neighbouring output rows share are then read from memory once, not once per XCD that happens to need them.
    const int nBlocks = static_cast<int>(gridDim.x);
    const int perXcd = (nBlocks + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    const int perBlock = (a.nGroups + nBlocks - 1) / nBlocks;
    const int gBegin = logical < nBlocks ? logical * perBlock : a.nGroups;
    const int gEnd = min(a.nGroups, gBegin + perBlock);
    const int planes = a.cin * a.H * a.W;

    const bool lin = (a.act == MSNH_ACT_LEAKY || a.act == MSNH_ACT_RELU || a.act == MSNH_ACT_NONE);
    const float slope = a.act == MSNH_ACT_LEAKY ? a.actParam : (a.act == MSNH_ACT_RELU ? 0.f : 1.f);

    for (int g = gBegin + static_cast<int>(threadIdx.x >> 6); g < gEnd; g += 4)
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
    hipLaunchKernelGGL(kern, dim3((blocks + 7) / 8 * 8), dim3(256), smem, st, a);      // a multiple of 8: the XCD regrouping is a bijection then
    MSNH_LAUNCH_CHECK();
    return 0;
}

// ---- 7x7 filters over 3 channels (the ResNet stems): K ordered by image rows ------------------------------------------------
// The gather kernel above issues one 4-byte load, one conversion and one select per K index and lane: 147 of each for a
// 7x7x3 filter, and the vector ALU, not memory, sets its time.  Here K is laid out as 21 (channel, filter row) pairs of
// 8 values each (7 taps + one zero): the 7 taps of a pair are 7 consecutive floats of one image row, so a lane fetches
// its half of a 16-wide K chunk with two 16-byte loads and converts it in place.  11 chunks (K = 176 with zero weights in
// the padding) instead of 10, but a fifth of the instructions.  Loads go through a buffer resource: a vector that starts
// left of the image or ends past the tensor reads zeros or a neighbouring row, and whatever lies outside the image is
// blanked before the conversion (only in groups that touch the border), the eighth value always.
// 16-byte load through a buffer resource: the hardware checks the byte offset against the resource size and returns zeros
// beyond it (an index that went negative wraps to an offset past the end)
typedef int stemI32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t stemRsrc(const void *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes), 0x00020000);
}
__device__ __forceinline__ f32x4 stemLoad16(__amdgpu_buffer_rsrc_t r, unsigned voffset)
{
    const stemI32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(voffset), 0, 0);
    return __builtin_bit_cast(f32x4, v);
}

constexpr int kRowChunks = 11;          // ceil(3 * 7 / 2) chunks of two (channel, filter row) pairs

struct StemRowsArgs
{
    const float *x;
    const f16   *wA;        // [mBlocks][kRowChunks][64 lanes][8]
    const float *scale;
    const float *shift;
    f16         *y;
    int B, H, W, OH, OW, outLd, stride, pad;
    int groupsPerRow, nGroups;
    unsigned xBytes;
    int act;
    float actParam, outMul;
    int rowOff[2 * kRowChunks];     // (ci * H + ky) * W of pair r; padding pair: 0
    int rowKy[2 * kRowChunks];      // ky of pair r; padding pair: 32767 (never inside the image)
};

template <int MBLK>
__global__ __launch_bounds__(256) void convStemRowsKernel(StemRowsArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    f16 *wl = reinterpret_cast<f16 *>(smem);                                        // [MBLK][kRowChunks][64][8]
    float *ssl = reinterpret_cast<float *>(smem + MBLK * kRowChunks * 1024);         // [2][MBLK*32]
    for (int i = threadIdx.x; i < MBLK * kRowChunks * 64; i += 256)
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
    // (contiguous runs of pixel groups per workgroup, XCD by XCD: see convStemMfmaKernel)
    const int nBlocks = static_cast<int>(gridDim.x);
    const int perXcd = (nBlocks + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    const int perBlock = (a.nGroups + nBlocks - 1) / nBlocks;
    const int gBegin = logical < nBlocks ? logical * perBlock : a.nGroups;
    const int gEnd = min(a.nGroups, gBegin + perBlock);
    const int planes = 3 * a.H * a.W;
    const __amdgpu_buffer_rsrc_t rx = stemRsrc(a.x, a.xBytes);

    const bool lin = (a.act == MSNH_ACT_LEAKY || a.act == MSNH_ACT_RELU || a.act == MSNH_ACT_NONE);
    const float slope = a.act == MSNH_ACT_LEAKY ? a.actParam : (a.act == MSNH_ACT_RELU ? 0.f : 1.f);

    for (int g = gBegin + static_cast<int>(threadIdx.x >> 6); g < gEnd; g += 4)
    {
        const int gx = g % a.groupsPerRow;
        const int row = g / a.groupsPerRow;
        const int oy = row % a.OH;
        const int b = row / a.OH;
        const int ox = gx * 32 + n;
        const int iy0 = oy * a.stride - a.pad;
        const int ix0 = ox * a.stride - a.pad;
        const int base = b * planes + iy0 * a.W + ix0;             // element index of the window's corner; may be negative
        f32x16 acc[MBLK];
#pragma unroll
        for (int mb = 0; mb < MBLK; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mb][r] = 0.f;

        // wave-uniform: every tap of every pixel of the group lies inside the image (no blanking then)
        const int ixFirst = gx * 32 * a.stride - a.pad;
        const int ixLast  = (gx * 32 + 31) * a.stride - a.pad;
        const bool interior = iy0 >= 0 && iy0 + 7 <= a.H && ixFirst >= 0 && ixLast + 7 <= a.W && gx * 32 + 31 < a.OW;
        staticFor<0, kRowChunks>([&](auto cTag) {
            constexpr int c = decltype(cTag)::value;
            const int off = base + (hi ? a.rowOff[2 * c + 1] : a.rowOff[2 * c]);
            const unsigned voff = static_cast<unsigned>(off) * 4u;  // a negative index wraps past the end of the buffer: zeros
            f32x4 lo4 = stemLoad16(rx, voff);
            f32x4 hi4 = stemLoad16(rx, voff + 16u);
            float v[8] = {lo4[0], lo4[1], lo4[2], lo4[3], hi4[0], hi4[1], hi4[2], 0.f};
            if (!interior)
            {
                const int ky = hi ? a.rowKy[2 * c + 1] : a.rowKy[2 * c];
                const bool rowOk = static_cast<unsigned>(iy0 + ky) < static_cast<unsigned>(a.H);
                if (off < 0 && rowOk)
                {
                    // the first image row of the first plane, left border: the 16-byte vectors would start in front of the
                    // tensor (and their offsets wrap), so the taps that exist are fetched one by one
#pragma unroll
                    for (int e = 0; e < 7; ++e)
                        v[e] = off + e >= 0 ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rx, (off + e) * 4, 0, 0)) : 0.f;
                }
#pragma unroll
                for (int e = 0; e < 7; ++e) v[e] = (rowOk && static_cast<unsigned>(ix0 + e) < static_cast<unsigned>(a.W)) ? v[e] : 0.f;
            }
            f16x8 bf;
#pragma unroll
            for (int e = 0; e < 8; ++e) bf[e] = static_cast<f16>(v[e]);
#pragma unroll
            for (int mb = 0; mb < MBLK; ++mb)
            {
                const f16x8 wa = *reinterpret_cast<const f16x8 *>(wl + ((static_cast<size_t>(mb) * kRowChunks + c) * 64 + lane) * 8);
                acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa, bf, acc[mb], 0, 0, 0);
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
                else activateArray<16>(t, a.act, a.actParam);
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

template <int MBLK>
int launchStemRows(const StemRowsArgs &a, unsigned blocks, hipStream_t st)
{
    const size_t smem = static_cast<size_t>(MBLK) * kRowChunks * 1024 + 2 * MBLK * 32 * sizeof(float);
    auto kern = convStemRowsKernel<MBLK>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, dim3((blocks + 7) / 8 * 8), dim3(256), smem, st, a);      // a multiple of 8: the XCD regrouping is a bijection then
    MSNH_LAUNCH_CHECK();
    return 0;
}

// the row-ordered kernel takes 7x7 filters over 3 channels whose whole input is addressable with 32-bit byte offsets
inline bool stemRowsOk(const msnh_conv_desc *d)
{
    return d->ksize == 7 && d->in_c == 3 && static_cast<long long>(d->batch) * 3 * d->in_h * d->in_w * 4 < 0x7fffffffLL;
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

size_t stemMfmaElems(const msnh_conv_desc *d)
{
    return static_cast<size_t>(d->out_c / 32) * (stemRowsOk(d) ? kRowChunks : stemKBlocks(d) * 2) * 64 * 8;
}

// packed[mb][kb16][lane][e] = W[channel(mb, lane % 32)][k = kb16*16 + 8*(lane/32) + e], k = tap*Cin + ci
void stemMfmaPack(const msnh_conv_desc *d, const float *oihw, _Float16 *packed)
{
    const int cin = d->in_c, kk = d->ksize * d->ksize, K = kk * cin, KB2 = stemKBlocks(d) * 2;
    if (stemRowsOk(d))
    {
        // packed[mb][chunk][lane][e] = W[channel(mb, lane % 32)][ci][ky][kx = e], (ci, ky) = pair 2 * chunk + lane / 32
        for (int mb = 0; mb < d->out_c / 32; ++mb)
            for (int c = 0; c < kRowChunks; ++c)
                for (int lane = 0; lane < 64; ++lane)
                    for (int e = 0; e < 8; ++e)
                    {
                        const int m = lane % 32;
                        const int oc = mb * 32 + 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3);
                        const int pair = 2 * c + lane / 32;
                        float v = 0.f;
                        if (pair < 21 && e < 7) v = oihw[(static_cast<size_t>(oc) * 3 + pair / 7) * 49 + (pair % 7) * 7 + e];
                        packed[((static_cast<size_t>(mb) * kRowChunks + c) * 64 + lane) * 8 + e] = static_cast<_Float16>(v);
                    }
        return;
    }
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
    if (stemRowsOk(d))
    {
        StemRowsArgs r;
        r.x = x; r.wA = wA; r.scale = scale; r.shift = shift; r.y = static_cast<f16 *>(y);
        r.B = d->batch; r.H = d->in_h; r.W = d->in_w; r.OH = d->out_h; r.OW = d->out_w; r.outLd = d->out_ld; r.stride = d->stride; r.pad = d->pad;
        r.groupsPerRow = (d->out_w + 31) / 32;
        const long long groups = static_cast<long long>(d->batch) * d->out_h * r.groupsPerRow;
        MSNH_REQUIRE(groups < (1LL << 31), "conv2d: stem tensor too large");
        r.nGroups = static_cast<int>(groups);
        r.xBytes = static_cast<unsigned>(static_cast<long long>(d->batch) * 3 * d->in_h * d->in_w * 4);
        r.act = d->act; r.actParam = d->act_param; r.outMul = d->out_mul;
        for (int p = 0; p < 2 * kRowChunks; ++p)
        {
            r.rowOff[p] = p < 21 ? ((p / 7) * d->in_h + p % 7) * d->in_w : 0;
            r.rowKy[p] = p < 21 ? p % 7 : 32767;
        }
        const long long want = (groups + 3) / 4;
        const unsigned blocks = static_cast<unsigned>(want < 256 * 4 ? (want < 1 ? 1 : want) : 256 * 4);     // (2..8 workgroups per CU measure alike)
        switch (d->out_c / 32)
        {
        case 1: return launchStemRows<1>(r, blocks, st);
        case 2: return launchStemRows<2>(r, blocks, st);
        default: return launchStemRows<4>(r, blocks, st);
        }
    }
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
