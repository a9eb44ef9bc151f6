// Depthwise 3x3 convolution (groups == channels), float16 NHWC, stride 1 or 2: the bandwidth kernel of the
// MobileNet family.  A thread owns 2 (4, 8) channels of a strip of 4 consecutive output pixels of one row:
//   * the nine filter taps of its 8 channels are loaded once (weights [tap][C]) instead of once per output pixel;
//   * per input row the strip needs 6 (stride 1) or 9 (stride 2) 16-byte pixel vectors, each used by up to three
//     outputs: 4.5 / 6.75 loads per output pixel instead of 9, all of them issued before the first use;
//   * loads go through a buffer resource, so pixels outside the image are an out-of-range offset that reads zeros:
//     no branches around the taps.
// Consecutive lanes take consecutive channel vectors of the same strip, so every load instruction of a wavefront
// covers whole pixels.
#include "common.hpp"
#include <cstdlib>

namespace msnh {

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned kOob = 0x80000000u;

struct DwArgs
{
    const f16 *x;
    const f16 *w;
    const float *scale;
    const float *shift;
    f16 *y;
    int H, W, inLd, OH, OW, outLd, C, pad;
    int strips;             // ceil(OW / 4)
    long long total;        // B * OH * strips * (C / channels per lane)
    unsigned xBytes;
    int act;
    float actParam, outMul;
};

template <int STRIDE, int CPL>
__global__ __launch_bounds__(256) void convDepthwise3x3Kernel(DwArgs a, int blocks)
{
    constexpr int COLS = 3 * STRIDE + 3;          // input columns feeding 4 outputs: (4 - 1) * STRIDE + 3
    typedef f16 HV __attribute__((ext_vector_type(CPL)));          // CPL channels per lane: one 16-, 8- or 4-byte access
    // Consecutive hardware workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.  Regrouped so that an XCD
    // works on one contiguous run of rows: the input rows an output row shares with the rows above and below it are then found
    // in the same L2 instead of being fetched from memory by three of them.
    const int perXcd = (blocks + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    if (logical >= blocks) return;
    const long long idx = static_cast<long long>(logical) * 256 + threadIdx.x;
    if (idx >= a.total) return;
    const int cv = a.C / CPL;
    const int c0 = static_cast<int>(idx % cv) * CPL;
    long long t = idx / cv;
    const int sx = static_cast<int>(t % a.strips);
    t /= a.strips;
    const int oy = static_cast<int>(t % a.OH);
    const int b  = static_cast<int>(t / a.OH);
    const int ox0 = sx * 4;
    const int iy0 = oy * STRIDE - a.pad;
    const int ix0 = ox0 * STRIDE - a.pad;

    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<f16 *>(a.x), 0, static_cast<int>(a.xBytes), 0x00020000);

    HV wv[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) wv[k] = *reinterpret_cast<const HV *>(a.w + static_cast<size_t>(k) * a.C + c0);

    // byte offset of input pixel (iy0, ix0), channel c0; may be "negative": it wraps back once a valid tap is added
    const unsigned base = static_cast<unsigned>(((static_cast<long long>(b) * a.H + iy0) * a.W + ix0) * a.inLd + c0) * 2u;
    unsigned colOff[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c)
    {
        const int ix = ix0 + c;
        colOff[c] = (ix >= 0 && ix < a.W) ? base + static_cast<unsigned>(c * a.inLd) * 2u : kOob;
    }
    float acc[4][CPL];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < CPL; ++e) acc[j][e] = 0.f;

    HV xv[3][COLS];
#pragma unroll
    for (int r = 0; r < 3; ++r)
    {
        const int iy = iy0 + r;
        const bool rowOk = iy >= 0 && iy < a.H;
        const unsigned rowOff = static_cast<unsigned>(r * a.W * a.inLd) * 2u;
#pragma unroll
        for (int c = 0; c < COLS; ++c)
        {
            const unsigned off = (rowOk && colOff[c] != kOob) ? colOff[c] + rowOff : kOob;
            if constexpr (CPL == 8) xv[r][c] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b128(rx, static_cast<int>(off), 0, 0));
            else if constexpr (CPL == 4) xv[r][c] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b64(rx, static_cast<int>(off), 0, 0));
            else xv[r][c] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b32(rx, static_cast<int>(off), 0, 0));
        }
    }
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int kx = 0; kx < 3; ++kx)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < CPL; ++e)
                    acc[j][e] += static_cast<float>(xv[r][j * STRIDE + kx][e]) * static_cast<float>(wv[r * 3 + kx][e]);

    float sc[CPL], sh[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e)
    {
        sc[e] = a.scale ? a.scale[c0 + e] : 1.f;
        sh[e] = a.shift ? a.shift[c0 + e] : 0.f;
    }
    const size_t prow = (static_cast<size_t>(b) * a.OH + oy) * a.OW;
    float v[4 * CPL];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < CPL; ++e) v[j * CPL + e] = acc[j][e] * sc[e] + sh[e];
    activateArray<4 * CPL>(v, a.act, a.actParam);
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        if (ox0 + j >= a.OW) break;
        HV o;
#pragma unroll
        for (int e = 0; e < CPL; ++e) o[e] = static_cast<f16>(a.outMul * v[j * CPL + e]);
        *reinterpret_cast<HV *>(a.y + (prow + ox0 + j) * a.outLd + c0) = o;
    }
}


// ---- the same strip kernel with 32-bit index arithmetic -------------------------------------------------------------------------
// With two channels per lane a lane produces eight outputs, and the kernel above spends more vector instructions on finding out
// which eight (three 64-bit divisions of the lane index, 64-bit address arithmetic for nine weight vectors and four stores) than on
// the 72 multiply-adds: it is bound by the vector ALU, not by memory.  Where everything fits 32 bits (lane count, input, output
// and weight bytes below 2^31 -- checked on the host) the divisions become multiplications by precomputed reciprocals
// (Granlund & Montgomery, "Division by invariant integers using multiplication", figure 4.1), every address a 32-bit buffer offset,
// and the stores past the row's end out-of-range offsets instead of branches.
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

struct DwFastArgs
{
    DwArgs d;
    FastDiv byCv, byStrips, byOH;
    unsigned wBytes, yBytes;
};

template <int STRIDE, int CPL>
__global__ __launch_bounds__(256) void convDepthwise3x3FastKernel(DwFastArgs g, int blocks)
{
    constexpr int COLS = 3 * STRIDE + 3;
    typedef f16 HV __attribute__((ext_vector_type(CPL)));
    const DwArgs &a = g.d;
    const int perXcd = (blocks + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    if (logical >= blocks) return;
    const unsigned idx = static_cast<unsigned>(logical) * 256u + threadIdx.x;
    if (idx >= static_cast<unsigned>(a.total)) return;
    const unsigned q1 = fastDiv(idx, g.byCv);
    const int c0 = static_cast<int>(idx - q1 * g.byCv.d) * CPL;
    const unsigned q2 = fastDiv(q1, g.byStrips);
    const int sx = static_cast<int>(q1 - q2 * g.byStrips.d);
    const unsigned q3 = fastDiv(q2, g.byOH);
    const int oy = static_cast<int>(q2 - q3 * g.byOH.d);
    const int b = static_cast<int>(q3);
    const int ox0 = sx * 4;
    const int iy0 = oy * STRIDE - a.pad;
    const int ix0 = ox0 * STRIDE - a.pad;

    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<f16 *>(a.x), 0, static_cast<int>(a.xBytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(const_cast<f16 *>(a.w), 0, static_cast<int>(g.wBytes), 0x00020000);
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, static_cast<int>(g.yBytes), 0x00020000);

    HV wv[9];
#pragma unroll
    for (int k = 0; k < 9; ++k)
    {
        const int off = static_cast<int>(static_cast<unsigned>(k * a.C + c0) * 2u);
        if constexpr (CPL == 4) wv[k] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b64(rw, off, 0, 0));
        else wv[k] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b32(rw, off, 0, 0));
    }

    // byte offset of input pixel (iy0, ix0), channel c0, modulo 2^32: it may lie in front of the tensor and comes back into range
    // once a valid tap's offset is added
    const unsigned base = (static_cast<unsigned>((b * a.H + iy0) * a.W + ix0) * static_cast<unsigned>(a.inLd) + static_cast<unsigned>(c0)) * 2u;
    const unsigned pixB = static_cast<unsigned>(a.inLd) * 2u;
    const unsigned rowB = static_cast<unsigned>(a.W) * pixB;
    HV xv[3][COLS];
#pragma unroll
    for (int r = 0; r < 3; ++r)
    {
        const bool rowOk = static_cast<unsigned>(iy0 + r) < static_cast<unsigned>(a.H);
#pragma unroll
        for (int c = 0; c < COLS; ++c)
        {
            const bool ok = rowOk && static_cast<unsigned>(ix0 + c) < static_cast<unsigned>(a.W);
            const unsigned off = ok ? base + static_cast<unsigned>(r) * rowB + static_cast<unsigned>(c) * pixB : kOob;
            if constexpr (CPL == 4) xv[r][c] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b64(rx, static_cast<int>(off), 0, 0));
            else xv[r][c] = __builtin_bit_cast(HV, __builtin_amdgcn_raw_buffer_load_b32(rx, static_cast<int>(off), 0, 0));
        }
    }
    float acc[4][CPL];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < CPL; ++e) acc[j][e] = 0.f;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int kx = 0; kx < 3; ++kx)
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < CPL; ++e)
                    acc[j][e] += static_cast<float>(xv[r][j * STRIDE + kx][e]) * static_cast<float>(wv[r * 3 + kx][e]);

    float sc[CPL], sh[CPL];
#pragma unroll
    for (int e = 0; e < CPL; ++e)
    {
        sc[e] = a.scale ? a.scale[c0 + e] : 1.f;
        sh[e] = a.shift ? a.shift[c0 + e] : 0.f;
    }
    float v[4 * CPL];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < CPL; ++e) v[j * CPL + e] = acc[j][e] * sc[e] + sh[e];
    activateArray<4 * CPL>(v, a.act, a.actParam);
    const unsigned obase = (static_cast<unsigned>((b * a.OH + oy) * a.OW + ox0) * static_cast<unsigned>(a.outLd) + static_cast<unsigned>(c0)) * 2u;
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        HV o;
#pragma unroll
        for (int e = 0; e < CPL; ++e) o[e] = static_cast<f16>(a.outMul * v[j * CPL + e]);
        const unsigned off = ox0 + j < a.OW ? obase + static_cast<unsigned>(j * a.outLd) * 2u : kOob;
        if constexpr (CPL == 4) __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u32x2, o), ry, static_cast<int>(off), 0, 0);
        else __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, o), ry, static_cast<int>(off), 0, 0);
    }
}

} // namespace

bool depthwise3x3Ok(const msnh_conv_desc *d, const void *x, const void *w, const void *y)
{
    const unsigned long long xb = ((static_cast<unsigned long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld + d->in_c) * 2ull;
    return d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16 && d->ksize == 3 && (d->stride == 1 || d->stride == 2) && d->dilation == 1 &&
           d->groups == d->in_c && d->out_c == d->in_c && d->in_c % 8 == 0 && d->in_ld % 8 == 0 && d->out_ld % 8 == 0 && !d->has_residual &&
           xb < 0x7fffffffull && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 &&
           reinterpret_cast<uintptr_t>(y) % 16 == 0;
}

int convDepthwise3x3(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, void *y, hipStream_t st)
{
    DwArgs a;
    a.x = static_cast<const f16 *>(x); a.w = static_cast<const f16 *>(w); a.scale = scale; a.shift = shift; a.y = static_cast<f16 *>(y);
    a.H = d->in_h; a.W = d->in_w; a.inLd = d->in_ld; a.OH = d->out_h; a.OW = d->out_w; a.outLd = d->out_ld; a.C = d->in_c; a.pad = d->pad;
    a.strips = (d->out_w + 3) / 4;
    // 2 channels per lane: a quarter of the registers of 8 (78 instead of 192), four times the wavefronts in flight -- the kernel
    // is bound by load latency, not by the number of load instructions (measured over MobileNetV2's 17 layers at batch 64:
    // 447 us with 8, 287 us with 4, 237 us with 2)
    constexpr int CPL = 2;
    a.total = static_cast<long long>(d->batch) * d->out_h * a.strips * (d->in_c / CPL);
    a.xBytes = static_cast<unsigned>(((static_cast<unsigned long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld + d->in_c) * 2ull);
    a.act = d->act; a.actParam = d->act_param; a.outMul = d->out_mul;
    const int blocks = static_cast<int>(gridFor(a.total, 256));
    const dim3 grid((blocks + 7) / 8 * 8);
    // everything below 2^31: the 32-bit form (d->tile == 1 keeps the general one, for comparison)
    const unsigned long long yBytes = ((static_cast<unsigned long long>(d->batch) * d->out_h * d->out_w - 1) * d->out_ld + d->in_c) * 2ull;
    const unsigned long long wBytes = 9ull * d->in_c * 2ull;
    static const bool generalOnly = std::getenv("MSNH_DEPTHWISE_GENERAL") != nullptr;      // (for A/B timing of whole networks)
    if (d->tile != 1 && !generalOnly && a.total < 0x7fffff00ll && yBytes < 0x7fffffffull && wBytes < 0x7fffffffull)
    {
        DwFastArgs g;
        g.d = a;
        g.byCv = makeFastDiv(static_cast<unsigned>(d->in_c / CPL));
        g.byStrips = makeFastDiv(static_cast<unsigned>(a.strips));
        g.byOH = makeFastDiv(static_cast<unsigned>(d->out_h));
        g.wBytes = static_cast<unsigned>(wBytes);
        g.yBytes = static_cast<unsigned>(yBytes);
        if (d->stride == 1) hipLaunchKernelGGL((convDepthwise3x3FastKernel<1, 2>), grid, dim3(256), 0, st, g, blocks);
        else                hipLaunchKernelGGL((convDepthwise3x3FastKernel<2, 2>), grid, dim3(256), 0, st, g, blocks);
        MSNH_LAUNCH_CHECK();
        return 0;
    }
    if (d->stride == 1) hipLaunchKernelGGL((convDepthwise3x3Kernel<1, CPL>), grid, dim3(256), 0, st, a, blocks);
    else                hipLaunchKernelGGL((convDepthwise3x3Kernel<2, CPL>), grid, dim3(256), 0, st, a, blocks);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
