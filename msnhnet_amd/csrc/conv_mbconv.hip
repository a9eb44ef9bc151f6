// The inverted-residual block of MobileNetV2 as one launch, float16: a 1x1 convolution that widens in_c to exp_c channels, a 3x3
// depthwise convolution (stride 1 or 2, pad 1) over the widened tensor, a 1x1 convolution that narrows it to out_c channels, each with
// its folded batch-norm and activation, and the block's residual add.  As three launches the widened tensor (six times the block's
// input) is written and read twice; here it never leaves the compute unit.
//
// A workgroup of eight wavefronts owns 7 x 7 output pixels of one image.  The (6 s + 3)^2 input pixels under them sit in LDS for the
// whole launch.  The widened channels are walked in chunks of 64:
//   1. expand: [64 channels] x [input pixels] = W1 chunk . X on the matrix cores; affine, activation and the widened tensor's
//      power-of-two scale on the accumulators; pixels outside the image become zeros (they are the depthwise layer's padding); the
//      chunk goes to LDS as float16, pixel-major;
//   2. depthwise: a thread owns one 8-channel vector of one output pixel: nine LDS vectors, float32 sums; affine,
//      activation, scale; to LDS as float16, pixel-major -- the operand layout of the next step;
//   3. project: [out_c] x [49 pixels] += W3[:, chunk] . (depthwise output) on the matrix cores, accumulators kept over the chunks.
// Everything a chunk needs beside the activations -- both 1x1 filters in matrix-core fragment order (rows permuted so that a lane's 16
// accumulators are 16 consecutive channels), the depthwise taps, the two affines -- is one contiguous record of the packed weights,
// copied into LDS by 16-byte-per-lane loads that deliver straight into LDS while the chunk before it is computed.
#include "conv_igemm.hpp"

namespace msnh {

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int MB_TO  = 7;      // output tile edge
constexpr int MB_CH  = 64;     // widened channels per chunk
constexpr int MB_NW  = 8;      // wavefronts per workgroup
constexpr int MB_ROW = 144;    // bytes of a pixel's 64-channel float16 row in LDS: 128 + 16, an odd number of 16-byte units, so that
                               // 16 consecutive pixels read at one channel offset fall on 16 different bank groups

struct MbArgs
{
    const f16           *x;
    const unsigned char *blob;
    const float         *scale3;
    const float         *shift3;
    const f16           *res;
    f16                 *y;
    int N, H, W, cin, inLd, cexp, cout, outLd, OH, OW, resLd;
    int tilesX, tilesY, total;
    int ks;                 // 16-wide K steps of the expand GEMM: ceil(in_c / 16)
    int mb;                 // 32-row blocks of the project GEMM: ceil(out_c / 32)
    int chunks;
    unsigned chunkBytes;    // one chunk's record in the packed weights
    unsigned xBytes, blobBytes;
    int act1, act2, act3, act4, hasRes;
    float act1Param, act2Param, act3Param, act4Param, outMul, resMul;
    float mul1, mul2;       // the widened tensors' scales, 1 where the packed affine already carries them (mbFolds)
    float cap1, cap2;       // relu6 with a folded scale clamps at 6 * scale
};

// For these activations act(m x) = m act(x) for a positive m (relu6: with the clamp moved to 6 m), so the power-of-two scale of a widened tensor is
// multiplied into the stage's scale and shift at pack time -- exactly, it is a power of two -- and costs no instruction per element.
__host__ __device__ inline bool mbFolds(int act) { return act == MSNH_ACT_NONE || act == MSNH_ACT_RELU || act == MSNH_ACT_LEAKY || act == MSNH_ACT_RELU6; }

template <int N> __device__ __forceinline__ void mbActivate(float (&v)[N], int act, float param, float cap, float mul)
{
    if (act == MSNH_ACT_RELU6)
    {
        // one median instruction per element; a NaN gives 0 as in activate()
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] = __builtin_amdgcn_fmed3f(v[e], 0.f, cap);
        return;
    }
    activateArray<N>(v, act, param);
    if (mul != 1.f)
    {
#pragma unroll
        for (int e = 0; e < N; ++e) v[e] *= mul;
    }
}

__host__ __device__ constexpr int mbRowOfChannel(int c) { return 8 * ((c & 15) >> 2) + 4 * (c >> 4) + (c & 3); }

// offsets inside a chunk's record
__host__ __device__ inline unsigned mbWpOff(int ks) { return static_cast<unsigned>(2 * ks) * 1024u; }
__host__ __device__ inline unsigned mbWdOff(int ks, int mb) { return static_cast<unsigned>(2 * ks + 4 * mb) * 1024u; }
__host__ __device__ inline unsigned mbAffOff(int ks, int mb) { return mbWdOff(ks, mb) + 9u * MB_CH * 2u; }
__host__ __device__ inline unsigned mbChunkBytes(int ks, int mb) { return static_cast<unsigned>(2 * ks + 4 * mb + 3) * 1024u; }

template <int S>
__global__ __launch_bounds__(64 * MB_NW) void mbconvKernel(MbArgs a)
{
    constexpr int IT = (MB_TO - 1) * S + 3;           // input tile edge: 9 or 15
    constexpr int IP = IT * IT;
    constexpr int NE = (IP + 31) / 32;                // 32-pixel column blocks of the expand GEMM
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const unsigned ldsBase = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)smem));

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, n = lane & 31;

    // workgroups are dealt to the XCDs in contiguous runs, so that the input rows neighbouring tiles share meet in one L2
    const int perXcd  = (a.total + 7) / 8;
    const int logical = (blockIdx.x % 8) * perXcd + blockIdx.x / 8;
    if (logical >= a.total) return;
    const int tx  = logical % a.tilesX;
    const int ty  = (logical / a.tilesX) % a.tilesY;
    const int img = logical / (a.tilesX * a.tilesY);
    const int gy0 = ty * MB_TO * S - 1, gx0 = tx * MB_TO * S - 1;      // image coordinates of input tile pixel (0, 0)

    const unsigned xStr = static_cast<unsigned>(a.ks) * 32u + 16u;      // bytes of an input pixel's row in LDS
    const unsigned xOff = 0;
    const unsigned eOff = (xOff + NE * 32u * xStr + 1023u) & ~1023u;    // (the input tile's region ends on a 1 KiB boundary: it is filled in 1 KiB deliveries)
    const unsigned yOff = eOff + NE * 32u * MB_ROW;
    const unsigned bOff = (yOff + 64u * MB_ROW + 1023u) & ~1023u;

    const i32x4 rxw = makeRsrcWords(a.x, a.xBytes);
    const i32x4 rb = makeRsrcWords(a.blob, a.blobBytes);
    const int pieces = static_cast<int>(a.chunkBytes / 1024u);
    auto issueBlob = [&](int chunk, unsigned dst) {
        for (int p = wave; p < pieces; p += MB_NW)
            dmaLoad16(rb, static_cast<unsigned>(p) * 1024u + static_cast<unsigned>(lane) * 16u, static_cast<unsigned>(chunk) * a.chunkBytes,
                      ldsBase + dst + static_cast<unsigned>(p) * 1024u);
    };
    issueBlob(0, bOff);

    // ---- the input tile, zeros outside the image and past in_c: delivered straight into LDS, 1 KiB per wavefront and load; a pixel's row
    // is 2 ks + 1 slots of 16 bytes, the last one padding (an out-of-range offset delivers zeros) -------------------------------------
    {
        const int slots = 2 * a.ks + 1;
        const int xPieces = static_cast<int>((eOff - xOff) / 1024u);
        for (int p = wave; p < xPieces; p += MB_NW)
        {
            const int q = p * 64 + lane;
            const int px = q / slots, v = q - px * slots;
            const int iy = px / IT, ix = px - iy * IT;
            const int gy = gy0 + iy, gx = gx0 + ix;
            const bool ok = px < IP && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && v * 8 < a.cin && v < slots - 1;
            const unsigned voff = ok ? (static_cast<unsigned>((img * a.H + gy) * a.W + gx) * a.inLd + v * 8) * 2u : kOobOffset;
            dmaLoad16(rxw, voff, 0u, ldsBase + xOff + static_cast<unsigned>(p) * 1024u);
        }
        // the depthwise output starts as zeros: its pixel rows 49..63 are operand columns whose results nobody stores, and the channel
        // vectors past exp_c of a last, partial chunk are never written (their filter values are zeros, but 0 * garbage may be a NaN)
        for (int idx = tid; idx < 64 * MB_ROW / 16; idx += 64 * MB_NW)
            *reinterpret_cast<f32x4 *>(smem + yOff + idx * 16) = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // this lane's pixel of every expand column block: inside the image?
    unsigned inImage = 0;
#pragma unroll
    for (int j = 0; j < NE; ++j)
    {
        const int px = 32 * j + n;
        const int iy = px / IT, ix = px - iy * IT;
        const int gy = gy0 + iy, gx = gx0 + ix;
        if (px < IP && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W) inImage |= 1u << j;
    }

    f32x16 accP;                                      // project: wavefront w owns block w / 2 of the output channels x column block w % 2
#pragma unroll
    for (int e = 0; e < 16; ++e) accP[e] = 0.f;

    dmaWait<0>();
    __syncthreads();

    // Per chunk of 64 widened channels: expand (matrix cores, all wavefronts) | barrier | depthwise (vector ALU) | barrier | project (matrix
    // cores, the first 2 mb wavefronts) together with the expand of the NEXT chunk, which touches neither the depthwise output the projection
    // reads nor anything the projection writes: two workgroup barriers per chunk, and the wavefronts without a projection block start the next
    // expand at once (its items are dealt from the last wavefront down).  The record of chunk c + 1 is asked for behind the first barrier of
    // chunk c -- its buffer held chunk c - 1, whose last reader, the projection, every wavefront has left by then -- and is complete at the
    // second one.
    const auto expandChunk = [&](int c) {
        const unsigned char *rec = smem + bOff + static_cast<unsigned>(c & 1) * a.chunkBytes;
        const float *aff = reinterpret_cast<const float *>(rec + mbAffOff(a.ks, a.mb));
        const int left = a.cexp - c * MB_CH;          // widened channels from this chunk on: a last chunk may be partial
        // ---- 1. expand (a 32-channel block past exp_c is skipped) ---------------------------------------------------------------------
        const int nmb = left > 32 ? 2 : 1;
        for (int it = MB_NW - 1 - wave; it < nmb * NE; it += MB_NW)
        {
            const int mblk = nmb == 2 ? (it & 1) : 0, j = nmb == 2 ? (it >> 1) : it;
            f32x16 acc;
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[e] = 0.f;
            const unsigned char *ap = rec + (mblk * a.ks) * 1024 + lane * 16;
            const unsigned char *bp = smem + xOff + (32 * j + n) * xStr + h * 16;
            for (int s = 0; s < a.ks; ++s)
                mfmaBlock(*reinterpret_cast<const f16x8 *>(ap + s * 1024), *reinterpret_cast<const f16x8 *>(bp + s * 32), acc);
            const int c0 = 32 * mblk + 16 * h;
            float v[16];
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const f32x4 sc = *reinterpret_cast<const f32x4 *>(aff + c0 + 4 * q);
                const f32x4 sh = *reinterpret_cast<const f32x4 *>(aff + MB_CH + c0 + 4 * q);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[4 * q + e] = acc[4 * q + e] * sc[e] + sh[e];
            }
            mbActivate<16>(v, a.act1, a.act1Param, a.cap1, a.mul1);
            // (a pixel outside the image is exactly zero, also where the activation of the shift is not: masked as bits)
            const unsigned keep = ((inImage >> j) & 1u) ? 0xffffffffu : 0u;
            f16x8 o0, o1;
#pragma unroll
            for (int e = 0; e < 8; ++e)
            {
                o0[e] = static_cast<f16>(v[e]);
                o1[e] = static_cast<f16>(v[8 + e]);
            }
            u32x4 b0 = __builtin_bit_cast(u32x4, o0), b1 = __builtin_bit_cast(u32x4, o1);
#pragma unroll
            for (int e = 0; e < 4; ++e) { b0[e] &= keep; b1[e] &= keep; }
            o0 = __builtin_bit_cast(f16x8, b0);
            o1 = __builtin_bit_cast(f16x8, b1);
            unsigned char *ep = smem + eOff + (32 * j + n) * MB_ROW + c0 * 2;
            *reinterpret_cast<f16x8 *>(ep) = o0;
            *reinterpret_cast<f16x8 *>(ep + 16) = o1;
        }
    };
    expandChunk(0);
    for (int c = 0; c < a.chunks; ++c)
    {
        const unsigned cur = bOff + static_cast<unsigned>(c & 1) * a.chunkBytes;
        const unsigned char *rec = smem + cur;
        const float *aff = reinterpret_cast<const float *>(rec + mbAffOff(a.ks, a.mb));
        const int left = a.cexp - c * MB_CH;
        __syncthreads();
        if (c + 1 < a.chunks) issueBlob(c + 1, bOff + static_cast<unsigned>((c + 1) & 1) * a.chunkBytes);

        // ---- 2. depthwise (the threads share out the channel vectors that exist) ---------------------------------------------------------
        {
            const int nv = left >= MB_CH ? 8 : (left + 7) / 8;
            int p = tid >> 3, v8 = tid & 7;
            if (nv != 8) { p = tid / nv; v8 = tid - p * nv; }
            if (p < MB_TO * MB_TO)
            {
                const unsigned char *wd = rec + mbWdOff(a.ks, a.mb) + v8 * 16;
                const int oy = p / MB_TO, ox = p - oy * MB_TO;
                const unsigned char *ep = smem + eOff + ((oy * S) * IT + ox * S) * MB_ROW + v8 * 16;
                float sum[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) sum[e] = 0.f;
#pragma unroll
                for (int t = 0; t < 9; ++t)
                {
                    const f16x8 xv = *reinterpret_cast<const f16x8 *>(ep + ((t / 3) * IT + t % 3) * MB_ROW);
                    const f16x8 wv = *reinterpret_cast<const f16x8 *>(wd + t * (MB_CH * 2));
#pragma unroll
                    for (int e = 0; e < 8; ++e) sum[e] += static_cast<float>(xv[e]) * static_cast<float>(wv[e]);
                }
                const f32x4 s0 = *reinterpret_cast<const f32x4 *>(aff + 2 * MB_CH + 8 * v8), s1 = *reinterpret_cast<const f32x4 *>(aff + 2 * MB_CH + 8 * v8 + 4);
                const f32x4 h0 = *reinterpret_cast<const f32x4 *>(aff + 3 * MB_CH + 8 * v8), h1 = *reinterpret_cast<const f32x4 *>(aff + 3 * MB_CH + 8 * v8 + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    sum[e]     = sum[e] * s0[e] + h0[e];
                    sum[4 + e] = sum[4 + e] * s1[e] + h1[e];
                }
                mbActivate<8>(sum, a.act2, a.act2Param, a.cap2, a.mul2);
                f16x8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = static_cast<f16>(sum[e]);
                *reinterpret_cast<f16x8 *>(smem + yOff + p * MB_ROW + v8 * 16) = o;
            }
        }
        dmaWait<0>();
        __syncthreads();

        // ---- 3. project --------------------------------------------------------------------------------------------------------
        if (wave < 2 * a.mb)
        {
            const int mblk = wave >> 1, j = wave & 1;
            const unsigned char *ap = rec + mbWpOff(a.ks) + (mblk * 4) * 1024 + lane * 16;
            const unsigned char *bp = smem + yOff + (32 * j + n) * MB_ROW + h * 16;
#pragma unroll
            for (int s = 0; s < MB_CH / 16; ++s)
                mfmaBlock(*reinterpret_cast<const f16x8 *>(ap + s * 1024), *reinterpret_cast<const f16x8 *>(bp + s * 32), accP);
        }
        if (c + 1 < a.chunks) expandChunk(c + 1);
    }

    // ---- epilogue: affine, activation, residual, second activation, scale; two 16-byte stores per lane ------------------------------
    if (wave < 2 * a.mb)
    {
        const int mblk = wave >> 1, j = wave & 1;
        const int p = 32 * j + n;
        const int oy = ty * MB_TO + p / MB_TO, ox = tx * MB_TO + p % MB_TO;
        if (p < MB_TO * MB_TO && oy < a.OH && ox < a.OW)
        {
            const size_t pix = static_cast<size_t>(img * a.OH + oy) * a.OW + ox;
#pragma unroll
            for (int g = 0; g < 2; ++g)
            {
                const int c0 = 32 * mblk + 16 * h + 8 * g;
                if (c0 >= a.cout) continue;
                float v[8];
                const f32x4 one = {1.f, 1.f, 1.f, 1.f}, zero = {0.f, 0.f, 0.f, 0.f};
                const f32x4 s0 = a.scale3 ? *reinterpret_cast<const f32x4 *>(a.scale3 + c0) : one, s1 = a.scale3 ? *reinterpret_cast<const f32x4 *>(a.scale3 + c0 + 4) : one;
                const f32x4 h0 = a.shift3 ? *reinterpret_cast<const f32x4 *>(a.shift3 + c0) : zero, h1 = a.shift3 ? *reinterpret_cast<const f32x4 *>(a.shift3 + c0 + 4) : zero;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    v[e]     = accP[8 * g + e] * s0[e] + h0[e];
                    v[4 + e] = accP[8 * g + 4 + e] * s1[e] + h1[e];
                }
                activateArray<8>(v, a.act3, a.act3Param);
                if (a.hasRes)
                {
                    const f16x8 r = *reinterpret_cast<const f16x8 *>(a.res + pix * a.resLd + c0);
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += a.resMul * static_cast<float>(r[e]);
                    activateArray<8>(v, a.act4, a.act4Param);
                }
                f16x8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = static_cast<f16>(a.outMul * v[e]);
                *reinterpret_cast<f16x8 *>(a.y + pix * a.outLd + c0) = o;
            }
        }
    }
}

size_t mbLdsBytes(const msnh_mbconv_desc *d)
{
    const int ks = (d->in_c + 15) / 16, mb = (d->out_c + 31) / 32;
    const int it = (MB_TO - 1) * d->stride + 3;
    const size_t ne = static_cast<size_t>((it * it + 31) / 32);
    const size_t xRegion = (ne * 32 * (static_cast<size_t>(ks) * 32 + 16) + 1023) & ~static_cast<size_t>(1023);
    const size_t acts = xRegion + ne * 32 * MB_ROW + 64 * MB_ROW;
    return ((acts + 1023) & ~static_cast<size_t>(1023)) + 2 * static_cast<size_t>(mbChunkBytes(ks, mb));
}

} // namespace

} // namespace msnh

using namespace msnh;

extern "C" {

int msnh_hip_mbconv_supported(const msnh_mbconv_desc *d)
{
    if (!d) return 0;
    const bool geometry = d->batch > 0 && d->in_h > 0 && d->in_w > 0 && (d->stride == 1 || d->stride == 2) &&
                          d->out_h == (d->in_h - 1) / d->stride + 1 && d->out_w == (d->in_w - 1) / d->stride + 1;
    const bool channels = d->in_c % 8 == 0 && d->in_c >= 8 && d->in_c <= 96 && d->exp_c % 8 == 0 && d->exp_c >= 8 && d->exp_c <= 4096 &&
                          d->out_c % 8 == 0 && d->out_c >= 8 && d->out_c <= 96 && d->in_ld % 8 == 0 && d->in_ld >= d->in_c &&
                          d->out_ld % 8 == 0 && d->out_ld >= d->out_c && (!d->has_residual || (d->res_ld % 8 == 0 && d->res_ld >= d->out_c));
    if (!geometry || !channels) return 0;
    if (!actOk(d->act1) || !actOk(d->act2) || !actOk(d->act3) || !actOk(d->act4)) return 0;
    const unsigned long long xb = (static_cast<unsigned long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld * 2ull + d->in_c * 2ull;
    if (xb >= 0x7fffffffull) return 0;
    return mbLdsBytes(d) <= 160 * 1024 ? 1 : 0;
}

size_t msnh_hip_mbconv_packed_bytes(const msnh_mbconv_desc *d)
{
    if (!msnh_hip_mbconv_supported(d)) return 0;
    const int ks = (d->in_c + 15) / 16, mb = (d->out_c + 31) / 32;
    return static_cast<size_t>((d->exp_c + MB_CH - 1) / MB_CH) * mbChunkBytes(ks, mb);
}

int msnh_hip_mbconv_pack(const msnh_mbconv_desc *d, const float *w_expand, const float *scale1, const float *shift1, const float *w_dw,
                         const float *scale2, const float *shift2, const float *w_project, void *packed)
{
    MSNH_REQUIRE(msnh_hip_mbconv_supported(d), "mbconv: block not supported (channels, stride or sizes)");
    MSNH_REQUIRE(w_expand && w_dw && w_project && packed, "mbconv pack: null pointer");
    const int ks = (d->in_c + 15) / 16, mb = (d->out_c + 31) / 32;
    const int chunks = (d->exp_c + MB_CH - 1) / MB_CH;
    const unsigned cb = mbChunkBytes(ks, mb);
    unsigned char *out = static_cast<unsigned char *>(packed);
    std::memset(out, 0, static_cast<size_t>(chunks) * cb);
    const auto half = [](float v) { return static_cast<f16>(v); };
    for (int c = 0; c < chunks; ++c)
    {
        unsigned char *rec = out + static_cast<size_t>(c) * cb;
        f16 *we = reinterpret_cast<f16 *>(rec);
        f16 *wp = reinterpret_cast<f16 *>(rec + mbWpOff(ks));
        f16 *wd = reinterpret_cast<f16 *>(rec + mbWdOff(ks, mb));
        float *aff = reinterpret_cast<float *>(rec + mbAffOff(ks, mb));
        for (int ch = 0; ch < MB_CH; ++ch)
        {
            const int ce = c * MB_CH + ch;
            if (ce >= d->exp_c) continue;
            // expand filter row ce -> block ch / 32, fragment row mbRowOfChannel(ch % 32); K value k sits in K step k / 16, half (k / 8) % 2
            const int mblk = ch / 32, row = mbRowOfChannel(ch % 32);
            for (int k = 0; k < d->in_c; ++k)
            {
                const int lane = row + 32 * ((k >> 3) & 1);
                we[(static_cast<size_t>(mblk * ks + (k >> 4)) * 64 + lane) * 8 + (k & 7)] = half(w_expand[static_cast<size_t>(ce) * d->in_c + k]);
            }
            for (int t = 0; t < 9; ++t) wd[t * MB_CH + ch] = half(w_dw[static_cast<size_t>(ce) * 9 + t]);
            const float m1 = mbFolds(d->act1) ? d->mul1 : 1.f, m2 = mbFolds(d->act2) ? d->mul2 : 1.f;
            aff[ch]             = m1 * (scale1 ? scale1[ce] : 1.f);
            aff[MB_CH + ch]     = m1 * (shift1 ? shift1[ce] : 0.f);
            aff[2 * MB_CH + ch] = m2 * (scale2 ? scale2[ce] : 1.f);
            aff[3 * MB_CH + ch] = m2 * (shift2 ? shift2[ce] : 0.f);
            // project filter column ce: K value ch of this chunk
            for (int co = 0; co < d->out_c; ++co)
            {
                const int lane = mbRowOfChannel(co % 32) + 32 * ((ch >> 3) & 1);
                wp[(static_cast<size_t>((co / 32) * 4 + (ch >> 4)) * 64 + lane) * 8 + (ch & 7)] = half(w_project[static_cast<size_t>(co) * d->exp_c + ce]);
            }
        }
    }
    return 0;
}

int msnh_hip_mbconv(const msnh_mbconv_desc *d, const void *x, const void *packed, const float *scale3, const float *shift3, const void *residual,
                    void *y, msnh_stream_t s)
{
    MSNH_REQUIRE(msnh_hip_mbconv_supported(d), "mbconv: block not supported (channels, stride or sizes)");
    MSNH_REQUIRE(x && packed && y && (!d->has_residual || residual), "mbconv: null pointer");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(packed) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                 (!d->has_residual || reinterpret_cast<uintptr_t>(residual) % 16 == 0), "mbconv: tensors must be 16-byte aligned");
    MbArgs a;
    a.x = static_cast<const f16 *>(x); a.blob = static_cast<const unsigned char *>(packed); a.scale3 = scale3; a.shift3 = shift3;
    a.res = static_cast<const f16 *>(residual); a.y = static_cast<f16 *>(y);
    a.N = d->batch; a.H = d->in_h; a.W = d->in_w; a.cin = d->in_c; a.inLd = d->in_ld; a.cexp = d->exp_c; a.cout = d->out_c; a.outLd = d->out_ld;
    a.OH = d->out_h; a.OW = d->out_w; a.resLd = d->res_ld;
    a.tilesX = (d->out_w + MB_TO - 1) / MB_TO; a.tilesY = (d->out_h + MB_TO - 1) / MB_TO;
    const long long total = static_cast<long long>(a.tilesX) * a.tilesY * d->batch;
    MSNH_REQUIRE(total < (1ll << 30), "mbconv: too many tiles");
    a.total = static_cast<int>(total);
    a.ks = (d->in_c + 15) / 16; a.mb = (d->out_c + 31) / 32; a.chunks = (d->exp_c + MB_CH - 1) / MB_CH;
    a.chunkBytes = mbChunkBytes(a.ks, a.mb);
    a.xBytes = static_cast<unsigned>((static_cast<unsigned long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld * 2ull + d->in_c * 2ull);
    a.blobBytes = static_cast<unsigned>(static_cast<size_t>(a.chunks) * a.chunkBytes);
    a.act1 = d->act1; a.act2 = d->act2; a.act3 = d->act3; a.act4 = d->act4; a.hasRes = d->has_residual ? 1 : 0;
    a.act1Param = d->act1_param; a.act2Param = d->act2_param; a.act3Param = d->act3_param; a.act4Param = d->act4_param;
    a.outMul = d->out_mul; a.resMul = d->res_mul;
    a.mul1 = mbFolds(d->act1) ? 1.f : d->mul1; a.mul2 = mbFolds(d->act2) ? 1.f : d->mul2;
    a.cap1 = 6.f * d->mul1; a.cap2 = 6.f * d->mul2;
    const size_t lds = mbLdsBytes(d);
    const unsigned blocks = static_cast<unsigned>((total + 7) / 8 * 8);
    hipStream_t st = resolveStream(s);
    if (d->stride == 1)
    {
        static bool raised = false;
        if (!raised) { MSNH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(mbconvKernel<1>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); raised = true; }
        hipLaunchKernelGGL((mbconvKernel<1>), dim3(blocks), dim3(64 * MB_NW), lds, st, a);
    }
    else
    {
        static bool raised = false;
        if (!raised) { MSNH_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(mbconvKernel<2>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); raised = true; }
        hipLaunchKernelGGL((mbconvKernel<2>), dim3(blocks), dim3(64 * MB_NW), lds, st, a);
    }
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // extern "C"
