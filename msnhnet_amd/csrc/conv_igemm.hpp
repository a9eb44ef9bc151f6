// Implicit-GEMM convolution on the gfx950 matrix cores.
//
// GEMM view per group:  D[m][p] = sum_k W[m][k] * X[k][p]
//     m = output channel (rows, operand A = packed weights [out_c][tap][cin_g], K contiguous)
//     p = output pixel over the whole batch, p = (b*OH + oy)*OW + ox (columns, operand B)
//     k = (tap, channel); the B operand is gathered on the fly from the NHWC input: for one tap the
//         cin_g channels of an input pixel are contiguous, so a 16-byte vector load per lane feeds the
//         MFMA operand registers without any transposition.
// A workgroup of 256, 512 or 768 threads (4, 8 or 12 wavefronts in a WM x WN grid) owns a BM x BN tile of D.  Per K step every
// wavefront issues 16-byte-per-lane buffer loads that deliver straight into LDS (no registers, no LDS store
// instructions); three LDS stages rotate so that the loads run two steps ahead of the MFMAs, with one barrier
// per step.  LDS rows are unpadded and XOR-swizzled so that both the 1 KiB deliveries and the 128-bit fragment
// reads are bank-conflict free.  Lanes outside the image, the channel range or the tensor carry an out-of-range
// offset and the hardware fills zeros.
// The epilogue applies folded batch-norm / bias, activation, residual add + second activation and the
// power-of-two output scale on the float32 accumulators and stores 8 consecutive channels per lane.
#pragma once
#include "common.hpp"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace msnh {

struct IgemmArgs
{
    const void  *x;
    const void  *w;
    const float *scale;
    const float *shift;
    const void  *res;
    void        *y;
    int batch, H, W, inLd;
    int OH, OW, outLd, resLd;
    int cinG, coutG, taps, ksize, stride, pad, dil;
    int P;                  // batch*OH*OW
    int cChunks;            // ceil(cinG / BK)
    int nIter;              // taps * cChunks
    int mTiles;             // ceil(coutG / BM)
    int patchRows;          // patch kernel: input pixels staged per tile = BN + 2*W + 2
    int patchOk;            // geometry is 3x3 stride 1 pad 1 dilation 1, ungrouped, same-size output
    int dryRun;             // validate the tile for this shape, launch nothing
    unsigned xBytes, wBytes; // extent of the input tensor / packed weights in bytes (buffer resources; < 2 GiB)
    int ragged;             // cinG is not a multiple of the tile's K step
    int splitMax;           // > 1: split-K requested, at most this many slices of the K loop (grid y)
    int splitK;             // slices actually used by the launch
    float *ws;              // split-K: float32 partial sums [slice][pixel][out_c]
    int wsLd;               // = out_c of the whole convolution
    int buffersOk;          // both extents fit a buffer resource
    int act, act2, hasRes, vecOk;
    float actParam, act2Param, resMul, outMul;
    FastDiv byOW, byOH;     // pixel index -> (image, row, column) without hardware-less integer division
    int xcdGm;              // > 1: the XCDs form an xcdGm x (8 / xcdGm) grid over (channel tiles, pixel tiles), see igemmTileOf
    int xcdMPer, xcdPPer;   // channel tiles / pixel tiles per XCD in that arrangement
    int up2;                // every result pixel goes to the 2 x 2 pixels of y it maps to under nearest-neighbour upsampling (y: [batch][2 OH][2 OW])
    unsigned yBytes;        // up2: extent of y in bytes
    // tail (tiles with TAIL = 1 only): a 1x1 stride-1 convolution z = zMul * act3(scale2 * (W2 . y) + shift2) of this convolution's
    // float16 result y, computed by the same workgroup from the copy of its y tile in LDS
    int tailOn;             // the launch carries a tail (set by the tail entry point, also for dry runs)
    const void  *w2;        // [cout2][coutG] float16, K contiguous
    const float *scale2, *shift2;
    void        *z;         // NHWC float16 with pixel stride zLd
    int cout2, zLd, act3, writeY;
    float act3Param, zMul;
    unsigned w2Bytes;
};

// Workgroup -> tile.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: id % 8 selects
// the XCD, id / 8 the position inside it.  Default arrangement (xcdGm <= 1): an XCD takes a contiguous run of tiles with the
// channel tiles of one pixel tile back to back, so an input pixel is fetched into one L2 once instead of once per channel
// tile and XCD -- and every XCD fetches every filter.  Where the filters outweigh the input (512 -> 1024 channels over
// 19 x 19 pixels: 9.4 MB against 3 MB) the host asks for an xcdGm x (8 / xcdGm) arrangement instead: an XCD owns a block of
// channel tiles and a block of pixel tiles and fetches only that share of the filters and that share of the input.
__device__ __forceinline__ bool igemmTileOf(const IgemmArgs &a, int nTilesP, int &mTile, int &pTile)
{
    const int xcd = blockIdx.x % 8, idx = blockIdx.x / 8;
    if (a.xcdGm <= 1)
    {
        const int total   = a.mTiles * nTilesP;
        const int perXcd  = (total + 7) / 8;
        const int logical = xcd * perXcd + idx;
        mTile = logical % a.mTiles;
        pTile = logical / a.mTiles;
        return logical < total;                       // padding ids of the last round
    }
    const int lp = idx / a.xcdMPer;
    mTile = (xcd % a.xcdGm) * a.xcdMPer + (idx - lp * a.xcdMPer);
    pTile = (xcd / a.xcdGm) * a.xcdPPer + lp;
    return lp < a.xcdPPer && mTile < a.mTiles && pTile < nTilesP;
}

// grid.x of a launch over a.mTiles x nTilesP tiles, and the XCD arrangement it runs under (see igemmTileOf).  a.xcdGm comes in as
// the caller's wish (msnh_conv_desc::xcd_blocks): 1, 2, 4, 8 are taken as they are; 0 picks the arrangement that makes the eight
// L2s fetch the fewest bytes, counted as (8 / g) x filters + g x input -- the default one stays unless another saves a quarter
// of that without more workgroup slots per XCD.  Grouped and split-K launches (plainGrid false) keep the default.
inline unsigned igemmGridX(IgemmArgs &a, int nTilesP, size_t es, bool plainGrid)
{
    static const bool off = std::getenv("MSNH_NO_XCD_BLOCKS") != nullptr;      // (for A/B timing of whole networks)
    const int wish = a.xcdGm;
    const int tiles = a.mTiles * nTilesP;
    const unsigned plain = static_cast<unsigned>((tiles + 7) / 8 * 8);
    a.xcdGm = 1; a.xcdMPer = a.mTiles; a.xcdPPer = nTilesP;
    if (!plainGrid || wish == 1 || (wish == 0 && off)) return plain;
    const double wB = static_cast<double>(a.coutG) * a.taps * a.cinG * es;
    const double xB = static_cast<double>(a.batch) * a.H * a.W * a.cinG * es;
    double best = 8 * wB + xB;
    const double need = 0.75 * best;
    unsigned grid = plain;
    for (int gm = 2; gm <= 8; gm *= 2)
    {
        const int gp = 8 / gm, mPer = (a.mTiles + gm - 1) / gm, pPer = (nTilesP + gp - 1) / gp;
        const double cost = gp * wB + gm * xB;
        const bool take = wish == gm || (wish == 0 && 8 * mPer * pPer <= static_cast<int>(plain) && cost < need && cost < best);
        if (take) { best = cost; a.xcdGm = gm; a.xcdMPer = mPer; a.xcdPPer = pPer; grid = 8u * mPer * pPer; }
    }
    return grid;
}

template <typename T> struct Frag;
template <> struct Frag<f16>   { typedef f16x8 V; static constexpr int VEC = 8; };
template <> struct Frag<float> { typedef f32x4 V; static constexpr int VEC = 4; };

// One "k-block": the 2 x 16 bytes of K that the two half-waves hold for a 32-row operand block.
__device__ __forceinline__ void mfmaBlock(const f16x8 &a, const f16x8 &b, f32x16 &c)
{
    c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void mfmaBlock(const f32x4 &a, const f32x4 &b, f32x16 &c)
{
    // lanes 0-31 carry k = 0..3, lanes 32-63 carry k = 4..7 of the block; A and B agree, so the four
    // 32x32x2 steps pair (j, 4+j) and together cover all eight k.
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], c, 0, 0, 0);
}

// 16-byte load through a buffer resource: the address is base + voffset + soffset with a hardware range check of
// voffset against the resource size, so a lane whose row, tap or channel falls outside the tensor simply carries an
// out-of-range voffset and reads zeros -- no branches, no 64-bit address arithmetic in the loop.
typedef int i32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned kOobOffset = 0x80000000u;      // beyond any resource this kernel accepts (sizes are < 2 GiB)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t makeRsrc(const void *base, unsigned bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, static_cast<int>(bytes), 0x00020000);
}

template <typename V> __device__ __forceinline__ V bufferLoad16(__amdgpu_buffer_rsrc_t r, unsigned voffset, unsigned soffset)
{
    const i32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(voffset), static_cast<int>(soffset), 0);
    return __builtin_bit_cast(V, v);
}

// Shared epilogue of the GEMM-shaped convolution kernels.  Nothing in it waits on a global load issued inside it
// except the residual, and that one is issued a whole staging pass ahead:
// 1. the per-channel affine (folded batch-norm / bias) was fetched before the main loop, one channel per thread,
//    and is now spread through LDS;
// 2. per 32-pixel column block the wavefront applies affine + activation on its float32 accumulators and stages
//    them pixel-major in LDS (the main loop's LDS is free after its last barrier), so that
// 3. every lane then owns 8 consecutive channels of a pixel: 16-byte residual loads and output stores through
//    range-checked buffer resources (pixels past the end of the tensor are dropped by the hardware), the lanes of
//    a pixel covering a contiguous run of channels.
template <typename T> struct Raw8;               // 8 consecutive elements as loaded / stored
template <> struct Raw8<f16>
{
    i32x4 r[1];
    __device__ __forceinline__ void toFloat(float (&v)[8]) const
    {
        const f16x8 h = __builtin_bit_cast(f16x8, r[0]);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = static_cast<float>(h[e]);
    }
    __device__ __forceinline__ void fromFloat(const float (&v)[8])
    {
        f16x8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = static_cast<f16>(v[e]);
        r[0] = __builtin_bit_cast(i32x4, h);
    }
};
template <> struct Raw8<float>
{
    i32x4 r[2];
    __device__ __forceinline__ void toFloat(float (&v)[8]) const
    {
        const f32x4 lo = __builtin_bit_cast(f32x4, r[0]), hi = __builtin_bit_cast(f32x4, r[1]);
#pragma unroll
        for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
    }
    __device__ __forceinline__ void fromFloat(const float (&v)[8])
    {
        f32x4 lo, hi;
#pragma unroll
        for (int e = 0; e < 4; ++e) { lo[e] = v[e]; hi[e] = v[4 + e]; }
        r[0] = __builtin_bit_cast(i32x4, lo);
        r[1] = __builtin_bit_cast(i32x4, hi);
    }
};

template <typename T> __device__ __forceinline__ Raw8<T> bufferLoad8(__amdgpu_buffer_rsrc_t rs, unsigned voffset)
{
    Raw8<T> o;
#pragma unroll
    for (int h = 0; h < static_cast<int>(sizeof(T)) / 2; ++h)
        o.r[h] = __builtin_amdgcn_raw_buffer_load_b128(rs, static_cast<int>(voffset + 16 * h), 0, 0);
    return o;
}

template <typename T> __device__ __forceinline__ void bufferStore8(const Raw8<T> &o, __amdgpu_buffer_rsrc_t rs, unsigned voffset)
{
#pragma unroll
    for (int h = 0; h < static_cast<int>(sizeof(T)) / 2; ++h)
        __builtin_amdgcn_raw_buffer_store_b128(o.r[h], rs, static_cast<int>(voffset + 16 * h), 0, 0);
}

// The affine of channel m0 + tid of group g, fetched by thread tid ahead of the main loop.
__device__ __forceinline__ void loadChannelAffine(const IgemmArgs &a, int g, int m0, int tid, int bm, float &sc, float &sh)
{
    sc = 1.f;
    sh = 0.f;
    const int m = m0 + tid;
    if (tid < bm && m < a.coutG)
    {
        if (a.scale) sc = a.scale[g * a.coutG + m];
        if (a.shift) sh = a.shift[g * a.coutG + m];
    }
}

// relu, leaky and identity are x > 0 ? x : slope * x with slope 0, param, 1
__device__ __forceinline__ bool actIsSlope(int act, float param, float &slope)
{
    slope = act == MSNH_ACT_LEAKY ? param : (act == MSNH_ACT_RELU ? 0.f : 1.f);
    return act == MSNH_ACT_LEAKY || act == MSNH_ACT_RELU || act == MSNH_ACT_NONE;
}

template <bool SLOPE> __device__ __forceinline__ float activateSel(float x, float slope, int act, float param)
{
    if (SLOPE) return x > 0.f ? x : slope * x;
    return activate(x, act, param);
}

// Loop whose index is a compile-time constant in the body (accumulator arrays must never be indexed dynamically,
// or they are demoted from registers to scratch memory).
template <int I, int N, typename F> __device__ __forceinline__ void staticFor(F &&f)
{
    if constexpr (I < N)
    {
        f(std::integral_constant<int, I>());
        staticFor<I + 1, N>(f);
    }
}

template <int BM, int TM, int NW = 4> constexpr size_t igemmEpilogueLds() { return (2 * BM + NW * 32 * (TM + 4)) * sizeof(float); }

// ssReady / stageOwn (the K-split epilogue): the affines already stand at ssReady, published by a barrier the caller has passed, and this
// wavefront stages in stageOwn (32 x (TM + 4) floats of its own) -- then the epilogue meets no workgroup barrier at all.
template <typename T, typename TOut, int BM, int BN, int TM, int TN>
__device__ __forceinline__ void igemmEpilogue(const IgemmArgs &a, f32x16 (&acc)[TM / 32][TN / 32], unsigned char *smemRaw, float chScale,
                                              float chShift, int m0, int p0, int wm, int wn, int wave, int lane, int g,
                                              float *ssReady = nullptr, float *stageOwn = nullptr)
{
    constexpr int MB  = TM / 32;
    constexpr int NB  = TN / 32;
    constexpr int LDE = TM + 4;                       // padded staging row (floats)
    constexpr int VPR = TM / 8;                       // lanes (8-channel vectors) per staged pixel
    constexpr int RPI = 64 / VPR;                     // pixels covered per pass of the wave
    constexpr int PASSES = 32 / RPI;
    static_assert(BM <= 256 && VPR <= 32, "epilogue geometry");
    float *ss    = ssReady ? ssReady : reinterpret_cast<float *>(smemRaw);                 // [BM] scale, [BM] shift
    float *stage = stageOwn ? stageOwn : ss + 2 * BM + wave * (32 * LDE);
    const int tid = wave * 64 + lane;
    if (!ssReady)
    {
        if (tid < BM) { ss[tid] = chScale; ss[BM + tid] = chShift; }
        __syncthreads();
    }

    const int chBase = g * a.coutG;
    const int vcol = (lane % VPR) * 8;
    const int mv   = m0 + wm * TM + vcol;             // first channel of this lane's vector (within the group)
    const bool chOk = mv < a.coutG;
    const bool full = a.vecOk && (mv + 7 < a.coutG);
    const unsigned ch = static_cast<unsigned>(chBase + mv);
    const int npix = min(a.P - p0, BN);
    TOut    *yBlock = static_cast<TOut *>(a.y) + static_cast<size_t>(p0) * a.outLd;
    const T *rBlock = static_cast<const T *>(a.res) + static_cast<size_t>(p0) * a.resLd;
    const __amdgpu_buffer_rsrc_t ry = a.up2 ? makeRsrc(a.y, a.yBytes) : makeRsrc(yBlock, static_cast<unsigned>(npix) * a.outLd * sizeof(TOut));
    const __amdgpu_buffer_rsrc_t rr = makeRsrc(a.hasRes ? rBlock : nullptr, a.hasRes ? static_cast<unsigned>(npix) * a.resLd * sizeof(T) : 0u);
    float slope1, slope2;
    const bool lin1 = actIsSlope(a.act, a.actParam, slope1);
    const bool lin2 = actIsSlope(a.act2, a.act2Param, slope2);

    staticFor<0, NB>([&](auto jTag) {
        constexpr int j = decltype(jTag)::value;
        const int pixBase = wn * TN + j * 32;         // first pixel of this column block inside the tile
        Raw8<T> resRaw[PASSES];
        if (a.hasRes)
        {
#pragma unroll
            for (int t = 0; t < PASSES; ++t)
            {
                const unsigned pl = pixBase + t * RPI + lane / VPR;
                resRaw[t] = bufferLoad8<T>(rr, full ? (pl * a.resLd + ch) * static_cast<unsigned>(sizeof(T)) : kOobOffset);
            }
        }
        auto stageBlock = [&](auto slopeTag) {
            constexpr bool SL = decltype(slopeTag)::value;
            if constexpr (SL)
            {
                staticFor<0, MB * 4>([&](auto iqTag) {
                        constexpr int i = decltype(iqTag)::value / 4;
                        constexpr int q = decltype(iqTag)::value % 4;
                        const int ml = i * 32 + q * 8 + (lane >> 5) * 4;       // channel inside the wave tile
                        const f32x4 sc = *reinterpret_cast<const f32x4 *>(ss + wm * TM + ml);
                        const f32x4 sh = *reinterpret_cast<const f32x4 *>(ss + BM + wm * TM + ml);
                        f32x4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = activateSel<true>(acc[i][j][q * 4 + e] * sc[e] + sh[e], slope1, a.act, a.actParam);
                        *reinterpret_cast<f32x4 *>(stage + (lane & 31) * LDE + ml) = v;
                });
            }
            else
            {
                // transcendental activations: affine on every accumulator first, then ONE choice of the activation for all of them
                float t[MB * 16];
                staticFor<0, MB * 4>([&](auto iqTag) {
                        constexpr int iq = decltype(iqTag)::value;
                        constexpr int i = iq / 4, q = iq % 4;
                        const int ml = i * 32 + q * 8 + (lane >> 5) * 4;
                        const f32x4 sc = *reinterpret_cast<const f32x4 *>(ss + wm * TM + ml);
                        const f32x4 sh = *reinterpret_cast<const f32x4 *>(ss + BM + wm * TM + ml);
#pragma unroll
                        for (int e = 0; e < 4; ++e) t[iq * 4 + e] = acc[i][j][q * 4 + e] * sc[e] + sh[e];
                });
                activateArray<MB * 16>(t, a.act, a.actParam);
                staticFor<0, MB * 4>([&](auto iqTag) {
                        constexpr int iq = decltype(iqTag)::value;
                        constexpr int i = iq / 4, q = iq % 4;
                        const int ml = i * 32 + q * 8 + (lane >> 5) * 4;
                        *reinterpret_cast<f32x4 *>(stage + (lane & 31) * LDE + ml) = f32x4{t[iq * 4], t[iq * 4 + 1], t[iq * 4 + 2], t[iq * 4 + 3]};
                });
            }
        };
        if (lin1) stageBlock(std::true_type()); else stageBlock(std::false_type());
        // the staging area belongs to this wavefront alone, and the LDS serves a wavefront's accesses in the order it issued them: the
        // reads below see the writes above without a workgroup barrier (a barrier here kept the twelve wavefronts of a tile in step
        // through their stores)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        auto storeBlock = [&](auto slopeTag) {
            constexpr bool SL = decltype(slopeTag)::value;
#pragma unroll
            for (int t = 0; t < PASSES; ++t)
            {
                const int row = t * RPI + lane / VPR;
                const unsigned pl = pixBase + row;
                float v[8];
                const f32x4 lo = *reinterpret_cast<const f32x4 *>(stage + row * LDE + vcol);
                const f32x4 hi = *reinterpret_cast<const f32x4 *>(stage + row * LDE + vcol + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
                if (full)
                {
                    if (a.hasRes)
                    {
                        float r[8];
                        resRaw[t].toFloat(r);
                        if constexpr (SL)
                        {
#pragma unroll
                            for (int e = 0; e < 8; ++e) v[e] = activateSel<true>(v[e] + a.resMul * r[e], slope2, a.act2, a.act2Param);
                        }
                        else
                        {
#pragma unroll
                            for (int e = 0; e < 8; ++e) v[e] += a.resMul * r[e];
                            activateArray<8>(v, a.act2, a.act2Param);
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] *= a.outMul;
                    Raw8<TOut> o;
                    o.fromFloat(v);
                    if (a.up2)
                    {
                        // pixel (image, row, column) -> the 2 x 2 pixels (2 row + dy, 2 column + dx) of the upsampled tensor
                        const unsigned p = static_cast<unsigned>(p0) + pl;
                        const unsigned t1 = fastDiv(p, a.byOW), bImg = fastDiv(t1, a.byOH);
                        const unsigned ox = p - t1 * a.OW, oy = t1 - bImg * a.OH;
                        const unsigned q = ((bImg * 2u * a.OH + 2u * oy) * 2u * a.OW + 2u * ox) * a.outLd + ch;
                        const unsigned rowStep = 2u * a.OW * a.outLd;
                        const unsigned es = static_cast<unsigned>(sizeof(TOut));
                        const bool in = static_cast<int>(pl) < npix;
                        bufferStore8<TOut>(o, ry, in ? q * es : kOobOffset);
                        bufferStore8<TOut>(o, ry, in ? (q + a.outLd) * es : kOobOffset);
                        bufferStore8<TOut>(o, ry, in ? (q + rowStep) * es : kOobOffset);
                        bufferStore8<TOut>(o, ry, in ? (q + rowStep + a.outLd) * es : kOobOffset);
                    }
                    else bufferStore8<TOut>(o, ry, (pl * a.outLd + ch) * static_cast<unsigned>(sizeof(TOut)));
                }
                else if (chOk && static_cast<int>(pl) < npix)
                {
                    const T *rp = rBlock + static_cast<size_t>(pl) * a.resLd + ch;
                    TOut *yp = yBlock + static_cast<size_t>(pl) * a.outLd + ch;
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (mv + e < a.coutG)
                        {
                            float o = v[e];
                            if (a.hasRes) o = activateSel<SL>(o + a.resMul * toF(rp[e]), slope2, a.act2, a.act2Param);
                            yp[e] = fromF<TOut>(a.outMul * o);
                        }
                }
            }
        };
        if (lin2) storeBlock(std::true_type()); else storeBlock(std::false_type());
        if (j + 1 < NB)
        {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    });
}

// Epilogue of the kernels whose wavefronts come in two groups that multiplied different k-blocks of the same 64 x 64 wave tile
// (kg = group, wt = wave tile index): group g keeps pixel block g of the tile, parks the other block's partial sums in LDS for
// its partner and adds what the partner parked for it; then the ordinary epilogue runs over 64 x 32 per wavefront.
// One workgroup barrier in all: the affines are written in front of it, into the area behind the wavefronts' regions, and a wavefront stages
// its block (32 pixels x 68 floats) in the region it has just emptied -- the one its partner filled for it, which nobody else touches.
// LDS: 32 x 68 floats per wavefront + the affines (igemmSwapLds).
constexpr int kSwapRegion = 32 * (64 + 4);         // floats per wavefront: the staging block of a 64-channel wave tile, which holds the 2048 parked sums
template <int NW, int BM> constexpr size_t igemmSwapLds() { return (static_cast<size_t>(NW) * kSwapRegion + 2 * BM) * sizeof(float); }

template <typename T, typename TOut, int BM, int BN>
__device__ __forceinline__ void igemmEpilogueSwap(const IgemmArgs &a, f32x16 (&acc)[2][2], unsigned char *smemRaw, float chScale, float chShift,
                                                  int m0, int p0, int wm, int wn, int kg, int wt, int wave, int lane, int g, int nWaves)
{
    float *xch = reinterpret_cast<float *>(smemRaw);
    float *ss  = xch + nWaves * kSwapRegion;
    const int tid = wave * 64 + lane;
    if (tid < BM) { ss[tid] = chScale; ss[BM + tid] = chShift; }
    f32x16 mine[2][1];
    float *stageOwn = nullptr;
    auto swap = [&](auto gTag) {
        constexpr int q = decltype(gTag)::value;
        float *put = xch + (wt * 2 + q) * kSwapRegion + lane;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) put[(i * 16 + r) * 64] = acc[i][1 - q][r];
        __syncthreads();
        stageOwn = xch + (wt * 2 + (1 - q)) * kSwapRegion;
        const float *get = stageOwn + lane;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) mine[i][0][r] = acc[i][q][r] + get[(i * 16 + r) * 64];
    };
    if (kg == 0) swap(std::integral_constant<int, 0>()); else swap(std::integral_constant<int, 1>());
    // (the partner's sums are in registers before the staging writes below reach the same region: one wavefront's LDS accesses are served in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    igemmEpilogue<T, TOut, BM, BN, 64, 32>(a, mine, smemRaw, chScale, chShift, m0, p0, wm, wn * 2 + kg, wave, lane, g, ss, stageOwn);
}

// Register budget: two workgroups per CU (one wave of each per SIMD) so that one workgroup's barrier and epilogue
// are covered by the other's MFMAs; smaller tiles, which serve the short-K bandwidth-bound layers, get three to six.
constexpr int igemmWavesPerSimd(int bm, int bn, int kv = 8, int ns = 3, int nw = 4)
{
    // eight-wavefront workgroups put two waves on every SIMD: one workgroup per CU, or two where registers (64 x 64 wave tile)
    // and LDS (at most 80 KiB) allow it
    if (nw == 12) return 3;
    if (nw == 8) return (bm * bn <= 256 * 128 && static_cast<size_t>(ns) * (bm + bn) * kv * 16 <= 80 * 1024) ? 4 : 2;
    // (two-stage 64-byte-row variants of the small tiles: LDS for six to eight workgroups per CU, for the short-K layers that
    // live on memory bandwidth)
    if (ns == 2 && kv == 4 && bm * bn <= 64 * 128) return bm * bn > 64 * 64 ? 6 : 8;
    return bm * bn > 128 * 128 ? 2 : (bm * bn > 64 * 128 ? 3 : (bm * bn > 64 * 64 ? 4 : 6));
}

// 16-byte-per-lane load from a buffer resource straight into LDS: the 64 lanes of the wave fill 1 KiB starting at
// ldsAddr (lane l at ldsAddr + 16 * l); lanes whose voffset is out of range store zeros.  No VGPRs and no LDS store
// instructions are involved (the LDS store path moves a quarter of what the load path delivers).  Written as inline
// assembly so that the compiler does not serialise later LDS reads of *other* stages behind it; completion is
// awaited explicitly with dmaWait<N>() (at most N younger loads of this wave still in flight).
__device__ __forceinline__ void dmaLoad16(i32x4 rsrc, unsigned voffset, unsigned soffset, unsigned ldsAddr)
{
    asm volatile("s_mov_b32 m0, %3\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voffset), "s"(rsrc), "s"(soffset), "s"(ldsAddr) : "memory");
}

template <int N> __device__ __forceinline__ void dmaWait()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__device__ __forceinline__ i32x4 makeRsrcWords(const void *base, unsigned bytes)
{
    const unsigned long long p = reinterpret_cast<unsigned long long>(base);
    i32x4 r;
    r[0] = static_cast<int>(static_cast<unsigned>(p));
    r[1] = static_cast<int>(static_cast<unsigned>(p >> 32) & 0xffffu);
    r[2] = static_cast<int>(bytes);
    r[3] = 0x00020000;
    return r;
}

// Epilogue of the tiles that carry a tail: the workgroup's tile covers every output channel of the convolution (one channel tile), so
// the 1x1 convolution that reads this convolution's result can be computed from the tile itself.
//   1. the residual tile arrives in LDS by direct-to-LDS loads, in the layout of the result tile: [pixel][BM channels] float16, rows
//      unpadded, 16-byte chunk c of row r at position c ^ (r % chunks per row); the main loop has asked for it already (resIssued)
//      unless its K loop is a single step;
//   2. affine + activation on the accumulators in place; then every lane adds the residual values under its accumulators (it reads
//      them from LDS as 8-byte pieces: 4 consecutive channels of a pixel), applies the block activation and the output scale, rounds
//      to float16 and writes the result back to the same place -- the LDS tile now holds exactly the bytes of y;
//   3. y leaves for memory as 16-byte vectors, a pixel's channels from consecutive lanes (skipped when nobody else reads y);
//   4. second GEMM: wavefront (channel block of 32, group of pixel blocks) multiplies W2 (fragments straight from global memory, asked
//      for before step 3) with the y tile (B fragments from LDS) in k order, as a separate 1x1 launch would;
//   5. its epilogue stages z as float16 in LDS the same way and stores 16-byte vectors.
// The rounding points are those of two separate launches: y is rounded to float16 before the second GEMM reads it.
// LDS map (the main loop of these tiles has two stages of STAGE bytes at [0, 2 STAGE); 160 KiB in all): 4 KiB of per-channel affines at 0; the y
// tile's last UPROWS pixel rows behind the loop's stages, where the residual can arrive while the loop still runs; its first LOWROWS rows
// (if the space behind the stages does not hold the whole tile) 4 KiB into the loop stage that the last tile step does not use -- that stage is
// free from the barrier of the last step but one, and the residual rows are asked for right there; the z tile 4 KiB into the other stage (into
// the first one when the y tile lies behind the stages entirely).
constexpr int kTailMaxOut = 128;                   // output channels of the tail convolution
template <int BM, int BN, unsigned STAGE> struct TailLds
{
    static constexpr unsigned TOTAL = 160 * 1024;
    static constexpr unsigned HEAD  = 4096;
    static constexpr int YROWB   = BM * 2;                                   // bytes per pixel row of the y tile
    static constexpr int RPS     = 1024 / YROWB;                             // rows per 1 KiB delivery
    static constexpr int FITROWS = static_cast<int>((TOTAL - 2 * STAGE) / YROWB) / RPS * RPS;
    static constexpr int UPROWS  = FITROWS > BN ? BN : FITROWS;
    static constexpr int LOWROWS = BN - UPROWS;
    static constexpr unsigned UPOFF = 2 * STAGE;
    static constexpr unsigned ZBYTES = BN * kTailMaxOut * 2;
    static_assert(1024 % YROWB == 0 && LOWROWS % RPS == 0, "whole deliveries");
    static_assert(HEAD + LOWROWS * YROWB <= STAGE && (LOWROWS == 0 ? HEAD + ZBYTES <= UPOFF : HEAD + ZBYTES <= STAGE), "tail tiles fit the loop's stages");
    static_assert(UPOFF + UPROWS * YROWB <= TOTAL, "y tile fits behind the stages");
    __device__ static unsigned lowOff(int freeStage) { return static_cast<unsigned>(freeStage) * STAGE + HEAD; }
    __device__ static unsigned zOff(int freeStage) { return (LOWROWS == 0 ? 0u : static_cast<unsigned>(1 - freeStage) * STAGE) + HEAD; }
    // byte offset of row 0 of the part that holds `row` (a row's address is this + row * YROWB)
    __device__ static unsigned partBase(int row, unsigned low) { return row < LOWROWS ? low : UPOFF - LOWROWS * YROWB; }
    static constexpr size_t bytes() { return LOWROWS > 0 ? TOTAL : (UPOFF + static_cast<size_t>(UPROWS) * YROWB); }
};

// The residual rows [LOWROWS, BN) (upper) or [0, LOWROWS) of the tile at pixel p0, straight into their places in the y tile: 1 KiB per wave
// instruction, chunk c of row r at position c ^ (r % chunks per row).  Rows past the tensor and channels past out_c arrive as zeros.
template <int BM, int BN, unsigned STAGE, int NW>
__device__ __forceinline__ void tailIssueResidual(const IgemmArgs &a, int p0, unsigned ldsBase, int wave, int lane, bool upper, unsigned low)
{
    typedef TailLds<BM, BN, STAGE> L;
    constexpr int YC = BM / 8;
    const int npix = min(a.P - p0, BN);
    const i32x4 rr = makeRsrcWords(static_cast<const f16 *>(a.res) + static_cast<size_t>(p0) * a.resLd, static_cast<unsigned>(npix) * a.resLd * 2u);
    const int sBegin = (upper ? L::LOWROWS : 0) / L::RPS, sEnd = (upper ? BN : L::LOWROWS) / L::RPS;
    const unsigned base = ldsBase + (upper ? L::UPOFF - L::LOWROWS * L::YROWB : low);
    for (int s = sBegin + wave; s < sEnd; s += NW)
    {
        const int row = s * L::RPS + lane / YC;
        const int c = (lane % YC) ^ (row % YC);
        // (the address is the same in every lane; said explicitly, because it has to travel in a scalar register)
        const unsigned ldsAddr = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(base + static_cast<unsigned>(s) * 1024u)));
        dmaLoad16(rr, c * 8 < a.coutG ? static_cast<unsigned>(row * a.resLd + c * 8) * 2u : kOobOffset, 0u, ldsAddr);
    }
}

template <int BM, int BN, int WM, int WN, unsigned STAGE>
__device__ __forceinline__ void igemmTailEpilogue(const IgemmArgs &a, f32x16 (&acc)[BM / WM / 32][BN / WN / 32], unsigned char *smemRaw, unsigned ldsBase,
                                                  float chScale, float chShift, float sc2, float sh2, int p0, int wm, int wn, int wave, int lane,
                                                  bool resIssued, int freeStage)
{
    typedef TailLds<BM, BN, STAGE> L;
    constexpr int NW    = WM * WN;
    constexpr int NT    = 64 * NW;
    constexpr int TM    = BM / WM, TN = BN / WN;
    constexpr int MB    = TM / 32, NB = TN / 32;
    constexpr int YROWB = BM * 2;                     // bytes per pixel row of the y tile
    constexpr int YC    = BM / 8;                     // 16-byte chunks per row
    constexpr int ZROWB = kTailMaxOut * 2, ZC = kTailMaxOut / 8;
    const unsigned LOW = L::lowOff(freeStage);
    const unsigned ZOFF = L::zOff(freeStage);
    constexpr int PG    = NW / 4;                     // groups of pixel blocks in the second GEMM (4 channel blocks of 32)
    constexpr int TN2   = BN / PG;
    constexpr int NB2   = TN2 / 32;
    constexpr int KB2   = BM / 16;                    // k-blocks of the second GEMM
    static_assert(NW % 4 == 0 && BN % PG == 0 && TN2 % 32 == 0 && (BN * YC) % NT == 0 && (BN * ZC) % NT == 0, "tail geometry");
    static_assert((2 * BM + 2 * kTailMaxOut) * 4 <= L::HEAD, "the affines fit in front of the tiles");

    float *ss = reinterpret_cast<float *>(smemRaw);   // [BM] scale, [BM] shift, [128] scale2, [128] shift2
    const int tid = wave * 64 + lane;
    const int npix = min(a.P - p0, BN);
    const int half = lane >> 5;
    if (tid < BM) { ss[tid] = chScale; ss[BM + tid] = chShift; }
    if (tid < kTailMaxOut) { ss[2 * BM + tid] = sc2; ss[2 * BM + kTailMaxOut + tid] = sh2; }

    // 1. residual tile -> LDS, unless the main loop asked for it
    if (a.hasRes && !resIssued)
    {
        tailIssueResidual<BM, BN, STAGE, NW>(a, p0, ldsBase, wave, lane, true, LOW);
        if (L::LOWROWS > 0) tailIssueResidual<BM, BN, STAGE, NW>(a, p0, ldsBase, wave, lane, false, LOW);
    }
    __syncthreads();                                  // affines visible

    // 2a. affine + activation in place
    float slope1, slope2, slope3;
    const bool lin1 = actIsSlope(a.act, a.actParam, slope1);
    const bool lin2 = actIsSlope(a.act2, a.act2Param, slope2);
    const bool lin3 = actIsSlope(a.act3, a.act3Param, slope3);
    staticFor<0, NB>([&](auto jTag) {
        constexpr int j = decltype(jTag)::value;
        float t[MB * 16];
        staticFor<0, MB * 4>([&](auto iqTag) {
            constexpr int iq = decltype(iqTag)::value;
            constexpr int i = iq / 4, q = iq % 4;
            const int ml = wm * TM + i * 32 + q * 8 + half * 4;
            const f32x4 sc = *reinterpret_cast<const f32x4 *>(ss + ml);
            const f32x4 sh = *reinterpret_cast<const f32x4 *>(ss + BM + ml);
#pragma unroll
            for (int e = 0; e < 4; ++e) t[iq * 4 + e] = acc[i][j][q * 4 + e] * sc[e] + sh[e];
        });
        if (lin1)
        {
#pragma unroll
            for (int e = 0; e < MB * 16; ++e) t[e] = activateSel<true>(t[e], slope1, a.act, a.actParam);
        }
        else activateArray<MB * 16>(t, a.act, a.actParam);
        staticFor<0, MB * 16>([&](auto eTag) { constexpr int e = decltype(eTag)::value; acc[e / 16][j][e % 16] = t[e]; });
    });
    dmaWait<0>();
    __syncthreads();                                  // residual tile complete

    // 2b. residual, block activation, scale, rounding; the y tile replaces the residual tile
    staticFor<0, NB>([&](auto jTag) {
        constexpr int j = decltype(jTag)::value;
        const int row = wn * TN + j * 32 + (lane & 31);
        unsigned char *rowPtr = smemRaw + L::partBase(row, LOW) + row * YROWB + half * 8;
        const int sw = row % YC;
        staticFor<0, MB * 4>([&](auto iqTag) {
            constexpr int iq = decltype(iqTag)::value;
            constexpr int i = iq / 4, q = iq % 4;
            const int c = (wm * TM + i * 32) / 8 + q;
            f16x4 *cell = reinterpret_cast<f16x4 *>(rowPtr + ((c ^ sw) * 16));
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e];
            if (a.hasRes)
            {
                const f16x4 r = *cell;
                if (lin2)
                {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = activateSel<true>(v[e] + a.resMul * static_cast<float>(r[e]), slope2, a.act2, a.act2Param);
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += a.resMul * static_cast<float>(r[e]);
                    activateArray<4>(v, a.act2, a.act2Param);
                }
            }
            f16x4 h;
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = static_cast<f16>(v[e] * a.outMul);
            *cell = h;
        });
    });

    // 4a. fragments of W2 for this wavefront's 32 output channels, all k-blocks (the accumulators' registers are free now)
    const int wm2 = wave % 4, wn2 = wave / 4;
    const __amdgpu_buffer_rsrc_t rw2 = makeRsrc(a.w2, a.w2Bytes);
    f16x8 fa2[KB2];
    {
        const int m2 = wm2 * 32 + (lane & 31);
#pragma unroll
        for (int kb = 0; kb < KB2; ++kb)
        {
            const int c = 2 * kb + half;
            fa2[kb] = bufferLoad16<f16x8>(rw2, (m2 < a.cout2 && c * 8 < a.coutG) ? static_cast<unsigned>(m2 * a.coutG + c * 8) * 2u : kOobOffset, 0u);
        }
    }
    __syncthreads();                                  // y tile complete

    // 3. y -> memory
    if (a.writeY)
    {
        const __amdgpu_buffer_rsrc_t ry = makeRsrc(static_cast<f16 *>(a.y) + static_cast<size_t>(p0) * a.outLd, static_cast<unsigned>(npix) * a.outLd * 2u);
#pragma unroll
        for (int k = 0; k < BN * YC / NT; ++k)
        {
            const int v = tid + NT * k;
            const int row = v / YC, c = v % YC;
            const i32x4 d = *reinterpret_cast<const i32x4 *>(smemRaw + L::partBase(row, LOW) + row * YROWB + ((c ^ (row % YC)) * 16));
            __builtin_amdgcn_raw_buffer_store_b128(d, ry, c * 8 < a.coutG ? (row * a.outLd + c * 8) * 2 : static_cast<int>(kOobOffset), 0, 0);
        }
    }

    // 4b. z tile = W2 . y tile
    f32x16 acc2[NB2];
#pragma unroll
    for (int j = 0; j < NB2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[j][r] = 0.f;
    const unsigned char *bBase[NB2];
    int bSw[NB2];
#pragma unroll
    for (int j = 0; j < NB2; ++j)
    {
        const int row = wn2 * TN2 + j * 32 + (lane & 31);
        bBase[j] = smemRaw + L::partBase(row, LOW) + row * YROWB;
        bSw[j] = row % YC;
    }
    staticFor<0, KB2>([&](auto kbTag) {
        constexpr int kb = decltype(kbTag)::value;
        f16x8 fb[NB2];
#pragma unroll
        for (int j = 0; j < NB2; ++j) fb[j] = *reinterpret_cast<const f16x8 *>(bBase[j] + (((2 * kb + half) ^ bSw[j]) * 16));
#pragma unroll
        for (int j = 0; j < NB2; ++j) mfmaBlock(fa2[kb], fb[j], acc2[j]);
    });

    // 5. z: affine, activation, scale, float16, staged in LDS, stored as 16-byte vectors
    staticFor<0, NB2>([&](auto jTag) {
        constexpr int j = decltype(jTag)::value;
        const int row = wn2 * TN2 + j * 32 + (lane & 31);
        unsigned char *rowPtr = smemRaw + ZOFF + row * ZROWB + half * 8;
        float t[16];
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            const int mch = wm2 * 32 + q * 8 + half * 4;
            const f32x4 sc = *reinterpret_cast<const f32x4 *>(ss + 2 * BM + mch);
            const f32x4 sh = *reinterpret_cast<const f32x4 *>(ss + 2 * BM + kTailMaxOut + mch);
#pragma unroll
            for (int e = 0; e < 4; ++e) t[q * 4 + e] = acc2[j][q * 4 + e] * sc[e] + sh[e];
        }
        if (lin3)
        {
#pragma unroll
            for (int e = 0; e < 16; ++e) t[e] = activateSel<true>(t[e], slope3, a.act3, a.act3Param);
        }
        else activateArray<16>(t, a.act3, a.act3Param);
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            f16x4 h;
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = static_cast<f16>(t[q * 4 + e] * a.zMul);
            *reinterpret_cast<f16x4 *>(rowPtr + (((wm2 * 4 + q) ^ (row % ZC)) * 16)) = h;
        }
    });
    __syncthreads();
    {
        const __amdgpu_buffer_rsrc_t rz = makeRsrc(static_cast<f16 *>(a.z) + static_cast<size_t>(p0) * a.zLd, static_cast<unsigned>(npix) * a.zLd * 2u);
#pragma unroll
        for (int k = 0; k < BN * ZC / NT; ++k)
        {
            const int v = tid + NT * k;
            const int row = v / ZC, c = v % ZC;
            const i32x4 d = *reinterpret_cast<const i32x4 *>(smemRaw + ZOFF + row * ZROWB + ((c ^ (row % ZC)) * 16));
            __builtin_amdgcn_raw_buffer_store_b128(d, rz, c * 8 < a.cout2 ? (row * a.zLd + c * 8) * 2 : static_cast<int>(kOobOffset), 0, 0);
        }
    }
}


// KG = 2: two groups of wavefronts share the WM x WN grid of (then 64 x 64) wave tiles and split the k-blocks of every tile step
// between them, which takes a third off the LDS fragment reads per MFMA against 32 x 64 wave tiles of the same workgroup tile.
// TAIL = 1: the epilogue also computes the 1x1 convolution that reads this one's result (igemmTailEpilogue); float16 only.
template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN, int NS, int KG = 1, int TAIL = 0>
__global__ __launch_bounds__(64 * WM * WN * KG)
__attribute__((amdgpu_waves_per_eu(KG == 2 ? (WM * WN * KG) / 4 : igemmWavesPerSimd(BM, BN, KV, NS, WM * WN),
                                   KG == 2 ? (WM * WN * KG == 4 ? 3 : (WM * WN * KG) / 4) : igemmWavesPerSimd(BM, BN, KV, NS, WM * WN))))
void convIgemmKernel(IgemmArgs a)
{
    typedef typename Frag<T>::V V;
    constexpr int VEC   = Frag<T>::VEC;
    constexpr int BK    = KV * VEC;               // K elements per tile step
    constexpr int NWT   = WM * WN;                // wave tiles
    constexpr int NT    = 64 * NWT * KG;          // threads: 4, 8 or 12 wavefronts
    constexpr int RPP   = NT / KV;                // rows loaded per pass of the workgroup
    constexpr int BML   = (BM + RPP - 1) / RPP * RPP; // A rows held in LDS: BM rounded up to whole passes (the surplus rows load nothing)
    constexpr int AROWS = BML / RPP;              // A rows (16-byte chunks) per thread per tile step
    constexpr int BNL   = (BN + RPP - 1) / RPP * RPP; // B rows held in LDS: BN rounded up to whole passes (the surplus rows load nothing)
    constexpr int BROWS = BNL / RPP;              // B rows per thread
    constexpr int NL    = AROWS + BROWS;          // loads per thread per tile step
    constexpr int TM    = BM / WM;                // wave tile
    constexpr int TN    = BN / WN;
    constexpr int MB    = TM / 32;
    constexpr int NB    = TN / 32;
    constexpr int S     = KV / 2 / KG;            // MFMA k-steps per tile step and wavefront (one k-block = two 16-byte chunks)
    constexpr unsigned ES = sizeof(T);
    constexpr int ROWB  = KV * 16;                // bytes per LDS row: unpadded
    constexpr int SWDIV = 16 / KV;                // rows per 256 bytes of LDS
    constexpr int A_BYTES = BML * ROWB;
    constexpr unsigned STAGE = (BML + BNL) * ROWB; // one LDS stage: A rows, then B rows
    static_assert(TM % 32 == 0 && TN % 32 == 0 && (NT == 256 || NT == 512 || NT == 768) && S % 2 == 0, "wave grid");
    static_assert(KG == 1 || (KG == 2 && TM == 64 && TN == 64), "the K-split variant works on 64 x 64 wave tiles");
    static_assert(NS >= 2 && NS <= 8, "LDS stages");

    extern __shared__ __attribute__((aligned(16))) unsigned char smemRaw[];
    const unsigned ldsBase = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)smemRaw));

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg   = wave / NWT;                  // which k-blocks of a tile step this wavefront multiplies
    const int wm   = (wave % NWT) / WN;
    const int wn   = (wave % NWT) % WN;
    const int g    = blockIdx.z;
    int mTile, pTile;
    if (!igemmTileOf(a, (a.P + BN - 1) / BN, mTile, pTile)) return;
    const int m0   = mTile * BM;
    const int p0   = pTile * BN;

    const unsigned gx = static_cast<unsigned>(g) * a.cinG * ES;
    const unsigned gw = static_cast<unsigned>(g) * a.coutG * a.taps * a.cinG * ES;
    const i32x4 rx = makeRsrcWords(static_cast<const unsigned char *>(a.x) + gx, a.xBytes - gx);
    const i32x4 rw = makeRsrcWords(static_cast<const unsigned char *>(a.w) + gw, a.wBytes - gw);

    float chScale, chShift;
    loadChannelAffine(a, g, m0, tid, BM, chScale, chShift);
    float sc2 = 1.f, sh2 = 0.f;                       // TAIL: the second convolution's affine of channel tid
    if constexpr (TAIL != 0)
        if (tid < kTailMaxOut && tid < a.cout2)
        {
            if (a.scale2) sc2 = a.scale2[tid];
            if (a.shift2) sh2 = a.shift2[tid];
        }

    // LDS layout of a stage: rows of KV 16-byte chunks without padding; chunk c of row r sits at chunk position
    // c ^ ((r / SWDIV) % KV).  With that XOR the 16 lanes the LDS serves per cycle hit 16 different 16-byte bank
    // groups when a wave reads one chunk column of 32 rows, while a wave's load fills 64 consecutive chunk
    // positions.  Thread tid owns chunk position tid % KV of row tid / KV (+ RPP rows per pass): byte tid * 16.
    const int ldRow = tid / KV;
    const int ldVec = (tid % KV) ^ ((ldRow / SWDIV) % KV);   // the logical chunk this thread fetches

    // Per-thread row state, fixed over the K loop: byte offset of the row's first tap (may be "negative", it wraps
    // back into range once a valid tap offset is added) and one bit per tap telling whether that tap lies inside
    // the image for this output pixel.
    unsigned bOff[BROWS];
    unsigned long long bMask[BROWS];
#pragma unroll
    for (int i = 0; i < BROWS; ++i)
    {
        const int p = p0 + ldRow + i * RPP;
        const bool ok = p < a.P && ldRow + i * RPP < BN;
        const int pp = ok ? p : 0;
        const int t  = static_cast<int>(fastDiv(static_cast<unsigned>(pp), a.byOW));
        const int ox = pp - t * a.OW;
        const int b  = static_cast<int>(fastDiv(static_cast<unsigned>(t), a.byOH));
        const int oy = t - b * a.OH;
        const int iy0 = oy * a.stride - a.pad;
        const int ix0 = ox * a.stride - a.pad;
        const long long pix = (static_cast<long long>(b) * a.H + iy0) * a.W + ix0;
        bOff[i] = static_cast<unsigned>((pix * a.inLd + ldVec * VEC) * static_cast<long long>(ES));
        // a tap lies inside the image when its row does and its column does: ksize row tests and ksize column tests instead of ksize^2 of both
        unsigned rowBits = 0, colBits = 0;
        for (int k = 0; k < a.ksize; ++k)
        {
            const int iy = iy0 + k * a.dil, ix = ix0 + k * a.dil;
            rowBits |= ((iy >= 0 && iy < a.H) ? 1u : 0u) << k;
            colBits |= ((ix >= 0 && ix < a.W) ? 1u : 0u) << k;
        }
        unsigned long long mask = 0;
        for (int ki = 0; ki < a.ksize; ++ki)
            if ((rowBits >> ki) & 1u) mask |= static_cast<unsigned long long>(colBits) << (ki * a.ksize);
        bMask[i] = ok ? mask : 0ull;
    }
    unsigned aOff[AROWS];
#pragma unroll
    for (int i = 0; i < AROWS; ++i)
    {
        const int m = m0 + ldRow + i * RPP;
        aOff[i] = (m < a.coutG && ldRow + i * RPP < BM) ? (static_cast<unsigned>(m) * a.taps * a.cinG + ldVec * VEC) * ES : kOobOffset;
    }

    unsigned bVoff[BROWS];                       // B offsets of the tap being loaded
    auto setTap = [&](int tap) {
        const int ki = tap / a.ksize;
        const int kj = tap - ki * a.ksize;
        const unsigned tapOff = static_cast<unsigned>((ki * a.dil * a.W + kj * a.dil) * a.inLd) * ES;
#pragma unroll
        for (int i = 0; i < BROWS; ++i) bVoff[i] = ((bMask[i] >> tap) & 1ull) ? bOff[i] + tapOff : kOobOffset;
    };
    // Load l of a tile step (A rows first, then B rows) into the LDS stage at byte offset stageOff.  `cut` blanks
    // the lane: past the last channel of a ragged K chunk, or a step past the end of K.
    const unsigned waveLds = ldsBase + wave * 1024;
    auto issueLoad = [&](auto lTag, unsigned sA, unsigned sB, bool cut, unsigned stageOff) {
        constexpr int l = decltype(lTag)::value;
        if constexpr (l < AROWS)
            dmaLoad16(rw, cut ? kOobOffset : aOff[l], sA, waveLds + stageOff + l * RPP * ROWB);
        else
            dmaLoad16(rx, cut ? kOobOffset : bVoff[l - AROWS], sB, waveLds + stageOff + A_BYTES + (l - AROWS) * RPP * ROWB);
    };
    int tapNext = 0, chunkNext = 0;              // the tile step whose loads were issued last
    unsigned sANext = 0, sBNext = 0;
    bool cutNext = false, pastEndNext = false;
    auto advance = [&](bool pastEnd) {
        pastEndNext = pastEnd;
        if (++chunkNext == a.cChunks) { chunkNext = 0; ++tapNext; if (tapNext < a.taps) setTap(tapNext); }
        sANext = (static_cast<unsigned>(tapNext) * a.cinG + chunkNext * BK) * ES;
        sBNext = static_cast<unsigned>(chunkNext * BK) * ES;
        cutNext = pastEnd || (a.ragged && (chunkNext * BK + ldVec * VEC >= a.cinG));
    };

    // fragment addresses: lane l feeds MFMA row l % 32 with chunk 2 * kb + l / 32 of k-step kb
    const int fragRow = lane & 31;
    const int fragSw  = (fragRow / SWDIV) % KV;
    unsigned aAddr[S], bAddr[S];
#pragma unroll
    for (int kb = 0; kb < S; ++kb)
    {
        const unsigned off = fragRow * ROWB + (((2 * (kg * S + kb) + (lane >> 5)) ^ fragSw) * 16);
        aAddr[kb] = wm * TM * ROWB + off;
        bAddr[kb] = A_BYTES + wn * TN * ROWB + off;
    }

    V fa[2][MB], fb[2][NB];                      // fragments of k-step s live in buffer s % 2
    auto readFrags = [&](unsigned stageOff, auto kbTag) {
        constexpr int kb = decltype(kbTag)::value;
        const unsigned char *ap = smemRaw + (aAddr[kb] + stageOff);
        const unsigned char *bp = smemRaw + (bAddr[kb] + stageOff);
#pragma unroll
        for (int i = 0; i < MB; ++i) fa[kb % 2][i] = *reinterpret_cast<const V *>(ap + i * 32 * ROWB);
#pragma unroll
        for (int j = 0; j < NB; ++j) fb[kb % 2][j] = *reinterpret_cast<const V *>(bp + j * 32 * ROWB);
    };

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // NS >= 3 LDS stages rotate: while tile step `it` is multiplied out of stage `cur`, steps it+1 .. it+NS-2 are
    // already (being) delivered into the following stages and the loads of step it+NS-1 go into the stage before
    // `cur`, whose last readers all passed the previous barrier.  How far ahead the loads must run is set by
    // Little's law: a CU has to keep (bytes per step) / (MFMA time per step) x (L2 latency) in flight, tens of KiB.
    // The NL loads of a step are spread evenly between the step's MFMAs (issued back to back they fill the memory
    // pipeline's queue and the wave, stuck on the issue, stops feeding the matrix core).
    // NS = 2: step it+2 goes into `cur` itself, which is free once the barrier of step `it` is passed, so all NL
    // loads follow that barrier, among the MFMAs of the last k-step, and must have landed by the next barrier.
    // Steps past the end of K are issued all the same with every lane out of range, so the count of loads in
    // flight is the same in every step.  LDS reads for k-step s+1 are issued before the MFMAs of k-step s, and
    // the single barrier sits before the last k-step, whose MFMAs cover the first fragment reads of step it+1.
    constexpr int PER  = MB * NB;                // MFMAs per k-step
    constexpr int TOT  = PER * S;                // MFMAs per tile step
    // NS >= 3: load l follows MFMA number l * TOT / NL, NPRE of them ahead of the barrier (numbers < TOT - PER);
    // NS = 2: load l follows MFMA number TOT - PER + l * PER / NL
    constexpr int NPRE = NS >= 3 ? ((TOT - PER) * NL + TOT - 1) / TOT : 0;
    constexpr int LBASE = NS >= 3 ? 0 : TOT - PER;
    constexpr int LSPAN = NS >= 3 ? TOT : PER;
    constexpr int AHEAD = NS >= 3 ? NS - 1 : 2;  // the loads issued during step `it` belong to step it + AHEAD
    constexpr int INFLIGHT = NS >= 3 ? (NS - 3) * NL + NPRE : 0;   // loads younger than step it+1's at the barrier

    // split-K: this workgroup multiplies tile steps [itBegin, itBegin + nLocal) of the K loop
    const int itBegin = a.splitK > 1 ? static_cast<int>(static_cast<long long>(blockIdx.y) * a.nIter / a.splitK) : 0;
    const int nLocal  = a.splitK > 1 ? static_cast<int>(static_cast<long long>(blockIdx.y + 1) * a.nIter / a.splitK) - itBegin : a.nIter;
    const bool tailPrefetch = TAIL != 0 && a.hasRes && nLocal >= 2;
    tapNext = itBegin / a.cChunks;
    chunkNext = itBegin - tapNext * a.cChunks - 1;            // advance() steps onto the first tile step
    setTap(tapNext);
    staticFor<0, AHEAD>([&](auto stTag) {
        constexpr int st = decltype(stTag)::value;
        advance(nLocal <= st);
        staticFor<0, NL>([&](auto lTag) { issueLoad(lTag, sANext, sBNext, cutNext, st * STAGE); });
    });
    dmaWait<(AHEAD - 1) * NL>();                 // step 0 has landed
    __syncthreads();
    readFrags(0, std::integral_constant<int, 0>());

    // cur: stage of step it; nxt: of step it+1; nn: where the loads issued during step it go
    unsigned cur = 0, nxt = STAGE, nn = NS >= 3 ? (NS - 1) * STAGE : 0;
    for (int it = 0; it < nLocal; ++it)
    {
        advance(it + AHEAD >= nLocal);          // sANext / sBNext / cutNext now describe step it + AHEAD
        readFrags(cur, std::integral_constant<int, 1>());
        __builtin_amdgcn_sched_barrier(0);
        staticFor<0, TOT>([&](auto gTag) {
            constexpr int gi = decltype(gTag)::value;
            constexpr int ks = gi / PER;
            if constexpr (gi % PER == 0 && ks >= 1)
            {
                if constexpr (ks < S - 1)
                    readFrags(cur, std::integral_constant<int, ks + 1>());
                else
                {
                    dmaWait<INFLIGHT>();         // all of step it+1 has landed; younger loads may be in flight
                    __syncthreads();
                    if constexpr (TAIL != 0)
                    {
                        // the residual tile of the epilogue: the rows that lie behind the loop's stages right away, the others into the
                        // stage of this step -- free from here on -- in the last step but one
                        if (tailPrefetch && it == 0) tailIssueResidual<BM, BN, STAGE, NT / 64>(a, p0, ldsBase, wave, lane, true, 0u);
                        if (tailPrefetch && it == nLocal - 2 && TailLds<BM, BN, STAGE>::LOWROWS > 0)
                            tailIssueResidual<BM, BN, STAGE, NT / 64>(a, p0, ldsBase, wave, lane, false, TailLds<BM, BN, STAGE>::lowOff(nLocal & 1));
                    }
                    readFrags(nxt, std::integral_constant<int, 0>());
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            mfmaBlock(fa[ks % 2][(gi % PER) / NB], fb[ks % 2][(gi % PER) % NB], acc[(gi % PER) / NB][(gi % PER) % NB]);
            if constexpr (gi >= LBASE)
            {
                // loads l with LBASE + l * LSPAN / NL == gi
                constexpr int first = ((gi - LBASE) * NL + LSPAN - 1) / LSPAN;
                constexpr int last  = ((gi - LBASE + 1) * NL + LSPAN - 1) / LSPAN;
                // (TAIL: the stages that steps past the end of K would zero receive residual rows instead)
                if (!(TAIL != 0 && pastEndNext))
                    staticFor<first, last>([&](auto lTag) { issueLoad(lTag, sANext, sBNext, cutNext, nn); });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        nn = NS >= 3 ? cur : nxt;
        cur = nxt;
        nxt = nxt + STAGE == NS * STAGE ? 0u : nxt + STAGE;
    }
    dmaWait<0>();
    __syncthreads();

    if constexpr (TAIL != 0)
    {
        static_assert(KG == 1 && NS == 2 && std::is_same<T, f16>::value && std::is_same<TOut, f16>::value, "the tail is a float16 epilogue of the unsplit two-stage kernel");
        igemmTailEpilogue<BM, BN, WM, WN, STAGE>(a, acc, smemRaw, ldsBase, chScale, chShift, sc2, sh2, p0, wm, wn, wave, lane, tailPrefetch, tailPrefetch ? (nLocal & 1) : 0);
        return;
    }
    if (a.splitK > 1)
    {
        // raw float32 partial sums of this K slice; affine, activation and residual follow in the reduction pass
        IgemmArgs e = a;
        e.act = MSNH_ACT_NONE; e.hasRes = 0; e.outMul = 1.f;
        e.y = a.ws + static_cast<size_t>(blockIdx.y) * a.P * a.wsLd;
        e.outLd = a.wsLd;
        e.vecOk = (a.wsLd % 8 == 0) && (a.coutG % 8 == 0 || gridDim.z == 1);
        if constexpr (KG == 2) igemmEpilogueSwap<T, float, BM, BN>(e, acc, smemRaw, 1.f, 0.f, m0, p0, wm, wn, kg, wave % NWT, wave, lane, g, NT / 64);
        else igemmEpilogue<T, float, BM, BN, TM, TN>(e, acc, smemRaw, 1.f, 0.f, m0, p0, wm, wn, wave, lane, g);
        return;
    }
    if constexpr (KG == 2) igemmEpilogueSwap<T, TOut, BM, BN>(a, acc, smemRaw, chScale, chShift, m0, p0, wm, wn, kg, wave % NWT, wave, lane, g, NT / 64);
    else igemmEpilogue<T, TOut, BM, BN, TM, TN>(a, acc, smemRaw, chScale, chShift, m0, p0, wm, wn, wave, lane, g);
}

// Split-K reduction: sums the K slices in slice order (so the result does not depend on timing) and applies the
// convolution's epilogue.  One thread per (pixel, 4 channels).
template <typename T, typename TOut>
__global__ __launch_bounds__(256) void splitKReduceKernel(IgemmArgs a, int outC, long long total)
{
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cq = outC / 4;
    const int c = static_cast<int>(idx % cq) * 4;
    const long long p = idx / cq;
    const float *w = a.ws + static_cast<size_t>(p) * a.wsLd + c;
    f32x4 acc = *reinterpret_cast<const f32x4 *>(w);
    for (int s = 1; s < a.splitK; ++s) acc += *reinterpret_cast<const f32x4 *>(w + static_cast<size_t>(s) * a.P * a.wsLd);
    const T *res = static_cast<const T *>(a.res);
    TOut *y = static_cast<TOut *>(a.y);
#pragma unroll
    for (int k = 0; k < 4; ++k)
    {
        const float sc = a.scale ? a.scale[c + k] : 1.f;
        const float sh = a.shift ? a.shift[c + k] : 0.f;
        float v = activate(acc[k] * sc + sh, a.act, a.actParam);
        if (a.hasRes) v = activate(v + a.resMul * toF(res[static_cast<size_t>(p) * a.resLd + c + k]), a.act2, a.act2Param);
        y[static_cast<size_t>(p) * a.outLd + c + k] = fromF<TOut>(a.outMul * v);
    }
}

constexpr int kSplitKMax = 8;

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN, int NS = 3, int KG = 1, int TAIL = 0>
inline int launchIgemm(IgemmArgs &a, int groups, hipStream_t st)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int BK  = KV * VEC;
    if (TAIL != 0 || a.tailOn)
    {
        // a launch with a tail needs a tile that has one, and the other way round; the tile must hold every output channel
        if (!(TAIL != 0 && a.tailOn) || groups != 1 || a.splitMax > 1 || a.coutG > BM || a.coutG % 8 != 0 || a.cout2 > kTailMaxOut || a.cout2 % 8 != 0 ||
            a.cout2 <= 0 || a.outLd % 8 != 0 || a.zLd % 8 != 0 || (a.hasRes && a.resLd % 8 != 0) || !a.vecOk)
        {
            setError("conv2d: this tile needs a 1x1 convolution behind it (msnh_hip_conv2d_tail), the others take none; ungrouped, channel counts that fit one tile");
            return 3;
        }
    }
    if (a.up2 && (TAIL != 0 || groups != 1 || a.hasRes || a.splitMax > 1 || (!a.vecOk && !a.dryRun) || a.coutG % 8 != 0))
    {
        setError("conv2d: the upsampling epilogue takes an ungrouped convolution without residual, channel counts multiples of 8");
        return 3;
    }
    a.cChunks = (a.cinG + BK - 1) / BK;
    a.nIter   = a.taps * a.cChunks;
    a.ragged  = (a.cinG % BK) != 0;
    if (a.taps > 64 || !a.buffersOk)
    {
        setError("conv2d: the implicit GEMM needs at most 64 filter taps and tensors below 2 GiB");
        return 3;
    }
    constexpr int RPP = 64 * WM * WN * KG / KV;
    const size_t smemLoop = static_cast<size_t>(NS) * ((BM + RPP - 1) / RPP * RPP + (BN + RPP - 1) / RPP * RPP) * KV * 16;
    size_t smemEpi = 0;
    if constexpr (TAIL != 0)
    {
        constexpr unsigned STAGE = static_cast<unsigned>(((BM + RPP - 1) / RPP * RPP + (BN + RPP - 1) / RPP * RPP) * KV * 16);
        smemEpi = TailLds<BM, BN, STAGE>::bytes();
    }
    else smemEpi = std::max(igemmEpilogueLds<BM, BM / WM, WM * WN * KG>(), KG == 2 ? igemmSwapLds<WM * WN * KG, BM>() : size_t(0));
    const size_t smem = smemLoop > smemEpi ? smemLoop : smemEpi;
    a.mTiles = (a.coutG + BM - 1) / BM;
    const int tiles = a.mTiles * ((a.P + BN - 1) / BN);
    a.splitK = 1;
    if (a.splitMax > 1)
    {
        // enough slices to give every CU two workgroups, each slice at least four tile steps long
        int want = (512 + tiles * groups - 1) / (tiles * groups);
        if (want > a.splitMax) want = a.splitMax;
        if (want > a.nIter / 4) want = a.nIter / 4;
        if (want < 2 || a.wsLd % 4 != 0)
        {
            setError("conv2d: split-K does not apply to this shape and tile");
            return 3;
        }
        a.splitK = want;
    }
    dim3 grid(igemmGridX(a, (a.P + BN - 1) / BN, sizeof(T), a.splitK == 1 && groups == 1), a.splitK, groups);
    if (a.dryRun) return 0;
    auto kern = convIgemmKernel<T, TOut, BM, BN, KV, WM, WN, NS, KG, TAIL>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, grid, dim3(64 * WM * WN * KG), smem, st, a);
    MSNH_LAUNCH_CHECK();
    if (a.splitK > 1)
    {
        const int outC = a.coutG * groups;
        const long long total = static_cast<long long>(a.P) * (outC / 4);
        hipLaunchKernelGGL((splitKReduceKernel<T, TOut>), dim3(gridFor(total, 256)), dim3(256), 0, st, a, outC, total);
        MSNH_LAUNCH_CHECK();
    }
    return 0;
}

} // namespace msnh

#include "conv_patch.hpp"
#include "conv_patch8.hpp"

namespace msnh {

// Tile configurations (BM x BN output tile, KV 16-byte vectors of K per step, WM x WN wavefront grid).
// Index 0 is "choose for me"; the others can be forced through msnh_conv_desc::tile, which is how the host
// library's per-layer search picks the fastest one at load time.
constexpr int kIgemmTiles = 65;
constexpr int kIgemmTailTileFirst = 64;         // tiles from here on carry a tail (msnh_hip_conv2d_tail)

template <typename T, typename TOut>
int igemmDispatch(IgemmArgs &a, int groups, int tile, hipStream_t st)
{
    switch (tile)
    {
    case 1:  return launchIgemm<T, TOut, 128, 128, 8, 2, 2>(a, groups, st);
    case 2:  return launchIgemm<T, TOut, 128, 128, 4, 2, 2>(a, groups, st);
    case 3:  return launchIgemm<T, TOut, 64, 256, 8, 1, 4>(a, groups, st);
    case 4:  return launchIgemm<T, TOut, 64, 256, 4, 1, 4>(a, groups, st);
    case 5:  return launchIgemm<T, TOut, 32, 256, 8, 1, 4>(a, groups, st);
    case 6:  return launchIgemm<T, TOut, 64, 64, 4, 2, 2>(a, groups, st);
    case 7:  return launchIgemm<T, TOut, 256, 128, 4, 2, 2>(a, groups, st);
    case 8:  return launchIgemm<T, TOut, 128, 64, 8, 2, 2>(a, groups, st);
    case 9:  return launchIgemm<T, TOut, 128, 64, 4, 2, 2>(a, groups, st);
    case 10: return launchIgemm<T, TOut, 64, 128, 8, 1, 4>(a, groups, st);
    case 11: return launchIgemm<T, TOut, 64, 128, 4, 1, 4>(a, groups, st);
    case 12: return launchIgemm<T, TOut, 64, 64, 8, 2, 2>(a, groups, st);
    case 13: return launchIgemm<T, TOut, 128, 256, 4, 2, 2>(a, groups, st);
    // 3x3 stride-1 pad-1 only: input patch resident in LDS, weights streamed per tap (last number: patch slices
    // per wave and step, 2 for wide images)
    case 14: return launchPatch<T, TOut, 128, 256, 4, 2, 2, 1>(a, groups, st);
    case 15: return launchPatch<T, TOut, 128, 256, 4, 2, 2, 2>(a, groups, st);
    case 16: return launchPatch<T, TOut, 128, 128, 4, 2, 2, 1>(a, groups, st);
    case 17: return launchPatch<T, TOut, 256, 128, 4, 2, 2, 1>(a, groups, st);
    case 18: return launchPatch<T, TOut, 64, 256, 4, 1, 4, 1>(a, groups, st);
    case 19: return launchPatch<T, TOut, 128, 128, 4, 2, 2, 2>(a, groups, st);
    // two LDS stages, 128-byte rows
    case 20: return launchIgemm<T, TOut, 128, 128, 8, 2, 2, 2>(a, groups, st);
    case 21: return launchIgemm<T, TOut, 256, 128, 8, 2, 2, 2>(a, groups, st);
    case 22: return launchIgemm<T, TOut, 128, 256, 8, 2, 2, 2>(a, groups, st);
    case 23: return launchIgemm<T, TOut, 128, 64, 8, 2, 2, 2>(a, groups, st);
    case 24: return launchIgemm<T, TOut, 64, 128, 8, 1, 4, 2>(a, groups, st);
    // deeper prefetch
    case 25: return launchIgemm<T, TOut, 128, 128, 4, 2, 2, 4>(a, groups, st);
    case 26: return launchIgemm<T, TOut, 256, 128, 4, 2, 2, 6>(a, groups, st);
    case 27: return launchIgemm<T, TOut, 128, 128, 8, 2, 2, 4>(a, groups, st);
    case 28: return launchIgemm<T, TOut, 128, 128, 4, 2, 2, 5>(a, groups, st);
    // small tiles at high occupancy for bandwidth-bound short-K layers
    case 29: return launchIgemm<T, TOut, 64, 128, 4, 1, 4, 2>(a, groups, st);
    case 30: return launchIgemm<T, TOut, 64, 64, 4, 2, 2, 2>(a, groups, st);
    case 31: return launchIgemm<T, TOut, 128, 64, 4, 2, 2, 2>(a, groups, st);
    // eight wavefronts (512 threads, two per SIMD): a second wave per SIMD covers the first one's barrier and LDS waits where
    // the launch has at most one workgroup per CU; pixel tiles of 192 and 96 bring the tile count of the 76x76 and 38x38
    // layers at batch 8 just under the CU count (241 and 242 tiles instead of 361 and 182)
    case 32: return launchIgemm<T, TOut, 256, 128, 8, 4, 2, 3>(a, groups, st);
    case 33: return launchIgemm<T, TOut, 128, 128, 8, 2, 4, 4>(a, groups, st);
    case 34: return launchIgemm<T, TOut, 256, 192, 8, 4, 2, 2>(a, groups, st);
    case 35: return launchIgemm<T, TOut, 256, 192, 4, 4, 2, 4>(a, groups, st);
    case 36: return launchIgemm<T, TOut, 256, 96, 8, 8, 1, 3>(a, groups, st);
    // twelve wavefronts (768 threads, three per SIMD) over 192-pixel tiles: 64 x 64 and 32 x 64 wave tiles
    case 37: return launchIgemm<T, TOut, 256, 192, 8, 4, 3, 2>(a, groups, st);
    case 38: return launchIgemm<T, TOut, 128, 192, 8, 4, 3, 3>(a, groups, st);
    // the LDS-patch kernel with eight wavefronts
    case 39: return launchPatch<T, TOut, 128, 384, 4, 2, 4, 1>(a, groups, st);
    case 40: return launchIgemm<T, TOut, 128, 128, 8, 2, 4, 3>(a, groups, st);
    // 64 channels x 256 pixels with eight wavefronts side by side, for the first layers of the detectors (32 -> 64 channels)
    case 41: return launchIgemm<T, TOut, 64, 256, 4, 1, 8, 3>(a, groups, st);
    // 128 channels x 384 pixels with twelve wavefronts: one round of tiles for 128-filter layers over many pixels
    case 42: return launchIgemm<T, TOut, 128, 384, 8, 2, 6, 2>(a, groups, st);
    // 3x3 stride-1 pad-1 only: input patch resident in LDS with 128-byte rows (last three numbers: wavefront grid rows x columns,
    // weight stages, patch slices per wavefront and tap step)
    case 43: return launchPatch8<T, TOut, 128, 192, 4, 3, 3, 1>(a, groups, st);
    case 44: return launchPatch8<T, TOut, 128, 192, 4, 2, 4, 1>(a, groups, st);
    case 45: return launchPatch8<T, TOut, 128, 192, 2, 2, 4, 2>(a, groups, st);
    case 46: return launchPatch8<T, TOut, 64, 384, 2, 6, 3, 1>(a, groups, st);
    case 47: return launchPatch8<T, TOut, 64, 384, 2, 4, 4, 2>(a, groups, st);
    case 48: return launchPatch8<T, TOut, 64, 256, 2, 4, 4, 1>(a, groups, st);
    case 49: return launchPatch8<T, TOut, 128, 256, 4, 2, 3, 1>(a, groups, st);
    case 50: return launchPatch8<T, TOut, 64, 192, 2, 2, 4, 2>(a, groups, st);
    case 51: return launchPatch8<T, TOut, 128, 384, 2, 4, 3, 2>(a, groups, st);
    // the same with the k-blocks of a tap step split between two groups of wavefronts over 64 x 64 wave tiles (the numbers are
    // the grid of wave tiles; twice as many wavefronts run)
    case 52: return launchPatch8<T, TOut, 64, 384, 1, 6, 3, 1, 0, 2>(a, groups, st);
    case 53: return launchPatch8<T, TOut, 128, 192, 2, 3, 3, 1, 0, 2>(a, groups, st);
    case 54: return launchPatch8<T, TOut, 64, 256, 1, 4, 4, 1, 0, 2>(a, groups, st);
    case 55: return launchPatch8<T, TOut, 128, 128, 2, 2, 4, 1, 0, 2>(a, groups, st);
    case 56: return launchPatch8<T, TOut, 64, 384, 1, 6, 4, 1, 0, 2>(a, groups, st);
    // the generic kernel with the same split (numbers: tile, 16-byte vectors of K per step, grid of 64 x 64 wave tiles, LDS stages)
    case 57: return launchIgemm<T, TOut, 128, 192, 8, 2, 3, 3, 2>(a, groups, st);
    case 58: return launchIgemm<T, TOut, 128, 128, 8, 2, 2, 4, 2>(a, groups, st);
    case 59: return launchIgemm<T, TOut, 64, 128, 8, 1, 2, 4, 2>(a, groups, st);
    case 60: return launchIgemm<T, TOut, 128, 64, 8, 2, 1, 4, 2>(a, groups, st);
    case 61: return launchIgemm<T, TOut, 64, 256, 8, 1, 4, 3, 2>(a, groups, st);
    case 62: return launchIgemm<T, TOut, 64, 384, 8, 1, 6, 2, 2>(a, groups, st);
    // the LDS-patch kernel over 256 channels x 192 pixels with twelve wavefronts: one round of tiles for the 76x76 128 -> 256 layers at batch 8
    // like tile 37, with a third fewer bytes delivered to LDS per tap step.  It fits the LDS with two weight stages only, the weight
    // tile of step it + 2 asked for behind the barrier of step it (see LATE in conv_patch8.hpp)
    case 63: return launchPatch8<T, TOut, 256, 192, 4, 3, 2, 1>(a, groups, st);
    // tiles whose epilogue also computes the 1x1 convolution that follows (msnh_hip_conv2d_tail only; float16): the tile holds every
    // output channel of the first convolution (at most 256 / 128)
    case 64:
    case 65:
        if constexpr (std::is_same<T, f16>::value && std::is_same<TOut, f16>::value)
        {
            if (tile == 64) return launchIgemm<T, TOut, 256, 192, 8, 4, 3, 2, 1, 1>(a, groups, st);
            return launchIgemm<T, TOut, 128, 192, 8, 4, 3, 2, 1, 1>(a, groups, st);
        }
        else
        {
            setError("conv2d: this tile needs float16 tensors and a 1x1 convolution behind it (msnh_hip_conv2d_tail)");
            return 3;
        }
    default: break;
    }
    setError("igemm: unknown tile %d", tile);
    return 2;
}

int igemmF16F16(IgemmArgs &a, int groups, int tile, hipStream_t st);
int igemmF16F32(IgemmArgs &a, int groups, int tile, hipStream_t st);
int igemmF32F32(IgemmArgs &a, int groups, int tile, hipStream_t st);

} // namespace msnh
