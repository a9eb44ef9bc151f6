// Implicit-GEMM convolution on the gfx950 matrix cores.
//
// GEMM view per group:  D[m][p] = sum_k W[m][k] * X[k][p]
//     m = output channel (rows, operand A = packed weights [out_c][tap][cin_g], K contiguous)
//     p = output pixel over the whole batch, p = (b*OH + oy)*OW + ox (columns, operand B)
//     k = (tap, channel); the B operand is gathered on the fly from the NHWC input: for one tap the
//         cin_g channels of an input pixel are contiguous, so a 16-byte vector load per lane feeds the
//         MFMA operand registers without any transposition.
// A workgroup of 256 threads (4 wavefronts in a WM x WN grid) owns a BM x BN tile of D.  Per K step each
// thread moves 16-byte vectors global -> registers -> LDS (two LDS buffers, one barrier per step) while
// the wavefronts issue 32x32 MFMA blocks from the other buffer.  LDS rows are padded by 16 bytes so the
// 128-bit fragment reads of 8 neighbouring lanes fall into distinct banks.
// The epilogue applies folded batch-norm / bias, activation, residual add + second activation and the
// power-of-two output scale on the float32 accumulators and stores 4 consecutive channels per lane.
#pragma once
#include "common.hpp"

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
    int act, act2, hasRes, vecOk;
    float actParam, act2Param, resMul, outMul;
};

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

// Shared epilogue of the GEMM-shaped convolution kernels:
// 1. folded batch-norm / bias + activation on the float32 accumulators, in registers;
// 2. each wavefront stages its TM x TN sub-tile as float32 in LDS, pixel-major (the main loop's LDS is free after
//    its last barrier), so that
// 3. every lane then owns 8 consecutive channels of a pixel: 16-byte residual loads and output stores, 8 lanes
//    covering a contiguous run of 64 channels.
template <typename T, typename TOut, int TM, int TN>
__device__ __forceinline__ void igemmEpilogue(const IgemmArgs &a, f32x16 (&acc)[TM / 32][TN / 32], unsigned char *smemRaw, int m0, int p0,
                                              int wm, int wn, int wave, int lane, int g)
{
    constexpr int MB = TM / 32;
    constexpr int NB = TN / 32;
    constexpr int LDE = TM + 4;                       // padded staging row (floats)
    float *stage = reinterpret_cast<float *>(smemRaw) + wave * (TN * LDE);
    const int chBase = g * a.coutG;
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
        for (int i = 0; i < MB; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int ml = i * 32 + q * 8 + (lane >> 5) * 4;           // channel inside the wave tile
                const int m = m0 + wm * TM + ml;
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    const int ch = chBase + m + e;
                    const bool ok = m + e < a.coutG;
                    const float sc = (ok && a.scale) ? a.scale[ch] : 1.f;
                    const float sh = (ok && a.shift) ? a.shift[ch] : 0.f;
                    v[e] = activate(acc[i][j][q * 4 + e] * sc + sh, a.act, a.actParam);
                }
                *reinterpret_cast<f32x4 *>(stage + (j * 32 + (lane & 31)) * LDE + ml) = v;
            }
    __syncthreads();

    const T *resg = static_cast<const T *>(a.res);
    TOut    *yg   = static_cast<TOut *>(a.y);
    constexpr int VPR = TM / 8;                       // 8-channel vectors per staged row
    constexpr int RPI = 64 / VPR;                     // rows covered per pass of the wave
    const int vcol = (lane % VPR) * 8;
    const int mv   = m0 + wm * TM + vcol;             // first channel of this lane's vector (within the group)
    if (mv < a.coutG)
    {
        const bool full = a.vecOk && (mv + 7 < a.coutG);
#pragma unroll
        for (int t = 0; t < TN / RPI; ++t)
        {
            const int row = t * RPI + lane / VPR;
            const int p = p0 + wn * TN + row;
            if (p >= a.P) continue;
            float v[8];
            const f32x4 lo = *reinterpret_cast<const f32x4 *>(stage + row * LDE + vcol);
            const f32x4 hi = *reinterpret_cast<const f32x4 *>(stage + row * LDE + vcol + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
            const size_t ch = static_cast<size_t>(chBase + mv);
            if (a.hasRes)
            {
                const T *rp = resg + static_cast<size_t>(p) * a.resLd + ch;
                if (full)
                {
                    typedef T ResV __attribute__((ext_vector_type(8)));
                    const ResV r = *reinterpret_cast<const ResV *>(rp);
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = activate(v[e] + a.resMul * toF(r[e]), a.act2, a.act2Param);
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (mv + e < a.coutG) v[e] = activate(v[e] + a.resMul * toF(rp[e]), a.act2, a.act2Param);
                }
            }
            TOut *yp = yg + static_cast<size_t>(p) * a.outLd + ch;
            if (full)
            {
                typedef TOut OutV __attribute__((ext_vector_type(8)));
                OutV o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = fromF<TOut>(a.outMul * v[e]);
                *reinterpret_cast<OutV *>(yp) = o;
            }
            else
            {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (mv + e < a.coutG) yp[e] = fromF<TOut>(a.outMul * v[e]);
            }
        }
    }
}

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN>
__global__ __launch_bounds__(256) void convIgemmKernel(IgemmArgs a)
{
    typedef typename Frag<T>::V V;
    constexpr int VEC   = Frag<T>::VEC;
    constexpr int BK    = KV * VEC;               // K elements per step
    constexpr int LDK   = BK + VEC;               // padded LDS row (elements)
    constexpr int RPP   = 256 / KV;               // rows loaded per pass
    constexpr int AROWS = (BM + RPP - 1) / RPP;   // A rows per thread (BM < RPP: only some threads load A)
    constexpr int BROWS = BN / RPP;               // B rows per thread
    constexpr int TM    = BM / WM;                // wave tile
    constexpr int TN    = BN / WN;
    constexpr int MB    = TM / 32;
    constexpr int NB    = TN / 32;
    constexpr int KBLK  = KV / 2;                 // k-blocks per step
    static_assert((BM % RPP == 0 || BM < RPP) && BN % RPP == 0, "tile rows must be a multiple of rows per pass");
    static_assert(TM % 32 == 0 && TN % 32 == 0 && WM * WN == 4, "wave grid");

    extern __shared__ __attribute__((aligned(16))) unsigned char smemRaw[];
    T *As = reinterpret_cast<T *>(smemRaw);                       // [2][BM][LDK]
    T *Bs = As + 2 * BM * LDK;                                    // [2][BN][LDK]

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm   = wave / WN;
    const int wn   = wave % WN;
    const int g    = blockIdx.z;
    // Workgroup -> tile mapping.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its own
    // L2.  Ids are therefore first regrouped per XCD (id % 8 selects the XCD, id / 8 the position inside it), and
    // inside an XCD the channel tiles of one pixel tile run back to back, so an input pixel is fetched into one L2
    // once instead of once per channel tile and XCD.
    const int nTilesP = (a.P + BN - 1) / BN;
    const int total   = a.mTiles * nTilesP;
    const int perXcd  = (total + 7) / 8;
    const int logical = (blockIdx.x % 8) * perXcd + blockIdx.x / 8;
    if (logical >= total) return;                     // padding ids of the last round
    const int m0   = (logical % a.mTiles) * BM;
    const int p0   = (logical / a.mTiles) * BN;

    const T *xg = static_cast<const T *>(a.x) + static_cast<size_t>(g) * a.cinG;
    const T *wg = static_cast<const T *>(a.w) + static_cast<size_t>(g) * a.coutG * a.taps * a.cinG;

    const int ldRow = tid / KV;
    const int ldVec = tid % KV;

    // per-thread row metadata, fixed over the K loop
    int    bIy0[BROWS], bIx0[BROWS];
    size_t bBase[BROWS];
    bool   bOk[BROWS];
#pragma unroll
    for (int i = 0; i < BROWS; ++i)
    {
        const int p = p0 + ldRow + i * RPP;
        bOk[i] = p < a.P;
        const int pp = bOk[i] ? p : 0;
        const int ox = pp % a.OW;
        const int t  = pp / a.OW;
        const int oy = t % a.OH;
        const int b  = t / a.OH;
        bIy0[i]  = oy * a.stride - a.pad;
        bIx0[i]  = ox * a.stride - a.pad;
        bBase[i] = static_cast<size_t>(b) * a.H * a.W;
    }
    size_t aBase[AROWS];
    bool   aOk[AROWS];
#pragma unroll
    for (int i = 0; i < AROWS; ++i)
    {
        const int m = m0 + ldRow + i * RPP;
        aOk[i]   = m < a.coutG && (ldRow + i * RPP) < BM;
        aBase[i] = static_cast<size_t>(aOk[i] ? m : 0) * a.taps * a.cinG;
    }

    V regA[AROWS], regB[BROWS];

    auto loadGlobal = [&](int it) {
        const int tap = it / a.cChunks;
        const int c   = (it - tap * a.cChunks) * BK + ldVec * VEC;
        const bool cOk = c < a.cinG;
        const int ki = tap / a.ksize;
        const int kj = tap - ki * a.ksize;
#pragma unroll
        for (int i = 0; i < AROWS; ++i)
        {
            V v = {0};
            if (aOk[i] && cOk)
                v = *reinterpret_cast<const V *>(wg + aBase[i] + static_cast<size_t>(tap) * a.cinG + c);
            regA[i] = v;
        }
#pragma unroll
        for (int i = 0; i < BROWS; ++i)
        {
            const int iy = bIy0[i] + ki * a.dil;
            const int ix = bIx0[i] + kj * a.dil;
            V v = {0};
            if (bOk[i] && cOk && iy >= 0 && iy < a.H && ix >= 0 && ix < a.W)
                v = *reinterpret_cast<const V *>(xg + (bBase[i] + static_cast<size_t>(iy) * a.W + ix) * a.inLd + c);
            regB[i] = v;
        }
    };

    auto storeLds = [&](int buf) {
        T *ad = As + buf * BM * LDK;
        T *bd = Bs + buf * BN * LDK;
#pragma unroll
        for (int i = 0; i < AROWS; ++i)
            if (BM % RPP == 0 || ldRow + i * RPP < BM)
                *reinterpret_cast<V *>(ad + (ldRow + i * RPP) * LDK + ldVec * VEC) = regA[i];
#pragma unroll
        for (int i = 0; i < BROWS; ++i)
            *reinterpret_cast<V *>(bd + (ldRow + i * RPP) * LDK + ldVec * VEC) = regB[i];
    };

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    loadGlobal(0);
    storeLds(0);
    __syncthreads();

    const int fragRow = lane & 31;
    const int fragCol = (lane >> 5) * VEC;

    for (int it = 0; it < a.nIter; ++it)
    {
        const int buf = it & 1;
        if (it + 1 < a.nIter) loadGlobal(it + 1);

        const T *ab = As + buf * BM * LDK + (wm * TM + fragRow) * LDK + fragCol;
        const T *bb = Bs + buf * BN * LDK + (wn * TN + fragRow) * LDK + fragCol;
#pragma unroll
        for (int kb = 0; kb < KBLK; ++kb)
        {
            V fa[MB], fb[NB];
#pragma unroll
            for (int i = 0; i < MB; ++i) fa[i] = *reinterpret_cast<const V *>(ab + i * 32 * LDK + kb * 2 * VEC);
#pragma unroll
            for (int j = 0; j < NB; ++j) fb[j] = *reinterpret_cast<const V *>(bb + j * 32 * LDK + kb * 2 * VEC);
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) mfmaBlock(fa[i], fb[j], acc[i][j]);
        }

        if (it + 1 < a.nIter) storeLds(buf ^ 1);
        __syncthreads();
    }

    igemmEpilogue<T, TOut, TM, TN>(a, acc, smemRaw, m0, p0, wm, wn, wave, lane, g);
}

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN>
inline int launchIgemm(IgemmArgs &a, int groups, hipStream_t st)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int BK  = KV * VEC;
    constexpr int LDK = BK + VEC;
    a.cChunks = (a.cinG + BK - 1) / BK;
    a.nIter   = a.taps * a.cChunks;
    const size_t smemLoop = static_cast<size_t>(2) * (BM + BN) * LDK * sizeof(T);
    const size_t smemEpi  = static_cast<size_t>(4) * (BN / WN) * (BM / WM + 4) * sizeof(float);
    const size_t smem = smemLoop > smemEpi ? smemLoop : smemEpi;
    a.mTiles = (a.coutG + BM - 1) / BM;
    const int tiles = a.mTiles * ((a.P + BN - 1) / BN);
    dim3 grid((tiles + 7) / 8 * 8, 1, groups);
    if (a.dryRun) return 0;
    auto kern = convIgemmKernel<T, TOut, BM, BN, KV, WM, WN>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh

#include "conv_patch.hpp"

namespace msnh {

// Tile configurations (BM x BN output tile, KV 16-byte vectors of K per step, WM x WN wavefront grid).
// Index 0 is "choose for me"; the others can be forced through msnh_conv_desc::tile, which is how the host
// library's per-layer search picks the fastest one at load time.
constexpr int kIgemmTiles = 19;

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
    case 6:  return launchIgemm<T, TOut, 32, 256, 4, 1, 4>(a, groups, st);
    case 7:  return launchIgemm<T, TOut, 256, 128, 4, 2, 2>(a, groups, st);
    case 8:  return launchIgemm<T, TOut, 128, 64, 8, 2, 2>(a, groups, st);
    case 9:  return launchIgemm<T, TOut, 128, 64, 4, 2, 2>(a, groups, st);
    case 10: return launchIgemm<T, TOut, 64, 128, 8, 1, 4>(a, groups, st);
    case 11: return launchIgemm<T, TOut, 64, 128, 4, 1, 4>(a, groups, st);
    case 12: return launchIgemm<T, TOut, 64, 64, 8, 2, 2>(a, groups, st);
    case 13: return launchIgemm<T, TOut, 256, 128, 8, 2, 2>(a, groups, st);
    // 3x3 stride-1 pad-1 only: input patch resident in LDS, weights streamed per tap
    case 14: return launchPatch<T, TOut, 128, 128, 8, 2, 2>(a, groups, st);
    case 15: return launchPatch<T, TOut, 128, 128, 4, 2, 2>(a, groups, st);
    case 16: return launchPatch<T, TOut, 64, 128, 8, 1, 4>(a, groups, st);
    case 17: return launchPatch<T, TOut, 64, 128, 4, 1, 4>(a, groups, st);
    case 18: return launchPatch<T, TOut, 256, 128, 4, 2, 2>(a, groups, st);
    case 19: return launchPatch<T, TOut, 128, 64, 8, 2, 2>(a, groups, st);
    default: break;
    }
    setError("igemm: unknown tile %d", tile);
    return 2;
}

int igemmF16F16(IgemmArgs &a, int groups, int tile, hipStream_t st);
int igemmF16F32(IgemmArgs &a, int groups, int tile, hipStream_t st);
int igemmF32F32(IgemmArgs &a, int groups, int tile, hipStream_t st);

} // namespace msnh
