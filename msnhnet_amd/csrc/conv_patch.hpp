// 3x3 stride-1 pad-1 convolution with the input patch resident in LDS.
//
// The generic implicit GEMM gathers the B operand (pixels x K) from global memory once per filter tap, so every
// input pixel crosses the L2 -> CU path nine times per channel tile.  Here a tile of BN consecutive output pixels
// (flattened over the batch) stages the contiguous run of BN + 2W + 2 input pixels it can touch -- one row above,
// one below, one pixel either side -- ONCE per channel chunk; the nine taps then read their operand fragments
// from that patch at a row offset of ti*W + tj, with lanes whose tap falls outside the image zeroed.  Only the
// weight tile of the current (chunk, tap) is streamed per step.  The next chunk's patch is brought in in eight
// slices interleaved with the tap steps (second LDS buffer), the next weight tile one step ahead.
#pragma once
#include "conv_igemm.hpp"

namespace msnh {

constexpr int kPatchSliceMax = 3;       // patch vectors a thread moves per tap step (upper bound)

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN>
__global__ __launch_bounds__(256) void convPatch3x3Kernel(IgemmArgs a)
{
    typedef typename Frag<T>::V V;
    constexpr int VEC  = Frag<T>::VEC;
    constexpr int BK   = KV * VEC;
    constexpr int LDK  = BK + VEC;
    constexpr int TM   = BM / WM;
    constexpr int TN   = BN / WN;
    constexpr int MB   = TM / 32;
    constexpr int NB   = TN / 32;
    constexpr int KBLK = KV / 2;
    constexpr int AV   = BM * KV / 256;           // weight vectors per thread per step
    static_assert(BM * KV % 256 == 0 && TM % 32 == 0 && TN % 32 == 0 && WM * WN == 4, "tile shape");

    extern __shared__ __attribute__((aligned(16))) unsigned char smemRaw[];
    const int R = a.patchRows;
    T *Ps = reinterpret_cast<T *>(smemRaw);               // [2][R][LDK]
    T *As = Ps + 2 * R * LDK;                              // [2][BM][LDK]

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm   = wave / WN;
    const int wn   = wave % WN;
    const int nTilesP = (a.P + BN - 1) / BN;
    const int total   = a.mTiles * nTilesP;
    const int perXcd  = (total + 7) / 8;
    const int logical = (blockIdx.x % 8) * perXcd + blockIdx.x / 8;
    if (logical >= total) return;
    const int m0 = (logical % a.mTiles) * BM;
    const int p0 = (logical / a.mTiles) * BN;

    float chScale, chShift;
    loadChannelAffine(a, 0, m0, tid, BM, chScale, chShift);

    const T *xg = static_cast<const T *>(a.x);
    const T *wg = static_cast<const T *>(a.w);
    const int W = a.W, H = a.H;
    const int q0 = p0 - W - 1;                            // input pixel held by patch row 0
    const int PV = R * KV;                                // vectors per patch chunk
    const int SV = (PV + 7) / 8;                          // vectors per slice

    // ---- loaders ----------------------------------------------------------------------------------------
    auto patchVec = [&](int idx, int chunk) -> V {
        const int r = idx / KV, v = idx - r * KV;
        const int q = q0 + r;
        const int c = chunk * BK + v * VEC;
        V val = {0};
        if (q >= 0 && q < a.P && c < a.cinG) val = *reinterpret_cast<const V *>(xg + static_cast<size_t>(q) * a.inLd + c);
        return val;
    };
    auto patchDst = [&](int idx, int buf) -> V * {
        const int r = idx / KV, v = idx - r * KV;
        return reinterpret_cast<V *>(Ps + (static_cast<size_t>(buf) * R + r) * LDK + v * VEC);
    };
    V regA[AV], regP[kPatchSliceMax];
    auto loadA = [&](int it) {
        const int chunk = it / 9, tap = it - chunk * 9;
#pragma unroll
        for (int i = 0; i < AV; ++i)
        {
            const int va = tid + i * 256;
            const int row = va / KV, v = va - row * KV;
            const int m = m0 + row;
            const int c = chunk * BK + v * VEC;
            V val = {0};
            if (m < a.coutG && c < a.cinG) val = *reinterpret_cast<const V *>(wg + (static_cast<size_t>(m) * 9 + tap) * a.cinG + c);
            regA[i] = val;
        }
    };
    auto storeA = [&](int buf) {
#pragma unroll
        for (int i = 0; i < AV; ++i)
        {
            const int va = tid + i * 256;
            const int row = va / KV, v = va - row * KV;
            *reinterpret_cast<V *>(As + (buf * BM + row) * LDK + v * VEC) = regA[i];
        }
    };
    auto loadSlice = [&](int slice, int chunk) {
        const int end = (slice + 1) * SV < PV ? (slice + 1) * SV : PV;
#pragma unroll
        for (int j = 0; j < kPatchSliceMax; ++j)
        {
            const int idx = slice * SV + tid + j * 256;
            V val = {0};
            if (idx < end) val = patchVec(idx, chunk);
            regP[j] = val;
        }
    };
    auto storeSlice = [&](int slice, int buf) {
        const int end = (slice + 1) * SV < PV ? (slice + 1) * SV : PV;
#pragma unroll
        for (int j = 0; j < kPatchSliceMax; ++j)
        {
            const int idx = slice * SV + tid + j * 256;
            if (idx < end) *patchDst(idx, buf) = regP[j];
        }
    };

    // ---- per-lane pixel metadata for the B fragments -----------------------------------------------------------
    int  nLocal[NB], oy[NB], ox[NB];
    bool pOk[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j)
    {
        nLocal[j] = wn * TN + j * 32 + (lane & 31);
        const int p = p0 + nLocal[j];
        pOk[j] = p < a.P;
        const int pp = pOk[j] ? p : 0;
        ox[j] = pp % W;
        oy[j] = (pp / W) % H;
    }

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // ---- prologue: whole patch of chunk 0, weight tile of step 0 -------------------------------------------------------
    for (int idx = tid; idx < PV; idx += 256) *patchDst(idx, 0) = patchVec(idx, 0);
    loadA(0);
    storeA(0);
    __syncthreads();

    const int fragRow = lane & 31;
    const int fragCol = (lane >> 5) * VEC;
    const int chunks = a.cChunks;

    for (int it = 0; it < a.nIter; ++it)
    {
        const int chunk = it / 9, tap = it - chunk * 9;
        const int ti = tap / 3, tj = tap - ti * 3;
        const bool moreChunks = chunk + 1 < chunks;
        if (it + 1 < a.nIter) loadA(it + 1);
        if (moreChunks && tap < 8) loadSlice(tap, chunk + 1);

        const T *ab = As + ((it & 1) * BM + wm * TM + fragRow) * LDK + fragCol;
        const T *pb = Ps + static_cast<size_t>(chunk & 1) * R * LDK + static_cast<size_t>(ti * W + tj) * LDK + fragCol;
        bool ok[NB];
#pragma unroll
        for (int j = 0; j < NB; ++j)
            ok[j] = pOk[j] && static_cast<unsigned>(oy[j] + ti - 1) < static_cast<unsigned>(H) &&
                    static_cast<unsigned>(ox[j] + tj - 1) < static_cast<unsigned>(W);
#pragma unroll
        for (int kb = 0; kb < KBLK; ++kb)
        {
            V fa[MB], fb[NB];
#pragma unroll
            for (int i = 0; i < MB; ++i) fa[i] = *reinterpret_cast<const V *>(ab + i * 32 * LDK + kb * 2 * VEC);
#pragma unroll
            for (int j = 0; j < NB; ++j)
            {
                V v = *reinterpret_cast<const V *>(pb + static_cast<size_t>(nLocal[j]) * LDK + kb * 2 * VEC);
                if (!ok[j]) v = V{0};
                fb[j] = v;
            }
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) mfmaBlock(fa[i], fb[j], acc[i][j]);
        }

        if (it + 1 < a.nIter) storeA((it + 1) & 1);
        if (moreChunks && tap < 8) storeSlice(tap, (chunk + 1) & 1);
        __syncthreads();
    }

    igemmEpilogue<T, TOut, BM, BN, TM, TN>(a, acc, smemRaw, chScale, chShift, m0, p0, wm, wn, wave, lane, 0);
}

// Host-side check shared by launch and tile enumeration.
template <typename T, int BM, int BN, int KV, int WM, int WN>
inline bool patchFits(const IgemmArgs &a, size_t *smemOut)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int LDK = KV * VEC + VEC;
    const int R = BN + 2 * a.W + 2;
    const size_t loop = (static_cast<size_t>(2) * R + 2 * BM) * LDK * sizeof(T);
    const size_t epi = igemmEpilogueLds<BM, BM / WM>();
    const size_t smem = loop > epi ? loop : epi;
    if (smemOut) *smemOut = smem;
    const int sv = (R * KV + 7) / 8;
    return a.patchOk && smem <= 160 * 1024 && (sv + 255) / 256 <= kPatchSliceMax;
}

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN>
inline int launchPatch(IgemmArgs &a, int groups, hipStream_t st)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int BK  = KV * VEC;
    size_t smem = 0;
    if (groups != 1 || !patchFits<T, BM, BN, KV, WM, WN>(a, &smem))
    {
        setError("conv2d: this tile needs a 3x3 stride-1 pad-1 ungrouped convolution whose input patch fits in LDS");
        return 3;
    }
    if (a.dryRun) return 0;
    a.patchRows = BN + 2 * a.W + 2;
    a.cChunks = (a.cinG + BK - 1) / BK;
    a.nIter   = 9 * a.cChunks;
    a.ragged  = (a.cinG % BK) != 0;
    a.mTiles  = (a.coutG + BM - 1) / BM;
    const int tiles = a.mTiles * ((a.P + BN - 1) / BN);
    dim3 grid((tiles + 7) / 8 * 8, 1, 1);
    auto kern = convPatch3x3Kernel<T, TOut, BM, BN, KV, WM, WN>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, grid, dim3(256), smem, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
