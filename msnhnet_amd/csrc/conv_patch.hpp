// 3x3 stride-1 pad-1 convolution with the input patch resident in LDS.
//
// The generic implicit GEMM gathers the B operand (pixels x K) from global memory once per filter tap, so every
// input pixel crosses the L2 -> CU path nine times per channel chunk, and it is the L2's request rate, not the
// matrix cores, that bounds those kernels.  Here a tile of BN consecutive output pixels (flattened over the
// batch) stages the contiguous run of R = BN + 2W + 2 input pixels it can touch -- one image row above, one
// below, one pixel either side -- ONCE per channel chunk; the nine taps then read their operand fragments from
// that patch at a row offset of ky*W + kx, and lanes whose tap falls outside the image read a zero chunk instead.
// Only the weight tile of the current (chunk, tap) is streamed per step.
//
// Data movement is the implicit GEMM's: 16-byte-per-lane buffer loads straight into LDS, XOR-swizzled unpadded
// rows, three rotating stages for the weight tile.  The patch has two stages; the patch of chunk c+1 arrives in
// 1 KiB slices (one wave instruction each), PS per wave and tap step over taps 0..7 of chunk c.  Every step
// issues the same number of loads per wave -- slices that do not exist go, out of range and therefore as
// zeros without touching memory, into a 1 KiB dump area that doubles as the zero chunk -- so the count of loads
// in flight at each barrier is a compile-time constant.
#pragma once
#include "conv_igemm.hpp"

namespace msnh {

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN, int PS>
__global__ __launch_bounds__(64 * WM * WN) __attribute__((amdgpu_waves_per_eu(2, 2)))
void convPatch3x3Kernel(IgemmArgs a)
{
    typedef typename Frag<T>::V V;
    constexpr int VEC   = Frag<T>::VEC;
    constexpr int BK    = KV * VEC;
    constexpr int NW    = WM * WN;                // wavefronts: 4 or 8
    constexpr int RPP   = 64 * NW / KV;
    constexpr int AL    = BM / RPP;               // weight loads per thread per step
    constexpr int NL    = AL + PS;                // loads per thread per step
    constexpr int TM    = BM / WM;
    constexpr int TN    = BN / WN;
    constexpr int MB    = TM / 32;
    constexpr int NB    = TN / 32;
    constexpr int S     = KV / 2;
    constexpr unsigned ES = sizeof(T);
    constexpr int ROWB  = KV * 16;
    constexpr int SWDIV = 16 / KV;
    constexpr unsigned A_STAGE = BM * ROWB;
    constexpr int RPS   = 64 / KV;                // patch rows per 1 KiB slice
    static_assert(KV == 4 && S == 2, "the slice arithmetic below assumes 64-byte rows");
    static_assert(BM % RPP == 0 && TM % 32 == 0 && TN % 32 == 0 && (NW == 4 || NW == 8), "tile shape");

    extern __shared__ __attribute__((aligned(16))) unsigned char smemRaw[];
    const unsigned ldsBase = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)smemRaw));
    // LDS: three weight stages | patch stage 0 | patch stage 1 | dump / zero area (1 KiB)
    const int nSlices = a.patchRows;              // 1 KiB slices per patch stage (host: ceil(R * KV / 64))
    const unsigned patchBytes = static_cast<unsigned>(nSlices) * 1024u;
    const unsigned patchOff0 = 3 * A_STAGE;
    const unsigned dumpOff = patchOff0 + 2 * patchBytes;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm   = wave / WN;
    const int wn   = wave % WN;
    int mTile, pTile;
    if (!igemmTileOf(a, (a.P + BN - 1) / BN, mTile, pTile)) return;
    const int m0 = mTile * BM;
    const int p0 = pTile * BN;

    const i32x4 rx = makeRsrcWords(a.x, a.xBytes);
    const i32x4 rw = makeRsrcWords(a.w, a.wBytes);

    float chScale, chShift;
    loadChannelAffine(a, 0, m0, tid, BM, chScale, chShift);

    if (tid < 64) *reinterpret_cast<f32x4 *>(smemRaw + dumpOff + tid * 16) = f32x4{0.f, 0.f, 0.f, 0.f};

    const int W = a.W, H = a.H;

    // ---- weight tile: thread tid owns chunk position tid % KV of row tid / KV (+ RPP rows per load) -----------
    const int ldRow = tid / KV;
    const int ldVec = (tid % KV) ^ ((ldRow / SWDIV) % KV);
    unsigned aOff[AL];
#pragma unroll
    for (int i = 0; i < AL; ++i)
    {
        const int m = m0 + ldRow + i * RPP;
        aOff[i] = m < a.coutG ? (static_cast<unsigned>(m) * 9u * a.cinG + ldVec * VEC) * ES : kOobOffset;
    }
    // ---- patch: slice s holds patch rows s*RPS .. s*RPS+RPS-1; lane l of the slice's load owns chunk position
    // l % KV of row s*RPS + l / KV, i.e. input pixel q0 + that row.  Pixels before the tensor give a negative
    // offset, which as unsigned is out of range like the pixels behind the tensor: zeros, no test needed.
    const int q0 = p0 - W - 1;                                  // input pixel of patch row 0
    const int pRow = lane / KV;
    const int pVec = (lane % KV) ^ ((pRow / SWDIV) % KV);       // (s*RPS + pRow) / SWDIV % KV does not depend on s
    const unsigned pBase = static_cast<unsigned>((static_cast<long long>(q0 + pRow) * a.inLd + pVec * VEC) * static_cast<long long>(ES));
    const unsigned sliceStride = static_cast<unsigned>(RPS) * a.inLd * ES;
    const unsigned waveDump = ldsBase + dumpOff;

    // slice number i of this wave (slices wave, wave+NW, ...) of the patch of channel chunk `chunk` into stage `st`
    auto issuePatch = [&](int i, int chunk, unsigned stOff) {
        const int s = wave + NW * i;
        const bool real = s < nSlices && chunk < a.cChunks;
        const bool cut = a.ragged && (chunk * BK + pVec * VEC >= a.cinG);
        const unsigned voff = (real && !cut) ? pBase + static_cast<unsigned>(s) * sliceStride : kOobOffset;
        dmaLoad16(rx, voff, static_cast<unsigned>(chunk * BK) * ES, real ? ldsBase + stOff + static_cast<unsigned>(s) * 1024u : waveDump);
    };
    const unsigned waveLds = ldsBase + wave * 1024;
    auto issueA = [&](auto lTag, unsigned sA, bool cut, unsigned stageOff) {
        constexpr int l = decltype(lTag)::value;
        dmaLoad16(rw, cut ? kOobOffset : aOff[l], sA, waveLds + stageOff + l * RPP * ROWB);
    };

    // ---- fragments ------------------------------------------------------------------------------------------
    const int fragRow = lane & 31;
    const int fragSw  = (fragRow / SWDIV) % KV;
    unsigned aAddr[S];
#pragma unroll
    for (int kb = 0; kb < S; ++kb) aAddr[kb] = wm * TM * ROWB + fragRow * ROWB + (((2 * kb + (lane >> 5)) ^ fragSw) * 16);
    // per 32-pixel block j of the wave tile: which of the nine taps lie inside the image for this lane's pixel
    unsigned tapOk[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j)
    {
        const int p = p0 + wn * TN + j * 32 + fragRow;
        unsigned m = 0;
        if (p < a.P)
        {
            const int t = static_cast<int>(fastDiv(static_cast<unsigned>(p), a.byOW));      // (same-size output: OW = W, OH = H)
            const int x = p - t * W;
            const int y = t - static_cast<int>(fastDiv(static_cast<unsigned>(t), a.byOH)) * H;
            const unsigned cols = (x > 0 ? 1u : 0u) | 2u | (x < W - 1 ? 4u : 0u);
            m = (y > 0 ? cols : 0u) | (cols << 3) | (y < H - 1 ? cols << 6 : 0u);
        }
        tapOk[j] = m;
    }
    const unsigned bRow0 = wn * TN + fragRow;     // patch row of this lane's pixel for tap (0,0), block 0

    V fa[2][MB], fb[2][NB];
    auto readA = [&](unsigned stageOff, auto kbTag) {
        constexpr int kb = decltype(kbTag)::value;
        const unsigned char *ap = smemRaw + (aAddr[kb] + stageOff);
#pragma unroll
        for (int i = 0; i < MB; ++i) fa[kb % 2][i] = *reinterpret_cast<const V *>(ap + i * 32 * ROWB);
    };
    // B fragments of tap `tap` from the patch stage at pOff
    auto readB = [&](unsigned pOff, int tap, auto kbTag) {
        constexpr int kb = decltype(kbTag)::value;
        const int ky = tap / 3;
        const unsigned row = bRow0 + static_cast<unsigned>(ky * W + (tap - 3 * ky));
        const unsigned sw = (row / SWDIV) % KV;   // rows 32 apart share it
        const unsigned addr = pOff + row * ROWB + (((2 * kb + (lane >> 5)) ^ sw) * 16);
        const unsigned bit = 1u << tap;
#pragma unroll
        for (int j = 0; j < NB; ++j)
        {
            const unsigned aj = (tapOk[j] & bit) ? addr + j * 32 * ROWB : dumpOff;
            fb[kb % 2][j] = *reinterpret_cast<const V *>(smemRaw + aj);
        }
    };

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    constexpr int PER = MB * NB;
    // all NL loads of a step are issued among the MFMAs of its first k-step, ahead of the barrier
    // ---- prologue: whole patch of chunk 0, weight tiles of steps 0 and 1 ----------------------------------------
    for (int i = 0; wave + NW * i < nSlices; ++i) issuePatch(i, 0, patchOff0);
    staticFor<0, AL>([&](auto lTag) { issueA(lTag, 0u, a.ragged && (ldVec * VEC >= a.cinG), 0u); });
    {
        const bool pastEnd = a.nIter < 2;         // never: nIter >= 9
        staticFor<0, AL>([&](auto lTag) { issueA(lTag, static_cast<unsigned>(a.cinG) * ES, pastEnd || (a.ragged && (ldVec * VEC >= a.cinG)), A_STAGE); });
    }
    dmaWait<0>();
    __syncthreads();
    readA(0, std::integral_constant<int, 0>());
    readB(patchOff0, 0, std::integral_constant<int, 0>());

    // step it = chunk * 9 + tap; weight stage of step it is (it % 3) * A_STAGE; patch stage of chunk is chunk % 2
    unsigned curA = 0, nxtA = A_STAGE, nnA = 2 * A_STAGE;
    unsigned curP = patchOff0, othP = patchOff0 + patchBytes;
    int tap = 0, chunk = 0;
    int tapL = 1, chunkL = 0;                     // (tap, chunk) of the step whose weight tile was issued last
    for (int it = 0; it < a.nIter; ++it)
    {
        // the weight tile of step it+2
        if (++tapL == 9) { tapL = 0; ++chunkL; }
        const unsigned sA = (static_cast<unsigned>(tapL) * a.cinG + chunkL * BK) * ES;
        const bool cutA = it + 2 >= a.nIter || (a.ragged && (chunkL * BK + ldVec * VEC >= a.cinG));
        // the next step's tap and patch stage
        const int tapN = tap == 8 ? 0 : tap + 1;
        const unsigned nextP = tap == 8 ? othP : curP;

        readA(curA, std::integral_constant<int, 1>());
        readB(curP, tap, std::integral_constant<int, 1>());
        __builtin_amdgcn_sched_barrier(0);
        staticFor<0, 2 * PER>([&](auto gTag) {
            constexpr int gi = decltype(gTag)::value;
            constexpr int ks = gi / PER;
            if constexpr (gi == PER)
            {
                dmaWait<NL>();                    // everything issued before this step has landed
                __syncthreads();
                readA(nxtA, std::integral_constant<int, 0>());
                readB(nextP, tapN, std::integral_constant<int, 0>());
                __builtin_amdgcn_sched_barrier(0);
            }
            mfmaBlock(fa[ks % 2][(gi % PER) / NB], fb[ks % 2][(gi % PER) % NB], acc[(gi % PER) / NB][(gi % PER) % NB]);
            if constexpr (gi < PER)
            {
                // loads l with l * PER / NL == gi: patch slices first, then the weight rows
                constexpr int first = (gi * NL + PER - 1) / PER;
                constexpr int last  = ((gi + 1) * NL + PER - 1) / PER;
                staticFor<first, last>([&](auto lTag) {
                    constexpr int l = decltype(lTag)::value;
                    if constexpr (l < PS)
                        issuePatch(tap == 8 ? (1 << 20) : tap * PS + l, chunk + 1, othP);
                    else
                        issueA(std::integral_constant<int, l - PS>(), sA, cutA, nnA);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        const unsigned t = curA;
        curA = nxtA;
        nxtA = nnA;
        nnA = t;
        if (tap == 8)
        {
            tap = 0;
            ++chunk;
            const unsigned tp = curP;
            curP = othP;
            othP = tp;
        }
        else
            ++tap;
    }
    dmaWait<0>();
    __syncthreads();

    igemmEpilogue<T, TOut, BM, BN, TM, TN>(a, acc, smemRaw, chScale, chShift, m0, p0, wm, wn, wave, lane, 0);
}

// Host-side check shared by launch and tile enumeration.
template <typename T, int BM, int BN, int KV, int WM, int WN, int PS>
inline bool patchFits(const IgemmArgs &a, size_t *smemOut, int *slicesOut)
{
    const int R = BN + 2 * a.W + 2;
    const int slices = (R * KV + 63) / 64;
    const size_t loop = static_cast<size_t>(3) * BM * KV * 16 + static_cast<size_t>(2) * slices * 1024 + 1024;
    const size_t epi = igemmEpilogueLds<BM, BM / WM, WM * WN>();
    const size_t smem = loop > epi ? loop : epi;
    if (smemOut) *smemOut = smem;
    if (slicesOut) *slicesOut = slices;
    // taps 0..7 of a chunk bring in the next patch: 8 * PS slices per wave
    return a.patchOk && a.buffersOk && smem <= 160 * 1024 && slices <= 8 * WM * WN * PS;
}

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN, int PS>
inline int launchPatch(IgemmArgs &a, int groups, hipStream_t st)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int BK  = KV * VEC;
    size_t smem = 0;
    int slices = 0;
    if (groups != 1 || a.splitMax > 1 || a.tailOn || !patchFits<T, BM, BN, KV, WM, WN, PS>(a, &smem, &slices))
    {
        setError("conv2d: this tile needs a 3x3 stride-1 pad-1 ungrouped convolution whose input patch fits in LDS");
        return 3;
    }
    if (a.dryRun) return 0;
    a.patchRows = slices;
    a.cChunks = (a.cinG + BK - 1) / BK;
    a.nIter   = 9 * a.cChunks;
    a.ragged  = (a.cinG % BK) != 0;
    a.mTiles  = (a.coutG + BM - 1) / BM;
    a.splitK  = 1;
    dim3 grid(igemmGridX(a, (a.P + BN - 1) / BN, sizeof(T), true), 1, 1);
    auto kern = convPatch3x3Kernel<T, TOut, BM, BN, KV, WM, WN, PS>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, grid, dim3(64 * WM * WN), smem, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
