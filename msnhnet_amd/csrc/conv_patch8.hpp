// 3x3 stride-1 pad-1 convolution with the input patch resident in LDS, 128-byte rows, 4 / 8 / 12 wavefronts.
//
// Why: the 3x3 layers of the detectors at 76x76 ... 19x19 are bound by what a CU can draw out of the L2 (about 20 bytes per
// clock and CU, measured), not by the matrix cores.  The generic implicit GEMM delivers (BM + BN) x 128 bytes to LDS per 64-deep
// K step and multiplies BM x BN x 64 with it; per filter tap it fetches the same input pixels again, shifted by one.  Here the
// run of BN + 2W + 2 input pixels that a tile of BN consecutive output pixels (flattened over the batch) can touch is delivered
// ONCE per 64-channel chunk and the nine taps read their B fragments from it at a row offset of ky*W + kx; only the weight tile
// (BM rows) streams per tap.  Bytes per MFMA fall by 2 - 2.8x against the generic kernel at the same tile, and the best shape
// moves to few channels x many pixels (the weights are what is left to stream, and they are amortised over the pixels).
// conv_patch.hpp is the same idea with 64-byte rows and four wavefronts; it loses to the generic kernel because its L2 requests
// are 64 bytes long (the L2 serves requests, not bytes), its weight tile arrives one step ahead only, and a single wavefront per
// SIMD has nothing to cover the barrier with.  This kernel differs in exactly those three points.
//
// LDS: NSA weight stages of BM x 128 B | patch of the current chunk | patch of the next chunk | 1 KiB of zeros.
// Data movement as in conv_igemm.hpp: 16-byte-per-lane buffer loads straight into LDS, XOR-swizzled unpadded rows, explicit
// vmcnt waits, one barrier per tap step.  The patch of chunk c+1 arrives in 1 KiB slices (8 pixels x 128 B, one wave
// instruction each), PS per wavefront and tap step over the first 11 - NSA taps of chunk c (8 with two weight stages); every tap step issues the same number
// of loads per wavefront (slices that do not exist go, out of range and therefore as zeros, into the zero area), so the count
// of loads in flight at each barrier is a compile-time constant.
#pragma once
#include "conv_igemm.hpp"

namespace msnh {

// DBG (timing experiments only, results are then meaningless; 0 in every instantiation the library ships): bit 0 leaves out the
// loads of the main loop, bit 1 its LDS fragment reads, bit 2 its barrier, bit 3 its MFMAs, bit 4 the epilogue, bit 5 the prologue's loads;
// bit 6 makes the first wavefront write the shader-clock and constant-clock ticks its main loop took to IgemmArgs::ws (two 64-bit words).
//
// KG = 2 splits the four k-blocks of every tap step between two groups of wavefronts that share the same WM x WN grid of wave
// tiles: a wavefront then owns a 64 x 64 tile over half of K instead of a 32 x 64 tile over all of it, which takes a third off
// the LDS fragment reads per MFMA (2 A + 2 B fragments per 4 MFMAs instead of 1 A + 2 B per 2); LDS is the busiest unit of this
// loop on the 38x38 and 19x19 layers.  After the loop the groups swap halves of their partial sums through LDS and each
// finishes one 32-pixel block of the wave tile.
template <typename T, typename TOut, int BM, int BN, int WM, int WN, int NSA, int PS, int DBG = 0, int KG = 1>
__global__ __launch_bounds__(64 * WM * WN * KG) __attribute__((amdgpu_waves_per_eu(WM * WN * KG / 4, WM * WN * KG / 4)))
void convPatch8Kernel(IgemmArgs a)
{
    typedef typename Frag<T>::V V;
    constexpr int VEC   = Frag<T>::VEC;
    constexpr int KV    = 8;
    constexpr int BK    = KV * VEC;
    constexpr int NWT   = WM * WN;                    // wave tiles
    constexpr int NW    = NWT * KG;
    constexpr int NT    = 64 * NW;
    constexpr int RPP   = NT / KV;                    // weight rows per load pass of the workgroup
    constexpr int AL    = (BM + RPP - 1) / RPP;       // weight loads per thread per tap step (whole passes of the workgroup)
    constexpr int NL    = AL + PS;                    // loads per thread per tap step
    constexpr int TM    = BM / WM;
    constexpr int TN    = BN / WN;
    constexpr int MB    = TM / 32;
    constexpr int NB    = TN / 32;
    constexpr int S     = KV / 2 / KG;                // MFMA k-blocks per tap step and wavefront
    constexpr unsigned ES = sizeof(T);
    constexpr int ROWB  = KV * 16;
    constexpr unsigned A_STAGE = BM * ROWB;           // the wavefronts whose rows of the last pass lie past BM aim at the zero area
    static_assert(BM % 8 == 0, "a wavefront's load covers eight weight rows");
    constexpr bool LATE = NSA == 2;                   // two weight stages: the tile of step it + 2 is asked for behind the barrier of step it, into the stage that barrier frees
    constexpr int PSTEPS = LATE ? 8 : 11 - NSA;       // tap steps of a chunk that bring in slices of the next chunk's patch
    static_assert(TM % 32 == 0 && TN % 32 == 0 && (NW == 4 || NW == 8 || NW == 12), "tile shape");
    static_assert(KG == 1 || (KG == 2 && TM == 64 && TN == 64), "the K-split variant works on 64 x 64 wave tiles");
    static_assert(NSA >= 2 && NSA <= 5, "weight stages");

    extern __shared__ __attribute__((aligned(16))) unsigned char smemRaw[];
    const unsigned ldsBase = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)smemRaw));
    const int nSlices = a.patchRows;                  // 1 KiB slices per patch stage (host: ceil((BN + 2W + 2) / 8))
    const unsigned patchBytes = static_cast<unsigned>(nSlices) * 1024u;
    const unsigned patchOff0 = NSA * A_STAGE;
    const unsigned patchStages = a.cChunks > 1 ? 2u : 1u;     // a single channel chunk never loads a second patch
    const unsigned dumpOff = patchOff0 + patchStages * patchBytes;

    const int tid  = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg   = wave / NWT;                      // which k-blocks of a tap step this wavefront multiplies
    const int wm   = (wave % NWT) / WN;
    const int wn   = (wave % NWT) % WN;
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

    // ---- weight tile: thread tid owns chunk position tid % 8 of row tid / 8 (+ RPP rows per pass); row r keeps logical chunk c
    // at position c ^ ((r / 2) % 8) ------------------------------------------------------------------------------------------
    const int ldRow = tid / KV;
    const int ldVec = (tid % KV) ^ ((ldRow / 2) % KV);
    unsigned aOff[AL];
#pragma unroll
    for (int i = 0; i < AL; ++i)
    {
        const int m = m0 + ldRow + i * RPP;
        aOff[i] = (m < a.coutG && ldRow + i * RPP < BM) ? (static_cast<unsigned>(m) * 9u * a.cinG + ldVec * VEC) * ES : kOobOffset;
    }
    // ---- patch: slice s holds patch rows 8s .. 8s+7 = input pixels q0 + 8s ..; lane l of the slice's load owns chunk position
    // l % 8 of row 8s + l / 8, whose swizzle is ((8s + l/8) / 2) % 8 = (l / 16) ^ 4*(s & 1).  A wavefront's slices are
    // wave, wave + NW, ...: NW is even, so the parity of s is the wavefront's and one base offset serves all its slices.
    // Pixels in front of the tensor give a negative offset, which as unsigned is out of range like the pixels behind it.
    const int q0 = p0 - W - 1;
    const int pRow = lane / KV;
    const int pVec = (lane % KV) ^ (lane / 16) ^ (4 * (wave & 1));
    const unsigned pBase = static_cast<unsigned>((static_cast<long long>(q0 + pRow) * a.inLd + pVec * VEC) * static_cast<long long>(ES));
    const unsigned sliceStride = 8u * static_cast<unsigned>(a.inLd) * ES;
    const unsigned waveDump = ldsBase + dumpOff;
    const bool pCutAlways = false;

    auto issuePatch = [&](int i, int chunk, unsigned stOff) {
        const int s = wave + NW * i;
        const bool real = s < nSlices && chunk < a.cChunks;
        const bool cut = a.ragged && (chunk * BK + pVec * VEC >= a.cinG);
        const unsigned voff = (real && !cut && !pCutAlways) ? pBase + static_cast<unsigned>(s) * sliceStride : kOobOffset;
        dmaLoad16(rx, voff, static_cast<unsigned>(chunk * BK) * ES, real ? ldsBase + stOff + static_cast<unsigned>(s) * 1024u : waveDump);
    };
    const unsigned waveLds = ldsBase + wave * 1024;
    auto issueA = [&](auto lTag, unsigned sA, bool cut, unsigned stageOff) {
        constexpr int l = decltype(lTag)::value;
        const bool real = wave * 8 + l * RPP < BM;    // else every lane's offset is out of range already: zeros onto zeros
        dmaLoad16(rw, cut ? kOobOffset : aOff[l], sA, real ? waveLds + stageOff + l * RPP * ROWB : waveDump);
    };

    // ---- fragments ----------------------------------------------------------------------------------------------------------
    const int fragRow = lane & 31;
    const int fragSw  = (fragRow / 2) % KV;
    unsigned aAddr[S];
#pragma unroll
    for (int kb = 0; kb < S; ++kb) aAddr[kb] = wm * TM * ROWB + fragRow * ROWB + (((2 * (kg * S + kb) + (lane >> 5)) ^ fragSw) * 16);
    const unsigned kvBase = 2 * kg * S + (lane >> 5); // this lane's 16-byte k-vector of local k-block 0
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
            // tap (ky, kx) lies inside the image when row y + ky - 1 and column x + kx - 1 do
            const unsigned cols = (x > 0 ? 1u : 0u) | 2u | (x < W - 1 ? 4u : 0u);
            m = (y > 0 ? cols : 0u) | (cols << 3) | (y < H - 1 ? cols << 6 : 0u);
        }
        tapOk[j] = m;
    }
    const unsigned bRow0 = wn * TN + fragRow;         // patch row of this lane's pixel for tap (0,0), block 0

    V fa[2][MB], fb[2][NB];
    auto readA = [&](unsigned stageOff, auto kbTag) {
        constexpr int kb = decltype(kbTag)::value;
        const unsigned char *ap = smemRaw + (aAddr[kb] + stageOff);
#pragma unroll
        for (int i = 0; i < MB; ++i) fa[kb % 2][i] = *reinterpret_cast<const V *>(ap + i * 32 * ROWB);
    };
    // B fragments of tap `tap` (row offset tapRow = ky*W + kx) from the patch stage at pOff; rows 32 apart share the swizzle.
    // A lane whose tap lies outside the image reads zeros from the zero area at the address bits that select the bank (stages,
    // patch and zero area start at multiples of 1 KiB), so it takes the bank its pixel would have taken: the lanes of a pass
    // stay on distinct banks.  (With one fixed zero address per lane every pass with a border pixel was a two-way conflict.)
    auto readB = [&](unsigned pOff, int tap, unsigned tapRow, auto kbTag) {
        constexpr int kb = decltype(kbTag)::value;
        const unsigned row = bRow0 + tapRow;
        const unsigned sw = (row / 2) % KV;
        const unsigned addr = pOff + row * ROWB + (((2 * kb + kvBase) ^ sw) * 16);
        const unsigned bit = 1u << tap;
        const unsigned zeroAddr = dumpOff + (addr & 255u);
#pragma unroll
        for (int j = 0; j < NB; ++j)
        {
            const unsigned aj = (tapOk[j] & bit) ? addr + j * 32 * ROWB : zeroAddr;
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

    constexpr int PER = MB * NB;                      // MFMAs per k-block
    constexpr int TOT = PER * S;
    constexpr int LSPAN = TOT - PER;                  // the loads of a step follow its MFMAs 0 .. LSPAN-1, ahead of the barrier
    // At the barrier of step `it` the weight tile of step it+1 must have landed: it was issued during step it+2-NSA, and the
    // loads of the NSA-2 steps since then may still be in flight.  Patch slices are issued during taps 0 .. PSTEPS-1 = 10-NSA and
    // are needed from the barrier of tap 8 on, NSA-2 steps later: covered by the same count.
    // Two stages (LATE): the weight tile of step it+2 goes into the stage of step `it` itself, which is free once the barrier of
    // step `it` is passed (the fragments of its last k-block are in registers by then): its loads follow that barrier, among the
    // MFMAs of the last k-block, and have until the next barrier to land; the patch slices of a step are issued ahead of its barrier
    // and may still be in flight there (the slices of taps 0 .. 7 are older than the weight tile that the barrier of tap 8 waits for).
    constexpr int INFLIGHT = LATE ? PS : (NSA - 2) * NL;
    constexpr int AHEADA = LATE ? 2 : NSA - 1;        // the weight loads issued during step `it` belong to step it + AHEADA

    // ---- prologue: whole patch of chunk 0, weight tiles of steps 0 .. NSA-2 -----------------------------------------------------
    if constexpr (!(DBG & 32))
        for (int i = 0; wave + NW * i < nSlices; ++i) issuePatch(i, 0, patchOff0);
    int tapL = -1, chunkL = 0;                        // (tap, chunk) of the step whose weight tile was issued last
    auto advanceA = [&](unsigned &sA, bool &cutA, int stepIndex) {
        if (++tapL == 9) { tapL = 0; ++chunkL; }
        sA = (static_cast<unsigned>(tapL) * a.cinG + chunkL * BK) * ES;
        cutA = stepIndex >= a.nIter || (a.ragged && (chunkL * BK + ldVec * VEC >= a.cinG));
    };
    staticFor<0, AHEADA>([&](auto stTag) {
        constexpr int st = decltype(stTag)::value;
        unsigned sA; bool cutA;
        advanceA(sA, cutA, st);
        if constexpr (!(DBG & 32)) staticFor<0, AL>([&](auto lTag) { issueA(lTag, sA, cutA, st * A_STAGE); });
    });
    dmaWait<0>();
    __syncthreads();
    readA(0, std::integral_constant<int, 0>());
    readB(patchOff0, 0, 0u, std::integral_constant<int, 0>());

    unsigned long long dbgT0 = 0, dbgR0 = 0;
    if constexpr (DBG & 64) { dbgT0 = __builtin_readcyclecounter(); dbgR0 = __builtin_amdgcn_s_memrealtime(); }
    unsigned curA = 0, nxtA = A_STAGE, nnA = (NSA - 1) * A_STAGE;
    unsigned curP = patchOff0, othP = patchStages > 1 ? patchOff0 + patchBytes : patchOff0;
    int it = 0;
    for (int chunk = 0; chunk < a.cChunks; ++chunk)
    {
        staticFor<0, 9>([&](auto tapTag) {
            constexpr int tap = decltype(tapTag)::value;
            constexpr int tapN = tap == 8 ? 0 : tap + 1;
            const unsigned tapRow = static_cast<unsigned>((tap / 3) * W + tap % 3);
            const unsigned tapRowN = static_cast<unsigned>((tapN / 3) * W + tapN % 3);
            const unsigned nextP = tap == 8 ? othP : curP;
            unsigned sA; bool cutA;
            advanceA(sA, cutA, it + AHEADA);          // the weight tile of step it + AHEADA

            if constexpr (!(DBG & 2))
            {
                readA(curA, std::integral_constant<int, 1>());
                readB(curP, tap, tapRow, std::integral_constant<int, 1>());
            }
            __builtin_amdgcn_sched_barrier(0);
            staticFor<0, TOT>([&](auto gTag) {
                constexpr int gi = decltype(gTag)::value;
                constexpr int ks = gi / PER;
                if constexpr (gi % PER == 0 && ks >= 1)
                {
                    if constexpr (ks < S - 1)
                    {
                        if constexpr (!(DBG & 2))
                        {
                            readA(curA, std::integral_constant<int, ks + 1>());
                            readB(curP, tap, tapRow, std::integral_constant<int, ks + 1>());
                        }
                    }
                    else
                    {
                        if constexpr (!(DBG & 1)) dmaWait<INFLIGHT>();
                        if constexpr (!(DBG & 4)) __syncthreads();
                        if constexpr (!(DBG & 2))
                        {
                            readA(nxtA, std::integral_constant<int, 0>());
                            readB(nextP, tapN, tapRowN, std::integral_constant<int, 0>());
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (!(DBG & 8)) mfmaBlock(fa[ks % 2][(gi % PER) / NB], fb[ks % 2][(gi % PER) % NB], acc[(gi % PER) / NB][(gi % PER) % NB]);
                else asm volatile("" : "+v"(fa[ks % 2][(gi % PER) / NB]), "+v"(fb[ks % 2][(gi % PER) % NB]));
                if constexpr (!LATE && gi < LSPAN && !(DBG & 1))
                {
                    // loads l with l * LSPAN / NL == gi: patch slices first, then the weight rows
                    constexpr int first = (gi * NL + LSPAN - 1) / LSPAN;
                    constexpr int last  = ((gi + 1) * NL + LSPAN - 1) / LSPAN;
                    staticFor<first, last>([&](auto lTag) {
                        constexpr int l = decltype(lTag)::value;
                        if constexpr (l < PS)
                            issuePatch(tap < PSTEPS ? tap * PS + l : (1 << 20), chunk + 1, othP);
                        else
                            issueA(std::integral_constant<int, l - PS>(), sA, cutA, nnA);
                    });
                }
                if constexpr (LATE && !(DBG & 1))
                {
                    if constexpr (gi < LSPAN)
                    {
                        // patch slices l with l * LSPAN / PS == gi, ahead of the barrier
                        constexpr int first = (gi * PS + LSPAN - 1) / LSPAN;
                        constexpr int last  = ((gi + 1) * PS + LSPAN - 1) / LSPAN;
                        staticFor<first, last>([&](auto lTag) {
                            constexpr int l = decltype(lTag)::value;
                            issuePatch(tap < PSTEPS ? tap * PS + l : (1 << 20), chunk + 1, othP);
                        });
                    }
                    else
                    {
                        // weight rows l with l * PER / AL == gi - LSPAN, behind the barrier, into the stage it has freed
                        constexpr int first = ((gi - LSPAN) * AL + PER - 1) / PER;
                        constexpr int last  = ((gi - LSPAN + 1) * AL + PER - 1) / PER;
                        staticFor<first, last>([&](auto lTag) { issueA(lTag, sA, cutA, curA); });
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            });
            nnA = curA;
            curA = nxtA;
            nxtA = nxtA + A_STAGE == NSA * A_STAGE ? 0u : nxtA + A_STAGE;
            ++it;
        });
        const unsigned tp = curP;
        curP = othP;
        othP = tp;
    }
    dmaWait<0>();
    __syncthreads();
    if constexpr (DBG & 64)
    {
        const unsigned long long t1 = __builtin_readcyclecounter(), r1 = __builtin_amdgcn_s_memrealtime();
        if (mTile == 0 && pTile == 0 && tid == 0)
        {
            reinterpret_cast<unsigned long long *>(a.ws)[0] = t1 - dbgT0;
            reinterpret_cast<unsigned long long *>(a.ws)[1] = r1 - dbgR0;
        }
    }

    if constexpr (DBG & 16)
    {
        // keep the accumulators alive without the staging and the stores
        float sum = 0.f;
        staticFor<0, MB * NB>([&](auto t) { constexpr int q = decltype(t)::value; sum += acc[q / NB][q % NB][0]; });
        if (sum == 123.456f) static_cast<float *>(a.y)[0] = sum;
        return;
    }
    if constexpr (KG == 1)
        igemmEpilogue<T, TOut, BM, BN, TM, TN>(a, acc, smemRaw, chScale, chShift, m0, p0, wm, wn, wave, lane, 0);
    else
        igemmEpilogueSwap<T, TOut, BM, BN>(a, acc, smemRaw, chScale, chShift, m0, p0, wm, wn, kg, wave % NWT, wave, lane, 0, NW);
}

// Host-side check shared by launch and tile enumeration.
template <typename T, int BM, int BN, int WM, int WN, int NSA, int PS, int KG = 1>
inline bool patch8Fits(const IgemmArgs &a, size_t *smemOut, int *slicesOut)
{
    constexpr int NW = WM * WN * KG;
    constexpr int BK = 8 * Frag<T>::VEC;
    const int R = BN + 2 * a.W + 2;
    const int slices = (R + 7) / 8;
    const int stages = a.cinG > BK ? 2 : 1;
    const size_t loop = static_cast<size_t>(NSA) * BM * 128 + static_cast<size_t>(stages) * slices * 1024 + 1024;
    const size_t swap = KG == 2 ? igemmSwapLds<NW, BM>() : 0;
    const size_t epiOnly = igemmEpilogueLds<BM, BM / WM, NW>();
    const size_t epi = epiOnly > swap ? epiOnly : swap;
    const size_t smem = loop > epi ? loop : epi;
    if (smemOut) *smemOut = smem;
    if (slicesOut) *slicesOut = slices;
    // the first 11 - NSA taps of a chunk (8 with two weight stages) bring in the next patch, PS slices per wavefront and tap
    return a.patchOk && a.buffersOk && smem <= 160 * 1024 && (stages == 1 || slices <= (NSA == 2 ? 8 : 11 - NSA) * NW * PS);
}

template <typename T, typename TOut, int BM, int BN, int WM, int WN, int NSA, int PS, int DBG = 0, int KG = 1>
inline int launchPatch8(IgemmArgs &a, int groups, hipStream_t st)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int BK  = 8 * VEC;
    size_t smem = 0;
    int slices = 0;
    if (groups != 1 || a.splitMax > 1 || a.tailOn || !patch8Fits<T, BM, BN, WM, WN, NSA, PS, KG>(a, &smem, &slices))
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
    auto kern = convPatch8Kernel<T, TOut, BM, BN, WM, WN, NSA, PS, DBG, KG>;
    if (smem > 48 * 1024)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
    }
    hipLaunchKernelGGL(kern, grid, dim3(64 * WM * WN * KG), smem, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
