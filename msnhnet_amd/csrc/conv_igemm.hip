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
    const int m0   = blockIdx.y * BM;
    const int p0   = blockIdx.x * BN;

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

    // ---- epilogue -------------------------------------------------------------------------------------
    const T *resg = static_cast<const T *>(a.res);
    TOut    *yg   = static_cast<TOut *>(a.y);
    const int chBase = g * a.coutG;
#pragma unroll
    for (int j = 0; j < NB; ++j)
    {
        const int p = p0 + wn * TN + j * 32 + (lane & 31);
        if (p >= a.P) continue;
#pragma unroll
        for (int i = 0; i < MB; ++i)
        {
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                const int m = m0 + wm * TM + i * 32 + q * 8 + (lane >> 5) * 4;
                if (m >= a.coutG) continue;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][q * 4 + e];
                const int ch = chBase + m;
                const bool full = a.vecOk && (m + 3 < a.coutG);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    if (m + e < a.coutG)
                    {
                        const float sc = a.scale ? a.scale[ch + e] : 1.f;
                        const float sh = a.shift ? a.shift[ch + e] : 0.f;
                        v[e] = activate(v[e] * sc + sh, a.act, a.actParam);
                    }
                }
                if (a.hasRes)
                {
                    const T *rp = resg + static_cast<size_t>(p) * a.resLd + ch;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m + e < a.coutG) v[e] = activate(v[e] + a.resMul * toF(rp[e]), a.act2, a.act2Param);
                }
                TOut *yp = yg + static_cast<size_t>(p) * a.outLd + ch;
                if (full)
                {
                    typedef TOut OutV __attribute__((ext_vector_type(4)));
                    OutV o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = fromF<TOut>(a.outMul * v[e]);
                    *reinterpret_cast<OutV *>(yp) = o;
                }
                else
                {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m + e < a.coutG) yp[e] = fromF<TOut>(a.outMul * v[e]);
                }
            }
        }
    }
}

template <typename T, typename TOut, int BM, int BN, int KV, int WM, int WN>
static int launchIgemm(IgemmArgs &a, int groups, hipStream_t st)
{
    constexpr int VEC = Frag<T>::VEC;
    constexpr int BK  = KV * VEC;
    constexpr int LDK = BK + VEC;
    a.cChunks = (a.cinG + BK - 1) / BK;
    a.nIter   = a.taps * a.cChunks;
    const size_t smem = static_cast<size_t>(2) * (BM + BN) * LDK * sizeof(T);
    dim3 grid((a.P + BN - 1) / BN, (a.coutG + BM - 1) / BM, groups);
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

template <typename T, typename TOut>
static int dispatchTile(IgemmArgs &a, int groups, hipStream_t st)
{
    // Tile choice: BM follows the output-channel count so narrow layers do not waste MFMA rows;
    // deep K (cinG >= 64) uses 8 vectors per row per step, shallow K 4.
    const bool deep = a.cinG >= 8 * Frag<T>::VEC;
    if (a.coutG <= 32)
        return deep ? launchIgemm<T, TOut, 32, 256, 8, 1, 4>(a, groups, st) : launchIgemm<T, TOut, 32, 256, 4, 1, 4>(a, groups, st);
    if (a.coutG <= 64)
        return deep ? launchIgemm<T, TOut, 64, 256, 8, 1, 4>(a, groups, st) : launchIgemm<T, TOut, 64, 256, 4, 1, 4>(a, groups, st);
    return deep ? launchIgemm<T, TOut, 128, 128, 8, 2, 2>(a, groups, st) : launchIgemm<T, TOut, 128, 128, 4, 2, 2>(a, groups, st);
}

int convIgemm(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
              const void *residual, void *y, hipStream_t st)
{
    IgemmArgs a;
    a.x = x; a.w = w; a.scale = scale; a.shift = shift; a.res = residual; a.y = y;
    a.batch = d->batch; a.H = d->in_h; a.W = d->in_w; a.inLd = d->in_ld;
    a.OH = d->out_h; a.OW = d->out_w; a.outLd = d->out_ld; a.resLd = d->res_ld;
    a.cinG = d->in_c / d->groups; a.coutG = d->out_c / d->groups;
    a.taps = d->ksize * d->ksize; a.ksize = d->ksize; a.stride = d->stride; a.pad = d->pad; a.dil = d->dilation;
    a.P = d->batch * d->out_h * d->out_w;
    a.act = d->act; a.act2 = d->act2; a.hasRes = (d->has_residual && residual) ? 1 : 0;
    a.actParam = d->act_param; a.act2Param = d->act2_param; a.resMul = d->res_mul; a.outMul = d->out_mul;
    const size_t outEl = dtypeSize(d->out_dtype);
    a.vecOk = (d->out_ld % 4 == 0) && ((d->out_c / d->groups) % 4 == 0) &&
              (reinterpret_cast<uintptr_t>(y) % (4 * outEl) == 0);
    if (d->dtype == MSNH_F16)
        return d->out_dtype == MSNH_F16 ? dispatchTile<f16, f16>(a, d->groups, st) : dispatchTile<f16, float>(a, d->groups, st);
    MSNH_REQUIRE(d->out_dtype == MSNH_F32, "igemm: float32 input needs float32 output");
    return dispatchTile<float, float>(a, d->groups, st);
}

} // namespace msnh
