// Winograd F(2x2,3x3) for 3x3 stride-1 pad-1 float16 layers as ONE launch: input transform on the way into LDS, the 16
// transformed-domain products on the matrix cores with all 16 accumulator sets of a tile held in registers, output transform and
// the full epilogue (folded batch-norm / bias, activation, residual, second activation, scale) straight from the accumulators.
// Nothing transformed crosses memory: the three-launch form (conv_winograd.hip) writes and reads V (16 x the input tiles) and M (16 x
// the output tiles, float32) through HBM and loses to the direct kernels for that reason alone.
//
// Work split.  A workgroup of 8 wavefronts owns 64 output channels x 64 output tiles (2 x 2 pixels each, consecutive in
// (image, tile row, tile column) order) for all 16 transform positions; wavefront w owns positions 2w and 2w + 1, i.e. two
// 64 x 64 accumulator sets (128 registers).  K = in_c runs in chunks of 16 channels:
//   * every thread owns one (tile, channel pair) of the chunk: it loads the 4 x 4 input patch of its tile (4-byte buffer loads;
//     positions outside the image carry an out-of-range offset and read zeros), applies B^T d B with packed float16 additions
//     (two roundings per value instead of the one of a float32 transform) and writes the 16 values into the V stage of the
//     chunk, [position][tile][16 channels], 32-byte rows whose halves are exchanged for every second group of eight tiles so that
//     the fragment reads of 16 lanes fall into 16 different bank groups;
//   * the filter operand U = G g G^T (packed [position][out_c][in_c] at load, the layout of the three-launch form) goes from
//     memory straight into fragment registers -- a wavefront's positions are its own, nothing is shared -- with the rows
//     permuted so that a lane's 16 accumulators are 16 consecutive output channels;
//   * per chunk a wavefront issues 8 MFMAs (2 positions x 2 channel blocks x 2 tile blocks); the loads of chunk c + 1 are in
//     flight meanwhile, its transform follows, one barrier per chunk, two V stages.
// After the loop the accumulators of 32 tiles at a time go through LDS ([position][tile][channel] float32, rows padded to 272
// bytes), and every thread combines the 9 positions one output pixel of a tile depends on for 8 channels: A^T M A, epilogue,
// one 16-byte store.
#include "conv_igemm.hpp"

namespace msnh {

struct WfArgs
{
    const f16   *x;
    const f16   *u;         // [16][out_c][in_c]
    const float *scale;
    const float *shift;
    const f16   *res;
    f16         *y;
    int B, H, W, C, inLd, OC, outLd, resLd;
    int TH, TW, T;          // tiles per image column / row, tiles in the batch
    int tileBlocks, coutBlocks;
    unsigned xBytes, uBytes;
    int act, act2, hasRes;
    float actParam, act2Param, resMul, outMul;
};

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

constexpr int WF_BM = 64, WF_NT = 64, WF_KC = 16, WF_THREADS = 512;
constexpr int WF_VSTAGE = 16 * WF_NT * WF_KC * 2;             // bytes of one V stage
constexpr int WF_MROW = 272;                                  // bytes of one (position, tile) row of the output staging: 64 floats + 16
constexpr int WF_MBYTES = 16 * 32 * WF_MROW;
constexpr int WF_LDS = WF_MBYTES > 2 * WF_VSTAGE ? WF_MBYTES : 2 * WF_VSTAGE;

__device__ __forceinline__ int wfChannelOfRow(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

__device__ __forceinline__ h2 loadPair(__amdgpu_buffer_rsrc_t r, unsigned voffset, unsigned soffset)
{
    const int v = __builtin_amdgcn_raw_buffer_load_b32(r, static_cast<int>(voffset), static_cast<int>(soffset), 0);
    return __builtin_bit_cast(h2, v);
}

__global__ __launch_bounds__(WF_THREADS) void convWinoFusedKernel(WfArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char wfSmem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, n = lane & 31;

    const int total = a.tileBlocks * a.coutBlocks;
    const int perXcd = (total + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    if (logical >= total) return;
    const int m0 = (logical % a.coutBlocks) * WF_BM;
    const int t0 = (logical / a.coutBlocks) * WF_NT;

    const __amdgpu_buffer_rsrc_t rx = makeRsrc(a.x, a.xBytes);
    const __amdgpu_buffer_rsrc_t ru = makeRsrc(a.u, a.uBytes);

    // ---- transform role: tile tid / 8, channel pair tid % 8 of the chunk --------------------------------------------------------
    const int trTile = tid >> 3, trPair = tid & 7;
    unsigned patchOff[16];                                      // byte offset of patch position (i, j), out of range where it lies outside the image
    {
        const int tg = t0 + trTile;
        const bool live = tg < a.T;
        const int tt = live ? tg : 0;
        const int tx = tt % a.TW;
        const int r = tt / a.TW;
        const int ty = r % a.TH;
        const int b = r / a.TH;
        const int iy0 = 2 * ty - 1, ix0 = 2 * tx - 1;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                const int iy = iy0 + i, ix = ix0 + j;
                const bool ok = live && iy >= 0 && iy < a.H && ix >= 0 && ix < a.W;
                patchOff[i * 4 + j] = ok ? static_cast<unsigned>(((b * a.H + iy) * a.W + ix) * a.inLd + 2 * trPair) * 2u : kOobOffset;
            }
    }
    // where this thread's 4 bytes of position 0 go inside a V stage
    const unsigned vWrite = static_cast<unsigned>(trTile * 32 + (((trPair >> 2) ^ ((trTile >> 3) & 1)) * 16) + (trPair & 3) * 4);
    h2 raw[16];
    auto loadRaw = [&](int chunk) {
        const unsigned so = static_cast<unsigned>(chunk * WF_KC) * 2u;
#pragma unroll
        for (int q = 0; q < 16; ++q) raw[q] = loadPair(rx, patchOff[q], so);
    };
    auto transformTo = [&](unsigned stageOff) {
        h2 t[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            t[0][j] = raw[0 * 4 + j] - raw[2 * 4 + j];
            t[1][j] = raw[1 * 4 + j] + raw[2 * 4 + j];
            t[2][j] = raw[2 * 4 + j] - raw[1 * 4 + j];
            t[3][j] = raw[1 * 4 + j] - raw[3 * 4 + j];
        }
        unsigned char *dst = wfSmem + stageOff + vWrite;
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            *reinterpret_cast<h2 *>(dst + (i * 4 + 0) * (WF_NT * 32)) = t[i][0] - t[i][2];
            *reinterpret_cast<h2 *>(dst + (i * 4 + 1) * (WF_NT * 32)) = t[i][1] + t[i][2];
            *reinterpret_cast<h2 *>(dst + (i * 4 + 2) * (WF_NT * 32)) = t[i][2] - t[i][1];
            *reinterpret_cast<h2 *>(dst + (i * 4 + 3) * (WF_NT * 32)) = t[i][1] - t[i][3];
        }
    };

    // ---- multiply role: positions 2 * wave, 2 * wave + 1 ------------------------------------------------------------------------------
    unsigned aOff[2];                                           // this lane's row of the two 32-channel blocks in U (position 0), bytes
#pragma unroll
    for (int i = 0; i < 2; ++i)
    {
        const int c = m0 + 32 * i + wfChannelOfRow(n);
        aOff[i] = c < a.OC ? static_cast<unsigned>(c * a.C + 8 * h) * 2u : kOobOffset;
    }
    const unsigned posStride = static_cast<unsigned>(a.OC) * static_cast<unsigned>(a.C) * 2u;
    const unsigned bRead = static_cast<unsigned>(2 * wave * (WF_NT * 32) + n * 32 + ((h ^ ((n >> 3) & 1)) * 16));
    f16x8 af[2][2];
    auto loadA = [&](int chunk) {
#pragma unroll
        for (int z = 0; z < 2; ++z)
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[z][i] = bufferLoad16<f16x8>(ru, aOff[i], static_cast<unsigned>(2 * wave + z) * posStride + static_cast<unsigned>(chunk * WF_KC) * 2u);
    };

    f32x16 acc[2][2][2];                                        // [position][channel block][tile block]
#pragma unroll
    for (int z = 0; z < 2; ++z)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[z][i][j][e] = 0.f;

    const int nChunks = a.C / WF_KC;
    loadRaw(0);
    loadA(0);
    transformTo(0);
    __syncthreads();
    for (int c = 0; c < nChunks; ++c)
    {
        const unsigned stage = static_cast<unsigned>(c & 1) * WF_VSTAGE;
        const bool more = c + 1 < nChunks;
        if (more) loadRaw(c + 1);
        f16x8 bf[2][2];
#pragma unroll
        for (int z = 0; z < 2; ++z)
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[z][j] = *reinterpret_cast<const f16x8 *>(wfSmem + stage + bRead + z * (WF_NT * 32) + j * 1024);
#pragma unroll
        for (int z = 0; z < 2; ++z)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) mfmaBlock(af[z][i], bf[z][j], acc[z][i][j]);
        if (more)
        {
            loadA(c + 1);
            transformTo(static_cast<unsigned>((c + 1) & 1) * WF_VSTAGE);
        }
        __syncthreads();
    }

    // ---- output: 32 tiles at a time through LDS, then one pixel x 8 channels per thread item ---------------------------------------
#pragma unroll
    for (int jh = 0; jh < 2; ++jh)
    {
        if (jh) __syncthreads();                                // the items of the first half have been read
#pragma unroll
        for (int z = 0; z < 2; ++z)
#pragma unroll
            for (int i = 0; i < 2; ++i)
            {
                unsigned char *dst = wfSmem + (2 * wave + z) * (32 * WF_MROW) + n * WF_MROW + (32 * i + 16 * h) * 4;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4)
                {
                    f32x4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = acc[z][i][jh][4 * e4 + e];
                    *reinterpret_cast<f32x4 *>(dst + e4 * 16) = v;
                }
            }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 2; ++k)
        {
            const int item = tid + k * WF_THREADS;
            const int g = item & 7, q = (item >> 3) & 3, t = item >> 5;
            const int c0 = m0 + 8 * g;
            const int tg = t0 + 32 * jh + t;
            if (tg >= a.T || c0 >= a.OC) continue;
            const int tx = tg % a.TW;
            const int r = tg / a.TW;
            const int ty = r % a.TH;
            const int b = r / a.TH;
            const int qy = q >> 1, qx = q & 1;
            const int oy = 2 * ty + qy, ox = 2 * tx + qx;
            if (oy >= a.H || ox >= a.W) continue;
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = 0.f;
            // A^T M A: pixel row 0 adds rows 0, 1, 2; pixel row 1 takes rows 1, -2, -3; columns likewise
#pragma unroll
            for (int rr = 0; rr < 3; ++rr)
#pragma unroll
                for (int cc = 0; cc < 3; ++cc)
                {
                    const int row = qy + rr, col = qx + cc;
                    const float sgn = ((qy && rr > 0) != (qx && cc > 0)) ? -1.f : 1.f;
                    const unsigned char *src = wfSmem + (row * 4 + col) * (32 * WF_MROW) + t * WF_MROW + g * 32;
                    const f32x4 lo = *reinterpret_cast<const f32x4 *>(src), hi = *reinterpret_cast<const f32x4 *>(src + 16);
#pragma unroll
                    for (int e = 0; e < 4; ++e) { v[e] += sgn * lo[e]; v[4 + e] += sgn * hi[e]; }
                }
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = v[e] * (a.scale ? a.scale[c0 + e] : 1.f) + (a.shift ? a.shift[c0 + e] : 0.f);
            activateArray<8>(v, a.act, a.actParam);
            const size_t p = (static_cast<size_t>(b) * a.H + oy) * a.W + ox;
            if (a.hasRes)
            {
                const f16x8 rv = *reinterpret_cast<const f16x8 *>(a.res + p * a.resLd + c0);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] += a.resMul * static_cast<float>(rv[e]);
                activateArray<8>(v, a.act2, a.act2Param);
            }
            f16x8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = static_cast<f16>(a.outMul * v[e]);
            *reinterpret_cast<f16x8 *>(a.y + p * a.outLd + c0) = o;
        }
    }
}

} // namespace

bool winogradFusedOk(const msnh_conv_desc *d)
{
    if (!(d->ksize == 3 && d->stride == 1 && d->dilation == 1 && d->groups == 1 && d->pad == 1 && d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16)) return false;
    if (d->in_h != d->out_h || d->in_w != d->out_w) return false;
    if (d->in_c % WF_KC != 0 || d->in_ld % 8 != 0 || d->out_c % 8 != 0 || d->out_ld % 8 != 0 || (d->has_residual && d->res_ld % 8 != 0)) return false;
    const long long xb = (static_cast<long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld * 2 + d->in_c * 2;
    const long long ub = 16LL * d->out_c * d->in_c * 2;
    const long long tiles = static_cast<long long>(d->batch) * ((d->out_h + 1) / 2) * ((d->out_w + 1) / 2);
    return xb < 0x7fffffffLL && ub < 0x7fffffffLL && tiles < (1LL << 30);
}

int convWinogradFused(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, const void *residual, void *y,
                      hipStream_t st)
{
    MSNH_REQUIRE(winogradFusedOk(d), "conv2d: shape not supported by the fused Winograd kernel");
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                     (!d->has_residual || reinterpret_cast<uintptr_t>(residual) % 16 == 0),
                 "conv2d: the fused Winograd kernel needs 16-byte aligned tensors");
    WfArgs a;
    a.x = static_cast<const f16 *>(x); a.u = static_cast<const f16 *>(w); a.scale = scale; a.shift = shift;
    a.res = static_cast<const f16 *>(residual); a.y = static_cast<f16 *>(y);
    a.B = d->batch; a.H = d->in_h; a.W = d->in_w; a.C = d->in_c; a.inLd = d->in_ld; a.OC = d->out_c; a.outLd = d->out_ld; a.resLd = d->res_ld;
    a.TH = (d->out_h + 1) / 2; a.TW = (d->out_w + 1) / 2; a.T = d->batch * a.TH * a.TW;
    a.tileBlocks = (a.T + WF_NT - 1) / WF_NT; a.coutBlocks = (a.OC + WF_BM - 1) / WF_BM;
    a.xBytes = static_cast<unsigned>((static_cast<long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld * 2 + d->in_c * 2);
    a.uBytes = static_cast<unsigned>(16LL * d->out_c * d->in_c * 2);
    a.act = d->act; a.act2 = d->act2; a.hasRes = (d->has_residual && residual) ? 1 : 0;
    a.actParam = d->act_param; a.act2Param = d->act2_param; a.resMul = d->res_mul; a.outMul = d->out_mul;
    static bool attrSet = false;        // (per process; the attribute belongs to the function on every device of this build's single-GPU use)
    if (!attrSet)
    {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(convWinoFusedKernel), hipFuncAttributeMaxDynamicSharedMemorySize, WF_LDS);
        if (e != hipSuccess) { setError("hipFuncSetAttribute: %s", hipGetErrorString(e)); return 1; }
        attrSet = true;
    }
    const int blocks = (a.tileBlocks * a.coutBlocks + 7) / 8 * 8;
    hipLaunchKernelGGL(convWinoFusedKernel, dim3(blocks), dim3(WF_THREADS), WF_LDS, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
