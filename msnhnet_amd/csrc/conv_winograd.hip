// Winograd F(2x2,3x3) convolution for 3x3 stride-1 pad-1 float16 layers: 2.25x fewer multiplications than the
// direct form, paid for with two extra passes over memory.  Three launches:
//
//   1. input transform   V[t][pos][ci] = (B^T d B)[pos]    d = the 4x4 input patch of output tile t (2x2 pixels),
//                                                          zero outside the image; pos = 4*row + col
//   2. 16 GEMMs          M[t][pos][co] = sum_ci U[pos][co][ci] * V[t][pos][ci]
//                        run as ONE grouped 1x1 convolution over T "pixels" with 16 groups on the implicit-GEMM
//                        MFMA kernel (V is laid out so that pos is the channel-group index), float32 out
//   3. output transform  y = epilogue((A^T M A))           2x2 pixels per tile; folded batch-norm / bias,
//                                                          activation, residual, second activation, output scale
//
// U = G g G^T is computed in float32 on the host when the weights are packed and rounded to float16 once.
// The transforms only add and subtract; they are done in float32 and rounded once, so the float16 operands of
// the GEMM carry the same rounding as the direct convolution's (|V| <= 4 max|d| stays far inside float16 range
// for activations scaled to <= 2^11).  It pays off where K is deep and the image small (few tiles, big GEMM);
// on large images the two extra passes cost more than the saved multiplications, and the per-layer search of the
// host library decides.
#include "common.hpp"
#include <vector>

namespace msnh {

int convIgemm(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
              const void *residual, void *y, hipStream_t st, bool dryRun);

namespace {

struct WinoGeom
{
    int B, H, W, C, inLd, OC, outLd, resLd;
    int TH, TW;            // tiles per image column / row
    long long T;           // tiles in the batch
};

inline WinoGeom geomOf(const msnh_conv_desc *d)
{
    WinoGeom g;
    g.B = d->batch; g.H = d->in_h; g.W = d->in_w; g.C = d->in_c; g.inLd = d->in_ld; g.OC = d->out_c; g.outLd = d->out_ld; g.resLd = d->res_ld;
    g.TH = (d->out_h + 1) / 2;
    g.TW = (d->out_w + 1) / 2;
    g.T = static_cast<long long>(d->batch) * g.TH * g.TW;
    return g;
}

inline size_t alignUp(size_t v) { return (v + 255) / 256 * 256; }

// thread = (tile, 4 channels)
__global__ __launch_bounds__(256) void winoInputKernel(const f16 *__restrict__ x, f16 *__restrict__ v, WinoGeom g, long long total)
{
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cq = g.C / 4;
    const int c = static_cast<int>(idx % cq) * 4;
    long long t = idx / cq;
    const int tx = static_cast<int>(t % g.TW);
    const long long r = t / g.TW;
    const int ty = static_cast<int>(r % g.TH);
    const int b = static_cast<int>(r / g.TH);
    float d[4][4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        const int iy = 2 * ty - 1 + i;
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            const int ix = 2 * tx - 1 + j;
            f16x4 q = {static_cast<f16>(0.f), static_cast<f16>(0.f), static_cast<f16>(0.f), static_cast<f16>(0.f)};
            if (iy >= 0 && iy < g.H && ix >= 0 && ix < g.W)
                q = *reinterpret_cast<const f16x4 *>(x + ((static_cast<size_t>(b) * g.H + iy) * g.W + ix) * g.inLd + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) d[i][j][e] = static_cast<float>(q[e]);
        }
    }
    f16 *vp = v + static_cast<size_t>(t) * 16 * g.C + c;
#pragma unroll
    for (int e = 0; e < 4; ++e)
    {
        // rows: B^T d
        float m[4][4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            m[0][j] = d[0][j][e] - d[2][j][e];
            m[1][j] = d[1][j][e] + d[2][j][e];
            m[2][j] = d[2][j][e] - d[1][j][e];
            m[3][j] = d[1][j][e] - d[3][j][e];
        }
        // columns: (B^T d) B
#pragma unroll
        for (int i = 0; i < 4; ++i)
        {
            d[i][0][e] = m[i][0] - m[i][2];
            d[i][1][e] = m[i][1] + m[i][2];
            d[i][2][e] = m[i][2] - m[i][1];
            d[i][3][e] = m[i][1] - m[i][3];
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            f16x4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = static_cast<f16>(d[i][j][e]);
            *reinterpret_cast<f16x4 *>(vp + static_cast<size_t>(i * 4 + j) * g.C) = o;
        }
}

struct WinoEpi
{
    const float *scale;
    const float *shift;
    int act, act2, hasRes;
    float actParam, act2Param, resMul, outMul;
};

// thread = (tile, 4 output channels)
template <typename TOut>
__global__ __launch_bounds__(256) void winoOutputKernel(const float *__restrict__ m, const f16 *__restrict__ res, TOut *__restrict__ y, WinoGeom g,
                                                        WinoEpi e, int OH, int OW, long long total)
{
    const long long idx = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total) return;
    const int cq = g.OC / 4;
    const int c = static_cast<int>(idx % cq) * 4;
    long long t = idx / cq;
    const int tx = static_cast<int>(t % g.TW);
    const long long r = t / g.TW;
    const int ty = static_cast<int>(r % g.TH);
    const int b = static_cast<int>(r / g.TH);
    const float *mp = m + static_cast<size_t>(t) * 16 * g.OC + c;
    f32x4 q[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) q[i][j] = *reinterpret_cast<const f32x4 *>(mp + static_cast<size_t>(i * 4 + j) * g.OC);
    // A^T M: 2 x 4
    f32x4 s[2][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        s[0][j] = q[0][j] + q[1][j] + q[2][j];
        s[1][j] = q[1][j] - q[2][j] - q[3][j];
    }
    f32x4 sc = {1.f, 1.f, 1.f, 1.f}, sh = {0.f, 0.f, 0.f, 0.f};
    if (e.scale) sc = *reinterpret_cast<const f32x4 *>(e.scale + c);
    if (e.shift) sh = *reinterpret_cast<const f32x4 *>(e.shift + c);
#pragma unroll
    for (int i = 0; i < 2; ++i)
    {
        const int oy = 2 * ty + i;
        if (oy >= OH) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
            const int ox = 2 * tx + j;
            if (ox >= OW) continue;
            const f32x4 acc = j == 0 ? s[i][0] + s[i][1] + s[i][2] : s[i][1] - s[i][2] - s[i][3];
            const size_t p = (static_cast<size_t>(b) * OH + oy) * OW + ox;
            f16x4 rv = {static_cast<f16>(0.f), static_cast<f16>(0.f), static_cast<f16>(0.f), static_cast<f16>(0.f)};
            if (e.hasRes) rv = *reinterpret_cast<const f16x4 *>(res + p * g.resLd + c);
            typedef TOut OutV __attribute__((ext_vector_type(4)));
            OutV o;
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                float v = activate(acc[k] * sc[k] + sh[k], e.act, e.actParam);
                if (e.hasRes) v = activate(v + e.resMul * static_cast<float>(rv[k]), e.act2, e.act2Param);
                o[k] = fromF<TOut>(e.outMul * v);
            }
            *reinterpret_cast<OutV *>(y + p * g.outLd + c) = o;
        }
    }
}

} // namespace

// the 16 GEMMs as one grouped 1x1 convolution over T pixels
void winogradGemmDesc(const msnh_conv_desc *d, msnh_conv_desc *gd)
{
    const WinoGeom g = geomOf(d);
    gd->dtype = MSNH_F16; gd->out_dtype = MSNH_F32;
    gd->batch = 1; gd->in_h = 1; gd->in_w = static_cast<int>(g.T); gd->in_c = 16 * g.C; gd->in_ld = 16 * g.C;
    gd->out_c = 16 * g.OC; gd->out_h = 1; gd->out_w = static_cast<int>(g.T); gd->out_ld = 16 * g.OC;
    gd->ksize = 1; gd->stride = 1; gd->pad = 0; gd->dilation = 1; gd->groups = 16;
    gd->act = MSNH_ACT_NONE; gd->act_param = 0.f; gd->has_residual = 0; gd->res_ld = 16 * g.OC; gd->act2 = MSNH_ACT_NONE; gd->act2_param = 0.f;
    gd->res_mul = 1.f; gd->out_mul = 1.f; gd->algo = MSNH_CONV_IGEMM; gd->tile = d->tile;
    gd->out_upsample = 0;
    gd->xcd_blocks = 0;
}

size_t winogradWorkspaceBytes(const msnh_conv_desc *d)
{
    const WinoGeom g = geomOf(d);
    return alignUp(static_cast<size_t>(g.T) * 16 * g.C * sizeof(f16)) + alignUp(static_cast<size_t>(g.T) * 16 * g.OC * sizeof(float));
}

// packed[pos][oc][ci] = (G g G^T)[pos], float16
void winogradPackWeights(const msnh_conv_desc *d, const float *oihw, void *packed)
{
    static const float G[4][3] = {{1.f, 0.f, 0.f}, {0.5f, 0.5f, 0.5f}, {0.5f, -0.5f, 0.5f}, {0.f, 0.f, 1.f}};
    _Float16 *o = static_cast<_Float16 *>(packed);
    const int C = d->in_c, OC = d->out_c;
    for (int oc = 0; oc < OC; ++oc)
        for (int ci = 0; ci < C; ++ci)
        {
            const float *g = oihw + (static_cast<size_t>(oc) * C + ci) * 9;
            float t[4][3];
            for (int i = 0; i < 4; ++i)
                for (int j = 0; j < 3; ++j) t[i][j] = G[i][0] * g[j] + G[i][1] * g[3 + j] + G[i][2] * g[6 + j];
            for (int i = 0; i < 4; ++i)
                for (int j = 0; j < 4; ++j)
                {
                    const float u = t[i][0] * G[j][0] + t[i][1] * G[j][1] + t[i][2] * G[j][2];
                    o[(static_cast<size_t>(i * 4 + j) * OC + oc) * C + ci] = static_cast<_Float16>(u);
                }
        }
}

int convWinograd(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift, const void *residual, void *y,
                 void *ws, size_t wsBytes, hipStream_t st)
{
    const WinoGeom g = geomOf(d);
    const size_t vBytes = alignUp(static_cast<size_t>(g.T) * 16 * g.C * sizeof(f16));
    MSNH_REQUIRE(ws != nullptr && wsBytes >= winogradWorkspaceBytes(d), "conv2d: Winograd needs a workspace of %zu bytes", winogradWorkspaceBytes(d));
    MSNH_REQUIRE(reinterpret_cast<uintptr_t>(ws) % 256 == 0 && reinterpret_cast<uintptr_t>(x) % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(w) % 16 == 0,
                 "conv2d: Winograd needs aligned tensors");
    MSNH_REQUIRE(!d->has_residual || (d->res_ld % 4 == 0 && reinterpret_cast<uintptr_t>(residual) % 8 == 0), "conv2d: Winograd needs an aligned residual");
    MSNH_REQUIRE(g.T * 16 * g.C * 2 < (1LL << 31) && g.T < (1LL << 31) / 16, "conv2d: too large for the Winograd path");
    f16 *v = static_cast<f16 *>(ws);
    float *m = reinterpret_cast<float *>(static_cast<unsigned char *>(ws) + vBytes);

    const long long inTotal = g.T * (g.C / 4);
    hipLaunchKernelGGL(winoInputKernel, dim3(gridFor(inTotal, 256)), dim3(256), 0, st, static_cast<const f16 *>(x), v, g, inTotal);
    MSNH_LAUNCH_CHECK();

    msnh_conv_desc gd;
    winogradGemmDesc(d, &gd);
    const int rc = convIgemm(&gd, v, w, nullptr, nullptr, nullptr, m, st, false);
    if (rc) return rc;

    WinoEpi e;
    e.scale = scale; e.shift = shift; e.act = d->act; e.act2 = d->act2; e.hasRes = (d->has_residual && residual) ? 1 : 0;
    e.actParam = d->act_param; e.act2Param = d->act2_param; e.resMul = d->res_mul; e.outMul = d->out_mul;
    const long long outTotal = g.T * (g.OC / 4);
    if (d->out_dtype == MSNH_F16)
        hipLaunchKernelGGL(winoOutputKernel<f16>, dim3(gridFor(outTotal, 256)), dim3(256), 0, st, m, static_cast<const f16 *>(residual),
                           static_cast<f16 *>(y), g, e, d->out_h, d->out_w, outTotal);
    else
        hipLaunchKernelGGL(winoOutputKernel<float>, dim3(gridFor(outTotal, 256)), dim3(256), 0, st, m, static_cast<const f16 *>(residual),
                           static_cast<float *>(y), g, e, d->out_h, d->out_w, outTotal);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace msnh
