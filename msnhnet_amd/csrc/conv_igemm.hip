// Host side of the implicit-GEMM convolution: argument marshalling and the default tile heuristic.
#include "conv_igemm.hpp"

namespace msnh {

// Default tile: BM follows the output-channel count so narrow layers do not waste MFMA rows; deep K
// (>= 8 vectors per tap) moves 8 vectors per row per step, shallow K 4.
int igemmHeuristicTile(const msnh_conv_desc *d)
{
    const int vec = d->dtype == MSNH_F16 ? 8 : 4;
    const int cinG = d->in_c / d->groups, coutG = d->out_c / d->groups;
    const bool deep = cinG >= 8 * vec;
    if (coutG <= 32) return deep ? 5 : 6;
    if (coutG <= 64) return deep ? 3 : 4;
    return deep ? 1 : 2;
}

int igemmTileCount() { return kIgemmTiles; }
int igemmTailTileFirst() { return kIgemmTailTileFirst; }

size_t igemmSplitKWorkspaceBytes(const msnh_conv_desc *d)
{
    return static_cast<size_t>(kSplitKMax) * d->batch * d->out_h * d->out_w * d->out_c * sizeof(float);
}

// tail != nullptr: the launch also computes the 1x1 convolution described there (msnh_hip_conv2d_tail); d->tile then names one of the
// tiles that carry a tail, 0 the first of them that takes the shape.
static int convIgemmAny(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
                        const void *residual, void *y, hipStream_t st, bool dryRun, void *splitWs, size_t splitWsBytes,
                        const msnh_conv_tail_desc *tail, const void *w2, const float *scale2, const float *shift2, void *z)
{
    IgemmArgs a;
    a.tailOn = tail ? 1 : 0;
    a.w2 = w2; a.scale2 = scale2; a.shift2 = shift2; a.z = z;
    a.cout2 = tail ? tail->out_c : 0; a.zLd = tail ? tail->out_ld : 0; a.act3 = tail ? tail->act : MSNH_ACT_NONE; a.writeY = tail ? (tail->write_y ? 1 : 0) : 1;
    a.act3Param = tail ? tail->act_param : 0.f; a.zMul = tail ? tail->out_mul : 1.f;
    a.w2Bytes = tail ? static_cast<unsigned>(tail->out_c) * static_cast<unsigned>(d->out_c) * 2u : 0u;
    a.x = x; a.w = w; a.scale = scale; a.shift = shift; a.res = residual; a.y = y;
    a.batch = d->batch; a.H = d->in_h; a.W = d->in_w; a.inLd = d->in_ld;
    a.OH = d->out_h; a.OW = d->out_w; a.outLd = d->out_ld; a.resLd = d->res_ld;
    a.cinG = d->in_c / d->groups; a.coutG = d->out_c / d->groups;
    a.taps = d->ksize * d->ksize; a.ksize = d->ksize; a.stride = d->stride; a.pad = d->pad; a.dil = d->dilation;
    a.P = d->batch * d->out_h * d->out_w;
    a.up2 = d->out_upsample == 2 ? 1 : 0;
    a.xcdGm = d->xcd_blocks;
    a.yBytes = a.up2 ? static_cast<unsigned>(static_cast<unsigned long long>(d->batch) * d->out_h * d->out_w * 4ull * d->out_ld * dtypeSize(d->out_dtype)) : 0u;
    a.byOW = makeFastDiv(static_cast<unsigned>(d->out_w));
    a.byOH = makeFastDiv(static_cast<unsigned>(d->out_h));
    a.patchOk = (d->ksize == 3 && d->stride == 1 && d->pad == 1 && d->dilation == 1 && d->groups == 1 && d->out_h == d->in_h && d->out_w == d->in_w) ? 1 : 0;
    a.patchRows = 0; a.mTiles = 0; a.cChunks = 0; a.nIter = 0;
    a.dryRun = dryRun ? 1 : 0;
    {
        const unsigned long long es = dtypeSize(d->dtype);
        const unsigned long long xb = ((static_cast<unsigned long long>(d->batch) * d->in_h * d->in_w - 1) * d->in_ld + d->in_c) * es;
        const unsigned long long wb = static_cast<unsigned long long>(d->out_c) * a.taps * a.cinG * es;
        a.buffersOk = xb < 0x7fffffffull && wb < 0x7fffffffull;
        a.xBytes = static_cast<unsigned>(xb);
        a.wBytes = static_cast<unsigned>(wb);
        a.ragged = 0;
    }
    a.act = d->act; a.act2 = d->act2; a.hasRes = (d->has_residual && residual) ? 1 : 0;
    a.actParam = d->act_param; a.act2Param = d->act2_param; a.resMul = d->res_mul; a.outMul = d->out_mul;
    const size_t outEl = dtypeSize(d->out_dtype);
    // 8-channel vector stores / residual loads need 8-element alignment of every row start
    a.vecOk = (d->out_ld % 8 == 0) && ((d->out_c / d->groups) % 8 == 0 || d->groups == 1) &&
              (reinterpret_cast<uintptr_t>(y) % (8 * outEl) == 0) &&
              (!a.hasRes || (d->res_ld % 8 == 0 && reinterpret_cast<uintptr_t>(residual) % 16 == 0));
    a.splitMax = 0; a.splitK = 1; a.ws = nullptr; a.wsLd = d->out_c;
    if (a.up2) MSNH_REQUIRE(d->algo != MSNH_CONV_IGEMM_SPLITK && !tail, "conv2d: the upsampling epilogue goes with the plain implicit GEMM");
    if (d->algo == MSNH_CONV_IGEMM_SPLITK)
    {
        MSNH_REQUIRE(d->out_c % 4 == 0, "conv2d: split-K needs out_c to be a multiple of 4");
        if (!dryRun)
        {
            MSNH_REQUIRE(splitWs && reinterpret_cast<uintptr_t>(splitWs) % 16 == 0 && splitWsBytes >= igemmSplitKWorkspaceBytes(d),
                         "conv2d: split-K needs a 16-byte aligned workspace of msnh_hip_conv2d_workspace_bytes() bytes");
        }
        a.splitMax = kSplitKMax;
        a.ws = static_cast<float *>(splitWs);
    }
    int tile = d->tile;
    if (tail)
    {
        MSNH_REQUIRE(d->dtype == MSNH_F16 && d->out_dtype == MSNH_F16 && d->groups == 1 && d->algo != MSNH_CONV_IGEMM_SPLITK, "conv2d_tail: float16, ungrouped, unsplit");
        if (tile <= 0) tile = d->out_c > 128 ? kIgemmTailTileFirst : kIgemmTailTileFirst + 1;
        MSNH_REQUIRE(tile >= kIgemmTailTileFirst && tile <= kIgemmTiles, "conv2d_tail: tile %d carries no tail", tile);
        if (!dryRun)
            MSNH_REQUIRE(reinterpret_cast<uintptr_t>(z) % 16 == 0 && reinterpret_cast<uintptr_t>(w2) % 16 == 0, "conv2d_tail: z and w2 must be 16-byte aligned");
        else a.vecOk = (d->out_ld % 8 == 0) && (d->out_c % 8 == 0) && (!d->has_residual || d->res_ld % 8 == 0);
    }
    if (tile <= 0 || tile > kIgemmTiles) tile = igemmHeuristicTile(d);
    if (d->dtype == MSNH_F16)
        return d->out_dtype == MSNH_F16 ? igemmF16F16(a, d->groups, tile, st) : igemmF16F32(a, d->groups, tile, st);
    MSNH_REQUIRE(d->out_dtype == MSNH_F32, "igemm: float32 input needs float32 output");
    return igemmF32F32(a, d->groups, tile, st);
}

int convIgemmWs(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
                const void *residual, void *y, hipStream_t st, bool dryRun, void *splitWs, size_t splitWsBytes)
{
    return convIgemmAny(d, x, w, scale, shift, residual, y, st, dryRun, splitWs, splitWsBytes, nullptr, nullptr, nullptr, nullptr, nullptr);
}

int convIgemmTail(const msnh_conv_desc *d, const msnh_conv_tail_desc *tail, const void *x, const void *w, const float *scale, const float *shift,
                  const void *residual, void *y, const void *w2, const float *scale2, const float *shift2, void *z, hipStream_t st, bool dryRun)
{
    return convIgemmAny(d, x, w, scale, shift, residual, y, st, dryRun, nullptr, 0, tail, w2, scale2, shift2, z);
}

int convIgemm(const msnh_conv_desc *d, const void *x, const void *w, const float *scale, const float *shift,
              const void *residual, void *y, hipStream_t st, bool dryRun)
{
    return convIgemmWs(d, x, w, scale, shift, residual, y, st, dryRun, nullptr, 0);
}

} // namespace msnh
