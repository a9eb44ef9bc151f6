// First layer + first down-sampling layer as ONE launch: a 3x3 stride-1 pad-1 convolution over the 3-channel NCHW float32 network
// input with 32 filters, followed by a 3x3 stride-2 pad-1 convolution with 32, 64 or 128 filters (the opening of the Darknet-53 and
// CSPDarknet-53 trunks: src/layers/MsnhConvolutionalLayer.cpp forwardGPU twice, with the full-resolution 32-channel tensor written
// to and read back from device memory in between).  Here that tensor never leaves the chip: for YOLOv3-608 at batch 8 it is 189 MB
// each way, more than the 35 MB the pair reads and the 95 MB it writes.
//
// A workgroup (4 wavefronts) owns a tile of 8 x 16 output pixels of the second convolution:
//   0. the 19 x 35 x 3 float32 input patch under it goes to LDS (zeros outside the image);
//   1. the 17 x 33 first-layer outputs the tile needs are computed on the matrix cores, 32 pixels per MFMA block (K = 27 padded to 32:
//      channel c's taps 0..7 in K group c, the three ninth taps in group 3), scaled / shifted / activated, set to zero where they fall
//      outside the image (they are the second layer's zero padding) and stored as float16 in LDS, 64 bytes per pixel, even and odd
//      columns apart so that the stride-2 reads of step 2 walk consecutive rows, 16-byte chunks XOR-swizzled against bank conflicts;
//   2. the second convolution reads its B fragments from that tile (one wavefront per 2 x 16 output pixels, K = 9 taps x 32 channels),
//      its A fragments (weights in MFMA lane order) straight from global memory one tap ahead, and writes NHWC float16.
// Both MFMA row orders are the channel permutation that makes a lane's 16 accumulators 16 consecutive channels (row 8q + 4h + e
// computes channel 16h + 4q + e).
//   3. (msnh_hip_conv_stem_down_tail) the 1x1 convolution with 32 filters that reads the pair's result -- the opening of Darknet-53's
//      first residual block -- computed by the same wavefront from its own 32 pixels without leaving the registers: a lane holds 16
//      consecutive channels of its pixel as float16, which is two 8-channel halves of the B operand of a 32x32x16 MFMA; the half the
//      lane's own operand slot does not take is the one its partner lane (same pixel, other half-wave) needs, and the other way round:
//      one v_permlane32_swap per register.  K runs over the channels in order, as a separate 1x1 launch would.
#include "common.hpp"

namespace msnh {

namespace {

constexpr int SD_TH = 8, SD_TW = 16;                  // output tile of the second convolution
constexpr int SD_SH = 2 * SD_TH + 1, SD_SW = 2 * SD_TW + 1;      // first-layer outputs under it: 17 x 33
constexpr int SD_IH = SD_SH + 2, SD_IW = SD_SW + 2;   // input patch: 19 x 35
constexpr int SD_IP = 36;                             // its row pitch in elements
constexpr int SD_NPIX = SD_SH * SD_SW;                // 561
constexpr int SD_EVEN = (SD_SW + 1) / 2;              // 17 even columns per tile row, then 16 odd ones
constexpr int SD_IMG_BYTES = 3 * SD_IH * SD_IP * 4;   // 8208 (a multiple of 16: the tile behind it holds 16-byte vectors)
constexpr int SD_TILE_BYTES = SD_NPIX * 64;           // 35904
constexpr int SD_MAXC2 = 128;

struct StemDownArgs
{
    const float *x;         // [B][3][H][W]
    const f16 *w1;          // [2][64][8]
    const float *scale1, *shift1;
    const f16 *w2;          // [9][2][C2/32][64][8]
    const float *scale2, *shift2;
    f16 *y;
    int B, H, W, OH, OW, outLd, tilesX, tilesY, total;
    int act1, act2;
    float act1Param, act2Param, midMul, outMul;
    // tail: z = zMul * act3(scale3 * (w3 . y) + shift3), 32 filters over the C2 channels of y
    const f16 *w3;          // [C2/32][2][64][8]
    const float *scale3, *shift3;
    f16 *z;
    int zLd, act3;
    float act3Param, zMul;
};

__device__ __forceinline__ unsigned sdSlotAddr(int slot, int chunk)
{
    return static_cast<unsigned>(slot) * 64u + static_cast<unsigned>((chunk ^ ((slot >> 1) & 3)) * 16);
}

template <int MB2, int TAIL = 0>
__global__ __launch_bounds__(256) void convStemDownKernel(StemDownArgs a)
{
    __shared__ __attribute__((aligned(16))) unsigned char smem[SD_IMG_BYTES + SD_TILE_BYTES];
    __shared__ float aff[2 * 32 + 2 * SD_MAXC2 + 2 * 32];
    float *imgL = reinterpret_cast<float *>(smem);
    unsigned char *tileL = smem + SD_IMG_BYTES;

    // workgroup ids are dealt round-robin to the 8 XCDs; regrouped so that an XCD works on one contiguous run of tiles (the halo rows
    // that neighbouring tiles share are then fetched into one L2)
    const int perXcd = (a.total + 7) / 8;
    const int logical = static_cast<int>(blockIdx.x % 8) * perXcd + static_cast<int>(blockIdx.x / 8);
    if (logical >= a.total) return;
    const int tx0 = (logical % a.tilesX) * SD_TW;
    const int ty0 = ((logical / a.tilesX) % a.tilesY) * SD_TH;
    const int b = logical / (a.tilesX * a.tilesY);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, g = lane >> 5;

    // ---- 0. input patch (four threads per (channel, patch row), nine consecutive columns each) and channel affines ---------------
    const int iy0 = 2 * ty0 - 2, ix0 = 2 * tx0 - 2;
    if (tid < 4 * 3 * SD_IH)
    {
        const int row = tid >> 2, c0 = (tid & 3) * 9;
        const int ci = row / SD_IH, r = row - ci * SD_IH;
        const int gy = iy0 + r;
        const bool rowOk = gy >= 0 && gy < a.H;
        const float *src = a.x + ((static_cast<size_t>(b) * 3 + ci) * a.H + (rowOk ? gy : 0)) * a.W;
        float *dst = imgL + row * SD_IP + c0;
        float v[9];
#pragma unroll
        for (int j = 0; j < 9; ++j)
        {
            const int gx = ix0 + c0 + j;
            v[j] = (rowOk && c0 + j < SD_IW && gx >= 0 && gx < a.W) ? src[gx] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 9; ++j) dst[j] = v[j];                  // (column 35 of the 36-wide row is padding)
    }
    // a positive power-of-two output scale commutes with relu / leaky / identity: folded into the channel affine then
    const bool hom1 = a.act1 == MSNH_ACT_NONE || a.act1 == MSNH_ACT_RELU || a.act1 == MSNH_ACT_LEAKY;
    const bool hom2 = a.act2 == MSNH_ACT_NONE || a.act2 == MSNH_ACT_RELU || a.act2 == MSNH_ACT_LEAKY;
    const float fold1 = hom1 ? a.midMul : 1.f, fold2 = hom2 ? a.outMul : 1.f;
    const float late1 = hom1 ? 1.f : a.midMul, late2 = hom2 ? 1.f : a.outMul;
    if (tid < 32) { aff[tid] = fold1 * (a.scale1 ? a.scale1[tid] : 1.f); aff[32 + tid] = fold1 * (a.shift1 ? a.shift1[tid] : 0.f); }
    if (tid < MB2 * 32) { aff[64 + tid] = fold2 * (a.scale2 ? a.scale2[tid] : 1.f); aff[64 + SD_MAXC2 + tid] = fold2 * (a.shift2 ? a.shift2[tid] : 0.f); }
    const bool hom3 = a.act3 == MSNH_ACT_NONE || a.act3 == MSNH_ACT_RELU || a.act3 == MSNH_ACT_LEAKY;
    const float fold3 = hom3 ? a.zMul : 1.f, late3 = hom3 ? 1.f : a.zMul;
    if (TAIL != 0 && tid < 32)
    {
        aff[64 + 2 * SD_MAXC2 + tid] = fold3 * (a.scale3 ? a.scale3[tid] : 1.f);
        aff[64 + 2 * SD_MAXC2 + 32 + tid] = fold3 * (a.shift3 ? a.shift3[tid] : 0.f);
    }
    const f16x8 w1a0 = *reinterpret_cast<const f16x8 *>(a.w1 + static_cast<size_t>(lane) * 8);
    const f16x8 w1a1 = *reinterpret_cast<const f16x8 *>(a.w1 + static_cast<size_t>(64 + lane) * 8);
    // the 1x1 tail's operand A, asked for here so that the epilogue does not wait for it
    f16x8 wa3[TAIL != 0 ? MB2 : 1][2];
    if constexpr (TAIL != 0)
    {
#pragma unroll
        for (int mb = 0; mb < MB2; ++mb)
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) wa3[mb][kb] = *reinterpret_cast<const f16x8 *>(a.w3 + static_cast<size_t>((mb * 2 + kb) * 64 + lane) * 8);
    }
    __syncthreads();

    // ---- 1. first layer over the 17 x 33 pixels under the tile ------------------------------------------------------------------
    for (int blk = wave; blk * 32 < SD_NPIX; blk += 4)
    {
        const int q = blk * 32 + n;
        const bool valid = q < SD_NPIX;
        const int sy = valid ? q / SD_SW : 0, sx = valid ? q % SD_SW : 0;
        const float *ip = imgL + sy * SD_IP + sx;
        f16x8 b0, b1;
        {
            // K group g of the first 16: channel g, taps 0..7
            const float *p = ip + g * (SD_IH * SD_IP);
#pragma unroll
            for (int e = 0; e < 8; ++e) b0[e] = static_cast<f16>(p[(e / 3) * SD_IP + e % 3]);
        }
        if (g == 0)
        {
            const float *p = ip + 2 * (SD_IH * SD_IP);             // K group 2: channel 2, taps 0..7
#pragma unroll
            for (int e = 0; e < 8; ++e) b1[e] = static_cast<f16>(p[(e / 3) * SD_IP + e % 3]);
        }
        else
        {
            const float *p = ip + 2 * SD_IP + 2;                    // K group 3: the ninth tap of the three channels, then zeros
#pragma unroll
            for (int e = 0; e < 8; ++e) b1[e] = e < 3 ? static_cast<f16>(p[e * (SD_IH * SD_IP)]) : static_cast<f16>(0.f);
        }
        f32x16 acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(w1a0, b0, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(w1a1, b1, acc, 0, 0, 0);
        const int gy = 2 * ty0 - 1 + sy, gx = 2 * tx0 - 1 + sx;
        const bool inside = valid && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W;
        float t[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) t[r] = acc[r] * aff[16 * g + r] + aff[32 + 16 * g + r];
        activateArray<16>(t, a.act1, a.act1Param);
        f16x8 o0, o1;
#pragma unroll
        for (int r = 0; r < 8; ++r) { o0[r] = static_cast<f16>(t[r] * late1); o1[r] = static_cast<f16>(t[8 + r] * late1); }
        if (!inside)
        {
#pragma unroll
            for (int r = 0; r < 8; ++r) { o0[r] = static_cast<f16>(0.f); o1[r] = static_cast<f16>(0.f); }
        }
        if (valid)
        {
            const int slot = sy * SD_SW + (sx & 1) * SD_EVEN + (sx >> 1);
            *reinterpret_cast<f16x8 *>(tileL + sdSlotAddr(slot, 2 * g)) = o0;
            *reinterpret_cast<f16x8 *>(tileL + sdSlotAddr(slot, 2 * g + 1)) = o1;
        }
    }
    __syncthreads();

    // ---- 2. second layer: this wavefront's 2 x 16 output pixels, all output channels ---------------------------------------------
    const int ty = 2 * wave + (n >> 4), tx = n & 15;
    const int slot0 = (2 * ty) * SD_SW + tx;
    f32x16 acc2[MB2];
#pragma unroll
    for (int mb = 0; mb < MB2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc2[mb][r] = 0.f;
    const f16 *wp = a.w2 + static_cast<size_t>(lane) * 8;
    f16x8 wa[2][2][MB2];                                            // [buffer][k block][channel block]
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int mb = 0; mb < MB2; ++mb) wa[0][kb][mb] = *reinterpret_cast<const f16x8 *>(wp + static_cast<size_t>((0 * 2 + kb) * MB2 + mb) * 512);
#pragma unroll
    for (int tap = 0; tap < 9; ++tap)
    {
        const int cur = tap & 1, nxt = cur ^ 1;
        if (tap + 1 < 9)
        {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int mb = 0; mb < MB2; ++mb)
                    wa[nxt][kb][mb] = *reinterpret_cast<const f16x8 *>(wp + static_cast<size_t>(((tap + 1) * 2 + kb) * MB2 + mb) * 512);
        }
        const int ky = tap / 3, kx = tap % 3;
        const int slot = slot0 + ky * SD_SW + (kx == 1 ? SD_EVEN : (kx == 2 ? 1 : 0));
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
        {
            const f16x8 bf = *reinterpret_cast<const f16x8 *>(tileL + sdSlotAddr(slot, 2 * kb + g));
#pragma unroll
            for (int mb = 0; mb < MB2; ++mb) acc2[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa[cur][kb][mb], bf, acc2[mb], 0, 0, 0);
        }
    }
    const int oy = ty0 + ty, ox = tx0 + tx;
    const bool store = oy < a.OH && ox < a.OW;
    const size_t pix = (static_cast<size_t>(b) * a.OH + (store ? oy : 0)) * a.OW + (store ? ox : 0);
    f16 *yp = a.y + pix * a.outLd + 16 * g;
    f32x16 accT;
#pragma unroll
    for (int r = 0; r < 16; ++r) accT[r] = 0.f;
#pragma unroll
    for (int mb = 0; mb < MB2; ++mb)
    {
        float t[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) t[r] = acc2[mb][r] * aff[64 + mb * 32 + 16 * g + r] + aff[64 + SD_MAXC2 + mb * 32 + 16 * g + r];
        activateArray<16>(t, a.act2, a.act2Param);
        f16x8 o0, o1;
#pragma unroll
        for (int r = 0; r < 8; ++r) { o0[r] = static_cast<f16>(t[r] * late2); o1[r] = static_cast<f16>(t[8 + r] * late2); }
        if (store)
        {
            *reinterpret_cast<f16x8 *>(yp + mb * 32) = o0;
            *reinterpret_cast<f16x8 *>(yp + mb * 32 + 8) = o1;
        }
        if constexpr (TAIL != 0)
        {
            // o0 / o1 = channels 16g .. 16g+7 / 16g+8 .. 16g+15 of this lane's pixel (within the 32 of block mb), as stored.  The B operand of
            // k-block kb wants channels 16 kb + 8g .. +7 from lane (pixel, g): after the swap x0 is that for kb = 0 and x1 for kb = 1
            // (g = 0 keeps o0 and receives its partner's o0 as x1; g = 1 keeps o1 and receives its partner's o1 as x0).
            typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
            typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
            u32x4 x0 = __builtin_bit_cast(u32x4, o0), x1 = __builtin_bit_cast(u32x4, o1);
#pragma unroll
            for (int d = 0; d < 4; ++d)
            {
                const u32x2 sw = __builtin_amdgcn_permlane32_swap(x0[d], x1[d], false, false);
                x0[d] = sw[0]; x1[d] = sw[1];
            }
            accT = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa3[mb][0], __builtin_bit_cast(f16x8, x0), accT, 0, 0, 0);
            accT = __builtin_amdgcn_mfma_f32_32x32x16_f16(wa3[mb][1], __builtin_bit_cast(f16x8, x1), accT, 0, 0, 0);
        }
    }
    if constexpr (TAIL != 0)
    {
        float t[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) t[r] = accT[r] * aff[64 + 2 * SD_MAXC2 + 16 * g + r] + aff[64 + 2 * SD_MAXC2 + 32 + 16 * g + r];
        activateArray<16>(t, a.act3, a.act3Param);
        f16x8 o0, o1;
#pragma unroll
        for (int r = 0; r < 8; ++r) { o0[r] = static_cast<f16>(t[r] * late3); o1[r] = static_cast<f16>(t[8 + r] * late3); }
        if (store)
        {
            f16 *zp = a.z + pix * a.zLd + 16 * g;
            *reinterpret_cast<f16x8 *>(zp) = o0;
            *reinterpret_cast<f16x8 *>(zp + 8) = o1;
        }
    }
}

// MFMA row m = 8q + 4h + e computes channel 16h + 4q + e
inline int sdChannelOfRow(int m) { return 16 * ((m >> 2) & 1) + 4 * (m >> 3) + (m & 3); }

inline uint16_t sdHalf(float f)
{
    const f16 h = static_cast<f16>(f);
    uint16_t u;
    std::memcpy(&u, &h, 2);
    return u;
}

} // namespace
} // namespace msnh

using namespace msnh;

extern "C" int msnh_hip_conv_stem_down_supported(int in_c, int c1, int k1, int s1, int p1, int c2, int k2, int s2, int p2)
{
    return in_c == 3 && c1 == 32 && k1 == 3 && s1 == 1 && p1 == 1 && (c2 == 32 || c2 == 64 || c2 == 128) && k2 == 3 && s2 == 2 && p2 == 1;
}

extern "C" size_t msnh_hip_conv_stem_down_packed_elems(int c2, int which)
{
    if (which == 0) return 2 * 64 * 8;
    return (c2 == 32 || c2 == 64 || c2 == 128) ? static_cast<size_t>(9) * 2 * (c2 / 32) * 64 * 8 : 0;
}

extern "C" int msnh_hip_conv_stem_down_pack(const float *w1, int c2, const float *w2, void *packed1, void *packed2)
{
    MSNH_REQUIRE(w1 && w2 && packed1 && packed2 && (c2 == 32 || c2 == 64 || c2 == 128), "conv_stem_down_pack: bad argument");
    uint16_t *p1 = static_cast<uint16_t *>(packed1), *p2 = static_cast<uint16_t *>(packed2);
    // first layer, w1[32][3][3][3] (filter, channel, ky, kx): K group G = 2 kb + lane / 32; G < 3: channel G, taps 0..7; G = 3: the ninth tap
    for (int kb = 0; kb < 2; ++kb)
        for (int lane = 0; lane < 64; ++lane)
            for (int e = 0; e < 8; ++e)
            {
                const int ch = sdChannelOfRow(lane & 31), G = 2 * kb + (lane >> 5);
                float v = 0.f;
                if (G < 3) v = w1[(ch * 3 + G) * 9 + e];
                else if (e < 3) v = w1[(ch * 3 + e) * 9 + 8];
                p1[(kb * 64 + lane) * 8 + e] = sdHalf(v);
            }
    // second layer, w2[c2][32][3][3]
    const int mb2 = c2 / 32;
    for (int tap = 0; tap < 9; ++tap)
        for (int kb = 0; kb < 2; ++kb)
            for (int mb = 0; mb < mb2; ++mb)
                for (int lane = 0; lane < 64; ++lane)
                    for (int e = 0; e < 8; ++e)
                    {
                        const int oc = mb * 32 + sdChannelOfRow(lane & 31), ic = kb * 16 + (lane >> 5) * 8 + e;
                        p2[((static_cast<size_t>(tap * 2 + kb) * mb2 + mb) * 64 + lane) * 8 + e] = sdHalf(w2[(static_cast<size_t>(oc) * 32 + ic) * 9 + tap]);
                    }
    return 0;
}

namespace {

int stemDownLaunch(int batch, int h, int w, const float *x, const void *packed1, const float *scale1, const float *shift1, int act1,
                   float act1_param, float mid_mul, int c2, const void *packed2, const float *scale2, const float *shift2, int act2,
                   float act2_param, float out_mul, void *y, int y_ld, const void *packed3, const float *scale3, const float *shift3, int act3,
                   float act3_param, float z_mul, void *z, int z_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(batch > 0 && h > 0 && w > 0 && x && packed1 && packed2 && y, "conv_stem_down: bad argument");
    MSNH_REQUIRE(c2 == 32 || c2 == 64 || c2 == 128, "conv_stem_down: the second layer must have 32, 64 or 128 filters");
    MSNH_REQUIRE(y_ld >= c2 && y_ld % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 && reinterpret_cast<uintptr_t>(packed1) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(packed2) % 16 == 0, "conv_stem_down: output and weights must be 16-byte aligned, y_ld a multiple of 8");
    const bool tail = packed3 != nullptr;
    if (tail)
        MSNH_REQUIRE(z && z_ld >= 32 && z_ld % 8 == 0 && reinterpret_cast<uintptr_t>(z) % 16 == 0 && reinterpret_cast<uintptr_t>(packed3) % 16 == 0 && actOk(act3),
                     "conv_stem_down_tail: z and the 1x1 filters must be 16-byte aligned, z_ld a multiple of 8");
    StemDownArgs a;
    a.x = x;
    a.w1 = static_cast<const f16 *>(packed1); a.scale1 = scale1; a.shift1 = shift1;
    a.w2 = static_cast<const f16 *>(packed2); a.scale2 = scale2; a.shift2 = shift2;
    a.y = static_cast<f16 *>(y);
    a.B = batch; a.H = h; a.W = w;
    a.OH = (h + 2 - 3) / 2 + 1; a.OW = (w + 2 - 3) / 2 + 1;
    a.outLd = y_ld;
    a.tilesX = (a.OW + SD_TW - 1) / SD_TW; a.tilesY = (a.OH + SD_TH - 1) / SD_TH;
    const long long total = static_cast<long long>(batch) * a.tilesX * a.tilesY;
    MSNH_REQUIRE(total < (1ll << 30), "conv_stem_down: too many tiles");
    a.total = static_cast<int>(total);
    a.act1 = act1; a.act1Param = act1_param; a.act2 = act2; a.act2Param = act2_param;
    a.midMul = mid_mul; a.outMul = out_mul;
    a.w3 = static_cast<const f16 *>(packed3); a.scale3 = scale3; a.shift3 = shift3; a.z = static_cast<f16 *>(z);
    a.zLd = z_ld; a.act3 = tail ? act3 : MSNH_ACT_NONE; a.act3Param = act3_param; a.zMul = z_mul;
    const dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8));
    hipStream_t st = resolveStream(s);
    if (tail)
    {
        if (c2 == 32) hipLaunchKernelGGL((convStemDownKernel<1, 1>), grid, dim3(256), 0, st, a);
        else if (c2 == 64) hipLaunchKernelGGL((convStemDownKernel<2, 1>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((convStemDownKernel<4, 1>), grid, dim3(256), 0, st, a);
    }
    else if (c2 == 32) hipLaunchKernelGGL((convStemDownKernel<1>), grid, dim3(256), 0, st, a);
    else if (c2 == 64) hipLaunchKernelGGL((convStemDownKernel<2>), grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((convStemDownKernel<4>), grid, dim3(256), 0, st, a);
    MSNH_LAUNCH_CHECK();
    return 0;
}

} // namespace

extern "C" int msnh_hip_conv_stem_down(int batch, int h, int w, const float *x, const void *packed1, const float *scale1, const float *shift1, int act1,
                                       float act1_param, float mid_mul, int c2, const void *packed2, const float *scale2, const float *shift2, int act2,
                                       float act2_param, float out_mul, void *y, int y_ld, msnh_stream_t s)
{
    return stemDownLaunch(batch, h, w, x, packed1, scale1, shift1, act1, act1_param, mid_mul, c2, packed2, scale2, shift2, act2, act2_param, out_mul, y, y_ld,
                          nullptr, nullptr, nullptr, MSNH_ACT_NONE, 0.f, 1.f, nullptr, 0, s);
}

extern "C" int msnh_hip_conv_stem_down_tail_supported(int c2, int c3, int k3, int s3, int p3)
{
    return (c2 == 32 || c2 == 64 || c2 == 128) && c3 == 32 && k3 == 1 && s3 == 1 && p3 == 0;
}

extern "C" size_t msnh_hip_conv_stem_down_tail_packed_elems(int c2)
{
    return (c2 == 32 || c2 == 64 || c2 == 128) ? static_cast<size_t>(c2 / 32) * 2 * 64 * 8 : 0;
}

extern "C" int msnh_hip_conv_stem_down_tail_pack(int c2, const float *w3, void *packed3)
{
    MSNH_REQUIRE(w3 && packed3 && (c2 == 32 || c2 == 64 || c2 == 128), "conv_stem_down_tail_pack: bad argument");
    // w3[32][c2] (filter, channel): operand A of k-block (mb, kb): lane (row, half) holds channels 32 mb + 16 kb + 8 half + 0..7 of filter sdChannelOfRow(row)
    uint16_t *p3 = static_cast<uint16_t *>(packed3);
    for (int mb = 0; mb < c2 / 32; ++mb)
        for (int kb = 0; kb < 2; ++kb)
            for (int lane = 0; lane < 64; ++lane)
                for (int e = 0; e < 8; ++e)
                {
                    const int oc = sdChannelOfRow(lane & 31), ic = mb * 32 + kb * 16 + (lane >> 5) * 8 + e;
                    p3[(static_cast<size_t>(mb * 2 + kb) * 64 + lane) * 8 + e] = sdHalf(w3[static_cast<size_t>(oc) * c2 + ic]);
                }
    return 0;
}

extern "C" int msnh_hip_conv_stem_down_tail(int batch, int h, int w, const float *x, const void *packed1, const float *scale1, const float *shift1, int act1,
                                            float act1_param, float mid_mul, int c2, const void *packed2, const float *scale2, const float *shift2, int act2,
                                            float act2_param, float out_mul, void *y, int y_ld, const void *packed3, const float *scale3, const float *shift3,
                                            int act3, float act3_param, float z_mul, void *z, int z_ld, msnh_stream_t s)
{
    MSNH_REQUIRE(packed3 && z, "conv_stem_down_tail: NULL pointer");
    return stemDownLaunch(batch, h, w, x, packed1, scale1, shift1, act1, act1_param, mid_mul, c2, packed2, scale2, shift2, act2, act2_param, out_mul, y, y_ld,
                          packed3, scale3, shift3, act3, act3_param, z_mul, z, z_ld, s);
}
