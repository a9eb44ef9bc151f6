// Timing diagnostics for convPatch8Kernel (include/msnh_hip_diag.h): the kernel instantiated with its timing switches.
// A library of its own, so that the kernel library carries only the switch-free instantiations.
#include "msnh_hip_diag.h"
#include "conv_igemm.hpp"        // (brings conv_patch8.hpp with it)
#include <cstring>

using namespace msnh;

namespace {

constexpr int kSwitches[] = {0, 1, 2, 3, 4, 5, 7, 8, 9, 10, 11, 15, 16, 31, 47, 63, 64, 65, 66, 71, 72};
constexpr int kCount = static_cast<int>(sizeof(kSwitches) / sizeof(kSwitches[0]));

template <int BM, int BN, int WM, int WN, int NSA, int PS, int KG, int I = 0>
int launchWith(int switches, IgemmArgs &a, hipStream_t st)
{
    if constexpr (I == kCount) return -1;
    else
    {
        if (switches == kSwitches[I]) return launchPatch8<f16, f16, BM, BN, WM, WN, NSA, PS, kSwitches[I], KG>(a, 1, st);
        return launchWith<BM, BN, WM, WN, NSA, PS, KG, I + 1>(switches, a, st);
    }
}

__global__ void emptyKernel(int *p)
{
    if (p && threadIdx.x == 0x7fffffff) *p = 1;
}

} // namespace

extern "C" int msnh_hip_diag_patch8_switches(int *out, int cap)
{
    for (int i = 0; i < kCount && i < cap; ++i)
        if (out) out[i] = kSwitches[i];
    return kCount;
}

extern "C" int msnh_hip_diag_empty_launch(int blocks, int threads, msnh_stream_t s)
{
    if (blocks < 1 || threads < 1 || threads > 1024) return 1;
    hipLaunchKernelGGL(emptyKernel, dim3(blocks), dim3(threads), 0, resolveStream(s), nullptr);
    return hipGetLastError() == hipSuccess ? 0 : 1;
}

extern "C" int msnh_hip_diag_patch8(int tile, int switches, int batch, int c, int h, int w, int oc, const void *x, const void *wt, const float *scale,
                                const float *shift, void *y, void *clocks, msnh_stream_t s)
{
    if (!x || !wt || !scale || !shift || !y) return 1;
    if (batch < 1 || h < 1 || w < 1 || c < 64 || c % 64 || oc < 64 || oc % 64) return 2;
    if ((switches & 64) && !clocks) return 3;
    const unsigned long long xBytes = static_cast<unsigned long long>(batch) * h * w * c * 2ull;
    const unsigned long long wBytes = static_cast<unsigned long long>(oc) * 9ull * c * 2ull;
    if (xBytes >= 0x7fffffffull || wBytes >= 0x7fffffffull || static_cast<unsigned long long>(batch) * h * w * oc * 2ull >= 0x7fffffffull) return 4;
    IgemmArgs a;
    std::memset(&a, 0, sizeof(a));
    a.x = x; a.w = wt; a.scale = scale; a.shift = shift; a.res = nullptr; a.y = y;
    a.batch = batch; a.H = h; a.W = w; a.inLd = c; a.OH = h; a.OW = w; a.outLd = oc; a.resLd = oc;
    a.cinG = c; a.coutG = oc; a.taps = 9; a.ksize = 3; a.stride = 1; a.pad = 1; a.dil = 1;
    a.P = batch * h * w; a.patchOk = 1; a.buffersOk = 1;
    a.byOW = makeFastDiv(static_cast<unsigned>(w));
    a.byOH = makeFastDiv(static_cast<unsigned>(h));
    a.xBytes = static_cast<unsigned>(xBytes);
    a.wBytes = static_cast<unsigned>(wBytes);
    a.act = MSNH_ACT_LEAKY; a.act2 = MSNH_ACT_NONE; a.actParam = 0.1f; a.resMul = 1.f; a.outMul = 1.f; a.vecOk = 1; a.wsLd = oc;
    a.ws = static_cast<float *>(clocks);
    hipStream_t st = resolveStream(s);
    int rc = -1;
    if (tile == 46) rc = launchWith<64, 384, 2, 6, 3, 1, 1>(switches, a, st);
    else if (tile == 52) rc = launchWith<64, 384, 1, 6, 3, 1, 2>(switches, a, st);
    else return 5;
    if (rc == -1) return 6;          // a combination that is not instantiated
    return rc == 0 ? 0 : 7;          // (the launcher's own refusal: the tile does not fit this shape)
}
