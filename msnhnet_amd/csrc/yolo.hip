// YOLO v3/v4 head decode fused with the [anchor][channel][pixel] -> [anchor][pixel][channel] reordering and
// the objectness threshold.  The NHWC head tensor already stores the (5+classes) values of one anchor of
// one pixel contiguously, so both the read and the write of a wavefront are contiguous runs.
#include "common.hpp"

namespace msnh {

struct Anchors { float v[6]; };

template <typename T>
__global__ __launch_bounds__(256) void yoloDecodeKernel(const T *__restrict__ x, int xLd, float xMul, Anchors an, float ratio,
                                                        float *__restrict__ decoded, float confThresh, int *__restrict__ candIdx,
                                                        int candCap, int candBase, int *__restrict__ candCnt, int W, int HW, int per,
                                                        long long total)
{
    long long idx = static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const int m = static_cast<int>(idx % per);
    long long t = idx / per;
    const int p = static_cast<int>(t % HW);
    t /= HW;
    const int a = static_cast<int>(t % 3);
    const int b = static_cast<int>(t / 3);
    const float v = xMul * toF(x[(static_cast<size_t>(b) * HW + p) * xLd + a * per + m]);
    float r;
    if (m == 0)      r = (1.f / (1.f + expf(-v)) + static_cast<float>(p % W)) * ratio;
    else if (m == 1) r = (1.f / (1.f + expf(-v)) + static_cast<float>(p / W)) * ratio;
    else if (m == 2) r = an.v[2 * a] * expf(v);
    else if (m == 3) r = an.v[2 * a + 1] * expf(v);
    else             r = 1.f / (1.f + expf(-v));
    decoded[idx] = r;
    if (m == 4 && candIdx != nullptr && r > confThresh)
    {
        const int pos = atomicAdd(candCnt + b, 1);
        if (pos < candCap) candIdx[static_cast<size_t>(b) * candCap + pos] = candBase + a * HW + p;
    }
}

} // namespace msnh

using namespace msnh;

extern "C" int msnh_hip_yolo_decode(int dtype, int batch, int h, int w, int classes, const void *x, int x_ld, float x_mul,
                                    const float *anchors6, float ratio, float *decoded, float conf_thresh, int *cand_idx,
                                    int cand_cap, int cand_base, int *cand_cnt, msnh_stream_t s)
{
    MSNH_REQUIRE(dtypeOk(dtype), "yolo_decode: bad dtype");
    MSNH_REQUIRE(batch > 0 && h > 0 && w > 0 && classes > 0, "yolo_decode: bad geometry");
    const int per = 5 + classes;
    MSNH_REQUIRE(x && decoded && anchors6 && x_ld >= 3 * per, "yolo_decode: bad argument");
    MSNH_REQUIRE(cand_idx == nullptr || (cand_cnt != nullptr && cand_cap > 0), "yolo_decode: candidate list without counter");
    Anchors an;
    for (int i = 0; i < 6; ++i) an.v[i] = anchors6[i];
    const long long total = static_cast<long long>(batch) * 3 * h * w * per;
    dim3 grid(gridFor(total, 256));
    hipStream_t st = resolveStream(s);
    if (dtype == MSNH_F16)
        hipLaunchKernelGGL((yoloDecodeKernel<f16>), grid, dim3(256), 0, st, static_cast<const f16 *>(x), x_ld, x_mul, an, ratio, decoded,
                           conf_thresh, cand_idx, cand_cap, cand_base, cand_cnt, w, h * w, per, total);
    else
        hipLaunchKernelGGL((yoloDecodeKernel<float>), grid, dim3(256), 0, st, static_cast<const float *>(x), x_ld, x_mul, an, ratio,
                           decoded, conf_thresh, cand_idx, cand_cap, cand_base, cand_cnt, w, h * w, per, total);
    MSNH_LAUNCH_CHECK();
    return 0;
}
