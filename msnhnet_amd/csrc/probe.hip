// A matrix-core ceiling probe: nothing but 32x32x16 float16 MFMAs on every SIMD, no memory traffic, with the shader clock read
// beside the constant-rate clock.  What it reports is the rate the matrix cores sustain on this part under full load (the
// published peak assumes the maximum engine clock, which a fully loaded part does not hold) -- the practical ceiling beside
// which the convolution kernels' rates are to be read.  Measurement only; no forward launches it.
#include "common.hpp"

namespace msnh {

typedef _Float16 probeH8 __attribute__((ext_vector_type(8)));
typedef float probeF16 __attribute__((ext_vector_type(16)));

// Each wavefront cycles over four independent accumulators (as the convolution kernels' 64 x 64 wave tiles do), so no MFMA
// waits for the previous one's result.
__global__ __launch_bounds__(256) void mfmaProbeKernel(int iters, float *sink, unsigned long long *clocks)
{
    probeH8 a, b;
    for (int i = 0; i < 8; ++i) { a[i] = static_cast<_Float16>(0.001f * (threadIdx.x & 7)); b[i] = static_cast<_Float16>(0.002f * (i + 1)); }
    probeF16 c0, c1, c2, c3;
    for (int i = 0; i < 16; ++i) { c0[i] = 0.f; c1[i] = 0.f; c2[i] = 0.f; c3[i] = 0.f; }
    const unsigned long long t0 = __builtin_readcyclecounter();
    const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it)
    {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c1, 0, 0, 0);
        c2 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c2, 0, 0, 0);
        c3 = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c3, 0, 0, 0);
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
    float s = 0.f;
    for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
    if (s == 12345.678f) sink[0] = s;                // keeps the MFMAs alive; never true
    if (blockIdx.x == 0 && threadIdx.x == 0) { clocks[0] = t1 - t0; clocks[1] = r1 - r0; }
}

} // namespace msnh

using namespace msnh;

// waves_per_simd: 1 .. 8 wavefronts resident on every SIMD (the grid is 256 CUs x waves_per_simd workgroups of four wavefronts;
// more workgroups than fit queue up, so values above the occupancy limit only lengthen the run).
extern "C" int msnh_hip_mfma_probe(int waves_per_simd, int iters, double *tflops, double *shader_mhz, double *seconds, msnh_stream_t s)
{
    MSNH_REQUIRE(waves_per_simd >= 1 && waves_per_simd <= 8 && iters >= 1 && iters <= (1 << 24), "mfma_probe: 1..8 wavefronts per SIMD, 1..2^24 iterations");
    MSNH_REQUIRE(tflops && shader_mhz && seconds, "mfma_probe: NULL result pointer");
    hipStream_t st = resolveStream(s);
    int cus = 0;
    MSNH_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
    float *sink = nullptr;
    unsigned long long *clocks = nullptr;
    MSNH_HIP_CHECK(hipMalloc(&sink, 256));
    if (hipMalloc(&clocks, 256) != hipSuccess) { (void)hipFree(sink); setError("mfma_probe: out of device memory"); return 1; }
    hipEvent_t e0 = nullptr, e1 = nullptr;
    MSNH_HIP_CHECK(hipEventCreate(&e0));
    MSNH_HIP_CHECK(hipEventCreate(&e1));
    const int grid = cus * waves_per_simd;
    hipLaunchKernelGGL(mfmaProbeKernel, dim3(grid), dim3(256), 0, st, iters / 8 + 1, sink, clocks);      // clocks up, caches warm
    MSNH_HIP_CHECK(hipEventRecord(e0, st));
    hipLaunchKernelGGL(mfmaProbeKernel, dim3(grid), dim3(256), 0, st, iters, sink, clocks);
    MSNH_HIP_CHECK(hipEventRecord(e1, st));
    MSNH_HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0.f;
    MSNH_HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    unsigned long long h[2] = {0, 0};
    MSNH_HIP_CHECK(hipMemcpy(h, clocks, sizeof(h), hipMemcpyDeviceToHost));
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    (void)hipFree(sink); (void)hipFree(clocks);
    const double flops = static_cast<double>(grid) * 4.0 * iters * 4.0 * (2.0 * 32 * 32 * 16);
    *seconds = ms * 1e-3;
    *tflops = flops / (ms * 1e-3) / 1e12;
    // the constant-rate clock runs at 100 MHz
    *shader_mhz = h[1] ? static_cast<double>(h[0]) / static_cast<double>(h[1]) * 100.0 : 0.0;
    return 0;
}
