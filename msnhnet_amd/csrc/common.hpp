// Shared device/host helpers of the gfx950 kernel library.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstdio>
#include <cstdarg>
#include <cstring>
#include <cfloat>
#include "msnh_hip.h"

namespace msnh {

// ---- error reporting ------------------------------------------------------------------------------
void setError(const char *fmt, ...);
hipStream_t resolveStream(msnh_stream_t s);
void yoloNmsSetupDevice();           // per-device set-up of the device NMS (csrc/yolo.hip) on the current device; failures are reported by the calls that need it

#define MSNH_HIP_CHECK(expr)                                                                      \
    do {                                                                                          \
        hipError_t err__ = (expr);                                                                \
        if (err__ != hipSuccess) {                                                                \
            msnh::setError("%s failed: %s (%s:%d)", #expr, hipGetErrorString(err__), __FILE__, __LINE__); \
            return 1;                                                                             \
        }                                                                                         \
    } while (0)

#define MSNH_REQUIRE(cond, ...)                                                                   \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            msnh::setError(__VA_ARGS__);                                                          \
            return 2;                                                                             \
        }                                                                                         \
    } while (0)

#define MSNH_LAUNCH_CHECK()                                                                       \
    do {                                                                                          \
        hipError_t err__ = hipGetLastError();                                                     \
        if (err__ != hipSuccess) {                                                                \
            msnh::setError("kernel launch failed: %s (%s:%d)", hipGetErrorString(err__), __FILE__, __LINE__); \
            return 1;                                                                             \
        }                                                                                         \
    } while (0)

// ---- element types --------------------------------------------------------------------------------
typedef _Float16 f16;
typedef f16   f16x2 __attribute__((ext_vector_type(2)));
typedef f16   f16x4 __attribute__((ext_vector_type(4)));
typedef f16   f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <typename T> struct DType;
template <> struct DType<float> { static constexpr int id = MSNH_F32; static constexpr int vec = 4; };
template <> struct DType<f16>   { static constexpr int id = MSNH_F16; static constexpr int vec = 8; };

inline size_t dtypeSize(int dtype) { return dtype == MSNH_F16 ? 2 : 4; }
inline bool   dtypeOk(int dtype) { return dtype == MSNH_F16 || dtype == MSNH_F32; }

__device__ __forceinline__ float toF(float v) { return v; }
__device__ __forceinline__ float toF(f16 v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T fromF(float v);
template <> __device__ __forceinline__ float fromF<float>(float v) { return v; }
template <> __device__ __forceinline__ f16 fromF<f16>(float v) { return static_cast<f16>(v); }

// ---- activations: the reference's scalar formulas (include/Msnhnet/layers/MsnhActivations.h:39-168), with the
// transcendental ones rearranged so that each costs one hardware exp2 and one hardware reciprocal (about 1e-6
// relative; on the epilogue of a bandwidth-bound convolution the library expf / logf / tanhf sequence of mish
// otherwise takes longer than the memory traffic):
//   logistic(x) = 1 / (1 + e^-x)
//   mish(x)     = x * tanh(softplus(x)) = x * n / (n + 2),  n = w (w + 2),  w = e^x
//                 (tanh(ln(1 + w)) = ((1+w)^2 - 1) / ((1+w)^2 + 1)); the reference's softplus thresholds at +-20 only
//                 guard its own overflow: beyond +20 the quotient is 1 to float precision, below -20 it is w
__device__ __forceinline__ float fastRcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ float logisticF(float x) { return fastRcp(1.f + __expf(-x)); }

__device__ __forceinline__ float mishF(float x)
{
    const float w = __expf(x < 20.f ? x : 20.f);
    const float n = w * (w + 2.f);
    return x * (n * fastRcp(n + 2.f));
}

__device__ __forceinline__ float activate(float x, int act, float param)
{
    switch (act)
    {
    case MSNH_ACT_LOGISTIC: return logisticF(x);
    case MSNH_ACT_RELU:     return x > 0.f ? x : 0.f * x;          // x*(x>0): keeps NaN, -0
    case MSNH_ACT_RELU6:    return (x > 0.f ? x : 0.f) > 6.f ? 6.f : (x > 0.f ? x : 0.f);
    case MSNH_ACT_LEAKY:    return x > 0.f ? x : param * x;
    case MSNH_ACT_SWISH:    return x * logisticF(x);
    case MSNH_ACT_HARD_SWISH:
    {
        const float t = x + 3.f;
        const float r = (t > 0.f ? t : 0.f) > 6.f ? 6.f : (t > 0.f ? t : 0.f);
        return x * r / 6.f;                                     // x*relu6(x+3)/6, evaluated in that order
    }
    case MSNH_ACT_MISH:     return mishF(x);
    default:                return x;
    }
}

// The same over a register array with the choice of the activation made once, outside the element loop: a kernel that
// calls activate() per element of an unrolled epilogue carries one copy of the whole switch per element.
template <int N> __device__ __forceinline__ void activateArray(float (&v)[N], int act, float param)
{
    switch (act)
    {
    case MSNH_ACT_NONE: break;
    case MSNH_ACT_RELU:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = v[i] > 0.f ? v[i] : 0.f * v[i];
        break;
    case MSNH_ACT_LEAKY:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = v[i] > 0.f ? v[i] : param * v[i];
        break;
    case MSNH_ACT_RELU6:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = activate(v[i], MSNH_ACT_RELU6, param);
        break;
    case MSNH_ACT_LOGISTIC:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = logisticF(v[i]);
        break;
    case MSNH_ACT_SWISH:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = v[i] * logisticF(v[i]);
        break;
    case MSNH_ACT_HARD_SWISH:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = activate(v[i], MSNH_ACT_HARD_SWISH, param);
        break;
    case MSNH_ACT_MISH:
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = mishF(v[i]);
        break;
    default: break;
    }
}

inline bool actOk(int act)
{
    return act == MSNH_ACT_LOGISTIC || act == MSNH_ACT_RELU || act == MSNH_ACT_RELU6 || act == MSNH_ACT_LEAKY ||
           act == MSNH_ACT_SWISH || act == MSNH_ACT_HARD_SWISH || act == MSNH_ACT_MISH || act == MSNH_ACT_NONE;
}

// Division of a 32-bit unsigned by a divisor known on the host: multiplication by a precomputed reciprocal (Granlund & Montgomery,
// "Division by invariant integers using multiplication", figure 4.1); exact for every 32-bit dividend.
struct FastDiv { unsigned m, s1, s2, d; };

inline FastDiv makeFastDiv(unsigned d)
{
    unsigned l = 0;
    while ((1ull << l) < d) ++l;                     // ceil(log2 d)
    FastDiv f;
    f.m = static_cast<unsigned>(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 1 ? l - 1 : 0;
    f.d = d;
    return f;
}

__device__ __forceinline__ unsigned fastDiv(unsigned n, const FastDiv &f)
{
    const unsigned t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

inline unsigned gridFor(long long n, int block)
{
    long long g = (n + block - 1) / block;
    if (g < 1) g = 1;
    return static_cast<unsigned>(g);
}

} // namespace msnh
