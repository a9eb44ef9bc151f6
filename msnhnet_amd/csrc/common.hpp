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

// ---- activations: the reference's scalar formulas (include/Msnhnet/layers/MsnhActivations.h:39-168) ----
__device__ __forceinline__ float softplusThr(float x, float thr)
{
    if (x > thr) return x;
    if (x < -thr) return expf(x);
    return logf(expf(x) + 1.f);
}

__device__ __forceinline__ float activate(float x, int act, float param)
{
    switch (act)
    {
    case MSNH_ACT_LOGISTIC: return 1.f / (1.f + expf(-x));
    case MSNH_ACT_RELU:     return x > 0.f ? x : 0.f * x;          // x*(x>0): keeps NaN, -0
    case MSNH_ACT_RELU6:    return (x > 0.f ? x : 0.f) > 6.f ? 6.f : (x > 0.f ? x : 0.f);
    case MSNH_ACT_LEAKY:    return x > 0.f ? x : param * x;
    case MSNH_ACT_SWISH:    return x * (1.f / (1.f + expf(-x)));
    case MSNH_ACT_MISH:     return x * tanhf(softplusThr(x, 20.f));
    default:                return x;
    }
}

inline bool actOk(int act)
{
    return act == MSNH_ACT_LOGISTIC || act == MSNH_ACT_RELU || act == MSNH_ACT_RELU6 || act == MSNH_ACT_LEAKY ||
           act == MSNH_ACT_SWISH || act == MSNH_ACT_MISH || act == MSNH_ACT_NONE;
}

inline unsigned gridFor(long long n, int block)
{
    long long g = (n + block - 1) / block;
    if (g < 1) g = 1;
    return static_cast<unsigned>(g);
}

} // namespace msnh
