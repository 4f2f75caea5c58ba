// hybrid_common.h — helpers shared by the hybrid-decoder kernels (csrc/hybrid/*.hip).
//
// Every kernel is instantiated for two activation element types: bfloat16 travelling as raw 16-bit words
// (uint16_t, as in csrc/kernels) and float.  Whatever the activation type, residual stream, norms, recurrent state,
// gates, router and attention scores are float.
#pragma once
#include "chronos_hip.h"

namespace chronos {
namespace hy {

template <typename T> __device__ __forceinline__ float ld(const T* p);
template <> __device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld<uint16_t>(const uint16_t* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void st(T* p, float v);
template <> __device__ __forceinline__ void st<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st<uint16_t>(uint16_t* p, float v) { *p = f2bf(v); }

// round a float through the activation type (what a value stored and read back would be)
template <typename T> __device__ __forceinline__ float rnd(float v);
template <> __device__ __forceinline__ float rnd<float>(float v) { return v; }
template <> __device__ __forceinline__ float rnd<uint16_t>(float v) { return bf2f(f2bf(v)); }

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
// log(sigmoid(z)) without overflow on either side
__device__ __forceinline__ float logsigmoidf_(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

constexpr int kActRelu2 = 0, kActGelu = 1;
__device__ __forceinline__ float act_apply(float z, int kind) {
    if (kind == kActRelu2) {
        const float r = fmaxf(z, 0.f);
        return r * r;
    }
    return 0.5f * z * (1.f + erff(z * 0.70710678118654752440f));
}

}  // namespace hy
}  // namespace chronos
