// post_norm.hip — the float32 residual stream of post-norm hybrid decoders and their gated feed-forward activation.
//
//   rms_norm          h = T(x / sqrt(mean(x^2) + eps) * w)                       (the model's final norm)
//   scale_add_rms     x <- (alpha x + y) / sqrt(mean((alpha x + y)^2) + eps) * w;  h = T(x)
//                     The norm sits AFTER the residual sum, so the stream itself is what the next sublayer reads:
//                     one kernel reads the sublayer output y (activation type) and the stream, does all arithmetic in
//                     float, rewrites the stream in place and emits its copy in the activation type.
//   glu               y = g sigmoid(slope g) (u + shift),  g = min(gate, limit),  u = clamp(up, -limit, limit), from
//                     a [T, 2F] projection whose first F columns are the gate and last F the up part.
//   decay_pow         z <- sigmoid(z)^p through exp(p log sigmoid(z)), float, in place (per-channel decays).
//
// Rows whose width is a multiple of 4 move 16 bytes (float) / 8 bytes (bfloat16) per lane and keep up to 16 values per
// thread in registers between the statistics pass and the write pass (d <= 4096 is read once).
#include "hybrid_common.h"

namespace chronos {
namespace hy {

template <typename T> __device__ __forceinline__ f32x4 ld4(const T* p);
template <> __device__ __forceinline__ f32x4 ld4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <> __device__ __forceinline__ f32x4 ld4<uint16_t>(const uint16_t* p) {
    const u16x4 v = *reinterpret_cast<const u16x4*>(p);
    return f32x4{bf2f(v[0]), bf2f(v[1]), bf2f(v[2]), bf2f(v[3])};
}
template <typename T> __device__ __forceinline__ void st4(T* p, const f32x4& v);
template <> __device__ __forceinline__ void st4<float>(float* p, const f32x4& v) { *reinterpret_cast<f32x4*>(p) = v; }
template <> __device__ __forceinline__ void st4<uint16_t>(uint16_t* p, const f32x4& v) {
    *reinterpret_cast<u16x4*>(p) = u16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}

// JOIN: v = alpha * x + y (y in TY), x <- norm(v) * w, h <- TH(x).   plain: v = x (float), h <- TH(norm(v) * w).
template <typename TY, typename TH, bool JOIN, bool VEC>
__global__ void __launch_bounds__(256) rms_norm_kernel(const TY* __restrict__ y, float* __restrict__ x,
                                                       const float* __restrict__ w, TH* __restrict__ h, int d,
                                                       float alpha, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float* xr = x + row * d;
    const TY* yr = JOIN ? y + row * d : nullptr;
    TH* hr = h != nullptr ? h + row * d : nullptr;
    float ss = 0.f;
    if constexpr (VEC) {
        f32x4 c[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            c[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (i < d) {
                f32x4 v = *reinterpret_cast<const f32x4*>(xr + i);
                if constexpr (JOIN) v = v * alpha + ld4<TY>(yr + i);
                c[j] = v;
                ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
            }
        }
        for (int i = (threadIdx.x + 1024) * 4; i < d; i += 1024) {
            f32x4 v = *reinterpret_cast<const f32x4*>(xr + i);
            if constexpr (JOIN) v = v * alpha + ld4<TY>(yr + i);
            ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        }
        const float rstd = 1.f / sqrtf(block_sum(ss, red) / (float)d + eps);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = (threadIdx.x + 256 * j) * 4;
            if (i < d) {
                const f32x4 v = c[j] * rstd * *reinterpret_cast<const f32x4*>(w + i);
                if constexpr (JOIN) *reinterpret_cast<f32x4*>(xr + i) = v;
                if (hr != nullptr) st4<TH>(hr + i, v);
            }
        }
        for (int i = (threadIdx.x + 1024) * 4; i < d; i += 1024) {
            f32x4 v = *reinterpret_cast<const f32x4*>(xr + i);
            if constexpr (JOIN) v = v * alpha + ld4<TY>(yr + i);
            v = v * rstd * *reinterpret_cast<const f32x4*>(w + i);
            if constexpr (JOIN) *reinterpret_cast<f32x4*>(xr + i) = v;
            if (hr != nullptr) st4<TH>(hr + i, v);
        }
    } else {
        for (int i = threadIdx.x; i < d; i += 256) {
            float v = xr[i];
            if constexpr (JOIN) v = v * alpha + ld<TY>(yr + i);
            ss += v * v;
        }
        const float rstd = 1.f / sqrtf(block_sum(ss, red) / (float)d + eps);
        for (int i = threadIdx.x; i < d; i += 256) {
            float v = xr[i];
            if constexpr (JOIN) v = v * alpha + ld<TY>(yr + i);
            v = v * rstd * w[i];
            if constexpr (JOIN) xr[i] = v;
            if (hr != nullptr) st<TH>(hr + i, v);
        }
    }
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256) glu_kernel(const T* __restrict__ gu, T* __restrict__ y, int64_t rows, int F,
                                                  float limit, float slope, float shift) {
    constexpr int E = VEC ? 4 : 1;
    const int64_t per = F / E;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * per) return;
    const int64_t r = i / per;
    const int c = (int)(i % per) * E;
    const T* g = gu + r * 2 * F + c;
    if constexpr (VEC) {
        const f32x4 gv = ld4<T>(g), uv = ld4<T>(g + F);
        f32x4 o;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float a = fminf(gv[k], limit), u = fminf(fmaxf(uv[k], -limit), limit);
            o[k] = a * sigmoidf_(slope * a) * (u + shift);
        }
        st4<T>(y + r * F + c, o);
    } else {
        const float a = fminf(ld<T>(g), limit), u = fminf(fmaxf(ld<T>(g + F), -limit), limit);
        st<T>(y + r * F + c, a * sigmoidf_(slope * a) * (u + shift));
    }
}

__global__ void __launch_bounds__(256) decay_pow_kernel(float* __restrict__ z, int64_t n, float p) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) z[i] = expf(logsigmoidf_(z[i]) * p);
}

}  // namespace hy

// y == nullptr: plain norm of x (h in float when out_f32, else bfloat16).  Otherwise the joined form; y is in the
// activation type (float when out_f32), h may be nullptr (float activations read the stream itself).
void launch_hy_rms_norm(const void* y, float* x, const float* w, void* h, bool out_f32, int rows, int d, float alpha,
                        float eps, hipStream_t s) {
    if (rows == 0) return;
    const bool vec = d % 4 == 0;
#define HY_RN(TY, TH, JOIN)                                                                                           \
    do {                                                                                                              \
        if (vec) hy::rms_norm_kernel<TY, TH, JOIN, true><<<rows, 256, 0, s>>>((const TY*)y, x, w, (TH*)h, d, alpha, eps); \
        else hy::rms_norm_kernel<TY, TH, JOIN, false><<<rows, 256, 0, s>>>((const TY*)y, x, w, (TH*)h, d, alpha, eps);    \
    } while (0)
    if (y != nullptr) {
        if (out_f32) HY_RN(float, float, true);
        else HY_RN(uint16_t, uint16_t, true);
    } else {
        if (out_f32) HY_RN(float, float, false);
        else HY_RN(float, uint16_t, false);
    }
#undef HY_RN
}

void launch_hy_glu(const void* gu, void* y, int64_t rows, int F, float limit, float slope, float shift, bool f32,
                   hipStream_t s) {
    if (rows == 0 || F == 0) return;
    const bool vec = F % 4 == 0;
    const int64_t n = rows * (vec ? F / 4 : F);
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (f32) {
        if (vec) hy::glu_kernel<float, true><<<blocks, 256, 0, s>>>((const float*)gu, (float*)y, rows, F, limit, slope, shift);
        else hy::glu_kernel<float, false><<<blocks, 256, 0, s>>>((const float*)gu, (float*)y, rows, F, limit, slope, shift);
    } else {
        if (vec) hy::glu_kernel<uint16_t, true><<<blocks, 256, 0, s>>>((const uint16_t*)gu, (uint16_t*)y, rows, F, limit, slope, shift);
        else hy::glu_kernel<uint16_t, false><<<blocks, 256, 0, s>>>((const uint16_t*)gu, (uint16_t*)y, rows, F, limit, slope, shift);
    }
}

void launch_hy_decay_pow(float* z, int64_t n, float p, hipStream_t s) {
    if (n == 0) return;
    hy::decay_pow_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(z, n, p);
}

}  // namespace chronos
