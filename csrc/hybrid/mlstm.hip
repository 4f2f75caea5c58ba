// mlstm.hip — the matrix-memory recurrence (mLSTM) over the engine's flattened token stream, prefill chunks and
// decode rows alike.  Per head: state S (D x Dv), normaliser n (D), running maximum m, all float and carried
// between steps in per-sequence state slots.
//
//   i_t = cap tanh(zi / cap)                       (log input gate)
//   f_t = logsigmoid(cap tanh(zf / cap))           (log forget gate)
//   m_t = max(f_t + m_{t-1}, i_t)                  a_t = exp(f_t + m_{t-1} - m_t)     b_t = exp(i_t - m_t)
//   S_t = a_t S_{t-1} + b_t k_t v_t^T              n_t = a_t n_{t-1} + b_t k_t
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),   q_t scaled by D^-1/2
//
// Three launches:
//   gate_scan    one wave per (sequence, head): the scalar recurrences a_t, b_t and the denominators (n lives in the
//                wave's lanes); sequential in t but only O(D) work per token;
//   state_scan   one workgroup per (sequence, head, 64 value columns): S in registers (lane = column, the D rows
//                split over 4 waves), tokens staged through LDS 8 at a time, the waves' partial read-outs summed
//                once per 8 tokens;
//   out_norm     per-head unit RMS of the read-out, the head-concatenated weight, the sigmoid output gate.
// A sequence whose first token in this step is at position 0 starts from the zero state (m = 0); otherwise from its
// slot.  Sequences with no tokens in the step are left alone.
#include "hybrid_common.h"

namespace chronos {
namespace hy {

template <typename T>
__global__ void __launch_bounds__(64) mlstm_gate_scan_kernel(
        const T* __restrict__ proj, int ldp, const float* __restrict__ gate_pre, const int32_t* __restrict__ q_start,
        const int32_t* __restrict__ pos0, const int32_t* __restrict__ slots, float* __restrict__ n_state,
        float* __restrict__ m_state, float* __restrict__ a_out, float* __restrict__ b_out, float* __restrict__ den_out,
        int H, int D, float cap) {
    const int b = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    if (t1 <= t0) return;
    const int slot = slots[b];
    const bool fresh = pos0[b] == 0;
    constexpr int NL = 8;  // D <= 512
    float n[NL];
    float* ns = n_state + ((int64_t)slot * H + hd) * D;
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int dd = lane + 64 * j;
        n[j] = (!fresh && dd < D) ? ns[dd] : 0.f;
    }
    float m = fresh ? 0.f : m_state[(int64_t)slot * H + hd];
    const float qs = 1.f / sqrtf((float)D);
    for (int t = t0; t < t1; ++t) {
        const float zi = gate_pre[(int64_t)t * 2 * H + hd], zf = gate_pre[(int64_t)t * 2 * H + H + hd];
        const float ig = cap * tanhf(zi / cap);
        const float fg = logsigmoidf_(cap * tanhf(zf / cap));
        const float mn = fmaxf(fg + m, ig);
        const float a = expf(fg + m - mn), bb = expf(ig - mn);
        m = mn;
        const T* q = proj + (int64_t)t * ldp + hd * D;
        const T* k = proj + (int64_t)t * ldp + H * D + hd * D;
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const int dd = lane + 64 * j;
            if (dd < D) {
                n[j] = a * n[j] + bb * ld<T>(k + dd);
                dot += n[j] * (ld<T>(q + dd) * qs);
            }
        }
        dot = wave_sum(dot);
        if (lane == 0) {
            a_out[(int64_t)t * H + hd] = a;
            b_out[(int64_t)t * H + hd] = bb;
            den_out[(int64_t)t * H + hd] = fmaxf(fabsf(dot), expf(-m)) + 1e-6f;
        }
    }
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int dd = lane + 64 * j;
        if (dd < D) ns[dd] = n[j];
    }
    if (lane == 0) m_state[(int64_t)slot * H + hd] = m;
}

// DR: state rows per wave (D <= 4 * DR).  TT tokens per LDS stage.
template <typename T, int DR>
__global__ void __launch_bounds__(256) mlstm_state_scan_kernel(
        const T* __restrict__ proj, int ldp, const float* __restrict__ a_in, const float* __restrict__ b_in,
        const float* __restrict__ den_in, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
        const int32_t* __restrict__ slots, float* __restrict__ S_state, float* __restrict__ o_out, int H, int D,
        int Dv) {
    constexpr int TT = 8, DP = 4 * DR;
    __shared__ __attribute__((aligned(16))) float qs_[TT][DP];
    __shared__ __attribute__((aligned(16))) float ks_[TT][DP];
    __shared__ float vs_[TT][64];
    __shared__ float ab_[TT][2];
    __shared__ float part_[4][TT][64];
    const int b = blockIdx.x, hd = blockIdx.y, c0 = blockIdx.z * 64;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    if (t1 <= t0) return;
    const int slot = slots[b];
    const bool fresh = pos0[b] == 0;
    const int c = c0 + lane;
    const bool cok = c < Dv;
    float* Ss = S_state + (((int64_t)slot * H + hd) * D) * Dv;
    const int d0 = wv * DR;
    float S[DR];
#pragma unroll
    for (int j = 0; j < DR; ++j) S[j] = (!fresh && cok && d0 + j < D) ? Ss[(int64_t)(d0 + j) * Dv + c] : 0.f;
    const float qscale = 1.f / sqrtf((float)D);
    const int qoff = hd * D, koff = H * D + hd * D, voff = 2 * H * D + hd * Dv;
    for (int tb = t0; tb < t1; tb += TT) {
        const int nt = min(TT, t1 - tb);
        __syncthreads();  // the previous stage's LDS is no longer read
        for (int i = threadIdx.x; i < TT * DP; i += 256) {
            const int tt = i / DP, dd = i % DP;
            const bool ok = tt < nt && dd < D;
            const T* row = proj + (int64_t)(tb + tt) * ldp;
            qs_[tt][dd] = ok ? ld<T>(row + qoff + dd) * qscale : 0.f;
            ks_[tt][dd] = ok ? ld<T>(row + koff + dd) : 0.f;
        }
        for (int i = threadIdx.x; i < TT * 64; i += 256) {
            const int tt = i >> 6, cc = c0 + (i & 63);
            vs_[tt][i & 63] = (tt < nt && cc < Dv) ? ld<T>(proj + (int64_t)(tb + tt) * ldp + voff + cc) : 0.f;
        }
        if (threadIdx.x < TT * 2) {
            const int tt = threadIdx.x >> 1, which = threadIdx.x & 1;
            float v = which ? 0.f : 1.f;  // past the range: a = 1, b = 0 (state unchanged)
            if (tt < nt) v = (which ? b_in : a_in)[(int64_t)(tb + tt) * H + hd];
            ab_[tt][which] = v;
        }
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float a = ab_[tt][0], bv = ab_[tt][1] * vs_[tt][lane];
            float acc = 0.f;
#pragma unroll
            for (int j = 0; j < DR; j += 4) {
                const f32x4 kk = *reinterpret_cast<const f32x4*>(&ks_[tt][d0 + j]);
                const f32x4 qq = *reinterpret_cast<const f32x4*>(&qs_[tt][d0 + j]);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    S[j + u] = a * S[j + u] + kk[u] * bv;
                    acc += S[j + u] * qq[u];
                }
            }
            part_[wv][tt][lane] = acc;
        }
        __syncthreads();
        for (int i = threadIdx.x; i < nt * 64; i += 256) {
            const int tt = i >> 6, l = i & 63;
            if (c0 + l < Dv) {
                const float num = (part_[0][tt][l] + part_[1][tt][l]) + (part_[2][tt][l] + part_[3][tt][l]);
                o_out[((int64_t)(tb + tt) * H + hd) * Dv + c0 + l] = num / den_in[(int64_t)(tb + tt) * H + hd];
            }
        }
    }
    if (cok) {
#pragma unroll
        for (int j = 0; j < DR; ++j)
            if (d0 + j < D) Ss[(int64_t)(d0 + j) * Dv + c] = S[j];
    }
}

// one wave per (token, head): y = o * rsqrt(mean(o^2) + eps) * w[head, :] * sigmoid(g[token, head, :])
template <typename T>
__global__ void __launch_bounds__(256) mlstm_out_kernel(const float* __restrict__ o, const T* __restrict__ proj, int ldp,
                                                        int g_off, const float* __restrict__ w, T* __restrict__ y,
                                                        int rows, int H, int Dv, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int64_t t = r / H;
    const int hd = (int)(r % H);
    const float* orow = o + r * Dv;
    float ss = 0.f;
    for (int i = lane; i < Dv; i += 64) ss += orow[i] * orow[i];
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)Dv + eps);
    const T* g = proj + t * ldp + g_off + hd * Dv;
    for (int i = lane; i < Dv; i += 64)
        st<T>(y + r * Dv + i, orow[i] * inv * w[hd * Dv + i] * sigmoidf_(ld<T>(g + i)));
}

}  // namespace hy

template <typename T>
static void mlstm_scan_t(const T* proj, int ldp, const float* gate_pre, const int32_t* q_start, const int32_t* pos0,
                         const int32_t* slots, float* S, float* n, float* m, float* a, float* b, float* den, float* o,
                         int B, int H, int D, int Dv, float cap, hipStream_t s) {
    hy::mlstm_gate_scan_kernel<T><<<dim3(B, H), 64, 0, s>>>(proj, ldp, gate_pre, q_start, pos0, slots, n, m, a, b, den,
                                                            H, D, cap);
    const dim3 grid(B, H, (Dv + 63) / 64);
#define HY_SCAN(DR) hy::mlstm_state_scan_kernel<T, DR><<<grid, 256, 0, s>>>(proj, ldp, a, b, den, q_start, pos0, slots, S, o, H, D, Dv)
    if (D <= 64) HY_SCAN(16);
    else if (D <= 128) HY_SCAN(32);
    else if (D <= 256) HY_SCAN(64);
    else HY_SCAN(128);
#undef HY_SCAN
}

// D <= 512.  a, b, den: float [T, H] scratch.
void launch_hy_mlstm_scan(const void* proj, int ldp, const float* gate_pre, const int32_t* q_start, const int32_t* pos0,
                          const int32_t* slots, float* S, float* n, float* m, float* a, float* b, float* den, float* o,
                          int B, int H, int D, int Dv, float cap, bool f32, hipStream_t s) {
    if (B == 0) return;
    if (f32) mlstm_scan_t<float>((const float*)proj, ldp, gate_pre, q_start, pos0, slots, S, n, m, a, b, den, o, B, H, D, Dv, cap, s);
    else mlstm_scan_t<uint16_t>((const uint16_t*)proj, ldp, gate_pre, q_start, pos0, slots, S, n, m, a, b, den, o, B, H, D, Dv, cap, s);
}

void launch_hy_mlstm_out(const float* o, const void* proj, int ldp, int g_off, const float* w, void* y, int T, int H,
                         int Dv, float eps, bool f32, hipStream_t s) {
    const int rows = T * H;
    if (rows == 0) return;
    const int blocks = (rows + 3) / 4;
    if (f32) hy::mlstm_out_kernel<float><<<blocks, 256, 0, s>>>(o, (const float*)proj, ldp, g_off, w, (float*)y, rows, H, Dv, eps);
    else hy::mlstm_out_kernel<uint16_t><<<blocks, 256, 0, s>>>(o, (const uint16_t*)proj, ldp, g_off, w, (uint16_t*)y, rows, H, Dv, eps);
}

}  // namespace chronos
