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

// Tokens are taken TG at a time (TG <= 64, a power of two): lane t evaluates the gates of token t (the tanh / log /
// exp work runs across the lanes, not along the sequence), the running maximum is a short scalar recurrence over the
// block, and the block's k and q rows are staged in LDS with coalesced loads, so the sequential n update never waits
// on global memory.  LDS: k rows [TG][D] | q rows [TG][D] in the activation type, then 5 float arrays of 64.
template <typename T>
__global__ void __launch_bounds__(256) mlstm_gate_scan_kernel(
        const T* __restrict__ proj, int ldp, const float* __restrict__ gate_pre, const int32_t* __restrict__ q_start,
        const int32_t* __restrict__ pos0, const int32_t* __restrict__ slots, float* __restrict__ n_state,
        float* __restrict__ m_state, float* __restrict__ a_out, float* __restrict__ b_out, float* __restrict__ den_out,
        int H, int D, float cap, int TG, int vec) {
    extern __shared__ __attribute__((aligned(16))) unsigned char gs_smem[];
    T* kst = reinterpret_cast<T*>(gs_smem);
    T* qst = kst + (size_t)TG * D;
    float* ig_s = reinterpret_cast<float*>(qst + (size_t)TG * D);
    float* fg_s = ig_s + 64;
    float* a_s = fg_s + 64;
    float* b_s = a_s + 64;
    float* em_s = b_s + 64;
    float* dots = em_s + 64;  // [TG][65]: lane l's partial n . q of token t at dots[t * 65 + l]
    // 256 threads stage the block's rows (16-byte loads, 8 in flight per thread); wave 0 runs the recurrences
    const int b = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x & 63;
    const bool w0 = threadIdx.x < 64;
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
    for (int tb = t0; tb < t1; tb += TG) {
        const int nt = min(TG, t1 - tb);
        __syncthreads();  // the previous block's rows are no longer read
        if (w0 && lane < nt) {
            const float zi = gate_pre[(int64_t)(tb + lane) * 2 * H + hd], zf = gate_pre[(int64_t)(tb + lane) * 2 * H + H + hd];
            ig_s[lane] = cap * tanhf(zi / cap);
            fg_s[lane] = logsigmoidf_(cap * tanhf(zf / cap));
        }
        if (vec) {
            constexpr int EV = 16 / (int)sizeof(T);
            const int vpr = D / EV, nvec = nt * 2 * vpr;  // vectors per row; per token: q row | k row
            for (int base = threadIdx.x; base < nvec; base += 256 * 8) {
                uint4 r[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int v = base + 256 * u;
                    if (v < nvec) {
                        const int tt = v / (2 * vpr), rem = v - tt * 2 * vpr;
                        const int part = rem >= vpr, off = (rem - part * vpr) * EV;
                        r[u] = *reinterpret_cast<const uint4*>(proj + (int64_t)(tb + tt) * ldp + (part ? H * D : 0) + hd * D + off);
                    }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int v = base + 256 * u;
                    if (v < nvec) {
                        const int tt = v / (2 * vpr), rem = v - tt * 2 * vpr;
                        const int part = rem >= vpr, off = (rem - part * vpr) * EV;
                        *reinterpret_cast<uint4*>((part ? kst : qst) + tt * D + off) = r[u];
                    }
                }
            }
        } else {
            for (int tt = 0; tt < nt; ++tt) {
                const T* row = proj + (int64_t)(tb + tt) * ldp + hd * D;
                for (int dd = threadIdx.x; dd < D; dd += 256) {
                    qst[tt * D + dd] = row[dd];
                    kst[tt * D + dd] = row[(int64_t)H * D + dd];
                }
            }
        }
        __syncthreads();
        if (!w0) continue;  // (the loop's first barrier keeps these waves in step)
        // running maximum: every lane walks the block, lane t keeps (m_{t-1}, m_t)
        float mp = m, mine_prev = m, mine = m;
        for (int tt = 0; tt < nt; ++tt) {
            const float mn = fmaxf(fg_s[tt] + mp, ig_s[tt]);
            if (tt == lane) {
                mine_prev = mp;
                mine = mn;
            }
            mp = mn;
        }
        m = mp;
        if (lane < nt) {
            const float a = expf(fg_s[lane] + mine_prev - mine), bb = expf(ig_s[lane] - mine);
            a_s[lane] = a;
            b_s[lane] = bb;
            em_s[lane] = expf(-mine);
            a_out[(int64_t)(tb + lane) * H + hd] = a;
            b_out[(int64_t)(tb + lane) * H + hd] = bb;
        }
        __builtin_amdgcn_wave_barrier();  // wave 0's own LDS writes above, read by its lanes below
        // the n update runs token by token, but no cross-lane reduction sits on that chain: every lane leaves its
        // partial n . q in LDS, and afterwards lane t adds up token t's 64 partials
        for (int tt = 0; tt < nt; ++tt) {
            const float a = a_s[tt], bb = b_s[tt];
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < NL; ++j) {
                const int dd = lane + 64 * j;
                if (dd < D) {
                    n[j] = a * n[j] + bb * ld<T>(kst + tt * D + dd);
                    dot += n[j] * (ld<T>(qst + tt * D + dd) * qs);
                }
            }
            dots[tt * 65 + lane] = dot;
        }
        __builtin_amdgcn_wave_barrier();
        if (lane < nt) {
            float dsum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int l = 0; l < 64; ++l) dsum[l & 3] += dots[lane * 65 + l];
            const float dot = (dsum[0] + dsum[1]) + (dsum[2] + dsum[3]);
            den_out[(int64_t)(tb + lane) * H + hd] = fmaxf(fabsf(dot), em_s[lane]) + 1e-6f;
        }
    }
#pragma unroll
    for (int j = 0; j < NL; ++j) {
        const int dd = lane + 64 * j;
        if (w0 && dd < D) ns[dd] = n[j];
    }
    if (threadIdx.x == 0) m_state[(int64_t)slot * H + hd] = m;
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

// The same scan with 16-byte global loads and the NEXT stage's loads in flight while the current stage's tokens are
// processed (the sequential token loop leaves one workgroup per CU alone with its memory latency otherwise).
// Needs rows of q, k, v that start and end on 16-byte boundaries (host-checked).  TT = 16 tokens per stage.
template <typename T, int DR>
__global__ void __launch_bounds__(256) mlstm_state_scan_vec_kernel(
        const T* __restrict__ proj, int ldp, const float* __restrict__ a_in, const float* __restrict__ b_in,
        const float* __restrict__ den_in, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
        const int32_t* __restrict__ slots, float* __restrict__ S_state, float* __restrict__ o_out, int H, int D,
        int Dv) {
    constexpr int TT = 16, DP = 4 * DR, EV = 16 / (int)sizeof(T);     // elements per 16-byte vector
    constexpr int QV = DP / EV, VV = 64 / EV, PV = 2 * QV + VV;       // vectors per token: q | k | v slice
    constexpr int NV = (TT * PV + 255) / 256;                         // vectors per thread and stage
    __shared__ __attribute__((aligned(16))) float qs_[TT][DP];
    __shared__ __attribute__((aligned(16))) float ks_[TT][DP];
    __shared__ __attribute__((aligned(16))) float vs_[TT][64];
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
    const int qoff = hd * D, koff = H * D + hd * D, voff = 2 * H * D + hd * Dv + c0;
    uint4 raw[NV];
    auto fetch = [&](int tb) {
        const int nt = min(TT, t1 - tb);
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int v = threadIdx.x + 256 * u;
            const int tt = v / PV, rem = v % PV;
            const int part = rem < QV ? 0 : (rem < 2 * QV ? 1 : 2);
            const int e = (part == 0 ? rem : (part == 1 ? rem - QV : rem - 2 * QV)) * EV;
            const bool ok = tt < nt && (part == 2 ? c0 + e < Dv : e < D);
            const T* src = proj + (int64_t)(tb + tt) * ldp + (part == 0 ? qoff : (part == 1 ? koff : voff)) + e;
            raw[u] = ok ? *reinterpret_cast<const uint4*>(src) : uint4{0u, 0u, 0u, 0u};
        }
    };
    auto store = [&]() {
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            const int v = threadIdx.x + 256 * u;
            const int tt = v / PV, rem = v % PV;
            if (tt >= TT) continue;
            const int part = rem < QV ? 0 : (rem < 2 * QV ? 1 : 2);
            const int e = (part == 0 ? rem : (part == 1 ? rem - QV : rem - 2 * QV)) * EV;
            float* dst = part == 0 ? &qs_[tt][e] : (part == 1 ? &ks_[tt][e] : &vs_[tt][e]);
            const float sc = part == 0 ? qscale : 1.f;
            float f[EV];
            if constexpr (sizeof(T) == 2) {
                const uint32_t w[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    f[2 * i] = __uint_as_float(w[i] << 16) * sc;
                    f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u) * sc;
                }
            } else {
                f[0] = __uint_as_float(raw[u].x) * sc; f[1] = __uint_as_float(raw[u].y) * sc;
                f[2] = __uint_as_float(raw[u].z) * sc; f[3] = __uint_as_float(raw[u].w) * sc;
            }
#pragma unroll
            for (int i = 0; i < EV; i += 4) *reinterpret_cast<f32x4*>(dst + i) = f32x4{f[i], f[i + 1], f[i + 2], f[i + 3]};
        }
    };
    fetch(t0);
    for (int tb = t0; tb < t1; tb += TT) {
        const int nt = min(TT, t1 - tb);
        __syncthreads();  // the previous stage's LDS is no longer read
        store();
        if (threadIdx.x < TT * 2) {
            const int tt = threadIdx.x >> 1, which = threadIdx.x & 1;
            float v = which ? 0.f : 1.f;
            if (tt < nt) v = (which ? b_in : a_in)[(int64_t)(tb + tt) * H + hd];
            ab_[tt][which] = v;
        }
        if (tb + TT < t1) fetch(tb + TT);  // in flight during this stage's token loop
        __syncthreads();
        for (int tt = 0; tt < nt; ++tt) {
            const float a = ab_[tt][0], bv = ab_[tt][1] * vs_[tt][lane];
            // the wave's DR k and q values: ONE per lane from LDS (two conflict-free reads per token), then handed
            // to every lane as scalar operands by lane reads — a broadcast LDS read per row costs the LDS pipe a
            // full 64-lane pass each and was the kernel's limit
            const int kreg = __float_as_int(ks_[tt][d0 + (lane & (DR - 1))]);
            const int qreg = __float_as_int(qs_[tt][d0 + (lane & (DR - 1))]);
            float acc[4] = {0.f, 0.f, 0.f, 0.f};  // independent chains: one wave per SIMD hides no FMA latency
#pragma unroll
            for (int j = 0; j < DR; ++j) {
                const float kj = __int_as_float(__builtin_amdgcn_readlane(kreg, j));
                const float qj = __int_as_float(__builtin_amdgcn_readlane(qreg, j));
                S[j] = a * S[j] + kj * bv;
                acc[j & 3] += S[j] * qj;
            }
            part_[wv][tt][lane] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
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
                                                        int rows, int H, int Dv, float eps, int silu) {
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
    for (int i = lane; i < Dv; i += 64) {
        const float gv = ld<T>(g + i);
        st<T>(y + r * Dv + i, orow[i] * inv * w[hd * Dv + i] * (silu ? gv * sigmoidf_(gv) : sigmoidf_(gv)));
    }
}

}  // namespace hy

template <typename T>
static void mlstm_scan_t(const T* proj, int ldp, const float* gate_pre, const int32_t* q_start, const int32_t* pos0,
                         const int32_t* slots, float* S, float* n, float* m, float* a, float* b, float* den, float* o,
                         int B, int H, int D, int Dv, float cap, hipStream_t s) {
    // tokens per gate-scan block: as many (<= 64) as keep the staged k and q rows within 40 KB
    int TG = 64;
    while (TG > 1 && (size_t)TG * 2 * D * sizeof(T) > 40 * 1024) TG >>= 1;
    const int gev = 16 / (int)sizeof(T);
    const int gvec = ldp % gev == 0 && D % gev == 0;  // q and k rows start and end on 16-byte boundaries
    hy::mlstm_gate_scan_kernel<T><<<dim3(B, H), 256, (size_t)TG * 2 * D * sizeof(T) + 5 * 64 * 4 + 64 * 65 * 4, s>>>(
        proj, ldp, gate_pre, q_start, pos0, slots, n, m, a, b, den, H, D, cap, TG, gvec);
    const dim3 grid(B, H, (Dv + 63) / 64);
    // rows of q, k, v on 16-byte boundaries: the vector-load kernel with the next stage prefetched (its LDS stays
    // within the static 64 KB up to D = 256); anything else: the plain one
    const int ev = 16 / (int)sizeof(T);
    const bool vec = ldp % ev == 0 && D % ev == 0 && Dv % ev == 0 && D <= 256;
#define HY_SCAN(DR)                                                                                                    \
    do {                                                                                                               \
        if (vec) hy::mlstm_state_scan_vec_kernel<T, DR><<<grid, 256, 0, s>>>(proj, ldp, a, b, den, q_start, pos0, slots, S, o, H, D, Dv); \
        else hy::mlstm_state_scan_kernel<T, DR><<<grid, 256, 0, s>>>(proj, ldp, a, b, den, q_start, pos0, slots, S, o, H, D, Dv);       \
    } while (0)
    if (D <= 64) HY_SCAN(16);
    else if (D <= 128) HY_SCAN(32);
    else if (D <= 256) HY_SCAN(64);
    else hy::mlstm_state_scan_kernel<T, 128><<<grid, 256, 0, s>>>(proj, ldp, a, b, den, q_start, pos0, slots, S, o, H, D, Dv);
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

// silu_gate: the gate columns pass SiLU instead of the sigmoid (the read-out of the linear-state mixers)
void launch_hy_head_norm_gate(const float* o, const void* proj, int ldp, int g_off, const float* w, void* y, int T, int H,
                              int Dv, float eps, bool silu_gate, bool f32, hipStream_t s) {
    const int rows = T * H;
    if (rows == 0) return;
    const int blocks = (rows + 3) / 4;
    if (f32) hy::mlstm_out_kernel<float><<<blocks, 256, 0, s>>>(o, (const float*)proj, ldp, g_off, w, (float*)y, rows, H, Dv, eps, silu_gate);
    else hy::mlstm_out_kernel<uint16_t><<<blocks, 256, 0, s>>>(o, (const uint16_t*)proj, ldp, g_off, w, (uint16_t*)y, rows, H, Dv, eps, silu_gate);
}

void launch_hy_mlstm_out(const float* o, const void* proj, int ldp, int g_off, const float* w, void* y, int T, int H,
                         int Dv, float eps, bool f32, hipStream_t s) {
    launch_hy_head_norm_gate(o, proj, ldp, g_off, w, y, T, H, Dv, eps, false, f32, s);
}

}  // namespace chronos
