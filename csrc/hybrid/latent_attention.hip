// latent_attention.hip — attention over a paged cache that holds ONE row per token: a low-rank latent (kv_rank
// columns, RMS-normed) followed by a rotated key part (R columns) shared by all heads.
//
// Keys and values are never materialised.  The caller carries each head's query into the latent space
// (q_u W_uk), so the score of head h against token j is  qa[h] . row_j  with qa = [q_u W_uk | rotated q_r], and the
// attention output is a weighted sum of the rows' latent columns, which the caller brings back through W_uv.  All
// heads therefore share the same key/value rows: one pass over the cache serves every head (a multi-query layout with
// key width rank + R and value width rank).
//
//   latent_prep       per token: RMS norm of the latent columns (float), rotation of the shared key part and of
//                     every head's rotated query columns (cos / sin from a float table made in double precision),
//                     cache write at the token's page and slot.
//   latent_attention  one workgroup per (sequence, block of up to 64 (token, head) rows): the rows are split
//                     over 4 waves; 64-key tiles of the cache are staged in LDS; lanes are keys for the scores
//                     (float accumulation, causal mask by each row's own position, online softmax in float) and
//                     latent columns for the output.  Serves prefill chunks and decode rows (a tile of one token).
#include <cstdlib>

#include "hybrid_common.h"

namespace chronos {
namespace hy {

template <typename T>
__global__ void __launch_bounds__(256) latent_prep_kernel(
        T* __restrict__ q, const T* __restrict__ dkv, const int32_t* __restrict__ pos, const int32_t* __restrict__ tok_seq,
        const int32_t* __restrict__ block_table, int max_blocks, const float* __restrict__ w_norm, float eps,
        const float* __restrict__ cos_sin, int dims, int rank, int R, int H, int D, T* __restrict__ cache, int BS) {
    __shared__ float red[16];
    const int64_t t = blockIdx.x;
    const int p = pos[t];
    const int blk = block_table[(int64_t)tok_seq[t] * max_blocks + p / BS];
    const int DK = rank + R;
    T* crow = cache + ((int64_t)blk * BS + p % BS) * DK;
    const T* drow = dkv + t * DK;
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += 256) {
        const float v = ld<T>(drow + i);
        ss += v * v;
    }
    const float inv = 1.f / sqrtf(block_sum(ss, red) / (float)rank + eps);
    for (int i = threadIdx.x; i < rank; i += 256) st<T>(crow + i, ld<T>(drow + i) * inv * w_norm[i]);
    const int half = dims / 2;
    const float* cs = cos_sin + (int64_t)p * dims;
    // the shared key part: pairs (i, i + half) rotated, the columns past `dims` copied
    for (int i = threadIdx.x; i < R; i += 256) {
        float v = ld<T>(drow + rank + i);
        if (i < half) v = v * cs[i] - ld<T>(drow + rank + i + half) * cs[half + i];
        else if (i < dims) v = v * cs[i - half] + ld<T>(drow + rank + i - half) * cs[i];
        st<T>(crow + rank + i, v);
    }
    // every head's rotated query columns, in place: each thread owns whole pairs
    for (int i = threadIdx.x; i < H * half; i += 256) {
        const int hd = i / half, k = i % half;
        T* qr = q + (t * H + hd) * (D + R) + D;
        const float u = ld<T>(qr + k), v = ld<T>(qr + k + half);
        st<T>(qr + k, u * cs[k] - v * cs[half + k]);
        st<T>(qr + k + half, v * cs[k] + u * cs[half + k]);
    }
}

// Words of 4 bytes: 2 bfloat16 or 1 float.
template <typename T> struct Word;
template <> struct Word<uint16_t> { static constexpr int E = 2; };
template <> struct Word<float> { static constexpr int E = 1; };
template <typename T> __device__ __forceinline__ void unpack(uint32_t w, float& a, float& b);
template <> __device__ __forceinline__ void unpack<uint16_t>(uint32_t w, float& a, float& b) {
    a = __uint_as_float(w << 16);
    b = __uint_as_float(w & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack<float>(uint32_t w, float& a, float& b) {
    a = __uint_as_float(w);
    b = 0.f;
}

// RW: rows per wave (<= 16), in groups of RB = 4.  DVL: latent columns per lane (rank <= 64 * DVL).
// KT: keys per LDS tile (<= 64).  LDS: K tile [KT][kstride words] | Q rows [rows][qwords] | P [4][64][4] floats.
template <typename T, int DVL>
__global__ void __launch_bounds__(256) latent_attention_kernel(
        const T* __restrict__ qa, const T* __restrict__ cache, const int32_t* __restrict__ block_table, int max_blocks,
        const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos, const float* __restrict__ gate,
        T* __restrict__ out, int H, int DK, int rank, int BS, int RBLK, int KT, int kstride, float scale) {
    constexpr int E = Word<T>::E, RB = 4, RWMAX = 16;
    extern __shared__ __attribute__((aligned(16))) uint32_t smem[];
    const int b = blockIdx.x;
    // rows of a sequence are (token * H + head); a workgroup takes RBLK (<= 64) consecutive rows, whatever H is
    const int t0 = q_start[b];
    const int rows_total = (q_start[b + 1] - t0) * H;
    const int rb0 = blockIdx.y * RBLK;
    if (rb0 >= rows_total) return;
    const int rows = min(RBLK, rows_total - rb0);
    const int qwords = DK / E;
    uint32_t* ks = smem;
    uint32_t* qsm = ks + KT * kstride;
    float* ps = reinterpret_cast<float*>(qsm + RBLK * qwords);
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int rw = (rows + 3) / 4;          // rows per wave, <= RWMAX (RBLK <= 64)
    const int r0 = wv * rw, r1 = min(rows, r0 + rw);
    // stage the tile's query rows (contiguous in qa)
    const uint32_t* qg = reinterpret_cast<const uint32_t*>(qa + ((int64_t)t0 * H + rb0) * DK);
    for (int i = threadIdx.x; i < rows * qwords; i += 256) qsm[i] = qg[i];
    const int pmax = pos[t0 + (rb0 + rows - 1) / H];
    const bool vec16 = (qwords % 4) == 0;  // rows start 16-byte aligned then (the cache base is)
    float O[RWMAX][DVL], mrow[RWMAX], lrow[RWMAX];
    int prow[RWMAX];
#pragma unroll
    for (int i = 0; i < RWMAX; ++i) {
        mrow[i] = -INFINITY;
        lrow[i] = 0.f;
        prow[i] = (r0 + i < r1) ? pos[t0 + (rb0 + r0 + i) / H] : -1;
#pragma unroll
        for (int v = 0; v < DVL; ++v) O[i][v] = 0.f;
    }
    float* pw = ps + wv * 64 * RB;
    const int32_t* bt = block_table + (int64_t)b * max_blocks;
    for (int k0 = 0; k0 <= pmax; k0 += KT) {
        __syncthreads();  // everyone is done with the previous key tile (and the query rows are staged)
        const int nk = min(KT, pmax + 1 - k0);
        // one wave per key row in turn (no index arithmetic per element; the page lookup is wave-uniform); 16-byte
        // global loads where the row length allows, 4-byte LDS stores into the odd-stride rows
        for (int j = wv; j < nk; j += 4) {
            const int key = k0 + j;
            const T* rowp = cache + ((int64_t)bt[key / BS] * BS + key % BS) * DK;
            uint32_t* dst = ks + j * kstride;
            if (vec16) {
                const uint4* src = reinterpret_cast<const uint4*>(rowp);
                for (int p = lane; p < qwords / 4; p += 64) {
                    const uint4 v = src[p];
                    dst[4 * p] = v.x; dst[4 * p + 1] = v.y; dst[4 * p + 2] = v.z; dst[4 * p + 3] = v.w;
                }
            } else {
                const uint32_t* src = reinterpret_cast<const uint32_t*>(rowp);
                for (int p = lane; p < qwords; p += 64) dst[p] = src[p];
            }
        }
        __syncthreads();
#pragma unroll
        for (int g = 0; g < RWMAX / RB; ++g) {
            if (r0 + g * RB < r1) {
                // scores: lane = key
                float sc[RB] = {0.f, 0.f, 0.f, 0.f};
                if (lane < nk) {
                    const uint32_t* kr = ks + lane * kstride;
                    const uint32_t* qr = qsm + (r0 + g * RB) * qwords;
                    for (int wd = 0; wd < qwords; ++wd) {
                        float ka, kb;
                        unpack<T>(kr[wd], ka, kb);
#pragma unroll
                        for (int u = 0; u < RB; ++u) {
                            float qa_, qb_;
                            // rows past r1 read staged rows of other waves or zero-initialised LDS: masked below
                            unpack<T>(qr[min(u, r1 - 1 - (r0 + g * RB)) * qwords + wd], qa_, qb_);
                            sc[u] += ka * qa_ + kb * qb_;
                        }
                    }
                }
                float corr[RB];
#pragma unroll
                for (int u = 0; u < RB; ++u) {
                    const int i = g * RB + u;
                    const bool seen = lane < nk && k0 + lane <= prow[i];
                    const float s = seen ? sc[u] * scale : -INFINITY;
                    const float mn = fmaxf(mrow[i], wave_max(s));
                    // a row that has seen no key yet keeps m = -inf: every weight 0, nothing to rescale
                    const float p = (mn == -INFINITY) ? 0.f : expf(s - mn);
                    corr[u] = (mn == -INFINITY) ? 1.f : expf(mrow[i] - mn);
                    lrow[i] = lrow[i] * corr[u] + wave_sum(p);
                    mrow[i] = mn;
                    pw[lane * RB + u] = p;
                }
                __builtin_amdgcn_wave_barrier();  // the wave's weights are in LDS before any lane reads them
                // output: lane = latent column(s); every wave reads only its own weights (no barrier: one wave)
#pragma unroll
                for (int u = 0; u < RB; ++u)
#pragma unroll
                    for (int v = 0; v < DVL; ++v) O[g * RB + u][v] *= corr[u];
                for (int j = 0; j < nk; ++j) {
                    const f32x4 pj = *reinterpret_cast<const f32x4*>(pw + j * RB);
#pragma unroll
                    for (int v = 0; v < DVL; ++v) {
                        const int col = lane + 64 * v;
                        float cv = 0.f;
                        if (col < rank) {
                            if constexpr (E == 2) {
                                const uint32_t wd = ks[j * kstride + (col >> 1)];
                                cv = (col & 1) ? __uint_as_float(wd & 0xffff0000u) : __uint_as_float(wd << 16);
                            } else {
                                cv = __uint_as_float(ks[j * kstride + col]);
                            }
                        }
#pragma unroll
                        for (int u = 0; u < RB; ++u) O[g * RB + u][v] += pj[u] * cv;
                    }
                }
                __builtin_amdgcn_wave_barrier();  // ... and read before the next row group overwrites them
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RWMAX; ++i) {
        const int r = r0 + i;
        if (r < r1) {
            const int64_t grow = (int64_t)t0 * H + rb0 + r;  // row of qa / gate / out
            float f = 1.f / lrow[i];
            if (gate != nullptr) f *= sigmoidf_(gate[grow]);
#pragma unroll
            for (int v = 0; v < DVL; ++v) {
                const int col = lane + 64 * v;
                if (col < rank) st<T>(out + grow * rank + col, O[i][v] * f);
            }
        }
    }
}

}  // namespace hy

void launch_hy_latent_prep(void* q, const void* dkv, const int32_t* pos, const int32_t* tok_seq, const int32_t* bt,
                           int max_blocks, const float* w_norm, float eps, const float* cos_sin, int dims, int rank,
                           int R, int H, int D, void* cache, int BS, int T, bool f32, hipStream_t s) {
    if (T == 0) return;
    if (f32) hy::latent_prep_kernel<float><<<T, 256, 0, s>>>((float*)q, (const float*)dkv, pos, tok_seq, bt, max_blocks, w_norm, eps, cos_sin, dims, rank, R, H, D, (float*)cache, BS);
    else hy::latent_prep_kernel<uint16_t><<<T, 256, 0, s>>>((uint16_t*)q, (const uint16_t*)dkv, pos, tok_seq, bt, max_blocks, w_norm, eps, cos_sin, dims, rank, R, H, D, (uint16_t*)cache, BS);
}

// Launch geometry of latent_attention for these sizes: RBLK (token, head) rows per workgroup (<= 64), KT keys per
// LDS tile, the K tile's row stride in words (odd, so lanes reading consecutive rows hit different banks), and the
// dynamic LDS bytes.  Returns false when not even 4 rows and 16 keys fit the LDS.
bool hy_latent_geometry(int H, int DK, int esize, int max_q, int lds_limit, int* RBLK, int* KT, int* kstride, int* bytes) {
    const int qwords = DK * esize / 4;
    const int ks = qwords | 1;
    int want = max_q * H;
    if (want > 64) want = 64;
    if (want < 1) want = 1;
    for (int kt = 64; kt >= 16; kt >>= 1) {
        for (int r = want; r >= 4 || r == want; r = r / 2) {
            const int b = (kt * ks + r * qwords) * 4 + 4 * 64 * 4 * 4;
            if (b <= lds_limit) {
                *RBLK = r; *KT = kt; *kstride = ks; *bytes = b;
                return true;
            }
            if (r <= 4) break;
        }
    }
    return false;
}

template <typename T, int DVL>
static void latent_attn_t(const T* qa, const T* cache, const int32_t* bt, int max_blocks, const int32_t* q_start,
                          const int32_t* pos, const float* gate, T* out, int B, int H, int DK, int rank, int BS,
                          int max_q, int RBLK, int KT, int kstride, int bytes, float scale, hipStream_t s) {
    auto kern = hy::latent_attention_kernel<T, DVL>;
    static int set_bytes = 0;
    if (bytes > set_bytes) {  // raise the dynamic-LDS ceiling of this instantiation once per size
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        set_bytes = bytes;
    }
    const dim3 grid(B, (max_q * H + RBLK - 1) / RBLK);
    kern<<<grid, 256, bytes, s>>>(qa, cache, bt, max_blocks, q_start, pos, gate, out, H, DK, rank, BS, RBLK, KT, kstride, scale);
}

bool launch_hy_latent_attention_mfma(const uint16_t*, const uint16_t*, const int32_t*, int, const int32_t*, const int32_t*,
                                     const float*, uint16_t*, int, int, int, int, int, int, float, int, float*, float*,
                                     int64_t, hipStream_t);
bool hy_latent_mfma_ok(int DK, int rank);

// whether this call goes to the matrix-core kernel (bfloat16 at its sizes; CHRONOS_LATENT_MFMA=0 keeps the general
// kernel, for A/B)
bool hy_latent_use_mfma(bool f32, int DK, int rank) {
    static const bool on = [] {
        const char* v = getenv("CHRONOS_LATENT_MFMA");
        return v == nullptr || v[0] != '0';
    }();
    return !f32 && on && hy_latent_mfma_ok(DK, rank);
}

bool launch_hy_latent_attention(const void* qa, const void* cache, const int32_t* bt, int max_blocks,
                                const int32_t* q_start, const int32_t* pos, const float* gate, void* out, int B, int H,
                                int DK, int rank, int BS, int max_q, float scale, bool f32, int nsplit, float* part_o,
                                float* part_ml, int64_t total_rows, hipStream_t s) {
    if (B == 0 || max_q == 0) return true;
    if (hy_latent_use_mfma(f32, DK, rank))
        return launch_hy_latent_attention_mfma((const uint16_t*)qa, (const uint16_t*)cache, bt, max_blocks, q_start, pos, gate,
                                               (uint16_t*)out, B, H, DK, rank, BS, max_q, scale, nsplit, part_o, part_ml,
                                               total_rows, s);
    int RBLK, KT, kstride, bytes;
    if (rank > 512 || !hy_latent_geometry(H, DK, f32 ? 4 : 2, max_q, 160 * 1024, &RBLK, &KT, &kstride, &bytes)) return false;
#define HY_LA(TT, DVL) latent_attn_t<TT, DVL>((const TT*)qa, (const TT*)cache, bt, max_blocks, q_start, pos, gate, (TT*)out, B, H, DK, rank, BS, max_q, RBLK, KT, kstride, bytes, scale, s)
    const int dvl = (rank + 63) / 64;
    if (f32) {
        if (dvl <= 1) HY_LA(float, 1); else if (dvl <= 2) HY_LA(float, 2); else if (dvl <= 4) HY_LA(float, 4); else HY_LA(float, 8);
    } else {
        if (dvl <= 1) HY_LA(uint16_t, 1); else if (dvl <= 2) HY_LA(uint16_t, 2); else if (dvl <= 4) HY_LA(uint16_t, 4); else HY_LA(uint16_t, 8);
    }
#undef HY_LA
    return true;
}

}  // namespace chronos
