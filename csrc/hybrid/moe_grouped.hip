// moe_grouped.hip — the experts of a mixture-of-experts layer as two grouped MFMA GEMMs (bfloat16), for any number of
// tokens: every expert's weights are streamed once per 128 of its tokens, never once per token.
//
//   align     one workgroup: counts the (token, choice) items of every expert with weights, gives each expert a run
//             of whole 128-row tiles in a sorted row space, and writes row -> item (or -1 for padding), item -> row
//             and the tile -> expert table.  Everything stays on the device: the GEMM grids are sized for the worst
//             case (items / 128 + experts tiles) and surplus workgroups leave at once, so the host never learns the
//             routing and the step captures into a graph.
//   up GEMM   Z[row, :] = act(h[token(row), :] W_up[e]^T): the x operand's rows are GATHERED by token through the
//             per-lane LDS-DMA source addresses; activation in the epilogue.
//   down GEMM Y[row, :] = Z[row, :] W_down[e]^T.
//   combine   out[t, :] = sum_k weight[t, k] * Y[row(t, k), :]  (+ weight * h[t, :] for an identity expert), summed
//             in the order of k in float: the result does not depend on what else is in the batch.
//
// Gated experts (act = gated unit): the up GEMM runs over W_gu [E, 2F, d] whose rows are PERMUTED at weight-packing
// time (moe_glu_row_order) so that every 128-row tile holds 64 gate rows and their 64 up rows in the accumulator
// positions of the same lane; the epilogue combines them and writes 64 columns of Z [rows, F] per tile.
//
// The tile loop is the 128 x 128 x 64 LDS-DMA ring of csrc/kernels/gemm.hip (4 waves as 2 x 2, 16x16x32 bf16 MFMAs,
// XOR-swizzled images, one barrier per k-step with a counted vmcnt).  Needs d % 128 == 0 and F % 128 == 0.
#include "hybrid_common.h"

namespace chronos {
namespace hy {

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) void* gbl_ptr_t;

constexpr int GBM = 128, GBN = 128, GBK = 64, GSTAGES = 3;
constexpr int kImg = 128 * GBK * 2;

template <int N>
__device__ __forceinline__ void wait_vm() {
    __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
}
__device__ __forceinline__ bf16x8 frag(const unsigned char* img, int row, int chunk) {
    return *reinterpret_cast<const bf16x8*>(img + row * 128 + ((chunk ^ (row & 7)) << 4));
}

// meta layout (int32): [0] tiles used | [1 .. 1+maxTiles) tile -> expert | then row -> item [maxTiles * 128] |
// then item -> row [items]
__global__ void __launch_bounds__(1024) moe_align_kernel(const int32_t* __restrict__ idx, int items, int E, int maxTiles,
                                                         int32_t* __restrict__ meta) {
    __shared__ int cnt[256], start[257], fill[256];
    int32_t* tile_e = meta + 1;
    int32_t* row_item = tile_e + maxTiles;
    int32_t* item_row = row_item + maxTiles * GBM;
    for (int e = threadIdx.x; e < E; e += blockDim.x) { cnt[e] = 0; fill[e] = 0; }
    __syncthreads();
    for (int i = threadIdx.x; i < items; i += blockDim.x) {
        const int e = idx[i];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int e = 0; e < E; ++e) {
            start[e] = t;
            const int n = (cnt[e] + GBM - 1) / GBM;
            for (int j = 0; j < n; ++j) tile_e[t + j] = e;
            t += n;
        }
        start[E] = t;
        meta[0] = t;
    }
    __syncthreads();
    const int used = start[E];
    for (int i = threadIdx.x; i < used * GBM; i += blockDim.x) row_item[i] = -1;
    __syncthreads();
    // which row of its expert's run an item takes does not matter: every row is computed on its own and found again
    // through item -> row, so the result is the same for any order
    for (int i = threadIdx.x; i < items; i += blockDim.x) {
        const int e = idx[i];
        if (e >= 0 && e < E) {
            const int r = start[e] * GBM + atomicAdd(&fill[e], 1);
            row_item[r] = i;
            item_row[i] = r;
        }
    }
    for (int i = threadIdx.x; i < items; i += blockDim.x) {
        const int e = idx[i];
        if (e < 0 || e >= E) item_row[i] = -1;
    }
}

// y[row, n] = sum_k x[src(row), k] * w[e][n, k]; GATHER: src(row) = row_item[row] / top (rows of h), else row.
// ACT >= 0: activation of that kind in the epilogue.  ACT == kActGlu: w holds N = 2F permuted gate / up rows, y is
// [rows, N / 2], and (limit, slope, shift) are the gated unit's constants.
constexpr int kActGlu = 2;
template <bool GATHER, int ACT>
__global__ void __launch_bounds__(256) moe_gemm_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                       uint16_t* __restrict__ y, const int32_t* __restrict__ meta,
                                                       int maxTiles, int top, int N, int K, float limit, float slope,
                                                       float shift) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    const int nt = N / GBN;
    const int tile = blockIdx.x / nt, tn = blockIdx.x % nt;
    if (tile >= meta[0]) return;
    const int e = meta[1 + tile];
    const int32_t* row_item = meta + 1 + maxTiles;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = tile * GBM;
    const uint16_t* we = w + (int64_t)e * N * K;
    const uint16_t* wsrc[4];
    const uint16_t* xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = 32 * wave + 8 * i + (lane >> 3);
        const int c = (lane & 7) ^ (r & 7);
        wsrc[i] = we + (int64_t)(tn * GBN + r) * K + c * 8;
        int64_t xr = m0 + r;
        if constexpr (GATHER) {
            const int it = row_item[m0 + r];
            xr = it < 0 ? 0 : it / top;  // padding rows read token 0 and are never stored
        }
        xsrc[i] = x + xr * K + c * 8;
    }
    auto issue = [&](int kt) {
        unsigned char* st = smem + (kt % GSTAGES) * 2 * kImg;
        const int koff = kt * GBK;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(wsrc[i] + koff), (lds_ptr_t)(st + (4 * wave + i) * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gbl_ptr_t)(xsrc[i] + koff), (lds_ptr_t)(st + kImg + (4 * wave + i) * 1024), 16, 0, 0);
        }
    };
    const int wn = wave >> 1, wm = wave & 1;
    f32x4 acc[4][4];
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[s][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int KT = K / GBK;
#pragma unroll
    for (int p = 0; p < GSTAGES - 1; ++p)
        if (p < KT) issue(p);
    for (int kt = 0; kt < KT; ++kt) {
        if (kt + GSTAGES - 2 < KT) wait_vm<8 * (GSTAGES - 2)>();
        else wait_vm<0>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (kt + GSTAGES - 1 < KT) issue(kt + GSTAGES - 1);
        const unsigned char* wimg = smem + (kt % GSTAGES) * 2 * kImg;
        const unsigned char* ximg = wimg + kImg;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int chunk = h * 4 + (lane >> 4);
            bf16x8 a[4], b[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) a[s] = frag(wimg, 64 * wn + 16 * s + (lane & 15), chunk);
#pragma unroll
            for (int t = 0; t < 4; ++t) b[t] = frag(ximg, 64 * wm + 16 * t + (lane & 15), chunk);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s], b[t], acc[s][t], 0, 0, 0);
        }
    }
    // lane holds D[n = 4 * (lane >> 4) + i][m = lane & 15] of each 16 x 16 tile = y[m][n .. n + 3]
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int m = m0 + 64 * wm + 16 * t + (lane & 15);
        if (row_item[m] < 0) continue;
        if constexpr (ACT == kActGlu) {
            // tile-local rows 64 wn + 16 s + j: s = 0, 1 are gate rows, s = 2, 3 the up rows of the same outputs
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                u16x4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float a = fminf(bf2f(f2bf(acc[s][t][i])), limit);
                    const float u = fminf(fmaxf(bf2f(f2bf(acc[s + 2][t][i])), -limit), limit);
                    o[i] = f2bf(a * sigmoidf_(slope * a) * (u + shift));
                }
                const int n = tn * 64 + 32 * wn + 16 * s + 4 * (lane >> 4);
                *reinterpret_cast<u16x4*>(y + (int64_t)m * (N / 2) + n) = o;
            }
            continue;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            u16x4 o;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float v = acc[s][t][i];
                if constexpr (ACT >= 0 && ACT != kActGlu) v = act_apply(bf2f(f2bf(v)), ACT);
                o[i] = f2bf(v);
            }
            const int n = tn * GBN + 64 * wn + 16 * s + 4 * (lane >> 4);
            *reinterpret_cast<u16x4*>(y + (int64_t)m * N + n) = o;
        }
    }
}

__global__ void __launch_bounds__(256) moe_combine_kernel(const uint16_t* __restrict__ h, const uint16_t* __restrict__ yrows,
                                                          const int32_t* __restrict__ idx, const float* __restrict__ wt,
                                                          const int32_t* __restrict__ item_row, uint16_t* __restrict__ out,
                                                          int d, int top, int E) {
    const int64_t t = blockIdx.x;
    for (int c = threadIdx.x * 8; c < d; c += 256 * 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int k = 0; k < top; ++k) {
            const int e = idx[t * top + k];
            const float g = wt[t * top + k];
            const uint16_t* src = e >= E ? h + t * d + c : yrows + (int64_t)item_row[t * top + k] * d + c;
            const u16x8 v = *reinterpret_cast<const u16x8*>(src);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] += g * bf2f(v[j]);
        }
        u16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = f2bf(acc[j]);
        *reinterpret_cast<u16x8*>(out + t * d + c) = o;
    }
}

}  // namespace hy

int hy_moe_max_tiles(int items, int E) { return (items + hy::GBM - 1) / hy::GBM + E; }

// meta: int32 [1 + maxTiles + maxTiles * 128 + items]; z: bf16 [maxTiles * 128, F]; yrows: bf16 [maxTiles * 128, d].
void launch_hy_moe_grouped(const uint16_t* h, const int32_t* idx, const float* wt, const uint16_t* w_up,
                           const uint16_t* w_down, uint16_t* out, int32_t* meta, uint16_t* z, uint16_t* yrows, int T,
                           int d, int F, int E, int top, int act, hipStream_t s) {
    if (T == 0) return;
    const int items = T * top, maxTiles = hy_moe_max_tiles(items, E);
    hy::moe_align_kernel<<<1, 1024, 0, s>>>(idx, items, E, maxTiles, meta);
    const int lds = hy::GSTAGES * 2 * hy::kImg;
    static bool attr = false;
    if (!attr) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(hy::moe_gemm_kernel<true, 0>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(hy::moe_gemm_kernel<true, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(hy::moe_gemm_kernel<false, -1>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        attr = true;
    }
    if (act == 0) hy::moe_gemm_kernel<true, 0><<<maxTiles * (F / hy::GBN), 256, lds, s>>>(h, w_up, z, meta, maxTiles, top, F, d, 0.f, 0.f, 0.f);
    else hy::moe_gemm_kernel<true, 1><<<maxTiles * (F / hy::GBN), 256, lds, s>>>(h, w_up, z, meta, maxTiles, top, F, d, 0.f, 0.f, 0.f);
    hy::moe_gemm_kernel<false, -1><<<maxTiles * (d / hy::GBN), 256, lds, s>>>(z, w_down, yrows, meta, maxTiles, top, d, F, 0.f, 0.f, 0.f);
    hy::moe_combine_kernel<<<T, 256, 0, s>>>(h, yrows, idx, wt, meta + 1 + maxTiles + maxTiles * hy::GBM, out, d, top, E);
}

// Gated experts.  w_gu: bf16 [E, 2F, d] in the tile order of moe_glu_row_order; z: bf16 [maxTiles * 128, F];
// needs d % 128 == 0 and F % 128 == 0 (the down GEMM's k-steps and the up GEMM's 64-output tiles).
void launch_hy_moe_glu_grouped(const uint16_t* h, const int32_t* idx, const float* wt, const uint16_t* w_gu,
                               const uint16_t* w_down, uint16_t* out, int32_t* meta, uint16_t* z, uint16_t* yrows, int T,
                               int d, int F, int E, int top, float limit, float slope, float shift, hipStream_t s) {
    if (T == 0) return;
    const int items = T * top, maxTiles = hy_moe_max_tiles(items, E);
    hy::moe_align_kernel<<<1, 1024, 0, s>>>(idx, items, E, maxTiles, meta);
    const int lds = hy::GSTAGES * 2 * hy::kImg;
    static bool attr = false;
    if (!attr) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(hy::moe_gemm_kernel<true, hy::kActGlu>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(hy::moe_gemm_kernel<false, -1>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        attr = true;
    }
    hy::moe_gemm_kernel<true, hy::kActGlu><<<maxTiles * (2 * F / hy::GBN), 256, lds, s>>>(h, w_gu, z, meta, maxTiles, top, 2 * F, d, limit, slope, shift);
    hy::moe_gemm_kernel<false, -1><<<maxTiles * (d / hy::GBN), 256, lds, s>>>(z, w_down, yrows, meta, maxTiles, top, d, F, 0.f, 0.f, 0.f);
    hy::moe_combine_kernel<<<T, 256, 0, s>>>(h, yrows, idx, wt, meta + 1 + maxTiles + maxTiles * hy::GBM, out, d, top, E);
}

}  // namespace chronos
