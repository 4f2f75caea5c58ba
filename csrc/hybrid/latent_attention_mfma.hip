// latent_attention_mfma.hip — the bfloat16 latent attention on the matrix cores (see latent_attention.hip for the
// math: one cached row per token, key = the whole row, value = its first `rank` columns, shared by all heads).
//
// One workgroup takes 64 (token, head) rows of one sequence — 16 per wave, rows are (token * H + head), so any head
// count tiles the same way — and walks the sequence's keys 64 at a time:
//   * the key tile is staged twice in LDS: row-major [64][DK] for the scores, and the value columns transposed
//     [rank][64] for the weighted sum (both MFMA operands want 8 consecutive k-values per lane: dims for the scores,
//     KEYS for the sum).  One pass of 16-byte global loads feeds both; the transposed image is written as 32-bit
//     words holding two neighbouring keys.
//   * scores  S^T = K Q^T : 16x16x32 MFMAs with the key rows as A operand and the wave's 16 query rows (held in
//     registers for the whole kernel) as B operand, so a lane ends up with 4 keys x 1 query row per 16-key tile;
//   * softmax in float per query row (lane & 15): causal mask by the row's own position, running maximum and sum,
//     reductions over the 4 lane groups by two shuffles;
//   * sum  O^T = V^T P^T : the lane's 8 weights of two neighbouring 16-key tiles ARE a B operand (the k index is a
//     fixed permutation of the 32 keys, the same one the transposed value image is read with), so the weights never
//     leave registers.  Accumulators: rank / 16 tiles x 4 registers.
// Sizes: DK % 32 == 0, rank % 16 == 0, DK <= 576, rank <= 512.  Everything else takes latent_attention.hip.
#include <cstdlib>

#include "hybrid_common.h"

namespace chronos {
namespace hy {

constexpr int MKT = 64;  // keys per tile at most

// NS: k-steps of the scores (DK / 32) at most; NCT: 16-column tiles of the output (rank / 16) at most; KT: keys per
// tile, 64 or 32 (32 halves the LDS images, so two workgroups share a CU at the widest rows and one stages while the
// other multiplies).
// NW: waves per workgroup, 4 or 8 (16 query rows each): with 8 a staged key tile serves 128 rows and every SIMD holds two
// waves, so one wave's softmax and staging run beside the other's MFMAs.
template <int NS, int NCT, int KT, int NW>
__global__ void __launch_bounds__(64 * NW) latent_attention_mfma_kernel(
        const uint16_t* __restrict__ qa, const uint16_t* __restrict__ cache, const int32_t* __restrict__ block_table,
        int max_blocks, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos,
        const float* __restrict__ gate, uint16_t* __restrict__ out, int H, int DK, int rank, int BS, float scale,
        int nsplit, float* __restrict__ part_o, float* __restrict__ part_ml, int bs_shift) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int b = blockIdx.x;
    const int t0 = q_start[b], t1 = q_start[b + 1];
    const int rows_total = (t1 - t0) * H;
    constexpr int NT = 64 * NW, RPB = 16 * NW;  // threads and query rows per workgroup
    const int rb0 = blockIdx.y * RPB;
    if (rb0 >= rows_total) return;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, g = lane >> 4, qi = lane & 15;
    const int ns = DK / 32, nct = rank / 16;
    const int krs = DK * 2 + 16;            // row-major image: bytes per key row
    constexpr int vts = KT * 2 + 8;         // transposed image: bytes per value column
    constexpr int PP = KT / 2;              // key pairs per tile
    __shared__ int krow[MKT];  // cache row (page * page size + slot) of each key of the tile
    unsigned char* kimg = smem;
    unsigned char* vimg = smem + KT * krs;
    // this lane's query row (for the B operand and for the softmax): row r of the sequence, token t0 + r / H
    const int r = rb0 + wv * 16 + qi;
    const bool rok = r < rows_total;
    const int rc = rok ? r : rows_total - 1;
    const int64_t grow = (int64_t)t0 * H + rc;              // row of qa / out / gate
    const int prow = rok ? pos[t0 + rc / H] : -1;
    const int last_row = min(rows_total, rb0 + RPB) - 1;
    const int pmax = pos[t0 + last_row / H];                // positions grow along the sequence
    bf16x8 qf[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s)
        if (s < ns) qf[s] = *reinterpret_cast<const bf16x8*>(qa + grow * DK + 32 * s + 8 * g);
    f32x4 O[NCT];
#pragma unroll
    for (int c = 0; c < NCT; ++c) O[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    float mrow = -INFINITY, lrow = 0.f;
    const int32_t* bt = block_table + (int64_t)b * max_blocks;
    const int chunks = DK / 8, vchunks = rank / 8;
    // key tiles are dealt round-robin to the nsplit workgroups of this row block (blockIdx.z): the context length is
    // only known on the device, and a split that gets no tile contributes an empty partial
    for (int k0 = blockIdx.z * KT; k0 <= pmax; k0 += KT * nsplit) {
        __syncthreads();
        // ---- cache rows of the tile's 64 keys (page lookup once per key, not once per staged vector: a lookup in
        // front of every data load made each of them wait for two trips to memory)
        if (threadIdx.x < KT) {
            const int key = min(k0 + (int)threadIdx.x, pmax);  // past the end: a real row, masked below
            krow[threadIdx.x] = bs_shift >= 0 ? ((bt[key >> bs_shift] << bs_shift) + (key & (BS - 1)))
                                              : (bt[key / BS] * BS + key % BS);
        }
        __syncthreads();
        // ---- stage: work item = (key pair jp, 8-dim chunk dc); lanes of a wave take consecutive key pairs; three
        // items' loads (six 16-byte vectors) are issued before any of them is written to LDS
        for (int it0 = threadIdx.x; it0 < PP * chunks; it0 += NT * 3) {
            u16x8 va[3], vb[3];
#pragma unroll
            for (int u = 0; u < 3; ++u) {
                const int it = it0 + NT * u;
                if (it < PP * chunks) {
                    const int jp = it & (PP - 1), dc = it / PP;
                    va[u] = *reinterpret_cast<const u16x8*>(cache + (int64_t)krow[2 * jp] * DK + dc * 8);
                    vb[u] = *reinterpret_cast<const u16x8*>(cache + (int64_t)krow[2 * jp + 1] * DK + dc * 8);
                }
            }
#pragma unroll
            for (int u = 0; u < 3; ++u) {
                const int it = it0 + NT * u;
                if (it < PP * chunks) {
                    const int jp = it & (PP - 1), dc = it / PP;
                    *reinterpret_cast<u16x8*>(kimg + (2 * jp) * krs + dc * 16) = va[u];
                    *reinterpret_cast<u16x8*>(kimg + (2 * jp + 1) * krs + dc * 16) = vb[u];
                    if (dc < vchunks) {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            *reinterpret_cast<uint32_t*>(vimg + (dc * 8 + e) * vts + jp * 4) =
                                (uint32_t)va[u][e] | ((uint32_t)vb[u][e] << 16);
                    }
                }
            }
        }
        __syncthreads();
        // ---- scores: KT / 16 key tiles of 16; lane gets keys 16 kt + 4 g + i of query row qi
        constexpr int NKT = KT / 16;
        f32x4 S[NKT];
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            S[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
            const unsigned char* arow = kimg + (16 * kt + qi) * krs + g * 16;
#pragma unroll
            for (int s = 0; s < NS; ++s)
                if (s < ns)
                    S[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8*>(arow + s * 64), qf[s],
                                                                    S[kt], 0, 0, 0);
        }
        // ---- softmax over the tile for query row qi (this lane and the 3 other lane groups hold its keys)
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k0 + 16 * kt + 4 * g + i;
                const float sv = key <= prow ? S[kt][i] * scale : -INFINITY;
                S[kt][i] = sv;
                mx = fmaxf(mx, sv);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mn = fmaxf(mrow, mx);
        const float corr = (mn == -INFINITY) ? 1.f : __expf(mrow - mn);
        float sum = 0.f;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = (mn == -INFINITY) ? 0.f : __expf(S[kt][i] - mn);
                S[kt][i] = p;
                sum += p;
            }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        lrow = lrow * corr + sum;
        mrow = mn;
        // ---- weighted sum of the value columns: k index of step u = [tile 2u keys 4g..4g+3 | tile 2u+1 keys 4g..4g+3]
        constexpr int NU = KT / 32;
        bf16x8 pf[NU];
#pragma unroll
        for (int u = 0; u < NU; ++u)
            pf[u] = bf16x8{(__bf16)S[2 * u][0], (__bf16)S[2 * u][1], (__bf16)S[2 * u][2], (__bf16)S[2 * u][3],
                           (__bf16)S[2 * u + 1][0], (__bf16)S[2 * u + 1][1], (__bf16)S[2 * u + 1][2], (__bf16)S[2 * u + 1][3]};
#pragma unroll
        for (int c = 0; c < NCT; ++c) {
            if (c < nct) {
                O[c] *= corr;
                const unsigned char* vrow = vimg + (16 * c + qi) * vts + g * 8;
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    const bf16x4 lo = *reinterpret_cast<const bf16x4*>(vrow + u * 64);
                    const bf16x4 hi = *reinterpret_cast<const bf16x4*>(vrow + u * 64 + 32);
                    const bf16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    O[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[u], O[c], 0, 0, 0);
                }
            }
        }
    }
    if (!rok) return;
    if (nsplit > 1) {  // unnormalised partial: the combine kernel merges the splits
        const int64_t pr = grow * nsplit + blockIdx.z;
        if (g == 0) {
            part_ml[pr * 2] = mrow;
            part_ml[pr * 2 + 1] = lrow;
        }
#pragma unroll
        for (int c = 0; c < NCT; ++c)
            if (c < nct) *reinterpret_cast<f32x4*>(part_o + pr * rank + 16 * c + 4 * g) = O[c];
        return;
    }
    float f = 1.f / lrow;
    if (gate != nullptr) f *= sigmoidf_(gate[grow]);
    // lane holds O^T[col = 16 c + 4 g + i][query row qi]
#pragma unroll
    for (int c = 0; c < NCT; ++c)
        if (c < nct) {
            const u16x4 o = u16x4{f2bf(O[c][0] * f), f2bf(O[c][1] * f), f2bf(O[c][2] * f), f2bf(O[c][3] * f)};
            *reinterpret_cast<u16x4*>(out + grow * rank + 16 * c + 4 * g) = o;
        }
}

// one wave per (token, head) row: out = sum_z exp(m_z - m) O_z / sum_z exp(m_z - m) l_z * sigmoid(gate)
__global__ void __launch_bounds__(256) latent_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                             const float* __restrict__ gate, uint16_t* __restrict__ out,
                                                             int64_t rows, int rank, int nsplit) {
    const int lane = threadIdx.x & 63;
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    float m = -INFINITY;
    for (int z = 0; z < nsplit; ++z) m = fmaxf(m, part_ml[(r * nsplit + z) * 2]);
    float l = 0.f;
    for (int z = 0; z < nsplit; ++z) {
        const float mz = part_ml[(r * nsplit + z) * 2];
        if (mz != -INFINITY) l += expf(mz - m) * part_ml[(r * nsplit + z) * 2 + 1];
    }
    float f = 1.f / l;
    if (gate != nullptr) f *= sigmoidf_(gate[r]);
    for (int c = lane; c < rank; c += 64) {
        float acc = 0.f;
        for (int z = 0; z < nsplit; ++z) {
            const float mz = part_ml[(r * nsplit + z) * 2];
            if (mz != -INFINITY) acc += expf(mz - m) * part_o[(r * nsplit + z) * rank + c];
        }
        out[r * rank + c] = f2bf(acc * f);
    }
}

}  // namespace hy

template <int NS, int NCT, int KT, int NW>
static void la_mfma_launch(const uint16_t* qa, const uint16_t* cache, const int32_t* bt, int max_blocks,
                           const int32_t* q_start, const int32_t* pos, const float* gate, uint16_t* out, int B, int H,
                           int DK, int rank, int BS, int max_q, float scale, int nsplit, float* part_o, float* part_ml,
                           hipStream_t s) {
    auto kern = hy::latent_attention_mfma_kernel<NS, NCT, KT, NW>;
    const int bytes = KT * (DK * 2 + 16) + rank * (KT * 2 + 8);
    static int set_bytes = 0;
    if (bytes > set_bytes) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
        set_bytes = bytes;
    }
    const dim3 grid(B, (max_q * H + 16 * NW - 1) / (16 * NW), nsplit);
    const int bs_shift = (BS & (BS - 1)) == 0 ? __builtin_ctz(BS) : -1;
    kern<<<grid, 64 * NW, bytes, s>>>(qa, cache, bt, max_blocks, q_start, pos, gate, out, H, DK, rank, BS, scale, nsplit, part_o,
                                  part_ml, bs_shift);
}

bool hy_latent_mfma_ok(int DK, int rank) { return !(DK % 32 || rank % 16 || DK > 576 || rank > 512 || rank > DK); }

// Splits of the key range (flash-decoding) for a launch of `wgs` workgroups over contexts of at most max_ctx keys:
// enough workgroups to cover the chip, at least 4 key tiles per split, at most 16.
int hy_latent_nsplit(int wgs, int max_ctx) {
    if (wgs >= 128) return 1;
    int want = (256 + wgs - 1) / wgs, cap = max_ctx / (4 * hy::MKT);
    if (want > 16) want = 16;
    if (want > cap) want = cap;
    return want < 1 ? 1 : want;
}

// false: these sizes are not served here (the caller takes the general kernel).  nsplit > 1: part_o float
// [T * H * nsplit, rank] and part_ml float [T * H * nsplit, 2] scratch.
bool launch_hy_latent_attention_mfma(const uint16_t* qa, const uint16_t* cache, const int32_t* bt, int max_blocks,
                                     const int32_t* q_start, const int32_t* pos, const float* gate, uint16_t* out, int B,
                                     int H, int DK, int rank, int BS, int max_q, float scale, int nsplit, float* part_o,
                                     float* part_ml, int64_t total_rows, hipStream_t s) {
    if (!hy_latent_mfma_ok(DK, rank)) return false;
    if (B == 0 || max_q == 0) return true;
#define HY_LAM(NS, NCT, KT, NW) la_mfma_launch<NS, NCT, KT, NW>(qa, cache, bt, max_blocks, q_start, pos, gate, out, B, H, DK, rank, BS, max_q, scale, nsplit, part_o, part_ml, s)
    // 64-key tiles (32-key tiles measured slower at every size: the per-tile softmax and barriers weigh more than the
    // second workgroup per CU gains; CHRONOS_LATENT_KT=32 keeps them for A/B).  8 waves per workgroup when a sequence
    // brings more than 64 rows (CHRONOS_LATENT_NW=4 / 8 forces one).
    static const int force_kt = [] { const char* v = getenv("CHRONOS_LATENT_KT"); return v ? atoi(v) : 0; }();
    static const int force_nw = [] { const char* v = getenv("CHRONOS_LATENT_NW"); return v ? atoi(v) : 0; }();
    const bool kt32 = force_kt == 32;
    const bool nw8 = force_nw == 8 || (force_nw != 4 && max_q * H > 64);
#define HY_LAM_T(NS, NCT)                                                            \
    do {                                                                             \
        if (kt32) { if (nw8) HY_LAM(NS, NCT, 32, 8); else HY_LAM(NS, NCT, 32, 4); }   \
        else { if (nw8) HY_LAM(NS, NCT, 64, 8); else HY_LAM(NS, NCT, 64, 4); }       \
    } while (0)
    if (DK <= 128 && rank <= 64) HY_LAM_T(4, 4);
    else if (DK <= 320 && rank <= 256) HY_LAM_T(10, 16);
    else HY_LAM_T(18, 32);
#undef HY_LAM_T
#undef HY_LAM
    if (nsplit > 1)
        hy::latent_combine_kernel<<<(unsigned)((total_rows + 3) / 4), 256, 0, s>>>(part_o, part_ml, gate, out, total_rows, rank, nsplit);
    return true;
}

}  // namespace chronos
