// Training forward of conv-attention on bf16 MFMA (gfx950).
//
// Workgroup = 4 waves = 128 query rows of one (batch, head); wave w owns rows
// i0 + 32w .. +31 and keeps their O^T accumulators, running max and partial row
// sums in registers for the whole key loop.  Per 64-key tile:
//   1. all waves stage K rows j0-8 .. j0+71 (row-major) and V rows j0 .. j0+63
//      (transposed, [d][key]) in LDS with 128-bit global loads;
//   2. each wave computes S^T = K Q^T for its 32 rows plus the 16 rows above
//      them (the query halo of the window), scales, applies the causal pre-mask
//      (zero) and writes the tile to its private LDS region as fp16;
//   3. convolution: c_q Toeplitz MFMAs per 16x16 block read the fp16 tile back
//      with the tap's row shift (see mfma_common.hpp);
//   4. post-mask (-inf), online softmax per query column of C^T (4 registers x
//      4 lane groups per row: two cross-lane steps for the max, sums stay
//      per-lane until the end);
//   5. O^T += V^T P^T with P^T taken straight from the softmax registers: the
//      MFMA k index is permuted (k = 8g+e <-> key 4g+e of block 0 for e < 4, of
//      block 1 for e >= 4) so no shuffle or LDS round trip is needed.
#include "mfma_common.hpp"

namespace convattn {
namespace {

constexpr int NW = 4;             // waves per workgroup
constexpr int WR = 32;            // output rows per wave
constexpr int BQ = NW * WR;       // 128
constexpr int BK = 64;            // output keys per tile
constexpr int SK = BK + 2 * kKeyHalo;  // score columns per tile (80)
constexpr int QH = 16;            // halo rows computed above a wave's rows
constexpr int SR = WR + QH;       // score rows per wave (48)
constexpr int SST = (SK + 8) * 2; // bytes per fp16 score row: 176 = 16 * odd
constexpr int VST = BK * 2 + 16;  // bytes per V^T row: 144

template <int D> struct FwdLds {
    static constexpr int KST = D * 2 + 16;  // bytes per K row (== 16 mod 256 for D = 128)
    static constexpr int k_bytes = SK * KST;
    static constexpr int v_bytes = D * VST;
    static constexpr int s_bytes = NW * SR * SST;
    static constexpr int total = k_bytes + v_bytes + s_bytes;
};

template <int D, int CQT, typename TO>
__global__ __launch_bounds__(NW * 64, 2) void fwd_mfma_kernel(
    Problem p, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const float *__restrict__ W, TO *__restrict__ O,
    float *__restrict__ M, float *__restrict__ L) {
    using Lds = FwdLds<D>;
    constexpr int KST = Lds::KST;
    constexpr int KS = D / 32;   // MFMA k-steps over the head dimension
    constexpr int DB = D / 16;   // 16-wide blocks of the head dimension
    constexpr int CPR = D / 8;   // 16-byte chunks per row
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem;
    unsigned char *Vt = smem + Lds::k_bytes;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    unsigned char *Ss = smem + Lds::k_bytes + Lds::v_bytes + wave * (SR * SST);

    const int h = blockIdx.y, b = blockIdx.z;
    const int qt = gridDim.x - 1 - blockIdx.x;  // longest (causal) tiles first
    const int i0 = qt * BQ, i0w = i0 + wave * WR;
    const int pk = p.pk, cq = p.c_q;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;

    // Toeplitz bands of this head, one fragment per query tap.
    f16x8 tf[CQT];
    load_bands<CQT>(tf, W + (size_t)h * cq * p.c_k, cq, p.c_k, pk, g, n, false);

    // Q^T fragments (B operand): rows i0w-16 .. i0w+31, resident for the whole loop.
    bf16x8 qf[3][KS];
#pragma unroll
    for (int rb = 0; rb < 3; ++rb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 raw = load_row16<D>(Qb, i0w - QH + rb * 16 + n, p.Nq, ks * 32 + g * 8);
            qf[rb][ks] = __builtin_bit_cast(bf16x8, raw);
        }

    f32x4 acc_o[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_o[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run[2] = {kNegInf, kNegInf};  // running max, in log2 units (C * log2 e)
    float l_run[2] = {0.f, 0.f};          // this lane's share of the row sum

    const float scale = p.scale * kLog2e;  // scores are kept in log2 units: the window is linear
    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    for (int j0 = 0; j0 < k_end; j0 += BK) {
        __syncthreads();
        // ---- stage K (row-major) and V (transposed) ----
        for (int c = tid; c < SK * CPR; c += NW * 64) {
            int row = c / CPR, cc = c - row * CPR;
            u32x4 v4 = load_row16<D>(Kb, j0 - kKeyHalo + row, p.Nk, cc * 8);
            *reinterpret_cast<u32x4 *>(Ks + row * KST + cc * 16) = v4;
        }
        for (int c = tid; c < BK * CPR; c += NW * 64) {
            int key = c & (BK - 1), cc = c >> 6;
            u32x4 v4 = load_row16<D>(Vb, j0 + key, p.Nk, cc * 8);
            unsigned short *dst = reinterpret_cast<unsigned short *>(Vt + (cc * 8) * VST + key * 2);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dst[(2 * e) * (VST / 2)] = (unsigned short)(v4[e] & 0xffffu);
                dst[(2 * e + 1) * (VST / 2)] = (unsigned short)(v4[e] >> 16);
            }
        }
        __syncthreads();
        if (causal && j0 > i0w + WR - 1) continue;  // every key of the tile is after this wave's rows

        // ---- S^T = K Q^T, scale, pre-mask, fp16 -> LDS ----
#pragma unroll
        for (int kb = 0; kb < SK / 16; ++kb) {
            f32x4 acc[3];
#pragma unroll
            for (int rb = 0; rb < 3; ++rb) acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8 kf = *reinterpret_cast<const bf16x8 *>(Ks + (kb * 16 + n) * KST + (ks * 32 + g * 8) * 2);
#pragma unroll
                for (int rb = 0; rb < 3; ++rb) acc[rb] = mfma_bf16(kf, qf[rb][ks], acc[rb]);
            }
            const int key0 = j0 - kKeyHalo + kb * 16 + 4 * g;
#pragma unroll
            for (int rb = 0; rb < 3; ++rb) {
                const int qpos = i0w - QH + rb * 16 + n;
                f16x4 hv;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float s = acc[rb][r] * scale;
                    if (causal && key0 + r > qpos) s = 0.f;
                    s = fminf(fmaxf(s, -kF16Max), kF16Max);
                    hv[r] = (_Float16)s;
                }
                *reinterpret_cast<f16x4 *>(Ss + (rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) = hv;
            }
        }
        __builtin_amdgcn_wave_barrier();

#pragma unroll
        for (int ob = 0; ob < 2; ++ob) {
            // ---- convolution: C^T block = sum_a T_a^T * S^T(rows shifted by a - pq) ----
            f32x4 c[BK / 16];
            const int srow = QH + ob * 16 + n - (CQT - 1);
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb) {
                c[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    f16x8 sf = *reinterpret_cast<const f16x8 *>(Ss + (srow + a) * SST + (kb * 16 + 8 * g) * 2);
                    c[kb] = mfma_f16(tf[a], sf, c[kb]);
                }
            }
            // ---- post-mask and online softmax (log2 domain) ----
            const int qpos = i0w + ob * 16 + n;
            float mx = kNegInf;
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = j0 + kb * 16 + 4 * g + r;
                    float x = c[kb][r];
                    if (key >= p.Nk || (causal && key > qpos)) x = kNegInf;
                    c[kb][r] = x;
                    mx = fmaxf(mx, x);
                }
            mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
            mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
            const float m_new = fmaxf(m_run[ob], mx);
            // rows with nothing visible yet keep m = -inf; use 0 as the exponent base there
            const float m_use = (m_new == kNegInf) ? 0.f : m_new;
            const float alpha = fast_exp2(m_run[ob] - m_use);
            m_run[ob] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float e = fast_exp2(c[kb][r] - m_use);
                    c[kb][r] = e;
                    psum += e;
                }
            l_run[ob] = l_run[ob] * alpha + psum;
#pragma unroll
            for (int db = 0; db < DB; ++db) acc_o[ob][db] *= alpha;
            // ---- O^T += V^T P^T ----
#pragma unroll
            for (int kp = 0; kp < BK / 32; ++kp) {
                bf16x8 pf;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pf[r] = (bf16_t)c[2 * kp][r];
                    pf[4 + r] = (bf16_t)c[2 * kp + 1][r];
                }
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const unsigned char *vrow = Vt + (db * 16 + n) * VST + (kp * 32 + 4 * g) * 2;
                    bf16x4 lo = *reinterpret_cast<const bf16x4 *>(vrow);
                    bf16x4 hi = *reinterpret_cast<const bf16x4 *>(vrow + 32);
                    bf16x8 vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    acc_o[ob][db] = mfma_bf16(vf, pf, acc_o[ob][db]);
                }
            }
        }
    }

    // ---- epilogue: finish the row sums, normalise, store O, M, L ----
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
        float l = l_run[ob];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        const int qpos = i0w + ob * 16 + n;
        if (qpos < p.Nq) {
            const float inv = 1.f / l;
            TO *orow = O + (bh * p.Nq + qpos) * D;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int col = db * 16 + 4 * g;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_o[ob][db][r] * inv);
                    *reinterpret_cast<bf16x4 *>(orow + col) = ov;
                } else {
                    f32x4 ov = acc_o[ob][db] * inv;
                    *reinterpret_cast<f32x4 *>(orow + col) = ov;
                }
            }
            if (g == 0) {
                M[bh * p.Nq + qpos] = m_run[ob] * (1.f / kLog2e);
                L[bh * p.Nq + qpos] = l;
            }
        }
    }
}

template <int D, int CQT, typename TO>
hipError_t launch_fwd(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                      void *o, float *m, float *l, hipStream_t s) {
    auto kern = fwd_mfma_kernel<D, CQT, TO>;
    constexpr int lds = FwdLds<D>::total;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
    }
    dim3 grid((p.Nq + BQ - 1) / BQ, p.H, p.B);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, w,
                                    (TO *)o, m, l);
    return hipGetLastError();
}

template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                   void *o, float *m, float *l, hipStream_t s) {
    if (p.c_q <= 3) return launch_fwd<D, 3, TO>(p, q, k, v, w, o, m, l, s);
    if (p.c_q <= 6) return launch_fwd<D, 6, TO>(p, q, k, v, w, o, m, l, s);
    return launch_fwd<D, 11, TO>(p, q, k, v, w, o, m, l, s);
}

}  // namespace

hipError_t mfma_fwd(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                    const float *w, void *o, float *m, float *l, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t>(p, q, k, v, w, o, m, l, s);
        return pick_cq<128, float>(p, q, k, v, w, o, m, l, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t>(p, q, k, v, w, o, m, l, s);
    return pick_cq<64, float>(p, q, k, v, w, o, m, l, s);
}

}  // namespace convattn
