// Backward of conv-attention on bf16 MFMA (gfx950): dK and dV.
//
// Workgroup = 4 waves = 128 keys of one (batch, head); wave w owns keys
// c0 = k0 + 32w .. c0+31 for dK and, because the convolved blocks sit 8 keys
// before the window-aligned ones, keys c0-8 .. c0+23 for dV (the shifted ranges
// of neighbouring waves and workgroups tile the key axis just the same).  The
// wave keeps its K and V fragments and both accumulators in registers and walks
// the queries in 32-row tiles that the workgroup stages in LDS (Q and dO
// row-major for the score / dP products, transposed for the dK / dV products).
// Per tile, with r0 its first row:
//   S^T  rows r0-16 .. r0+47, keys c0-16 .. c0+47    K Q^T, pre-masked, fp16 -> LDS
//   C    rows r0 .. r0+47, keys c0-8 .. c0+39        Toeplitz MFMAs, here oriented
//        [query][key] so that a lane holds one key and 4 query rows: that is the
//        operand layout the dV and dK products need, no transposition in between
//   P = exp(C - LSE), dP = dO V^T, dC = P (dP - D): fp16 -> LDS (2-byte stores)
//   dV^T += dO^T P        (rows r0 .. r0+31, keys c0-8 .. c0+23)
//   dS   rows r0 .. r0+31, keys c0 .. c0+31: flipped-band MFMAs over dC, causal zero
//   dK^T += Q^T dS
#include "mfma_common.hpp"

namespace convattn {
namespace {

constexpr int NW = 4;
constexpr int WK = 32;                 // own keys per wave
constexpr int BKW = NW * WK;           // 128 keys per workgroup
constexpr int BR = 32;                 // query rows per tile
constexpr int S_ROWS = BR + 32;        // 64
constexpr int S_COLS = WK + 32;        // 64
constexpr int C_ROWS = BR + 16;        // 48
constexpr int C_COLS = WK + 16;        // 48
constexpr int SST = (S_COLS + 8) * 2;  // 144
constexpr int CST = (C_COLS + 8) * 2;  // 112
constexpr int TST = BR * 2 + 16;       // 80 bytes per row of Q^T / dO^T

template <int D> struct KvLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int q_bytes = S_ROWS * RST;
    static constexpr int g_bytes = C_ROWS * RST;
    static constexpr int qt_bytes = D * TST;
    static constexpr int gt_bytes = D * TST;
    static constexpr int stat_bytes = 2 * C_ROWS * 4;
    static constexpr int wave_bytes = S_ROWS * SST + C_ROWS * CST;
    static constexpr int total = q_bytes + g_bytes + qt_bytes + gt_bytes + stat_bytes + NW * wave_bytes;
};

__device__ __forceinline__ void store_transposed(unsigned char *dst_base, int tst, int col8, int row,
                                                 u32x4 v4) {
    unsigned short *dst = reinterpret_cast<unsigned short *>(dst_base + (col8 * 8) * tst + row * 2);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        dst[(2 * e) * (tst / 2)] = (unsigned short)(v4[e] & 0xffffu);
        dst[(2 * e + 1) * (tst / 2)] = (unsigned short)(v4[e] >> 16);
    }
}

template <int D, int CQT, typename TO>
__global__ __launch_bounds__(NW * 64) void bwd_dkdv_mfma_kernel(
    Problem p, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const bf16_t *__restrict__ dO, const float *__restrict__ Dl,
    const float *__restrict__ LSE, const float *__restrict__ W, TO *__restrict__ dK,
    TO *__restrict__ dV) {
    using Lds = KvLds<D>;
    constexpr int RST = Lds::RST;
    constexpr int KS = D / 32, DB = D / 16, CPR = D / 8;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Qs = smem;
    unsigned char *Gs = Qs + Lds::q_bytes;
    unsigned char *Qt = Gs + Lds::g_bytes;
    unsigned char *Gt = Qt + Lds::qt_bytes;
    float *lse_s = reinterpret_cast<float *>(Gt + Lds::gt_bytes);
    float *dl_s = lse_s + C_ROWS;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    unsigned char *Ss = Gt + Lds::gt_bytes + Lds::stat_bytes + wave * Lds::wave_bytes;
    unsigned char *Cs = Ss + S_ROWS * SST;

    const int h = blockIdx.y, b = blockIdx.z;
    const int k0 = blockIdx.x * BKW, c0 = k0 + wave * WK;
    const int pk = p.pk, cq = p.c_q, ck = p.c_k;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;
    const bf16_t *dOb = dO + bh * p.Nq * D;
    const float *lse_b = LSE + bh * p.Nq;
    const float *dl_b = Dl + bh * p.Nq;

    f16x8 tf[CQT], tfl[CQT];
    load_bands<CQT>(tf, W + (size_t)h * cq * ck, cq, ck, pk, g, n, false, 1.f);
    load_bands<CQT>(tfl, W + (size_t)h * cq * ck, cq, ck, pk, g, n, true, 1.f);

    bf16x8 kf[4][KS];  // K rows c0-16 .. c0+47
    bf16x8 vf[3][KS];  // V rows c0-8 .. c0+39
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            kf[kb][ks] = __builtin_bit_cast(bf16x8, load_row16<D>(Kb, c0 - 16 + kb * 16 + n, p.Nk, ks * 32 + g * 8));
#pragma unroll
    for (int kb = 0; kb < 3; ++kb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            vf[kb][ks] = __builtin_bit_cast(bf16x8, load_row16<D>(Vb, c0 - 8 + kb * 16 + n, p.Nk, ks * 32 + g * 8));

    f32x4 acc_k[2][DB], acc_v[2][DB];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            acc_k[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
            acc_v[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }

    const float scale = p.scale;
    const float scale2 = p.scale * kLog2e;  // score tile in log2 units (the window is linear)
    // Causal: rows before the first key this workgroup touches (k0 - 8) see none of its keys.
    const int r_begin = causal ? (max(0, k0 - 8) / BR) * BR : 0;
    for (int r0 = r_begin; r0 < p.Nq; r0 += BR) {
        __syncthreads();
        for (int c = tid; c < S_ROWS * CPR; c += NW * 64) {
            int row = c / CPR, cc = c - row * CPR;
            u32x4 v4 = load_row16<D>(Qb, r0 - 16 + row, p.Nq, cc * 8);
            *reinterpret_cast<u32x4 *>(Qs + row * RST + cc * 16) = v4;
            if (row >= 16 && row < 16 + BR) store_transposed(Qt, TST, cc, row - 16, v4);
        }
        for (int c = tid; c < C_ROWS * CPR; c += NW * 64) {
            int row = c / CPR, cc = c - row * CPR;
            u32x4 v4 = load_row16<D>(dOb, r0 + row, p.Nq, cc * 8);
            *reinterpret_cast<u32x4 *>(Gs + row * RST + cc * 16) = v4;
            if (row < BR) store_transposed(Gt, TST, cc, row, v4);
        }
        if (tid < C_ROWS) {
            int qr = r0 + tid;
            lse_s[tid] = qr < p.Nq ? lse_b[qr] * kLog2e : 0.f;
            dl_s[tid] = qr < p.Nq ? dl_b[qr] : 0.f;
        }
        __syncthreads();
        if (causal && r0 + BR - 1 < c0 - 8) continue;  // none of the tile's own rows sees the wave's keys

        // ---- S^T tile -> fp16 LDS ----
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            f32x4 acc[4];
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) acc[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8 qf = *reinterpret_cast<const bf16x8 *>(Qs + (rb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
#pragma unroll
                for (int kb = 0; kb < 4; ++kb) acc[kb] = mfma_bf16(kf[kb][ks], qf, acc[kb]);
            }
            const int qpos = r0 - 16 + rb * 16 + n;
#pragma unroll
            for (int kb = 0; kb < 4; ++kb) {
                const int key0 = c0 - 16 + kb * 16 + 4 * g;
                f16x4 hv;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float s = acc[kb][r] * scale2;
                    if (causal && key0 + r > qpos) s = 0.f;
                    s = fminf(fmaxf(s, -kF16Max), kF16Max);
                    hv[r] = (_Float16)s;
                }
                *reinterpret_cast<f16x4 *>(Ss + (rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) = hv;
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- C, P, dP, dC ([query][key] orientation: lane = key, registers = 4 rows) ----
        f32x4 pkeep[2][2];
#pragma unroll
        for (int rb = 0; rb < 3; ++rb) {
            const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(lse_s + rb * 16 + 4 * g);
            const f32x4 dl4 = *reinterpret_cast<const f32x4 *>(dl_s + rb * 16 + 4 * g);
            const int srow = 16 + rb * 16 + n - (CQT - 1);
#pragma unroll
            for (int kb = 0; kb < 3; ++kb) {
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    f16x8 sf = *reinterpret_cast<const f16x8 *>(Ss + (srow + a) * SST + (kb * 16 + 8 * g) * 2);
                    c = mfma_f16(sf, tf[a], c);
                }
                f32x4 dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    bf16x8 gf = *reinterpret_cast<const bf16x8 *>(Gs + (rb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
                    dp = mfma_bf16(gf, vf[kb][ks], dp);
                }
                const int key = c0 - 8 + kb * 16 + n;
                f32x4 pr;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int qpos = r0 + rb * 16 + 4 * g + r;
                    float e = fast_exp2(c[r] - lse4[r]);
                    float dc = e * (dp[r] - dl4[r]);
                    if (key < 0 || key >= p.Nk || qpos >= p.Nq || (causal && key > qpos)) { e = 0.f; dc = 0.f; }
                    dc = fminf(fmaxf(dc, -kF16Max), kF16Max);
                    pr[r] = e;
                    *reinterpret_cast<_Float16 *>(Cs + (rb * 16 + 4 * g + r) * CST + (kb * 16 + n) * 2) = (_Float16)dc;
                }
                if (rb < 2 && kb < 2) pkeep[rb][kb] = pr;
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- dV^T += dO^T P  (keys c0-8 .. c0+23) ----
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            bf16x8 pf;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pf[r] = (bf16_t)pkeep[0][kb][r];
                pf[4 + r] = (bf16_t)pkeep[1][kb][r];
            }
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const unsigned char *grow = Gt + (db * 16 + n) * TST + (4 * g) * 2;
                bf16x4 lo = *reinterpret_cast<const bf16x4 *>(grow);
                bf16x4 hi = *reinterpret_cast<const bf16x4 *>(grow + 32);
                bf16x8 gf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                acc_v[kb][db] = mfma_bf16(gf, pf, acc_v[kb][db]);
            }
        }

        // ---- dS (keys c0 .. c0+31) and dK^T += Q^T dS ----
        f32x4 ds[2][2];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    f16x8 cf = *reinterpret_cast<const f16x8 *>(Cs + (ob * 16 + n + (CQT - 1) - a) * CST + (m * 16 + 8 * g) * 2);
                    s = mfma_f16(cf, tfl[a], s);
                }
                if (causal) {
                    const int key = c0 + m * 16 + n;
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (key > r0 + ob * 16 + 4 * g + r) s[r] = 0.f;
                }
                ds[ob][m] = s;
            }
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            bf16x8 sf;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                sf[r] = (bf16_t)ds[0][m][r];
                sf[4 + r] = (bf16_t)ds[1][m][r];
            }
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const unsigned char *qrow = Qt + (db * 16 + n) * TST + (4 * g) * 2;
                bf16x4 lo = *reinterpret_cast<const bf16x4 *>(qrow);
                bf16x4 hi = *reinterpret_cast<const bf16x4 *>(qrow + 32);
                bf16x8 qf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                acc_k[m][db] = mfma_bf16(qf, sf, acc_k[m][db]);
            }
        }
    }

    // ---- stores: lane = key, 4 consecutive head-dim columns per block ----
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const int key_k = c0 + m * 16 + n;
        const int key_v = c0 - 8 + m * 16 + n;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int col = db * 16 + 4 * g;
            if (key_k < p.Nk) {
                TO *dst = dK + (bh * p.Nk + key_k) * D + col;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_k[m][db][r] * scale);
                    *reinterpret_cast<bf16x4 *>(dst) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(dst) = acc_k[m][db] * scale;
                }
            }
            if (key_v >= 0 && key_v < p.Nk) {
                TO *dst = dV + (bh * p.Nk + key_v) * D + col;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)acc_v[m][db][r];
                    *reinterpret_cast<bf16x4 *>(dst) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(dst) = acc_v[m][db];
                }
            }
        }
    }
}

template <int D, int CQT, typename TO>
hipError_t launch_kv(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                     const float *Dl, const float *lse, const float *w, void *dk, void *dv,
                     hipStream_t s) {
    auto kern = bwd_dkdv_mfma_kernel<D, CQT, TO>;
    constexpr int lds = KvLds<D>::total;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    // + 8: the last workgroup's dV range starts 8 keys early, so the key axis needs 8 more
    dim3 grid((p.Nk + 8 + BKW - 1) / BKW, p.H, p.B);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v,
                                    (const bf16_t *)d_o, Dl, lse, w, (TO *)dk, (TO *)dv);
    return hipGetLastError();
}

template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                   const float *Dl, const float *lse, const float *w, void *dk, void *dv,
                   hipStream_t s) {
    if (p.c_q <= 3) return launch_kv<D, 3, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
    if (p.c_q <= 6) return launch_kv<D, 6, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
    return launch_kv<D, 11, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
}

}  // namespace

hipError_t mfma_bwd_dkdv(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                         const void *d_o, const float *Dl, const float *lse, const float *w, void *dk,
                         void *dv, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
        return pick_cq<128, float>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
    return pick_cq<64, float>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
}

}  // namespace convattn
