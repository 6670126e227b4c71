// Backward of conv-attention on bf16 MFMA (gfx950): dQ and the dW partials.
//
// Workgroup = 4 waves = 128 query rows of one (batch, head); wave w owns rows
// r0 = i0 + 32w .. r0+31 and walks the keys in 64-wide tiles.  Everything a
// tile needs beyond K/V (staged once per workgroup) is private to the wave, so
// there is no barrier inside a tile.  With c0 the tile's first key:
//   S^T   rows r0-16 .. r0+47, keys c0-16 .. c0+79   scale*K Q^T, pre-masked, fp16 -> LDS
//   C^T   rows r0    .. r0+47, keys c0-8  .. c0+71   Toeplitz MFMAs over the fp16 tile
//   P     = exp(C - LSE) (0 where masked); dP^T = V dO^T on the same blocks
//   dC^T  = P * (dP - D), fp16 -> LDS (rows r0 .. r0+47: own rows plus the rows
//           below them that the transposed window reaches)
//   dS^T  rows r0 .. r0+31, keys c0 .. c0+63: Toeplitz MFMAs with the flipped taps
//           over dC rows shifted down by pad_q - a, then the causal zero
//   dQ^T += K^T dS^T  (K^T staged transposed in LDS; dS^T straight from registers)
//   dW[a][b] += sum over own rows i and keys j' in the tile of
//           S_m[i+a-pq][j'] * dC[i][j'-b+pk]: one MFMA chain with M = a, N = b and
//           the (row, 8 keys) pairs as the contraction; the dC operand is read
//           from LDS at a 2-byte granular offset.
// Every (dC row, S key) pair belongs to exactly one (wave, tile), so the dW
// partials of the waves add up to the full gradient; they are summed over the
// workgroup in a fixed order and stored per workgroup.
#include "mfma_common.hpp"

namespace convattn {
namespace {

constexpr int NW = 4;
constexpr int WR = 32;                 // own query rows per wave
constexpr int BQ = NW * WR;            // 128
constexpr int BK = 64;                 // own keys per tile
constexpr int S_ROWS = WR + 32;        // 64: 16 above, 16 below
constexpr int S_COLS = BK + 32;        // 96: 16 either side
constexpr int C_ROWS = WR + 16;        // 48
constexpr int C_COLS = BK + 16;        // 80: 8 either side
constexpr int SST = (S_COLS + 8) * 2;  // 208 bytes per fp16 score row
constexpr int CST = (C_COLS + 8) * 2;  // 176 bytes per fp16 dC row
constexpr int TST = BK * 2 + 16;       // 144 bytes per K^T row

template <int D> struct DqLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int k_bytes = S_COLS * RST;
    static constexpr int v_bytes = C_COLS * RST;
    static constexpr int kt_bytes = D * TST;
    static constexpr int wave_bytes = S_ROWS * SST + C_ROWS * CST;
    static constexpr int total = k_bytes + v_bytes + kt_bytes + NW * wave_bytes;
};

template <int D, int CQT, typename TO>
__global__ __launch_bounds__(NW * 64) void bwd_dq_mfma_kernel(
    Problem p, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const bf16_t *__restrict__ dO, const float *__restrict__ Dl,
    const float *__restrict__ LSE, const float *__restrict__ W, TO *__restrict__ dQ,
    float *__restrict__ dW_part) {
    using Lds = DqLds<D>;
    constexpr int RST = Lds::RST;
    constexpr int KS = D / 32, DB = D / 16, CPR = D / 8;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem;
    unsigned char *Vs = Ks + Lds::k_bytes;
    unsigned char *Kt = Vs + Lds::v_bytes;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    unsigned char *Ss = Kt + Lds::kt_bytes + wave * Lds::wave_bytes;
    unsigned char *Cs = Ss + S_ROWS * SST;

    const int h = blockIdx.y, b = blockIdx.z;
    const int qt = gridDim.x - 1 - blockIdx.x;
    const int i0 = qt * BQ, r0 = i0 + wave * WR;
    const int pq = p.pq, pk = p.pk, cq = p.c_q, ck = p.c_k;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;
    const bf16_t *dOb = dO + bh * p.Nq * D;

    f16x8 tf[CQT], tfl[CQT];  // forward band and flipped (transposed-window) band per tap slot
    load_bands<CQT>(tf, W + (size_t)h * cq * ck, cq, ck, pk, g, n, false, 1.f);
    load_bands<CQT>(tfl, W + (size_t)h * cq * ck, cq, ck, pk, g, n, true, 1.f);

    bf16x8 qf[4][KS];   // Q rows r0-16 .. r0+47
    bf16x8 gf[3][KS];   // dO rows r0 .. r0+47
    float lse2[3], dl[3];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qf[rb][ks] = __builtin_bit_cast(bf16x8, load_row16<D>(Qb, r0 - 16 + rb * 16 + n, p.Nq, ks * 32 + g * 8));
#pragma unroll
    for (int rb = 0; rb < 3; ++rb) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            gf[rb][ks] = __builtin_bit_cast(bf16x8, load_row16<D>(dOb, r0 + rb * 16 + n, p.Nq, ks * 32 + g * 8));
        const int qpos = r0 + rb * 16 + n;
        lse2[rb] = qpos < p.Nq ? LSE[bh * p.Nq + qpos] * kLog2e : 0.f;
        dl[rb] = qpos < p.Nq ? Dl[bh * p.Nq + qpos] : 0.f;
    }

    f32x4 acc_q[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_q[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    f32x4 acc_w = {0.f, 0.f, 0.f, 0.f};
    const int bcl = n < ck ? n : ck - 1;  // lanes past the last key tap re-read a valid one

    const float scale = p.scale;
    const float scale2 = p.scale * kLog2e;  // score tile in log2 units (the window is linear)
    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    for (int c0 = 0; c0 < k_end; c0 += BK) {
        __syncthreads();
        for (int c = tid; c < S_COLS * CPR; c += NW * 64) {
            int row = c / CPR, cc = c - row * CPR;
            u32x4 v4 = load_row16<D>(Kb, c0 - 16 + row, p.Nk, cc * 8);
            *reinterpret_cast<u32x4 *>(Ks + row * RST + cc * 16) = v4;
            if (row >= 16 && row < 16 + BK) {  // own keys also go in transposed
                unsigned short *dst = reinterpret_cast<unsigned short *>(Kt + (cc * 8) * TST + (row - 16) * 2);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dst[(2 * e) * (TST / 2)] = (unsigned short)(v4[e] & 0xffffu);
                    dst[(2 * e + 1) * (TST / 2)] = (unsigned short)(v4[e] >> 16);
                }
            }
        }
        for (int c = tid; c < C_COLS * CPR; c += NW * 64) {
            int row = c / CPR, cc = c - row * CPR;
            u32x4 v4 = load_row16<D>(Vb, c0 - 8 + row, p.Nk, cc * 8);
            *reinterpret_cast<u32x4 *>(Vs + row * RST + cc * 16) = v4;
        }
        __syncthreads();
        if (causal && c0 > r0 + WR - 1) continue;

        // ---- S^T tile -> fp16 LDS ----
#pragma unroll
        for (int kb = 0; kb < S_COLS / 16; ++kb) {
            f32x4 acc[4];
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8 kf = *reinterpret_cast<const bf16x8 *>(Ks + (kb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) acc[rb] = mfma_bf16(kf, qf[rb][ks], acc[rb]);
            }
            const int key0 = c0 - 16 + kb * 16 + 4 * g;
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const int qpos = r0 - 16 + rb * 16 + n;
                f16x4 hv;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float s = acc[rb][r] * scale2;
                    if (causal && key0 + r > qpos) s = 0.f;
                    s = fminf(fmaxf(s, -kF16Max), kF16Max);
                    hv[r] = (_Float16)s;
                }
                *reinterpret_cast<f16x4 *>(Ss + (rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) = hv;
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- C^T, P, dP^T, dC^T -> fp16 LDS ----
#pragma unroll
        for (int rb = 0; rb < 3; ++rb) {
            const int qpos = r0 + rb * 16 + n;
            const int srow = 16 + rb * 16 + n - (CQT - 1);  // S-tile row of tap slot 0
#pragma unroll
            for (int kb = 0; kb < C_COLS / 16; ++kb) {
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    // keys c0-8+16kb .. need S keys from 8 before: S-tile column 16kb
                    f16x8 sf = *reinterpret_cast<const f16x8 *>(Ss + (srow + a) * SST + (kb * 16 + 8 * g) * 2);
                    c = mfma_f16(tf[a], sf, c);
                }
                f32x4 dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    bf16x8 vf = *reinterpret_cast<const bf16x8 *>(Vs + (kb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
                    dp = mfma_bf16(vf, gf[rb][ks], dp);
                }
                f16x4 hv;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = c0 - 8 + kb * 16 + 4 * g + r;
                    float pr = fast_exp2(c[r] - lse2[rb]);
                    float dc = pr * (dp[r] - dl[rb]);
                    if (key < 0 || key >= p.Nk || qpos >= p.Nq || (causal && key > qpos)) dc = 0.f;
                    dc = fminf(fmaxf(dc, -kF16Max), kF16Max);
                    hv[r] = (_Float16)dc;
                }
                *reinterpret_cast<f16x4 *>(Cs + (rb * 16 + n) * CST + (kb * 16 + 4 * g) * 2) = hv;
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- dS^T (transposed window) and dQ^T += K^T dS^T ----
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) {
            const int qpos = r0 + ob * 16 + n;
            f32x4 ds[BK / 16];
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb) {
                ds[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    f16x8 cf = *reinterpret_cast<const f16x8 *>(Cs + (ob * 16 + n + (CQT - 1) - a) * CST + (kb * 16 + 8 * g) * 2);
                    ds[kb] = mfma_f16(tfl[a], cf, ds[kb]);
                }
                if (causal) {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (c0 + kb * 16 + 4 * g + r > qpos) ds[kb][r] = 0.f;
                }
            }
#pragma unroll
            for (int kp = 0; kp < BK / 32; ++kp) {
                bf16x8 sf;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    sf[r] = (bf16_t)ds[2 * kp][r];
                    sf[4 + r] = (bf16_t)ds[2 * kp + 1][r];
                }
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const unsigned char *krow = Kt + (db * 16 + n) * TST + (kp * 32 + 4 * g) * 2;
                    bf16x4 lo = *reinterpret_cast<const bf16x4 *>(krow);
                    bf16x4 hi = *reinterpret_cast<const bf16x4 *>(krow + 32);
                    bf16x8 kf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    acc_q[ob][db] = mfma_bf16(kf, sf, acc_q[ob][db]);
                }
            }
        }

        // ---- dW: rows m = tap a, columns n = tap b, contraction over (own row, 8 keys) ----
        {
            // A: S_m[i + a - pq][c0 + 32jb + 8g ..]   (S-tile row 16 + i + a - pq, column 16 + ...)
            // B: dC[i][c0 + 32jb + 8g - b + pk ..]    (dC-tile column 8 + ... - b + pk)
            const unsigned char *abase = Ss + (16 + n - pq) * SST + (16 + 8 * g) * 2;
            const unsigned char *bbase = Cs + (8 + 8 * g - bcl + pk) * 2;
            for (int i = 0; i < WR; ++i) {
#pragma unroll
                for (int jb = 0; jb < BK / 32; ++jb) {
                    f16x8 af = *reinterpret_cast<const f16x8 *>(abase + i * SST + jb * 64);
                    f16x8 bf = reinterpret_cast<const F16x8U *>(bbase + i * CST + jb * 64)->v;
                    acc_w = mfma_f16(af, bf, acc_w);
                }
            }
        }
    }

    // ---- dQ = scale * acc ----
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
        const int qpos = r0 + ob * 16 + n;
        if (qpos < p.Nq) {
            TO *orow = dQ + (bh * p.Nq + qpos) * D;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int col = db * 16 + 4 * g;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_q[ob][db][r] * scale);
                    *reinterpret_cast<bf16x4 *>(orow + col) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(orow + col) = acc_q[ob][db] * scale;
                }
            }
        }
    }

    // ---- dW partial of this workgroup: ordered sum over the 4 waves ----
    __syncthreads();
    float *red = reinterpret_cast<float *>(smem);  // [NW][16][16]
#pragma unroll
    for (int r = 0; r < 4; ++r) red[(wave * 16 + 4 * g + r) * 16 + n] = acc_w[r];
    __syncthreads();
    const int ntap = cq * ck;
    if (tid < ntap) {
        const int a = tid / ck, bb = tid - a * ck;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[(w * 16 + a) * 16 + bb];
        dW_part[(bh * gridDim.x + qt) * ntap + tid] = s * (1.f / kLog2e);  // S tile was in log2 units
    }
}

template <int D, int CQT, typename TO>
hipError_t launch_dq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                     const float *Dl, const float *lse, const float *w, void *dq, float *dw_part,
                     hipStream_t s) {
    auto kern = bwd_dq_mfma_kernel<D, CQT, TO>;
    constexpr int lds = DqLds<D>::total;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    dim3 grid(mfma_dq_tiles(p), p.H, p.B);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v,
                                    (const bf16_t *)d_o, Dl, lse, w, (TO *)dq, dw_part);
    return hipGetLastError();
}

template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                   const float *Dl, const float *lse, const float *w, void *dq, float *dw_part,
                   hipStream_t s) {
    if (p.c_q <= 3) return launch_dq<D, 3, TO>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
    if (p.c_q <= 6) return launch_dq<D, 6, TO>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
    return launch_dq<D, 11, TO>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
}

}  // namespace

hipError_t mfma_bwd_dq_dw(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                          const void *d_o, const float *Dl, const float *lse, const float *w, void *dq,
                          float *dw_part, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
        return pick_cq<128, float>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
    return pick_cq<64, float>(p, q, k, v, d_o, Dl, lse, w, dq, dw_part, s);
}

}  // namespace convattn
