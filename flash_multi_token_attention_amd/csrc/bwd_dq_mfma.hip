// Backward of conv-attention on bf16 MFMA (gfx950): dQ and the dW partials.
//
// Workgroup = 4 waves = 128 query rows of one (batch, head); wave w owns rows
// r0 = i0 + 32w .. r0+31 and walks the keys in 64-wide tiles.  Everything a
// tile needs beyond K/V (staged once per workgroup, row-major) is private to
// the wave, so there is no barrier inside a tile.  With c0 the tile's first key:
//   S^T   rows r0-16 .. r0+47, keys c0-16 .. c0+79   raw K Q^T, pre-masked, fp16 -> LDS
//   C^T   rows r0    .. r0+47, keys c0-8  .. c0+71   Toeplitz MFMAs over the fp16 tile
//         (bands carry scale * log2 e, so C comes out in log2 units)
//   P     = exp2(C - LSE) (0 where masked); dP^T = V dO^T on the same blocks
//   dC^T  = P * (dP - D), fp16 -> LDS (rows r0 .. r0+47: own rows plus the rows
//           below them that the transposed window reaches)
//   dS^T  rows r0 .. r0+31, keys c0 .. c0+63: Toeplitz MFMAs with the flipped bands
//           (carrying scale) over dC rows shifted down by the tap, then the causal zero
//   dQ^T += K^T dS^T  (K^T fragments by LDS transpose reads of the row-major K tile;
//           dS^T straight from registers)
//   dW[a][b] += sum over own rows i and keys j' in the tile of
//           S[i+a-pq][j'] * dC[i][j'-b+pk]: an MFMA contraction with M = a, N = b and
//           the (row, 8 keys) pairs as the k index; the dC operand is read from LDS at
//           a 2-byte granular offset.  Four accumulators break the dependency chain.
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
constexpr int NCB = C_COLS / 16;       // 5 key blocks of C / dP / dC

template <int D> struct DqLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int k_bytes = S_COLS * RST;
    static constexpr int v_bytes = C_COLS * RST;
    static constexpr int wave_bytes = S_ROWS * SST + C_ROWS * CST;
    static constexpr int total = k_bytes + v_bytes + NW * wave_bytes;
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
    constexpr int K_CH = S_COLS * CPR, V_CH = C_COLS * CPR;
    constexpr int K_LD = (K_CH + NW * 64 - 1) / (NW * 64);
    constexpr int V_LD = (V_CH + NW * 64 - 1) / (NW * 64);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem;
    unsigned char *Vs = Ks + Lds::k_bytes;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    unsigned char *Ss = Vs + Lds::v_bytes + wave * Lds::wave_bytes;
    unsigned char *Cs = Ss + S_ROWS * SST;

    // x = head, y = batch, z = query tile: longest (causal) tiles of every (batch, head) first
    const int h = blockIdx.x, b = blockIdx.y;
    const int n_qt = gridDim.z, qt = n_qt - 1 - blockIdx.z;
    const int i0 = qt * BQ, r0 = i0 + wave * WR;
    const int pq = p.pq, pk = p.pk, cq = p.c_q, ck = p.c_k;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;
    const bf16_t *dOb = dO + bh * p.Nq * D;

    // forward bands carry scale*log2(e) (C in log2 units), flipped bands carry scale
    // (dS then already holds the factor dQ needs)
    f16x8 tf[CQT], tfl[CQT];
    load_bands<CQT>(tf, W + (size_t)h * cq * ck, cq, ck, pk, g, n, false, p.scale * kLog2e);
    load_bands<CQT>(tfl, W + (size_t)h * cq * ck, cq, ck, pk, g, n, true, p.scale);

    // dC is carried as fp16 times a power of two taken from D (dc_scale_log2_from_d): log2 of it comes
    // off LSE, its inverse goes onto dQ and the dW partial
    const float dcs_log2 = dc_scale_log2_from_d(Dl + bh * p.Nq, p.Nq, tid, NW * 64, reinterpret_cast<float *>(smem));
    const float dcs_inv = exp2f(-dcs_log2);
    bf16x8 qf[4][KS];   // Q rows r0-16 .. r0+47
    bf16x8 gf[3][KS];   // dO rows r0 .. r0+47
    float lse2[3], dl[3];
#pragma unroll
    for (int rb = 0; rb < 4; ++rb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qf[rb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Qb, r0 - 16 + rb * 16 + n, p.Nq, ks * 32 + g * 8));
#pragma unroll
    for (int rb = 0; rb < 3; ++rb) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            gf[rb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(dOb, r0 + rb * 16 + n, p.Nq, ks * 32 + g * 8));
        const int qpos = r0 + rb * 16 + n;
        lse2[rb] = qpos < p.Nq ? LSE[bh * p.Nq + qpos] * kLog2e - dcs_log2 : 0.f;
        dl[rb] = qpos < p.Nq ? Dl[bh * p.Nq + qpos] : 0.f;
    }

    f32x4 acc_q[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_q[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    f32x4 acc_w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc_w[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int bcl = n < ck ? n : ck - 1;  // lanes past the last key tap re-read a valid one

    // Staging registers: every thread holds its 16-byte chunks of the next K / V tile
    // (K rows c0-16 .. c0+79, V rows c0-8 .. c0+71), loaded while the current tile is computed.
    u32x4 kr[K_LD], vr[V_LD];
    auto load_tile = [&](int c0) {
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = min(tid + i * NW * 64, K_CH - 1), row = c / CPR, cc = c % CPR;
            kr[i] = load_row16_clamped<D>(Kb, c0 - 16 + row, p.Nk, cc * 8);
        }
#pragma unroll
        for (int i = 0; i < V_LD; ++i) {
            const int c = min(tid + i * NW * 64, V_CH - 1), row = c / CPR, cc = c % CPR;
            vr[i] = load_row16_clamped<D>(Vb, c0 - 8 + row, p.Nk, cc * 8);
        }
    };

    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    load_tile(0);
    for (int c0 = 0; c0 < k_end; c0 += BK) {
        __syncthreads();
        if (c0 == 0 || c0 + BK + 16 > p.Nk) {  // rows outside the sequence count as zeros
#pragma unroll
            for (int i = 0; i < K_LD; ++i) {
                const int row = c0 - 16 + (tid + i * NW * 64) / CPR;
                kr[i] = zero_unless(row >= 0 && row < p.Nk, kr[i]);
            }
#pragma unroll
            for (int i = 0; i < V_LD; ++i) {
                const int row = c0 - 8 + (tid + i * NW * 64) / CPR;
                vr[i] = zero_unless(row >= 0 && row < p.Nk, vr[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            if (c < K_CH) *reinterpret_cast<u32x4 *>(Ks + row * RST + cc * 16) = kr[i];
        }
#pragma unroll
        for (int i = 0; i < V_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            if (c < V_CH) *reinterpret_cast<u32x4 *>(Vs + row * RST + cc * 16) = vr[i];
        }
        __syncthreads();
        load_tile(c0 + BK);  // unconditional (rows are clamped into the sequence): a conditional load keeps the old registers alive
        if (causal && c0 > r0 + WR - 1) continue;
        // masks matter only where the tile can reach the diagonal or the end of the keys
        const bool edge = c0 == 0 || (causal && c0 + BK + 16 > r0 - 16) || (c0 + BK + 8 > p.Nk) ||
                          (r0 + C_ROWS > p.Nq);  // c0 == 0: the dC blocks start 8 keys before key 0

        // ---- S^T tile (raw) -> fp16 LDS; K fragments one key block ahead ----
        {
            bf16x8 kf[2][KS];
            auto load_kf = [&](int buf, int kb) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    kf[buf][ks] = *reinterpret_cast<const bf16x8 *>(Ks + (kb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
            };
            load_kf(0, 0);
            SCHED_DS_READ(KS);
#pragma unroll
            for (int kb = 0; kb < S_COLS / 16; ++kb) {
                const int cur = kb & 1;
                if (kb + 1 < S_COLS / 16) {
                    load_kf(cur ^ 1, kb + 1);
                    SCHED_DS_READ(KS);
                }
                f32x4 acc[4];
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int rb = 0; rb < 4; ++rb) acc[rb] = mfma_bf16(kf[cur][ks], qf[rb][ks], acc[rb]);
                SCHED_MFMA(4 * KS);
                const int key0 = c0 - 16 + kb * 16 + 4 * g;
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) {
                    if (edge && causal) {
                        const int qpos = r0 - 16 + rb * 16 + n;
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (key0 + r > qpos) acc[rb][r] = 0.f;
                    }
                    *reinterpret_cast<u32x2 *>(Ss + (rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) = pack_scores_f16(acc[rb]);
                }
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- per row block: C^T (5 chains over the taps), dP^T (5 chains over d), dC^T -> LDS ----
#pragma unroll
        for (int rb = 0; rb < 3; ++rb) {
            const int qpos = r0 + rb * 16 + n;
            f32x4 c[NCB], dp[NCB];
#pragma unroll
            for (int kb = 0; kb < NCB; ++kb) {
                c[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
                dp[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
            {
                // keys c0-8+16kb .. need S keys from 8 before: S-tile column 16kb
                const unsigned char *sbase = Ss + (16 + rb * 16 + n - (CQT - 1)) * SST + (8 * g) * 2;
                f16x8 sf[2][NCB];
                auto load_sf = [&](int buf, int a) {
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb)
                        sf[buf][kb] = *reinterpret_cast<const f16x8 *>(sbase + a * SST + kb * 32);
                };
                load_sf(0, 0);
                SCHED_DS_READ(NCB);
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    if (a + 1 < CQT) {
                        load_sf((a + 1) & 1, a + 1);
                        SCHED_DS_READ(NCB);
                    }
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb) c[kb] = mfma_f16(tf[a], sf[a & 1][kb], c[kb]);
                    SCHED_MFMA(NCB);
                }
            }
            {
                bf16x8 vf[2][NCB];
                auto load_vf = [&](int buf, int ks) {
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb)
                        vf[buf][kb] = *reinterpret_cast<const bf16x8 *>(Vs + (kb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
                };
                load_vf(0, 0);
                SCHED_DS_READ(NCB);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks + 1 < KS) {
                        load_vf((ks + 1) & 1, ks + 1);
                        SCHED_DS_READ(NCB);
                    }
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb) dp[kb] = mfma_bf16(vf[ks & 1][kb], gf[rb][ks], dp[kb]);
                    SCHED_MFMA(NCB);
                }
            }
#pragma unroll
            for (int kb = 0; kb < NCB; ++kb) {
                f32x4 dc;
#pragma unroll
                for (int r = 0; r < 4; ++r) dc[r] = fast_exp2(c[kb][r] - lse2[rb]) * (dp[kb][r] - dl[rb]);
                if (edge) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = c0 - 8 + kb * 16 + 4 * g + r;
                        if (key < 0 || key >= p.Nk || qpos >= p.Nq || (causal && key > qpos)) dc[r] = 0.f;
                    }
                }
                f16x4 hv;
#pragma unroll
                for (int r = 0; r < 4; ++r) hv[r] = (_Float16)__builtin_amdgcn_fmed3f(dc[r], -kF16Max, kF16Max);
                *reinterpret_cast<f16x4 *>(Cs + (rb * 16 + n) * CST + (kb * 16 + 4 * g) * 2) = hv;
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- dS^T (transposed window): 8 chains over the taps ----
        f32x4 ds[2][BK / 16];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb) ds[ob][kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        {
            constexpr int NST = 2 * CQT;  // stage = (tap slot, row block)
            f16x8 cf[2][BK / 16];
            auto load_cf = [&](int buf, int st) {
                const int a = st >> 1, ob = st & 1;
                const unsigned char *base = Cs + (ob * 16 + n + (CQT - 1) - a) * CST + (8 * g) * 2;
#pragma unroll
                for (int kb = 0; kb < BK / 16; ++kb) cf[buf][kb] = *reinterpret_cast<const f16x8 *>(base + kb * 32);
            };
            load_cf(0, 0);
            SCHED_DS_READ(BK / 16);
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (st + 1 < NST) {
                    load_cf((st + 1) & 1, st + 1);
                    SCHED_DS_READ(BK / 16);
                }
#pragma unroll
                for (int kb = 0; kb < BK / 16; ++kb)
                    ds[st & 1][kb] = mfma_f16(tfl[st >> 1], cf[st & 1][kb], ds[st & 1][kb]);
                SCHED_MFMA(BK / 16);
            }
        }
        if (edge && causal) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (c0 + kb * 16 + 4 * g + r > r0 + ob * 16 + n) ds[ob][kb][r] = 0.f;
        }
        // ---- dQ^T += K^T dS^T ----
        {
            bf16x8 sf[2][BK / 32];
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int kp = 0; kp < BK / 32; ++kp)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        sf[ob][kp][r] = (bf16_t)ds[ob][2 * kp][r];
                        sf[ob][kp][4 + r] = (bf16_t)ds[ob][2 * kp + 1][r];
                    }
            bf16x8 kf[2];
            auto load_kt = [&](int buf, int st) {  // stage = (key pair, head-dim block); own keys start at K-tile row 16
                const int kp = st / DB, db = st % DB;
                bf16x4 lo = lds_read_tr4x16(Ks, RST, 16 + kp * 32 + 4 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Ks, RST, 16 + kp * 32 + 16 + 4 * g, db * 16, n);
                kf[buf] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            };
            load_kt(0, 0);
            SCHED_DS_READ(2);
#pragma unroll
            for (int st = 0; st < (BK / 32) * DB; ++st) {
                if (st + 1 < (BK / 32) * DB) {
                    load_kt((st + 1) & 1, st + 1);
                    SCHED_DS_READ(2);
                }
                const int kp = st / DB, db = st % DB;
#pragma unroll
                for (int ob = 0; ob < 2; ++ob) acc_q[ob][db] = mfma_bf16(kf[st & 1], sf[ob][kp], acc_q[ob][db]);
                SCHED_MFMA(2);
            }
        }

        // ---- dW: rows m = tap a, columns n = tap b, contraction over (own row, 8 keys) ----
        {
            // A: S[i + a - pq][c0 + 32jb + 8g ..]   (S-tile row 16 + i + a - pq, column 16 + ...)
            // B: dC[i][c0 + 32jb + 8g - b + pk ..]  (dC-tile column 8 + ... - b + pk)
            const unsigned char *abase = Ss + (16 + n - pq) * SST + (16 + 8 * g) * 2;
            // LDS reads at odd 2-byte offsets are slow: read 5 dwords from the even
            // element below and funnel-shift by 0 or 16 bits per lane instead.
            const int boff = 8 + 8 * g - bcl + pk;
            const unsigned char *bbase = Cs + (boff & ~1) * 2;
            const unsigned int bsh = (boff & 1) * 16;
#pragma unroll 1
            for (int i = 0; i < WR; i += 2) {
                f16x8 af[4];
                u32x4 bw[4];
                unsigned int bx[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int ii = i + (u >> 1), jb = u & 1;
                    af[u] = *reinterpret_cast<const f16x8 *>(abase + ii * SST + jb * 64);
                    lds_read_dwords5(bbase + ii * CST + jb * 64, bw[u], bx[u]);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    u32x4 sh;
                    sh[0] = __builtin_amdgcn_alignbit(bw[u][1], bw[u][0], bsh);
                    sh[1] = __builtin_amdgcn_alignbit(bw[u][2], bw[u][1], bsh);
                    sh[2] = __builtin_amdgcn_alignbit(bw[u][3], bw[u][2], bsh);
                    sh[3] = __builtin_amdgcn_alignbit(bx[u], bw[u][3], bsh);
                    acc_w[u] = mfma_f16(af[u], __builtin_bit_cast(f16x8, sh), acc_w[u]);
                }
            }
        }
    }

    // ---- dQ (the flipped bands already carried the scale) ----
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
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_q[ob][db][r] * dcs_inv);
                    *reinterpret_cast<bf16x4 *>(orow + col) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(orow + col) = acc_q[ob][db] * dcs_inv;
                }
            }
        }
    }

    // ---- dW partial of this workgroup: ordered sum over the 4 waves; S was raw, so * scale ----
    __syncthreads();
    float *red = reinterpret_cast<float *>(smem);  // [NW][16][16]
#pragma unroll
    for (int r = 0; r < 4; ++r)
        red[(wave * 16 + 4 * g + r) * 16 + n] = (acc_w[0][r] + acc_w[1][r]) + (acc_w[2][r] + acc_w[3][r]);
    __syncthreads();
    const int ntap = cq * ck;
    if (tid < ntap) {
        const int a = tid / ck, bb = tid - a * ck;
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) s += red[(w * 16 + a) * 16 + bb];
        dW_part[(bh * n_qt + qt) * ntap + tid] = s * p.scale * dcs_inv;
    }
}

template <int D, int CQT, typename TO>
hipError_t launch_dq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                     const float *Dl, const float *lse, const float *w, void *dq, float *dw_part,
                     hipStream_t s) {
    auto kern = bwd_dq_mfma_kernel<D, CQT, TO>;
    constexpr int lds = DqLds<D>::total;
    hipError_t e = set_max_lds_once<bwd_dq_mfma_kernel<D, CQT, TO>>(lds);
    if (e != hipSuccess) return e;
    dim3 grid(p.H, p.B, mfma_dq_tiles(p));
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
