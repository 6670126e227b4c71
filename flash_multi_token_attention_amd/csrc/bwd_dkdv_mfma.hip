// Backward of conv-attention on bf16 MFMA (gfx950): dK and dV.
//
// Workgroup = 4 waves = 128 keys of one (batch, head); wave w owns keys
// c0 = k0 + 32w .. c0+31 for dK and, because the convolved blocks sit 8 keys
// before the window-aligned ones, keys c0-8 .. c0+23 for dV (the shifted ranges
// of neighbouring waves and workgroups tile the key axis just the same).  The
// wave keeps its K and V fragments and both accumulators in registers and walks
// the queries in 64-row tiles that the workgroup stages row-major in LDS (Q
// and dO; their transposes for the dK / dV products come from LDS transpose
// reads).  Per tile, with r0 its first row:
//   S^T  rows r0-16 .. r0+63, keys c0-16 .. c0+47    raw K Q^T, pre-masked, fp16 -> LDS
//   C    rows r0 .. r0+63, keys c0-8 .. c0+39        Toeplitz MFMAs, here oriented
//        [query][key] so that a lane holds one key and 4 query rows: that is the
//        operand layout the dV and dK products need, no transposition in between
//   P = exp2(C - LSE), dP = dO V^T, dC = P (dP - D): fp16 -> LDS (2-byte stores), below the
//        16 dC rows kept from the previous tile
//   dV^T += dO^T P        (rows r0 .. r0+63, keys c0-8 .. c0+23)
//   dS   rows r0-16 .. r0+47, keys c0 .. c0+31: flipped-band MFMAs over dC, causal zero.  dS of
//        a row needs the dC rows up to c_q-1 below it, so this product trails the tile by 16
//        rows instead of recomputing C / dP / dC for a 16-row halo below every tile; one short
//        tile after the last row finishes the last 16 rows
//   dK^T += Q^T dS        (the flipped bands carry the softmax scale)
//
// (bwd_ws_mfma.hip is the whole-backward relative of this kernel: same tiles, two waves per SIMD.)
#include <type_traits>

#include "mfma_common.hpp"

#ifndef CONVATTN_DKDV_UNIT
#define CONVATTN_DKDV_UNIT 0
#endif

namespace convattn {
namespace {

constexpr int NW = 4;
constexpr int WK = 32;                 // own keys per wave
constexpr int BKW = NW * WK;           // 128 keys per workgroup
constexpr int BR = 64;                 // query rows per tile
constexpr int HT = 16;                 // rows staged above a tile's own rows (>= c_q - 1)
constexpr int S_ROWS = BR + HT;        // 80 score rows: r0-16 .. r0+63
constexpr int S_COLS = WK + 32;        // 64
constexpr int C_ROWS = BR + HT;        // 80 dC rows: 16 carried over from the previous tile + 64 new
constexpr int C_COLS = WK + 16;        // 48
constexpr int SST = (S_COLS + 8) * 2;  // 144
constexpr int CST = (C_COLS + 8) * 2;  // 112
constexpr int NSB = S_COLS / 16;       // 4 key blocks of S
constexpr int NCB = C_COLS / 16;       // 3 key blocks of C / dP / dC
constexpr int NRB = BR / 16;           // 4 own row blocks per tile
static_assert(BKW == kKvKeysPerWg, "grid size");

template <int D, int CQT> struct KvLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int q_bytes = S_ROWS * RST;
    static constexpr int g_bytes = BR * RST;
    static constexpr int stat_bytes = 2 * BR * 4;
    static constexpr int wave_bytes = S_ROWS * SST + C_ROWS * CST;
    static constexpr int total = q_bytes + g_bytes + stat_bytes + NW * wave_bytes;
};

template <int D, int CQT, typename TO>
__global__ __launch_bounds__(NW * 64) void bwd_dkdv_mfma_kernel(
    Problem p, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const bf16_t *__restrict__ dO, const float *__restrict__ Dl,
    const float *__restrict__ LSE, const float *__restrict__ W, TO *__restrict__ dK,
    TO *__restrict__ dV) {
    using Lds = KvLds<D, CQT>;
    constexpr int RST = Lds::RST;
    constexpr int KS = D / 32, DB = D / 16, CPR = D / 8;
    constexpr int Q_CH = S_ROWS * CPR, G_CH = BR * CPR;
    constexpr int Q_LD = (Q_CH + NW * 64 - 1) / (NW * 64);
    constexpr int G_LD = (G_CH + NW * 64 - 1) / (NW * 64);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Qs = smem;
    unsigned char *Gs = Qs + Lds::q_bytes;
    float *lse_s = reinterpret_cast<float *>(Gs + Lds::g_bytes);
    float *dl_s = lse_s + BR;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    unsigned char *Ss = Gs + Lds::g_bytes + Lds::stat_bytes + wave * Lds::wave_bytes;
    unsigned char *Cs = Ss + S_ROWS * SST;

    // x = head, y = batch, z = key tile: the first key tiles see the most rows and go first
    const int h = blockIdx.x, b = blockIdx.y;
    const int k0 = blockIdx.z * BKW, c0 = k0 + wave * WK;
    const int pk = p.pk, cq = p.c_q, ck = p.c_k;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;
    const bf16_t *dOb = dO + bh * p.Nq * D;
    const float *lse_b = LSE + bh * p.Nq;
    const float *dl_b = Dl + bh * p.Nq;

    // dC is carried as fp16 times a power of two taken from D (dc_scale_log2_from_d): log2 of it comes
    // off the staged LSE, its inverse goes onto dK and dV
    const float dcs_log2 = dc_scale_log2_from_d(dl_b, p.Nq, tid, NW * 64, reinterpret_cast<float *>(smem));
    const float dcs_inv = exp2f(-dcs_log2);

    f16x8 tf[CQT], tfl[CQT];
    load_bands<CQT>(tf, W + (size_t)h * cq * ck, cq, ck, pk, g, n, false, p.scale * kLog2e);
    load_bands<CQT>(tfl, W + (size_t)h * cq * ck, cq, ck, pk, g, n, true, p.scale);

    bf16x8 kf[NSB][KS];  // K rows c0-16 .. c0+47
    bf16x8 vf[NCB][KS];  // V rows c0-8 .. c0+39
#pragma unroll
    for (int kb = 0; kb < NSB; ++kb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            kf[kb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Kb, c0 - 16 + kb * 16 + n, p.Nk, ks * 32 + g * 8));
#pragma unroll
    for (int kb = 0; kb < NCB; ++kb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            vf[kb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Vb, c0 - 8 + kb * 16 + n, p.Nk, ks * 32 + g * 8));

    f32x4 acc_k[2][DB], acc_v[2][DB];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            acc_k[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
            acc_v[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }

    // Causal: rows before the first key this workgroup touches (k0 - 8) see none of its keys.
    const int r_begin = causal ? (max(0, k0 - 8) / BR) * BR : 0;
    // dS / dK of a row need the dC rows below it, so they trail the tiles by 16 rows: one more
    // (short) tile when the last 16 rows of the sequence are not covered otherwise.
    const int r_end = p.Nq + HT;
    for (int c = lane; c < HT * (CST / 16); c += 64)  // no dC before the first tile
        *reinterpret_cast<u32x4 *>(Cs + (c / (CST / 16)) * CST + (c % (CST / 16)) * 16) = (u32x4){0u, 0u, 0u, 0u};
    // Staging registers: this thread's 16-byte chunks of the next Q / dO tile and its LSE / D entry.
    u32x4 qr[Q_LD], gr[G_LD];
    float ls = 0.f, dd = 0.f;
    auto load_tile = [&](int r0) {
#pragma unroll
        for (int i = 0; i < Q_LD; ++i) {
            const int c = min(tid + i * NW * 64, Q_CH - 1), row = c / CPR, cc = c % CPR;
            qr[i] = load_row16_clamped<D>(Qb, r0 - HT + row, p.Nq, cc * 8);
        }
#pragma unroll
        for (int i = 0; i < G_LD; ++i) {
            const int c = min(tid + i * NW * 64, G_CH - 1), row = c / CPR, cc = c % CPR;
            gr[i] = load_row16_clamped<D>(dOb, r0 + row, p.Nq, cc * 8);
        }
        ls = 1e30f; dd = 0.f;  // rows past the end: exp2(C - LSE) = 0
        if (tid < BR && r0 + tid < p.Nq) { ls = lse_b[r0 + tid] * kLog2e - dcs_log2; dd = dl_b[r0 + tid]; }
    };
    load_tile(r_begin);
    // One row tile.  EDGE tiles apply the causal / sequence-end masks; the others are far enough
    // from the diagonal and from both ends of the key axis to need none (rows past the end of the
    // sequence are dealt with by the staged values: zero Q / dO rows and a huge LSE give P = dC = 0).
    auto tile = [&](const int r0, auto edge_tag) {
        constexpr bool EDGE = decltype(edge_tag)::value;
        __syncthreads();
        if (r0 == 0 || r0 + BR > p.Nq) {  // rows outside the sequence count as zeros
#pragma unroll
            for (int i = 0; i < Q_LD; ++i) {
                const int row = r0 - HT + (tid + i * NW * 64) / CPR;
                qr[i] = zero_unless(row >= 0 && row < p.Nq, qr[i]);
            }
#pragma unroll
            for (int i = 0; i < G_LD; ++i) gr[i] = zero_unless(r0 + (tid + i * NW * 64) / CPR < p.Nq, gr[i]);
        }
#pragma unroll
        for (int i = 0; i < Q_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            if (c < Q_CH) *reinterpret_cast<u32x4 *>(Qs + row * RST + cc * 16) = qr[i];
        }
#pragma unroll
        for (int i = 0; i < G_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            if (c < G_CH) *reinterpret_cast<u32x4 *>(Gs + row * RST + cc * 16) = gr[i];
        }
        if (tid < BR) { lse_s[tid] = ls; dl_s[tid] = dd; }
        __syncthreads();
        load_tile(r0 + BR);  // unconditional (rows are clamped into the sequence): a conditional load keeps the old registers alive
        if (causal && r0 + BR - 1 < c0 - 8) return;  // none of the tile's rows sees the wave's keys (only on masked tiles)
        // Past the last row only the dS / dK work of the 16 carried rows is left.
        const bool tail = EDGE && r0 >= p.Nq;
        f32x4 pkeep[NRB][2];
        if (tail) {
            // the tile has no dC rows of its own: zeros below the carried ones
            for (int c = lane; c < 16 * (CST / 16); c += 64)
                *reinterpret_cast<u32x4 *>(Cs + (HT + c / (CST / 16)) * CST + (c % (CST / 16)) * 16) = (u32x4){0u, 0u, 0u, 0u};
        } else {

        // ---- S^T tile (raw) -> fp16 LDS; Q fragments one row block ahead.  (Taking the first 16 rows
        // over from the previous tile instead of recomputing them was measured: no gain.) ----
        {
            bf16x8 qf[2][KS];
            auto load_qf = [&](int buf, int rb) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    qf[buf][ks] = *reinterpret_cast<const bf16x8 *>(Qs + (rb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
            };
            load_qf(0, 0);
            SCHED_DS_READ_ID(KS, 10);
            static_for<S_ROWS / 16>([&](auto rb_c) {
                constexpr int rb = decltype(rb_c)::value;
                constexpr int cur = rb & 1;
                if constexpr (rb + 1 < S_ROWS / 16) {
                    load_qf(cur ^ 1, rb + 1);
                    SCHED_DS_READ_ID(KS, 11 + rb);
                }
                f32x4 acc[NSB];
#pragma unroll
                for (int kb = 0; kb < NSB; ++kb) acc[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int kb = 0; kb < NSB; ++kb) acc[kb] = mfma_bf16(kf[kb][ks], qf[cur][ks], acc[kb]);
                SCHED_MFMA_ID(NSB * KS, 10 + rb);
                const int qpos = r0 - HT + rb * 16 + n;
#pragma unroll
                for (int kb = 0; kb < NSB; ++kb) {
                    if (EDGE && causal) {
                        const int key0 = c0 - 16 + kb * 16 + 4 * g;
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (key0 + r > qpos) acc[kb][r] = 0.f;
                    }
                    *reinterpret_cast<u32x2 *>(Ss + (rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) = pack_scores_f16(acc[kb]);
                }
            });
        }
        __builtin_amdgcn_wave_barrier();

        // ---- C, P, dP, dC ([query][key] orientation: lane = key, registers = 4 rows) ----
        static_for<NRB>([&](auto rb_c) {
            constexpr int rb = decltype(rb_c)::value;
            constexpr int SID = 20 + rb;  // scheduling pipeline of this row block
            const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(lse_s + rb * 16 + 4 * g);
            const f32x4 dl4 = *reinterpret_cast<const f32x4 *>(dl_s + rb * 16 + 4 * g);
            SCHED_DS_READ_ID(2, SID);
            f32x4 c[NCB], dp[NCB];
#pragma unroll
            for (int kb = 0; kb < NCB; ++kb) {
                c[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
                dp[kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
            {
                const unsigned char *sbase = Ss + (HT + rb * 16 + n - (CQT - 1)) * SST + (8 * g) * 2;
                f16x8 sf[2][NCB];
                auto load_sf = [&](int buf, int a) {
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb)
                        sf[buf][kb] = *reinterpret_cast<const f16x8 *>(sbase + a * SST + kb * 32);
                };
                load_sf(0, 0);
                SCHED_DS_READ_ID(NCB, SID);
#pragma unroll
                for (int a = 0; a < CQT; ++a) {
                    if (a + 1 < CQT) {
                        load_sf((a + 1) & 1, a + 1);
                        SCHED_DS_READ_ID(NCB, SID);
                    }
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb) c[kb] = mfma_f16(sf[a & 1][kb], tf[a], c[kb]);
                    SCHED_MFMA_ID(NCB, SID);
                }
            }
            {
                bf16x8 gf[2];
                auto load_gf = [&](int buf, int ks) {
                    gf[buf] = *reinterpret_cast<const bf16x8 *>(Gs + (rb * 16 + n) * RST + (ks * 32 + g * 8) * 2);
                };
                load_gf(0, 0);
                SCHED_DS_READ_ID(1, SID);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks + 1 < KS) {
                        load_gf((ks + 1) & 1, ks + 1);
                        SCHED_DS_READ_ID(1, SID);
                    }
#pragma unroll
                    for (int kb = 0; kb < NCB; ++kb) dp[kb] = mfma_bf16(gf[ks & 1], vf[kb][ks], dp[kb]);
                    SCHED_MFMA_ID(NCB, SID);
                }
            }
#pragma unroll
            for (int kb = 0; kb < NCB; ++kb) {
                f32x4 pr, dc;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pr[r] = fast_exp2(c[kb][r] - lse4[r]);
                    dc[r] = pr[r] * (dp[kb][r] - dl4[r]);
                }
                if constexpr (EDGE) {
                    const int key = c0 - 8 + kb * 16 + n;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int qpos = r0 + rb * 16 + 4 * g + r;
                        if (key < 0 || key >= p.Nk || qpos >= p.Nq || (causal && key > qpos)) { pr[r] = 0.f; dc[r] = 0.f; }
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    *reinterpret_cast<_Float16 *>(Cs + (HT + rb * 16 + 4 * g + r) * CST + (kb * 16 + n) * 2) =
                        (_Float16)__builtin_amdgcn_fmed3f(dc[r], -kF16Max, kF16Max);
                if (kb < 2) pkeep[rb][kb] = pr;
            }
        });
        __builtin_amdgcn_wave_barrier();

        // ---- dV^T += dO^T P  (keys c0-8 .. c0+23); dO^T by transpose reads of the dO tile ----
        {
            bf16x8 pf[NRB / 2][2];
#pragma unroll
            for (int kp = 0; kp < NRB / 2; ++kp)
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        pf[kp][kb][r] = (bf16_t)pkeep[2 * kp][kb][r];
                        pf[kp][kb][4 + r] = (bf16_t)pkeep[2 * kp + 1][kb][r];
                    }
            constexpr int NST = (NRB / 2) * DB;  // stage = (row pair, head-dim block)
            bf16x8 gt[2];
            auto load_gt = [&](int buf, int st) {
                const int kp = st / DB, db = st % DB;
                bf16x4 lo = lds_read_tr4x16(Gs, RST, kp * 32 + 4 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Gs, RST, kp * 32 + 16 + 4 * g, db * 16, n);
                gt[buf] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            };
            load_gt(0, 0);
            SCHED_DS_READ_ID(2, 30);
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (st + 1 < NST) {
                    load_gt((st + 1) & 1, st + 1);
                    SCHED_DS_READ_ID(2, 30);
                }
                const int kp = st / DB, db = st % DB;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) acc_v[kb][db] = mfma_bf16(gt[st & 1], pf[kp][kb], acc_v[kb][db]);
                SCHED_MFMA_ID(2, 30);
            }
        }
        }  // !tail
        __builtin_amdgcn_wave_barrier();

        // ---- dS, rows r0-16 .. r0+47 (keys c0 .. c0+31): 4 chains over the taps.  The rows are the
        // ones whose window (c_q - 1 rows down) is complete with this tile's dC; the dC tile starts
        // at row r0-16 with the 16 rows carried over from the previous tile. ----
        f32x4 ds[NRB][2];
#pragma unroll
        for (int ob = 0; ob < NRB; ++ob)
#pragma unroll
            for (int m = 0; m < 2; ++m) ds[ob][m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        {
            constexpr int NST = NRB * CQT;  // stage = (tap slot, row block)
            f16x8 cf[2][2];
            auto load_cf = [&](int buf, int st) {
                const int a = st / NRB, ob = st % NRB;
                const unsigned char *base = Cs + (ob * 16 + n + (CQT - 1) - a) * CST + (8 * g) * 2;
                cf[buf][0] = *reinterpret_cast<const f16x8 *>(base);
                cf[buf][1] = *reinterpret_cast<const f16x8 *>(base + 32);
            };
            load_cf(0, 0);
            SCHED_DS_READ_ID(2, 31);
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (st + 1 < NST) {
                    load_cf((st + 1) & 1, st + 1);
                    SCHED_DS_READ_ID(2, 31);
                }
#pragma unroll
                for (int m = 0; m < 2; ++m) ds[st % NRB][m] = mfma_f16(cf[st & 1][m], tfl[st / NRB], ds[st % NRB][m]);
                SCHED_MFMA_ID(2, 31);
            }
        }
        if (EDGE && causal) {
#pragma unroll
            for (int ob = 0; ob < NRB; ++ob)
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (c0 + m * 16 + n > r0 - HT + ob * 16 + 4 * g + r) ds[ob][m][r] = 0.f;
        }
        // ---- dK^T += Q^T dS; Q^T by transpose reads (the Q tile starts at row r0-16 as well) ----
        {
            bf16x8 sf[NRB / 2][2];
#pragma unroll
            for (int kp = 0; kp < NRB / 2; ++kp)
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        sf[kp][m][r] = (bf16_t)ds[2 * kp][m][r];
                        sf[kp][m][4 + r] = (bf16_t)ds[2 * kp + 1][m][r];
                    }
            constexpr int NST = (NRB / 2) * DB;
            bf16x8 qt[2];
            auto load_qt = [&](int buf, int st) {
                const int kp = st / DB, db = st % DB;
                bf16x4 lo = lds_read_tr4x16(Qs, RST, kp * 32 + 4 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Qs, RST, 16 + kp * 32 + 4 * g, db * 16, n);
                qt[buf] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            };
            load_qt(0, 0);
            SCHED_DS_READ_ID(2, 32);
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (st + 1 < NST) {
                    load_qt((st + 1) & 1, st + 1);
                    SCHED_DS_READ_ID(2, 32);
                }
                const int kp = st / DB, db = st % DB;
#pragma unroll
                for (int m = 0; m < 2; ++m) acc_k[m][db] = mfma_bf16(qt[st & 1], sf[kp][m], acc_k[m][db]);
                SCHED_MFMA_ID(2, 32);
            }
        }

        // ---- the last 16 dC rows become the first 16 of the next tile ----
        __builtin_amdgcn_wave_barrier();
        for (int c = lane; c < HT * (CST / 16); c += 64) {
            const int off = (c / (CST / 16)) * CST + (c % (CST / 16)) * 16;
            *reinterpret_cast<u32x4 *>(Cs + off) = *reinterpret_cast<const u32x4 *>(Cs + BR * CST + off);
        }
        __builtin_amdgcn_wave_barrier();
    };
    // keys before 0 or past the end in reach: every tile masks; else only the tiles near the diagonal
    // and the last, partial ones
    const bool always_edge = c0 == 0 || c0 + 40 > p.Nk;
    int r0 = r_begin;
    for (; r0 < r_end && (always_edge || r0 == 0 || (causal && r0 < c0 + 64)); r0 += BR) tile(r0, std::true_type{});
    for (; r0 + BR <= p.Nq; r0 += BR) tile(r0, std::false_type{});
    for (; r0 < r_end; r0 += BR) tile(r0, std::true_type{});

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
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_k[m][db][r] * dcs_inv);
                    *reinterpret_cast<bf16x4 *>(dst) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(dst) = acc_k[m][db] * dcs_inv;
                }
            }
            if (key_v >= 0 && key_v < p.Nk) {
                TO *dst = dV + (bh * p.Nk + key_v) * D + col;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_v[m][db][r] * dcs_inv);
                    *reinterpret_cast<bf16x4 *>(dst) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(dst) = acc_v[m][db] * dcs_inv;
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
    constexpr int lds = KvLds<D, CQT>::total;
    hipError_t e = set_max_lds_once<bwd_dkdv_mfma_kernel<D, CQT, TO>>(lds);
    if (e != hipSuccess) return e;
    dim3 grid(p.H, p.B, mfma_kv_tiles(p));
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v,
                                    (const bf16_t *)d_o, Dl, lse, w, (TO *)dk, (TO *)dv);
    return hipGetLastError();
}

}  // namespace

// This file is built as two objects so that they compile in parallel: CONVATTN_DKDV_UNIT = 1
// holds the 11-tap-slot instantiations (the slowest), 0 the others and the entry point.
template <int D, typename TO>
hipError_t dkdv_wide(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                     const float *Dl, const float *lse, const float *w, void *dk, void *dv,
                     hipStream_t s);

#if CONVATTN_DKDV_UNIT == 1
template <int D, typename TO>
hipError_t dkdv_wide(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                     const float *Dl, const float *lse, const float *w, void *dk, void *dv,
                     hipStream_t s) {
    return launch_kv<D, 11, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
}
#define CONVATTN_INST(D, TO)                                                                          \
    template hipError_t dkdv_wide<D, TO>(const Problem &, const void *, const void *, const void *,   \
                                         const void *, const float *, const float *, const float *,   \
                                         void *, void *, hipStream_t);
CONVATTN_INST(128, bf16_t) CONVATTN_INST(128, float) CONVATTN_INST(64, bf16_t) CONVATTN_INST(64, float)
#undef CONVATTN_INST
#else
namespace {
template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                   const float *Dl, const float *lse, const float *w, void *dk, void *dv,
                   hipStream_t s) {
    if (p.c_q <= 3) return launch_kv<D, 3, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
    if (p.c_q <= 6) return launch_kv<D, 6, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
    return dkdv_wide<D, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, s);
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
#endif

}  // namespace convattn
