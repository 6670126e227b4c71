// Whole backward of conv-attention on bf16 MFMA (gfx950), two waves per SIMD.
//
// Same mathematics, tiles and workspace layout as the whole-backward variant of
// bwd_dkdv_mfma.hip (dK, dV, dW partials and the bf16 dS blocks that bwd_dq_gemm.hip turns into
// dQ), reorganised so that two waves share a SIMD: an MFMA occupies its wave's issue slot for
// the whole instruction, so a wave alone on a SIMD cannot overlap its MFMAs with its own VALU or
// LDS work, and the one-wave kernel needs all 512 registers.  Here a workgroup is 8 waves = 4
// pairs; pair p owns keys c0 = k0 + 32p .. c0+31 (dV: c0-8 .. c0+23), and the work of a
// 32-row tile is split between the two waves of the pair:
//   producer (even waves): keeps the K / V fragments; S^T = K Q^T (rows r0-16 .. r0+31) -> LDS,
//       C by Toeplitz MFMAs, P = exp2(C - LSE), dP = dO V^T, dC = P (dP - D) -> LDS, P -> LDS
//   consumer (odd waves):  keeps the dK / dV / dW accumulators; one tile behind the producer:
//       dV^T += dO^T P, dS (rows r0-16 .. r0+15, flipped-band MFMAs over dC) -> workspace,
//       dK^T += Q^T dS, dW += S (x) dC
// One workgroup barrier per tile.  In iteration `it` every thread stages tile it+1 (Q, dO, LSE, D:
// global loads issued an iteration earlier), the producers work on tile it and the consumers on
// tile it-1, so three tiles are alive in LDS: Q sits in a ring of seven 16-row blocks (the 16 rows
// above a tile are the previous tile's, never loaded twice), dO in three tile slots, S in a ring of
// five 16-row blocks and dC in a ring of three 32-row slots per pair (a tile's 48-row window = its
// own rows + the last 16 of the previous tile, never copied or recomputed), P in two buffers.  Both
// roles run the same number of iterations.  dS / dK trail their tile by 16 rows (they need the dC
// rows below).
#include <type_traits>

#include "mfma_common.hpp"

namespace convattn {
namespace {

constexpr int NP = 4;                  // wave pairs = key ranges per workgroup
constexpr int NT = 2 * NP * 64;        // 512 threads
constexpr int WK = 32;                 // own keys per pair
constexpr int BKW = NP * WK;           // 128 keys per workgroup
constexpr int BR = 32;                 // query rows per tile
constexpr int HT = 16;                 // rows staged above a tile's own rows (>= c_q - 1)
constexpr int S_ROWS = BR + HT;        // 48 score rows in a tile's window: r0-16 .. r0+31

constexpr int S_COLS = WK + 32;        // 64
constexpr int C_COLS = WK + 16;        // 48
constexpr int SST = (S_COLS + 8) * 2;  // 144
constexpr int CST = (C_COLS + 8) * 2;  // 112
constexpr int NSB = S_COLS / 16;       // 4 key blocks of S
constexpr int NCB = C_COLS / 16;       // 3 key blocks of C / dP / dC
constexpr int NRB = BR / 16;           // 2 own row blocks per tile
constexpr int P_BYTES = 2 * 64 * 16;   // P of a tile as two MFMA operands per lane
constexpr int C_RING = 3 * BR;         // dC ring of a pair: three tiles of 32 rows
constexpr int S_RING = 5 * 16;         // S ring of a pair: five blocks of 16 rows
constexpr int Q_BLOCKS = 7;            // Q ring of the workgroup: seven blocks of 16 rows
static_assert(BKW == kKvKeysPerWg && WK == kDsKeys && kDsRows == 2 * BR && kDsRowShift == HT, "dS workspace layout");

template <int D> struct WsLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int q_bytes = Q_BLOCKS * 16 * RST;        // Q ring
    static constexpr int g_bytes = 3 * BR * RST;               // dO: three tile slots
    static constexpr int stat_bytes = 2 * (2 * BR * 4);        // LSE and D of a tile: two slots
    static constexpr int stage_bytes = q_bytes + g_bytes + stat_bytes;
    static constexpr int pair_bytes = S_RING * SST + C_RING * CST + 2 * P_BYTES;
    static constexpr int total = stage_bytes + NP * pair_bytes;
};

template <int D, int CQT, typename TO>
__global__ __launch_bounds__(NT) void bwd_ws_mfma_kernel(
    Problem p, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const bf16_t *__restrict__ dO, const float *__restrict__ Dl,
    const float *__restrict__ LSE, const float *__restrict__ W, TO *__restrict__ dK,
    TO *__restrict__ dV, bf16_t *__restrict__ dS_ws, float *__restrict__ dW_part) {
    using Lds = WsLds<D>;
    constexpr int RST = Lds::RST;
    constexpr int KS = D / 32, DB = D / 16, CPR = D / 8;
    constexpr int Q_CH = BR * CPR, G_CH = BR * CPR;
    constexpr int Q_LD = (Q_CH + NT - 1) / NT, G_LD = (G_CH + NT - 1) / NT;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    const bool producer = (wave & 1) == 0;   // (measured: this assignment beats waves 0-3 / 4-7)
    const int pr = wave >> 1;
    // Rows are numbered in blocks of 16 from row r_begin - 16: tile t owns blocks 2t+1 and 2t+2, and
    // its 48-row window (the 16 rows above it included) is blocks 2t .. 2t+2.  In iteration `it` the
    // workgroup stages tile it+1, the producers work on tile it and the consumers on tile it-1, so
    // blocks 2it-2 .. 2it+4 of Q (seven), tiles it-1 .. it+1 of dO (three) and blocks 2it-2 .. 2it+2
    // of S (five) are alive between two barriers; dC, which the consumer reads as rows of tile it-1
    // and the half tile above it, has a ring of three tile slots.
    auto q_block = [&](int blk) { return smem + (blk % Q_BLOCKS) * (16 * RST); };
    auto stage_g = [&](int t) { return smem + Lds::q_bytes + (t % 3) * (BR * RST); };
    auto stage_lse = [&](int t) {
        return reinterpret_cast<float *>(smem + Lds::q_bytes + Lds::g_bytes + (t & 1) * (2 * BR * 4));
    };
    unsigned char *pair_base = smem + Lds::stage_bytes + pr * Lds::pair_bytes;
    unsigned char *s_ring = pair_base;
    unsigned char *c_ring = pair_base + S_RING * SST;
    // S: ring row of window row rho of tile t is (32 t + rho) mod 80; with base = 32 t mod 80 and
    // rho < 80 that is the unsigned minimum of base + rho and base + rho - 80.
    auto s_base = [](int t) { return (t % 5) * 32 % S_RING; };
    auto s_row = [](int base, int rho) { return (int)min((unsigned)(base + rho), (unsigned)(base + rho - S_RING)); };
    // dC: row rho of a tile's window is ring row (rho < 16 ? ring_hb(t) : ring_tb(t)) + rho; the two
    // bases differ only when the window wraps around the ring.
    auto ring_tb = [](int t) { return (t % 3) * BR - HT; };
    auto ring_hb = [](int t) { return ((t + 2) % 3) * BR + HT; };
    auto pair_p = [&](int buf) { return pair_base + S_RING * SST + C_RING * CST + buf * P_BYTES; };

    // x = head, y = batch, z = key tile: the first key tiles see the most rows and go first
    const int h = blockIdx.x, b = blockIdx.y;
    const int k0 = blockIdx.z * BKW, c0 = k0 + pr * WK;
    const int pk = p.pk, cq = p.c_q, ck = p.c_k;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *dOb = dO + bh * p.Nq * D;
    const float *lse_b = LSE + bh * p.Nq;
    const float *dl_b = Dl + bh * p.Nq;

    // dC is carried as fp16 times a power of two taken from D (dc_scale_log2_from_d): log2 of it comes
    // off the staged LSE, its inverse goes onto dK, dV, the dW partial and (in the dQ product) dQ
    const float dcs_log2 = dc_scale_log2_from_d(dl_b, p.Nq, tid, NT, reinterpret_cast<float *>(smem));
    const float dcs_inv = exp2f(-dcs_log2);

    // no dC before the first tile, and nothing but zeros where a tile was skipped
    for (int c = tid; c < NP * Lds::pair_bytes / 16; c += NT)
        *reinterpret_cast<u32x4 *>(smem + Lds::stage_bytes + c * 16) = (u32x4){0u, 0u, 0u, 0u};

    // Causal: rows before the first key this workgroup touches (k0 - 8) see none of its keys.
    const int r_begin = causal ? (max(0, k0 - 8) / BR) * BR : 0;
    // dS / dK trail the tiles by 16 rows: tiles run until row Nq + 16, and the consumer runs one
    // iteration behind the producer.
    const int n_tiles = (p.Nq + HT - r_begin + BR - 1) / BR;
    // masks are needed next to the diagonal, at both ends of the key axis and past the last row
    const bool always_edge = c0 == 0 || c0 + 40 > p.Nk;
    auto is_edge = [&](int r0) { return always_edge || r0 == 0 || (causal && r0 < c0 + 64) || r0 + BR > p.Nq; };
    auto is_skipped = [&](int r0) { return causal && r0 + BR - 1 < c0 - 8; };

    // Staging registers: this thread's 16-byte chunks of the next Q / dO tile and its LSE / D entry.
    u32x4 qr[Q_LD], gr[G_LD];
    float ls = 0.f, dd = 0.f;
    // Buffer loads: rows before the first or after the last query row are outside the descriptor's
    // range and read as zeros, which is what the window's zero padding and the tail tile ask for.
    const __amdgpu_buffer_rsrc_t q_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)Qb, 0, p.Nq * D * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t g_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)dOb, 0, p.Nq * D * 2, 0x00020000);
    auto load_tile = [&](int r0) {
#pragma unroll
        for (int i = 0; i < Q_LD; ++i) {
            const int c = min(tid + i * NT, Q_CH - 1), row = c / CPR, cc = c % CPR;
            qr[i] = __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, ((r0 + row) * D + cc * 8) * 2, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < G_LD; ++i) {
            const int c = min(tid + i * NT, G_CH - 1), row = c / CPR, cc = c % CPR;
            gr[i] = __builtin_amdgcn_raw_buffer_load_b128(g_rsrc, ((r0 + row) * D + cc * 8) * 2, 0, 0);
        }
        ls = 1e30f; dd = 0.f;  // rows past the end: exp2(C - LSE) = 0
        if (tid < BR && r0 + tid < p.Nq) { ls = lse_b[r0 + tid] * kLog2e - dcs_log2; dd = dl_b[r0 + tid]; }
    };
    // Both roles: the registers of tile t into its Q blocks, dO slot and LSE / D slot.
    auto stage_tile = [&](int t) {
        unsigned char *Q1 = q_block(2 * t + 1), *Q2 = q_block(2 * t + 2), *Gs = stage_g(t);
        float *lse_s = stage_lse(t);
#pragma unroll
        for (int i = 0; i < Q_LD; ++i) {
            const int c = tid + i * NT, row = c / CPR, cc = c % CPR;
            if (c < Q_CH) *reinterpret_cast<u32x4 *>((row < 16 ? Q1 : Q2) + (row & 15) * RST + cc * 16) = qr[i];
        }
#pragma unroll
        for (int i = 0; i < G_LD; ++i) {
            const int c = tid + i * NT, row = c / CPR, cc = c % CPR;
            if (c < G_CH) *reinterpret_cast<u32x4 *>(Gs + row * RST + cc * 16) = gr[i];
        }
        if (tid < BR) { lse_s[tid] = ls; lse_s[BR + tid] = dd; }
    };

    // Q rows r_begin-16 .. r_begin-1 (block 0), then tile 0; tile 1 waits in the registers
    for (int c = tid; c < 16 * CPR; c += NT) {
        const int row = c / CPR, cc = c % CPR;
        *reinterpret_cast<u32x4 *>(q_block(0) + row * RST + cc * 16) =
            __builtin_amdgcn_raw_buffer_load_b128(q_rsrc, ((r_begin - HT + row) * D + cc * 8) * 2, 0, 0);
    }
    load_tile(r_begin);
    stage_tile(0);
    load_tile(r_begin + BR);
    // One barrier per iteration: it makes tile `it` (staged in the previous iteration) and the
    // previous tile's S / dC / P visible, and frees what iteration it-1 read.  The first one also
    // covers the zero-filled pair buffers.

    if (producer) {
        // ================================ producer ================================
        const bf16_t *Kb = K + bh * p.Nk * D;
        const bf16_t *Vb = V + bh * p.Nk * D;
        f16x8 tf[CQT];
        load_bands<CQT>(tf, W + (size_t)h * cq * ck, cq, ck, pk, g, n, false, p.scale * kLog2e);
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

        for (int it = 0; it <= n_tiles; ++it) {
            const int r0 = r_begin + it * BR;
            __syncthreads();
            if (it + 1 < n_tiles) stage_tile(it + 1);
            load_tile(r0 + 2 * BR);  // unconditional: rows past the end read as zeros, and a conditional
                                     // load would keep the previous tile's registers alive through the tile
            if (it == n_tiles || is_skipped(r0)) continue;
            // the tile body exists twice: with the masks (tiles on the diagonal or at an end of a
            // sequence) and without, as straight-line code
            auto ptile = [&](auto edge_tag) {
            constexpr bool edge = decltype(edge_tag)::value;
            const unsigned char *Gs = stage_g(it);
            const float *lse_s = stage_lse(it), *dl_s = lse_s + BR;
            unsigned char *Ps = pair_p(it & 1);
            const int tb = ring_tb(it), sb = s_base(it);

            // a wave in an MFMA phase gets the issue slot before the SIMD's other wave (which is in
            // the same role, somewhere else in its tile); element-wise phases run at priority 0
            __builtin_amdgcn_s_setprio(1);
            // ---- S^T tile (raw) -> fp16 LDS; Q fragments one row block ahead.  The first 16 rows
            // are the last 16 of the previous tile (masks depend on positions only): taken over from
            // the other buffer when that tile was computed. ----
            {
                const bool carry_s = it > 0 && !is_skipped(r0 - BR);
                bf16x8 qf[2][KS];
                auto load_qf = [&](int buf, int rb) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        qf[buf][ks] = *reinterpret_cast<const bf16x8 *>(q_block(2 * it + rb) + n * RST + (ks * 32 + g * 8) * 2);
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
                    if (rb == 0 && carry_s) return;
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
                        if (edge && causal) {
                            const int key0 = c0 - 16 + kb * 16 + 4 * g;
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                if (key0 + r > qpos) acc[kb][r] = 0.f;
                        }
                        *reinterpret_cast<u32x2 *>(s_ring + s_row(sb, rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) =
                            pack_scores_f16(acc[kb]);
                    }
                });
            }
            __builtin_amdgcn_wave_barrier();

            // ---- C, P, dP, dC ([query][key] orientation: lane = key, registers = 4 rows) ----
            f32x4 pkeep[NRB][2];
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
                    // tap a reads window row HT + rb*16 + n - (CQT-1) + a
                    const int srow = HT + rb * 16 + n - (CQT - 1);
                    f16x8 sf[2][NCB];
                    auto load_sf = [&](int buf, int a) {
                        const unsigned char *base = s_ring + s_row(sb, srow + a) * SST + (8 * g) * 2;
#pragma unroll
                        for (int kb = 0; kb < NCB; ++kb)
                            sf[buf][kb] = *reinterpret_cast<const f16x8 *>(base + kb * 32);
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
                __builtin_amdgcn_s_setprio(0);
#pragma unroll
                for (int kb = 0; kb < NCB; ++kb) {
                    f32x4 prob, dc;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        prob[r] = fast_exp2(c[kb][r] - lse4[r]);
                        dc[r] = prob[r] * (dp[kb][r] - dl4[r]);
                    }
                    if (edge) {
                        const int key = c0 - 8 + kb * 16 + n;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int qpos = r0 + rb * 16 + 4 * g + r;
                            if (key < 0 || key >= p.Nk || qpos >= p.Nq || (causal && key > qpos)) { prob[r] = 0.f; dc[r] = 0.f; }
                        }
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        *reinterpret_cast<_Float16 *>(c_ring + (tb + HT + rb * 16 + 4 * g + r) * CST + (kb * 16 + n) * 2) =
                            (_Float16)__builtin_amdgcn_fmed3f(dc[r], -kF16Max, kF16Max);
                    if (kb < 2) pkeep[rb][kb] = prob;
                }
                if (rb + 1 < NRB) __builtin_amdgcn_s_setprio(1);
            });
            // P of the tile as the consumer's MFMA operand: lane = key, elements = rows 4g.. of the
            // two row blocks
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
                bf16x8 pf;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pf[r] = (bf16_t)pkeep[0][kb][r];
                    pf[4 + r] = (bf16_t)pkeep[1][kb][r];
                }
                *reinterpret_cast<bf16x8 *>(Ps + (kb * 64 + lane) * 16) = pf;
            }
            };
            if (is_edge(r0)) ptile(std::true_type{});
            else ptile(std::false_type{});
        }
    } else {
    // ================================ consumer ================================
    f16x8 tfl[CQT];
    load_bands<CQT>(tfl, W + (size_t)h * cq * ck, cq, ck, pk, g, n, true, p.scale);
    f32x4 acc_k[2][DB], acc_v[2][DB];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            acc_k[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
            acc_v[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
    // dW: one accumulator per row of a group of RPL rows (see the dW loop)
    constexpr int RPL = 4;
    f32x4 acc_w[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) acc_w[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const int bcl = n < ck ? n : ck - 1;  // dW: lanes past the last key tap re-read a valid one
    const int pq = p.pq;
    // dS workspace blocks of this pair: [key tile][row tile of 64][32 keys][64 rows]
    const int n_rt = mfma_ds_row_tiles(p);
    bf16_t *ds_pair = dS_ws + ((bh * gridDim.z * NP + blockIdx.z * NP + pr) * n_rt) * (size_t)(WK * kDsRows);

    for (int it = 0; it <= n_tiles; ++it) {
        __syncthreads();
        if (it + 1 < n_tiles) stage_tile(it + 1);
        load_tile(r_begin + (it + 2) * BR);
        if (it == 0) continue;
        const int r0 = r_begin + (it - 1) * BR;   // the tile the producer finished in the last iteration
        if (is_skipped(r0)) continue;
        const bool edge = is_edge(r0);
        // the Q rows of this tile's dS (r0-16 .. r0+15) are blocks 2(it-1) and 2(it-1)+1
        const unsigned char *Qa = q_block(2 * (it - 1)), *Qb2 = q_block(2 * (it - 1) + 1), *Gs = stage_g(it - 1);
        const unsigned char *Ps = pair_p((it - 1) & 1);
        const int tb = ring_tb(it - 1), hb = ring_hb(it - 1), sb = s_base(it - 1);

        // ---- dS, rows r0-16 .. r0+15 (keys c0 .. c0+31): chains over the taps; the dC buffer
        // starts at row r0-16 ----
        f32x4 ds[NRB][2];
#pragma unroll
        for (int ob = 0; ob < NRB; ++ob)
#pragma unroll
            for (int m = 0; m < 2; ++m) ds[ob][m] = (f32x4){0.f, 0.f, 0.f, 0.f};
        {
            constexpr int NST = NRB * CQT;  // stage = (tap slot, row block)
            f16x8 cf[3][2];  // fragments two stages ahead
            auto load_cf = [&](int b2, int st) {
                const int a = st / NRB, ob = st % NRB;
                const int crow = ob * 16 + n + (CQT - 1) - a;  // window row: above the tile's own rows if < 16
                const unsigned char *base = c_ring + ((crow < HT ? hb : tb) + crow) * CST + (8 * g) * 2;
                cf[b2][0] = *reinterpret_cast<const f16x8 *>(base);
                cf[b2][1] = *reinterpret_cast<const f16x8 *>(base + 32);
            };
            load_cf(0, 0);
            load_cf(1, 1);
            SCHED_DS_READ_ID(4, 31);
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (st + 2 < NST) {
                    load_cf((st + 2) % 3, st + 2);
                    SCHED_DS_READ_ID(2, 31);
                }
#pragma unroll
                for (int m = 0; m < 2; ++m) ds[st % NRB][m] = mfma_f16(cf[st % 3][m], tfl[st / NRB], ds[st % NRB][m]);
                SCHED_MFMA_ID(2, 31);
            }
        }
        if (edge && causal) {
#pragma unroll
            for (int ob = 0; ob < NRB; ++ob)
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (c0 + m * 16 + n > r0 - HT + ob * 16 + 4 * g + r) ds[ob][m][r] = 0.f;
        }
        __builtin_amdgcn_s_setprio(1);  // the dense MFMA phase of the consumer
        // ---- dK^T += Q^T dS (the Q tile starts at row r0-16 as well) and dV ----
        {
            bf16x8 sf[2];
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    sf[m][r] = (bf16_t)ds[0][m][r];
                    sf[m][4 + r] = (bf16_t)ds[1][m][r];
                }
            // dS to the workspace: lane = key m*16+n holds rows 4g.. of the two 16-row blocks
            // r0-16.. and r0.., which is exactly one 16-byte piece of the key's row tile (row tile rt
            // starts at row 64 rt - 16; position 32k + 8g + 4h + r holds its row 32k + 16h + 4g + r).
#pragma unroll
            for (int m = 0; m < 2; ++m)
                *reinterpret_cast<bf16x8 *>(ds_pair + (size_t)(r0 / kDsRows) * (WK * kDsRows) +
                                            (m * 16 + n) * kDsRows + (r0 % kDsRows) + 8 * g) = sf[m];
            // dV^T += dO^T P (keys c0-8 .. c0+23) shares the loop: dO^T and Q^T by transpose reads of
            // the row-major tiles, four independent MFMAs per head-dim block
            bf16x8 pf[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) pf[kb] = *reinterpret_cast<const bf16x8 *>(Ps + (kb * 64 + lane) * 16);
            bf16x8 qt[2], gt[2];
            auto load_qg = [&](int b2, int db) {
                bf16x4 lo = lds_read_tr4x16(Qa, RST, 4 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Qb2, RST, 4 * g, db * 16, n);
                qt[b2] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                lo = lds_read_tr4x16(Gs, RST, 4 * g, db * 16, n);
                hi = lds_read_tr4x16(Gs, RST, 16 + 4 * g, db * 16, n);
                gt[b2] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            };
            load_qg(0, 0);
            SCHED_DS_READ_ID(6, 32);
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                if (db + 1 < DB) {
                    load_qg((db + 1) & 1, db + 1);
                    SCHED_DS_READ_ID(4, 32);
                }
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    acc_k[m][db] = mfma_bf16(qt[db & 1], sf[m], acc_k[m][db]);
                    acc_v[m][db] = mfma_bf16(gt[db & 1], pf[m], acc_v[m][db]);
                }
                SCHED_MFMA_ID(4, 32);
            }
        }

        __builtin_amdgcn_s_setprio(0);
        // ---- dW: rows m = tap a, columns n = tap b, contraction over (own row, 8 own keys) ----
        if (r0 < p.Nq) {
            // A: S[i + a - pq][c0 + 8g ..]        (S-tile row HT + i + a - pq, column 16 + 8g)
            // B: dC[i][c0 + 8g - b + pk ..]       (dC-tile row HT + i, column 8 + 8g - b + pk)
            const unsigned char *abase = s_ring + (16 + 8 * g) * 2;
            // LDS reads at odd 2-byte offsets are slow, and so are 128-bit reads off a 16-byte
            // boundary: read 5 single dwords from the even element below and funnel-shift by 0 or
            // 16 bits per lane instead.
            const int boff = 8 + 8 * g - bcl + pk;
            const unsigned char *bbase = c_ring + (tb + HT) * CST + (boff & ~1) * 2;
            const unsigned int bsh = (boff & 1) * 16;
            // The S operand is read once per group of RPL rows: lane m holds S row i + m - pq, which
            // for row i + u of the group is the row of tap a = m - u.  Row u of every group
            // therefore accumulates into its own accumulator, whose row m belongs to tap m - u; the
            // accumulators are added up with that shift once, after the tile loop.  Only rows
            // m - u < c_q matter, and (c_q - 1) + (RPL - 1) <= 15.
            static_assert(BR % RPL == 0 && (CQT - 1) + (RPL - 1) <= 15, "dW row groups");
#pragma unroll 1
            for (int i = 0; i < BR; i += RPL) {
                const u32x4 af = *reinterpret_cast<const u32x4 *>(abase + s_row(sb, HT + n - pq + i) * SST);
                u32x4 bw[RPL];
                unsigned int bx[RPL];
#pragma unroll
                for (int u = 0; u < RPL; ++u) {
                    lds_read_dwords5(bbase + (i + u) * CST, bw[u], bx[u]);
                }
#pragma unroll
                for (int u = 0; u < RPL; ++u) {
                    u32x4 sh;
                    sh[0] = __builtin_amdgcn_alignbit(bw[u][1], bw[u][0], bsh);
                    sh[1] = __builtin_amdgcn_alignbit(bw[u][2], bw[u][1], bsh);
                    sh[2] = __builtin_amdgcn_alignbit(bw[u][3], bw[u][2], bsh);
                    sh[3] = __builtin_amdgcn_alignbit(bx[u], bw[u][3], bsh);
                    acc_w[u] = mfma_f16(__builtin_bit_cast(f16x8, af), __builtin_bit_cast(f16x8, sh), acc_w[u]);
                }
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

    // ---- dW of this pair into its own LDS (over the tile buffers nobody reads any more): first the
    // RPL accumulators as [u][row m][tap b], then dW[a][b] = sum_u acc_u[a + u][b] as [16][16] ----
    float *red = reinterpret_cast<float *>(pair_base);
    static_assert(RPL * 1024 <= Lds::pair_bytes, "room for the dW accumulators");
#pragma unroll
    for (int u = 0; u < RPL; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[u * 256 + (4 * g + r) * 16 + n] = acc_w[u][r];
    __builtin_amdgcn_wave_barrier();
    float dw_out[4];
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
        const int o = lane + 64 * q4, a = o >> 4;
        float sum = 0.f;
#pragma unroll
        for (int u = 0; u < RPL; ++u) sum += (a + u < 16) ? red[u * 256 + o + 16 * u] : 0.f;
        dw_out[q4] = sum;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) red[lane + 64 * q4] = dw_out[q4];
    }  // consumer

    // ---- dW partial of this workgroup: ordered sum over the 4 pairs; S was raw, so * scale ----
    __syncthreads();
    const int ntap = cq * ck;
    if (tid < ntap) {
        const int a = tid / ck, bb = tid - a * ck;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NP; ++w)
            sum += reinterpret_cast<const float *>(smem + Lds::stage_bytes + w * Lds::pair_bytes)[a * 16 + bb];
        dW_part[(bh * gridDim.z + blockIdx.z) * ntap + tid] = sum * p.scale * dcs_inv;
    }
}

template <int D, int CQT, typename TO>
hipError_t launch_ws(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                     const float *Dl, const float *lse, const float *w, void *dk, void *dv, void *ds_ws,
                     float *dw_part, hipStream_t s) {
    auto kern = bwd_ws_mfma_kernel<D, CQT, TO>;
    constexpr int lds = WsLds<D>::total;
    static_assert(lds <= 160 * 1024, "LDS budget");
    hipError_t e = set_max_lds_once<bwd_ws_mfma_kernel<D, CQT, TO>>(lds);
    if (e != hipSuccess) return e;
    dim3 grid(p.H, p.B, mfma_kv_tiles(p));
    kern<<<grid, NT, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v,
                               (const bf16_t *)d_o, Dl, lse, w, (TO *)dk, (TO *)dv, (bf16_t *)ds_ws, dw_part);
    return hipGetLastError();
}

template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                   const float *Dl, const float *lse, const float *w, void *dk, void *dv, void *ds_ws,
                   float *dw_part, hipStream_t s) {
    if (p.c_q <= 3) return launch_ws<D, 3, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
    if (p.c_q <= 6) return launch_ws<D, 6, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
    return launch_ws<D, 11, TO>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
}

}  // namespace

hipError_t mfma_bwd_fused_ws(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                             const void *d_o, const float *Dl, const float *lse, const float *w, void *dk,
                             void *dv, void *ds_ws, float *dw_part, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
        return pick_cq<128, float>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
    return pick_cq<64, float>(p, q, k, v, d_o, Dl, lse, w, dk, dv, ds_ws, dw_part, s);
}

}  // namespace convattn
