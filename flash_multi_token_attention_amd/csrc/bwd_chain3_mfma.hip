// Whole backward of conv-attention on bf16 MFMA (gfx950), windows of up to 6 query taps: the
// key-stationary kernel of bwd_chain_mfma.hip with three waves per SIMD instead of two.
//
// A workgroup of 12 waves owns 128 keys of one (batch, head) and walks down the query rows in tiles
// of 32.  Triple p (waves p, p+4, p+8: one SIMD) owns keys c0 = k0 + 32p .. c0+31 for dK and dS,
// c0-8 .. c0+23 for dV and dW:
//   score wave (waves 0-3), tile it: dP^T = V dO^T - D; S^T (raw, pre-masked, packed to fp16); the
//       convolution as Toeplitz MFMAs on the packed S^T, row-shifted by DPP moves; P = exp2(C - LSE),
//       dC = P dP.  P (bf16), dC and S (fp16) go to LDS as [row][key] tiles;
//   value wave (waves 4-7), tile it-1: dV^T += dO^T P and dW += dC^T S (operands through LDS transpose
//       reads).  The last triple's value wave takes no part in dW; it computes, for tile it, the
//       C / dP / dC block after the workgroup's keys (the transposed convolution of a triple's 32 keys
//       needs dC on the 16 keys after them: for the other triples that is the next triple's first block);
//   key wave (waves 8-11), tile it-2: dS^T by flipped-band MFMAs over the packed dC^T of tiles it-2
//       and it-1, dS -> workspace and -> LDS, dK^T += Q^T dS.  The value and key waves issue the
//       loads of the Q / dO tile it+1 (global memory -> LDS); the last key wave stages LSE / D.
// One workgroup barrier per tile.  With 168 registers per wave every role keeps its operands and
// accumulators in registers, and a SIMD always has two other waves to issue from while one waits
// for LDS data, the matrix pipe or the barrier.
#include <type_traits>

#include "chain_common.hpp"

namespace convattn {
namespace {

using namespace chain;

constexpr int NT3 = 3 * NP * 64;  // 768 threads
// Wave priorities (s_setprio): the wave of a SIMD that has the least slack before the barrier issues first.
#ifndef C3_PRIO_SCORE
#define C3_PRIO_SCORE 1   // score waves, MFMA phases (0 in the P / dC arithmetic)
#endif
#ifndef C3_PRIO_EXTRA
#define C3_PRIO_EXTRA 3   // the value wave that also computes the block after the workgroup's keys
#endif
#ifndef C3_PRIO_VALUE
#define C3_PRIO_VALUE 1   // value waves
#endif
#ifndef C3_PRIO_KEY
#define C3_PRIO_KEY 0     // key waves
#endif
// LDS: the layout of the two-role kernel, then the V fragments of the block after the workgroup's keys
// (16 rows; the wave that computes that block has no registers to keep them in)
template <int D, int CQT> struct Chain3Lds : ChainLds<D, CQT> {
    static constexpr int e_off = ChainLds<D, CQT>::total;
    static constexpr int e_bytes = 16 * D * 2;
    static constexpr int total3 = e_off + e_bytes;
};

// One role of the workgroup: ROLE 0 = score waves, 1 = value waves (dV, dW, the block after the
// workgroup's keys), 2 = key waves (dS, dK).  WANT: bit 0 = dK and dV, bit 1 = dS (for dQ) and dW.
template <int D, int CQT, typename TO, int ROLE, int WANT>
__device__ __forceinline__ void chain3_role(const CHAIN_CONST_AS ChainArgs *args_in) {
    const unsigned long long av = reinterpret_cast<unsigned long long>(args_in);
    const unsigned long long as =
        ((unsigned long long)(unsigned int)__builtin_amdgcn_readfirstlane((int)(av >> 32)) << 32) |
        (unsigned int)__builtin_amdgcn_readfirstlane((int)(unsigned int)av);
    const ChainArgs args = *reinterpret_cast<const CHAIN_CONST_AS ChainArgs *>(as);
    const Problem p = args.p;
    const bf16_t *__restrict__ Q = args.Q, *__restrict__ K = args.K, *__restrict__ V = args.V, *__restrict__ dO = args.dO;
    const float *__restrict__ Dl = args.Dl, *__restrict__ LSE = args.LSE, *__restrict__ W = args.W;
    const float *__restrict__ dc_scale = args.dc_scale;
    TO *__restrict__ dK = static_cast<TO *>(args.dK), *__restrict__ dV = static_cast<TO *>(args.dV);
    bf16_t *__restrict__ dS_ws = args.dS_ws;
    float *__restrict__ dW_part = args.dW_part;
    const int n_rt = args.n_rt;
    using Lds = Chain3Lds<D, CQT>;
    constexpr int KS = D / 32, DB = D / 16;
    static_assert(CQT <= 6 && (2 * CQT) % 6 == 0, "whole dW units per value wave and half");
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    constexpr bool WANT_KV = (WANT & 1) != 0, WANT_QW = (WANT & 2) != 0;
    const int pr = wave & (NP - 1);

    auto q_slot = [&](int t) { return smem + Lds::q_off + (t & 3) * Lds::tile_bytes; };
    auto g_slot = [&](int t) { return smem + Lds::g_off + (t % 3) * Lds::tile_bytes; };
    auto stat_slot = [&](int t) { return reinterpret_cast<float *>(smem + Lds::stat_off + (t & 1) * (2 * BR * 4)); };
    unsigned char *pair_base = smem + Lds::pair_off + pr * Lds::pair_bytes;
    unsigned char *s_ring = pair_base;
    auto c_stage = [&](int t) { return pair_base + Lds::s_bytes + (t & 1) * (BR * CST); };
    auto p_stage = [&](int t) { return pair_base + Lds::s_bytes + Lds::c_bytes + (t & 1) * (BR * PST); };
    unsigned char *ds_tile = pair_base + Lds::s_bytes + Lds::c_bytes + Lds::p_bytes;

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
    // dC scale (a power of two): given by the caller, or, without one, taken from D = rowsum(dO O)
    float dcs, dcs_log2;
    if (dc_scale) {
        dcs = dc_scale[2 * bh];
        dcs_log2 = dc_scale[2 * bh + 1];
    } else {
        dcs_log2 = dc_scale_log2_from_d(dl_b, p.Nq, tid, NT3, reinterpret_cast<float *>(smem + Lds::stat_off));
        dcs = exp2f(dcs_log2);
    }

    // Causal: rows before the first key this workgroup touches (k0 - 8) see none of its keys.
    const int r_begin = causal ? (max(0, k0 - 8) / BR) * BR : 0;
    const int n_tiles = (p.Nq - r_begin + BR - 1) / BR;
    // masks are needed next to the diagonal, at both ends of the key axis and past the last row
    const bool always_edge = c0 < 8 || c0 + 40 > p.Nk;
    auto is_edge = [&](int r0) { return always_edge || (causal && r0 < c0 + 64) || r0 + BR > p.Nq; };
    // no (row, key) pair of the tile is visible: only its scores are needed, by the tile below
    auto is_skipped = [&](int r0) { return causal && r0 + BR - 1 < c0 - 8; };

    // Q / dO tiles: global memory -> LDS without passing through registers, issued by the eight value
    // and key waves (the score waves start on the tile right after the barrier).  A tile is 2 KBT units
    // of 1 KB (KBT of Q, then KBT of dO; unit 2 ks + f = the 16 row pairs of one k-step and parity).
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    constexpr int KBT = Lds::tile_bytes / 1024;
    static_assert(KBT == 2 * KS && ((2 * KBT) % (2 * NP) == 0 || 2 * KBT < 2 * NP), "whole units per loading wave");
    auto dma_rsrc = [&](const bf16_t *ptr) {
        const unsigned long long a = reinterpret_cast<unsigned long long>(ptr);
        return (i32x4){(int)(unsigned int)a, (int)(unsigned int)(a >> 32), p.Nq * D * 2, 0x00020000};
    };
    const i32x4 q_dma = dma_rsrc(Qb), g_dma = dma_rsrc(dOb);
    const unsigned int lds0 = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) unsigned char *)smem;
    auto fetch_tile = [&](int t) {
        if constexpr (ROLE != 0) {
            const int ln = (int)opaque((unsigned int)lane);
#pragma unroll
            for (int j0 = 0; j0 < 2 * KBT; j0 += 2 * NP) {
                const int j = j0 + wave - NP, m = j / KBT, kb = j - m * KBT;
                if (j >= 2 * KBT) break;   // (head dimension 32: four units for eight waves)
                const int row = 2 * (ln >> 2) + (kb & 1), chunk = (kb >> 1) * 4 + ((ln & 3) ^ ((ln >> 4) & 3));
                const int voff = ((r_begin + t * BR + row) * D + chunk * 8) * 2;
                const unsigned int dst = lds0 + (m ? Lds::g_off + (t % 3) * Lds::tile_bytes : Lds::q_off + (t & 3) * Lds::tile_bytes) + kb * 1024;
                const i32x4 rsrc = m ? g_dma : q_dma;
                // (M0 is written here and read by the load that follows; nothing else of this kernel uses it)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                             :: "s"(dst), "v"(voff), "s"(rsrc) : "memory");
            }
        }
    };
    // Every tile this wave has asked for is in LDS (to be followed by the workgroup barrier).  Vector
    // memory operations complete in the order of their issue: `younger` = the global stores the wave
    // has issued since the tile loads (the dS block of an iteration: exactly NDB * 2 stores), which need
    // not be waited for.
    auto tiles_landed = [&](bool younger) {
        if constexpr (ROLE != 0) {
            if (younger) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NDB * 2) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    };
    // LSE and D of a tile: loaded by the first 32 lanes of the last key wave one iteration before they
    // are written to LDS.  (A wave-uniform test, i.e. a branch: the other waves must not touch `ls` / `dd`.)
    const bool stat_wave = ROLE == 2 && pr == NP - 1;
    float ls = 0.f, dd = 0.f;
    auto load_stats = [&](int r0) {
        if constexpr (ROLE == 2) {
            if (stat_wave) {
                // raw values: arithmetic on them here would wait for the loads in this iteration
                const int tt = (int)opaque((unsigned int)lane);
                ls = 1e30f; dd = 0.f;  // rows past the end: exp2(C - LSE) = 0
                if (tt < BR && r0 + tt < p.Nq) { ls = lse_b[r0 + tt]; dd = dl_b[r0 + tt]; }
            }
        }
    };
    auto stage_stats = [&](int t) {
        if constexpr (ROLE == 2) {
            if (stat_wave) {
                const int tt = (int)opaque((unsigned int)lane);
                float *st = stat_slot(t);
                if (tt < BR) { st[tt] = ls * kLog2e - dcs_log2; st[BR + tt] = dd; }
            }
        }
    };
    // Lane parts of the fragment addresses inside a tile (see ChainLds).
    auto row_frag_off = [&] { return (unsigned int)(n * 64 + ((g ^ ((n >> 2) & 3)) << 4)); };
    auto tr_frag_off = [&] {
        return (unsigned int)(((n >> 2) & 1) * 1024 + (2 * g + (n >> 3)) * 64 + ((((n >> 1) & 1) ^ (g >> 1)) << 4) + (n & 1) * 8);
    };
    auto read_tr_t = [&](const unsigned char *lane_ptr, int db) {   // (db: a constant after unrolling)
        bf16x4 lo = lds_tr64(lane_ptr + (db >> 1) * 2048 + ((db & 1) << 5));
        bf16x4 hi = lds_tr64(lane_ptr + (db >> 1) * 2048 + (((db & 1) ^ 1) << 5) + 512);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };

    fetch_tile(0);
    load_stats(r_begin);

    // ---- The score chain of a tile for the score blocks KB0 .. KB0 + NKB - 1 (keys c0 - 16 + 16 kb ..) and the
    // C / dP / dC blocks CB0 .. CB0 + NCBL - 1 (keys c0 - 8 + 16 cb ..; block cb needs score blocks cb and cb + 1).
    // Score waves: blocks 0..2 and 0..1; the last value wave: blocks 2..3 and 2.  Runs the whole tile
    // loop when DRIVER (score waves), else `tile(it)` is called from the caller's loop. ----
    auto score_chain = [&](auto kb0_tag, auto nkb_tag, auto cb0_tag, auto ncb_tag, auto &&per_tile) {
        constexpr int KB0 = decltype(kb0_tag)::value, NKB = decltype(nkb_tag)::value;
        constexpr int CB0 = decltype(cb0_tag)::value, NCBL = decltype(ncb_tag)::value;
        static_assert(CB0 >= KB0 && CB0 - KB0 + NCBL + 1 <= NKB, "score blocks cover the C blocks");
        const bf16_t *Kb = K + bh * p.Nk * D;
        const bf16_t *Vb = V + bh * p.Nk * D;
        const unsigned char *bands = smem + opaque((unsigned int)Lds::band_off + lane * 16);
        // (the score waves keep their V fragments in registers; the value wave that computes the block after
        // the workgroup's keys parks them in LDS, in fragment order: one conflict-free 16-byte read per k-step)
        constexpr bool VLDS = KB0 != 0;
        static_assert(!VLDS || NCBL == 1, "LDS room for one block of V fragments");
        bf16x8 kf[NKB][KS], vf[NCBL][KS];
        unsigned char *v_park = smem + opaque((unsigned int)Lds::e_off + lane * 16);
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kf[kb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Kb, c0 - 16 + (KB0 + kb) * 16 + n, p.Nk, ks * 32 + g * 8));
#pragma unroll
        for (int cb = 0; cb < NCBL; ++cb)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                vf[cb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Vb, c0 - 8 + (CB0 + cb) * 16 + n, p.Nk, ks * 32 + g * 8));
        if constexpr (VLDS) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) *reinterpret_cast<bf16x8 *>(v_park + ks * 1024) = vf[0][ks];
        }
        // Q rows of the 32 rows above the first tile
        bf16x8 q_above[2][KS];
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                q_above[f][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Qb, r_begin - BR + 2 * n + f, p.Nq, ks * 32 + g * 8));

        unsigned int prev_pd[NKB][2][2];
        // S^T of the 32 rows r0 .. r0+31 (ring tile tp), pre-masked, packed and stored for dW
        auto s_phase = [&](int r0, int tp, unsigned int (&pd)[NKB][2][2], auto edge_tag, auto &&load_qf) {
            constexpr bool EDGE = decltype(edge_tag)::value;
            f32x4 acc[NKB][2];
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int f = 0; f < 2; ++f) acc[kb][f] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                bf16x8 qf[2];
#pragma unroll
                for (int f = 0; f < 2; ++f) qf[f] = load_qf(f, ks);
#pragma unroll
                for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                    for (int f = 0; f < 2; ++f) acc[kb][f] = mfma_bf16(kf[kb][ks], qf[f], acc[kb][f]);
            }
            const int rbase = (tp * BR) % S_RING;
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int f = 0; f < 2; ++f) {
                    if constexpr (EDGE) {
                        if (causal) {
                            const int qpos = r0 + 2 * n + f, key0 = c0 - 16 + (KB0 + kb) * 16 + 4 * g;
#pragma unroll
                            for (int r = 0; r < 4; ++r)
                                if (key0 + r > qpos) acc[kb][f][r] = 0.f;
                        }
                    }
                    // rounded exactly as the forward rounds its scores
                    const u32x2 two = pack_scores_f16(acc[kb][f]);
                    pd[kb][f][0] = two[0];
                    pd[kb][f][1] = two[1];
                    // (the ring holds the blocks 0..2 of a triple, written by its score wave)
                    if constexpr (KB0 == 0) {
                        if (WANT_QW && kb < 3) {
                            const int rr = rbase + 2 * n + f;
                            *reinterpret_cast<u32x2 *>(s_ring + (rr >= S_RING ? rr - S_RING : rr) * SST + (kb * 16 + 4 * g) * 2) =
                                (u32x2){pd[kb][f][0], pd[kb][f][1]};
                        }
                    }
                }
        };
        // the 32 rows above the first tile: their scores are the window's halo for tile 0
        s_phase(r_begin - BR, 0, prev_pd, std::true_type{}, [&](int f, int ks) { return q_above[f][ks]; });

        auto tile = [&](int it) {
            const int r0 = r_begin + it * BR;
            // dC of a tile that has none (entirely above the diagonal, or the one after the last):
            // zeros, so that the key waves read every tile alike
            auto zero_dc = [&] {
                const unsigned int ln = opaque((unsigned int)lane);
                unsigned char *Cs = c_stage(it) + 2 * (ln & 15) * CST + (ln >> 4) * 8;
#pragma unroll
                for (int cb = 0; cb < NCBL; ++cb)
#pragma unroll
                    for (int ob = 0; ob < 2; ++ob)
                        *reinterpret_cast<u32x2 *>(Cs + ob * CST + (CB0 + cb) * 32) = (u32x2){0u, 0u};
            };
            if (it == n_tiles) zero_dc();
            if (it >= n_tiles) return;
            auto ptile = [&](auto edge_tag, auto full_tag) {
                constexpr bool EDGE = decltype(edge_tag)::value;
                constexpr bool FULL = decltype(full_tag)::value;
                const unsigned char *Qs = smem + opaque((unsigned int)(q_slot(it) - smem) + row_frag_off());
                const unsigned char *Gs = smem + opaque((unsigned int)(g_slot(it) - smem) + row_frag_off());
                __builtin_amdgcn_s_setprio(VLDS ? C3_PRIO_EXTRA : C3_PRIO_SCORE);
                f32x4 dp[NCBL][2];
                float2 l2 = {0.f, 0.f};
                if constexpr (FULL) l2 = *reinterpret_cast<const float2 *>(stat_slot(it) + 2 * n);
                // ---- S^T ----
                unsigned int pd[NKB][2][2];
                s_phase(r0, it + 1, pd, edge_tag, [&](int f, int ks) {
                    return *reinterpret_cast<const bf16x8 *>(Qs + f * 1024 + ks * 2048);
                });
                // (the instance beside the dV accumulators has no registers for phases that overlap)
                if constexpr (VLDS) __builtin_amdgcn_sched_barrier(0);
                if constexpr (FULL) {
                    unsigned char *Cs = c_stage(it), *Ps = p_stage(it);
                    // ---- convolution: C^T block cb from score blocks cb (k slots 0..3 of a lane
                    // group) and cb+1 (4..7).  Operand of row offset delta = DL - (CQT-1): fragment
                    // f = delta & 1 shifted s = (f - delta) / 2 lanes down; it serves output parity
                    // 0 with tap slot DL and parity 1 with tap slot DL - 1. ----
                    f32x4 c[NCBL][2];
#pragma unroll
                    for (int cb = 0; cb < NCBL; ++cb) {
                        c[cb][0] = (f32x4){-l2.x, -l2.x, -l2.x, -l2.x};
                        c[cb][1] = (f32x4){-l2.y, -l2.y, -l2.y, -l2.y};
                    }
                    f16x8 tf_prev = (f16x8)(_Float16)0.f;
                    static_for<CQT + 1>([&](auto DL) {
                        constexpr int t0 = decltype(DL)::value;
                        constexpr int delta = t0 - (CQT - 1);
                        constexpr int f = delta & 1, s = (f - delta) / 2;
                        f16x8 tf_cur = tf_prev;
                        if constexpr (t0 < CQT) tf_cur = *reinterpret_cast<const f16x8 *>(bands + t0 * 1024);
                        unsigned int sh[NKB][2];
#pragma unroll
                        for (int kb = CB0 - KB0; kb < CB0 - KB0 + NCBL + 1; ++kb)
#pragma unroll
                            for (int dw = 0; dw < 2; ++dw) sh[kb][dw] = win_up<s>(prev_pd[kb][f][dw], pd[kb][f][dw]);
#pragma unroll
                        for (int cb = 0; cb < NCBL; ++cb) {
                            constexpr int o = CB0 - KB0;
                            const u32x4 bv = {sh[o + cb][0], sh[o + cb][1], sh[o + cb + 1][0], sh[o + cb + 1][1]};
                            if constexpr (t0 < CQT) c[cb][0] = mfma_f16(tf_cur, __builtin_bit_cast(f16x8, bv), c[cb][0]);
                            if constexpr (t0 >= 1) c[cb][1] = mfma_f16(tf_prev, __builtin_bit_cast(f16x8, bv), c[cb][1]);
                        }
                        tf_prev = tf_cur;
                    });
#pragma unroll
                    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                        for (int f = 0; f < 2; ++f) { prev_pd[kb][f][0] = pd[kb][f][0]; prev_pd[kb][f][1] = pd[kb][f][1]; }
                    // ---- dP^T = V dO^T - D, after the convolution (the shifted score windows are no longer live) ----
                    if constexpr (VLDS) __builtin_amdgcn_sched_barrier(0);
                    {
                        const float2 d2 = *reinterpret_cast<const float2 *>(stat_slot(it) + BR + 2 * n);
#pragma unroll
                        for (int cb = 0; cb < NCBL; ++cb) {
                            dp[cb][0] = (f32x4){-d2.x, -d2.x, -d2.x, -d2.x};
                            dp[cb][1] = (f32x4){-d2.y, -d2.y, -d2.y, -d2.y};
                        }
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks) {
                            bf16x8 gf[2];
#pragma unroll
                            for (int f = 0; f < 2; ++f)
                                gf[f] = *reinterpret_cast<const bf16x8 *>(Gs + f * 1024 + ks * 2048);
#pragma unroll
                            for (int cb = 0; cb < NCBL; ++cb) {
                                bf16x8 vk = vf[cb][ks];
                                if constexpr (VLDS) vk = *reinterpret_cast<const bf16x8 *>(v_park + ks * 1024);
#pragma unroll
                                for (int f = 0; f < 2; ++f) dp[cb][f] = mfma_bf16(vk, gf[f], dp[cb][f]);
                            }
                        }
                    }
                    // ---- P = exp2(C - LSE) (times the dC scale), dC = P dP ----
                    if constexpr (VLDS) __builtin_amdgcn_sched_barrier(0);
                    static_for<NCBL>([&](auto CB) {
                        constexpr int cb = decltype(CB)::value, cba = CB0 + cb;
                        __builtin_amdgcn_s_setprio(VLDS ? C3_PRIO_EXTRA : 0);
#pragma unroll
                        for (int ob = 0; ob < 2; ++ob) {
                            f32x4 prob, dc;
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                prob[r] = fast_exp2(c[cb][ob][r]);
                                dc[r] = prob[r] * dp[cb][ob][r];
                            }
                            if constexpr (EDGE) {
                                const int qpos = r0 + 2 * n + ob;
#pragma unroll
                                for (int r = 0; r < 4; ++r) {
                                    const int key = c0 - 8 + cba * 16 + 4 * g + r;
                                    if (key < 0 || key >= p.Nk || (causal && key > qpos)) { prob[r] = 0.f; dc[r] = 0.f; }
                                }
                            }
                            *reinterpret_cast<u32x2 *>(Cs + (2 * n + ob) * CST + (cba * 16 + 4 * g) * 2) =
                                (u32x2){pack_f16_rtz(dc[0], dc[1]), pack_f16_rtz(dc[2], dc[3])};
                            if constexpr (WANT_KV && cba < 2) {
                                bf16x4 pv;
#pragma unroll
                                for (int r = 0; r < 4; ++r) pv[r] = (bf16_t)prob[r];
                                *reinterpret_cast<bf16x4 *>(Ps + (2 * n + ob) * PST + (cba * 16 + 4 * g) * 2) = pv;
                            }
                        }
                    });
                } else {
#pragma unroll
                    for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                        for (int f = 0; f < 2; ++f) { prev_pd[kb][f][0] = pd[kb][f][0]; prev_pd[kb][f][1] = pd[kb][f][1]; }
                    zero_dc();
                }
            };
            if (is_skipped(r0)) ptile(std::true_type{}, std::false_type{});
            else if (is_edge(r0)) ptile(std::true_type{}, std::true_type{});
            else ptile(std::false_type{}, std::true_type{});
        };
        per_tile(tile);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;

    if constexpr (ROLE == 0) {
        // ================================ score waves ================================
        // bands (times scale * log2 e: the convolved scores come out in log2 units) in LDS, one KB
        // per tap slot, the slots dealt out to the four waves; the first barrier of the tile loop
        // publishes them
        for (int t = pr; t < CQT; t += NP)
            *reinterpret_cast<f16x8 *>(smem + Lds::band_off + t * 1024 + lane * 16) =
                band_frag<CQT>(t, W + (size_t)h * cq * ck, cq, ck, pk, g, n, false, p.scale * kLog2e);
        score_chain(I0{}, I3{}, I0{}, I2{}, [&](auto &&tile) {
            for (int it = 0; it <= n_tiles + 1; ++it) {
                __syncthreads();
                tile(it);
            }
        });
        __syncthreads();  // the value waves' barrier before they hand over their dW accumulators
        __syncthreads();  // ... and the one after it
        // ---- dW partial of this workgroup: G[m][n] of half x belongs to key tap b = n - m + 16 x - 8 + pk;
        // the sum runs over the pair groups, the halves and the diagonals' elements in a fixed order.
        // S was raw, so * scale; dC was scaled, so / dcs. ----
        static_assert(2 * CQT * 2 * 1024 <= NP * ChainLds<D, CQT>::pair_bytes, "room for the dW accumulators");
        // Four lanes per tap (pair group, half), each adds its diagonal's elements in index order; the
        // four sums are added as (0 + 1) + (2 + 3).
        const int ntap = cq * ck;
        for (int q = tid; WANT_QW && (q >> 2) < ntap; q += NP * 64) {
            const int tap = q >> 2, a = tap / ck, bb = tap - a * ck, t = a + CQT - cq;
            const int pgi = (q >> 1) & 1, x = q & 1;
            const float *red = reinterpret_cast<const float *>(smem + Lds::pair_off) + ((pgi * CQT + t) * 2 + x) * 256;
            float sum = 0.f;
#pragma unroll
            for (int m = 0; m < 16; ++m) {
                const int nn = bb + m - 16 * x + 8 - pk;
                const float val = red[m * 16 + min(max(nn, 0), 15)];
                if (nn >= 0 && nn < 16) sum += val;
            }
            sum += __shfl_xor(sum, 1);
            sum += __shfl_xor(sum, 2);
            if ((q & 3) == 0) dW_part[(bh * gridDim.z + blockIdx.z) * ntap + tap] = sum * p.scale / dcs;
        }
    } else if constexpr (ROLE == 1) {
        // ================================ value waves ================================
        f32x4 acc_v[2][DB];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int db = 0; db < DB; ++db) acc_v[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // dV^T += dO^T P of tile u (keys c0-8 .. c0+23)
        auto dv_phase = [&](int u, auto prio_tag) {
            const unsigned char *Ps = smem + opaque((unsigned int)(p_stage(u) - smem) + tr_lane_off(PST, g, n));
            const unsigned char *Gs = smem + opaque((unsigned int)(g_slot(u) - smem) + tr_frag_off());
            __builtin_amdgcn_s_setprio(decltype(prio_tag)::value);
            constexpr int PF = 3;
            bf16x8 pf[2], gq[PF + 1];
#pragma unroll
            for (int cb = 0; cb < 2; ++cb) pf[cb] = read_tr(Ps, PST, cb * 16);
#pragma unroll
            for (int db = 0; db < PF && db < DB; ++db) gq[db] = read_tr_t(Gs, db);
            static_for<DB>([&](auto DBI) {
                constexpr int db = decltype(DBI)::value;
                if constexpr (db + PF < DB) {
                    gq[(db + PF) % (PF + 1)] = read_tr_t(Gs, db + PF);
                    SCHED_DS_READ_ID(2, 60 + db);
                }
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) acc_v[cb][db] = mfma_bf16(gq[db % (PF + 1)], pf[cb], acc_v[cb][db]);
                SCHED_MFMA_ID(2, 60 + db);
            });
        };
        auto store_dv = [&] {
            const float inv = 1.f / dcs;
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                const int key_v = c0 - 8 + m * 16 + n;
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const int col = db * 16 + 4 * g;
                    if (WANT_KV && key_v >= 0 && key_v < p.Nk) {
                        TO *dst = dV + (bh * p.Nk + key_v) * D + col;
                        if constexpr (sizeof(TO) == 2) {
                            bf16x4 ov;
#pragma unroll
                            for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_v[m][db][r] * inv);
                            *reinterpret_cast<bf16x4 *>(dst) = ov;
                        } else {
                            *reinterpret_cast<f32x4 *>(dst) = acc_v[m][db] * inv;
                        }
                    }
                }
            }
        };
        if (pr == NP - 1) {
            // the last triple: no dW; the score chain of the block after the workgroup's keys instead
            score_chain(I2{}, I2{}, I2{}, I1{}, [&](auto &&tile) {
                for (int it = 0; it <= n_tiles + 1; ++it) {
                    tiles_landed(false);
                    __syncthreads();
                    if (it + 1 < n_tiles) fetch_tile(it + 1);
                    const int u = it - 1;
                    if (WANT_KV && it >= 1 && u < n_tiles && !is_skipped(r_begin + u * BR)) dv_phase(u, std::integral_constant<int, C3_PRIO_EXTRA>{});
                    __builtin_amdgcn_sched_barrier(0);
                    tile(it);
                }
            });
            __syncthreads();
            __syncthreads();
            store_dv();
        } else {
            // dW: a unit is the key blocks of two triples (pair group) times one tap slot; the waves 0 .. 2
            // take 2 CQT / 3 consecutive units each, in two passes of NU units of one pair group.
            constexpr int NU = CQT / 3, NPASS = 2, TH = NU * NPASS;
            int dw_pg[NPASS], dw_t[NPASS];
#pragma unroll
            for (int ps = 0; ps < NPASS; ++ps) {
                const int q = pr * TH + ps * NU;
                dw_pg[ps] = q / CQT;
                dw_t[ps] = q - dw_pg[ps] * CQT;
            }
            f32x4 acc_w[TH][2];
#pragma unroll
            for (int t = 0; t < TH; ++t) acc_w[t][0] = acc_w[t][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
            for (int it = 0; it <= n_tiles + 1; ++it) {
                tiles_landed(false);
                __syncthreads();
                if (it + 1 < n_tiles) fetch_tile(it + 1);
                const int u = it - 1;
                const bool u_in = it >= 1 && u < n_tiles;
                if (WANT_KV && u_in && !is_skipped(r_begin + u * BR)) dv_phase(u, std::integral_constant<int, C3_PRIO_VALUE>{});
                // ---- dW, key blocks jb = 0..3 of the triples 2 pg and 2 pg + 1 (block jb = dC block jb & 1 of
                // triple 2 pg + jb / 2, keys k0 + 64 pg - 8 + 16 jb ..), tap slots t_lo .. t_lo + NU - 1:
                // G_t[j][j'] += sum_rows dC[row][j] S[row + t - (CQT-1)][j'] with j' in the score block
                // 8 keys before the dC block (x = 0) and the one 8 keys after it (x = 1) ----
                if (WANT_QW && u_in) static_for<NPASS>([&](auto PS) {
                    constexpr int ps = decltype(PS)::value;
                    const int pg = dw_pg[ps], t_lo = dw_t[ps];
                    const int wbase = ((u + 1) * BR - (CQT - 1) + S_RING) % S_RING;
                    const unsigned int c_lane = opaque(tr_lane_off(CST, g, n));
                    const unsigned int ring0 = Lds::pair_off + 2 * pg * Lds::pair_bytes + 4 * (n & 3) * 2;
                    unsigned int a_lo[NU], a_hi[NU];
#pragma unroll
                    for (int tt = 0; tt < NU; ++tt) {
                        const unsigned int ra = wbase + 4 * g + (n >> 2) + min(t_lo + tt, CQT - 1), rb = ra + 16;
                        a_lo[tt] = opaque(ring0 + min(ra, ra - S_RING) * SST);
                        a_hi[tt] = opaque(ring0 + min(rb, rb - S_RING) * SST);
                    }
                    const unsigned int off4 = pg == NP / 2 - 1 ? Lds::pair_bytes + 64 : 2 * Lds::pair_bytes;
                    unsigned int a4_lo[NU], a4_hi[NU];
#pragma unroll
                    for (int tt = 0; tt < NU; ++tt) { a4_lo[tt] = a_lo[tt] + off4; a4_hi[tt] = a_hi[tt] + off4; }
                    auto s_frag = [&](auto JBP, int tt) {
                        constexpr int jbp = decltype(JBP)::value;
                        constexpr int off = (jbp >> 1) * Lds::pair_bytes + (jbp & 1) * 32;
                        bf16x4 l4, h4;
                        if constexpr (jbp < 4) {
                            l4 = lds_tr64(smem + a_lo[tt] + off);
                            h4 = lds_tr64(smem + a_hi[tt] + off);
                        } else {
                            l4 = lds_tr64(smem + a4_lo[tt]);
                            h4 = lds_tr64(smem + a4_hi[tt]);
                        }
                        return __builtin_bit_cast(f16x8, __builtin_shufflevector(l4, h4, 0, 1, 2, 3, 4, 5, 6, 7));
                    };
                    auto c_frag = [&](int jb) {
                        const int dq = jb >> 1;
                        return __builtin_bit_cast(
                            f16x8, read_tr(smem + Lds::pair_off + 2 * pg * Lds::pair_bytes + Lds::s_bytes + (u & 1) * (BR * CST) +
                                               c_lane + dq * Lds::pair_bytes, CST, (jb & 1) * 16));
                    };
                    f16x8 af = c_frag(0), b0[NU], b1[NU];
#pragma unroll
                    for (int tt = 0; tt < NU; ++tt) {
                        b0[tt] = s_frag(std::integral_constant<int, 0>{}, tt);
                        b1[tt] = s_frag(std::integral_constant<int, 1>{}, tt);
                    }
                    static_for<4>([&](auto JB) {
                        constexpr int jb = decltype(JB)::value;
                        f16x8 af_n = af, b2[NU];
#pragma unroll
                        for (int tt = 0; tt < NU; ++tt) b2[tt] = b1[tt];
                        if constexpr (jb < 3) {
                            af_n = c_frag(jb + 1);
#pragma unroll
                            for (int tt = 0; tt < NU; ++tt) b2[tt] = s_frag(std::integral_constant<int, jb + 2>{}, tt);
                            SCHED_DS_READ_ID(2 + 2 * NU, 40 + 4 * ps + jb);
                        }
#pragma unroll
                        for (int tt = 0; tt < NU; ++tt) {
                            acc_w[ps * NU + tt][0] = mfma_f16(af, b0[tt], acc_w[ps * NU + tt][0]);
                            acc_w[ps * NU + tt][1] = mfma_f16(af, b1[tt], acc_w[ps * NU + tt][1]);
                        }
                        SCHED_MFMA_ID(2 * NU, 40 + 4 * ps + jb);
                        af = af_n;
#pragma unroll
                        for (int tt = 0; tt < NU; ++tt) { b0[tt] = b1[tt]; b1[tt] = b2[tt]; }
                    });
                });
            }
            // ---- dW accumulators of this wave to LDS as [pair group][tap slot][x][m][n], once every
            // wave is done with the tiles ----
            __syncthreads();
            float *red = reinterpret_cast<float *>(smem + Lds::pair_off);
#pragma unroll
            for (int ps = 0; ps < NPASS; ++ps)
#pragma unroll
                for (int tt = 0; tt < NU; ++tt)
#pragma unroll
                    for (int x = 0; x < 2; ++x)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (WANT_QW && dw_t[ps] + tt < CQT)
                                red[(((dw_pg[ps] * CQT + dw_t[ps] + tt) * 2 + x) * 16 + 4 * g + r) * 16 + n] = acc_w[ps * NU + tt][x][r];
            __syncthreads();  // the score waves add the dW partial up while the others store dK and dV
            store_dv();
        }
    } else {
        // ================================ key waves ================================
        const float *w_head = W + (size_t)h * cq * ck;
        // flipped bands (times the softmax scale) in LDS, one KB per tap slot, dealt out to the four waves
        unsigned char *bands = smem + opaque((unsigned int)Lds::band_off + CQT * 1024 + lane * 16);
        for (int t = pr; t < CQT; t += NP)
            *reinterpret_cast<f16x8 *>(bands + t * 1024) = band_frag<CQT>(t, w_head, cq, ck, pk, g, n, true, p.scale);
        stage_stats(0);
        load_stats(r_begin + BR);
        f32x4 acc_k[NDB][DB];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int db = 0; db < DB; ++db) acc_k[m][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
        unsigned int prev_dc[NCB][2][2];
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int f = 0; f < 2; ++f) prev_dc[cb][f][0] = prev_dc[cb][f][1] = 0u;
        const int n_kt = gridDim.z * NP, kt = blockIdx.z * NP + pr;
        // (causal: the pair's first block is row tile kt - 1)
        bf16_t *ds_pair = dS_ws + (bh * (size_t)chain_ds_block_off(causal, n_rt, n_kt) + (size_t)chain_ds_block_off(causal, n_rt, kt) -
                                   chain_ds_first_rt(causal, kt)) * (WK * BR);

        bool ds_stored = false;  // the last iteration stored a dS block (after its tile loads)
        for (int it = 0; it <= n_tiles + 1; ++it) {
            tiles_landed(ds_stored);
            ds_stored = false;
            __syncthreads();
            // (the LSE / D loads before the tile loads: the counted wait above relies on that order)
            if (it + 1 < n_tiles) stage_stats(it + 1);
            load_stats(r_begin + (it + 2) * BR);
            if (it + 1 < n_tiles) fetch_tile(it + 1);
            const int u = it - 1, v = it - 2;
            const int r0v = r_begin + v * BR;
            const bool v_ok = it >= 2 && !is_skipped(r0v);
            // packed dC^T of tile u, as the score wave's lanes held it (zeros when the tile has none)
            unsigned int cur_dc[NCB][2][2];
            {
                // read unconditionally: the score waves write zeros for a tile without dC; what the first
                // iteration reads (nothing written yet) is dropped before any use
                const unsigned char *Cl = smem + opaque((unsigned int)(c_stage(max(u, 0)) - smem) + 2 * n * CST + 4 * g * 2);
                // the block after the triple's own keys: the first block of the next triple's stage (the last
                // triple's value wave writes it to its own stage)
                const unsigned char *Cn = Cl + (pr == NP - 1 ? 2 * 32 : Lds::pair_bytes);
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                    for (int f = 0; f < 2; ++f) {
                        const u32x2 t2 = *reinterpret_cast<const u32x2 *>(cb < 2 ? Cl + f * CST + cb * 32 : Cn + f * CST);
                        cur_dc[cb][f][0] = t2[0];
                        cur_dc[cb][f][1] = t2[1];
                    }
            }
            if (v_ok) {
                bf16_t *ds_blk = ds_pair + (size_t)(r0v / BR) * (WK * BR);
                __builtin_amdgcn_s_setprio(C3_PRIO_KEY);
                // ---- dS^T of tile v: rows below it come from tile v+1.  Operand of row offset
                // e = parity + (CQT-1 - tap slot): fragment e & 1 shifted e >> 1 lanes up. ----
                f32x4 ds[NDB][2];
#pragma unroll
                for (int sb = 0; sb < NDB; ++sb) ds[sb][0] = ds[sb][1] = (f32x4){0.f, 0.f, 0.f, 0.f};
                auto band_of = [&](int e) { return *reinterpret_cast<const f16x8 *>(bands + (CQT - 1 - e) * 1024); };
                f16x8 tbq[4];   // bands of steps e-1 .. e+2
                tbq[0] = band_of(0);
                tbq[1] = band_of(CQT >= 2 ? 1 : 0);
                tbq[2] = tbq[3] = tbq[0];
                static_for<CQT + 1>([&](auto E) {
                    constexpr int e = decltype(E)::value, f = e & 1, s = e >> 1;
                    if constexpr (e + 2 <= CQT - 1) tbq[(e + 2) % 4] = band_of(e + 2);
                    const f16x8 tb_cur = tbq[e % 4], tb_prev = tbq[(e + 3) % 4];
                    unsigned int sh[NCB][2];
#pragma unroll
                    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                        for (int dw = 0; dw < 2; ++dw) sh[cb][dw] = win_down<s>(prev_dc[cb][f][dw], cur_dc[cb][f][dw]);
#pragma unroll
                    for (int sb = 0; sb < NDB; ++sb) {
                        const u32x4 bv = {sh[sb][0], sh[sb][1], sh[sb + 1][0], sh[sb + 1][1]};
                        if constexpr (e <= CQT - 1) ds[sb][0] = mfma_f16(tb_cur, __builtin_bit_cast(f16x8, bv), ds[sb][0]);
                        if constexpr (e >= 1) ds[sb][1] = mfma_f16(tb_prev, __builtin_bit_cast(f16x8, bv), ds[sb][1]);
                    }
                });
                auto ds_out = [&](auto edge_tag) {
                    constexpr bool EDGE = decltype(edge_tag)::value;
#pragma unroll
                    for (int sb = 0; sb < NDB; ++sb)
#pragma unroll
                        for (int ob = 0; ob < 2; ++ob) {
                            if constexpr (EDGE) {
#pragma unroll
                                for (int r = 0; r < 4; ++r)
                                    if (c0 + sb * 16 + 4 * g + r > r0v + 2 * n + ob) ds[sb][ob][r] = 0.f;
                            }
                            bf16x4 sv;
#pragma unroll
                            for (int r = 0; r < 4; ++r) sv[r] = (bf16_t)ds[sb][ob][r];
                            // block layout [row parity][key half][16 row pairs][16 keys]: the 64 lanes of a store
                            // write 512 contiguous bytes
                            // (non-temporal: the blocks are read once, by another kernel; kept out of the L2 they do not
                            // push out the Q / dO tiles the other workgroups of this head are still reading)
                            if constexpr (WANT_QW)
                                __builtin_nontemporal_store(__builtin_bit_cast(u32x2, sv),
                                                            reinterpret_cast<u32x2 *>(ds_blk + ((ob * 2 + sb) * 16 + n) * 16 + 4 * g));
                            if constexpr (WANT_KV) *reinterpret_cast<bf16x4 *>(ds_tile + (2 * n + ob) * PST + (sb * 16 + 4 * g) * 2) = sv;
                        }
                };
                if (causal && is_edge(r0v)) ds_out(std::true_type{});
                else ds_out(std::false_type{});
                if constexpr (WANT_QW) ds_stored = true;
            }
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int f = 0; f < 2; ++f) { prev_dc[cb][f][0] = cur_dc[cb][f][0]; prev_dc[cb][f][1] = cur_dc[cb][f][1]; }
            if (WANT_KV && v_ok) {
                const unsigned char *Qs = smem + opaque((unsigned int)(q_slot(v) - smem) + tr_frag_off());
                const unsigned char *Dsl = smem + opaque((unsigned int)(ds_tile - smem) + tr_lane_off(PST, g, n));
                asm volatile("" ::: "memory");
                __builtin_amdgcn_wave_barrier();
                // ---- dK^T += Q^T dS ----
                {
                    constexpr int PF = 3;
                    bf16x8 sf[2], qq[PF + 1];
#pragma unroll
                    for (int db = 0; db < PF && db < DB; ++db) qq[db] = read_tr_t(Qs, db);
#pragma unroll
                    for (int sb = 0; sb < 2; ++sb) sf[sb] = read_tr(Dsl, PST, sb * 16);
                    static_for<DB>([&](auto DBI) {
                        constexpr int db = decltype(DBI)::value;
                        if constexpr (db + PF < DB) {
                            qq[(db + PF) % (PF + 1)] = read_tr_t(Qs, db + PF);
                            SCHED_DS_READ_ID(2, 70 + db);
                        }
#pragma unroll
                        for (int sb = 0; sb < 2; ++sb) acc_k[sb][db] = mfma_bf16(qq[db % (PF + 1)], sf[sb], acc_k[sb][db]);
                        SCHED_MFMA_ID(2, 70 + db);
                    });
                }
                asm volatile("" ::: "memory");
                __builtin_amdgcn_wave_barrier();
            }
        }
        __syncthreads();
        __syncthreads();
        // ---- dK: lane = key, 4 consecutive head-dim columns per block ----
        const float inv = 1.f / dcs;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const int key_k = c0 + m * 16 + n;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int col = db * 16 + 4 * g;
                if (WANT_KV && key_k < p.Nk) {
                    TO *dst = dK + (bh * p.Nk + key_k) * D + col;
                    if constexpr (sizeof(TO) == 2) {
                        bf16x4 ov;
#pragma unroll
                        for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc_k[m][db][r] * inv);
                        *reinterpret_cast<bf16x4 *>(dst) = ov;
                    } else {
                        *reinterpret_cast<f32x4 *>(dst) = acc_k[m][db] * inv;
                    }
                }
            }
        }
    }
}

template <int D, int CQT, typename TO, int WANT>
__global__ __launch_bounds__(NT3) void bwd_chain3_kernel(ChainArgs args) {
#if defined(__HIP_DEVICE_COMPILE__)
    const CHAIN_CONST_AS ChainArgs *ap =
        (const CHAIN_CONST_AS ChainArgs *)__builtin_amdgcn_kernarg_segment_ptr();
#else
    const ChainArgs *ap = &args;
#endif
    const int role = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) / NP;
    if (role == 0) chain3_role<D, CQT, TO, 0, WANT>(ap);
    else if (role == 1) chain3_role<D, CQT, TO, 1, WANT>(ap);
    else chain3_role<D, CQT, TO, 2, WANT>(ap);
}

template <int D, int CQT, typename TO, int WANT>
hipError_t launch_chain3(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                         const float *Dl, const float *lse, const float *w, const float *dc_scale, void *dk,
                         void *dv, void *ds_ws, float *dw_part, hipStream_t s) {
    auto kern = bwd_chain3_kernel<D, CQT, TO, WANT>;
    constexpr int lds = Chain3Lds<D, CQT>::total3;
    static_assert(lds <= 160 * 1024, "LDS budget");
    hipError_t e = set_max_lds_once<bwd_chain3_kernel<D, CQT, TO, WANT>>(lds);
    if (e != hipSuccess) return e;
    dim3 grid(p.H, p.B, mfma_kv_tiles(p));
    ChainArgs args{p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, (const bf16_t *)d_o, Dl, lse, w,
                   dc_scale, dk, dv, (bf16_t *)ds_ws, dw_part, chain_row_tiles(p)};
    kern<<<grid, NT3, lds, s>>>(args);
    return hipGetLastError();
}

template <int D, typename TO, int WANT>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const void *d_o,
                   const float *Dl, const float *lse, const float *w, const float *dc_scale, void *dk, void *dv,
                   void *ds_ws, float *dw_part, hipStream_t s) {
    if (p.c_q <= 3) return launch_chain3<D, 3, TO, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    return launch_chain3<D, 6, TO, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
}

template <int WANT>
hipError_t pick_shape(const Problem &p, int out_dt, const void *q, const void *k, const void *v, const void *d_o,
                      const float *Dl, const float *lse, const float *w, const float *dc_scale, void *dk, void *dv,
                      void *ds_ws, float *dw_part, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
        return pick_cq<128, float, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    }
    if (p.d == 32) {
        if (out_dt == CONVATTN_BF16) return pick_cq<32, bf16_t, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
        return pick_cq<32, float, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    return pick_cq<64, float, WANT>(p, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
}

}  // namespace

// This file is compiled once per value of CONVATTN_CHAIN_UNIT (1 = dK and dV only, 2 = dS and dW
// only, 3 = everything), so that the three sets of instances build in parallel.
#ifndef CONVATTN_CHAIN_UNIT
#define CONVATTN_CHAIN_UNIT 3
#endif
#if CONVATTN_CHAIN_UNIT == 1
#define CHAIN3_ENTRY mfma_bwd_chain3_kv
#elif CONVATTN_CHAIN_UNIT == 2
#define CHAIN3_ENTRY mfma_bwd_chain3_qw
#else
#define CHAIN3_ENTRY mfma_bwd_chain3_all
#endif
hipError_t CHAIN3_ENTRY(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                        const void *d_o, const float *Dl, const float *lse, const float *w,
                        const float *dc_scale, void *dk, void *dv, void *ds_ws, float *dw_part, hipStream_t s) {
    return pick_shape<CONVATTN_CHAIN_UNIT>(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
}

}  // namespace convattn
