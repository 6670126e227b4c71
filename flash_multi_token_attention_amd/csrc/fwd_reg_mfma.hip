// Training forward of conv-attention on bf16 MFMA (gfx950): the scores never leave the registers.
//
// Workgroup = 4 waves of one (batch, head); a wave computes scores for 32 consecutive query rows
// (the first CQT-1 of them only as the window's halo above its 33-CQT output rows) and keeps
// O^T, the row sums and the softmax bases of its rows in registers for the whole key loop.
// Lane n of score fragment f holds row base + 2n + f.  Per 32-key step:
//   1. all waves issue the loads of the next step's K / V rows, which go from global memory
//      straight into the LDS buffer the step before this one has just left (buffer loads with the
//      LDS modifier: no staging registers, no LDS writes by the waves; a tile is kept as
//      [k-step][row][64 bytes] with the four 16-byte chunks XOR-swizzled with the row index, so that
//      one lane address per matrix serves every fragment; one barrier per step);
//   2. S^T = K Q^T for two 16-key blocks; the accumulator layout (lane = query row, 4 keys per
//      lane group) is, packed to fp16 after the causal pre-mask, already the B operand layout of
//      the convolution MFMA: k slots 0..3 of a lane group come from one block, 4..7 from the next
//      (the Toeplitz bands are built for that order), so a window of 32 input keys is two packed
//      blocks and the output block sits 8 keys into it.  The last block of a step is carried to
//      the next step; no score is computed twice along the keys;
//   3. convolution: C^T += T_a^T S^T(rows shifted by the tap).  A shift by an even number of
//      rows is a DPP row shift of the packed registers, by an odd number the other fragment
//      shifted; rows shifted in from above the wave's first row are zeros and only reach halo rows;
//   4. post-mask (-inf) and softmax numerators against a per-row base that is only raised (with
//      a rescale of O and the row sums) when a score exceeds it by more than 2^6: no cross-lane
//      traffic otherwise.  The true row maximum is kept per lane for the M output;
//   5. O^T += V^T P^T: V^T fragments through the LDS transpose read, P^T straight from the
//      softmax registers.
#include "mfma_common.hpp"

namespace convattn {
namespace {


// DPP move (CTRL 0x110+s: row_shr:s, lane n of a row of 16 gets lane n-s); lanes without a
// source lane get 0.
template <int CTRL>
__device__ __forceinline__ unsigned int dpp_zero(unsigned int src) {
    return (unsigned int)__builtin_amdgcn_update_dpp(0, (int)src, CTRL, 0xf, 0xf, true);
}

__device__ __forceinline__ unsigned int opaque_u32(unsigned int x) {
    asm volatile("" : "+v"(x));
    return x;
}
__device__ __forceinline__ bf16x4 lds_tr64(__attribute__((address_space(3))) const unsigned char *ptr) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(ptr));
    return __builtin_bit_cast(bf16x4, v);
}

constexpr int NW = 4;             // waves per workgroup
constexpr int BK = 32;            // keys per step
constexpr float kMaxSlack = 6.f;  // log2 units a score may exceed its row's exponent base by
// A wave computes scores for 32 consecutive rows; the first CQT-1 of them are only the
// window's halo, the other 33-CQT are its output rows.
constexpr int wave_rows(int cqt) { return 33 - cqt; }

constexpr int kFwdPfv = 2;    // V^T fragments read ahead of their MFMAs in the P V phase
constexpr int kFwdNbuf = 2;   // LDS buffers: the rows of step u+1 arrive during step u (3, two steps ahead, measured no faster)
template <int D> struct FwdLds {
    // K / V rows go from global memory straight into LDS (buffer loads with the LDS modifier: the
    // 64 lanes of a load fill 1 KB of consecutive LDS, which rules out padded rows).  A tile of 32
    // rows is kept as [k-step ks][row][64 bytes]: the 4 chunks of 16 bytes that a row holds of
    // head-dim columns 32 ks .. 32 ks + 31, chunk c at position c ^ s(row) with s = row / 4 mod 4 for
    // K and the same two bits swapped for V.  The row fragments of K (lane n reads row n) and the
    // transposed fragments of V then touch every bank equally often, and k-step, row block and head-dim
    // block are constant offsets from one lane address.
    static constexpr int KST = D * 2;              // bytes of a row in global memory
    static constexpr int k_bytes = BK * KST;
    static constexpr int buf_bytes = 2 * k_bytes;  // K rows, then V rows
    static constexpr int n_buf = kFwdNbuf;         // steps u, u+1 (and u+2) resident or on their way
    static constexpr int total = n_buf * buf_bytes;
};

template <int D, int CQT, typename TO>
__global__ __launch_bounds__(NW * 64, 2) void fwd_reg_mfma_kernel(
    Problem p, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const float *__restrict__ W, TO *__restrict__ O,
    float *__restrict__ M, float *__restrict__ L) {
    using Lds = FwdLds<D>;
    constexpr int KST = Lds::KST;
    constexpr int KS = D / 32;   // MFMA k-steps over the head dimension
    constexpr int DB = D / 16;   // 16-wide blocks of the head dimension
    constexpr int WR = wave_rows(CQT), BQ = NW * WR;
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;  // wave-uniform for the compiler too
    const int g = lane >> 4, n = lane & 15;

    // x = head, y = batch, z = query tile: the dispatcher hands out every (batch, head) of the
    // longest (causal) tiles first, so the tail of the launch is made of short tiles
    const int h = blockIdx.x, b = blockIdx.y;
    const int qt = gridDim.z - 1 - blockIdx.z;
    const int i0 = qt * BQ, i0w = i0 + wave * WR;
    const int base = i0w - (CQT - 1);  // first score row of the wave
    const int pk = p.pk, cq = p.c_q;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;

    // Toeplitz bands of this head, one fragment per tap slot, pre-multiplied by
    // scale * log2(e): the convolved scores come out in log2 units.  k slot 8g+e of a window
    // is key 4g+e of its first 16-key block for e < 4, key 4g+e-4 of its second for e >= 4.
    f16x8 tf[CQT];
    {
        const float *w_head = W + (size_t)h * cq * p.c_k;
        // (unconditional loads from clamped indices, all in flight together; the select happens on the values)
        float wv[CQT][8];
#pragma unroll
        for (int t = 0; t < CQT; ++t) {
            const int a = t - (CQT - cq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int kappa = e < 4 ? 4 * g + e : 16 + 4 * g + e - 4;
                const int bb = kappa - kKeyHalo - n + pk;
                wv[t][e] = w_head[max(a, 0) * p.c_k + min(max(bb, 0), p.c_k - 1)];
            }
        }
#pragma unroll
        for (int t = 0; t < CQT; ++t) {
            const int a = t - (CQT - cq);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int kappa = e < 4 ? 4 * g + e : 16 + 4 * g + e - 4;
                const int bb = kappa - kKeyHalo - n + pk;
                tf[t][e] = (_Float16)((a >= 0 && bb >= 0 && bb < p.c_k) ? wv[t][e] * (p.scale * kLog2e) : 0.f);
            }
        }
    }

    // Q^T fragments (B operand), resident for the whole loop: lane n of fragment f holds row
    // base + 2n + f, so a shift of the score rows by an even number of rows is a shift of
    // lanes and by an odd number a change of fragment as well.
    bf16x8 qf[2][KS];
#pragma unroll
    for (int f = 0; f < 2; ++f)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qf[f][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Qb, base + 2 * n + f, p.Nq, ks * 32 + g * 8));

    f32x4 acc_o[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_o[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_ref[2] = {kNegInf, kNegInf};   // exponent base of the row, in log2 units (same in the row's 4 lanes)
    float m_true[2] = {kNegInf, kNegInf};  // maximum of the scores this lane has seen
    // The convolution accumulates on top of minus the exponent base (0 while the row has none),
    // so its result is already the exponent; slack[ob]: how far it may go above 0 before the base
    // is raised (-inf while the row has no base: any visible score sets one).
    f32x4 neg_base[2] = {(f32x4){0.f, 0.f, 0.f, 0.f}, (f32x4){0.f, 0.f, 0.f, 0.f}};
    float slack[2] = {kNegInf, kNegInf};
    float l_run[2] = {0.f, 0.f};           // this lane's share of the row sum, relative to m_ref

    // Step u: score blocks 2u, 2u+1 (keys 32u-8 .. 32u+23, K rows of the step) and output blocks
    // 2u-1, 2u (keys 32u-16 .. 32u+15, V rows of the step); an output block needs the score
    // block 8 keys before it and the one 8 keys after it, so the packed scores of block 2u-1
    // are carried from the previous step.
    // K / V rows: buffer loads with the LDS modifier.  Rows before the first or after the last key
    // are outside the descriptor's range and arrive as zeros, which is what the window's zero
    // padding asks for.
    // A tile is 2 KS units of 1 KB (unit 2 ks + blk = rows 16 blk .. 16 blk + 15 of k-step ks); wave w
    // issues the units w, w + NW, ...  Lane l of a load fills chunk position l % 4 of row l / 4.
    // (head dimension 32: two units, issued by the waves 0 and 1)
    constexpr int UNITS = Lds::k_bytes / 1024, N_LD = UNITS >= NW ? UNITS / NW : 1;
    static_assert(UNITS == 2 * KS && (UNITS % NW == 0 || UNITS < NW) && NW == 4, "whole units per wave");
    const bool dma_wave = UNITS >= NW || wave < UNITS;
    // (K rows are read as row fragments, 16 rows of one chunk column at a time: swizzle value row / 4 mod 4;
    // V rows through transpose reads, 8 rows x 32 bytes per half wave: the same value with its two bits
    // swapped, so that rows r and r + 4 use different halves of their 64 bytes)
    const int dma_row = (16 * (wave & 1) + (lane >> 2)) * KST;
    const int dma_off = dma_row + (((wave >> 1) * 4 + ((lane & 3) ^ ((lane >> 4) & 3))) << 4);
    const int dma_off_v = dma_row + (((wave >> 1) * 4 + ((lane & 3) ^ ((((lane >> 4) & 1) << 1) | ((lane >> 5) & 1)))) << 4);
    // rows of step u: issued right after the barrier that ends step u - 1 (their buffer is free then),
    // landed by the barrier that starts step u (the barrier waits for the wave's loads)
    // (issued as inline assembly: for the builtin the compiler makes every later LDS read wait for the
    // load, since it cannot tell the two buffers apart; the wait is written out before the barrier instead)
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    auto dma_rsrc = [&](const bf16_t *ptr) {
        const unsigned long long a = reinterpret_cast<unsigned long long>(ptr);
        return (i32x4){(int)(unsigned int)a, (int)(unsigned int)(a >> 32), p.Nk * D * 2, 0x00020000};
    };
    const i32x4 k_dma = dma_rsrc(Kb), v_dma = dma_rsrc(Vb);
    const unsigned int lds_u = (unsigned int)(unsigned long long)(__attribute__((address_space(3))) unsigned char *)smem;
    const unsigned int lds_base = lds_u + wave * 1024;
    // unit i of the wave: k-step + 2 i = 128 bytes further along the row (the instruction's offset
    // field, which the hardware adds to the LDS address as well as to the global one), 4 KB further in
    // LDS; the step's first row is the scalar offset of the load
    auto dma16 = [&](const i32x4 &rsrc, unsigned int lds_addr, int voffset, int soffset, auto I) {
        constexpr int i = decltype(I)::value;
        // (M0 is written here and read by the load that follows; nothing else of this kernel uses it)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen offset:%4 lds"
                     :: "s"(__builtin_amdgcn_readfirstlane((int)lds_addr + i * (4096 - 128))), "v"(voffset), "s"(rsrc),
                        "s"(__builtin_amdgcn_readfirstlane(soffset)), "n"(i * 128) : "memory");
    };
    // step 0 starts before the first key: those rows have negative offsets, which only the vector
    // offset (a wrapping 32-bit sum made here) may carry; later steps pass theirs as the scalar offset
    auto fetch_step = [&](int u) {
        const unsigned int Ks = lds_base + (u % Lds::n_buf) * Lds::buf_bytes, Vs = Ks + Lds::k_bytes;
        const int k0 = (32 * u - 8) * KST, v0 = (32 * u - 16) * KST;
        if (dma_wave) static_for<N_LD>([&](auto I) {
            if (u == 0) {
                dma16(k_dma, Ks, dma_off + k0, 0, I);
                dma16(v_dma, Vs, dma_off_v + v0, 0, I);
            } else {
                // (a scalar offset past the end is held at the end: everything is out of range then,
                // whichever way the range check treats a scalar offset beyond the number of records)
                dma16(k_dma, Ks, dma_off, min(k0, p.Nk * KST), I);
                dma16(v_dma, Vs, dma_off_v, min(v0, p.Nk * KST), I);
            }
        });
    };
    // lane addresses (absolute LDS addresses) of the fragment reads inside the buffer of the step; they
    // are moved to the other buffer at the end of every step.  K row fragment: row n, chunk 4 ks + g;
    // row block and k-step are constant offsets.  V^T fragment: rows 4g + n/4 (+ 16), 8 bytes at byte
    // column 32 db + 8 (n % 4): head-dim blocks 2 x and 2 x + 1 differ in bit 5 of the lane part.
    unsigned int ka = opaque_u32(lds_u + n * 64 + ((g ^ ((n >> 2) & 3)) << 4));
    unsigned int va[2];
    va[0] = opaque_u32(lds_u + Lds::k_bytes + (4 * g + (n >> 2)) * 64 + ((((n >> 1) & 1) ^ (((g & 1) << 1) | (g >> 1))) << 4) + (n & 1) * 8);
    va[1] = opaque_u32(va[0] ^ 32u);
    typedef __attribute__((address_space(3))) const bf16x8 *lds_bf16x8_ptr;
    typedef __attribute__((address_space(3))) const unsigned char *lds_byte_ptr;

    // packed fp16 scores of the last score block of the previous step:
    // carry[f][dword] = row base + 2n + f, keys 4g .. 4g+3 of the block
    unsigned int carry[2][2] = {{0u, 0u}, {0u, 0u}};

    // One step of the wave; EDGE = the step touches the diagonal or an end of the keys
    // (wave-uniform), only then are the masks evaluated.
    auto step = [&](int u, auto edge_tag) {
        constexpr bool EDGE = decltype(edge_tag)::value;
        const int jk = 32 * u - 8, jv = 32 * u - 16;
        f32x4 c[2][2];
        bf16x8 kf[KS];  // K fragments of one score block; the second block's are read during the first's convolution
        unsigned int pd[2][2][2];  // [score block of the step][f][dword]
        auto load_kf = [&](int blk) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kf[ks] = *(lds_bf16x8_ptr)(size_t)(ka + blk * 1024 + ks * 2048);
        };
        load_kf(0);
        static_for<2>([&](auto BL) {
            constexpr int blk = decltype(BL)::value;
            // ---- S^T = K Q^T (raw), pre-mask, pack two keys per dword ----
            f32x4 acc[2];
#pragma unroll
            for (int f = 0; f < 2; ++f) acc[f] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int f = 0; f < 2; ++f) acc[f] = mfma_bf16(kf[ks], qf[f][ks], acc[f]);
            if constexpr (blk == 0) {
                load_kf(1);
                SCHED_DS_READ(KS);
                SCHED_MFMA(2 * CQT);
            }
            const int key0 = jk + blk * 16 + 4 * g;
#pragma unroll
            for (int f = 0; f < 2; ++f) {
                if constexpr (EDGE) {
                    if (causal) {
                        const int qpos = base + 2 * n + f;
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (key0 + r > qpos) acc[f][r] = 0.f;
                    }
                }
                const u32x2 two = pack_scores_f16(acc[f]);
                pd[blk][f][0] = two[0];
                pd[blk][f][1] = two[1];
            }
            // ---- convolution of output block blk: one B operand per row offset
            //      delta = (output row parity) + (tap slot) - (CQT-1): rows base + 2n + delta =
            //      fragment f shifted s lanes down (zeros shifted in: those lanes are halo rows,
            //      whose outputs are not used); k slots 0..3 of a lane group from the score block
            //      before, 4..7 from this one ----
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) c[ob][blk] = neg_base[ob];
            static_for<CQT + 1>([&](auto DL) {
                constexpr int delta = decltype(DL)::value - (CQT - 1);
                constexpr int f = delta & 1, s = (f - delta) / 2;
                u32x4 bv;
#pragma unroll
                for (int half = 0; half < 2; ++half)
#pragma unroll
                    for (int dw = 0; dw < 2; ++dw) {
                        const unsigned int own = half ? pd[blk][f][dw] : (blk ? pd[0][f][dw] : carry[f][dw]);
                        if constexpr (s == 0) bv[2 * half + dw] = own;
                        else bv[2 * half + dw] = dpp_zero<0x110 + s>(own);
                    }
                constexpr int t0 = delta + (CQT - 1);  // tap slot of output parity 0
                if constexpr (t0 < CQT) c[0][blk] = mfma_f16(tf[t0], __builtin_bit_cast(f16x8, bv), c[0][blk]);
                if constexpr (t0 >= 1) c[1][blk] = mfma_f16(tf[t0 - 1], __builtin_bit_cast(f16x8, bv), c[1][blk]);
            });
        });
#pragma unroll
        for (int f = 0; f < 2; ++f)
#pragma unroll
            for (int dw = 0; dw < 2; ++dw) carry[f][dw] = pd[1][f][dw];
        // V^T fragments of the first kFwdPfv head-dim blocks: in flight during the softmax
        constexpr int PFV = kFwdPfv < DB ? kFwdPfv : DB;
        bf16x8 vf[PFV + 1];
        auto load_vf = [&](int buf, int db) {
            bf16x4 lo = lds_tr64((lds_byte_ptr)(size_t)(va[db & 1] + (db >> 1) * 2048));
            bf16x4 hi = lds_tr64((lds_byte_ptr)(size_t)(va[db & 1] + (db >> 1) * 2048 + 1024));
            vf[buf] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        };
#pragma unroll
        for (int db = 0; db < PFV; ++db) load_vf(db, db);
        // The two waves of a SIMD are at different places of their steps: the one in an MFMA
        // phase (P V, S^T, the convolution) gets the issue slot first, the one in the softmax
        // arithmetic fills the gaps (measured: 1.5 % over equal priorities; the reverse is slower).
        __builtin_amdgcn_s_setprio(0);
        // ---- post-mask and softmax numerators (log2 domain).  The exponent base m_ref of a row
        //      only follows the row's maximum when some score exceeds it by more than kMaxSlack
        //      (then every lane group of the wave exchanges its maxima and rescales); otherwise no
        //      lane talks to another.  The true maximum is tracked per lane for the M output. ----
        float mloc[2];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) {
            if constexpr (EDGE) {
                const int qpos = base + 2 * n + ob;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = jv + kb * 16 + 4 * g + r;
                        if (key < 0 || key >= p.Nk || (causal && key > qpos)) c[ob][kb][r] = kNegInf;
                    }
            }
            float mx = kNegInf;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, c[ob][kb][r]);
            mloc[ob] = mx;                                           // relative to the base
            m_true[ob] = fmaxf(m_true[ob], mx - neg_base[ob][0]);   // absolute
        }
        if (__builtin_amdgcn_ballot_w64(mloc[0] > slack[0] || mloc[1] > slack[1]) != 0) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) {
                const float old_use = -neg_base[ob][0];
                float mx = mloc[ob] + old_use;
                mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
                mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
                const float m_new = fmaxf(m_ref[ob], mx);
                // rows with nothing visible yet keep m = -inf; 0 is the exponent base there
                const float new_use = (m_new == kNegInf) ? 0.f : m_new;
                const float alpha = fast_exp2(m_ref[ob] - new_use);
                const float delta = new_use - old_use;
                m_ref[ob] = m_new;
                slack[ob] = (m_new == kNegInf) ? kNegInf : kMaxSlack;
                neg_base[ob] = (f32x4){-new_use, -new_use, -new_use, -new_use};
                l_run[ob] *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db) acc_o[ob][db] *= alpha;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) c[ob][kb][r] -= delta;
            }
        }
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) {
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float e = fast_exp2(c[ob][kb][r]);
                    c[ob][kb][r] = e;
                    psum += e;
                }
            l_run[ob] += psum;
        }
        // ---- O^T += V^T P^T: V^T fragments through the LDS transpose read, P^T straight from
        //      the softmax registers (k slot 8g+e <-> key 4g+e of output block 0 for e < 4, of
        //      output block 1 for e >= 4) ----
        __builtin_amdgcn_s_setprio(1);
        bf16x8 pf[2];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pf[ob][r] = (bf16_t)c[ob][0][r];
                pf[ob][4 + r] = (bf16_t)c[ob][1][r];
            }
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            if (db + PFV < DB) {
                load_vf((db + PFV) % (PFV + 1), db + PFV);
                SCHED_DS_READ(2);
            }
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) acc_o[ob][db] = mfma_bf16(vf[db % (PFV + 1)], pf[ob], acc_o[ob][db]);
            SCHED_MFMA(2);
        }
    };

    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    const int n_steps = (k_end + 16 + BK - 1) / BK;
    fetch_step(0);
    if constexpr (Lds::n_buf == 3) fetch_step(1);
    // Along the keys a wave's steps are: step 0 (keys before the first one to mask), steps whose
    // keys all lie at or before its first score row (no masks), steps on the diagonal or at the
    // end of the keys (masks), and steps entirely after its rows (it only takes part in the
    // staging).  One loop per kind, so that each loop body has the accumulators in place.
    auto run = [&](int ua, int ub, auto kind) {
        constexpr int KIND = decltype(kind)::value;
#pragma unroll 1
        for (int u = ua; u < ub; ++u) {
            // this wave's rows of step u have landed (with three buffers those of step u + 1 may be on their way:
            // 2 * N_LD loads per step, and the loop body issues no other vector memory operation before this wait)
            if constexpr (Lds::n_buf == 3) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * N_LD) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();  // step u-1 is done everywhere: its buffer is free, and step u's is written
            fetch_step(u + Lds::n_buf - 1);
            if constexpr (KIND != 2) step(u, std::integral_constant<bool, KIND == 1>{});
            const int to_other = (u % Lds::n_buf == Lds::n_buf - 1) ? -(Lds::n_buf - 1) * Lds::buf_bytes : Lds::buf_bytes;
            ka += to_other;
            va[0] += to_other;
            va[1] += to_other;
        }
    };
    const int u_diag = base < 23 ? 1 : (base - 23) / 32 + 1;    // first u >= 1 with 32u + 23 > base
    const int u_tail = p.Nk < 24 ? 1 : (p.Nk - 24) / 32 + 1;    // first u >= 1 with 32u + 24 > Nk
    const int u1 = min(causal ? min(u_diag, u_tail) : u_tail, n_steps);
    const int u2 = max(u1, causal ? min((i0w + WR + 15) / 32 + 1, n_steps) : n_steps);  // 32u - 16 > i0w + WR - 1
    run(0, 1, std::integral_constant<int, 1>{});
    run(1, u1, std::integral_constant<int, 0>{});
    run(u1, u2, std::integral_constant<int, 1>{});
    run(u2, n_steps, std::integral_constant<int, 2>{});
    // ---- epilogue: finish the row sums and maxima, normalise, store O, M, L ----
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
        float l = l_run[ob];
        l += __shfl_xor(l, 16, kWave);
        l += __shfl_xor(l, 32, kWave);
        float mt = m_true[ob];
        mt = fmaxf(mt, __shfl_xor(mt, 16, kWave));
        mt = fmaxf(mt, __shfl_xor(mt, 32, kWave));
        const int qpos = base + 2 * n + ob;
        if (qpos >= i0w && qpos < p.Nq) {
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
                M[bh * p.Nq + qpos] = mt * (1.f / kLog2e);
                L[bh * p.Nq + qpos] = l * fast_exp2(m_ref[ob] - mt);
            }
        }
    }
}

template <int D, int CQT, typename TO>
hipError_t launch_fwd(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                      void *o, float *m, float *l, hipStream_t s) {
    auto kern = fwd_reg_mfma_kernel<D, CQT, TO>;
    constexpr int lds = FwdLds<D>::total;
    if (lds > 64 * 1024) {
        hipError_t e = set_max_lds_once<fwd_reg_mfma_kernel<D, CQT, TO>>(lds);
        if (e != hipSuccess) return e;
    }
    constexpr int BQ = NW * wave_rows(CQT);
    dim3 grid(p.H, p.B, (p.Nq + BQ - 1) / BQ);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, w,
                                    (TO *)o, m, l);
    return hipGetLastError();
}

template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                   void *o, float *m, float *l, hipStream_t s) {
    if (p.c_q <= 3) return launch_fwd<D, 3, TO>(p, q, k, v, w, o, m, l, s);
    if (p.c_q <= 6) return launch_fwd<D, 6, TO>(p, q, k, v, w, o, m, l, s);
    if (p.c_q <= 8) return launch_fwd<D, 8, TO>(p, q, k, v, w, o, m, l, s);
    return launch_fwd<D, 11, TO>(p, q, k, v, w, o, m, l, s);
}

}  // namespace


hipError_t mfma_fwd(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                    const float *w, void *o, float *m, float *l, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t>(p, q, k, v, w, o, m, l, s);
        return pick_cq<128, float>(p, q, k, v, w, o, m, l, s);
    }
    if (p.d == 32) {
        if (out_dt == CONVATTN_BF16) return pick_cq<32, bf16_t>(p, q, k, v, w, o, m, l, s);
        return pick_cq<32, float>(p, q, k, v, w, o, m, l, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t>(p, q, k, v, w, o, m, l, s);
    return pick_cq<64, float>(p, q, k, v, w, o, m, l, s);
}

}  // namespace convattn
