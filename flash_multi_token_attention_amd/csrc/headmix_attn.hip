// Head-mixing attention ("head_conv_attn" of the reference) on the matrix cores of gfx950.
//
//   S_h' = scale Q_h' K_h'^T,   Z_h = sum_h' w[h][h'] S_h',   P_h = softmax_j(Z_h + causal mask),
//   O_h = P_h V_h.
// The heads of a (batch, row, key) triple are coupled before the softmax, so a workgroup handles
// ALL heads of 16 query rows (forward, dQ + dW) or of 16 keys (dK / dV) of one batch entry and
// walks the other axis in tiles of 16.  Products of two inputs (Q K^T, dO V^T) run on the bf16 MFMA
// (exact products, fp32 accumulation); scores, the head mix, the softmax and dW stay fp32
// (v_mfma_f32_16x16x4_f32 for the mix and dW); products of a computed tile with an input (P V,
// P^T dO, dS K, dS^T Q) round the tile to bf16 and run on v_mfma_f32_16x16x16_bf16.
//
// Per 16 x 16 tile (8 waves):
//   1. waves take heads: S_h' from Q / K row fragments read straight from global memory
//      (16 bytes of a row are a lane's operand of the bf16 MFMA as they lie in memory)    -> LDS;
//   2. waves take rows: Z = W S as a product over the head index (A = W, B = the scores of one
//      row across the heads), mask, softmax (or P = exp(Z - LSE) in the backward)        -> LDS;
//   3. waves take heads again: P V (forward), dP = dO V^T, dV += P^T dO, dZ = P (dP - D);
//   4. (backward) waves take rows: dW += dZ S^T over the tile's elements, dS = W^T dZ in place;
//   5. (backward) waves take heads: dQ += dS K or dK += dS^T Q.
// Operands that are read along their rows (V, K, Q, dO as the right-hand side) are staged per wave
// in a 16-row bf16 tile.  Accumulators (O, dQ, dK / dV of up to 4 heads per wave) stay in registers
// for the whole loop; nothing is accumulated through global memory and there are no atomics
// (the reference's Triton kernels read-modify-write O per key block, fwd_kernel.py:214-250, and add
// dW with tl.atomic_add, bwd_dq_dw.py:370): dW partials are summed in a fixed order.
#include "mfma_common.hpp"

namespace convattn {
namespace {

typedef short short4_t __attribute__((ext_vector_type(4)));

// waves per workgroup: 16 in the forward (one or two heads per wave: half the accumulators and fragments per
// wave, four waves per SIMD to hide the latencies between the phases) and in the backward with 16 heads up to
// d = 64, where 128 registers per wave hold that without much scratch; otherwise 8 (two or four heads per wave;
// with 32 heads the dW accumulators of 16 waves would not fit the LDS either)
template <int H, int D, bool BWD> constexpr int kHmWaves = (!BWD || (H == 16 && D <= 64)) ? 16 : 8;
constexpr int HT = 16;           // rows / keys per tile
constexpr int SST = 20;          // floats per row of a score tile in LDS
constexpr int HST = HT * SST + 16;   // floats per head of a score array (== 16 mod 32: see the reads in phase 2)

__device__ __forceinline__ f32x4 mfma4(float a, float b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

struct HmArgs {
    int B, H, N, causal;
    float scale;
};

// XT: staging tiles per wave (1, or one per head of the wave where K tiles are staged a phase early)
template <int H, int D, int XT, int HW, int ARRS = 2> struct HmLds {
    static constexpr int WST = H + 4;                       // floats per row of W
    static constexpr int XST = D * 2 + 32;                  // bytes per row of a staged bf16 tile
    static constexpr int arr_bytes = H * HST * 4;           // one score array
    static constexpr int s_off = 0;                         // S (forward: then P in place)
    static constexpr int p_off = s_off + arr_bytes;         // backward: P, then dZ, then dS
    static constexpr int w_off = s_off + ARRS * arr_bytes;   // (the forward has no second array)
    static constexpr int x_off = w_off + H * WST * 4;       // per-wave staging tiles
    static constexpr int stat_off = x_off + HW * XT * HT * XST;  // three [H][16] float arrays
    static constexpr int total = stat_off + 3 * H * HT * 4;
};

// 8 consecutive bf16 of row `row` at column `col`; zeros for rows outside [0, N)
template <int D>
__device__ __forceinline__ bf16x8 row_frag(const bf16_t *__restrict__ base, int row, int N, int col) {
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (row >= 0 && row < N) raw = *reinterpret_cast<const u32x4 *>(base + (size_t)row * D + col);
    return __builtin_bit_cast(bf16x8, raw);
}

// C[16 x 16] (lane (g, n): rows 4g .. 4g+3, column n) = X Y^T for two row-major bf16 matrices in global
// memory: rows x0 + n of X against rows y0 + n of Y; the operands of the bf16 MFMA are the rows as
// they lie in memory (lane (g, n): 8 consecutive columns at 32 blk + 8 g).
template <int D>
__device__ __forceinline__ f32x4 rows_times_rows(const bf16_t *__restrict__ X, int x0, const bf16_t *__restrict__ Y,
                                                 int y0, int N, int g, int n) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int blk = 0; blk < D / 32; ++blk)
        acc = mfma_bf16(row_frag<D>(X, x0 + n, N, blk * 32 + 8 * g), row_frag<D>(Y, y0 + n, N, blk * 32 + 8 * g), acc);
    return acc;
}

// The same in two steps, for loads issued a tile ahead of their use: the row fragments of a 16-row tile ...
template <int D>
__device__ __forceinline__ void load_frags(bf16x8 (&f)[D / 32], const bf16_t *__restrict__ X, int x0, int N, int g, int n) {
#pragma unroll
    for (int blk = 0; blk < D / 32; ++blk) f[blk] = row_frag<D>(X, x0 + n, N, blk * 32 + 8 * g);
}
template <int D>
__device__ __forceinline__ f32x4 frags_dot(const bf16x8 (&x)[D / 32], const bf16x8 (&y)[D / 32]) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int blk = 0; blk < D / 32; ++blk) acc = mfma_bf16(x[blk], y[blk], acc);
    return acc;
}
// ... and the 16-byte chunks of 16 rows that a lane stages (chunk c of the tile: row c / (D / 8))
template <int D>
__device__ __forceinline__ void load_chunks(u32x4 (&r)[(HT * D / 8 + 63) / 64], const bf16_t *__restrict__ base, int r0,
                                            int N, int lane) {
    constexpr int CPR = D / 8;
#pragma unroll
    for (int i = 0; i < (HT * CPR + 63) / 64; ++i) {
        const int c = lane + i * 64, row = c / CPR, cc = c % CPR;
        r[i] = (u32x4){0u, 0u, 0u, 0u};
        if (c < HT * CPR && r0 + row >= 0 && r0 + row < N)
            r[i] = *reinterpret_cast<const u32x4 *>(base + (size_t)(r0 + row) * D + cc * 8);
    }
}
template <int D>
__device__ __forceinline__ void stage_chunks(unsigned char *xt, int xst, const u32x4 (&r)[(HT * D / 8 + 63) / 64], int lane) {
    constexpr int CPR = D / 8;
#pragma unroll
    for (int i = 0; i < (HT * CPR + 63) / 64; ++i) {
        const int c = lane + i * 64, row = c / CPR, cc = c % CPR;
        if (c < HT * CPR) *reinterpret_cast<u32x4 *>(xt + row * xst + cc * 16) = r[i];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Rows r0 .. r0+15 of a [N][D] bf16 matrix into this wave's staging tile (zeros outside [0, N)).
template <int D>
__device__ __forceinline__ void stage_rows(unsigned char *xt, int xst, const bf16_t *__restrict__ base, int r0, int N,
                                           int lane) {
    constexpr int CPR = D / 8;
#pragma unroll
    for (int c = lane; c < HT * CPR; c += 64) {
        const int row = c / CPR, cc = c % CPR;
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (r0 + row >= 0 && r0 + row < N) raw = *reinterpret_cast<const u32x4 *>(base + (size_t)(r0 + row) * D + cc * 8);
        *reinterpret_cast<u32x4 *>(xt + row * xst + cc * 16) = raw;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// acc[db] (lane (g, n): tile row 4g .. 4g+3, head-dim column 16 db + n) += A X, with A a 16 x 16 fp32 tile
// in LDS (element (m, k) at a[m * a_rs + k * a_cs]; rounded to bf16 here) and X this wave's staged
// 16-row bf16 tile, read with transpose reads (lane (g, n): rows 4g .. 4g+3 of column 16 db + n).
template <int D>
__device__ __forceinline__ void tile_times_staged(f32x4 (&acc)[D / 16], const float *a, int a_rs, int a_cs,
                                                  const unsigned char *xt, int xst, int g, int n) {
    bf16x4 av;
#pragma unroll
    for (int e = 0; e < 4; ++e) av[e] = (bf16_t)a[n * a_rs + (4 * g + e) * a_cs];
#pragma unroll
    for (int db = 0; db < D / 16; ++db)
        acc[db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, av),
                                                             __builtin_bit_cast(short4_t, lds_read_tr4x16(xt, xst, 4 * g, db * 16, n)),
                                                             acc[db], 0, 0, 0);
}

// Max / sum over the 16 lanes of a lane group (all of them get the result, bit for bit: at every step the
// lanes are paired the same way from either side).  Rotations of the row of 16 by 8, 4, 2 and 1 lanes as DPP
// moves: vector-ALU speed, where a shuffle through the LDS crossbar costs its latency eight times in a row.
template <int ROR> __device__ __forceinline__ float row16_rot(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x120 + ROR, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, row16_rot<8>(v));
    v = fmaxf(v, row16_rot<4>(v));
    v = fmaxf(v, row16_rot<2>(v));
    return fmaxf(v, row16_rot<1>(v));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += row16_rot<8>(v);
    v += row16_rot<4>(v);
    v += row16_rot<2>(v);
    return v + row16_rot<1>(v);
}

// Workgroup barrier for data that is exchanged through LDS only: waits for this wave's LDS operations, not for
// its global loads (__syncthreads() drains those too, which would expose the latency of every load that is
// issued ahead of its use at the next barrier).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int H, int HW> __device__ __forceinline__ void load_w(float *Wl, int wst, const float *__restrict__ W, int tid) {
    for (int i = tid; i < H * H; i += HW * 64) Wl[(i / H) * wst + (i % H)] = W[i];
}

// Phase 1: scaled scores of the heads wave, wave + 8, ... for rows i0.. and keys j0.. -> S[h'][i][j]
template <int H, int D, int HW>
__device__ __forceinline__ void scores_phase(float *S, const HmArgs &a, const bf16_t *__restrict__ Qb,
                                             const bf16_t *__restrict__ Kb, int i0, int j0, int wave, int g, int n) {
#pragma unroll
    for (int t = 0; t < H / HW; ++t) {
        const int h = wave + t * HW;
        const f32x4 acc = rows_times_rows<D>(Qb + (size_t)h * a.N * D, i0, Kb + (size_t)h * a.N * D, j0, a.N, g, n);
#pragma unroll
        for (int r = 0; r < 4; ++r) S[h * HST + (4 * g + r) * SST + n] = acc[r] * a.scale;
    }
}

// Z (or its transpose-weighted counterpart) of tile row i for every head: out[hb] (lane (g, n): head
// 16 hb + 4g + r, key n) = sum_k Wt(16 hb + m, k) X[k][i][n], Wt(m, k) = Wl[m * w_rs + k * w_cs].
template <int H>
__device__ __forceinline__ void mix_row(f32x4 (&out)[H / 16], const float *Wl, int w_rs, int w_cs, const float *X,
                                        int i, int g, int n) {
#pragma unroll
    for (int hb = 0; hb < H / 16; ++hb) out[hb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k0 = 0; k0 < H; k0 += 4) {
        const float b = X[(k0 + g) * HST + i * SST + n];
#pragma unroll
        for (int hb = 0; hb < H / 16; ++hb) out[hb] = mfma4(Wl[(hb * 16 + n) * w_rs + (k0 + g) * w_cs], b, out[hb]);
    }
}

// ------------------------------------------------------------------ forward
template <int H, int D, typename TO>
__global__ __launch_bounds__((kHmWaves<H, D, false> * 64)) void headmix_fwd_kernel(HmArgs a, const bf16_t *__restrict__ Q,
                                                              const bf16_t *__restrict__ K, const bf16_t *__restrict__ V,
                                                              const float *__restrict__ W, TO *__restrict__ O,
                                                              float *__restrict__ L, float *__restrict__ M) {
    constexpr int HW = kHmWaves<H, D, false>;
    using Lds = HmLds<H, D, 1, HW, 1>;
    constexpr int DB = D / 16, HPW = H / HW, RPW = HT / HW;  // heads and rows per wave
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *S = reinterpret_cast<float *>(smem + Lds::s_off);
    float *Wl = reinterpret_cast<float *>(smem + Lds::w_off);
    float *al = reinterpret_cast<float *>(smem + Lds::stat_off);   // alpha[h][i], at the end 1 / l
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, n = lane & 15;
    unsigned char *xt = smem + Lds::x_off + wave * HT * Lds::XST;
    const int b = blockIdx.y, i0 = (gridDim.x - 1 - blockIdx.x) * HT;   // longest (causal) tiles first
    const size_t bo = (size_t)b * a.H * a.N * D;
    const bf16_t *Qb = Q + bo, *Kb = K + bo, *Vb = V + bo;

    load_w<H, HW>(Wl, Lds::WST, W, tid);
    f32x4 acc_o[HPW][DB];
#pragma unroll
    for (int t = 0; t < HPW; ++t)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_o[t][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // softmax state of this wave's rows (phase 2): [row][head block][r], the same in the 16 lanes of a group
    float m_run[RPW][H / 16][4], l_run[RPW][H / 16][4];
#pragma unroll
    for (int rl = 0; rl < RPW; ++rl)
#pragma unroll
        for (int hb = 0; hb < H / 16; ++hb)
#pragma unroll
            for (int r = 0; r < 4; ++r) { m_run[rl][hb][r] = kNegInf; l_run[rl][hb][r] = 0.f; }

    // Where the registers allow it the Q fragments of the wave's heads stay resident, the K fragments
    // of a tile are loaded while the tile before it is worked on, and the V rows of a tile are on their
    // way during its score and softmax phases: a workgroup fills its CU alone, so nothing else hides
    // the latency of these loads.  (16 heads only: with 32 heads the softmax state of the mixed rows takes twice
    // the registers, the fragments held ahead went to scratch memory and cost more than they hid: B2 N2048 d64
    // 2.17 ms with them, 1.05 ms without, 0.82 ms with Q alone resident and K as whole rows.)
    constexpr bool AHEAD = HPW * (D / 32) <= 8 && H == 16;
    constexpr bool QRES = !AHEAD;   // the Q fragments alone stay resident
    constexpr int NCH = (HT * D / 8 + 63) / 64;
    // (K rows as whole rows, 1 KB of consecutive memory per load, and from the wave's staging tile into the
    // fragments: a fragment load straight from memory takes 64 bytes of each of 16 rows, half of every cache line
    // it touches, and the vector memory pipe of the CU, which a workgroup's loads pass one after the other, is what
    // the score phase waits for)
    bf16x8 qf[(AHEAD || QRES) ? HPW : 1][D / 32];
    u32x4 kr[AHEAD ? HPW : 1][NCH], vr[AHEAD ? HPW : 1][NCH];
    if constexpr (AHEAD) {
#pragma unroll
        for (int t = 0; t < HPW; ++t) {
            load_frags<D>(qf[t], Qb + (size_t)(wave + t * HW) * a.N * D, i0, a.N, g, n);
            load_chunks<D>(kr[t], Kb + (size_t)(wave + t * HW) * a.N * D, 0, a.N, lane);
        }
    }
    if constexpr (QRES) {
#pragma unroll
        for (int t = 0; t < HPW; ++t) load_frags<D>(qf[t], Qb + (size_t)(wave + t * HW) * a.N * D, i0, a.N, g, n);
    }

    const int j_end = a.causal ? min(a.N, i0 + HT) : a.N;
    for (int j0 = 0; j0 < j_end; j0 += HT) {
        lds_barrier();   // the last tile's P has been used (and, first, W is in place)
        if constexpr (AHEAD) {
            // (the products first: they wait for the K fragments, which were asked for a tile ago; a wait placed
            // after this tile's loads would be for those as well)
            f32x4 sc[HPW];
#pragma unroll
            for (int t = 0; t < HPW; ++t) {
                stage_chunks<D>(xt, Lds::XST, kr[t], lane);
                bf16x8 kf[D / 32];
#pragma unroll
                for (int blk = 0; blk < D / 32; ++blk)
                    kf[blk] = *reinterpret_cast<const bf16x8 *>(xt + n * Lds::XST + (blk * 32 + 8 * g) * 2);
                sc[t] = frags_dot<D>(qf[t], kf);
                __builtin_amdgcn_wave_barrier();
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < HPW; ++t) {
                const int h = wave + t * HW;
                load_chunks<D>(kr[t], Kb + (size_t)h * a.N * D, j0 + HT, a.N, lane);
#pragma unroll
                for (int r = 0; r < 4; ++r) S[h * HST + (4 * g + r) * SST + n] = sc[t][r] * a.scale;
            }
        } else if constexpr (QRES) {
#pragma unroll
            for (int t = 0; t < HPW; ++t) {
                const int h = wave + t * HW;
                // (K as whole rows through the wave's staging tile, as above)
                bf16x8 kf[D / 32];
                {
                    u32x4 kc[NCH];
                    load_chunks<D>(kc, Kb + (size_t)h * a.N * D, j0, a.N, lane);
                    stage_chunks<D>(xt, Lds::XST, kc, lane);
#pragma unroll
                    for (int blk = 0; blk < D / 32; ++blk)
                        kf[blk] = *reinterpret_cast<const bf16x8 *>(xt + n * Lds::XST + (blk * 32 + 8 * g) * 2);
                    __builtin_amdgcn_wave_barrier();
                }
                const f32x4 acc = frags_dot<D>(qf[t], kf);
#pragma unroll
                for (int r = 0; r < 4; ++r) S[h * HST + (4 * g + r) * SST + n] = acc[r] * a.scale;
            }
        } else {
            scores_phase<H, D, HW>(S, a, Qb, Kb, i0, j0, wave, g, n);
        }
        lds_barrier();
        // (the V rows of the tile are asked for here rather than with the K fragments: the vector memory pipe of
        // the CU takes a workgroup's loads one after the other, and this phase has no other use for it)
        if constexpr (AHEAD) {
#pragma unroll
            for (int t = 0; t < HPW; ++t) load_chunks<D>(vr[t], Vb + (size_t)(wave + t * HW) * a.N * D, j0, a.N, lane);
        }
#pragma unroll
        for (int rl = 0; rl < RPW; ++rl) {
            const int i = wave * RPW + rl;
            f32x4 z[H / 16];
            mix_row<H>(z, Wl, Lds::WST, 1, S, i, g, n);
            const bool visible = j0 + n < a.N && !(a.causal && j0 + n > i0 + i);
#pragma unroll
            for (int hb = 0; hb < H / 16; ++hb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float zv = visible ? z[hb][r] : kNegInf;
                    const float m_old = m_run[rl][hb][r];
                    const float m_new = fmaxf(m_old, row16_max(zv));
                    const float pv = m_new == kNegInf ? 0.f : __expf(zv - m_new);
                    const float alpha = m_old == kNegInf ? 0.f : __expf(m_old - m_new);
                    l_run[rl][hb][r] = l_run[rl][hb][r] * alpha + row16_sum(pv);
                    m_run[rl][hb][r] = m_new;
                    const int h = hb * 16 + 4 * g + r;
                    S[h * HST + i * SST + n] = pv;   // P in place: this wave alone reads and writes row i
                    if (n == 0) al[h * HT + i] = alpha;
                }
        }
        lds_barrier();
#pragma unroll
        for (int t = 0; t < HPW; ++t) {
            const int h = wave + t * HW;
            if constexpr (AHEAD) stage_chunks<D>(xt, Lds::XST, vr[t], lane);
            else stage_rows<D>(xt, Lds::XST, Vb + (size_t)h * a.N * D, j0, a.N, lane);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float alpha = al[h * HT + 4 * g + r];
#pragma unroll
                for (int db = 0; db < DB; ++db) acc_o[t][db][r] *= alpha;
            }
            tile_times_staged<D>(acc_o[t], S + h * HST, SST, 1, xt, Lds::XST, g, n);
            __builtin_amdgcn_wave_barrier();
        }
    }
    // row sums and maxima from the row waves to the head waves
    __syncthreads();
    float *lf = al, *mf = al + H * HT;
#pragma unroll
    for (int rl = 0; rl < RPW; ++rl)
#pragma unroll
        for (int hb = 0; hb < H / 16; ++hb)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (n == 0) {
                    const int h = hb * 16 + 4 * g + r, i = wave * RPW + rl;
                    lf[h * HT + i] = l_run[rl][hb][r];
                    mf[h * HT + i] = m_run[rl][hb][r];
                }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < HPW; ++t) {
        const int h = wave + t * HW;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = i0 + 4 * g + r;
            if (i < a.N) {
                const float inv = 1.f / lf[h * HT + 4 * g + r];
                TO *orow = O + bo + ((size_t)h * a.N + i) * D;
#pragma unroll
                for (int db = 0; db < DB; ++db) orow[db * 16 + n] = from_f32<TO>(acc_o[t][db][r] * inv);
            }
        }
    }
    for (int idx = tid; idx < H * HT; idx += HW * 64) {
        const int h = idx / HT, i = i0 + idx % HT;
        if (i < a.N) {
            L[((size_t)b * a.H + h) * a.N + i] = lf[idx];
            M[((size_t)b * a.H + h) * a.N + i] = mf[idx];
        }
    }
}

template <int H, int D, int WHAT> constexpr bool bwd_ahead() {
    constexpr int HW = kHmWaves<H, D, true>;
    return WHAT == 0 && (H / HW) * (D / 32) <= 8 && HmLds<H, D, H / HW, HW>::total <= 160 * 1024;
}
// dK + dV, where LDS allows three staging tiles per wave: the Q and dO tiles of the products with dS^T
// and P^T are staged from the row fragments that the score and dP products load anyway, and the
// fragments of two heads are loaded before the first of them is used.
template <int H, int D, int WHAT> constexpr bool bwd_frag_staging() {
    return WHAT == 1 && HmLds<H, D, 3, kHmWaves<H, D, true>>::total <= 160 * 1024;
}
template <int D>
__device__ __forceinline__ void stage_frags(unsigned char *xt, int xst, const bf16x8 (&f)[D / 32], int g, int n) {
#pragma unroll
    for (int blk = 0; blk < D / 32; ++blk)
        *reinterpret_cast<u32x4 *>(xt + n * xst + (blk * 32 + 8 * g) * 2) = __builtin_bit_cast(u32x4, f[blk]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// ----------------------------------------------------------------- backward
// WHAT = 0: dQ and the dW partial of a row tile (grid: row tiles x batch);
// WHAT = 1: dK and dV of 16 heads (blockIdx.z) of a key tile (grid: key tiles x batch x H / 16).
template <int H, int D, int WHAT>
__global__ __launch_bounds__((kHmWaves<H, D, true> * 64)) void headmix_bwd_kernel(HmArgs a, const bf16_t *__restrict__ Q,
                                                              const bf16_t *__restrict__ K, const bf16_t *__restrict__ V,
                                                              const float *__restrict__ W, const bf16_t *__restrict__ dO,
                                                              const float *__restrict__ LSE, const float *__restrict__ Dl,
                                                              float *__restrict__ out0, float *__restrict__ out1) {
    constexpr int HW = kHmWaves<H, D, true>;
    constexpr int DB = D / 16, HPW = H / HW, RPW = HT / HW, HB = H / 16;
    constexpr int OPW = 16 / HW;   // WHAT = 1: heads of this workgroup's 16 that a wave accumulates for
    constexpr int PU = HPW >= 2 ? 2 : 1;   // heads whose fragments are loaded before the first of them is used
    // dQ + dW, where registers and LDS allow: the Q / dO fragments of the wave's heads stay resident, the
    // K / V fragments of a key tile are loaded while the tile before it is worked on, dP is taken in the
    // score phase and the K tile is staged for the last phase from the fragments (no second load).
    constexpr bool AHEAD = bwd_ahead<H, D, WHAT>();
    constexpr bool FSTAGE = bwd_frag_staging<H, D, WHAT>();
    constexpr int XTILES = AHEAD ? HPW : (FSTAGE ? 3 : 1);   // FSTAGE: tile 0 = dO of the head at hand, 1 + x = Q of output head x
    using Lds = HmLds<H, D, XTILES, HW>;
    // (where loads are issued a tile ahead of their use the barriers must not wait for them; the other instances
    // measured faster with the full barrier)
    auto tile_barrier = [] {
        if constexpr (AHEAD || FSTAGE) lds_barrier();
        else __syncthreads();
    };
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    float *S = reinterpret_cast<float *>(smem + Lds::s_off);
    float *P = reinterpret_cast<float *>(smem + Lds::p_off);
    float *Wl = reinterpret_cast<float *>(smem + Lds::w_off);
    float *lse_s = reinterpret_cast<float *>(smem + Lds::stat_off), *d_s = lse_s + H * HT;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, g = lane >> 4, n = lane & 15;
    unsigned char *xt = smem + Lds::x_off + wave * XTILES * HT * Lds::XST;
    const int b = blockIdx.y, hs = blockIdx.z;
    const size_t bo = (size_t)b * a.H * a.N * D;
    const bf16_t *Qb = Q + bo, *Kb = K + bo, *Vb = V + bo, *Gb = dO + bo;
    const int fixed0 = (WHAT == 0 ? gridDim.x - 1 - blockIdx.x : blockIdx.x) * HT;   // own row tile (0) or key tile (1)

    load_w<H, HW>(Wl, Lds::WST, W, tid);
    constexpr int NACC = WHAT == 0 ? HPW : 2 * OPW;
    f32x4 acc[NACC][DB];   // WHAT 0: dQ of the wave's heads; WHAT 1: dK then dV of its output heads
#pragma unroll
    for (int t = 0; t < NACC; ++t)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[t][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    f32x4 acc_w[HB][HB];
#pragma unroll
    for (int x = 0; x < HB; ++x)
#pragma unroll
        for (int y = 0; y < HB; ++y) acc_w[x][y] = (f32x4){0.f, 0.f, 0.f, 0.f};

    auto load_stats = [&](int i0) {
        for (int idx = tid; idx < H * HT; idx += HW * 64) {
            const int h = idx / HT, i = i0 + idx % HT;
            const size_t at = ((size_t)b * a.H + h) * a.N + i;
            lse_s[idx] = i < a.N ? LSE[at] : 0.f;
            d_s[idx] = i < a.N ? Dl[at] : 0.f;
        }
    };
    if (WHAT == 0) load_stats(fixed0);
    constexpr int NF = AHEAD ? HPW : 1;
    bf16x8 qf[NF][D / 32], gf[NF][D / 32], kf[NF][D / 32], vf[NF][D / 32];
    if constexpr (AHEAD) {
#pragma unroll
        for (int t = 0; t < HPW; ++t) {
            const size_t ho = (size_t)(wave + t * HW) * a.N * D;
            load_frags<D>(qf[t], Qb + ho, fixed0, a.N, g, n);
            load_frags<D>(gf[t], Gb + ho, fixed0, a.N, g, n);
            load_frags<D>(kf[t], Kb + ho, 0, a.N, g, n);
            load_frags<D>(vf[t], Vb + ho, 0, a.N, g, n);
        }
    }

    // the other axis: keys up to the diagonal (dQ) or rows from the diagonal on (dK / dV)
    const int lo = WHAT == 0 ? 0 : (a.causal ? fixed0 : 0);
    const int hi = WHAT == 0 ? (a.causal ? min(a.N, fixed0 + HT) : a.N) : a.N;
    // dK + dV with fragment staging: the fragments of the first pair of heads are asked for two phases before
    // their products (Q / K of the next row tile during the last two phases of this one, dO / V during the
    // probability phase), in the registers that the other pair of fragment sets has just left
    constexpr int NPF = FSTAGE ? PU : 1;
    bf16x8 pq[NPF][D / 32], pk[NPF][D / 32], pg[NPF][D / 32], pv[NPF][D / 32];
    auto prefetch_qk = [&](int i0n) {
        if constexpr (FSTAGE) {
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                const size_t ho = (size_t)(wave + u * HW) * a.N * D;
                load_frags<D>(pq[u], Qb + ho, i0n, a.N, g, n);
                load_frags<D>(pk[u], Kb + ho, fixed0, a.N, g, n);
            }
        }
    };
    auto prefetch_gv = [&](int i0n) {
        if constexpr (FSTAGE) {
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                const size_t ho = (size_t)(wave + u * HW) * a.N * D;
                load_frags<D>(pg[u], Gb + ho, i0n, a.N, g, n);
                load_frags<D>(pv[u], Vb + ho, fixed0, a.N, g, n);
            }
        }
    };
    prefetch_qk(lo);
    for (int o0 = lo; o0 < hi; o0 += HT) {
        const int i0 = WHAT == 0 ? fixed0 : o0, j0 = WHAT == 0 ? o0 : fixed0;
        tile_barrier();   // the last tile's dS has been used (and, first, W and the statistics are in place)
        if (WHAT == 1) load_stats(i0);
        f32x4 dp_early[NF];
        if constexpr (AHEAD) {
#pragma unroll
            for (int t = 0; t < HPW; ++t) {
                const int h = wave + t * HW;
                const f32x4 sc = frags_dot<D>(qf[t], kf[t]);
#pragma unroll
                for (int r = 0; r < 4; ++r) S[h * HST + (4 * g + r) * SST + n] = sc[r] * a.scale;
                dp_early[t] = frags_dot<D>(gf[t], vf[t]);
                // the K rows of the tile, as the fragments hold them, for dQ += dS K
                stage_frags<D>(xt + t * HT * Lds::XST, Lds::XST, kf[t], g, n);
                if (o0 + HT < hi) {
                    load_frags<D>(kf[t], Kb + (size_t)h * a.N * D, j0 + HT, a.N, g, n);
                    load_frags<D>(vf[t], Vb + (size_t)h * a.N * D, j0 + HT, a.N, g, n);
                }
            }
        } else if constexpr (FSTAGE) {
#pragma unroll
            for (int t0 = 0; t0 < HPW; t0 += PU) {
                bf16x8 xq[PU][D / 32], xk[PU][D / 32];
#pragma unroll
                for (int u = 0; u < PU; ++u) {
                    if (t0 == 0) {
#pragma unroll
                        for (int blk = 0; blk < D / 32; ++blk) { xq[u][blk] = pq[u][blk]; xk[u][blk] = pk[u][blk]; }
                    } else {
                        const size_t ho = (size_t)(wave + (t0 + u) * HW) * a.N * D;
                        load_frags<D>(xq[u], Qb + ho, i0, a.N, g, n);
                        load_frags<D>(xk[u], Kb + ho, j0, a.N, g, n);
                    }
                }
#pragma unroll
                for (int u = 0; u < PU; ++u) {
                    const int t = t0 + u, h = wave + t * HW;
                    const f32x4 sc = frags_dot<D>(xq[u], xk[u]);
#pragma unroll
                    for (int r = 0; r < 4; ++r) S[h * HST + (4 * g + r) * SST + n] = sc[r] * a.scale;
                    if (h / 16 == hs) stage_frags<D>(xt + (1 + t % OPW) * HT * Lds::XST, Lds::XST, xq[u], g, n);
                }
            }
        } else {
            scores_phase<H, D, HW>(S, a, Qb, Kb, i0, j0, wave, g, n);
        }
        tile_barrier();
        prefetch_gv(i0);
        // ---- P = exp(Z - LSE), rows of this wave ----
#pragma unroll
        for (int rl = 0; rl < RPW; ++rl) {
            const int i = wave * RPW + rl;
            f32x4 z[HB];
            mix_row<H>(z, Wl, Lds::WST, 1, S, i, g, n);
            const bool visible = i0 + i < a.N && j0 + n < a.N && !(a.causal && j0 + n > i0 + i);
#pragma unroll
            for (int hb = 0; hb < HB; ++hb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int h = hb * 16 + 4 * g + r;
                    P[h * HST + i * SST + n] = visible ? __expf(z[hb][r] - lse_s[h * HT + i]) : 0.f;
                }
        }
        tile_barrier();
        // ---- heads of this wave: dP = dO V^T, (dV += P^T dO), dZ = P (dP - D) in place of P ----
        if constexpr (FSTAGE) {
#pragma unroll
            for (int t0 = 0; t0 < HPW; t0 += PU) {
                bf16x8 xg[PU][D / 32], xv[PU][D / 32];
#pragma unroll
                for (int u = 0; u < PU; ++u) {
                    if (t0 == 0) {
#pragma unroll
                        for (int blk = 0; blk < D / 32; ++blk) { xg[u][blk] = pg[u][blk]; xv[u][blk] = pv[u][blk]; }
                    } else {
                        const size_t ho = (size_t)(wave + (t0 + u) * HW) * a.N * D;
                        load_frags<D>(xg[u], Gb + ho, i0, a.N, g, n);
                        load_frags<D>(xv[u], Vb + ho, j0, a.N, g, n);
                    }
                }
#pragma unroll
                for (int u = 0; u < PU; ++u) {
                    const int t = t0 + u, h = wave + t * HW;
                    const f32x4 dp = frags_dot<D>(xg[u], xv[u]);
                    if (h / 16 == hs) {
                        stage_frags<D>(xt, Lds::XST, xg[u], g, n);
                        tile_times_staged<D>(acc[OPW + (t % OPW)], P + h * HST, 1, SST, xt, Lds::XST, g, n);
                        __builtin_amdgcn_wave_barrier();
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        float *pp = P + h * HST + (4 * g + r) * SST + n;
                        *pp = *pp * (dp[r] - d_s[h * HT + 4 * g + r]);
                    }
                }
            }
        } else {
#pragma unroll
        for (int t = 0; t < HPW; ++t) {
            const int h = wave + t * HW;
            f32x4 dp;
            if constexpr (AHEAD) dp = dp_early[t];
            else dp = rows_times_rows<D>(Gb + (size_t)h * a.N * D, i0, Vb + (size_t)h * a.N * D, j0, a.N, g, n);
            if constexpr (WHAT == 1) {
                // heads wave + 8t of the half hs: t = 2 hs, 2 hs + 1 (H = 32) or t = 0, 1 (H = 16)
                if (h / 16 == hs) {
                    stage_rows<D>(xt, Lds::XST, Gb + (size_t)h * a.N * D, i0, a.N, lane);
                    // dV[j][:] += sum_i P[i][j] dO[i][:]: A(m = j, k = i)
                    tile_times_staged<D>(acc[OPW + (t % OPW)], P + h * HST, 1, SST, xt, Lds::XST, g, n);
                    __builtin_amdgcn_wave_barrier();
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float *pp = P + h * HST + (4 * g + r) * SST + n;
                *pp = *pp * (dp[r] - d_s[h * HT + 4 * g + r]);
            }
        }
        }
        tile_barrier();
        // (unconditionally, past the last row too, where the loads are switched off lane by lane: fragments that
        // may or may not be replaced here would have to stay in their registers through the whole tile)
        if constexpr (WHAT == 1) prefetch_qk(o0 + HT);
        // ---- rows of this wave: dW += dZ S^T over its elements, then dS = scale W^T dZ in place ----
#pragma unroll
        for (int rl = 0; rl < RPW; ++rl) {
            const int i = wave * RPW + rl;
            if constexpr (WHAT == 0) {
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int x = 0; x < HB; ++x) {
                        const float av = P[(x * 16 + n) * HST + i * SST + 4 * s + g];
#pragma unroll
                        for (int y = 0; y < HB; ++y)
                            acc_w[x][y] = mfma4(av, S[(y * 16 + n) * HST + i * SST + 4 * s + g], acc_w[x][y]);
                    }
            }
            f32x4 ds[HB];
            mix_row<H>(ds, Wl, 1, Lds::WST, P, i, g, n);   // W^T: element (m = h', k = h) is W[h][h']
#pragma unroll
            for (int hb = 0; hb < HB; ++hb)
#pragma unroll
                for (int r = 0; r < 4; ++r) P[(hb * 16 + 4 * g + r) * HST + i * SST + n] = ds[hb][r] * a.scale;
        }
        tile_barrier();
        // ---- heads of this wave: dQ += dS K, or dK += dS^T Q ----
        if constexpr (WHAT == 0) {
#pragma unroll
            for (int t = 0; t < HPW; ++t) {
                const int h = wave + t * HW;
                if constexpr (AHEAD) {
                    tile_times_staged<D>(acc[t], P + h * HST, SST, 1, xt + t * HT * Lds::XST, Lds::XST, g, n);
                } else {
                    stage_rows<D>(xt, Lds::XST, Kb + (size_t)h * a.N * D, j0, a.N, lane);
                    tile_times_staged<D>(acc[t], P + h * HST, SST, 1, xt, Lds::XST, g, n);
                    __builtin_amdgcn_wave_barrier();
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < HPW; ++t) {
                const int h = wave + t * HW;
                if (h / 16 == hs) {
                    if constexpr (FSTAGE) {
                        tile_times_staged<D>(acc[t % OPW], P + h * HST, 1, SST, xt + (1 + t % OPW) * HT * Lds::XST, Lds::XST, g, n);
                    } else {
                        stage_rows<D>(xt, Lds::XST, Qb + (size_t)h * a.N * D, i0, a.N, lane);
                        tile_times_staged<D>(acc[t % OPW], P + h * HST, 1, SST, xt, Lds::XST, g, n);
                        __builtin_amdgcn_wave_barrier();
                    }
                }
            }
        }
    }

    // ---- stores: lane (g, n) holds tile rows 4g .. 4g+3 at head-dim columns 16 db + n ----
    if constexpr (WHAT == 0) {
#pragma unroll
        for (int t = 0; t < HPW; ++t) {
            const int h = wave + t * HW;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = fixed0 + 4 * g + r;
                if (i < a.N) {
                    float *row = out0 + bo + ((size_t)h * a.N + i) * D;
#pragma unroll
                    for (int db = 0; db < DB; ++db) row[db * 16 + n] = acc[t][db][r];
                }
            }
        }
        // dW partial of the workgroup: the eight waves' accumulators added in wave order
        __syncthreads();
        float *red = S;   // [wave][h][h']
#pragma unroll
        for (int x = 0; x < HB; ++x)
#pragma unroll
            for (int y = 0; y < HB; ++y)
#pragma unroll
                for (int r = 0; r < 4; ++r) red[(wave * H + x * 16 + 4 * g + r) * H + y * 16 + n] = acc_w[x][y][r];
        __syncthreads();
        float *part = out1 + ((size_t)b * gridDim.x + blockIdx.x) * H * H;
        for (int idx = tid; idx < H * H; idx += HW * 64) {
            float s = 0.f;
#pragma unroll
            for (int w8 = 0; w8 < HW; ++w8) s += red[w8 * H * H + idx];
            part[idx] = s;
        }
    } else {
#pragma unroll
        for (int t = 0; t < HPW; ++t) {
            const int h = wave + t * HW;
            if (h / 16 != hs) continue;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = fixed0 + 4 * g + r;
                if (j < a.N) {
                    float *krow = out0 + bo + ((size_t)h * a.N + j) * D, *vrow = out1 + bo + ((size_t)h * a.N + j) * D;
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        krow[db * 16 + n] = acc[t % OPW][db][r];
                        vrow[db * 16 + n] = acc[OPW + (t % OPW)][db][r];
                    }
                }
            }
        }
    }
}

// dW[h][h'] = sum of the partials in a fixed order: a workgroup takes 64 entries (lane = entry), wave w
// adds the partials w, w + 4, ... in four independent chains, the waves' sums are added in wave order.
__global__ __launch_bounds__(256) void headmix_dw_reduce_kernel(int n_part, int hh, const float *__restrict__ part,
                                                                float *__restrict__ dW) {
    __shared__ float red[4][64];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, idx = blockIdx.x * 64 + lane;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (idx < hh) {
        int q = wave;
        for (; q + 12 < n_part; q += 16) {
#pragma unroll
            for (int c = 0; c < 4; ++c) s[c] += part[(size_t)(q + 4 * c) * hh + idx];
        }
        for (int c = 0; q < n_part; q += 4, ++c) s[c] += part[(size_t)q * hh + idx];
    }
    red[wave][lane] = (s[0] + s[1]) + (s[2] + s[3]);
    __syncthreads();
    if (wave == 0 && idx < hh) dW[idx] = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
}

template <int H, int D>
hipError_t launch_fwd(const HmArgs &a, int out_dt, const void *q, const void *k, const void *v, const float *w, void *o,
                      float *l, float *m, hipStream_t s) {
    constexpr int HW = kHmWaves<H, D, false>, lds = HmLds<H, D, 1, HW, 1>::total;
    static_assert(lds <= 160 * 1024, "LDS budget");
    dim3 grid((a.N + HT - 1) / HT, a.B);
    if (out_dt == CONVATTN_BF16) {
        hipError_t e = set_max_lds_once<headmix_fwd_kernel<H, D, bf16_t>>(lds);
        if (e != hipSuccess) return e;
        headmix_fwd_kernel<H, D, bf16_t><<<grid, HW * 64, lds, s>>>(a, (const bf16_t *)q, (const bf16_t *)k,
                                                                     (const bf16_t *)v, w, (bf16_t *)o, l, m);
    } else {
        hipError_t e = set_max_lds_once<headmix_fwd_kernel<H, D, float>>(lds);
        if (e != hipSuccess) return e;
        headmix_fwd_kernel<H, D, float><<<grid, HW * 64, lds, s>>>(a, (const bf16_t *)q, (const bf16_t *)k,
                                                                   (const bf16_t *)v, w, (float *)o, l, m);
    }
    return hipGetLastError();
}

template <int H, int D, int WHAT>
hipError_t launch_bwd(const HmArgs &a, const void *q, const void *k, const void *v, const float *w, const void *d_o,
                      const float *lse, const float *Dl, float *out0, float *out1, hipStream_t s) {
    constexpr int HW = kHmWaves<H, D, true>;
    constexpr int lds = HmLds<H, D, bwd_ahead<H, D, WHAT>() ? H / HW : (bwd_frag_staging<H, D, WHAT>() ? 3 : 1), HW>::total;
    static_assert(lds <= 160 * 1024, "LDS budget");
    static_assert(HW * H * H * 4 <= HmLds<H, D, 1, HW>::arr_bytes, "room for the dW accumulators of the waves");
    hipError_t e = set_max_lds_once<headmix_bwd_kernel<H, D, WHAT>>(lds);
    if (e != hipSuccess) return e;
    dim3 grid((a.N + HT - 1) / HT, a.B, WHAT == 1 ? H / 16 : 1);
    headmix_bwd_kernel<H, D, WHAT><<<grid, HW * 64, lds, s>>>(a, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v,
                                                              w, (const bf16_t *)d_o, lse, Dl, out0, out1);
    return hipGetLastError();
}

#define HM_DISPATCH(CALL)                                    \
    do {                                                     \
        if (a.H == 16 && d == 32) return CALL(16, 32);       \
        if (a.H == 16 && d == 64) return CALL(16, 64);       \
        if (a.H == 16 && d == 128) return CALL(16, 128);     \
        if (a.H == 32 && d == 32) return CALL(32, 32);       \
        if (a.H == 32 && d == 64) return CALL(32, 64);       \
        if (a.H == 32 && d == 128) return CALL(32, 128);     \
        return hipErrorInvalidValue;                         \
    } while (0)

}  // namespace

hipError_t headmix_fwd(int B, int H, int N, int d, float scale, int causal, int out_dt, const void *q, const void *k,
                       const void *v, const float *w, void *o, float *l, float *m, hipStream_t s) {
    const HmArgs a{B, H, N, causal, scale};
#define CALL(HH, DD) launch_fwd<HH, DD>(a, out_dt, q, k, v, w, o, l, m, s)
    HM_DISPATCH(CALL);
#undef CALL
}

hipError_t headmix_bwd_dq_dw(int B, int H, int N, int d, float scale, int causal, const void *q, const void *k,
                             const void *v, const float *w, const void *d_o, const float *lse, const float *Dl, float *dq,
                             float *dw_part, float *dw, hipStream_t s) {
    const HmArgs a{B, H, N, causal, scale};
    hipError_t e = [&]() -> hipError_t {
#define CALL(HH, DD) launch_bwd<HH, DD, 0>(a, q, k, v, w, d_o, lse, Dl, dq, dw_part, s)
        HM_DISPATCH(CALL);
#undef CALL
    }();
    if (e != hipSuccess) return e;
    const int n_part = B * ((N + HT - 1) / HT), hh = H * H;
    headmix_dw_reduce_kernel<<<(hh + 63) / 64, 256, 0, s>>>(n_part, hh, dw_part, dw);
    return hipGetLastError();
}

hipError_t headmix_bwd_dkdv(int B, int H, int N, int d, float scale, int causal, const void *q, const void *k,
                            const void *v, const float *w, const void *d_o, const float *lse, const float *Dl, float *dk,
                            float *dv, hipStream_t s) {
    const HmArgs a{B, H, N, causal, scale};
#define CALL(HH, DD) launch_bwd<HH, DD, 1>(a, q, k, v, w, d_o, lse, Dl, dk, dv, s)
    HM_DISPATCH(CALL);
#undef CALL
}

int headmix_row_tiles(int N) { return (N + HT - 1) / HT; }

}  // namespace convattn
