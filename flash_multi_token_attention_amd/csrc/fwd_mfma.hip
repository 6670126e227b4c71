// Training forward of conv-attention on bf16 MFMA (gfx950), scores staged in LDS: the kernel for
// windows of 7 to 11 query taps (narrower ones: fwd_reg_mfma.hip).
//
// Workgroup = 4 waves = 128 query rows of one (batch, head); wave w owns rows
// i0 + 32w .. +31 and keeps their O^T accumulators, running max and partial row
// sums in registers for the whole key loop.  Per 64-key tile:
//   1. all waves stage K rows j0-8 .. j0+71 and V rows j0 .. j0+63 row-major in
//      LDS: every thread first issues all of its 128-bit global loads, then
//      waits once and writes them out;
//   2. each wave computes the raw products S^T = K Q^T for its 32 rows plus the
//      16 rows above them (the query halo of the window), applies the causal
//      pre-mask (zero) and writes the tile to its private LDS region as fp16
//      (the softmax scale and log2 e live in the Toeplitz bands instead);
//   3. convolution: per tap one Toeplitz MFMA per 16x16 block reads the fp16 tile
//      back with the tap's row shift (see mfma_common.hpp); the 8 blocks of the
//      wave form 8 independent accumulation chains;
//   4. post-mask (-inf), online softmax per query column of C^T (4 registers x
//      4 lane groups per row: two cross-lane steps for the max, sums stay
//      per-lane until the end); O is rescaled only when some row's max moved;
//   5. O^T += V^T P^T: V^T fragments come from the row-major V tile through the
//      LDS transpose read, P^T straight from the softmax registers (the MFMA k
//      index is permuted: k = 8g+e <-> key 4g+e of block 0 for e < 4, of block 1
//      for e >= 4), so nothing is transposed or shuffled in between.
// LDS fragment reads are issued one stage ahead of the MFMAs that consume them.
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

template <int D> struct FwdLds {
    static constexpr int KST = D * 2 + 16;  // bytes per K / V row (== 16 mod 256 for D = 128)
    static constexpr int k_bytes = SK * KST;
    static constexpr int v_bytes = BK * KST;
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
    constexpr int NKB = SK / 16; // score key blocks per tile (5)
    constexpr int K_CH = SK * CPR, V_CH = BK * CPR;          // 16-byte chunks per tile
    constexpr int K_LD = (K_CH + NW * 64 - 1) / (NW * 64);   // chunks per thread
    constexpr int V_LD = (V_CH + NW * 64 - 1) / (NW * 64);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char *Ks = smem;
    unsigned char *Vs = smem + Lds::k_bytes;

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    unsigned char *Ss = smem + Lds::k_bytes + Lds::v_bytes + wave * (SR * SST);

    // x = head, y = batch, z = query tile: the dispatcher hands out every (batch, head) of the
    // longest (causal) tiles first, so the tail of the launch is made of short tiles
    const int h = blockIdx.x, b = blockIdx.y;
    const int qt = gridDim.z - 1 - blockIdx.z;
    const int i0 = qt * BQ, i0w = i0 + wave * WR;
    const int pk = p.pk, cq = p.c_q;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *Vb = V + bh * p.Nk * D;

    // Toeplitz bands of this head, one fragment per tap slot, pre-multiplied by
    // scale * log2(e): the convolved scores come out in log2 units.
    f16x8 tf[CQT];
    load_bands<CQT>(tf, W + (size_t)h * cq * p.c_k, cq, p.c_k, pk, g, n, false, p.scale * kLog2e);

    // Q^T fragments (B operand): rows i0w-16 .. i0w+31, resident for the whole loop.
    bf16x8 qf[3][KS];
#pragma unroll
    for (int rb = 0; rb < 3; ++rb)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qf[rb][ks] = __builtin_bit_cast(bf16x8, load_row16_nb<D>(Qb, i0w - QH + rb * 16 + n, p.Nq, ks * 32 + g * 8));

    f32x4 acc_o[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc_o[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m_run[2] = {kNegInf, kNegInf};  // running max, in log2 units
    float l_run[2] = {0.f, 0.f};          // this lane's share of the row sum

    // Staging registers: every thread holds its 16-byte chunks of the next K / V tile.
    u32x4 kr[K_LD], vr[V_LD];
    auto load_tile = [&](int j0) {
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = min(tid + i * NW * 64, K_CH - 1), row = c / CPR, cc = c % CPR;
            kr[i] = load_row16_clamped<D>(Kb, j0 - kKeyHalo + row, p.Nk, cc * 8);
        }
#pragma unroll
        for (int i = 0; i < V_LD; ++i) {
            const int c = min(tid + i * NW * 64, V_CH - 1), row = c / CPR, cc = c % CPR;
            vr[i] = load_row16_clamped<D>(Vb, j0 + row, p.Nk, cc * 8);
        }
    };

    // One tile of the wave; `edge` = the tile touches the diagonal or the end of the keys
    // (wave-uniform), only then are the masks evaluated.
    auto tile = [&](int j0, bool edge, bool skip, bool more) {
        if (skip) {
            if (more) load_tile(j0 + BK);
            return;
        }
        // ---- S^T = K Q^T (raw), pre-mask, fp16 -> LDS; K fragments one block ahead ----
        {
            bf16x8 kf[2][KS];
            f32x4 acc[3];
            auto load_kf = [&](int buf, int kb) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    kf[buf][ks] = *reinterpret_cast<const bf16x8 *>(Ks + (kb * 16 + n) * KST + (ks * 32 + g * 8) * 2);
            };
            auto store_s = [&](int kb) {
                const int key0 = j0 - kKeyHalo + kb * 16 + 4 * g;
#pragma unroll
                for (int rb = 0; rb < 3; ++rb) {
                    const int qpos = i0w - QH + rb * 16 + n;
                    f16x4 hv;
                    if (edge && causal) {
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (key0 + r > qpos) acc[rb][r] = 0.f;
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        hv[r] = (_Float16)__builtin_amdgcn_fmed3f(acc[rb][r], -kF16Max, kF16Max);
                    *reinterpret_cast<f16x4 *>(Ss + (rb * 16 + n) * SST + (kb * 16 + 4 * g) * 2) = hv;
                }
            };
            load_kf(0, 0);
            SCHED_DS_READ(KS);
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
                const int cur = kb & 1;
                if (kb + 1 < NKB) {
                    load_kf(cur ^ 1, kb + 1);
                    SCHED_DS_READ(KS);
                }
#pragma unroll
                for (int rb = 0; rb < 3; ++rb) acc[rb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int rb = 0; rb < 3; ++rb) acc[rb] = mfma_bf16(kf[cur][ks], qf[rb][ks], acc[rb]);
                SCHED_MFMA(3 * KS);
                store_s(kb);
            }
        }
        __builtin_amdgcn_wave_barrier();

        // ---- convolution: 8 chains C^T[ob][kb] += T_a^T * S^T(rows shifted by the tap) ----
        f32x4 c[2][BK / 16];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb) c[ob][kb] = (f32x4){0.f, 0.f, 0.f, 0.f};
        {
            // stage st = (tap slot, row block, key-block pair): 2 fragments, read one stage ahead
            constexpr int NST = 4 * CQT;
            f16x8 sf[2][2];
            auto load_sf = [&](int buf, int st) {
                const int a = st >> 2, ob = (st >> 1) & 1, kh = st & 1;
                const unsigned char *base = Ss + (QH + ob * 16 + n - (CQT - 1) + a) * SST + (kh * 32 + 8 * g) * 2;
                sf[buf][0] = *reinterpret_cast<const f16x8 *>(base);
                sf[buf][1] = *reinterpret_cast<const f16x8 *>(base + 32);
            };
            load_sf(0, 0);
            SCHED_DS_READ(2);
#pragma unroll
            for (int st = 0; st < NST; ++st) {
                if (st + 1 < NST) {
                    load_sf((st + 1) & 1, st + 1);
                    SCHED_DS_READ(2);
                }
                const int a = st >> 2, ob = (st >> 1) & 1, kh = st & 1;
                c[ob][2 * kh] = mfma_f16(tf[a], sf[st & 1][0], c[ob][2 * kh]);
                c[ob][2 * kh + 1] = mfma_f16(tf[a], sf[st & 1][1], c[ob][2 * kh + 1]);
                SCHED_MFMA(2);
            }
        }
        // next tile's K / V: in flight during the softmax and the P.V products
        if (more) load_tile(j0 + BK);
        // ---- post-mask and online softmax (log2 domain) ----
        float alpha[2];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob) {
            const int qpos = i0w + ob * 16 + n;
            if (edge) {
#pragma unroll
                for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = j0 + kb * 16 + 4 * g + r;
                        if (key >= p.Nk || (causal && key > qpos)) c[ob][kb][r] = kNegInf;
                    }
            }
            float mx = kNegInf;
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) mx = fmaxf(mx, c[ob][kb][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
            mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
            const float m_new = fmaxf(m_run[ob], mx);
            // rows with nothing visible yet keep m = -inf; use 0 as the exponent base there
            const float m_use = (m_new == kNegInf) ? 0.f : m_new;
            alpha[ob] = fast_exp2(m_run[ob] - m_use);
            m_run[ob] = m_new;
            float psum = 0.f;
#pragma unroll
            for (int kb = 0; kb < BK / 16; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float e = fast_exp2(c[ob][kb][r] - m_use);
                    c[ob][kb][r] = e;
                    psum += e;
                }
            l_run[ob] = l_run[ob] * alpha[ob] + psum;
        }
        if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.f || alpha[1] != 1.f) != 0) {
#pragma unroll
            for (int ob = 0; ob < 2; ++ob)
#pragma unroll
                for (int db = 0; db < DB; ++db) acc_o[ob][db] *= alpha[ob];
        }
        // ---- O^T += V^T P^T ----
        bf16x8 pf[2][BK / 32];
#pragma unroll
        for (int ob = 0; ob < 2; ++ob)
#pragma unroll
            for (int kp = 0; kp < BK / 32; ++kp)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    pf[ob][kp][r] = (bf16_t)c[ob][2 * kp][r];
                    pf[ob][kp][4 + r] = (bf16_t)c[ob][2 * kp + 1][r];
                }
        {
            bf16x8 vf[2];
            auto load_vf = [&](int buf, int st) {  // stage st = (key pair, head-dim block)
                const int kp = st / DB, db = st % DB;
                bf16x4 lo = lds_read_tr4x16(Vs, KST, kp * 32 + 4 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Vs, KST, kp * 32 + 16 + 4 * g, db * 16, n);
                vf[buf] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            };
            load_vf(0, 0);
            SCHED_DS_READ(2);
#pragma unroll
            for (int st = 0; st < (BK / 32) * DB; ++st) {
                if (st + 1 < (BK / 32) * DB) {
                    load_vf((st + 1) & 1, st + 1);
                    SCHED_DS_READ(2);
                }
                const int kp = st / DB, db = st % DB;
#pragma unroll
                for (int ob = 0; ob < 2; ++ob) acc_o[ob][db] = mfma_bf16(vf[st & 1], pf[ob][kp], acc_o[ob][db]);
                SCHED_MFMA(2);
            }
        }
    };

    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    load_tile(0);
    for (int j0 = 0; j0 < k_end; j0 += BK) {
        __syncthreads();
        // ---- K and V of this tile were loaded during the previous one: write them to LDS ----
        if (j0 == 0 || j0 + BK + kKeyHalo > p.Nk) {  // rows outside the sequence count as zeros
#pragma unroll
            for (int i = 0; i < K_LD; ++i) {
                const int kr_row = j0 - kKeyHalo + (tid + i * NW * 64) / CPR;
                kr[i] = zero_unless(kr_row >= 0 && kr_row < p.Nk, kr[i]);
            }
#pragma unroll
            for (int i = 0; i < V_LD; ++i) vr[i] = zero_unless(j0 + (tid + i * NW * 64) / CPR < p.Nk, vr[i]);
        }
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            if (c < K_CH) *reinterpret_cast<u32x4 *>(Ks + row * KST + cc * 16) = kr[i];
        }
#pragma unroll
        for (int i = 0; i < V_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            if (c < V_CH) *reinterpret_cast<u32x4 *>(Vs + row * KST + cc * 16) = vr[i];
        }
        __syncthreads();
        const bool skip = causal && j0 > i0w + WR - 1;  // every key of the tile is after this wave's rows
        const bool edge = (causal && j0 + BK + kKeyHalo > i0w - QH) || (j0 + BK > p.Nk);
        tile(j0, edge, skip, j0 + BK < k_end);
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
    dim3 grid(p.H, p.B, (p.Nq + BQ - 1) / BQ);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k, (const bf16_t *)v, w,
                                    (TO *)o, m, l);
    return hipGetLastError();
}

template <int D, typename TO>
hipError_t pick_cq(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                   void *o, float *m, float *l, hipStream_t s) {
    return launch_fwd<D, 11, TO>(p, q, k, v, w, o, m, l, s);
}

}  // namespace

hipError_t mfma_fwd(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                    const float *w, void *o, float *m, float *l, hipStream_t s) {
    // (its buffer descriptors count bytes in 32 bits)
    if (p.c_q <= kMfmaFwdRegMaxCq && (size_t)p.Nk * p.d * 2 < (1ull << 31))
        return mfma_fwd_reg(p, out_dt, q, k, v, w, o, m, l, s);
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return pick_cq<128, bf16_t>(p, q, k, v, w, o, m, l, s);
        return pick_cq<128, float>(p, q, k, v, w, o, m, l, s);
    }
    if (out_dt == CONVATTN_BF16) return pick_cq<64, bf16_t>(p, q, k, v, w, o, m, l, s);
    return pick_cq<64, float>(p, q, k, v, w, o, m, l, s);
}

}  // namespace convattn
