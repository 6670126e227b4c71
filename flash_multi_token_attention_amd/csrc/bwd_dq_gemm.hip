// dQ = dS K on bf16 MFMA (gfx950), second step of the one-pass backward.
//
// dS comes from the fused dK/dV kernel as bf16 blocks [key tile of 32][row tile of 64] of
// [32 keys][64 rows in the producer's order, see ds_row_of_pos] (the softmax scale is already in it).  Workgroup = 4 waves = 128 query
// rows of one (batch, head); wave w owns rows i0 + 32w .. +31 and all D columns.  Per step of
// 64 keys the workgroup stages the K rows (row-major) and the four dS blocks (as [key][128
// rows]) in LDS; both MFMA operands are LDS transpose reads with the keys as the k index:
//   dQ^T[d][row] += K^T[d][key] dS^T[key][row]
// Two LDS buffers, one barrier per step, the global loads of the next two steps in flight during
// the MFMAs (two register sets, the step loop unrolled by two).  Blocks the fused kernel never wrote (key tile entirely after the row tile under the
// causal mask, or past the last key) are not used: zeros are staged in their place.
#include "mfma_common.hpp"

namespace convattn {
namespace {

constexpr int NW = 4;
constexpr int BQ = 128;   // rows per workgroup
constexpr int BKS = 64;   // keys per step
constexpr int TST = BQ * 2 + 16;  // bytes per key of the staged dS^T tile

template <int D> struct GemmLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int k_bytes = BKS * RST;
    static constexpr int t_bytes = BKS * TST;
    static constexpr int total = 2 * (k_bytes + t_bytes);
};

template <int D, typename TO>
__global__ __launch_bounds__(NW * 64) void dq_from_ds_kernel(Problem p, const bf16_t *__restrict__ K,
                                                             const bf16_t *__restrict__ dS_ws,
                                                             const float *__restrict__ Dl, int n_kt,
                                                             int n_rt, TO *__restrict__ dQ) {
    using Lds = GemmLds<D>;
    constexpr int RST = Lds::RST;
    constexpr int DB = D / 16, CPR = D / 8;
    constexpr int K_CH = BKS * CPR;                 // 16-byte chunks of a K step
    constexpr int K_LD = K_CH / (NW * 64);          // 4 (D = 128) or 2 (D = 64)
    constexpr int BLK = kDsKeys * kDsRows;          // elements per dS block
    static_assert(BLK * 2 / 16 == NW * 64, "one chunk of a dS block per thread");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    const int h = blockIdx.x, b = blockIdx.y;
    const int qt = gridDim.z - 1 - blockIdx.z;  // longest (causal) row tiles first
    const int i0 = qt * BQ - kDsRowShift, rw = i0 + wave * 32;  // the dS row tiles start 16 rows early
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *ws = dS_ws + bh * n_kt * n_rt * (size_t)BLK;
    // the dS blocks carry the dC scale of their (batch, head): the same power of two, from the same D
    const float dcs_inv = exp2f(-dc_scale_log2_from_d(Dl + bh * p.Nq, p.Nq, tid, NW * 64, reinterpret_cast<float *>(smem)));

    f32x4 acc[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    const int n_steps = (k_end + BKS - 1) / BKS;

    // this thread's chunk of each of the 4 dS blocks of a step: key tid/8, rows 8*(tid%8) .. +7
    const int t_key = tid >> 3, t_ch = tid & 7;
    // two register sets: the loads of steps s+1 and s+2 are in flight while step s is multiplied
    // (one step of MFMAs is shorter than the memory latency)
    u32x4 kr_a[K_LD], tr_a[4], kr_b[K_LD], tr_b[4];
    bool tv_a[4], tv_b[4];
    auto load_step = [&](int s, u32x4 (&kr)[K_LD], u32x4 (&tr)[4], bool (&tv)[4]) {
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            kr[i] = load_row16_clamped<D>(Kb, s * BKS + row, p.Nk, cc * 8);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int kt = s * 2 + (i >> 1), rt = qt * 2 + (i & 1);
            tv[i] = kt * kDsKeys < p.Nk && rt < n_rt &&
                    (!causal || kt * kDsKeys < (rt + 1) * kDsRows - kDsRowShift);  // first key <= last row of the block
            const size_t blk = (size_t)min(kt, n_kt - 1) * n_rt + min(rt, n_rt - 1);
            // every dS block is read once: non-temporal, so that it does not push K out of the caches
            tr[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(ws + blk * BLK + t_key * kDsRows + t_ch * 8));
        }
    };

    // loads past the last step re-read clamped addresses and are never staged
    auto run_step = [&](int s, u32x4 (&kr)[K_LD], u32x4 (&tr)[4], bool (&tv)[4]) {
        unsigned char *Ks = smem + (s & 1) * (Lds::k_bytes + Lds::t_bytes);
        unsigned char *Ts = Ks + Lds::k_bytes;
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            *reinterpret_cast<u32x4 *>(Ks + row * RST + cc * 16) = zero_unless(s * BKS + row < p.Nk, kr[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<u32x4 *>(Ts + ((i >> 1) * kDsKeys + t_key) * TST + ((i & 1) * kDsRows + t_ch * 8) * 2) =
                zero_unless(tv[i], tr[i]);
        __syncthreads();
        load_step(s + 2, kr, tr, tv);
        if (causal && s * BKS > rw + 31) return;  // every key of the step is after the wave's rows

#pragma unroll
        for (int kp = 0; kp < BKS / 32; ++kp) {
            bf16x8 sf[2];
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) {
                bf16x4 lo = lds_read_tr4x16(Ts, TST, kp * 32 + 4 * g, wave * 32 + ob * 16, n);
                bf16x4 hi = lds_read_tr4x16(Ts, TST, kp * 32 + 16 + 4 * g, wave * 32 + ob * 16, n);
                sf[ob] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                bf16x4 lo = lds_read_tr4x16(Ks, RST, kp * 32 + 4 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Ks, RST, kp * 32 + 16 + 4 * g, db * 16, n);
                const bf16x8 kf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int ob = 0; ob < 2; ++ob) acc[ob][db] = mfma_bf16(kf, sf[ob], acc[ob][db]);
            }
        }
    };
    load_step(0, kr_a, tr_a, tv_a);
    load_step(1, kr_b, tr_b, tv_b);
    for (int s = 0; s < n_steps; s += 2) {
        run_step(s, kr_a, tr_a, tv_a);
        if (s + 1 < n_steps) run_step(s + 1, kr_b, tr_b, tv_b);
    }

    // lane = position ob*16+n of the wave's 32 rows in the dS blocks' row order;
    // 4 consecutive head-dim columns per block
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
        const int qpos = rw + ds_row_of_pos(ob * 16 + n);
        if (qpos >= 0 && qpos < p.Nq) {
            TO *orow = dQ + (bh * p.Nq + qpos) * D;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int col = db * 16 + 4 * g;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc[ob][db][r] * dcs_inv);
                    *reinterpret_cast<bf16x4 *>(orow + col) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(orow + col) = acc[ob][db] * dcs_inv;
                }
            }
        }
    }
}

template <int D, typename TO>
hipError_t launch(const Problem &p, const void *k, const void *ds_ws, const float *Dl, void *dq, hipStream_t s) {
    auto kern = dq_from_ds_kernel<D, TO>;
    constexpr int lds = GemmLds<D>::total;
    hipError_t e = set_max_lds_once<dq_from_ds_kernel<D, TO>>(lds);
    if (e != hipSuccess) return e;
    dim3 grid(p.H, p.B, (p.Nq + kDsRowShift + BQ - 1) / BQ);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)k, (const bf16_t *)ds_ws, Dl, mfma_ds_key_tiles(p),
                                    mfma_ds_row_tiles(p), (TO *)dq);
    return hipGetLastError();
}

}  // namespace

hipError_t mfma_dq_from_ds(const Problem &p, int out_dt, const void *k, const void *ds_ws, const float *Dl,
                           void *dq, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return launch<128, bf16_t>(p, k, ds_ws, Dl, dq, s);
        return launch<128, float>(p, k, ds_ws, Dl, dq, s);
    }
    if (out_dt == CONVATTN_BF16) return launch<64, bf16_t>(p, k, ds_ws, Dl, dq, s);
    return launch<64, float>(p, k, ds_ws, Dl, dq, s);
}

}  // namespace convattn
