// dQ = dS K on bf16 MFMA (gfx950), second step of the one-pass backward of bwd_chain_mfma.hip.
//
// dS comes from the key-stationary kernel as bf16 blocks [key tile of 32][row tile of 32] of
// 32 rows x 32 keys, laid out [row parity][key half][row pair][16 keys] (the order in which that
// kernel's lanes hold it: each of its stores and each load here covers whole 128-byte lines; the
// softmax scale and the dC scale are already in it).  Workgroup
// = 4 waves = 128 query rows of one (batch, head); wave w owns rows i0 + 32w .. +31 and all D
// columns.  The product is dQ^T[d][row] += K^T[d][key] dS^T[key][row]: 16 bytes of a block are 8
// keys of one row, which is the B operand of a lane as it lies in memory, so dS goes from global
// memory straight into the MFMA operand registers (every block is read once, by one wave, in
// whole 1 KB pieces).  Only K passes through LDS (row-major, read with transpose reads), staged
// per step of 64 keys in two buffers with one barrier per step; the loads of the next two steps
// are in flight during the MFMAs.  Blocks the first kernel never wrote (key tile entirely after
// the row tile under the causal mask, or past the last key or row) are not read.
#include "mfma_common.hpp"

namespace convattn {
namespace {

constexpr int NW = 4;
constexpr int BQ = 128;   // rows per workgroup
constexpr int BKS = 64;   // keys per step
constexpr int BLK = kChainKeys * kChainRows;  // elements per dS block

template <int D> struct RowsLds {
    static constexpr int RST = D * 2 + 16;
    static constexpr int k_bytes = BKS * RST;
    static constexpr int total = 2 * k_bytes;
};

template <int D, typename TO>
__global__ __launch_bounds__(NW * 64) void dq_rows_kernel(Problem p, const bf16_t *__restrict__ K,
                                                          const bf16_t *__restrict__ dS_ws,
                                                          const float *__restrict__ dc_scale, int n_kt,
                                                          int n_rt, TO *__restrict__ dQ) {
    using Lds = RowsLds<D>;
    constexpr int RST = Lds::RST;
    constexpr int DB = D / 16, CPR = D / 8;
    constexpr int K_CH = BKS * CPR;                 // 16-byte chunks of a K step
    constexpr int K_LD = K_CH / (NW * 64);          // 4 (D = 128) or 2 (D = 64)
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    const int h = blockIdx.x, b = blockIdx.y;
    const int qt = gridDim.z - 1 - blockIdx.z;  // longest (causal) row tiles first
    const int i0 = qt * BQ, rw = i0 + wave * 32, rt = rw / kChainRows;
    const bool causal = p.causal != 0;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Kb = K + bh * p.Nk * D;
    const bf16_t *ws = dS_ws + bh * (size_t)chain_ds_block_off(causal, n_rt, n_kt) * BLK;

    f32x4 acc[2][DB];
#pragma unroll
    for (int ob = 0; ob < 2; ++ob)
#pragma unroll
        for (int db = 0; db < DB; ++db) acc[ob][db] = (f32x4){0.f, 0.f, 0.f, 0.f};

    const int k_end = causal ? min(p.Nk, i0 + BQ) : p.Nk;
    const int n_steps = (k_end + BKS - 1) / BKS;
    const bool row_ok = rt < n_rt;

    // the dS loads of steps s+1 and s+2 (two register sets) and the K loads of step s+1 (K comes from the
    // L2, which the other row tiles of the head keep it in) are in flight while step s is multiplied
    u32x4 kr[K_LD], sr_a[2][2], sr_b[2][2];
    auto load_k = [&](int s) {
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            kr[i] = load_row16_clamped<D>(Kb, s * BKS + row, p.Nk, cc * 8);
        }
    };
    auto load_ds = [&](int s, u32x4 (&sr)[2][2]) {
#pragma unroll
        for (int kp = 0; kp < 2; ++kp) {
            const int kt = s * 2 + kp;
            // (a block that does not exist: any block that does; the registers are cleared before their use)
            const int rt_c = min(rt, n_rt - 1), kt_c = causal ? min(kt, rt_c) : min(kt, n_kt - 1);
            const size_t blk = (size_t)chain_ds_block_off(causal, n_rt, kt_c) + rt_c - chain_ds_first_rt(causal, kt_c);
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) {
                // every dS block is read once: non-temporal, so that it does not push K out of the caches.
                // Raw: blocks that do not exist are cleared where the registers are used (a select here
                // would wait for the load within this step)
                sr[kp][ob] = __builtin_nontemporal_load(
                    reinterpret_cast<const u32x4 *>(ws + blk * BLK + ((ob * 2 + (g >> 1)) * 16 + n) * 16 + 8 * (g & 1)));
            }
        }
    };

    auto run_step = [&](int s, u32x4 (&sr)[2][2]) {
        unsigned char *Ks = smem + (s & 1) * Lds::k_bytes;
#pragma unroll
        for (int i = 0; i < K_LD; ++i) {
            const int c = tid + i * NW * 64, row = c / CPR, cc = c % CPR;
            *reinterpret_cast<u32x4 *>(Ks + row * RST + cc * 16) = zero_unless(s * BKS + row < p.Nk, kr[i]);
        }
        bf16x8 sf[2][2];
#pragma unroll
        for (int kp = 0; kp < 2; ++kp) {
            const int kt = s * 2 + kp;
            // the block exists when its first key is a key and (causal) not after the tile's last row
            const bool ok = row_ok && kt * kChainKeys < p.Nk && (!causal || kt * kChainKeys <= rw + 31);
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) sf[kp][ob] = __builtin_bit_cast(bf16x8, zero_unless(ok, sr[kp][ob]));
        }
        __syncthreads();
        load_k(s + 1);
        load_ds(s + 2, sr);
        if (causal && s * BKS > rw + 31) return;  // every key of the step is after the wave's rows

#pragma unroll
        for (int kp = 0; kp < BKS / 32; ++kp) {
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                // k slot 8g+e = key 8g+e of the 32-key tile, as in the dS rows
                bf16x4 lo = lds_read_tr4x16(Ks, RST, kp * 32 + 8 * g, db * 16, n);
                bf16x4 hi = lds_read_tr4x16(Ks, RST, kp * 32 + 8 * g + 4, db * 16, n);
                const bf16x8 kf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int ob = 0; ob < 2; ++ob) acc[ob][db] = mfma_bf16(kf, sf[kp][ob], acc[ob][db]);
            }
        }
    };
    load_k(0);
    load_ds(0, sr_a);
    load_ds(1, sr_b);
    for (int s = 0; s < n_steps; s += 2) {
        run_step(s, sr_a);
        if (s + 1 < n_steps) run_step(s + 1, sr_b);
    }

    // lane n of block ob = row 2 n + ob of the wave's 32; 4 consecutive head-dim columns per block
    const float inv = dc_scale ? 1.f / dc_scale[2 * bh] : 1.f;
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
        const int qpos = rw + 2 * n + ob;
        if (qpos < p.Nq) {
            TO *orow = dQ + (bh * p.Nq + qpos) * D;
#pragma unroll
            for (int db = 0; db < DB; ++db) {
                const int col = db * 16 + 4 * g;
                if constexpr (sizeof(TO) == 2) {
                    bf16x4 ov;
#pragma unroll
                    for (int r = 0; r < 4; ++r) ov[r] = (bf16_t)(acc[ob][db][r] * inv);
                    *reinterpret_cast<bf16x4 *>(orow + col) = ov;
                } else {
                    *reinterpret_cast<f32x4 *>(orow + col) = acc[ob][db] * inv;
                }
            }
        }
    }
}

template <int D, typename TO>
hipError_t launch(const Problem &p, const void *k, const void *ds_ws, const float *dc_scale, void *dq,
                  hipStream_t s) {
    auto kern = dq_rows_kernel<D, TO>;
    constexpr int lds = RowsLds<D>::total;
    dim3 grid(p.H, p.B, (p.Nq + BQ - 1) / BQ);
    kern<<<grid, NW * 64, lds, s>>>(p, (const bf16_t *)k, (const bf16_t *)ds_ws, dc_scale, chain_key_tiles(p),
                                    chain_row_tiles(p), (TO *)dq);
    return hipGetLastError();
}

}  // namespace

hipError_t mfma_dq_from_rows(const Problem &p, int out_dt, const void *k, const void *ds_ws, const float *dc_scale,
                           void *dq, hipStream_t s) {
    if (p.d == 128) {
        if (out_dt == CONVATTN_BF16) return launch<128, bf16_t>(p, k, ds_ws, dc_scale, dq, s);
        return launch<128, float>(p, k, ds_ws, dc_scale, dq, s);
    }
    if (p.d == 32) {
        if (out_dt == CONVATTN_BF16) return launch<32, bf16_t>(p, k, ds_ws, dc_scale, dq, s);
        return launch<32, float>(p, k, ds_ws, dc_scale, dq, s);
    }
    if (out_dt == CONVATTN_BF16) return launch<64, bf16_t>(p, k, ds_ws, dc_scale, dq, s);
    return launch<64, float>(p, k, ds_ws, dc_scale, dq, s);
}

}  // namespace convattn
