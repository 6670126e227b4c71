// Decode step of conv-attention as an HBM stream (gfx950).
//
// One output row per (batch, head): c[j] = sum_ab W[a][b] * scale * <q_a, k_{j+b-pk}>
// over the whole KV cache, softmax over j, times V.  K and V are read exactly once
// from HBM, 16 bytes per lane, straight into registers (no LDS staging):
//   * workgroup = 4 waves = one (split, head, batch); each wave walks its own
//     contiguous share of the split's keys, 64 keys per iteration, with no
//     barrier in the loop;
//   * scores of the <= 16 resident query rows against 16 keys are one MFMA chain
//     (K rows are the A operand in the layout the global loads deliver);
//   * the wave keeps an fp32 score strip [tap row][80 keys] in LDS: 16 keys carried
//     over from the previous iteration + 64 new ones, so the +-pad_k key halo costs
//     no second read of K; the window is applied from that strip on the VALU, one
//     key per lane;
//   * online softmax per wave (max by cross-lane butterfly, sums kept per lane);
//   * P.V on the VALU: a lane owns 8 head-dim columns and every (64*8/D)-th key,
//     the key phases are summed across lanes once at the end;
//   * K of the next iteration and V of this one are in flight while the scores,
//     window and softmax of this iteration are computed.
// The 4 waves merge their (m, l, o) in LDS and store one un-normalised partial
// per split; convattn_decode_combine merges the splits.
//
// Where the rows live is a parameter of the kernel (KvArgs): query heads may share KV heads
// (head h reads KV head h / group), the rows of a (batch, KV head) may be contiguous or come in
// pages named by a block table (PAGED instance: one table lookup per row load; the lookups of the
// rows a lane loads next are independent of everything else in the iteration), and every batch
// entry may have its own number of keys.
#include "mfma_common.hpp"

namespace convattn {
namespace {

// Non-temporal loads below: every K / V row is read exactly once, and keeping it out of the
// caches' replacement order is worth 10 % of the stream's bandwidth here.

constexpr int NW = 4;
constexpr int IT = 64;             // keys per wave iteration
constexpr int SW = IT + 16;        // score strip width: 16 carried + 64 new
constexpr int SROW = SW + 4;       // floats per strip row (84)

__device__ __forceinline__ float bf16_lo(unsigned int w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(unsigned int w) { return __uint_as_float(w & 0xffff0000u); }

template <int D, bool PAGED>
__global__ __launch_bounds__(NW * 64) void decode_stream_kernel(
    Problem p, KvArgs kv, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const float *__restrict__ W, float *__restrict__ O_part,
    float *__restrict__ M_part, float *__restrict__ L_part) {
    constexpr int KS = D / 32;
    constexpr int CPR = D / 8;       // 16-byte chunks per K/V row
    constexpr int RPI = 64 / CPR;    // V rows one load instruction of the wave covers
    constexpr int VT = IT / RPI;     // V loads per lane per iteration
    __shared__ __attribute__((aligned(16))) float s_strip[NW][16 * SROW];
    __shared__ __attribute__((aligned(16))) float s_p[NW][IT];
    __shared__ float s_w[kMaxCq * 17];
    __shared__ __attribute__((aligned(16))) float s_o[NW][D];
    __shared__ float s_ml[NW][2];

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    const int sp = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int cq = p.c_q, ck = p.c_k, pk = p.pk;
    const size_t bh = (size_t)b * p.H + h;
    const bf16_t *Qb = Q + bh * p.Nq * D;
    const int hk = h / kv.group;
    const int Nk = kv.seq_lens ? min(max(kv.seq_lens[b], 0), p.Nk) : p.Nk;   // keys of this batch entry
    const bf16_t *Kb = K + (PAGED ? 0 : b * p.kv_bstride) + hk * p.kv_hstride;
    const bf16_t *Vb = V + (PAGED ? 0 : b * p.kv_bstride) + hk * p.kv_hstride;
    const int *tbl = PAGED ? kv.table + (size_t)b * kv.table_stride : nullptr;
    // 8 bf16 at column `col` of the row nearest to `row` inside [0, Nk)
    auto load_row = [&](const bf16_t *base, int row, int col) -> u32x4 {
        const int rr = min(max(row, 0), Nk - 1);
        const bf16_t *src;
        if constexpr (PAGED)
            src = base + (size_t)tbl[rr >> kv.page_shift] * kv.page_stride + (size_t)(rr & ((1 << kv.page_shift) - 1)) * D;
        else
            src = base + (size_t)rr * D;
        return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + col));
    };
    float *strip = s_strip[wave];

    for (int i = tid; i < cq * ck; i += NW * 64) s_w[i] = W[(size_t)h * cq * ck + i];

    // Tap row a reads resident row Nq - c_q + a (zero row if it does not exist).
    bf16x8 qf[KS];
    {
        const int ri = p.Nq - cq + n;
        const bool ok = n < cq && ri >= 0;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 raw = {0u, 0u, 0u, 0u};
            if (ok) raw = *reinterpret_cast<const u32x4 *>(Qb + (size_t)ri * D + ks * 32 + g * 8);
            qf[ks] = __builtin_bit_cast(bf16x8, raw);
        }
    }
    // Causal variant: tap row a sits at position Nk - c_q + a and sees no later key.
    const int row_pos = p.causal ? Nk - cq + n : 0x7fffffff;

    // Key range of this wave: the split's chunk cut into 4 runs of whole iterations.
    const int chunk = (Nk + p.n_splits - 1) / p.n_splits;
    const int s_lo = sp * chunk, s_hi = min(Nk, s_lo + chunk);
    const int per_wave = ((chunk + NW - 1) / NW + IT - 1) / IT * IT;
    const int lo = s_lo + wave * per_wave, hi = min(s_hi, lo + per_wave);

    const int cc = lane % CPR, gph = lane / CPR;  // this lane's V column chunk and key phase
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    float m_run = kNegInf, l_run = 0.f;
    const float scale = p.scale;
    __syncthreads();  // s_w

    if (lo < hi) {
        // strip columns 0..15 <- scores of keys lo-8 .. lo+7
        {
            f32x4 a4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                // (keys before the first or after the last one score zero: the window's padding)
                const int row = lo - 8 + n;
                u32x4 raw = load_row(Kb, row, ks * 32 + g * 8);
                if (row < 0 || row >= Nk) raw = (u32x4){0u, 0u, 0u, 0u};
                a4 = mfma_bf16(__builtin_bit_cast(bf16x8, raw), qf[ks], a4);
            }
            if (n < cq) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = lo - 8 + 4 * g + r;
                    a4[r] = (key > row_pos) ? 0.f : a4[r] * scale;
                }
                *reinterpret_cast<f32x4 *>(strip + n * SROW + 4 * g) = a4;
            }
        }
        // K of the first iteration: keys lo+8 .. lo+71
        u32x4 kreg[4][KS];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kreg[blk][ks] = load_row(Kb, lo + 8 + blk * 16 + n, ks * 32 + g * 8);

        for (int j0 = lo; j0 < hi; j0 += IT) {
            // V of this iteration: keys j0 .. j0+63
            u32x4 vreg[VT];
#pragma unroll
            for (int t = 0; t < VT; ++t) vreg[t] = load_row(Vb, j0 + RPI * t + gph, cc * 8);

            // scores of keys j0+8 .. j0+71 -> strip columns 16 .. 79
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
                f32x4 a4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    a4 = mfma_bf16(__builtin_bit_cast(bf16x8, kreg[blk][ks]), qf[ks], a4);
                if (n < cq) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = j0 + 8 + blk * 16 + 4 * g + r;
                        a4[r] = (key > row_pos) ? 0.f : a4[r] * scale;
                    }
                    if (j0 + IT + 8 > Nk) {  // keys past the end of the cache score zero (K rows were clamped)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (j0 + 8 + blk * 16 + 4 * g + r >= Nk) a4[r] = 0.f;
                    }
                    *reinterpret_cast<f32x4 *>(strip + n * SROW + 16 + blk * 16 + 4 * g) = a4;
                }
            }
            // K of the next iteration (zeros past the cache end)
            if (j0 + IT < hi) {
#pragma unroll
                for (int blk = 0; blk < 4; ++blk)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        kreg[blk][ks] = load_row(Kb, j0 + IT + 8 + blk * 16 + n, ks * 32 + g * 8);
            }
            __builtin_amdgcn_wave_barrier();

            // window: lane j -> key j0 + j; strip column of key x is x - (j0 - 8)
            float c = 0.f;
            {
                const float *srow = strip + lane + 8 - pk;
                for (int a = 0; a < cq; ++a) {
                    const float *wr = s_w + a * ck;
                    for (int bb = 0; bb < ck; ++bb) c = fmaf(wr[bb], srow[bb], c);
                    srow += SROW;
                }
            }
            if (j0 + lane >= hi) c = kNegInf;
            const float m_new = fmaxf(m_run, wave_max(c));
            const float e = (c == kNegInf) ? 0.f : __expf(c - m_new);
            const float alpha = (m_run == kNegInf) ? 0.f : __expf(m_run - m_new);
            m_run = m_new;
            l_run = l_run * alpha + e;
            // hand p to the lanes that own each key's V row: phase-major order
            s_p[wave][(lane % RPI) * VT + lane / RPI] = e;
            __builtin_amdgcn_wave_barrier();
            // carry the last 16 score columns to the front for the next iteration
            if (lane < 16) {
                for (int a = 0; a < cq; ++a) strip[a * SROW + lane] = strip[a * SROW + IT + lane];
            }
            float pv[VT];
#pragma unroll
            for (int t = 0; t < VT; t += 4) {
                f32x4 p4 = *reinterpret_cast<const f32x4 *>(&s_p[wave][gph * VT + t]);
                pv[t] = p4[0]; pv[t + 1] = p4[1]; pv[t + 2] = p4[2]; pv[t + 3] = p4[3];
            }
#pragma unroll
            for (int e8 = 0; e8 < 8; ++e8) acc[e8] *= alpha;
#pragma unroll
            for (int t = 0; t < VT; ++t) {
#pragma unroll
                for (int w2 = 0; w2 < 4; ++w2) {
                    acc[2 * w2] = fmaf(pv[t], bf16_lo(vreg[t][w2]), acc[2 * w2]);
                    acc[2 * w2 + 1] = fmaf(pv[t], bf16_hi(vreg[t][w2]), acc[2 * w2 + 1]);
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        // sum the key phases (lanes with the same column chunk) and the row sums
#pragma unroll
        for (int o = CPR; o < 64; o <<= 1) {
#pragma unroll
            for (int e8 = 0; e8 < 8; ++e8) acc[e8] += __shfl_xor(acc[e8], o, kWave);
        }
        l_run = wave_sum(l_run);
    }

    // merge the 4 waves: o = sum o_w e^{m_w - m}, l = sum l_w e^{m_w - m}
    if (lane < CPR) {
#pragma unroll
        for (int e8 = 0; e8 < 8; ++e8) s_o[wave][lane * 8 + e8] = acc[e8];
    }
    if (lane == 0) { s_ml[wave][0] = m_run; s_ml[wave][1] = l_run; }
    __syncthreads();
    float m = kNegInf;
#pragma unroll
    for (int w = 0; w < NW; ++w) m = fmaxf(m, s_ml[w][0]);
    const size_t slot = bh * p.n_splits + sp;
    if (tid < D) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w)
            if (s_ml[w][0] != kNegInf) o = fmaf(s_o[w][tid], __expf(s_ml[w][0] - m), o);
        O_part[slot * D + tid] = o;
    }
    if (tid == 0) {
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w)
            if (s_ml[w][0] != kNegInf) l = fmaf(s_ml[w][1], __expf(s_ml[w][0] - m), l);
        M_part[slot] = m;
        L_part[slot] = l;
    }
}

}  // namespace

bool decode_stream_ok(const Problem &p, int in_dt, unsigned flags) {
    return in_dt == CONVATTN_BF16 && !(flags & CONVATTN_FLAG_EXACT) && (p.d == 64 || p.d == 128) &&
           p.pk <= 8 && p.c_q <= 16;
}

hipError_t decode_stream_kv(const Problem &p, const KvArgs &kv, const void *q, const void *k, const void *v,
                            const float *w, float *o_part, float *m_part, float *l_part, hipStream_t s) {
    dim3 grid(p.n_splits, p.H, p.B);
#define CONVATTN_DECODE_LAUNCH(DD, PG)                                                                       \
    decode_stream_kernel<DD, PG><<<grid, NW * 64, 0, s>>>(p, kv, (const bf16_t *)q, (const bf16_t *)k,         \
                                                         (const bf16_t *)v, w, o_part, m_part, l_part)
    if (p.d == 128) {
        if (kv.table) CONVATTN_DECODE_LAUNCH(128, true);
        else CONVATTN_DECODE_LAUNCH(128, false);
    } else {
        if (kv.table) CONVATTN_DECODE_LAUNCH(64, true);
        else CONVATTN_DECODE_LAUNCH(64, false);
    }
#undef CONVATTN_DECODE_LAUNCH
    return hipGetLastError();
}

hipError_t decode_stream(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                         float *o_part, float *m_part, float *l_part, hipStream_t s) {
    KvArgs kv = {};
    kv.group = 1;
    return decode_stream_kv(p, kv, q, k, v, w, o_part, m_part, l_part, s);
}

}  // namespace convattn
