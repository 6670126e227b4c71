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
// pages named by a block table (PAGED instance: the page numbers of the 80 rows around a 64-key
// iteration are fetched by scalar loads one iteration ahead and handed to the lanes through LDS,
// so the lookups do not sit in the vector-load queue between the K / V loads), and every batch
// entry may have its own number of keys.  With shared KV heads a workgroup takes HG = 2 or 4 query
// heads of one KV head (windows of up to 8 query taps): two heads' tap rows fill one 16-row MFMA
// (rows 0..7 and 8..15), so the K / V stream of the KV head is read once for all of them, and only
// the window, the softmax and P.V are repeated per head.
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

template <int D, bool PAGED, int HG>
__global__ __launch_bounds__(NW * 64) void decode_stream_kernel(
    Problem p, KvArgs kv, const bf16_t *__restrict__ Q, const bf16_t *__restrict__ K,
    const bf16_t *__restrict__ V, const float *__restrict__ W, float *__restrict__ O_part,
    float *__restrict__ M_part, float *__restrict__ L_part) {
    constexpr int KS = D / 32;
    constexpr int CPR = D / 8;       // 16-byte chunks per K/V row
    constexpr int RPI = 64 / CPR;    // V rows one load instruction of the wave covers
    constexpr int VT = IT / RPI;     // V loads per lane per iteration
    constexpr int MG = (HG + 1) / 2;   // 16-row MFMA groups: one head (HG = 1) or two heads each
    __shared__ __attribute__((aligned(16))) float s_strip[NW][MG][16 * SROW];
    __shared__ __attribute__((aligned(16))) float s_p[NW][HG][IT];
    // window weights, one row of 20 floats per tap row: key tap b sits at column 8 - pk + b of the
    // 17 columns around a key (zeros elsewhere), so that the window loop has a fixed trip count
    __shared__ __attribute__((aligned(16))) float s_w[HG][kMaxCq][20];
    __shared__ __attribute__((aligned(16))) float s_o[NW][HG][D];
    __shared__ float s_ml[NW][HG][2];
    __shared__ int s_pid[NW][2][8];   // PAGED: page numbers of the row windows of two iterations

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int g = lane >> 4, n = lane & 15;
    const int sp = blockIdx.x, h = blockIdx.y * HG, b = blockIdx.z;   // h: first query head of the workgroup
    const int cq = p.c_q, ck = p.c_k, pk = p.pk;
    const size_t bh = (size_t)b * p.H + h;
    const int hk = h / kv.group;
    // MFMA row n of a group: tap row_tap of head 2 m + row_head of the workgroup
    const int row_head = HG == 1 ? 0 : (n >> 3), row_tap = HG == 1 ? n : (n & 7);
    const int Nk = kv.seq_lens ? min(max(kv.seq_lens[b], 0), p.Nk) : p.Nk;   // keys of this batch entry
    const bf16_t *Kb = K + (PAGED ? 0 : b * p.kv_bstride) + hk * p.kv_hstride;
    const bf16_t *Vb = V + (PAGED ? 0 : b * p.kv_bstride) + hk * p.kv_hstride;
    // PAGED: the window of a 64-key iteration starting at key w0 (a multiple of 64) is rows
    // w0-8 .. w0+71: at most 6 pages of 16 or more keys.  fetch_pages(w0) reads their numbers with
    // scalar loads (the table is read-only: constant address space) and leaves them in the wave's
    // slot (w0 / 64) & 1; load_row(w0, ...) looks a row's page up there.
#if defined(__HIP_DEVICE_COMPILE__)
    typedef const __attribute__((address_space(4))) int *tbl_ptr_t;
#else
    typedef const int *tbl_ptr_t;
#endif
    tbl_ptr_t tbl = PAGED ? (tbl_ptr_t)(kv.table + (size_t)b * kv.table_stride) : (tbl_ptr_t) nullptr;
    auto fetch_pages = [&](int w0) {
        if constexpr (PAGED) {
            const int first = max(w0 - 8, 0) >> kv.page_shift, last = (Nk - 1) >> kv.page_shift;
            int mine = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int id = tbl[min(first + i, last)];
                mine = lane == i ? id : mine;
            }
            if (lane < 8) s_pid[wave][(w0 >> 6) & 1][lane] = mine;
            asm volatile("" ::: "memory");
            __builtin_amdgcn_wave_barrier();
        }
    };
    // 8 bf16 at column `col` of the row nearest to `row` inside [0, Nk)
    auto load_row = [&](int w0, const bf16_t *base, int row, int col) -> u32x4 {
        const int rr = min(max(row, 0), Nk - 1);
        const bf16_t *src;
        if constexpr (PAGED) {
            const int first = max(w0 - 8, 0) >> kv.page_shift;
            const int page = s_pid[wave][(w0 >> 6) & 1][(rr >> kv.page_shift) - first];
            src = base + (size_t)page * kv.page_stride + (size_t)(rr & ((1 << kv.page_shift) - 1)) * D;
        } else {
            src = base + (size_t)rr * D;
        }
        return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + col));
    };
    for (int i = tid; i < HG * kMaxCq * 20; i += NW * 64) {
        const int hh = i / (kMaxCq * 20), a = i / 20 % kMaxCq, bb = i % 20 - (8 - pk);
        s_w[hh][a][i % 20] = (a < cq && bb >= 0 && bb < ck) ? W[((size_t)(h + hh) * cq + a) * ck + bb] : 0.f;
    }

    // Tap row a reads resident row Nq - c_q + a (zero row if it does not exist).
    bf16x8 qf[MG][KS];
#pragma unroll
    for (int m = 0; m < MG; ++m) {
        const int ri = p.Nq - cq + row_tap, hh = 2 * m + row_head;
        const bool ok = row_tap < cq && ri >= 0 && hh < HG;
        const bf16_t *Qb = Q + (bh + hh) * p.Nq * D;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 raw = {0u, 0u, 0u, 0u};
            if (ok) raw = *reinterpret_cast<const u32x4 *>(Qb + (size_t)ri * D + ks * 32 + g * 8);
            qf[m][ks] = __builtin_bit_cast(bf16x8, raw);
        }
    }
    // Causal variant: tap row a sits at position Nk - c_q + a and sees no later key.
    const int row_pos = p.causal ? Nk - cq + row_tap : 0x7fffffff;

    // Key range of this wave: the split's chunk cut into 4 runs of whole iterations.
    // (PAGED: splits start at multiples of 64 keys, so that an iteration's rows are a fixed window)
    const int chunk = PAGED ? ((Nk + p.n_splits - 1) / p.n_splits + IT - 1) / IT * IT : (Nk + p.n_splits - 1) / p.n_splits;
    const int s_lo = sp * chunk, s_hi = min(Nk, s_lo + chunk);
    const int per_wave = ((chunk + NW - 1) / NW + IT - 1) / IT * IT;
    const int lo = s_lo + wave * per_wave, hi = min(s_hi, lo + per_wave);

    const int cc = lane % CPR, gph = lane / CPR;  // this lane's V column chunk and key phase
    float acc[HG][8], m_run[HG], l_run[HG];
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[hh][e] = 0.f;
        m_run[hh] = kNegInf;
        l_run[hh] = 0.f;
    }
    const float scale = p.scale;
    __syncthreads();  // s_w

    if (lo < hi) {
        fetch_pages(lo);
        // strip columns 0..15 <- scores of keys lo-8 .. lo+7
        {
            f32x4 a4[MG];
#pragma unroll
            for (int m = 0; m < MG; ++m) a4[m] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                // (keys before the first or after the last one score zero: the window's padding)
                const int row = lo - 8 + n;
                u32x4 raw = load_row(lo, Kb, row, ks * 32 + g * 8);
                if (row < 0 || row >= Nk) raw = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
                for (int m = 0; m < MG; ++m) a4[m] = mfma_bf16(__builtin_bit_cast(bf16x8, raw), qf[m][ks], a4[m]);
            }
            if (row_tap < cq) {
#pragma unroll
                for (int m = 0; m < MG; ++m) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int key = lo - 8 + 4 * g + r;
                        a4[m][r] = (key > row_pos) ? 0.f : a4[m][r] * scale;
                    }
                    *reinterpret_cast<f32x4 *>(s_strip[wave][m] + n * SROW + 4 * g) = a4[m];
                }
            }
        }
        // K of the first iteration: keys lo+8 .. lo+71
        u32x4 kreg[4][KS];
#pragma unroll
        for (int blk = 0; blk < 4; ++blk)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kreg[blk][ks] = load_row(lo, Kb, lo + 8 + blk * 16 + n, ks * 32 + g * 8);

        for (int j0 = lo; j0 < hi; j0 += IT) {
            // V of this iteration: keys j0 .. j0+63
            u32x4 vreg[VT];
#pragma unroll
            for (int t = 0; t < VT; ++t) vreg[t] = load_row(j0, Vb, j0 + RPI * t + gph, cc * 8);
            if (j0 + IT < hi) fetch_pages(j0 + IT);   // for the K loads below and the next iteration's V loads

            // scores of keys j0+8 .. j0+71 -> strip columns 16 .. 79
#pragma unroll
            for (int blk = 0; blk < 4; ++blk) {
#pragma unroll
                for (int m = 0; m < MG; ++m) {
                    f32x4 a4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        a4 = mfma_bf16(__builtin_bit_cast(bf16x8, kreg[blk][ks]), qf[m][ks], a4);
                    if (row_tap < cq) {
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
                        *reinterpret_cast<f32x4 *>(s_strip[wave][m] + n * SROW + 16 + blk * 16 + 4 * g) = a4;
                    }
                }
            }
            // K of the next iteration (zeros past the cache end)
            if (j0 + IT < hi) {
#pragma unroll
                for (int blk = 0; blk < 4; ++blk)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        kreg[blk][ks] = load_row(j0 + IT, Kb, j0 + IT + 8 + blk * 16 + n, ks * 32 + g * 8);
            }
            __builtin_amdgcn_wave_barrier();

            // window: lane j -> key j0 + j; strip column of key x is x - (j0 - 8)
            float alpha[HG];
#pragma unroll
            for (int hh = 0; hh < HG; ++hh) {
                // (17 columns around the key whatever c_k is: the reads of a tap row are independent
                // of each other and issued together; with run-time bounds every tap waited for its own)
                float c = 0.f;
                {
                    const float *srow = s_strip[wave][hh >> 1] + (HG == 1 ? 0 : 8 * (hh & 1)) * SROW + lane;
                    for (int a = 0; a < cq; ++a) {
                        float wv[20], sv[17];
#pragma unroll
                        for (int q4 = 0; q4 < 5; ++q4)
                            *reinterpret_cast<f32x4 *>(wv + 4 * q4) = *reinterpret_cast<const f32x4 *>(&s_w[hh][a][4 * q4]);
#pragma unroll
                        for (int bb = 0; bb < 17; ++bb) sv[bb] = srow[bb];
                        float c0 = 0.f, c1 = 0.f;
#pragma unroll
                        for (int bb = 0; bb < 16; bb += 2) { c0 = fmaf(wv[bb], sv[bb], c0); c1 = fmaf(wv[bb + 1], sv[bb + 1], c1); }
                        c += c0 + fmaf(wv[16], sv[16], c1);
                        srow += SROW;
                    }
                }
                if (j0 + lane >= hi) c = kNegInf;
                const float m_new = fmaxf(m_run[hh], wave_max(c));
                const float e = (c == kNegInf) ? 0.f : __expf(c - m_new);
                alpha[hh] = (m_run[hh] == kNegInf) ? 0.f : __expf(m_run[hh] - m_new);
                m_run[hh] = m_new;
                l_run[hh] = l_run[hh] * alpha[hh] + e;
                // hand p to the lanes that own each key's V row: phase-major order
                s_p[wave][hh][(lane % RPI) * VT + lane / RPI] = e;
            }
            __builtin_amdgcn_wave_barrier();
            // carry the last 16 score columns to the front for the next iteration
            if (lane < 16) {
#pragma unroll
                for (int m = 0; m < MG; ++m) {
                    float cv[16];
#pragma unroll
                    for (int a = 0; a < 16; ++a) cv[a] = s_strip[wave][m][a * SROW + IT + lane];
#pragma unroll
                    for (int a = 0; a < 16; ++a) s_strip[wave][m][a * SROW + lane] = cv[a];
                }
            }
#pragma unroll
            for (int hh = 0; hh < HG; ++hh) {
                float pv[VT];
#pragma unroll
                for (int t = 0; t < VT; t += 4) {
                    f32x4 p4 = *reinterpret_cast<const f32x4 *>(&s_p[wave][hh][gph * VT + t]);
                    pv[t] = p4[0]; pv[t + 1] = p4[1]; pv[t + 2] = p4[2]; pv[t + 3] = p4[3];
                }
#pragma unroll
                for (int e8 = 0; e8 < 8; ++e8) acc[hh][e8] *= alpha[hh];
#pragma unroll
                for (int t = 0; t < VT; ++t) {
#pragma unroll
                    for (int w2 = 0; w2 < 4; ++w2) {
                        acc[hh][2 * w2] = fmaf(pv[t], bf16_lo(vreg[t][w2]), acc[hh][2 * w2]);
                        acc[hh][2 * w2 + 1] = fmaf(pv[t], bf16_hi(vreg[t][w2]), acc[hh][2 * w2 + 1]);
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }
        // sum the key phases (lanes with the same column chunk) and the row sums
#pragma unroll
        for (int hh = 0; hh < HG; ++hh) {
#pragma unroll
            for (int o = CPR; o < 64; o <<= 1) {
#pragma unroll
                for (int e8 = 0; e8 < 8; ++e8) acc[hh][e8] += __shfl_xor(acc[hh][e8], o, kWave);
            }
            l_run[hh] = wave_sum(l_run[hh]);
        }
    }

    // merge the 4 waves: o = sum o_w e^{m_w - m}, l = sum l_w e^{m_w - m}
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) {
        if (lane < CPR) {
#pragma unroll
            for (int e8 = 0; e8 < 8; ++e8) s_o[wave][hh][lane * 8 + e8] = acc[hh][e8];
        }
        if (lane == 0) { s_ml[wave][hh][0] = m_run[hh]; s_ml[wave][hh][1] = l_run[hh]; }
    }
    __syncthreads();
#pragma unroll
    for (int hh = 0; hh < HG; ++hh) {
        float m = kNegInf;
#pragma unroll
        for (int w = 0; w < NW; ++w) m = fmaxf(m, s_ml[w][hh][0]);
        const size_t slot = (bh + hh) * p.n_splits + sp;
        if (tid < D) {
            float o = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w)
                if (s_ml[w][hh][0] != kNegInf) o = fmaf(s_o[w][hh][tid], __expf(s_ml[w][hh][0] - m), o);
            O_part[slot * D + tid] = o;
        }
        if (tid == 0) {
            float l = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w)
                if (s_ml[w][hh][0] != kNegInf) l = fmaf(s_ml[w][hh][1], __expf(s_ml[w][hh][0] - m), l);
            M_part[slot] = m;
            L_part[slot] = l;
        }
    }
}

}  // namespace

bool decode_stream_ok(const Problem &p, int in_dt, unsigned flags) {
    return in_dt == CONVATTN_BF16 && !(flags & CONVATTN_FLAG_EXACT) && (p.d == 32 || p.d == 64 || p.d == 128) &&
           p.pk <= 8 && p.c_q <= 16;
}

// Query heads a workgroup takes together: 4 or 2 heads of one KV head when the window's query taps
// fit half an MFMA (8 rows), else 1.
int decode_heads_per_wg(const Problem &p, int group) {
    if (p.c_q > 8) return 1;
    return group % 4 == 0 ? 4 : group % 2 == 0 ? 2 : 1;
}

hipError_t decode_stream_kv(const Problem &p, const KvArgs &kv, const void *q, const void *k, const void *v,
                            const float *w, float *o_part, float *m_part, float *l_part, hipStream_t s) {
    const int hg = decode_heads_per_wg(p, kv.group);
    dim3 grid(p.n_splits, p.H / hg, p.B);
#define CONVATTN_DECODE_LAUNCH(DD, PG, HH)                                                                   \
    decode_stream_kernel<DD, PG, HH><<<grid, NW * 64, 0, s>>>(p, kv, (const bf16_t *)q, (const bf16_t *)k,     \
                                                             (const bf16_t *)v, w, o_part, m_part, l_part)
#define CONVATTN_DECODE_PICK_HG(DD, PG)                                                                      \
    do {                                                                                                     \
        if (hg == 4) CONVATTN_DECODE_LAUNCH(DD, PG, 4);                                                       \
        else if (hg == 2) CONVATTN_DECODE_LAUNCH(DD, PG, 2);                                                  \
        else CONVATTN_DECODE_LAUNCH(DD, PG, 1);                                                               \
    } while (0)
    if (p.d == 128) {
        if (kv.table) CONVATTN_DECODE_PICK_HG(128, true);
        else CONVATTN_DECODE_PICK_HG(128, false);
    } else if (p.d == 32) {
        if (kv.table) CONVATTN_DECODE_PICK_HG(32, true);
        else CONVATTN_DECODE_PICK_HG(32, false);
    } else {
        if (kv.table) CONVATTN_DECODE_PICK_HG(64, true);
        else CONVATTN_DECODE_PICK_HG(64, false);
    }
#undef CONVATTN_DECODE_PICK_HG
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
