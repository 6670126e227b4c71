// fp32-arithmetic conv-attention kernels for gfx950: every supported shape and
// both input types.  These are the "exact" path (CONVATTN_FLAG_EXACT, fp32
// inputs, shapes the bf16 MFMA kernels do not cover): all operands, scores and
// probabilities are fp32.  The dot products (Q K^T, P V, dO V^T, dS K, dS^T Q,
// P^T dO) run on v_mfma_f32_16x16x4_f32 with both operands read from fp32 LDS
// tiles; the convolution, its transpose, dW and the softmax run on the vector
// ALUs.  Accumulators stay in registers for the whole key (or query) loop, and
// nothing is accumulated through HBM or with atomics.
//
// Index conventions (per batch b, head h): query row i, key column j, tap
// (a, b) of W[h] looks at S_m[i + a - pq][j + b - pk].  A workgroup owns
// kGenTR query rows (forward, dQ) or kGenBwdTC keys (dK/dV) and walks the other
// axis in tiles, loading each tile with the halo the window needs.
#include "common.hpp"

namespace convattn {
namespace {

constexpr int TR = kGenTR;
constexpr int NT = 256;  // threads per workgroup
constexpr int NWV = NT / 64;

// dst[r][c] (row stride `stride`) = src[(row0 + r) * d + c], zero outside [0, N): eight elements (d is
// a multiple of 8) per thread and turn.
__device__ __forceinline__ void load8_f32(const float *src, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4 *>(src), b = *reinterpret_cast<const float4 *>(src + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8_f32(const bf16_t *src, float (&v)[8]) {
    const uint4 raw = *reinterpret_cast<const uint4 *>(src);
    const unsigned int w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <typename T>
__device__ __forceinline__ void load_rows(float *dst, int stride, const T *src, int row0, int nrows,
                                          int N, int d) {
    const int cpr = d / 8;
    for (int idx = threadIdx.x; idx < nrows * cpr; idx += NT) {
        const int r = idx / cpr, c = (idx - r * cpr) * 8;
        const int g = row0 + r;
        float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (g >= 0 && g < N) load8_f32(src + (size_t)g * d + c, v);
        float *out = dst + r * stride + c;
        if ((stride & 3) == 0) {
            *reinterpret_cast<float4 *>(out) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(out + 4) = make_float4(v[4], v[5], v[6], v[7]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) out[i] = v[i];
        }
    }
}

// The same in two steps, for tiles that are loaded while the tile before them is worked on: issue()
// starts the loads of this thread's pieces (8 elements each, MAXP pieces at most), commit() converts
// them and writes them to LDS.
template <typename T, int MAXP>
struct RowPieces {
    static constexpr int Q = sizeof(T) == 2 ? 1 : 2;   // 16-byte quantities per piece
    uint4 raw[MAXP * Q];
    __device__ __forceinline__ void issue(const T *src, int row0, int nrows, int N, int d) {
        const int cpr = d / 8;
#pragma unroll
        for (int i = 0; i < MAXP; ++i) {
            const int idx = threadIdx.x + i * NT, r = idx / cpr, c = (idx - r * cpr) * 8, g = row0 + r;
#pragma unroll
            for (int q = 0; q < Q; ++q) raw[i * Q + q] = make_uint4(0u, 0u, 0u, 0u);
            if (idx < nrows * cpr && g >= 0 && g < N) {
                const uint4 *ptr = reinterpret_cast<const uint4 *>(src + (size_t)g * d + c);
#pragma unroll
                for (int q = 0; q < Q; ++q) raw[i * Q + q] = ptr[q];
            }
        }
    }
    __device__ __forceinline__ void commit(float *dst, int stride, int nrows, int d) const {
        const int cpr = d / 8;
#pragma unroll
        for (int i = 0; i < MAXP; ++i) {
            const int idx = threadIdx.x + i * NT, r = idx / cpr, c = (idx - r * cpr) * 8;
            if (idx < nrows * cpr) {
                float4 lo, hi;
                if constexpr (Q == 1) {
                    const unsigned int w[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
                    lo = make_float4(__uint_as_float(w[0] << 16), __uint_as_float(w[0] & 0xffff0000u),
                                     __uint_as_float(w[1] << 16), __uint_as_float(w[1] & 0xffff0000u));
                    hi = make_float4(__uint_as_float(w[2] << 16), __uint_as_float(w[2] & 0xffff0000u),
                                     __uint_as_float(w[3] << 16), __uint_as_float(w[3] & 0xffff0000u));
                } else {
                    lo = make_float4(__uint_as_float(raw[2 * i].x), __uint_as_float(raw[2 * i].y),
                                     __uint_as_float(raw[2 * i].z), __uint_as_float(raw[2 * i].w));
                    hi = make_float4(__uint_as_float(raw[2 * i + 1].x), __uint_as_float(raw[2 * i + 1].y),
                                     __uint_as_float(raw[2 * i + 1].z), __uint_as_float(raw[2 * i + 1].w));
                }
                float *out = dst + r * stride + c;   // (strides of the tiles loaded this way are multiples of 4 floats)
                *reinterpret_cast<float4 *>(out) = lo;
                *reinterpret_cast<float4 *>(out + 4) = hi;
            }
        }
    }
};
constexpr int pieces_per_thread(int rows) { return (rows * (kMaxD / 8) + NT - 1) / NT; }

// S[r][c] = scale * <A[r], Kt[c]> for r < nr, c < nc on the vector ALUs (the decode kernel's few rows);
// the causal pre-mask zeroes keys after the row's own position.
__device__ __forceinline__ void score_tile(float *S, int sstride, const float *A, int astride,
                                           const float *Kt, int kstride, int nr, int nc, int d,
                                           int row_pos0, int col_pos0, float scale, int causal) {
    for (int idx = threadIdx.x; idx < nr * nc; idx += NT) {
        int r = idx / nc, c = idx - r * nc;
        const float *a = A + r * astride;
        const float *k = Kt + c * kstride;
        float acc = 0.f;
        for (int t = 0; t < d; ++t) acc = fmaf(a[t], k[t], acc);
        if (causal && (col_pos0 + c) > (row_pos0 + r)) acc = 0.f;
        S[r * sstride + c] = acc * scale;
    }
}

typedef float f32x4 __attribute__((ext_vector_type(4)));

// Four adjacent outputs of the convolution, out[k] = sum_ab W[a][b] * X[a rows down][k + b columns on],
// with `x` pointing at the window's first element for output 0: one new tile element and one weight
// are read per four multiply-adds, and the four sums are independent.  CK > 0: the number of key taps
// as a constant, so that the reads of a tap row are all issued before its multiply-adds (with a
// run-time bound every few taps wait for their LDS reads).  FLIP: the transposed convolution,
// out[k] = sum_ab W[a][b] * X[a rows UP][k - b columns], `x` at the element under output 0 for tap (0, 0).
template <int CK, bool FLIP>
__device__ __forceinline__ void conv4_impl(float (&out)[4], const float *Ws, int c_q, int c_k, const float *x, int xstride) {
    out[0] = out[1] = out[2] = out[3] = 0.f;
    const int ck = CK > 0 ? CK : c_k;
    for (int a = 0; a < c_q; ++a) {
        const float *row = FLIP ? x - a * xstride : x + a * xstride, *w = Ws + a * ck;
        if constexpr (CK > 0) {
            float seg[CK + 3], wv[CK];
#pragma unroll
            for (int i = 0; i < CK + 3; ++i) seg[i] = FLIP ? row[3 - i] : row[i];   // FLIP: seg[i] = X[.. 3 - i]
#pragma unroll
            for (int bb = 0; bb < CK; ++bb) wv[bb] = w[bb];
#pragma unroll
            for (int bb = 0; bb < CK; ++bb) {
#pragma unroll
                for (int k = 0; k < 4; ++k) out[k] = fmaf(wv[bb], FLIP ? seg[3 - k + bb] : seg[k + bb], out[k]);
            }
        } else if constexpr (!FLIP) {
            float s0 = row[0], s1 = row[1], s2 = row[2];
#pragma unroll 4
            for (int bb = 0; bb < ck; ++bb) {
                const float s3 = row[bb + 3], wv = w[bb];
                out[0] = fmaf(wv, s0, out[0]);
                out[1] = fmaf(wv, s1, out[1]);
                out[2] = fmaf(wv, s2, out[2]);
                out[3] = fmaf(wv, s3, out[3]);
                s0 = s1; s1 = s2; s2 = s3;
            }
        } else {
            float s1 = row[1], s2 = row[2], s3 = row[3];
#pragma unroll 4
            for (int bb = 0; bb < ck; ++bb) {
                const float s0 = row[-bb], wv = w[bb];
                out[0] = fmaf(wv, s0, out[0]);
                out[1] = fmaf(wv, s1, out[1]);
                out[2] = fmaf(wv, s2, out[2]);
                out[3] = fmaf(wv, s3, out[3]);
                s3 = s2; s2 = s1; s1 = s0;
            }
        }
    }
}
template <bool FLIP>
__device__ __forceinline__ void conv4_any(float (&out)[4], const float *Ws, int c_q, int c_k, const float *x, int xstride) {
    switch (c_k) {   // (workgroup-uniform)
        case 3: conv4_impl<3, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        case 5: conv4_impl<5, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        case 7: conv4_impl<7, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        case 9: conv4_impl<9, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        case 11: conv4_impl<11, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        case 13: conv4_impl<13, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        case 15: conv4_impl<15, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
        default: conv4_impl<0, FLIP>(out, Ws, c_q, c_k, x, xstride); break;
    }
}
__device__ __forceinline__ void conv4(float (&out)[4], const float *Ws, int c_q, int c_k, const float *x, int xstride) {
    conv4_any<false>(out, Ws, c_q, c_k, x, xstride);
}
__device__ __forceinline__ void conv4_t(float (&out)[4], const float *Ws, int c_q, int c_k, const float *x, int xstride) {
    conv4_any<true>(out, Ws, c_q, c_k, x, xstride);
}

// NB 16 x 16 blocks at once that share the left operand: acc[u] (lane (g, n): rows 4g .. 4g+3, column n)
// += A B_u over k < K (a multiple of 4), operands fp32 in LDS.  `ap` / `bp[u]` are this lane's operand
// pointers at k = 0 (A: row n at k = g; B: column n at k = g), a_ks / b_ks the strides per unit of k.  Independent accumulators keep the
// matrix pipe busy where one chain of dependent MFMAs would wait for itself.
template <int NB>
__device__ __forceinline__ void lds_mma_n(f32x4 (&acc)[NB], const float *ap, int a_ks, const float *const (&bp)[NB],
                                          int b_ks, int K) {
    for (int k = 0; k < K; k += 4) {
        const float a = ap[k * a_ks];
#pragma unroll
        for (int u = 0; u < NB; ++u) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bp[u][k * b_ks], acc[u], 0, 0, 0);
    }
}

// S[r][c] = scale * <A[r], Kt[c]> for r < nr, c < nc on the matrix cores: a wave takes strips of one
// 16-row block times three 16-column blocks; the causal pre-mask zeroes keys after the row's own position.
__device__ __forceinline__ void score_tile_mma(float *S, int sstride, const float *A, int astride, const float *Kt,
                                               int kstride, int nr, int nc, int d, int row_pos0, int col_pos0,
                                               float scale, int causal) {
    constexpr int CBW = 3;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, g = lane >> 4, n = lane & 15;
    const int nrb = (nr + 15) / 16, ncb = (nc + 15) / 16, ncs = (ncb + CBW - 1) / CBW;
    for (int strip = wave; strip < nrb * ncs; strip += NWV) {
        const int rb = strip / ncs, cb0 = (strip - rb * ncs) * CBW;
        f32x4 acc[CBW];
        const float *bp[CBW];
#pragma unroll
        for (int u = 0; u < CBW; ++u) {
            acc[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
            bp[u] = Kt + min((cb0 + u) * 16 + n, nc - 1) * kstride + g;   // (blocks past the last one repeat it)
        }
        lds_mma_n<CBW>(acc, A + min(rb * 16 + n, nr - 1) * astride + g, 1, bp, 1, d);
#pragma unroll
        for (int u = 0; u < CBW; ++u) {
            const int c = (cb0 + u) * 16 + n;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const int r = rb * 16 + 4 * g + rr;
                if (r < nr && c < nc && cb0 + u < ncb)
                    S[r * sstride + c] = (causal && (col_pos0 + c) > (row_pos0 + r)) ? 0.f : acc[u][rr] * scale;
            }
        }
    }
}

// LDS carve-up of the forward.  Row strides: == 4 mod 32 floats where the 16 lanes of an MFMA operand
// read 16 rows at one column (Q, K), == 16 mod 32 where they read one row at 16 columns and the lane
// groups 4 rows (V as the right-hand side of P V).
struct FwdLds {
    float *Qs, *KVs, *Ss, *Ps, *Ws, *m_s, *l_s, *al_s;
    int qst, kst, vst, sst, pst;
};
__host__ __device__ inline size_t fwd_lds_floats(int d, int pq, int pk, int ntap) {
    const int QR = TR + pq, SC = kGenFwdTC + 2 * pk;
    const size_t kv = (size_t)SC * (d + 4) > (size_t)kGenFwdTC * (d + 16) ? (size_t)SC * (d + 4) : (size_t)kGenFwdTC * (d + 16);
    return (size_t)QR * (d + 4) + kv + (size_t)QR * (SC + 1) + (size_t)TR * (kGenFwdTC + 4) + ntap + 3 * TR;
}
__device__ __forceinline__ FwdLds carve_fwd(float *lds, const Problem &p) {
    FwdLds t;
    const int d = p.d, QR = TR + p.pq, SC = kGenFwdTC + 2 * p.pk;
    t.qst = d + 4; t.kst = d + 4; t.vst = d + 16; t.sst = SC + 1; t.pst = kGenFwdTC + 4;
    const int kv = max(SC * t.kst, kGenFwdTC * t.vst);
    t.Qs = lds;
    t.KVs = t.Qs + QR * t.qst;
    t.Ss = t.KVs + kv;
    t.Ps = t.Ss + QR * t.sst;
    t.Ws = t.Ps + TR * t.pst;
    t.m_s = t.Ws + p.c_q * p.c_k;
    t.l_s = t.m_s + TR;
    t.al_s = t.l_s + TR;
    return t;
}

// ------------------------------------------------------------------ forward
template <typename TI, typename TO>
__global__ __launch_bounds__(NT) void gen_fwd_kernel(Problem p, const TI *__restrict__ Q,
                                                     const TI *__restrict__ K,
                                                     const TI *__restrict__ V,
                                                     const float *__restrict__ W, TO *__restrict__ O,
                                                     float *__restrict__ M, float *__restrict__ L) {
    constexpr int TC = kGenFwdTC;
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
    const int r0 = blockIdx.x * TR;
    const int pq = p.pq, pk = p.pk, d = p.d;
    const int QR = TR + pq, SC = TC + 2 * pk;
    const FwdLds t = carve_fwd(lds, p);
    const int ntap = p.c_q * p.c_k;
    float *Qs = t.Qs, *KVs = t.KVs, *Ss = t.Ss, *Ps = t.Ps, *Ws = t.Ws, *m_s = t.m_s, *l_s = t.l_s, *al_s = t.al_s;
    const int qst = t.qst, kst = t.kst, vst = t.vst, sst = t.sst, pst = t.pst;

    const size_t bh = (size_t)b * p.H + h;
    const TI *Qb = Q + bh * p.Nq * d;
    const TI *Kb = K + bh * p.Nk * d;
    const TI *Vb = V + bh * p.Nk * d;

    load_rows(Qs, qst, Qb, r0 - pq, QR, p.Nq, d);
    for (int i = tid; i < ntap; i += NT) Ws[i] = W[(size_t)h * ntap + i];
    if (tid < TR) { m_s[tid] = kNegInf; l_s[tid] = 0.f; }

    // O: a wave holds the 16 x 16 blocks wave, wave + 4 of the head dimension (lane (g, n): rows 4g .. 4g+3)
    const int wave = tid >> 6, lane = tid & 63, g = lane >> 4, n = lane & 15;
    f32x4 acc[kMaxD / 16 / NWV];
#pragma unroll
    for (int u = 0; u < kMaxD / 16 / NWV; ++u) acc[u] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // The K rows of a tile are loaded during the tile before it, its V rows during its score phase.
    RowPieces<TI, pieces_per_thread(kGenFwdTC + 2 * ((kMaxCk - 1) / 2))> kp;
    RowPieces<TI, pieces_per_thread(kGenFwdTC)> vp;
    const int kend = p.causal ? min(p.Nk, r0 + TR) : p.Nk;
    kp.issue(Kb, -pk, SC, p.Nk, d);
    for (int c0 = 0; c0 < kend; c0 += TC) {
        kp.commit(KVs, kst, SC, d);
        vp.issue(Vb, c0, TC, p.Nk, d);
        __syncthreads();
        score_tile_mma(Ss, sst, Qs, qst, KVs, kst, QR, SC, d, r0 - pq, c0 - pk, p.scale, p.causal);
        __syncthreads();
        vp.commit(KVs, vst, TC, d);  // V replaces K
        if (c0 + TC < kend) kp.issue(Kb, c0 + TC - pk, SC, p.Nk, d);
        for (int idx = tid; idx < TR * TC / 4; idx += NT) {
            const int i = idx / (TC / 4), j = (idx - i * (TC / 4)) * 4;
            float c[4];
            conv4(c, Ws, p.c_q, p.c_k, Ss + i * sst + j, sst);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int qi = r0 + i, kj = c0 + j + k;
                Ps[i * pst + j + k] = (kj < p.Nk && !(p.causal && kj > qi)) ? c[k] : kNegInf;
            }
        }
        __syncthreads();
        {   // online softmax: one wave per 4 rows, one lane per key of the tile
            for (int rr = 0; rr < 4; ++rr) {
                int i = wave * 4 + rr;
                float c = Ps[i * pst + lane];
                float m_old = m_s[i];
                float m_new = fmaxf(m_old, wave_max(c));
                float e = (c == kNegInf) ? 0.f : __expf(c - m_new);
                float sum = wave_sum(e);
                float al = (m_old == kNegInf) ? 0.f : __expf(m_old - m_new);
                Ps[i * pst + lane] = e;
                if (lane == 0) { m_s[i] = m_new; l_s[i] = l_s[i] * al + sum; al_s[i] = al; }
            }
        }
        __syncthreads();
        {
            // P (16 x TC; keys past the end are 0) times V (rows zero-filled past the end); columns past d
            // repeat the last one and are not stored
            const float *bp[kMaxD / 16 / NWV];
#pragma unroll
            for (int u = 0; u < kMaxD / 16 / NWV; ++u) {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) acc[u][rr] *= al_s[4 * g + rr];
                bp[u] = KVs + g * vst + min((wave + NWV * u) * 16 + n, d - 1);
            }
            lds_mma_n<kMaxD / 16 / NWV>(acc, Ps + n * pst + g, 1, bp, vst, TC);
        }
        __syncthreads();
    }
#pragma unroll
    for (int u = 0; u < kMaxD / 16 / NWV; ++u) {
        const int dc = (wave + NWV * u) * 16 + n;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int qi = r0 + 4 * g + rr;
            if (qi < p.Nq && dc < d) O[(bh * p.Nq + qi) * d + dc] = from_f32<TO>(acc[u][rr] / l_s[4 * g + rr]);
        }
    }
    if (tid < TR && r0 + tid < p.Nq) { M[bh * p.Nq + r0 + tid] = m_s[tid]; L[bh * p.Nq + r0 + tid] = l_s[tid]; }
}

// ----------------------------------------------------------------- backward
// LDS carve-up shared by the two backward kernels (row strides as in the forward).
struct BwdLds {
    float *Qs, *dOs, *KVs, *Ss, *dCs, *Ps, *dSs, *Ws, *lse_s, *D_s, *red;
    int qst, gst, kst, kst2, sst, cst, pst;
};
constexpr int kDwRowGroups = 8;   // dW: a work item is one tap over TR / 8 rows of a tile
constexpr int kDwItemsPerThread = (kMaxCq * kMaxCk * kDwRowGroups + NT - 1) / NT;

__host__ __device__ inline size_t bwd_lds_floats(int d, int pq, int pk, int ntap) {
    constexpr int TC = kGenBwdTC;
    const size_t kv = (size_t)(TC + 4 * pk) * (d + 4) > (size_t)TC * (d + 16) ? (size_t)(TC + 4 * pk) * (d + 4)
                                                                               : (size_t)TC * (d + 16);
    return (size_t)(TR + 2 * pq) * (d + 4) + (size_t)(TR + pq) * (d + 4) + kv +
           (size_t)(TR + 2 * pq) * (TC + 4 * pk + 1) + (size_t)(TR + pq) * (TC + 2 * pk + 1) + 2 * (size_t)TR * (TC + 4) +
           ntap + 2 * (TR + pq) + (size_t)kDwRowGroups * ntap;
}

template <int TC>
__device__ __forceinline__ BwdLds carve_bwd(float *lds, const Problem &p) {
    BwdLds t;
    const int d = p.d, pq = p.pq, pk = p.pk, ntap = p.c_q * p.c_k;
    t.qst = d + 4; t.gst = d + 4; t.kst = d + 4; t.kst2 = d + 16;
    t.sst = TC + 4 * pk + 1;
    t.cst = TC + 2 * pk + 1;
    t.pst = TC + 4;
    const int kv = max((TC + 4 * pk) * t.kst, TC * t.kst2);
    t.Qs = lds;
    t.dOs = t.Qs + (TR + 2 * pq) * t.qst;
    t.KVs = t.dOs + (TR + pq) * t.gst;
    t.Ss = t.KVs + kv;
    t.dCs = t.Ss + (TR + 2 * pq) * t.sst;
    t.Ps = t.dCs + (TR + pq) * t.cst;
    t.dSs = t.Ps + TR * t.pst;
    t.Ws = t.dSs + TR * t.pst;
    t.lse_s = t.Ws + ntap;
    t.D_s = t.lse_s + (TR + pq);
    t.red = t.D_s + (TR + pq);   // dW partial sums of the row groups
    return t;
}

// What depends on the query tile: Q rows r0-pq .. r0+TR+pq-1, dO / LSE / D rows r0 .. r0+TR+pq-1
// (TR + pq <= 31 rows: one LSE / D entry per thread), loaded in two steps like the tiles.
template <typename TI>
struct QSide {
    RowPieces<TI, pieces_per_thread(TR + 2 * (kMaxCq - 1))> qp;
    RowPieces<TI, pieces_per_thread(TR + kMaxCq - 1)> gp;
    float ls, dd;
    __device__ __forceinline__ void issue(const Problem &p, const TI *Qb, const TI *dOb, const float *lse, const float *D,
                                          int r0) {
        qp.issue(Qb, r0 - p.pq, TR + 2 * p.pq, p.Nq, p.d);
        gp.issue(dOb, r0, TR + p.pq, p.Nq, p.d);
        const int g = r0 + (int)threadIdx.x;
        ls = 0.f; dd = 0.f;
        if ((int)threadIdx.x < TR + p.pq && g < p.Nq) { ls = lse[g]; dd = D[g]; }
    }
    __device__ __forceinline__ void commit(const BwdLds &t, const Problem &p) const {
        qp.commit(t.Qs, t.qst, TR + 2 * p.pq, p.d);
        gp.commit(t.dOs, t.gst, TR + p.pq, p.d);
        if ((int)threadIdx.x < TR + p.pq) { t.lse_s[threadIdx.x] = ls; t.D_s[threadIdx.x] = dd; }
    }
};

// For query tile r0 and key tile c0 (query side already in LDS) leaves in LDS:
//   Ss  = S_m  rows r0-pq .. r0+TR+pq-1, keys c0-2pk .. c0+TC+2pk-1
//   dCs = dC   rows r0    .. r0+TR+pq-1, keys c0-pk  .. c0+TC+pk-1
//   Ps  = P    rows r0    .. r0+TR-1,    keys c0     .. c0+TC-1
// Ends with a barrier; KVs is free afterwards.  The K rows (c0-2pk .. c0+TC+2pk-1) are on their way in `kp`
// when this is called; the V rows are loaded during the score phase; `after_v` is where the caller starts
// the loads it needs next.
template <typename TI, int TC, typename KP, typename VP, typename Hook>
__device__ __forceinline__ void bwd_tile(const BwdLds &t, const Problem &p, KP &kp, VP &vp, const TI *Vb, int r0, int c0,
                                         Hook &&after_v) {
    const int pq = p.pq, pk = p.pk, d = p.d;
    kp.commit(t.KVs, t.kst, TC + 4 * pk, d);
    vp.issue(Vb, c0 - pk, TC + 2 * pk, p.Nk, d);
    __syncthreads();
    score_tile_mma(t.Ss, t.sst, t.Qs, t.qst, t.KVs, t.kst, TR + 2 * pq, TC + 4 * pk, d, r0 - pq, c0 - 2 * pk,
                   p.scale, p.causal);
    __syncthreads();
    vp.commit(t.KVs, t.kst, TC + 2 * pk, d);
    after_v();
    __syncthreads();
    const int nr = TR + pq, nc = TC + 2 * pk;
    // dP = dO V^T into dCs (scale 1, no mask), then dC = P (dP - D) in place
    score_tile_mma(t.dCs, t.cst, t.dOs, t.gst, t.KVs, t.kst, nr, nc, d, 0, 0, 1.f, 0);
    __syncthreads();
    const int ng = (nc + 3) / 4;   // groups of four adjacent keys per row
    for (int idx = threadIdx.x; idx < nr * ng; idx += NT) {
        const int i = idx / ng, j0 = (idx - i * ng) * 4;
        float c[4];
        conv4(c, t.Ws, p.c_q, p.c_k, t.Ss + i * t.sst + j0, t.sst);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int j = j0 + k, qi = r0 + i, kj = c0 - pk + j;
            if (j < nc) {
                float P = 0.f, dC = 0.f;
                if (qi < p.Nq && kj >= 0 && kj < p.Nk && !(p.causal && kj > qi)) {
                    P = __expf(c[k] - t.lse_s[i]);
                    dC = P * (t.dCs[i * t.cst + j] - t.D_s[i]);
                }
                t.dCs[i * t.cst + j] = dC;
                if (i < TR && j >= pk && j < pk + TC) t.Ps[i * t.pst + j - pk] = P;
            }
        }
    }
    __syncthreads();
}

// dSs[r][c] = sum_ab W[a][b] * dC[r - a + pq][c - b + pk], zero on the causal future.
template <int TC>
__device__ __forceinline__ void dscore_tile(const BwdLds &t, const Problem &p, int r0, int c0) {
    const int pq = p.pq, pk = p.pk;
    for (int idx = threadIdx.x; idx < TR * TC / 4; idx += NT) {
        const int r = idx / (TC / 4), c = (idx - r * (TC / 4)) * 4;
        float s[4];
        conv4_t(s, t.Ws, p.c_q, p.c_k, t.dCs + (r + pq) * t.cst + c + 2 * pk, t.cst);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int qi = r0 + r, kj = c0 + c + k;
            t.dSs[r * t.pst + c + k] = (qi < p.Nq && kj < p.Nk && !(p.causal && kj > qi)) ? s[k] : 0.f;
        }
    }
}

template <typename TI, typename TO>
__global__ __launch_bounds__(NT) void gen_dq_dw_kernel(
    Problem p, const TI *__restrict__ Q, const TI *__restrict__ K, const TI *__restrict__ V,
    const TI *__restrict__ dO, const float *__restrict__ D, const float *__restrict__ LSE,
    const float *__restrict__ W, TO *__restrict__ dQ, float *__restrict__ dW_part) {
    constexpr int TC = kGenBwdTC;
    extern __shared__ float lds[];
    const BwdLds t = carve_bwd<TC>(lds, p);
    const int tid = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z, qt = blockIdx.x;
    const int r0 = qt * TR;
    const int d = p.d, pk = p.pk, ntap = p.c_q * p.c_k;
    const size_t bh = (size_t)b * p.H + h;
    const TI *Qb = Q + bh * p.Nq * d, *dOb = dO + bh * p.Nq * d;
    const TI *Kb = K + bh * p.Nk * d, *Vb = V + bh * p.Nk * d;

    for (int i = tid; i < ntap; i += NT) t.Ws[i] = W[(size_t)h * ntap + i];
    {
        QSide<TI> qs;
        qs.issue(p, Qb, dOb, LSE + bh * p.Nq, D + bh * p.Nq, r0);
        qs.commit(t, p);
    }
    constexpr int PKM = (kMaxCk - 1) / 2;
    RowPieces<TI, pieces_per_thread(TC + 4 * PKM)> kp;   // K rows of the next tile
    RowPieces<TI, pieces_per_thread(TC + 2 * PKM)> vp;   // V rows of this tile
    RowPieces<TI, pieces_per_thread(TC)> op;             // this tile's own keys again, for dQ += dS K

    // dQ: a wave holds the 16 x 16 blocks wave, wave + 4 of the head dimension
    const int wave = tid >> 6, lane = tid & 63, g = lane >> 4, n = lane & 15;
    f32x4 acc[kMaxD / 16 / NWV];
#pragma unroll
    for (int u = 0; u < kMaxD / 16 / NWV; ++u) acc[u] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // dW: thread t adds up the work items t, t + NT, ... (item = tap * 8 + row group) over all tiles
    float dw_acc[kDwItemsPerThread];
#pragma unroll
    for (int u = 0; u < kDwItemsPerThread; ++u) dw_acc[u] = 0.f;

    const int kend = p.causal ? min(p.Nk, r0 + TR) : p.Nk;
    kp.issue(Kb, -2 * pk, TC + 4 * pk, p.Nk, d);
    for (int c0 = 0; c0 < kend; c0 += TC) {
        bwd_tile<TI, TC>(t, p, kp, vp, Vb, r0, c0, [&] { op.issue(Kb, c0, TC, p.Nk, d); });
        op.commit(t.KVs, t.kst2, TC, d);
        if (c0 + TC < kend) kp.issue(Kb, c0 + TC - 2 * pk, TC + 4 * pk, p.Nk, d);
        dscore_tile<TC>(t, p, r0, c0);
        // dW[a][b] += dC[i][j] * S_m[i + a - pq][j + b - pk] over this tile's own (row, key) pairs,
        // always in the same order
#pragma unroll
        for (int u = 0; u < kDwItemsPerThread; ++u) {
            const int item = tid + u * NT;
            if (item < ntap * kDwRowGroups) {
                const int tap = item / kDwRowGroups, rg = item - tap * kDwRowGroups;
                const int a = tap / p.c_k, bb = tap - a * p.c_k;
                float s4[4] = {0.f, 0.f, 0.f, 0.f};   // four independent sums, added in a fixed order
                for (int i = rg * (TR / kDwRowGroups); i < (rg + 1) * (TR / kDwRowGroups); ++i) {
                    const float *dc = t.dCs + i * t.cst + pk, *sr = t.Ss + (i + a) * t.sst + pk + bb;
#pragma unroll 2
                    for (int j = 0; j < TC; j += 4) {
                        s4[0] = fmaf(dc[j], sr[j], s4[0]);
                        s4[1] = fmaf(dc[j + 1], sr[j + 1], s4[1]);
                        s4[2] = fmaf(dc[j + 2], sr[j + 2], s4[2]);
                        s4[3] = fmaf(dc[j + 3], sr[j + 3], s4[3]);
                    }
                }
                dw_acc[u] += (s4[0] + s4[1]) + (s4[2] + s4[3]);
            }
        }
        __syncthreads();
        {
            const float *bp[kMaxD / 16 / NWV];
#pragma unroll
            for (int u = 0; u < kMaxD / 16 / NWV; ++u) bp[u] = t.KVs + g * t.kst2 + min((wave + NWV * u) * 16 + n, d - 1);
            lds_mma_n<kMaxD / 16 / NWV>(acc, t.dSs + n * t.pst + g, 1, bp, t.kst2, TC);
        }
        __syncthreads();
    }
#pragma unroll
    for (int u = 0; u < kMaxD / 16 / NWV; ++u) {
        const int dc = (wave + NWV * u) * 16 + n;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int qi = r0 + 4 * g + rr;
            if (qi < p.Nq && dc < d) dQ[(bh * p.Nq + qi) * d + dc] = from_f32<TO>(acc[u][rr] * p.scale);
        }
    }
    // the row groups' sums, added in group order
#pragma unroll
    for (int u = 0; u < kDwItemsPerThread; ++u) {
        const int item = tid + u * NT;
        if (item < ntap * kDwRowGroups) t.red[item] = dw_acc[u];   // [tap][row group]
    }
    __syncthreads();
    float *part = dW_part + (bh * gridDim.x + qt) * ntap;
    for (int tap = tid; tap < ntap; tap += NT) {
        float sum = 0.f;
#pragma unroll
        for (int rg = 0; rg < kDwRowGroups; ++rg) sum += t.red[tap * kDwRowGroups + rg];
        part[tap] = sum;
    }
}

template <typename TI, typename TO>
__global__ __launch_bounds__(NT) void gen_dkdv_kernel(
    Problem p, const TI *__restrict__ Q, const TI *__restrict__ K, const TI *__restrict__ V,
    const TI *__restrict__ dO, const float *__restrict__ D, const float *__restrict__ LSE,
    const float *__restrict__ W, TO *__restrict__ dK, TO *__restrict__ dV) {
    constexpr int TC = kGenBwdTC;
    extern __shared__ float lds[];
    const BwdLds t = carve_bwd<TC>(lds, p);
    const int tid = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
    const int c0 = blockIdx.x * TC;
    const int d = p.d, pq = p.pq, ntap = p.c_q * p.c_k;
    const size_t bh = (size_t)b * p.H + h;
    const TI *Qb = Q + bh * p.Nq * d, *dOb = dO + bh * p.Nq * d;
    const TI *Kb = K + bh * p.Nk * d, *Vb = V + bh * p.Nk * d;

    for (int i = tid; i < ntap; i += NT) t.Ws[i] = W[(size_t)h * ntap + i];

    // dK, dV: TC keys x d = (TC / 16) x (d / 16) blocks each; a wave holds the blocks wave, wave + 4, ...
    // (block x: keys 16 (x % (TC / 16)) .., head-dim columns 16 (x / (TC / 16)) ..; lane (g, n): keys 4g .. 4g+3)
    constexpr int KB = TC / 16, NBLK = KB * (kMaxD / 16) / NWV;
    const int wave = tid >> 6, lane = tid & 63, g = lane >> 4, n = lane & 15;
    f32x4 acc_k[NBLK], acc_v[NBLK];
#pragma unroll
    for (int u = 0; u < NBLK; ++u) acc_k[u] = acc_v[u] = (f32x4){0.f, 0.f, 0.f, 0.f};

    constexpr int PKM = (kMaxCk - 1) / 2;
    RowPieces<TI, pieces_per_thread(TC + 4 * PKM)> kp;   // the K rows (the same for every row tile: KVs also holds V)
    RowPieces<TI, pieces_per_thread(TC + 2 * PKM)> vp;
    QSide<TI> qs;                                        // the next row tile's Q, dO, LSE, D
    const int pk = p.pk;
    // Causal: rows before the tile's first key see none of its keys.
    const int rstart = p.causal ? (c0 / TR) * TR : 0;
    kp.issue(Kb, c0 - 2 * pk, TC + 4 * pk, p.Nk, d);
    qs.issue(p, Qb, dOb, LSE + bh * p.Nq, D + bh * p.Nq, rstart);
    for (int r0 = rstart; r0 < p.Nq; r0 += TR) {
        __syncthreads();
        qs.commit(t, p);
        bwd_tile<TI, TC>(t, p, kp, vp, Vb, r0, c0, [&] {
            if (r0 + TR < p.Nq) {
                kp.issue(Kb, c0 - 2 * pk, TC + 4 * pk, p.Nk, d);
                qs.issue(p, Qb, dOb, LSE + bh * p.Nq, D + bh * p.Nq, r0 + TR);
            }
        });
        dscore_tile<TC>(t, p, r0, c0);
        __syncthreads();
        // dV[key][:] += sum_r P[r][key] dO[r][:], dK[key][:] += sum_r dS[r][key] Q[r][:]  (A(m = key, k = r));
        // eight independent accumulators per wave
        for (int k = 0; k < TR; k += 4) {
#pragma unroll
            for (int u = 0; u < NBLK; ++u) {
                const int x = wave + NWV * u, kb = x % KB, dc = min((x / KB) * 16 + n, d - 1);
                acc_v[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(t.Ps[(k + g) * t.pst + kb * 16 + n],
                                                                t.dOs[(k + g) * t.gst + dc], acc_v[u], 0, 0, 0);
                acc_k[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(t.dSs[(k + g) * t.pst + kb * 16 + n],
                                                                t.Qs[(k + g + pq) * t.qst + dc], acc_k[u], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < NBLK; ++u) {
        const int x = wave + NWV * u, kb = x % KB, dc = (x / KB) * 16 + n;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int kj = c0 + kb * 16 + 4 * g + rr;
            if (kj < p.Nk && dc < d) {
                dK[(bh * p.Nk + kj) * d + dc] = from_f32<TO>(acc_k[u][rr] * p.scale);
                dV[(bh * p.Nk + kj) * d + dc] = from_f32<TO>(acc_v[u][rr]);
            }
        }
    }
}

// ------------------------------------------------------------------- decode
// One workgroup per (split, head, batch): un-normalised partial of the last
// query row over the split's keys.  Resident rows sit at positions
// Nk-Nq .. Nk-1; tap a reads resident row Nq - c_q + a (a zero row if negative).
template <typename TI>
__global__ __launch_bounds__(NT) void gen_decode_kernel(Problem p, const TI *__restrict__ Q,
                                                        const TI *__restrict__ K,
                                                        const TI *__restrict__ V,
                                                        const float *__restrict__ W,
                                                        float *__restrict__ O_part,
                                                        float *__restrict__ M_part,
                                                        float *__restrict__ L_part) {
    constexpr int TC = kGenDecTC;
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int sp = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int pk = p.pk, d = p.d, cq = p.c_q;
    const int SC = TC + 2 * pk, kst = d + 1, sst = SC + 1, ntap = cq * p.c_k;
    float *Qs = lds;               // cq * d
    float *Ks = Qs + cq * d;       // SC * kst
    float *Ss = Ks + SC * kst;     // cq * sst
    float *Ps = Ss + cq * sst;     // TC
    float *Ws = Ps + TC;           // ntap
    float *st = Ws + ntap;         // m, l, alpha

    const size_t bh = (size_t)b * p.H + h;
    const TI *Qb = Q + bh * p.Nq * d;
    const TI *Kb = K + b * p.kv_bstride + h * p.kv_hstride;
    const TI *Vb = V + b * p.kv_bstride + h * p.kv_hstride;
    load_rows(Qs, d, Qb, p.Nq - cq, cq, p.Nq, d);
    for (int i = tid; i < ntap; i += NT) Ws[i] = W[(size_t)h * ntap + i];
    if (tid == 0) { st[0] = kNegInf; st[1] = 0.f; }

    const int chunk = (p.Nk + p.n_splits - 1) / p.n_splits;
    const int k_lo = sp * chunk, k_hi = min(p.Nk, k_lo + chunk);
    float acc = 0.f;
    for (int c0 = k_lo; c0 < k_hi; c0 += TC) {
        load_rows(Ks, kst, Kb, c0 - pk, SC, p.Nk, d);
        __syncthreads();
        // position of tap row a is Nk - c_q + a; the causal variant zeroes keys after it
        score_tile(Ss, sst, Qs, d, Ks, kst, cq, SC, d, p.Nk - cq, c0 - pk, p.scale, p.causal);
        __syncthreads();
        if (tid < TC) {
            int kj = c0 + tid;
            float c = kNegInf;
            if (kj < k_hi) {
                c = 0.f;
                for (int a = 0; a < cq; ++a)
                    for (int bb = 0; bb < p.c_k; ++bb)
                        c = fmaf(Ws[a * p.c_k + bb], Ss[a * sst + tid + bb], c);
            }
            float m_old = st[0];
            float m_new = fmaxf(m_old, wave_max(c));
            float e = (c == kNegInf) ? 0.f : __expf(c - m_new);
            float sum = wave_sum(e);
            float al = (m_old == kNegInf) ? 0.f : __expf(m_old - m_new);
            Ps[tid] = e;
            if (tid == 0) { st[0] = m_new; st[1] = st[1] * al + sum; st[2] = al; }
        }
        __syncthreads();
        if (tid < d) {
            float s = acc * st[2];
            const int n = min(TC, k_hi - c0);
            for (int j = 0; j < n; ++j) s = fmaf(Ps[j], to_f32(Vb[(size_t)(c0 + j) * d + tid]), s);
            acc = s;
        }
        __syncthreads();
    }
    const size_t slot = bh * p.n_splits + sp;
    if (tid < d) O_part[slot * d + tid] = acc;
    if (tid == 0) { M_part[slot] = st[0]; L_part[slot] = st[1]; }
}

template <typename F>
hipError_t allow_lds(F kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

}  // namespace

size_t generic_fwd_lds(const Problem &p) { return fwd_lds_floats(p.d, p.pq, p.pk, p.c_q * p.c_k) * sizeof(float); }

size_t generic_bwd_lds(const Problem &p) { return bwd_lds_floats(p.d, p.pq, p.pk, p.c_q * p.c_k) * sizeof(float); }

size_t generic_decode_lds(const Problem &p) {
    const int SC = kGenDecTC + 2 * p.pk;
    size_t f = (size_t)p.c_q * p.d + (size_t)SC * (p.d + 1) + (size_t)p.c_q * (SC + 1) + kGenDecTC +
               p.c_q * p.c_k + 4;
    return f * sizeof(float);
}

#define CONVATTN_DISPATCH_IO(in_dt, out_dt, CALL)                                   \
    do {                                                                            \
        if (in_dt == CONVATTN_BF16 && out_dt == CONVATTN_BF16) { CALL(bf16_t, bf16_t); } \
        else if (in_dt == CONVATTN_BF16 && out_dt == CONVATTN_F32) { CALL(bf16_t, float); } \
        else if (in_dt == CONVATTN_F32 && out_dt == CONVATTN_BF16) { CALL(float, bf16_t); } \
        else { CALL(float, float); }                                                \
    } while (0)

hipError_t generic_fwd(const Problem &p, int in_dt, int out_dt, const void *q, const void *k,
                       const void *v, const float *w, void *o, float *m, float *l, hipStream_t s) {
    const size_t lds = generic_fwd_lds(p);
    dim3 grid(generic_q_tiles(p), p.H, p.B);
#define CALL(TI, TO)                                                                         \
    {                                                                                        \
        hipError_t e = allow_lds(gen_fwd_kernel<TI, TO>, lds);                               \
        if (e != hipSuccess) return e;                                                       \
        gen_fwd_kernel<TI, TO><<<grid, NT, lds, s>>>(p, (const TI *)q, (const TI *)k,        \
                                                     (const TI *)v, w, (TO *)o, m, l);       \
    }
    CONVATTN_DISPATCH_IO(in_dt, out_dt, CALL);
#undef CALL
    return hipGetLastError();
}

hipError_t generic_bwd_dq_dw(const Problem &p, int in_dt, int out_dt, const void *q, const void *k,
                             const void *v, const void *d_o, const float *D, const float *lse,
                             const float *w, void *dq, float *dw_part, hipStream_t s) {
    const size_t lds = generic_bwd_lds(p);
    dim3 grid(generic_q_tiles(p), p.H, p.B);
#define CALL(TI, TO)                                                                          \
    {                                                                                         \
        hipError_t e = allow_lds(gen_dq_dw_kernel<TI, TO>, lds);                              \
        if (e != hipSuccess) return e;                                                        \
        gen_dq_dw_kernel<TI, TO><<<grid, NT, lds, s>>>(p, (const TI *)q, (const TI *)k,       \
                                                       (const TI *)v, (const TI *)d_o, D, lse, \
                                                       w, (TO *)dq, dw_part);                 \
    }
    CONVATTN_DISPATCH_IO(in_dt, out_dt, CALL);
#undef CALL
    return hipGetLastError();
}

hipError_t generic_bwd_dkdv(const Problem &p, int in_dt, int out_dt, const void *q, const void *k,
                            const void *v, const void *d_o, const float *D, const float *lse,
                            const float *w, void *dk, void *dv, hipStream_t s) {
    const size_t lds = generic_bwd_lds(p);
    dim3 grid((p.Nk + kGenBwdTC - 1) / kGenBwdTC, p.H, p.B);
#define CALL(TI, TO)                                                                         \
    {                                                                                        \
        hipError_t e = allow_lds(gen_dkdv_kernel<TI, TO>, lds);                              \
        if (e != hipSuccess) return e;                                                       \
        gen_dkdv_kernel<TI, TO><<<grid, NT, lds, s>>>(p, (const TI *)q, (const TI *)k,       \
                                                      (const TI *)v, (const TI *)d_o, D, lse, \
                                                      w, (TO *)dk, (TO *)dv);                \
    }
    CONVATTN_DISPATCH_IO(in_dt, out_dt, CALL);
#undef CALL
    return hipGetLastError();
}

hipError_t generic_decode(const Problem &p, int in_dt, const void *q, const void *k, const void *v,
                          const float *w, float *o_part, float *m_part, float *l_part,
                          hipStream_t s) {
    const size_t lds = generic_decode_lds(p);
    dim3 grid(p.n_splits, p.H, p.B);
    if (in_dt == CONVATTN_BF16) {
        hipError_t e = allow_lds(gen_decode_kernel<bf16_t>, lds);
        if (e != hipSuccess) return e;
        gen_decode_kernel<bf16_t><<<grid, NT, lds, s>>>(p, (const bf16_t *)q, (const bf16_t *)k,
                                                        (const bf16_t *)v, w, o_part, m_part, l_part);
    } else {
        hipError_t e = allow_lds(gen_decode_kernel<float>, lds);
        if (e != hipSuccess) return e;
        gen_decode_kernel<float><<<grid, NT, lds, s>>>(p, (const float *)q, (const float *)k,
                                                       (const float *)v, w, o_part, m_part, l_part);
    }
    return hipGetLastError();
}

}  // namespace convattn
