// fp32-arithmetic conv-attention kernels for gfx950: every supported shape and
// both input types.  These are the "exact" path (CONVATTN_FLAG_EXACT, fp32
// inputs, shapes the MFMA kernels do not cover): all dot products, the
// convolution and the softmax run in fp32 on the vector ALUs out of LDS tiles,
// accumulators stay in registers for the whole key (or query) loop, and nothing
// is accumulated through HBM or with atomics.
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

// dst[r][c] (row stride `stride`) = src[(row0 + r) * d + c], zero outside [0, N).
template <typename T>
__device__ __forceinline__ void load_rows(float *dst, int stride, const T *src, int row0, int nrows,
                                          int N, int d) {
    for (int idx = threadIdx.x; idx < nrows * d; idx += NT) {
        int r = idx / d, c = idx - r * d;
        int g = row0 + r;
        dst[r * stride + c] = (g >= 0 && g < N) ? to_f32(src[(size_t)g * d + c]) : 0.f;
    }
}

// S[r][c] = scale * <A[r], Kt[c]> for r < nr, c < nc; rows/cols outside the
// sequence are zero because their operands were zero-filled; the causal
// pre-mask zeroes keys after the row's own position.
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
    const int kst = d + 1, sst = SC + 1, ntap = p.c_q * p.c_k;
    float *Qs = lds;
    float *KVs = Qs + QR * d;
    float *Ss = KVs + SC * kst;
    float *Ps = Ss + QR * sst;
    float *Ws = Ps + TR * TC;
    float *m_s = Ws + ntap;
    float *l_s = m_s + TR;
    float *al_s = l_s + TR;

    const size_t bh = (size_t)b * p.H + h;
    const TI *Qb = Q + bh * p.Nq * d;
    const TI *Kb = K + bh * p.Nk * d;
    const TI *Vb = V + bh * p.Nk * d;

    load_rows(Qs, d, Qb, r0 - pq, QR, p.Nq, d);
    for (int i = tid; i < ntap; i += NT) Ws[i] = W[(size_t)h * ntap + i];
    if (tid < TR) { m_s[tid] = kNegInf; l_s[tid] = 0.f; }

    const int orow = tid >> 4, ocol = tid & 15;  // this thread's output row and column phase
    float acc[kMaxD / 16];
#pragma unroll
    for (int u = 0; u < kMaxD / 16; ++u) acc[u] = 0.f;

    const int kend = p.causal ? min(p.Nk, r0 + TR) : p.Nk;
    for (int c0 = 0; c0 < kend; c0 += TC) {
        load_rows(KVs, kst, Kb, c0 - pk, SC, p.Nk, d);
        __syncthreads();
        score_tile(Ss, sst, Qs, d, KVs, kst, QR, SC, d, r0 - pq, c0 - pk, p.scale, p.causal);
        __syncthreads();
        load_rows(KVs, kst, Vb, c0, TC, p.Nk, d);  // V replaces K
        for (int idx = tid; idx < TR * TC; idx += NT) {
            int i = idx / TC, j = idx - i * TC;
            int qi = r0 + i, kj = c0 + j;
            float c = kNegInf;
            if (kj < p.Nk && !(p.causal && kj > qi)) {
                c = 0.f;
                for (int a = 0; a < p.c_q; ++a)
                    for (int bb = 0; bb < p.c_k; ++bb)
                        c = fmaf(Ws[a * p.c_k + bb], Ss[(i + a) * sst + j + bb], c);
            }
            Ps[idx] = c;
        }
        __syncthreads();
        {   // online softmax: one wave per 4 rows, one lane per key of the tile
            const int wv = tid >> 6, lane = tid & 63;
            for (int rr = 0; rr < 4; ++rr) {
                int i = wv * 4 + rr;
                float c = Ps[i * TC + lane];
                float m_old = m_s[i];
                float m_new = fmaxf(m_old, wave_max(c));
                float e = (c == kNegInf) ? 0.f : __expf(c - m_new);
                float sum = wave_sum(e);
                float al = (m_old == kNegInf) ? 0.f : __expf(m_old - m_new);
                Ps[i * TC + lane] = e;
                if (lane == 0) { m_s[i] = m_new; l_s[i] = l_s[i] * al + sum; al_s[i] = al; }
            }
        }
        __syncthreads();
        {
            const float al = al_s[orow];
            const float *prow = Ps + orow * TC;
#pragma unroll
            for (int u = 0; u < kMaxD / 16; ++u) {
                int dc = ocol + 16 * u;
                if (dc < d) {
                    float s = acc[u] * al;
                    for (int j = 0; j < TC; ++j) s = fmaf(prow[j], KVs[j * kst + dc], s);
                    acc[u] = s;
                }
            }
        }
        __syncthreads();
    }
    const int qi = r0 + orow;
    if (qi < p.Nq) {
        const float inv = 1.f / l_s[orow];
#pragma unroll
        for (int u = 0; u < kMaxD / 16; ++u) {
            int dc = ocol + 16 * u;
            if (dc < d) O[(bh * p.Nq + qi) * d + dc] = from_f32<TO>(acc[u] * inv);
        }
        if (ocol == 0) { M[bh * p.Nq + qi] = m_s[orow]; L[bh * p.Nq + qi] = l_s[orow]; }
    }
}

// ----------------------------------------------------------------- backward
// LDS carve-up shared by the two backward kernels.
struct BwdLds {
    float *Qs, *dOs, *KVs, *Ss, *dCs, *Ps, *dSs, *Ws, *lse_s, *D_s;
    int kst, sst, cst, pst;
};

template <int TC>
__device__ __forceinline__ BwdLds carve_bwd(float *lds, const Problem &p) {
    BwdLds t;
    const int d = p.d, pq = p.pq, pk = p.pk;
    t.kst = d + 1;
    t.sst = TC + 4 * pk + 1;
    t.cst = TC + 2 * pk + 1;
    t.pst = TC + 1;
    t.Qs = lds;
    t.dOs = t.Qs + (TR + 2 * pq) * d;
    t.KVs = t.dOs + (TR + pq) * d;
    t.Ss = t.KVs + (TC + 4 * pk) * t.kst;
    t.dCs = t.Ss + (TR + 2 * pq) * t.sst;
    t.Ps = t.dCs + (TR + pq) * t.cst;
    t.dSs = t.Ps + TR * t.pst;
    t.Ws = t.dSs + TR * t.pst;
    t.lse_s = t.Ws + p.c_q * p.c_k;
    t.D_s = t.lse_s + (TR + pq);
    return t;
}

// Loads what depends on the query tile: Q rows r0-pq .. r0+TR+pq-1, dO / LSE / D
// rows r0 .. r0+TR+pq-1.
template <typename TI>
__device__ __forceinline__ void load_q_side(const BwdLds &t, const Problem &p, const TI *Qb,
                                            const TI *dOb, const float *lse, const float *D, int r0) {
    load_rows(t.Qs, p.d, Qb, r0 - p.pq, TR + 2 * p.pq, p.Nq, p.d);
    load_rows(t.dOs, p.d, dOb, r0, TR + p.pq, p.Nq, p.d);
    for (int i = threadIdx.x; i < TR + p.pq; i += NT) {
        int g = r0 + i;
        t.lse_s[i] = g < p.Nq ? lse[g] : 0.f;
        t.D_s[i] = g < p.Nq ? D[g] : 0.f;
    }
}

// For query tile r0 and key tile c0 (query side already in LDS) leaves in LDS:
//   Ss  = S_m  rows r0-pq .. r0+TR+pq-1, keys c0-2pk .. c0+TC+2pk-1
//   dCs = dC   rows r0    .. r0+TR+pq-1, keys c0-pk  .. c0+TC+pk-1
//   Ps  = P    rows r0    .. r0+TR-1,    keys c0     .. c0+TC-1
// Ends with a barrier; KVs is free afterwards.
template <typename TI, int TC>
__device__ __forceinline__ void bwd_tile(const BwdLds &t, const Problem &p, const TI *Kb,
                                         const TI *Vb, int r0, int c0) {
    const int pq = p.pq, pk = p.pk, d = p.d;
    load_rows(t.KVs, t.kst, Kb, c0 - 2 * pk, TC + 4 * pk, p.Nk, d);
    __syncthreads();
    score_tile(t.Ss, t.sst, t.Qs, d, t.KVs, t.kst, TR + 2 * pq, TC + 4 * pk, d, r0 - pq, c0 - 2 * pk,
               p.scale, p.causal);
    __syncthreads();
    load_rows(t.KVs, t.kst, Vb, c0 - pk, TC + 2 * pk, p.Nk, d);
    __syncthreads();
    const int nr = TR + pq, nc = TC + 2 * pk;
    for (int idx = threadIdx.x; idx < nr * nc; idx += NT) {
        int i = idx / nc, j = idx - i * nc;
        int qi = r0 + i, kj = c0 - pk + j;
        float P = 0.f, dC = 0.f;
        if (qi < p.Nq && kj >= 0 && kj < p.Nk && !(p.causal && kj > qi)) {
            float c = 0.f;
            for (int a = 0; a < p.c_q; ++a)
                for (int bb = 0; bb < p.c_k; ++bb)
                    c = fmaf(t.Ws[a * p.c_k + bb], t.Ss[(i + a) * t.sst + j + bb], c);
            P = __expf(c - t.lse_s[i]);
            const float *g = t.dOs + i * d;
            const float *vv = t.KVs + j * t.kst;
            float dP = 0.f;
            for (int x = 0; x < d; ++x) dP = fmaf(g[x], vv[x], dP);
            dC = P * (dP - t.D_s[i]);
        }
        t.dCs[i * t.cst + j] = dC;
        if (i < TR && j >= pk && j < pk + TC) t.Ps[i * t.pst + j - pk] = P;
    }
    __syncthreads();
}

// dSs[r][c] = sum_ab W[a][b] * dC[r - a + pq][c - b + pk], zero on the causal future.
template <int TC>
__device__ __forceinline__ void dscore_tile(const BwdLds &t, const Problem &p, int r0, int c0) {
    const int pq = p.pq, pk = p.pk;
    for (int idx = threadIdx.x; idx < TR * TC; idx += NT) {
        int r = idx / TC, c = idx - r * TC;
        int qi = r0 + r, kj = c0 + c;
        float s = 0.f;
        if (qi < p.Nq && kj < p.Nk && !(p.causal && kj > qi)) {
            for (int a = 0; a < p.c_q; ++a)
                for (int bb = 0; bb < p.c_k; ++bb)
                    s = fmaf(t.Ws[a * p.c_k + bb], t.dCs[(r - a + pq) * t.cst + c - bb + 2 * pk], s);
        }
        t.dSs[r * t.pst + c] = s;
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
    load_q_side(t, p, Qb, dOb, LSE + bh * p.Nq, D + bh * p.Nq, r0);

    const int orow = tid >> 4, ocol = tid & 15;
    float acc[kMaxD / 16];
#pragma unroll
    for (int u = 0; u < kMaxD / 16; ++u) acc[u] = 0.f;
    constexpr int kTapsPerThread = (kMaxCq * kMaxCk + NT - 1) / NT;
    float dw_acc[kTapsPerThread];
#pragma unroll
    for (int u = 0; u < kTapsPerThread; ++u) dw_acc[u] = 0.f;

    const int kend = p.causal ? min(p.Nk, r0 + TR) : p.Nk;
    for (int c0 = 0; c0 < kend; c0 += TC) {
        bwd_tile<TI, TC>(t, p, Kb, Vb, r0, c0);
        load_rows(t.KVs, t.kst, Kb, c0, TC, p.Nk, d);  // own keys, for dQ += dS K
        dscore_tile<TC>(t, p, r0, c0);
        // dW[a][b] += dC[i][j] * S_m[i + a - pq][j + b - pk] over this tile's own
        // (row, key) pairs; a thread owns whole taps, so the order is fixed.
#pragma unroll
        for (int u = 0; u < kTapsPerThread; ++u) {
            int tap = tid + u * NT;
            if (tap < ntap) {
                int a = tap / p.c_k, bb = tap - a * p.c_k;
                float s = dw_acc[u];
                for (int i = 0; i < TR; ++i)
                    for (int j = 0; j < TC; ++j)
                        s = fmaf(t.dCs[i * t.cst + j + pk], t.Ss[(i + a) * t.sst + j + pk + bb], s);
                dw_acc[u] = s;
            }
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kMaxD / 16; ++u) {
            int dc = ocol + 16 * u;
            if (dc < d) {
                float s = acc[u];
                for (int c = 0; c < TC; ++c) s = fmaf(t.dSs[orow * t.pst + c], t.KVs[c * t.kst + dc], s);
                acc[u] = s;
            }
        }
        __syncthreads();
    }
    const int qi = r0 + orow;
    if (qi < p.Nq) {
#pragma unroll
        for (int u = 0; u < kMaxD / 16; ++u) {
            int dc = ocol + 16 * u;
            if (dc < d) dQ[(bh * p.Nq + qi) * d + dc] = from_f32<TO>(acc[u] * p.scale);
        }
    }
    float *part = dW_part + (bh * gridDim.x + qt) * ntap;
#pragma unroll
    for (int u = 0; u < kTapsPerThread; ++u) {
        int tap = tid + u * NT;
        if (tap < ntap) part[tap] = dw_acc[u];
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

    const int ocol = tid >> 3, oph = tid & 7;  // this thread's key and column phase
    float acc_k[kMaxD / 8], acc_v[kMaxD / 8];
#pragma unroll
    for (int u = 0; u < kMaxD / 8; ++u) { acc_k[u] = 0.f; acc_v[u] = 0.f; }

    // Causal: rows before the tile's first key see none of its keys.
    const int rstart = p.causal ? (c0 / TR) * TR : 0;
    for (int r0 = rstart; r0 < p.Nq; r0 += TR) {
        __syncthreads();
        load_q_side(t, p, Qb, dOb, LSE + bh * p.Nq, D + bh * p.Nq, r0);
        bwd_tile<TI, TC>(t, p, Kb, Vb, r0, c0);
        dscore_tile<TC>(t, p, r0, c0);
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kMaxD / 8; ++u) {
            int dc = oph + 8 * u;
            if (dc < d) {
                float sk = acc_k[u], sv = acc_v[u];
                for (int r = 0; r < TR; ++r) {
                    sv = fmaf(t.Ps[r * t.pst + ocol], t.dOs[r * d + dc], sv);
                    sk = fmaf(t.dSs[r * t.pst + ocol], t.Qs[(r + pq) * d + dc], sk);
                }
                acc_k[u] = sk;
                acc_v[u] = sv;
            }
        }
    }
    const int kj = c0 + ocol;
    if (kj < p.Nk) {
#pragma unroll
        for (int u = 0; u < kMaxD / 8; ++u) {
            int dc = oph + 8 * u;
            if (dc < d) {
                dK[(bh * p.Nk + kj) * d + dc] = from_f32<TO>(acc_k[u] * p.scale);
                dV[(bh * p.Nk + kj) * d + dc] = from_f32<TO>(acc_v[u]);
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

size_t generic_fwd_lds(const Problem &p) {
    const int QR = TR + p.pq, SC = kGenFwdTC + 2 * p.pk;
    size_t f = (size_t)QR * p.d + (size_t)SC * (p.d + 1) + (size_t)QR * (SC + 1) + TR * kGenFwdTC +
               p.c_q * p.c_k + 3 * TR;
    return f * sizeof(float);
}

size_t generic_bwd_lds(const Problem &p) {
    constexpr int TC = kGenBwdTC;
    size_t f = (size_t)(TR + 2 * p.pq) * p.d + (size_t)(TR + p.pq) * p.d +
               (size_t)(TC + 4 * p.pk) * (p.d + 1) + (size_t)(TR + 2 * p.pq) * (TC + 4 * p.pk + 1) +
               (size_t)(TR + p.pq) * (TC + 2 * p.pk + 1) + 2 * TR * (TC + 1) + p.c_q * p.c_k +
               2 * (TR + p.pq);
    return f * sizeof(float);
}

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
