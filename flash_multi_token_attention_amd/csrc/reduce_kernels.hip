// Small bandwidth-bound helpers around the conv-attention kernels:
// backward preparation (D, LSE), the ordered dW reduction and the decode
// split merge.
#include "common.hpp"

namespace convattn {
namespace {

// D = <dO, O>, LSE = M + log L.  16 lanes per query row, 8 elements (16 or 32 bytes) per lane:
// a wave reads 4 rows at a time with full-width loads; d is a multiple of 8 and at most 128.
template <typename T>
__device__ __forceinline__ void load8(const T *__restrict__ ptr, float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        const uint4 raw = *reinterpret_cast<const uint4 *>(ptr);
        const unsigned int w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
        }
    } else {
        const float4 a = *reinterpret_cast<const float4 *>(ptr);
        const float4 b = *reinterpret_cast<const float4 *>(ptr + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
}

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void preprocess_kernel(size_t rows, int d, const TO *__restrict__ O,
                                                         const TI *__restrict__ dO,
                                                         const float *__restrict__ M,
                                                         const float *__restrict__ L,
                                                         float *__restrict__ D, float *__restrict__ LSE) {
    const size_t row = (size_t)blockIdx.x * 16 + (threadIdx.x >> 4);
    const int sub = threadIdx.x & 15;
    float s = 0.f;
    if (row < rows && sub * 8 < d) {
        float o[8], g[8];
        load8(O + row * d + sub * 8, o);
        load8(dO + row * d + sub * 8, g);
#pragma unroll
        for (int i = 0; i < 8; ++i) s = fmaf(o[i], g[i], s);
    }
#pragma unroll
    for (int m = 8; m >= 1; m >>= 1) s += __shfl_xor(s, m, 16);
    if (row < rows && sub == 0) {
        D[row] = s;
        LSE[row] = M[row] + __logf(L[row]);
    }
}

// dW[h][tap] = sum over (batch, tile) of the partials, in a fixed order: a workgroup takes 64 taps
// of one head (lane = tap, so a partial is read with contiguous loads); wave w adds the partials
// w, w+4, ... in four independent chains, and the four waves' sums are added in wave order.
__global__ __launch_bounds__(256) void dw_reduce_kernel(int B, int H, int n_tiles, int ntap,
                                                        const float *__restrict__ part, float *__restrict__ dW) {
    __shared__ float red[4][64];
    const int h = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int tap = blockIdx.y * 64 + lane;
    const int n = B * n_tiles;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (tap < ntap) {
        auto at = [&](int q) {
            const int b = q / n_tiles, t = q - b * n_tiles;
            return part[(((size_t)b * H + h) * n_tiles + t) * ntap + tap];
        };
        int q = wave;
        for (; q + 12 < n; q += 16) {
#pragma unroll
            for (int c = 0; c < 4; ++c) s[c] += at(q + 4 * c);
        }
        for (int c = 0; q < n; q += 4, ++c) s[c] += at(q);
    }
    red[wave][lane] = (s[0] + s[1]) + (s[2] + s[3]);
    __syncthreads();
    if (wave == 0 && tap < ntap)
        dW[(size_t)h * ntap + tap] = (red[0][lane] + red[1][lane]) + (red[2][lane] + red[3][lane]);
}

// Merge of a few decode splits: one workgroup per (batch, head), one thread per output column walks the splits.
template <typename TO>
__global__ void combine_few_kernel(int n_splits, int d, const float *__restrict__ O_part,
                                   const float *__restrict__ M_part, const float *__restrict__ L_part,
                                   TO *__restrict__ O, float *__restrict__ M, float *__restrict__ L) {
    const size_t bh = blockIdx.x;
    const float *mp = M_part + bh * n_splits;
    const float *lp = L_part + bh * n_splits;
    float m = kNegInf;
    for (int s = 0; s < n_splits; ++s) m = fmaxf(m, mp[s]);
    float l = 0.f;
    for (int s = 0; s < n_splits; ++s) l += (mp[s] == kNegInf) ? 0.f : lp[s] * __expf(mp[s] - m);
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        float o = 0.f;
        for (int s = 0; s < n_splits; ++s)
            if (mp[s] != kNegInf) o = fmaf(O_part[(bh * n_splits + s) * d + c], __expf(mp[s] - m), o);
        O[bh * d + c] = from_f32<TO>(o / l);
    }
    if (threadIdx.x == 0) { M[bh] = m; L[bh] = l; }
}

// Merge of many decode splits: m = max m_s, l = sum l_s e^{m_s - m}, o = sum o_s e^{m_s - m} / l.
// A workgroup takes 32 output columns of one (batch, head).  All 256 threads scan the splits'
// (m_s, l_s) together (every workgroup of a head repeats this: at most 1024 pairs); for the
// outputs thread (g, c) adds the splits g, g+8, ... of column c, so a split's row is read with
// 128-byte loads and eight rows are in flight per pass, and the eight sums are added in order of g.
template <typename TO>
__global__ __launch_bounds__(256) void combine_kernel(int n_splits, int d, const float *__restrict__ O_part,
                                                      const float *__restrict__ M_part,
                                                      const float *__restrict__ L_part, TO *__restrict__ O,
                                                      float *__restrict__ M, float *__restrict__ L) {
    __shared__ float red_m[4], red_l[4], acc[8][32];
    const size_t bh = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *mp = M_part + bh * n_splits;
    const float *lp = L_part + bh * n_splits;
    float m = kNegInf;
    for (int s = tid; s < n_splits; s += 256) m = fmaxf(m, mp[s]);
#pragma unroll
    for (int x = 32; x >= 1; x >>= 1) m = fmaxf(m, __shfl_xor(m, x));
    if (lane == 0) red_m[wave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red_m[0], red_m[1]), fmaxf(red_m[2], red_m[3]));
    float l = 0.f;
    for (int s = tid; s < n_splits; s += 256) {
        const float ms = mp[s];
        if (ms != kNegInf) l = fmaf(lp[s], __expf(ms - m), l);
    }
#pragma unroll
    for (int x = 32; x >= 1; x >>= 1) l += __shfl_xor(l, x);
    if (lane == 0) red_l[wave] = l;
    __syncthreads();
    l = (red_l[0] + red_l[1]) + (red_l[2] + red_l[3]);

    const int c = tid & 31, g = tid >> 5, col = blockIdx.y * 32 + c;
    float o = 0.f;
    if (col < d) {
        const float *op = O_part + bh * n_splits * d + col;
#pragma unroll 4
        for (int s = g; s < n_splits; s += 8) {
            const float ms = mp[s];
            if (ms != kNegInf) o = fmaf(op[(size_t)s * d], __expf(ms - m), o);
        }
    }
    acc[g][c] = o;
    __syncthreads();
    if (tid < 32 && col < d) {
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += acc[i][c];
        O[bh * d + col] = from_f32<TO>(sum / l);
    }
    if (tid == 0 && blockIdx.y == 0) { M[bh] = m; L[bh] = l; }
}

}  // namespace

hipError_t bwd_preprocess(const Problem &p, int in_dt, int out_dt, const void *o, const void *d_o,
                          const float *m, const float *l, float *D, float *lse, hipStream_t s) {
    const size_t rows = (size_t)p.B * p.H * p.Nq;
    const unsigned grid = (unsigned)((rows + 15) / 16);
#define CALL(TI, TO) \
    preprocess_kernel<TI, TO><<<grid, 256, 0, s>>>(rows, p.d, (const TO *)o, (const TI *)d_o, m, l, D, lse)
    if (in_dt == CONVATTN_BF16 && out_dt == CONVATTN_BF16) CALL(bf16_t, bf16_t);
    else if (in_dt == CONVATTN_BF16) CALL(bf16_t, float);
    else if (out_dt == CONVATTN_BF16) CALL(float, bf16_t);
    else CALL(float, float);
#undef CALL
    return hipGetLastError();
}

hipError_t dw_reduce(const Problem &p, int n_tiles, const float *dw_part, float *dw, hipStream_t s) {
    dw_reduce_kernel<<<dim3(p.H, (p.c_q * p.c_k + 63) / 64), 256, 0, s>>>(p.B, p.H, n_tiles, p.c_q * p.c_k, dw_part, dw);
    return hipGetLastError();
}

hipError_t decode_combine(const Problem &p, int out_dt, const float *o_part, const float *m_part,
                          const float *l_part, void *o, float *m, float *l, hipStream_t s) {
    // (a serving step with many (batch, head) pairs has a handful of splits: the walk over them is shorter than
    // the second kernel's two reductions; few pairs over a long cache have hundreds)
    if (p.n_splits <= 8) {
        const unsigned few = (unsigned)(p.B * p.H);
        if (out_dt == CONVATTN_BF16)
            combine_few_kernel<bf16_t><<<few, 128, 0, s>>>(p.n_splits, p.d, o_part, m_part, l_part, (bf16_t *)o, m, l);
        else
            combine_few_kernel<float><<<few, 128, 0, s>>>(p.n_splits, p.d, o_part, m_part, l_part, (float *)o, m, l);
        return hipGetLastError();
    }
    const dim3 grid((unsigned)(p.B * p.H), (unsigned)((p.d + 31) / 32));
    if (out_dt == CONVATTN_BF16)
        combine_kernel<bf16_t><<<grid, 256, 0, s>>>(p.n_splits, p.d, o_part, m_part, l_part, (bf16_t *)o, m, l);
    else
        combine_kernel<float><<<grid, 256, 0, s>>>(p.n_splits, p.d, o_part, m_part, l_part, (float *)o, m, l);
    return hipGetLastError();
}

}  // namespace convattn
