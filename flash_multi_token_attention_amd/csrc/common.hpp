// Internal declarations shared by the conv-attention HIP sources (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "convattn.h"

namespace convattn {

// Problem as the kernels see it (derived from convattn_desc once, on the host).
struct Problem {
    int B, H, Nq, Nk, d;
    int c_q, c_k, pq, pk;  // pq = c_q-1 rows back, pk = (c_k-1)/2 keys either side
    float scale;
    int causal;
    int n_splits;
    // decode only: elements between consecutive batches / heads of K and V (a dense [B,H,Nk,d]
    // tensor has H*Nk*d and Nk*d; a view of a longer cache has the cache's)
    long long kv_bstride, kv_hstride;
};

typedef __bf16 bf16_t;

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

constexpr int kWave = 64;
constexpr float kNegInf = -__builtin_inff();

// 64-lane butterfly reductions.
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// ---- fp32-arithmetic kernels (generic_kernels.hip): any supported shape ----
constexpr int kGenTR = 16;       // query rows a workgroup owns
constexpr int kGenFwdTC = 64;    // keys per forward tile
constexpr int kGenBwdTC = 32;    // keys per backward tile
constexpr int kGenDecTC = 64;    // keys per decode tile
constexpr int kMaxD = 128;
constexpr int kMaxCq = 16;
constexpr int kMaxCk = 33;
constexpr size_t kLdsBytes = 160 * 1024;

size_t generic_fwd_lds(const Problem &p);
size_t generic_bwd_lds(const Problem &p);
size_t generic_decode_lds(const Problem &p);

hipError_t generic_fwd(const Problem &p, int in_dt, int out_dt, const void *q, const void *k,
                       const void *v, const float *w, void *o, float *m, float *l, hipStream_t s);
hipError_t generic_bwd_dq_dw(const Problem &p, int in_dt, int out_dt, const void *q, const void *k,
                             const void *v, const void *d_o, const float *D, const float *lse,
                             const float *w, void *dq, float *dw_part, hipStream_t s);
hipError_t generic_bwd_dkdv(const Problem &p, int in_dt, int out_dt, const void *q, const void *k,
                            const void *v, const void *d_o, const float *D, const float *lse,
                            const float *w, void *dk, void *dv, hipStream_t s);
hipError_t generic_decode(const Problem &p, int in_dt, const void *q, const void *k, const void *v,
                          const float *w, float *o_part, float *m_part, float *l_part, hipStream_t s);
inline int generic_q_tiles(const Problem &p) { return (p.Nq + kGenTR - 1) / kGenTR; }

// ---- shape-independent helpers (reduce_kernels.hip) ----
hipError_t bwd_preprocess(const Problem &p, int in_dt, int out_dt, const void *o, const void *d_o,
                          const float *m, const float *l, float *D, float *lse, hipStream_t s);
hipError_t dw_reduce(const Problem &p, int n_tiles, const float *dw_part, float *dw, hipStream_t s);
hipError_t decode_combine(const Problem &p, int out_dt, const float *o_part, const float *m_part,
                          const float *l_part, void *o, float *m, float *l, hipStream_t s);

// ---- head-mixing attention (headmix_attn.hip) ----
hipError_t headmix_fwd(int B, int H, int N, int d, float scale, int causal, int out_dt, const void *q, const void *k,
                       const void *v, const float *w, void *o, float *l, float *m, hipStream_t s);
hipError_t headmix_bwd_dq_dw(int B, int H, int N, int d, float scale, int causal, const void *q, const void *k,
                             const void *v, const float *w, const void *d_o, const float *lse, const float *Dl, float *dq,
                             float *dw_part, float *dw, hipStream_t s);
hipError_t headmix_bwd_dkdv(int B, int H, int N, int d, float scale, int causal, const void *q, const void *k,
                            const void *v, const float *w, const void *d_o, const float *lse, const float *Dl, float *dk,
                            float *dv, hipStream_t s);
int headmix_row_tiles(int N);

}  // namespace convattn
