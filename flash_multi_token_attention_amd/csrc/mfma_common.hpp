// Building blocks of the bf16 MFMA conv-attention kernels (gfx950, wave64).
//
// MFMA 16x16x32 register layout (lane = 16*g + n, g = 0..3, n = 0..15):
//   A operand: row n of the 16 x 32 tile, k = 8g .. 8g+7   (8 x 16-bit, one b128)
//   B operand: column n of the 32 x 16 tile, k = 8g .. 8g+7
//   C/D:       column n, rows 4g .. 4g+3                    (4 x fp32)
//
// The key-axis part of the (c_q x c_k) window is a banded Toeplitz matrix, so the
// convolution of a score tile is c_q MFMAs per 16 x 16 output block: for query
// tap a, C^T[16 out keys][16 queries] += T_a^T[16 x 32] * S^T[32 in keys][16
// queries shifted by a - pad_q rows].  The 32 input keys start 8 before the
// block's first output key (a 16-byte-aligned LDS column), which covers
// pad_k <= 8.  Scores are staged in LDS as fp16 (11-bit significand; bf16's 8
// bits would cost ~1e-2 in the softmax argument).
#pragma once
#include <atomic>
#include <type_traits>

#include "common.hpp"

namespace convattn {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
// Five consecutive dwords at a 4-byte boundary of LDS, as 32-bit reads (the compiler pairs them
// into ds_read2_b32).  A 128-bit LDS read that is not 16-byte aligned is legal on gfx950 but slow:
// measured with four waves reading, one costs about 66 clocks of the LDS pipe against about 12 for
// the five dwords read separately.
__device__ __forceinline__ void lds_read_dwords5(const unsigned char *p, u32x4 &lo, unsigned int &hi) {
    const unsigned int *q = reinterpret_cast<const unsigned int *>(p);
    lo = (u32x4){q[0], q[1], q[2], q[3]};
    hi = q[4];
}

constexpr int kKeyHalo = 8;          // LDS columns before a block's first output key
constexpr int kMfmaMaxPk = 8;        // so c_k <= 17 on the MFMA path
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kF16Max = 65504.f;   // what a score beyond fp16's range is rounded to

__device__ __forceinline__ f32x4 mfma_bf16(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4 mfma_f16(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Scheduling hints: the sequence of these calls in program order is the order in which the
// backend lays out groups of LDS reads and MFMAs.  Used as "reads of stage s+1, then MFMAs
// of stage s" so that fragment reads stay one stage ahead instead of sinking next to their use.
#define SCHED_DS_READ(n) __builtin_amdgcn_sched_group_barrier(0x100, (n), 0)
#define SCHED_MFMA(n) __builtin_amdgcn_sched_group_barrier(0x008, (n), 0)
#define SCHED_VALU(n) __builtin_amdgcn_sched_group_barrier(0x002, (n), 0)
// The same with an explicit pipeline id: groups are only ordered against groups of their own id,
// and the backend places long pipelines badly, so every row block of a phase gets its own.
#define SCHED_DS_READ_ID(n, id) __builtin_amdgcn_sched_group_barrier(0x100, (n), (id))
#define SCHED_MFMA_ID(n, id) __builtin_amdgcn_sched_group_barrier(0x008, (n), (id))
#define SCHED_VALU_ID(n, id) __builtin_amdgcn_sched_group_barrier(0x002, (n), (id))

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a
// constant expression in the body (the scheduling-group builtins need one).
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Lane n of every 16-lane row gets the value lane n+1 of that row holds (lane 15 gets 0):
// DPP row_shl:1.
__device__ __forceinline__ unsigned int lane_from_next(unsigned int v) {
    return (unsigned int)__builtin_amdgcn_update_dpp(0, (int)v, 0x101, 0xf, 0xf, true);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Four raw scores to fp16, two per dword (one v_cvt_pkrtz_f16_f32 per pair).  Rounded toward zero:
// a finite score beyond fp16's range becomes +-65504 instead of infinity, so no clamp is needed.
// Every kernel of the forward and the backward rounds its scores with this function: P = exp2(C - LSE)
// only sums to one over a row if C is the C the forward's LSE was taken from.
__device__ __forceinline__ u32x2 pack_scores_f16(f32x4 s) {
    return (u32x2){__builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_pkrtz(s[0], s[1])),
                   __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_pkrtz(s[2], s[3]))};
}

// Toeplitz fragment of query tap `a` for this lane: element e is
// W[a][b], b = (8g + e) - 8 - n + pk, zero outside the window.  `flip` builds the
// transposed-convolution band instead (b -> c_k - 1 - b).
__device__ __forceinline__ f16x8 toeplitz_frag(const float *__restrict__ w_row, int c_k, int pk,
                                               int g, int n, bool flip) {
    f16x8 t;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        int b = 8 * g + e - kKeyHalo - n + pk;
        float v = 0.f;
        if (b >= 0 && b < c_k) v = w_row[flip ? (c_k - 1 - b) : b];
        t[e] = (_Float16)v;
    }
    return t;
}

// Bands for a compile-time tap count CQT >= c_q: the window is padded with zero
// taps in FRONT (older query rows), so tap slot t stands for tap a = t - (CQT - c_q)
// and reads score row  i + t - (CQT - 1); the padded slots read rows that exist
// (the halo above the tile) and multiply them by zero.  No run-time tap loop.
template <int CQT>
__device__ __forceinline__ void load_bands(f16x8 (&tf)[CQT], const float *__restrict__ w_head, int c_q,
                                           int c_k, int pk, int g, int n, bool flip, float mul) {
#pragma unroll
    for (int t = 0; t < CQT; ++t) {
        const int a = t - (CQT - c_q);
        f16x8 f = (f16x8)(_Float16)0.f;
        if (a >= 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                int b = 8 * g + e - kKeyHalo - n + pk;
                float v = 0.f;
                if (b >= 0 && b < c_k) v = w_head[a * c_k + (flip ? (c_k - 1 - b) : b)] * mul;
                f[e] = (_Float16)v;
            }
        }
        tf[t] = f;
    }
}

// 8 bf16 of row `row`, zeros outside [0, N); branch-free so a batch of loads can be in flight.
template <int D>
__device__ __forceinline__ u32x4 load_row16_nb(const bf16_t *__restrict__ base, int row, int N, int col) {
    const int rr = min(max(row, 0), N - 1);
    u32x4 v = *reinterpret_cast<const u32x4 *>(base + (size_t)rr * D + col);
    if (rr != row) v = (u32x4){0u, 0u, 0u, 0u};
    return v;
}

// 8 bf16 of the row nearest to `row` inside [0, N): nothing depends on the loaded value, so the
// load stays in flight until its consumer; rows outside the sequence are zeroed by the consumer
// (only tiles at the ends of the sequence have any).
template <int D>
__device__ __forceinline__ u32x4 load_row16_clamped(const bf16_t *__restrict__ base, int row, int N, int col) {
    const int rr = min(max(row, 0), N - 1);
    return *reinterpret_cast<const u32x4 *>(base + (size_t)rr * D + col);
}
__device__ __forceinline__ u32x4 zero_unless(bool keep, u32x4 v) {
    return keep ? v : (u32x4){0u, 0u, 0u, 0u};
}

// LDS transpose read (ds_read_b64_tr_b16): the 16 lanes of a group pass the
// addresses of a 4-row x 16-column block of 16-bit elements (lane p: row p/4,
// columns 4(p%4) .. +3) and lane p gets column p of the 4 rows.  With
// `row0`/`col0` the block origin inside a row-major tile of row stride `stride`
// bytes this yields, for MFMA operands whose k index runs over the tile's rows,
// k = row0 .. row0+3 for column col0 + (lane % 16).
__device__ __forceinline__ bf16x4 lds_read_tr4x16(const unsigned char *tile, int stride, int row0, int col0,
                                                  int n) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const unsigned char *ptr = tile + (row0 + (n >> 2)) * stride + (col0 + 4 * (n & 3)) * 2;
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(ptr));
    return __builtin_bit_cast(bf16x4, v);
}

// 8 bf16 (16 bytes) of row `row` at element offset `col` of a dense [N][D]
// matrix, zeros when the row is outside [0, N).
template <int D>
__device__ __forceinline__ u32x4 load_row16(const bf16_t *__restrict__ base, int row, int N, int col) {
    u32x4 z = {0u, 0u, 0u, 0u};
    if (row < 0 || row >= N) return z;
    return *reinterpret_cast<const u32x4 *>(base + (size_t)row * D + col);
}

// fp32-arithmetic fallbacks are chosen when this is false.
inline bool mfma_shape_ok(const Problem &p, int in_dt, unsigned flags) {
    return in_dt == CONVATTN_BF16 && !(flags & CONVATTN_FLAG_EXACT) && (p.d == 32 || p.d == 64 || p.d == 128) &&
           p.pk <= kMfmaMaxPk && p.c_q <= 11;
}
// The forward addresses K and V of one (batch, head) through buffer descriptors, which count
// bytes in 32 bits.
// Row / key tiles sit on the z dimension of the grids (at most 65535): the smallest forward tile has
// 88 rows, the backward kernels' tiles 128 rows or keys.
constexpr int kMaxGridZ = 65535;
inline bool mfma_fwd_shape_ok(const Problem &p, int in_dt, unsigned flags) {
    return mfma_shape_ok(p, in_dt, flags) && (size_t)p.Nk * p.d * 2 < (1ull << 31) &&
           ((long long)p.Nq + 87) / 88 <= kMaxGridZ;
}
// The backward kernels put the key taps on one 16-wide MFMA dimension.
inline bool mfma_bwd_shape_ok(const Problem &p, int in_dt, unsigned flags) {
    // (the one-pass kernel addresses Q and dO of one (batch, head) with 32-bit byte offsets)
    // (head dimension 32: the key-stationary kernels only, i.e. not the low-memory dQ pass)
    const bool d32_ok = p.d != 32 || !(flags & CONVATTN_FLAG_LOW_MEMORY);
    return mfma_shape_ok(p, in_dt, flags) && d32_ok && p.c_k <= 15 && (size_t)p.Nq * p.d * 2 < (1ull << 31) &&
           ((long long)p.Nq + 16 + 127) / 128 <= kMaxGridZ && ((long long)p.Nk + 8 + 127) / 128 <= kMaxGridZ;
}

#if defined(__HIPCC__)
// log2 of the dC scale of one (batch, head), taken from D = rowsum(dO o O) of its rows: D is linear
// in dO and of the magnitude of dP, so the power of two s with s |D|max ~ 2^8 keeps the fp16 dC
// tiles (dC = P (dP - D), times s) in fp16's normal range whatever the magnitude of dO is, which
// makes the backward linear in dO.  Every kernel of a backward pass derives the same s from the
// same D.  Called by all `nthreads` threads of a workgroup; `red` is LDS room for one float per
// wave that nothing else uses until the call returns (two barriers inside).
__device__ __forceinline__ float dc_scale_log2_from_d(const float *__restrict__ dl_b, int Nq, int tid, int nthreads,
                                                      float *red) {
    float mx = 0.f;
    for (int i = tid; i < Nq; i += nthreads) mx = fmaxf(mx, fabsf(dl_b[i]));
    mx = wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    mx = 0.f;
    for (int w2 = 0; w2 < nthreads / 64; ++w2) mx = fmaxf(mx, red[w2]);
    __syncthreads();
    return (mx > 0.f && mx < 3e38f) ? fminf(fmaxf(floorf(8.f - __log2f(mx)), -100.f), 100.f) : 0.f;
}
#endif

// Raises a kernel's dynamic LDS limit once per device (the attribute is sticky; setting it on every
// launch costs a driver call).  One instance, and one flag word, per kernel instantiation.
template <auto Kern>
inline hipError_t set_max_lds_once(int bytes) {
    static std::atomic<unsigned long long> done{0};   // one bit per device ordinal (mod 64)
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

// ---- bf16 MFMA kernels ----
hipError_t mfma_fwd(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                    const float *w, void *o, float *m, float *l, hipStream_t s);

constexpr int kMfmaDqRows = 128;   // query rows per dQ/dW workgroup (= one dW partial)
inline int mfma_dq_tiles(const Problem &p) { return (p.Nq + kMfmaDqRows - 1) / kMfmaDqRows; }
hipError_t mfma_bwd_dq_dw(const Problem &p, int out_dt, const void *q, const void *k, const void *v,
                          const void *d_o, const float *Dl, const float *lse, const float *w, void *dq,
                          float *dw_part, hipStream_t s);

// ---- whole backward with the score chain in registers (bwd_chain_mfma.hip, bwd_chain3_mfma.hip, bwd_dq_rows.hip) ----
constexpr int kKvKeysPerWg = 128;
inline int mfma_kv_tiles(const Problem &p) { return (p.Nk + 8 + kKvKeysPerWg - 1) / kKvKeysPerWg; }
// The key-stationary kernel's workgroups cover 128 keys each (+ 8:
// the dV ranges start 8 keys early); it leaves one dW partial per workgroup and dS as bf16 blocks
// [key tile of 32][row tile of 32][32 rows][32 keys], which mfma_dq_from_rows multiplies with K.
// dc_scale holds {s, log2 s} per (batch, head): the power of two dC is carried at (mfma_dc_scale).
constexpr int kChainKeys = 32, kChainRows = 32;
inline int chain_key_tiles(const Problem &p) { return mfma_kv_tiles(p) * (kKvKeysPerWg / kChainKeys); }
__host__ __device__ inline int chain_row_tiles(const Problem &p) { return (p.Nq + kChainRows - 1) / kChainRows; }
// The dS blocks of one (batch, head) are kept as [key tile][row tile]; under the causal mask key tile kt has
// only the row tiles from kt - 1 on (the rows before them see none of its keys), and only those are kept.
__host__ __device__ inline int chain_ds_first_rt(bool causal, int kt) { return causal && kt > 1 ? kt - 1 : 0; }
// blocks before key tile kt (with kt = the number of key tiles: blocks of a (batch, head))
__host__ __device__ inline long long chain_ds_block_off(bool causal, int n_rt, int kt) {
    if (!causal || kt <= 1) return (long long)kt * n_rt;
    const long long k = kt < n_rt + 1 ? kt : n_rt + 1;   // key tiles from n_rt + 1 on have no blocks
    return k * n_rt - (k - 1) * (k - 2) / 2;
}
inline size_t chain_ds_bytes(const Problem &p) {
    return (size_t)p.B * p.H * (size_t)chain_ds_block_off(p.causal != 0, chain_row_tiles(p), chain_key_tiles(p)) *
           kChainKeys * kChainRows * 2;
}
// {s, log2 s} per (batch, head) followed by 32 x 2 partial maxima per (batch, head)
inline size_t chain_scale_bytes(const Problem &p) { return (size_t)p.B * p.H * (2 + 64) * sizeof(float); }
hipError_t mfma_dc_scale(const Problem &p, const void *d_o, const void *v, float *dc_scale, hipStream_t s);
// want: bit 0 = dK and dV, bit 1 = dS blocks (for dQ) and the dW partial; dc_scale may be null when
// bit 1 is clear (the kernel then takes the scale from D).
#define CHAIN_DECL(name)                                                                                   \
    hipError_t name(const Problem &p, int out_dt, const void *q, const void *k, const void *v, const void *d_o, \
                    const float *Dl, const float *lse, const float *w, const float *dc_scale, void *dk, void *dv, \
                    void *ds_ws, float *dw_part, hipStream_t s)
CHAIN_DECL(mfma_bwd_chain_kv);
CHAIN_DECL(mfma_bwd_chain_qw);
CHAIN_DECL(mfma_bwd_chain_all);
// the same with three waves per SIMD (bwd_chain3_mfma.hip): windows of up to 6 query taps
CHAIN_DECL(mfma_bwd_chain3_kv);
CHAIN_DECL(mfma_bwd_chain3_qw);
CHAIN_DECL(mfma_bwd_chain3_all);
#undef CHAIN_DECL
inline hipError_t mfma_bwd_chain(const Problem &p, int out_dt, int want, const void *q, const void *k, const void *v,
                                 const void *d_o, const float *Dl, const float *lse, const float *w,
                                 const float *dc_scale, void *dk, void *dv, void *ds_ws, float *dw_part,
                                 hipStream_t s) {
    if (p.c_q <= 6) {
        if (want == 1) return mfma_bwd_chain3_kv(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
        if (want == 2) return mfma_bwd_chain3_qw(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
        return mfma_bwd_chain3_all(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    }
    if (want == 1) return mfma_bwd_chain_kv(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    if (want == 2) return mfma_bwd_chain_qw(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
    return mfma_bwd_chain_all(p, out_dt, q, k, v, d_o, Dl, lse, w, dc_scale, dk, dv, ds_ws, dw_part, s);
}
hipError_t mfma_dq_from_rows(const Problem &p, int out_dt, const void *k, const void *ds_ws,
                             const float *dc_scale, void *dq, hipStream_t s);

// ---- decode as an HBM stream (decode_stream.hip) ----
bool decode_stream_ok(const Problem &p, int in_dt, unsigned flags);
// Where the decode kernel finds K and V rows beyond Problem's batch / head strides.
struct KvArgs {
    const int *table;       // block table [B][table_stride] of page numbers, or null: contiguous rows
    const int *seq_lens;    // keys per batch entry [B] (clamped to Problem::Nk), or null: Nk for all
    long long page_stride;  // elements between pages of the pool
    int table_stride;
    int page_shift;         // log2 of the keys per page
    int group;              // query heads per KV head (>= 1)
};
int decode_heads_per_wg(const Problem &p, int group);
hipError_t decode_stream_kv(const Problem &p, const KvArgs &kv, const void *q, const void *k, const void *v,
                            const float *w, float *o_part, float *m_part, float *l_part, hipStream_t s);
hipError_t decode_stream(const Problem &p, const void *q, const void *k, const void *v, const float *w,
                         float *o_part, float *m_part, float *l_part, hipStream_t s);

}  // namespace convattn
