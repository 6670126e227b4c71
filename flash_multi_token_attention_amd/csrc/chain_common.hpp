// Shared pieces of the key-stationary backward kernels (bwd_chain_mfma.hip, bwd_chain3_mfma.hip): LDS layout,
// fragment addressing, DPP row windows, Toeplitz bands for the packed operand order, the argument block.
#pragma once
#include <type_traits>

#include "mfma_common.hpp"

namespace convattn {
namespace chain {

constexpr int NP = 4;            // wave pairs = 32-key ranges per workgroup
constexpr int WK = 32;           // own keys per pair
constexpr int BKW = NP * WK;     // 128 keys per workgroup
constexpr int BR = 32;           // query rows per tile
constexpr int NSB = 4;           // S^T blocks of a pair: keys c0-16+16kb
constexpr int NCB = 3;           // C / dP / dC blocks: keys c0-8+16cb
constexpr int NDB = 2;           // dS blocks: keys c0+16sb
constexpr int SST = 112;         // bytes per row of the S tile in LDS (48 keys fp16 + 16)
constexpr int S_RING = 72;       // rows of the S ring: a tile being written, the tile before it and 8 rows more (>= c_q - 1)
constexpr int kBandTab = 352;    // bytes of a compact band table: 44 slots of 4 fp16 (see band_tab_build)
constexpr int CST = 112;         // bytes per row of the dC tile (48 keys fp16 + 16)
constexpr int PST = 72;          // bytes per row of the P and dS tiles (32 keys bf16 + 8)
static_assert(BKW == kKvKeysPerWg && WK == kChainKeys && BR == kChainRows, "dS workspace layout");

template <int D, int CQT> struct ChainLds {
    // Q / dO tiles are filled by buffer loads with the LDS modifier (64 lanes = 1 KB of consecutive
    // LDS), which rules out padded rows.  A tile of 32 rows is kept as [k-step ks][row parity f]
    // [row pair n][64 bytes]: the 4 chunks of 16 bytes that row 2n + f holds of head-dim columns
    // 32 ks .. 32 ks + 31, chunk c at position c ^ (n / 4 mod 4).  Row fragments (lane n reads row
    // 2n + f) and transposed fragments then touch every bank equally often, and k-step, parity and
    // head-dim block are constant offsets from one lane address.
    static constexpr int RST = D * 2;                               // bytes per Q / dO row
    static constexpr int tile_bytes = BR * RST;
    static constexpr int q_off = 0, q_slots = 4;                    // tiles it-2 .. it+1
    static constexpr int g_off = q_off + q_slots * tile_bytes, g_slots = 3;  // tiles it-1 .. it+1
    static constexpr int stat_off = g_off + g_slots * tile_bytes;   // LSE and D of a tile: two slots
    static constexpr int stat_bytes = 2 * (2 * BR * 4);
    // bands, then flipped bands: one KB of ready-made fragments per tap slot, or (windows of more than 8
    // query taps, where those do not fit) one compact table per tap slot that the lanes read their fragments from
    static constexpr bool compact_bands = CQT > 8;
    static constexpr int band_slot = compact_bands ? kBandTab : 1024;
    static constexpr int band_off = stat_off + stat_bytes;
    static constexpr int band_bytes = 2 * CQT * band_slot;
    static constexpr int pair_off = band_off + band_bytes;
    static constexpr int ring_rows = CQT > 9 ? S_RING + 4 : S_RING;   // >= 64 + CQT - 1
    static constexpr int s_bytes = ring_rows * SST;
    static constexpr int c_bytes = 2 * BR * CST;
    static constexpr int p_bytes = 2 * BR * PST;
    static constexpr int ds_bytes = BR * PST;
    static constexpr int pair_bytes = s_bytes + c_bytes + p_bytes + ds_bytes;
    static constexpr int total = pair_off + NP * pair_bytes;
    static_assert(2 * CQT * 2 * 1024 <= NP * pair_bytes, "room for the dW accumulators (they take the place of the pairs' tiles)");
};

// A lane-dependent LDS offset the compiler may not fold or hoist: what is added to it afterwards
// stays a constant and ends up in the instructions' offset fields instead of one address register
// per fragment.
__device__ __forceinline__ unsigned int opaque(unsigned int x) {
    asm volatile("" : "+v"(x));
    return x;
}

__device__ __forceinline__ bf16x4 lds_tr64(const unsigned char *ptr) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(ptr));
    return __builtin_bit_cast(bf16x4, v);
}
// Transposed fragment of a row-major tile of 16-bit elements with `stride` bytes per row:
// k = rows 4g .. 4g+3 then 16+4g .. 16+4g+3, column col0 + n.  `lane_ptr` is the tile's address plus
// tr_lane_off(stride, g, n).
__device__ __forceinline__ unsigned int tr_lane_off(int stride, int g, int n) {
    return (4 * g + (n >> 2)) * stride + 4 * (n & 3) * 2;
}
__device__ __forceinline__ bf16x8 read_tr(const unsigned char *lane_ptr, int stride, int col0) {
    bf16x4 lo = lds_tr64(lane_ptr + col0 * 2);
    bf16x4 hi = lds_tr64(lane_ptr + 16 * stride + col0 * 2);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

template <int CTRL>
__device__ __forceinline__ unsigned int dpp_keep(unsigned int old, unsigned int src) {
    return (unsigned int)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, 0xf, 0xf, false);
}
// A DPP move that writes every lane (rotations): no previous value to keep.
template <int CTRL>
__device__ __forceinline__ unsigned int dpp_mov(unsigned int src) {
    return (unsigned int)__builtin_amdgcn_mov_dpp((int)src, CTRL, 0xf, 0xf, true);
}
// Lane n of a row of 16 gets cur[n - S] for n >= S and prev[16 + n - S] below: a window that
// starts S lanes before `cur` in the sequence prev | cur.
template <int S>
__device__ __forceinline__ unsigned int win_up(unsigned int prev, unsigned int cur) {
    if constexpr (S == 0) {
        return cur;
    } else {
        const unsigned int x = dpp_mov<0x120 + S>(prev);  // row_ror:S
        return dpp_keep<0x110 + S>(x, cur);               // row_shr:S, lanes below S keep x
    }
}
// Lane n gets a[n + S] for n + S < 16 and b[n + S - 16] above: a window that starts S lanes into
// `a` in the sequence a | b.
template <int S>
__device__ __forceinline__ unsigned int win_down(unsigned int a, unsigned int b) {
    if constexpr (S == 0) {
        return a;
    } else {
        const unsigned int x = dpp_mov<0x120 + 16 - S>(b);  // row_ror:(16-S)
        return dpp_keep<0x100 + S>(x, a);                   // row_shl:S, the last S lanes keep x
    }
}

__device__ __forceinline__ unsigned int pack_f16_rtz(float a, float b) {
    return __builtin_bit_cast(unsigned int, __builtin_amdgcn_cvt_pkrtz(a, b));
}

// Toeplitz bands for the packed operand order: k slot 8g+e of a 32-key window is key 4g+e of its
// first 16-key block for e < 4 and key 4g+e-4 of its second for e >= 4; the output block starts 8
// keys into the window.  Tap slot t stands for query tap a = t - (CQT - c_q) (zero taps in front).
// `flip` builds the bands of the transposed convolution.
template <int CQT>
__device__ __forceinline__ f16x8 band_frag(int t, const float *__restrict__ w_head, int c_q, int c_k, int pk,
                                           int g, int n, bool flip, float mul) {
    const int a = t - (CQT - c_q);
    // (unconditional loads from clamped indices: the eight of a fragment are in flight together)
    const float *row = w_head + max(a, 0) * c_k;
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int kappa = e < 4 ? 4 * g + e : 16 + 4 * g + e - 4;
        const int off = kappa - kKeyHalo - n;
        const int bb = flip ? pk - off : pk + off;
        v[e] = row[min(max(bb, 0), c_k - 1)];
        if (a < 0 || bb < 0 || bb >= c_k) v[e] = 0.f;
    }
    f16x8 f;
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = (_Float16)(v[e] * mul);
    return f;
}

// The same bands as compact tables.  A fragment is Toeplitz in (slot, lane): its value at k slot e of lane
// (g, n) is T[x] with x = kappa(e, g) - n in [-15, 31], T[x] = w[a][pk +- (x - 8)] (zero outside the window),
// and the eight k slots of a lane are x0 .. x0+3 and x0+16 .. x0+19 with x0 = 4g - n.  A table holds T as 44
// slots of 4 fp16: slot 4k + r (k = 0..10, r = 0..3) = T[4k + r - 15 .. 4k + r - 12], so that lane (g, n) finds
// its two groups at the slots 4k + r and 4(k + 4) + r with k = g - n/4 + 3, r = 3 - n%4: two aligned 8-byte
// reads, 128 bytes apart, and the 28 distinct addresses of a wave fall into distinct banks.
__device__ __forceinline__ unsigned int band_tab_lane_off(int g, int n) {
    return (unsigned int)(((g - (n >> 2) + 3) * 4 + 3 - (n & 3)) * 8);
}
__device__ __forceinline__ f16x8 band_tab_read(const unsigned char *lane_ptr) {
    const u32x2 lo = *reinterpret_cast<const u32x2 *>(lane_ptr), hi = *reinterpret_cast<const u32x2 *>(lane_ptr + 128);
    return __builtin_bit_cast(f16x8, (u32x4){lo[0], lo[1], hi[0], hi[1]});
}
// Tables of all tap slots: CQT direct ones (times mul_direct), then CQT flipped ones (times mul_flipped), built
// by all `nthreads` threads of the workgroup; a barrier has to follow before they are read.
template <int CQT>
__device__ __forceinline__ void band_tab_build(unsigned char *tabs, const float *__restrict__ w_head, int c_q, int c_k,
                                               int pk, float mul_direct, float mul_flipped, int tid, int nthreads) {
    constexpr int PER = kBandTab / 2;   // fp16 entries per table
    for (int i = tid; i < 2 * CQT * PER; i += nthreads) {
        const int td = i / PER, q = i - td * PER, flip = td >= CQT, t = td - flip * CQT;
        const int a = t - (CQT - c_q), x = q - (q >> 2) * 3 - 15;   // entry e of slot s: x = s + e - 15
        const int bb = flip ? pk - (x - kKeyHalo) : pk + (x - kKeyHalo);
        float v = 0.f;
        if (a >= 0 && bb >= 0 && bb < c_k) v = w_head[a * c_k + bb] * (flip ? mul_flipped : mul_direct);
        reinterpret_cast<_Float16 *>(tabs)[i] = (_Float16)v;
    }
}

// Kernel arguments as one block: each role reads them from the kernel argument segment with
// scalar loads (arguments of a device function would arrive in vector registers).
struct ChainArgs {
    Problem p;
    const bf16_t *Q, *K, *V, *dO;
    const float *Dl, *LSE, *W, *dc_scale;
    void *dK, *dV;
    bf16_t *dS_ws;
    float *dW_part;
    int n_rt;
};

// The kernel argument segment lives in the constant address space; host passes of the compiler
// do not know that attribute.
#if defined(__HIP_DEVICE_COMPILE__)
#define CHAIN_CONST_AS __attribute__((address_space(4)))
#else
#define CHAIN_CONST_AS
#endif

}  // namespace chain
}  // namespace convattn
