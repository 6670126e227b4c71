// C ABI of the conv-attention library: host-side argument checks, kernel-family
// selection and launches.  Nothing here allocates or synchronises.
#include <math.h>
#include <string.h>

#include <mutex>

#include "common.hpp"
#include "mfma_common.hpp"

using namespace convattn;

namespace {

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_dtype(int dt) { return (dt == CONVATTN_BF16 || dt == CONVATTN_F32) ? 0 : CONVATTN_ERR_DTYPE; }

int validate(const convattn_desc *d, int op, Problem *out) {
    if (!d) return CONVATTN_ERR_NULL;
    if (op != CONVATTN_OP_FWD && op != CONVATTN_OP_BWD && op != CONVATTN_OP_DECODE)
        return CONVATTN_ERR_SHAPE;
    if (d->B <= 0 || d->H <= 0 || d->Nq <= 0 || d->Nk <= 0 || d->d <= 0) return CONVATTN_ERR_SHAPE;
    if (d->d % 8 != 0 || d->d > kMaxD) return CONVATTN_ERR_HEAD_DIM;
    if (d->c_q < 1 || d->c_q > kMaxCq || d->c_k < 1 || d->c_k > kMaxCk || d->c_k % 2 == 0)
        return CONVATTN_ERR_KERNEL_SIZE;
    if (check_dtype(d->in_dtype) || check_dtype(d->out_dtype)) return CONVATTN_ERR_DTYPE;
    if (!isfinite(d->scale)) return CONVATTN_ERR_SCALE;
    if ((long long)d->B * d->H > 0x7fffffffLL / 64) return CONVATTN_ERR_TOO_LARGE;
    if (d->B > 65535 || d->H > 65535) return CONVATTN_ERR_TOO_LARGE;
    Problem p;
    p.B = d->B; p.H = d->H; p.Nq = d->Nq; p.Nk = d->Nk; p.d = d->d;
    p.c_q = d->c_q; p.c_k = d->c_k; p.pq = d->c_q - 1; p.pk = (d->c_k - 1) / 2;
    p.scale = d->scale; p.causal = d->causal ? 1 : 0; p.n_splits = 1;
    p.kv_hstride = (long long)d->Nk * d->d; p.kv_bstride = p.kv_hstride * d->H;
    if (op == CONVATTN_OP_DECODE) {
        if (d->Nq > 16) return CONVATTN_ERR_QROWS;
        if (d->n_splits < 1 || d->n_splits > d->Nk || d->n_splits > 1024) return CONVATTN_ERR_SPLITS;
        p.n_splits = d->n_splits;
        if (generic_decode_lds(p) > kLdsBytes) return CONVATTN_ERR_LDS;
    } else {
        if (p.causal && d->Nq != d->Nk) return CONVATTN_ERR_CAUSAL_SHAPE;
        const size_t lds = (op == CONVATTN_OP_FWD) ? generic_fwd_lds(p) : generic_bwd_lds(p);
        if (lds > kLdsBytes) return CONVATTN_ERR_LDS;
    }
    if (out) *out = p;
    return CONVATTN_OK;
}

// 0 = fp32-arithmetic kernels, 1 = bf16 MFMA kernels.
int pick_path(const convattn_desc *d, const Problem &p, int op) {
    if (op == CONVATTN_OP_FWD) return mfma_fwd_shape_ok(p, d->in_dtype, d->flags) ? 1 : 0;
    if (op == CONVATTN_OP_BWD) return mfma_bwd_shape_ok(p, d->in_dtype, d->flags) ? 1 : 0;
    if (op == CONVATTN_OP_DECODE) return decode_stream_ok(p, d->in_dtype, d->flags) ? 1 : 0;
    return 0;
}

int dw_tiles(const convattn_desc *d, const Problem &p) {
    return pick_path(d, p, CONVATTN_OP_BWD) == 1 ? mfma_dq_tiles(p) : generic_q_tiles(p);
}

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
size_t fused_dw_bytes(const Problem &p) {
    return (size_t)p.B * p.H * mfma_kv_tiles(p) * p.c_q * p.c_k * sizeof(float);
}

// Scratch of convattn_decode_noalloc: the split partials of one decode step, held by every GPU
// the library runs on until the process ends.  Host code reaches it only through the address
// hipGetSymbolAddress returns for the current device (kept per device).
constexpr size_t kDecodeScratchBytes = CONVATTN_DECODE_NOALLOC_MAX_BYTES;
static __device__ __align__(256) unsigned char scratch[kDecodeScratchBytes];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up once per device); hipError_t in *err.
void *decode_scratch(hipError_t *err) {
    int dev = -1;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) { *err = hipErrorInvalidDevice; return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        *err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (*err != hipSuccess) return nullptr;
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

#define REQUIRE_PTR(x)                                   \
    do {                                                 \
        if (!(x)) return CONVATTN_ERR_NULL;              \
        if (!aligned16(x)) return CONVATTN_ERR_ALIGN;    \
    } while (0)

}  // namespace

extern "C" {

int convattn_version(void) { return CONVATTN_VERSION; }

const char *convattn_strerror(int code) {
    switch (code) {
        case CONVATTN_OK: return "ok";
        case CONVATTN_ERR_NULL: return "a required pointer is NULL";
        case CONVATTN_ERR_SHAPE: return "B, H, Nq, Nk and d must be positive";
        case CONVATTN_ERR_HEAD_DIM: return "Unsupported head dimension: d must be a multiple of 8 and at most 128";
        case CONVATTN_ERR_KERNEL_SIZE: return "Unsupported kernel size: c_q must be in 1..16 and c_k odd in 1..33";
        case CONVATTN_ERR_DTYPE: return "tensors must be bfloat16 or float32";
        case CONVATTN_ERR_ALIGN: return "device pointers must be 16-byte aligned";
        case CONVATTN_ERR_SPLITS: return "k_splits must be positive and cannot be larger than seq_len_k (or 1024)";
        case CONVATTN_ERR_QROWS: return "Q sequence length must be between 1 and 16 for inference";
        case CONVATTN_ERR_SCALE: return "scale must be finite";
        case CONVATTN_ERR_CAUSAL_SHAPE: return "causal conv-attention needs seq_len_q == seq_len_k";
        case CONVATTN_ERR_LDS: return "convolution window too large for the 160 KB of LDS at this head dimension";
        case CONVATTN_ERR_TOO_LARGE: return "batch or head count too large for one launch";
        case CONVATTN_ERR_KV_LAYOUT: return "KV layout rejected: H must be a multiple of H_kv, page_size a power of two >= 16, strides multiples of 8 that cover a page / a sequence, the block table long enough, and the descriptor one of the streaming decode kernel (bf16, d 32, 64 or 128, c_k <= 17)";
        case CONVATTN_ERR_HEADMIX: return "head-mixing attention: n_heads must be 16 or 32, d_model 32, 64 or 128, inputs bf16";
        case CONVATTN_ERR_SCRATCH: return "the split partials of this decode step do not fit the library's built-in scratch (convattn_decode_noalloc): use fewer splits or convattn_decode";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "unknown convattn status";
}

int convattn_validate(const convattn_desc *desc, int op) { return validate(desc, op, nullptr); }

int convattn_kernel_path(const convattn_desc *desc, int op) {
    Problem p;
    int rc = validate(desc, op, &p);
    if (rc) return rc;
    return pick_path(desc, p, op);
}

int convattn_fwd(const convattn_desc *desc, const void *q, const void *k, const void *v,
                 const float *w, void *o, float *m, float *l, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_FWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(w);
    REQUIRE_PTR(o); REQUIRE_PTR(m); REQUIRE_PTR(l);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pick_path(desc, p, CONVATTN_OP_FWD) == 1)
        return (int)mfma_fwd(p, desc->out_dtype, q, k, v, w, o, m, l, s);
    return (int)generic_fwd(p, desc->in_dtype, desc->out_dtype, q, k, v, w, o, m, l, s);
}

int convattn_bwd_preprocess(const convattn_desc *desc, const void *o, const void *d_o,
                            const float *m, const float *l, float *D, float *lse, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(o); REQUIRE_PTR(d_o); REQUIRE_PTR(m); REQUIRE_PTR(l); REQUIRE_PTR(D); REQUIRE_PTR(lse);
    return (int)bwd_preprocess(p, desc->in_dtype, desc->out_dtype, o, d_o, m, l, D, lse,
                               static_cast<hipStream_t>(stream));
}

// Workspace of the one-pass backward on the MFMA path: dS blocks, dW partials and the dC scale of
// every (batch, head), each part 256-byte aligned.
struct FusedWs {
    size_t ds_bytes, part_off, scale_off, total;
};
static FusedWs fused_ws(const Problem &p) {
    FusedWs w;
    w.ds_bytes = chain_ds_bytes(p);
    w.part_off = align256(w.ds_bytes);
    w.scale_off = w.part_off + align256(fused_dw_bytes(p));
    w.total = w.scale_off + align256(chain_scale_bytes(p));
    return w;
}

// The dQ + dW pass on the MFMA path is the key-stationary kernel without its dK / dV half plus the
// dQ = dS K product: its "dW partial buffer" is the one-pass backward's workspace (dS blocks, dW
// partials, dC scales).  With CONVATTN_FLAG_LOW_MEMORY it is the query-stationary kernel of
// bwd_dq_mfma.hip, whose buffer holds dW partials only.
static bool dq_dw_uses_chain(const convattn_desc *desc, const Problem &p) {
    return pick_path(desc, p, CONVATTN_OP_BWD) == 1 && !(desc->flags & CONVATTN_FLAG_LOW_MEMORY);
}

size_t convattn_dw_partial_bytes(const convattn_desc *desc) {
    Problem p;
    if (validate(desc, CONVATTN_OP_BWD, &p)) return 0;
    if (dq_dw_uses_chain(desc, p)) return fused_ws(p).total;
    return (size_t)p.B * p.H * dw_tiles(desc, p) * p.c_q * p.c_k * sizeof(float);
}

int convattn_bwd_dq_dw(const convattn_desc *desc, const void *q, const void *k, const void *v,
                       const void *d_o, const float *D, const float *lse, const float *w, void *dq,
                       float *dw_partial, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(d_o); REQUIRE_PTR(D);
    REQUIRE_PTR(lse); REQUIRE_PTR(w); REQUIRE_PTR(dq); REQUIRE_PTR(dw_partial);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dq_dw_uses_chain(desc, p)) {
        unsigned char *ws = reinterpret_cast<unsigned char *>(dw_partial);
        const FusedWs lay = fused_ws(p);
        float *scale = reinterpret_cast<float *>(ws + lay.scale_off);
        hipError_t e = mfma_dc_scale(p, d_o, v, scale, s);
        if (e == hipSuccess)
            e = mfma_bwd_chain(p, desc->out_dtype, 2, q, k, v, d_o, D, lse, w, scale, nullptr, nullptr, ws,
                               reinterpret_cast<float *>(ws + lay.part_off), s);
        if (e == hipSuccess) e = mfma_dq_from_rows(p, desc->out_dtype, k, ws, scale, dq, s);
        return (int)e;
    }
    if (pick_path(desc, p, CONVATTN_OP_BWD) == 1)
        return (int)mfma_bwd_dq_dw(p, desc->out_dtype, q, k, v, d_o, D, lse, w, dq, dw_partial, s);
    return (int)generic_bwd_dq_dw(p, desc->in_dtype, desc->out_dtype, q, k, v, d_o, D, lse, w, dq,
                                  dw_partial, s);
}

int convattn_dw_reduce(const convattn_desc *desc, const float *dw_partial, float *dw, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(dw_partial); REQUIRE_PTR(dw);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dq_dw_uses_chain(desc, p)) {
        const unsigned char *ws = reinterpret_cast<const unsigned char *>(dw_partial);
        return (int)dw_reduce(p, mfma_kv_tiles(p), reinterpret_cast<const float *>(ws + fused_ws(p).part_off), dw, s);
    }
    return (int)dw_reduce(p, dw_tiles(desc, p), dw_partial, dw, s);
}

int convattn_bwd_dkdv(const convattn_desc *desc, const void *q, const void *k, const void *v,
                      const void *d_o, const float *D, const float *lse, const float *w, void *dk,
                      void *dv, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(d_o); REQUIRE_PTR(D);
    REQUIRE_PTR(lse); REQUIRE_PTR(w); REQUIRE_PTR(dk); REQUIRE_PTR(dv);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pick_path(desc, p, CONVATTN_OP_BWD) == 1)   // the key-stationary kernel without dS and dW; it scales dC by D
        return (int)mfma_bwd_chain(p, desc->out_dtype, 1, q, k, v, d_o, D, lse, w, nullptr, dk, dv, nullptr, nullptr, s);
    return (int)generic_bwd_dkdv(p, desc->in_dtype, desc->out_dtype, q, k, v, d_o, D, lse, w, dk, dv, s);
}

size_t convattn_bwd_fused_workspace_bytes(const convattn_desc *desc) {
    Problem p;
    if (validate(desc, CONVATTN_OP_BWD, &p)) return 0;
    if (pick_path(desc, p, CONVATTN_OP_BWD) != 1) return align256(convattn_dw_partial_bytes(desc));
    return fused_ws(p).total;
}

int convattn_bwd_fused_dkdv(const convattn_desc *desc, const void *q, const void *k, const void *v,
                            const void *d_o, const float *D, const float *lse, const float *w, void *dk,
                            void *dv, void *workspace, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(d_o); REQUIRE_PTR(D);
    REQUIRE_PTR(lse); REQUIRE_PTR(w); REQUIRE_PTR(dk); REQUIRE_PTR(dv); REQUIRE_PTR(workspace);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pick_path(desc, p, CONVATTN_OP_BWD) != 1)
        return (int)generic_bwd_dkdv(p, desc->in_dtype, desc->out_dtype, q, k, v, d_o, D, lse, w, dk, dv, s);
    unsigned char *ws = static_cast<unsigned char *>(workspace);
    const FusedWs lay = fused_ws(p);
    float *part = reinterpret_cast<float *>(ws + lay.part_off);
    float *scale = reinterpret_cast<float *>(ws + lay.scale_off);
    hipError_t e = mfma_dc_scale(p, d_o, v, scale, s);
    if (e != hipSuccess) return (int)e;
    return (int)mfma_bwd_chain(p, desc->out_dtype, 3, q, k, v, d_o, D, lse, w, scale, dk, dv, ws, part, s);
}

int convattn_bwd_fused_dq(const convattn_desc *desc, const void *q, const void *k, const void *v,
                          const void *d_o, const float *D, const float *lse, const float *w, void *dq,
                          void *workspace, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(k); REQUIRE_PTR(dq); REQUIRE_PTR(workspace);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pick_path(desc, p, CONVATTN_OP_BWD) != 1) {
        // fp32-arithmetic kernels: the separate dQ pass, its dW partials go to the workspace
        REQUIRE_PTR(q); REQUIRE_PTR(v); REQUIRE_PTR(d_o); REQUIRE_PTR(D); REQUIRE_PTR(lse); REQUIRE_PTR(w);
        return (int)generic_bwd_dq_dw(p, desc->in_dtype, desc->out_dtype, q, k, v, d_o, D, lse, w, dq,
                                      static_cast<float *>(workspace), s);
    }
    const FusedWs lay = fused_ws(p);
    const float *scale = reinterpret_cast<const float *>(static_cast<const unsigned char *>(workspace) + lay.scale_off);
    return (int)mfma_dq_from_rows(p, desc->out_dtype, k, workspace, scale, dq, s);
}

int convattn_bwd_fused_dw(const convattn_desc *desc, const void *workspace, float *dw, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_BWD, &p);
    if (rc) return rc;
    REQUIRE_PTR(workspace); REQUIRE_PTR(dw);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pick_path(desc, p, CONVATTN_OP_BWD) != 1)
        return (int)dw_reduce(p, dw_tiles(desc, p), static_cast<const float *>(workspace), dw, s);
    const unsigned char *ws = static_cast<const unsigned char *>(workspace);
    return (int)dw_reduce(p, mfma_kv_tiles(p), reinterpret_cast<const float *>(ws + fused_ws(p).part_off), dw, s);
}

int convattn_bwd_fused(const convattn_desc *desc, const void *q, const void *k, const void *v,
                       const void *d_o, const float *D, const float *lse, const float *w, void *dq,
                       void *dk, void *dv, float *dw, void *workspace, void *stream) {
    int rc = convattn_bwd_fused_dkdv(desc, q, k, v, d_o, D, lse, w, dk, dv, workspace, stream);
    if (rc == 0) rc = convattn_bwd_fused_dq(desc, q, k, v, d_o, D, lse, w, dq, workspace, stream);
    if (rc == 0) rc = convattn_bwd_fused_dw(desc, workspace, dw, stream);
    return rc;
}

size_t convattn_decode_partial_bytes(const convattn_desc *desc) {
    Problem p;
    if (validate(desc, CONVATTN_OP_DECODE, &p)) return 0;
    return (size_t)p.B * p.H * p.n_splits * p.d * sizeof(float);
}

int convattn_decode(const convattn_desc *desc, const void *q, const void *k, const void *v,
                    const float *w, float *o_part, float *m_part, float *l_part, void *stream) {
    if (!desc) return CONVATTN_ERR_NULL;
    const long long hs = (long long)desc->Nk * desc->d;
    return convattn_decode_strided(desc, q, k, v, w, hs * desc->H, hs, o_part, m_part, l_part, stream);
}

int convattn_decode_strided(const convattn_desc *desc, const void *q, const void *k, const void *v,
                            const float *w, long long kv_batch_stride, long long kv_head_stride,
                            float *o_part, float *m_part, float *l_part, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_DECODE, &p);
    if (rc) return rc;
    // rows of a head stay dense (d elements apart) and 16-byte aligned; heads and batches must not overlap
    if (kv_head_stride < (long long)p.Nk * p.d || kv_head_stride % 8 != 0 || kv_batch_stride % 8 != 0 ||
        (p.B > 1 && kv_batch_stride < (long long)p.Nk * p.d))
        return CONVATTN_ERR_SHAPE;
    p.kv_bstride = kv_batch_stride; p.kv_hstride = kv_head_stride;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(w);
    REQUIRE_PTR(o_part); REQUIRE_PTR(m_part); REQUIRE_PTR(l_part);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (pick_path(desc, p, CONVATTN_OP_DECODE) == 1)
        return (int)decode_stream(p, q, k, v, w, o_part, m_part, l_part, s);
    return (int)generic_decode(p, desc->in_dtype, q, k, v, w, o_part, m_part, l_part, s);
}

int convattn_decode_kv(const convattn_desc *desc, const void *q, const void *k, const void *v,
                       const convattn_kv_layout *kv, const float *w, float *o_part, float *m_part,
                       float *l_part, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_DECODE, &p);
    if (rc) return rc;
    if (!kv) return CONVATTN_ERR_NULL;
    if (pick_path(desc, p, CONVATTN_OP_DECODE) != 1) return CONVATTN_ERR_KV_LAYOUT;
    const int h_kv = kv->H_kv > 0 ? kv->H_kv : p.H;
    if (h_kv > p.H || p.H % h_kv != 0 || kv->reserved != 0) return CONVATTN_ERR_KV_LAYOUT;
    KvArgs a = {};
    a.group = p.H / h_kv;
    a.seq_lens = kv->seq_lens;
    const long long row = p.d;
    if (kv->page_size == 0) {
        // contiguous rows per (batch, KV head); KV heads and batches must not overlap
        if (kv->head_stride < (long long)p.Nk * row || kv->head_stride % 8 != 0 || kv->batch_stride % 8 != 0 ||
            (p.B > 1 && kv->batch_stride < (long long)p.Nk * row))
            return CONVATTN_ERR_KV_LAYOUT;
        p.kv_bstride = kv->batch_stride;
    } else {
        const int ps = kv->page_size;
        if (ps < 16 || (ps & (ps - 1)) != 0 || !kv->block_table || kv->head_stride < (long long)ps * row ||
            kv->head_stride % 8 != 0 || kv->page_stride % 8 != 0 || kv->page_stride < (long long)ps * row ||
            (long long)kv->table_stride * ps < p.Nk)
            return CONVATTN_ERR_KV_LAYOUT;
        a.table = kv->block_table;
        a.table_stride = kv->table_stride;
        a.page_stride = kv->page_stride;
        a.page_shift = __builtin_ctz((unsigned)ps);
        p.kv_bstride = 0;
    }
    p.kv_hstride = kv->head_stride;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(w);
    REQUIRE_PTR(o_part); REQUIRE_PTR(m_part); REQUIRE_PTR(l_part);
    return (int)decode_stream_kv(p, a, q, k, v, w, o_part, m_part, l_part, static_cast<hipStream_t>(stream));
}

size_t convattn_decode_noalloc_bytes(const convattn_desc *desc) {
    Problem p;
    if (validate(desc, CONVATTN_OP_DECODE, &p)) return 0;
    const size_t slots = (size_t)p.B * p.H * p.n_splits;
    return align256(slots * p.d * sizeof(float)) + 2 * align256(slots * sizeof(float));
}

int convattn_decode_noalloc(const convattn_desc *desc, const void *q, const void *k, const void *v,
                            const float *w, long long kv_batch_stride, long long kv_head_stride, void *o,
                            float *m, float *l, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_DECODE, &p);
    if (rc) return rc;
    REQUIRE_PTR(o); REQUIRE_PTR(m); REQUIRE_PTR(l);
    if (convattn_decode_noalloc_bytes(desc) > kDecodeScratchBytes) return CONVATTN_ERR_SCRATCH;
    hipError_t err = hipSuccess;
    unsigned char *base = static_cast<unsigned char *>(decode_scratch(&err));
    if (!base) return (int)err;
    const size_t slots = (size_t)p.B * p.H * p.n_splits;
    float *o_part = reinterpret_cast<float *>(base);
    float *m_part = reinterpret_cast<float *>(base + align256(slots * p.d * sizeof(float)));
    float *l_part = reinterpret_cast<float *>(base + align256(slots * p.d * sizeof(float)) + align256(slots * sizeof(float)));
    // every (batch, head, split) slot is written by the first kernel before the second reads it:
    // nothing of the previous call's contents is used
    rc = convattn_decode_strided(desc, q, k, v, w, kv_batch_stride, kv_head_stride, o_part, m_part, l_part, stream);
    if (rc) return rc;
    return convattn_decode_combine(desc, o_part, m_part, l_part, o, m, l, stream);
}

int convattn_decode_combine(const convattn_desc *desc, const float *o_part, const float *m_part,
                            const float *l_part, void *o, float *m, float *l, void *stream) {
    Problem p;
    int rc = validate(desc, CONVATTN_OP_DECODE, &p);
    if (rc) return rc;
    REQUIRE_PTR(o_part); REQUIRE_PTR(m_part); REQUIRE_PTR(l_part);
    REQUIRE_PTR(o); REQUIRE_PTR(m); REQUIRE_PTR(l);
    return (int)decode_combine(p, desc->out_dtype, o_part, m_part, l_part, o, m, l,
                               static_cast<hipStream_t>(stream));
}

// ---- head-mixing attention ----
static int headmix_check(const convattn_headmix_desc *d) {
    if (!d) return CONVATTN_ERR_NULL;
    if (d->B <= 0 || d->N <= 0) return CONVATTN_ERR_SHAPE;
    if ((d->H != 16 && d->H != 32) || (d->d != 32 && d->d != 64 && d->d != 128)) return CONVATTN_ERR_HEADMIX;
    if (d->in_dtype != CONVATTN_BF16) return CONVATTN_ERR_HEADMIX;
    if (d->out_dtype != CONVATTN_BF16 && d->out_dtype != CONVATTN_F32) return CONVATTN_ERR_DTYPE;
    if (!(d->scale == d->scale) || d->scale - d->scale != 0.f) return CONVATTN_ERR_SCALE;
    if ((long long)d->B > 65535) return CONVATTN_ERR_TOO_LARGE;
    return 0;
}
struct HeadmixWs {
    size_t stat_bytes, part_off, total;
};
static HeadmixWs headmix_ws(const convattn_headmix_desc *d) {
    HeadmixWs w;
    w.stat_bytes = align256((size_t)d->B * d->H * d->N * sizeof(float));
    w.part_off = 2 * w.stat_bytes;
    w.total = w.part_off + align256((size_t)d->B * headmix_row_tiles(d->N) * d->H * d->H * sizeof(float));
    return w;
}
// D = rowsum(dO o O) and LSE = M + log L of every row into the workspace
static int headmix_prepare(const convattn_headmix_desc *d, const void *o, const void *d_o, const float *l, const float *m,
                           void *workspace, hipStream_t s) {
    Problem p{};
    p.B = d->B; p.H = d->H; p.Nq = p.Nk = d->N; p.d = d->d;
    float *Dl = static_cast<float *>(workspace);
    float *lse = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + headmix_ws(d).stat_bytes);
    return (int)bwd_preprocess(p, d->in_dtype, d->out_dtype, o, d_o, m, l, Dl, lse, s);
}

int convattn_headmix_validate(const convattn_headmix_desc *desc) { return headmix_check(desc); }

int convattn_headmix_fwd(const convattn_headmix_desc *desc, const void *q, const void *k, const void *v,
                         const float *w, void *o, float *l, float *m, void *stream) {
    int rc = headmix_check(desc);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(w); REQUIRE_PTR(o); REQUIRE_PTR(l); REQUIRE_PTR(m);
    return (int)headmix_fwd(desc->B, desc->H, desc->N, desc->d, desc->scale, desc->causal, desc->out_dtype, q, k, v, w, o,
                            l, m, static_cast<hipStream_t>(stream));
}

size_t convattn_headmix_bwd_workspace_bytes(const convattn_headmix_desc *desc) {
    return headmix_check(desc) ? 0 : headmix_ws(desc).total;
}

int convattn_headmix_bwd_dq_dw(const convattn_headmix_desc *desc, const void *q, const void *k, const void *v,
                               const float *w, const void *o, const void *d_o, const float *l, const float *m,
                               void *workspace, float *dq, float *dw, void *stream) {
    int rc = headmix_check(desc);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(w); REQUIRE_PTR(o); REQUIRE_PTR(d_o);
    REQUIRE_PTR(l); REQUIRE_PTR(m); REQUIRE_PTR(workspace); REQUIRE_PTR(dq); REQUIRE_PTR(dw);
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = headmix_prepare(desc, o, d_o, l, m, workspace, s);
    if (rc) return rc;
    const HeadmixWs ws = headmix_ws(desc);
    unsigned char *base = static_cast<unsigned char *>(workspace);
    return (int)headmix_bwd_dq_dw(desc->B, desc->H, desc->N, desc->d, desc->scale, desc->causal, q, k, v, w, d_o,
                                  reinterpret_cast<const float *>(base + ws.stat_bytes), reinterpret_cast<const float *>(base),
                                  dq, reinterpret_cast<float *>(base + ws.part_off), dw, s);
}

int convattn_headmix_bwd_dkdv(const convattn_headmix_desc *desc, const void *q, const void *k, const void *v,
                              const float *w, const void *o, const void *d_o, const float *l, const float *m,
                              void *workspace, float *dk, float *dv, void *stream) {
    int rc = headmix_check(desc);
    if (rc) return rc;
    REQUIRE_PTR(q); REQUIRE_PTR(k); REQUIRE_PTR(v); REQUIRE_PTR(w); REQUIRE_PTR(o); REQUIRE_PTR(d_o);
    REQUIRE_PTR(l); REQUIRE_PTR(m); REQUIRE_PTR(workspace); REQUIRE_PTR(dk); REQUIRE_PTR(dv);
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = headmix_prepare(desc, o, d_o, l, m, workspace, s);
    if (rc) return rc;
    const HeadmixWs ws = headmix_ws(desc);
    unsigned char *base = static_cast<unsigned char *>(workspace);
    return (int)headmix_bwd_dkdv(desc->B, desc->H, desc->N, desc->d, desc->scale, desc->causal, q, k, v, w, d_o,
                                 reinterpret_cast<const float *>(base + ws.stat_bytes), reinterpret_cast<const float *>(base),
                                 dk, dv, s);
}

}  // extern "C"
