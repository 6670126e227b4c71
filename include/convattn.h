/*
 * convattn.h - C ABI of the MI355X (gfx950) fused conv-attention library.
 *
 * Conv-attention: scores S = scale * Q K^T pass through a per-head causal 2-D
 * cross-correlation over a (c_q x c_k) query/key window before the softmax:
 *
 *   S_m[i,j] = S[i,j]                       (0 where causal and j > i)
 *   C[i,j]   = sum_{a<c_q} sum_{b<c_k} W[h,a,b] * S_m[i+a-(c_q-1), j+b-(c_k-1)/2]
 *   C[i,j]   = -inf where causal and j > i
 *   M = rowmax C, L = rowsum exp(C-M), O = softmax(C) V
 *
 * Conventions
 *   - Every tensor pointer is a DEVICE address of a dense row-major array:
 *     Q [B,H,Nq,d], K,V [B,H,Nk,d], W [H,c_q,c_k] (always fp32), statistics
 *     M, L, D, LSE [B,H,Nq] (always fp32).  Pointers must be 16-byte aligned.
 *   - The library never allocates or frees device memory: the caller owns
 *     inputs, outputs and the work buffers whose sizes the *_bytes() queries
 *     return.  One exception, convattn_decode_noalloc, keeps its scratch in a
 *     built-in device array of fixed size (see its declaration).
 *   - Every launch is asynchronous on the hipStream_t passed as `stream`
 *     (NULL = the null stream); no entry point synchronises the device.
 *   - Return value: 0 = ok, < 0 = convattn_status (argument rejected before any
 *     HIP call), > 0 = hipError_t of a failed launch.
 *   - The functions are re-entrant and keep no state between calls, except
 *     convattn_decode_noalloc: calls that overlap on one GPU share its scratch.
 *
 * Each entry point names the interface of Gusanidas/flash-multi-token-attention
 * that it replaces (paths relative to flash_multi_token_attention/).
 */
#ifndef CONVATTN_H
#define CONVATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CONVATTN_VERSION 300 /* major*10000 + minor*100 + patch */

typedef enum convattn_dtype {
    CONVATTN_BF16 = 0,
    CONVATTN_F32 = 1
} convattn_dtype;

typedef enum convattn_op {
    CONVATTN_OP_FWD = 0,
    CONVATTN_OP_BWD = 1,
    CONVATTN_OP_DECODE = 2
} convattn_op;

typedef enum convattn_status {
    CONVATTN_OK = 0,
    CONVATTN_ERR_NULL = -1,        /* a required pointer is NULL */
    CONVATTN_ERR_SHAPE = -2,       /* B, H, Nq, Nk or d not positive / mismatched */
    CONVATTN_ERR_HEAD_DIM = -3,    /* d not a multiple of 8 or > 128 */
    CONVATTN_ERR_KERNEL_SIZE = -4, /* c_q not in 1..16, c_k even or not in 1..33 */
    CONVATTN_ERR_DTYPE = -5,       /* unknown dtype code */
    CONVATTN_ERR_ALIGN = -6,       /* pointer not 16-byte aligned */
    CONVATTN_ERR_SPLITS = -7,      /* decode: n_splits not in 1..Nk (or > 1024) */
    CONVATTN_ERR_QROWS = -8,       /* decode: resident query rows not in 1..16 */
    CONVATTN_ERR_SCALE = -9,       /* scale is not finite */
    CONVATTN_ERR_CAUSAL_SHAPE = -10, /* causal training pass needs Nq == Nk */
    CONVATTN_ERR_LDS = -11,        /* the window needs more LDS than a CU has */
    CONVATTN_ERR_TOO_LARGE = -12,  /* a launch dimension would overflow */
    CONVATTN_ERR_SCRATCH = -13,    /* convattn_decode_noalloc: partials larger than the built-in scratch */
    CONVATTN_ERR_HEADMIX = -15,    /* convattn_headmix_*: H not 16 or 32, d not 32 / 64 / 128, or inputs not bf16 */
    CONVATTN_ERR_KV_LAYOUT = -14   /* convattn_decode_kv: bad KV-head count, page size, stride or table, or a
                                      descriptor outside the streaming decode kernel (bf16, d 64 / 128, c_k <= 17) */
} convattn_status;

/* Flags for convattn_desc.flags */
#define CONVATTN_FLAG_EXACT 1u /* force the fp32-arithmetic kernels (no MFMA, no
                                  fp16 score tile); what "fp32 mode" runs */
#define CONVATTN_FLAG_LOW_MEMORY 2u /* convattn_bwd_dq_dw: keep the partial buffer O(N) (the
                                  query-stationary kernel) instead of the faster pass whose
                                  buffer holds the bf16 dS matrix, O(N^2) */

/*
 * Problem descriptor (plain data, passed by pointer, read during the call only).
 * Training passes: Nq == Nk when causal.  Decode: Nq = number of resident query
 * rows (the last Nq positions, 1..16), Nk = KV-cache length; one output row.
 */
typedef struct convattn_desc {
    int32_t B, H, Nq, Nk, d;
    int32_t c_q, c_k;   /* window: c_q query taps (pad_q = c_q-1 rows back),
                           c_k key taps (pad_k = (c_k-1)/2 either side, c_k odd) */
    float scale;        /* softmax scale, usually 1/sqrt(d) */
    int32_t causal;     /* 0 / 1 */
    int32_t in_dtype;   /* Q, K, V, dO */
    int32_t out_dtype;  /* O, dQ, dK, dV */
    int32_t n_splits;   /* decode only: partitions of the key range (>= 1) */
    uint32_t flags;
} convattn_desc;

/* Library version (CONVATTN_VERSION it was built from). */
int convattn_version(void);

/* Text for a return code of this library (negative) or of HIP (positive). */
const char *convattn_strerror(int code);

/*
 * Host-only argument check for one operation; touches no GPU state.  Mirrors the
 * TORCH_CHECKs of conv_attn/kernels/fwd_wrapper.cu:25-33,72,94,
 * dq_bwd_wrapper.cu:25-43 and fwd_inference_wrapper.cu:25-66.
 */
int convattn_validate(const convattn_desc *desc, int op);

/*
 * Which kernel family a call with this descriptor runs: 0 = fp32-arithmetic
 * kernels, 1 = bf16 MFMA kernels.  Negative = convattn_status.
 */
int convattn_kernel_path(const convattn_desc *desc, int op);

/*
 * Training forward.  Replaces flash_conv_attention_forward
 * (conv_attn/kernels/fwd_wrapper.cu:15-100, bound as `forward` in
 * conv_attn/bindings.cpp:46-48) and fwd_kernel (conv_attn/kernels/fwd.cu:21-310).
 * Writes O [B,H,Nq,d] (out_dtype), M, L [B,H,Nq] fp32.
 */
int convattn_fwd(const convattn_desc *desc, const void *q, const void *k, const void *v,
                 const float *w, void *o, float *m, float *l, void *stream);

/*
 * Backward preparation: D = rowsum(dO * O), LSE = M + log L, both fp32.  Replaces
 * the unfused torch ops of FlashConvAttentionCUDAFunction.backward
 * (conv_attn/conv_attention_cuda.py:130,144).  `o` is out_dtype, `d_o` in_dtype.
 */
int convattn_bwd_preprocess(const convattn_desc *desc, const void *o, const void *d_o,
                            const float *m, const float *l, float *D, float *lse,
                            void *stream);

/*
 * Bytes of the work buffer convattn_bwd_dq_dw needs (0 on a bad descriptor).  On the
 * bf16 matrix-core path this is the whole workspace of the
 * key-stationary kernel: the bf16 dS matrix, B*H*Nq*Nk*2 bytes (causal: its lower triangle, 1.1 GB at B4 H16 N4096),
 * plus the dW partials and the dC scales.  With CONVATTN_FLAG_LOW_MEMORY in desc->flags
 * (and on every other path) it is the dW partials only, O(B*H*Nq/128) floats.
 */
size_t convattn_dw_partial_bytes(const convattn_desc *desc);

/*
 * dQ and the per-tile partial sums of dW.  Replaces flash_conv_attention_dq_backward
 * (conv_attn/kernels/dq_bwd_wrapper.cu:11-93, bound as `dq_backward` in
 * conv_attn/bindings.cpp:50-52) and dq_kernel (conv_attn/kernels/dq_bwd.cu:20-587).
 * The reference adds dW with float atomics (dq_bwd.cu:498-501); here every tile
 * stores its own partial and convattn_dw_reduce sums them in a fixed order.
 */
int convattn_bwd_dq_dw(const convattn_desc *desc, const void *q, const void *k, const void *v,
                       const void *d_o, const float *D, const float *lse, const float *w,
                       void *dq, float *dw_partial, void *stream);

/* dW [H,c_q,c_k] fp32 = ordered sum of the partials over batch and query tiles. */
int convattn_dw_reduce(const convattn_desc *desc, const float *dw_partial, float *dw,
                       void *stream);

/*
 * dK and dV.  Replaces flash_conv_attention_dkdv_backward
 * (conv_attn/kernels/dkdv_wrapper.cu:12-89, bound as `dkdv_backward` in
 * conv_attn/bindings.cpp:54-56) and dk_dv_kernel (conv_attn/kernels/dkdv_kernel.cu:18-527).
 */
int convattn_bwd_dkdv(const convattn_desc *desc, const void *q, const void *k, const void *v,
                      const void *d_o, const float *D, const float *lse, const float *w,
                      void *dk, void *dv, void *stream);

/*
 * The whole backward in one call: dQ, dK, dV and dW from one pass over the score tiles.
 * Same results as convattn_bwd_dq_dw + convattn_dw_reduce + convattn_bwd_dkdv, which recompute
 * the scores, the convolution and dC once each; this entry computes them once, keeps dS
 * (bf16) in `workspace` and forms dQ = dS K from it.  It is what the autograd function of
 * the reference (conv_attn/conv_attention_cuda.py:119-190, which calls dq_backward and then
 * dkdv_backward) amounts to when both results are wanted.  `workspace` is device memory of
 * convattn_bwd_fused_workspace_bytes(desc) bytes, 256-byte aligned; its contents need not be
 * initialised and mean nothing afterwards.  dW is written (not accumulated).
 */
size_t convattn_bwd_fused_workspace_bytes(const convattn_desc *desc);
int convattn_bwd_fused(const convattn_desc *desc, const void *q, const void *k, const void *v,
                       const void *d_o, const float *D, const float *lse, const float *w,
                       void *dq, void *dk, void *dv, float *dw, void *workspace, void *stream);

/*
 * The three steps of convattn_bwd_fused, for callers that order or time them themselves.
 * They must run in this order on one stream (or with the caller's own dependencies) and share
 * one workspace: _dkdv writes dK, dV and, into the workspace, dS and the dW partials; _dq
 * forms dQ from the workspace (the arguments other than k, dq and workspace are only read
 * for shapes the fp32-arithmetic kernels handle, where this step is the separate dQ pass);
 * _dw sums the partials into dW.  Counterparts in the reference as for convattn_bwd_dkdv
 * (conv_attn/kernels/dkdv_wrapper.cu:12-89), convattn_bwd_dq_dw
 * (conv_attn/kernels/dq_bwd_wrapper.cu:11-93) and the float-atomic accumulation of dW
 * (conv_attn/kernels/dq_bwd.cu:498-501).
 */
int convattn_bwd_fused_dkdv(const convattn_desc *desc, const void *q, const void *k, const void *v,
                            const void *d_o, const float *D, const float *lse, const float *w,
                            void *dk, void *dv, void *workspace, void *stream);
int convattn_bwd_fused_dq(const convattn_desc *desc, const void *q, const void *k, const void *v,
                          const void *d_o, const float *D, const float *lse, const float *w,
                          void *dq, void *workspace, void *stream);
int convattn_bwd_fused_dw(const convattn_desc *desc, const void *workspace, float *dw, void *stream);

/* Bytes of o_part (fp32 [B,H,n_splits,d]); m_part and l_part are fp32 [B,H,n_splits]. */
size_t convattn_decode_partial_bytes(const convattn_desc *desc);

/*
 * Decode step over a KV cache: un-normalised per-split partials of the last
 * query row.  Replaces flash_conv_attention_inference
 * (conv_attn/kernels/fwd_inference_wrapper.cu:13-120, bound as
 * `forward_inference` in conv_attn/fwd_inference_bindings.cpp:20-23) and
 * fwd_inference_kernel (conv_attn/kernels/fwd_inference.cu:19-283).
 * q is [B,H,Nq,d] with Nq resident rows (no front padding needed).
 */
int convattn_decode(const convattn_desc *desc, const void *q, const void *k, const void *v,
                    const float *w, float *o_part, float *m_part, float *l_part, void *stream);

/*
 * The same over K and V that are views of a longer cache: rows of one head are dense
 * ([Nk][d]), consecutive heads are kv_head_stride elements apart and consecutive batches
 * kv_batch_stride (both multiples of 8, kv_head_stride >= Nk*d).  A cache allocated as
 * [B,H,N_max,d] and read as cache[:, :, :Nk] has kv_head_stride = N_max*d and
 * kv_batch_stride = H*N_max*d.  The reference requires contiguous K and V
 * (CHECK_CONTIGUOUS, conv_attn/kernels/fwd_inference_wrapper.cu:8,28-30), so its callers copy
 * such a view on every step; convattn_decode is this call with the dense strides.
 */
int convattn_decode_strided(const convattn_desc *desc, const void *q, const void *k, const void *v,
                            const float *w, long long kv_batch_stride, long long kv_head_stride,
                            float *o_part, float *m_part, float *l_part, void *stream);

/*
 * Where K and V of a decode step live, beyond the dense and strided [B,H,Nk,d] forms above: shared
 * KV heads (grouped-query attention), a paged cache and per-sequence lengths.  The reference has
 * none of the three (its shim takes dense [B,H,Nk,d] tensors, conv_attn/
 * flash_conv_attention_inference.py:33-93); this is the widening of its decode entry for serving.
 *   H_kv          KV heads (0 = H).  H % H_kv == 0; query head h reads KV head h / (H / H_kv).  W stays
 *                 per query head.
 *   page_size     0: the rows of one (batch, KV head) are contiguous, batches batch_stride and KV heads
 *                 head_stride elements apart (as in convattn_decode_strided).
 *                 > 0 (a power of two >= 16): k and v are pools of pages; page p of KV head g starts at
 *                 p * page_stride + g * head_stride and holds page_size rows of d elements; keys
 *                 [i * page_size, (i+1) * page_size) of batch entry b are page block_table[b * table_stride + i]
 *                 (device memory, int32).  A pool laid out [n_pages][H_kv][page_size][d] has
 *                 page_stride = H_kv*page_size*d and head_stride = page_size*d.
 *   seq_lens      optional device int32 [B]: number of keys of every batch entry (1 .. desc->Nk); NULL =
 *                 desc->Nk for all.  desc->Nk is the longest sequence; splits cut every sequence evenly.
 * Strides are multiples of 8 elements.  Only descriptors that run the streaming decode kernel are
 * accepted (bf16 K and V, d 32, 64 or 128, c_k <= 17: convattn_kernel_path(desc, CONVATTN_OP_DECODE) == 1).
 */
typedef struct convattn_kv_layout {
    int32_t H_kv;
    int32_t page_size;
    int64_t batch_stride;
    int64_t head_stride;
    int64_t page_stride;
    const int32_t *block_table;
    int32_t table_stride;
    int32_t reserved;          /* 0 */
    const int32_t *seq_lens;
} convattn_kv_layout;

/* convattn_decode with K and V described by `kv`; partials and convattn_decode_combine as above. */
int convattn_decode_kv(const convattn_desc *desc, const void *q, const void *k, const void *v,
                       const convattn_kv_layout *kv, const float *w, float *o_part, float *m_part,
                       float *l_part, void *stream);

/*
 * Log-sum-exp merge of the split partials into O [B,H,1,d] (out_dtype), M, L
 * [B,H,1] fp32.  Replaces combine_splits_kernel (conv_attn/kernels/
 * fwd_inference.cu:286-369); unlike the reference it also runs for n_splits == 1,
 * so O is always normalised.
 */
int convattn_decode_combine(const convattn_desc *desc, const float *o_part, const float *m_part,
                            const float *l_part, void *o, float *m, float *l, void *stream);

/*
 * A whole decode step (convattn_decode_strided + convattn_decode_combine) that allocates nothing
 * and needs no partial buffers from the caller: O [B,H,1,d] (out_dtype), M, L [B,H,1] fp32 from
 * Q, K, V, W.  It has no counterpart in the reference; it is for callers that cannot allocate
 * device memory around the call (code under HIP graph capture, serving loops with a fixed memory
 * plan, harnesses that forbid hipMalloc).  The split partials live in a buffer built into the
 * library, CONVATTN_DECODE_NOALLOC_MAX_BYTES per GPU for the life of the process:
 * convattn_decode_noalloc_bytes(desc) is what a descriptor needs (B*H*n_splits*(d+2) floats, each
 * part rounded up to 256 bytes; 0 on a bad descriptor); a step that needs more is rejected with
 * CONVATTN_ERR_SCRATCH.  Every call on one GPU uses the same buffer: calls that overlap on one
 * GPU (two streams, two threads) race, calls on one stream do not.  kv_batch_stride and
 * kv_head_stride as in convattn_decode_strided (Nk*d*H and Nk*d for dense K and V).
 */
#define CONVATTN_DECODE_NOALLOC_MAX_BYTES (8u << 20)
size_t convattn_decode_noalloc_bytes(const convattn_desc *desc);
int convattn_decode_noalloc(const convattn_desc *desc, const void *q, const void *k, const void *v,
                            const float *w, long long kv_batch_stride, long long kv_head_stride,
                            void *o, float *m, float *l, void *stream);

/* ------------------------------------------------------------------------------------------
 * Head-mixing attention, the reference's second variant (head_conv_attn/): the scores of all
 * heads of a (batch, row, key) triple are mixed by a dense [H][H] matrix before the softmax,
 *   Z[b,h] = sum_h' w[h][h'] * scale * Q[b,h'] K[b,h']^T,  P = softmax(Z + causal mask),  O = P V
 * (head_conv_attn/head_conv_fn_pytorch.py:7-54).  q, k, v, o, d_o: dense [B,H,N,d]; w: fp32
 * [H][H] (out head, in head); l, m: fp32 [B,H,N] with m the row maximum of Z and
 * l = sum_j exp(Z - m), as the reference returns them.  H is 16 or 32 (fwd_kernel.py:289),
 * d 32, 64 or 128, inputs bf16, O bf16 or fp32, gradients fp32 (bwd_dq_dw.py:381-382).
 * ------------------------------------------------------------------------------------------ */
typedef struct convattn_headmix_desc {
    int32_t B, H, N, d;
    float scale;
    int32_t causal;
    int32_t in_dtype;   /* CONVATTN_BF16 */
    int32_t out_dtype;  /* dtype of O */
} convattn_headmix_desc;

/* Host-only check of a descriptor: 0 or a negative convattn_status. */
int convattn_headmix_validate(const convattn_headmix_desc *desc);

/*
 * Forward.  Replaces head_conv_attention_forward and head_conv_attn_fwd_kernel
 * (head_conv_attn/fwd_kernel.py:7-365): O stays in registers for the whole key loop instead of
 * being read and written back per key block (fwd_kernel.py:214-250).
 */
int convattn_headmix_fwd(const convattn_headmix_desc *desc, const void *q, const void *k, const void *v,
                         const float *w, void *o, float *l, float *m, void *stream);

/* Bytes of the scratch buffer the two backward entry points need (D and LSE of every row, the dW
 * partials of every row tile); its contents need not be initialised.  0 on a bad descriptor. */
size_t convattn_headmix_bwd_workspace_bytes(const convattn_headmix_desc *desc);

/*
 * dQ [B,H,N,d] fp32 and dW [H][H] fp32.  Replaces head_conv_attention_bwd_dq_dw
 * (head_conv_attn/bwd_dq_dw.py:7-470).  dW is summed over per-tile partials in a fixed order
 * (the reference adds it with tl.atomic_add, bwd_dq_dw.py:370).
 */
int convattn_headmix_bwd_dq_dw(const convattn_headmix_desc *desc, const void *q, const void *k, const void *v,
                               const float *w, const void *o, const void *d_o, const float *l, const float *m,
                               void *workspace, float *dq, float *dw, void *stream);

/* dK, dV [B,H,N,d] fp32.  Replaces head_conv_attention_bwd_dkdv (head_conv_attn/bwd_dk_dv.py:7-500). */
int convattn_headmix_bwd_dkdv(const convattn_headmix_desc *desc, const void *q, const void *k, const void *v,
                              const float *w, const void *o, const void *d_o, const float *l, const float *m,
                              void *workspace, float *dk, float *dv, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CONVATTN_H */
