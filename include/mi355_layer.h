/*
 * mi355_layer.h -- C ABI of libmi355_layer.so: hand-written gfx950 (MI355X) kernels for the
 * transformer-layer hot path (attention core forward/backward/decode, rotary, RMSNorm, SwiGLU).
 *
 * The reference (Aleph-Alpha/scaling) is pure Python; it has no FFI for this path.  Each entry
 * point below names the reference call site (path under src/scaling/) whose arithmetic it
 * replaces.  A Python host binds these with ctypes; nothing here depends on libtorch.
 *
 * Conventions
 *   - every function returns MI_OK (0) or a negative mi_status; it never throws, aborts or
 *     synchronises the device.  mi_last_error() returns a thread-local description of the last
 *     failure on the calling thread.
 *   - all kernels are launched asynchronously on `stream` (a hipStream_t passed as void*;
 *     NULL = the default stream).
 *   - the library allocates no device memory and keeps no mutable global state: scratch space is
 *     passed in by the caller (see the *_workspace_bytes helpers), so calls are re-entrant.
 *   - tensors: innermost dimension contiguous, base pointers 16-byte aligned, every stride
 *     (given in ELEMENTS) a multiple of 8 elements for 16-bit types (4 for fp32).
 *   - "token" axes are the flattened (batch seq) axis of the reference's [b, s, ...] tensors;
 *     cumulative sequence lengths are int32 offsets on that axis exactly as produced by
 *     transformer/data/utils.py:40-74.
 */
#ifndef MI355_LAYER_H
#define MI355_LAYER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_LAYER_VERSION 100

typedef enum mi_status {
    MI_OK = 0,
    MI_E_NULL = -1,        /* a required pointer is NULL */
    MI_E_DTYPE = -2,       /* dtype code not supported by this entry point */
    MI_E_SHAPE = -3,       /* size / head_dim / head-count combination not supported */
    MI_E_ALIGN = -4,       /* pointer or stride violates the alignment contract */
    MI_E_WORKSPACE = -5,   /* workspace missing or too small */
    MI_E_LAUNCH = -6,      /* the HIP runtime refused the launch (mi_last_error has details) */
    MI_E_ARCH = -7         /* current device is not gfx950 */
} mi_status;

typedef enum mi_dtype { MI_BF16 = 0, MI_F16 = 1, MI_F32 = 2 } mi_dtype;

int mi_version(void);
const char* mi_last_error(void);
const char* mi_status_string(int status);
/* MI_OK when the current HIP device is a gfx950 part, MI_E_ARCH otherwise. */
int mi_check_device(void);

/* ------------------------------------------------------------------------------------------
 * RMSNorm.  Replaces core/nn/norm/rms_norm.py:47-50:  y = x * rsqrt(mean(x^2, -1) + eps) * weight.
 * Arithmetic in fp32, one rounding to `dtype` on store.  x, y: [n_rows, hidden]; weight: [hidden].
 * rstd (optional, may be NULL): fp32 [n_rows], receives rsqrt(mean(x^2)+eps).
 * Algorithmic HBM bytes: fwd 2*n_rows*hidden*e, bwd 3*n_rows*hidden*e (e = element size).
 * ------------------------------------------------------------------------------------------ */
int mi_rmsnorm_fwd(const void* x, const void* weight, void* y, float* rstd,
                   int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream);

/* Residual add fused into the norm that follows it (transformer/model/layers/layer.py:252-293 with
 * core/nn/residual.py:49-65 at inference): sum_out = x + residual rounded to `dtype`, y = rmsnorm(sum_out) * weight
 * exactly as mi_rmsnorm_fwd computes it from the stored sum.  sum_out may alias x or residual; y may not alias.
 * Forward only.  Algorithmic HBM bytes: 4 * n_rows * hidden * e. */
int mi_add_rmsnorm_fwd(const void* x, const void* residual, const void* weight, void* sum_out, void* y,
                       int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream);

/* Backward of the above (what autograd derives from rms_norm.py:47-50):
 *   dx = rstd * (dy*w) - x * rstd^3 * mean(dy*w*x),   dweight = sum_rows dy * x * rstd.
 * rstd is recomputed from x.  `workspace` holds per-block fp32 partial sums of dweight and must be
 * at least mi_rmsnorm_bwd_workspace_bytes(n_rows, hidden) bytes; the partials are reduced in a
 * fixed order (bit-reproducible).  dweight is written in `dtype`. */
size_t mi_rmsnorm_bwd_workspace_bytes(int64_t n_rows, int64_t hidden);
int mi_rmsnorm_bwd(const void* x, const void* weight, const void* dy, void* dx, void* dweight,
                   void* workspace, size_t workspace_bytes,
                   int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * LayerNorm.  Replaces core/nn/norm/layernorm.py:75-86 (torch.nn.functional.layer_norm over the last
 * dimension):  y = (x - mean) * rsqrt(var + eps) * weight + bias, biased variance, fp32 arithmetic, one
 * rounding to `dtype` on store.  bias may be NULL.  `mean` / `rstd` (fp32 [n_rows], both or neither; may be
 * NULL) receive the row statistics, the two tensors torch.native_layer_norm saves for its backward.
 *   dx = rstd * (dy*w - mean(dy*w) - xhat * mean(dy*w*xhat)),  dweight = sum_rows dy*xhat,  dbias = sum_rows dy
 * (dbias may be NULL).  The backward takes the saved `mean` / `rstd` (then a row needs one reduction instead
 * of two) or, when both are NULL, recomputes them from x.  `workspace`: fp32, at least
 * mi_layernorm_bwd_workspace_bytes(n_rows, hidden) bytes; partial sums are reduced in a fixed order.
 * Algorithmic HBM bytes as for RMSNorm.
 * ------------------------------------------------------------------------------------------ */
int mi_layernorm_fwd(const void* x, const void* weight, const void* bias, void* y, float* mean, float* rstd,
                     int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream);
size_t mi_layernorm_bwd_workspace_bytes(int64_t n_rows, int64_t hidden);
int mi_layernorm_bwd(const void* x, const void* weight, const void* dy, const float* mean, const float* rstd,
                     void* dx, void* dweight, void* dbias, void* workspace, size_t workspace_bytes,
                     int64_t n_rows, int64_t hidden, float eps, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * GELU activation of the default MLP.  Replaces core/nn/mlp.py:135-139 with
 * core/nn/activation_function.py:13-14 (torch.nn.functional.gelu, exact erf form):
 *   y = 0.5 * x * (1 + erf(x / sqrt 2)),   dx = dy * (0.5 * (1 + erf(x / sqrt 2)) + x * exp(-x^2/2) / sqrt(2 pi)).
 * Algorithmic HBM bytes: fwd 2*n_elem*e, bwd 3*n_elem*e.
 * ------------------------------------------------------------------------------------------ */
int mi_gelu_fwd(const void* x, void* y, int64_t n_elem, int dtype, void* stream);
int mi_gelu_bwd(const void* x, const void* dy, void* dx, int64_t n_elem, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Token-level cross entropy over vocabulary rows.  Replaces transformer/model/losses/cross_entropy.py:18-32
 * (torch.nn.functional.cross_entropy(logits.float(), target, reduction="none")) and the argmax of :84, and
 * produces what autograd derives from them.  Per row r with target t (fp32 arithmetic on `dtype` logits):
 *   lse = log sum_i exp(x_i),  losses[r] = lse - x_t,  argmax[r] = first index of max_i x_i,
 *   dlogits[r][i] = row_scale[r] * (exp(x_i - lse) - [i == t])        (only when dlogits != NULL)
 * row_scale (fp32, NULL = 1) carries loss_weight[r] / sum(loss_weights) times the upstream gradient
 * (cross_entropy.py:30).  A target outside [0, vocab) marks an ignored row (loss 0, zero gradient; -100 is
 * torch's ignore_index).  losses / lse / argmax / dlogits may each be NULL; dlogits may alias logits
 * (in-place gradient for a chunked LM head).  Row strides are in elements; rows need not be 16-byte aligned nor a
 * whole number of 16-byte vectors.  With a gradient, rows of more than 16384 vectors (131072 bf16 logits) and rows
 * that are not aligned whole vectors are served by two launches that hand the log-sum-exp over in `lse`: pass it
 * (with at most 65535 rows, logits and dlogits rows at the same offset from a 16-byte boundary), or such rows fall
 * back to a slow scalar kernel.
 * Algorithmic HBM bytes: n_rows*vocab*e read, plus the same written when dlogits is given (and read once more
 * by the two-launch path).
 * ------------------------------------------------------------------------------------------ */
int mi_cross_entropy(const void* logits, const int64_t* targets, const float* row_scale, float* losses, float* lse,
                     int32_t* argmax, void* dlogits, int64_t n_rows, int64_t vocab, int64_t logits_row_stride,
                     int64_t dlogits_row_stride, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * SwiGLU activation.  Replaces core/nn/mlp.py:248-249:  out = silu(a) * gate, elementwise over
 * n_elem contiguous elements.  Backward: da = dout*gate*sig(a)*(1 + a*(1 - sig(a))), dgate = dout*silu(a).
 * Algorithmic HBM bytes: fwd 3*n_elem*e, bwd 5*n_elem*e.
 * ------------------------------------------------------------------------------------------ */
int mi_swiglu_fwd(const void* a, const void* gate, void* out, int64_t n_elem, int dtype, void* stream);
int mi_swiglu_bwd(const void* a, const void* gate, const void* dout, void* da, void* dgate,
                  int64_t n_elem, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Rotary embedding (rotate-half pairing i <-> i + rot_dim/2), stand-alone kernel.
 * Replaces core/nn/rotary.py:117-139 / :176-213 (cos/sin row gather by position id, then
 * x*cos + rotate_half(x)*sin on the first rot_dim features, the rest copied).
 * x, out: [n_tokens, n_heads, head_dim] with element strides (token, head); out may alias x.
 * cos, sin: [table_rows, rot_dim] contiguous, in `table_dtype` (the reference keeps them in the
 * module dtype).  position_ids: int64 [n_tokens] or NULL (then token t of every sequence uses
 * row t % seq_len_for_null_ids).  inverse != 0 rotates by the negative angle (= the backward).
 * Algorithmic HBM bytes: 2*n_tokens*n_heads*head_dim*e + table rows touched + 8*n_tokens.
 * ------------------------------------------------------------------------------------------ */
int mi_rotary(const void* x, void* out, const void* cos, const void* sin, const int64_t* position_ids,
              int64_t n_tokens, int32_t n_heads, int32_t head_dim, int32_t rot_dim,
              int64_t x_stride_token, int64_t x_stride_head, int64_t out_stride_token, int64_t out_stride_head,
              int64_t table_rows, int64_t seq_len_for_null_ids, int inverse,
              int dtype, int table_dtype, void* stream);

/* Interleaved ("complex") rotary, pairs (2i, 2i+1) over the whole head, fp32 arithmetic.
 * Replaces core/nn/rotary.py:45-90 / :216-255 (RotaryEmbeddingComplex): cos / sin are the real / imaginary
 * parts of freqs_cis, fp32 [table_rows, head_dim/2].  Other arguments as mi_rotary. */
int mi_rotary_complex(const void* x, void* out, const float* cos, const float* sin, const int64_t* position_ids,
                      int64_t n_tokens, int32_t n_heads, int32_t head_dim,
                      int64_t x_stride_token, int64_t x_stride_head, int64_t out_stride_token, int64_t out_stride_head,
                      int64_t table_rows, int64_t seq_len_for_null_ids, int inverse, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Attention core.  Replaces core/nn/attention/attention.py:108-213 (multi_head_attention) with
 * core/nn/masked_softmax/masked_softmax.py:14-34 as softmax and :76-105 as mask, plus repeat_kv
 * (:60-69) and, when cos/sin are given, the rotary call at :836-845.  Interface precedent for a
 * fused kernel inside the reference: flash_attention(), attention.py:216-271.
 *
 * Layout: q [total_q, n_q_heads, head_dim], k/v [total_k, n_kv_heads, head_dim], o like q, element
 * strides (token, head) per tensor.  Query head h reads kv head h / (n_q_heads / n_kv_heads).
 * Mask predicate (never materialised): query token t of document j (cu_seqlens_q[j] <= t <
 * cu_seqlens_q[j+1]) may attend key token u iff cu_seqlens_k[j] <= u < cu_seqlens_k[j+1] and, when
 * causal, (u - cu_seqlens_k[j]) <= (t - cu_seqlens_q[j]) + (len_k - len_q).  For len_k == len_q this
 * is exactly the reference's block-diagonal lower-triangular mask; for len_q == 1 it is the
 * unmasked cached-decode case.  Softmax is evaluated in fp32 with scores scaled by softmax_scale
 * (= query_key_scaling_factor * masked_softmax.scale); probabilities are rounded to bf16 before
 * P*V as in the reference (attention.py:211).  A row without any allowed key yields zeros.
 * lse: fp32 [n_q_heads, total_q], natural-log sum-exp of the scaled scores (needed by backward).
 *
 * Fused rotary (optional): if rotary_cos != NULL, q and k are rotated on load (rotate-half, the
 * whole head_dim; tables [rotary_table_rows, head_dim] in the I/O dtype; position ids int64 per
 * token).  position_ids_k == NULL means that k is rotated already and only q is rotated here: the cheaper
 * arrangement whenever k can be rotated once beforehand (mi_rotary), because a K tile is loaded by every query
 * block of every query head of its group and a Q row only once; it is also the only one that combines with
 * dropout.  q_rot_out receives the rotated q for the backward.  With rotary_interleaved != 0 the rotation is the interleaved-pair ("complex")
 * one of core/nn/rotary.py:59-90 instead: pairs (2i, 2i+1), fp32 tables [rotary_table_rows,
 * head_dim / 2] (real and imaginary part of freqs_cis), fp32 arithmetic, one rounding -- the same
 * bits as mi_rotary_complex followed by the plain call.  Fused rotary needs head_dim in {64, 128}.
 * Supported: dtype MI_BF16 or MI_F16 (the same kernels built on the bf16 / f16 MFMA), head_dim in {32, 64, 96, 128};
 * dtype MI_F32 (the reference's default `precision`, transformer/context/config.py:346): separate kernels on the
 * fp32 MFMA with fp32 probabilities throughout (probs.to(value.dtype) is the identity there), same masks, layouts,
 * lse and workspace contract, strides multiples of 4 elements, no dropout, no fused rotary, flags ignored.
 * Algorithmic work: 4 * head_dim * n_q_heads * P flop forward, 10 * head_dim * n_q_heads * P backward,
 * P = number of allowed (query, key) pairs per head.
 * ------------------------------------------------------------------------------------------ */
#define MI_ATTN_QG1 1   /* forward: one group of 32 queries per wavefront (128 per workgroup) */
#define MI_ATTN_QG2 2   /* forward: two groups of 32 queries per wavefront (256 per workgroup) */
/* Accuracy mode, forward and backward: every bf16 operand that the kernels form themselves (the probabilities P in
 * P V and dV = P^T dO, dS in dQ = dS K and dK = dS^T Q) enters its MFMA as two bf16 terms hi + lo, so these products
 * carry 16 mantissa bits instead of 8 (the reference rounds P once to the value dtype, attention.py:211).  Costs a
 * second pass over those MFMAs (forward 1.5 x, backward 1.4 x the MFMA work).  No dropout; fused rotary on q only.
 * Accuracy: without rotary, outputs and gradients are within max-abs 2e-2 / mean-relative 1e-3 of the reference
 * evaluated in fp32.  With the fused rotary they are not: the rotated q and k are rounded once to the I/O dtype
 * before the score product (as the reference rounds them, rotary.py:117-139, but at other values than the
 * reference's fp32 evaluation attends with), which leaves mean-relative errors of about 2e-3 in either mode. */
#define MI_ATTN_SPLIT_P 4
/* backward: run only the named kernels (for per-kernel timing; all three when none of the bits is set) */
#define MI_ATTN_BWD_DELTA 16
#define MI_ATTN_BWD_DKDV 32
#define MI_ATTN_BWD_DQ 64

typedef struct mi_attn_args {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    float* lse;
    const int32_t* cu_seqlens_q;   /* device, [n_docs + 1] */
    const int32_t* cu_seqlens_k;   /* device, [n_docs + 1]; NULL = same as cu_seqlens_q */
    int32_t n_docs;
    int32_t causal;
    int64_t total_q;
    int64_t total_k;
    int32_t n_q_heads;
    int32_t n_kv_heads;
    int32_t head_dim;
    int32_t dtype;
    int64_t q_stride_token, q_stride_head;
    int64_t k_stride_token, k_stride_head;
    int64_t v_stride_token, v_stride_head;
    int64_t o_stride_token, o_stride_head;
    float softmax_scale;
    int32_t flags;                 /* 0 = library chooses; MI_ATTN_* bits above */
    /* optional fused rotary */
    const void* rotary_cos;
    const void* rotary_sin;
    const int64_t* position_ids_q;
    const int64_t* position_ids_k;
    int64_t rotary_table_rows;
    void* stream;
    /* dropout on the attention probabilities (attention.py:204-207): 0 = off.  Element (head, query, key) is
     * dropped iff byte(lowbias32(head_base + (query >> 1) * 0x9E3779B1 + (key >> 1) * 0x85EBCA77)
     *                  >> (16 * (query & 1) + 8 * (key & 1))) < T,  T = round(256 * dropout_p) clamped to 1..255,
     * head_base = lowbias32(seed32 ^ lowbias32(head * 0x9E3779B9 + 0x7F4A7C15)), seed32 = low ^ high word of
     * dropout_seed; query / key are token indices on the flattened axes.  The effective drop probability is
     * T / 256 and kept probabilities are scaled by 256 / (256 - T).  The backward call must pass the same values. */
    float dropout_p;
    uint64_t dropout_seed;
    int32_t rotary_interleaved;    /* fused rotary: 0 = rotate-half, 1 = interleaved pairs with fp32 tables */
    void* q_rot_out;               /* forward with fused rotary: optional copy of the rotated q (strides of q), what
                                      mi_attn_bwd takes as q; NULL = not stored */
} mi_attn_args;

/* total_q == 0 and total_k == 0 (an empty batch) is not an error: nothing is launched, MI_OK (mi_attn_bwd likewise). */
int mi_attn_fwd(const mi_attn_args* args);

/* Backward of mi_attn_fwd.  Extra inputs: o and lse from the forward, d_o (layout/strides of o).
 * Outputs dq (strides of q), dk, dv (strides given).  With rotary (fwd.rotary_cos != NULL; both position id arrays
 * required): fwd.q and fwd.k are the ROTATED tensors the forward attended with (its q_rot_out, and the rotated k), and
 * dq / dk are the gradients of the unrotated ones: each row is rotated back (by minus its position's angles, what
 * autograd derives from core/nn/rotary.py:117-139 / :59-90) in fp32 before its single rounding.  GQA: dk/dv are summed over the query heads of
 * each group inside the kernel, in a fixed order (no atomics; bit-reproducible).
 * workspace: fp32 scratch of mi_attn_bwd_workspace_bytes() bytes (row sums of d_o * o). */
typedef struct mi_attn_bwd_args {
    mi_attn_args fwd;              /* q,k,v,o,lse,cu_seqlens,... as in the forward call */
    const void* d_o;
    void* dq;
    void* dk;
    void* dv;
    int64_t dk_stride_token, dk_stride_head;
    int64_t dv_stride_token, dv_stride_head;
    void* workspace;
    size_t workspace_bytes;
} mi_attn_bwd_args;

size_t mi_attn_bwd_workspace_bytes(int64_t total_q, int32_t n_q_heads, int32_t head_dim);
/* Workspace that also holds the fp32 partial dK / dV of a launch with fewer than 8 KV heads (multi-query attention,
 * GQA with 2 or 4 KV heads): with at least this much, the dK/dV kernel splits the query heads of a group over
 * workgroups (8 x more of them for one KV head) and a second launch sums the partials in a fixed order; with
 * only mi_attn_bwd_workspace_bytes() it loops over the whole group in one workgroup per key block, which leaves
 * most compute units idle (6.3 ms against 1.1 ms for 32 query heads on one KV head at 8192 tokens).  Equal to
 * mi_attn_bwd_workspace_bytes() for 8 or more KV heads. */
size_t mi_attn_bwd_workspace_bytes_kv(int64_t total_q, int64_t total_k, int32_t n_q_heads, int32_t n_kv_heads,
                                      int32_t head_dim);
int mi_attn_bwd(const mi_attn_bwd_args* args);

/* ------------------------------------------------------------------------------------------
 * Decode attention over a pre-allocated KV cache (one new query token per sequence).
 * Replaces the cache branch attention.py:852-873 followed by multi_head_attention with a
 * [1,1,1,1] all-false mask: softmax over every cached key.  The reference grows the cache by
 * torch.cat per step and supports batch 1 only; here the cache is [batch, max_ctx, n_kv_heads,
 * head_dim] (element strides batch/token/head), holds post-rotary K, and ctx_len[b] (int32, device)
 * gives the number of valid keys of sequence b INCLUDING the token appended in this call.
 *
 * If k_new/v_new != NULL the kernel first appends them at position ctx_len[b]-1 (in-place append
 * instead of torch.cat); with rotary_cos != NULL it rotates q and k_new by position_ids[b] before
 * use/append (fused rotary; rotary_interleaved selects the pairing and table format as in mi_attn_args).
 * o: [batch, n_q_heads, head_dim] contiguous; q likewise unless q_stride_batch is set.
 * A workgroup serves up to 16 query heads of one KV head, so every K / V element is read once per 16 heads of its
 * group (once in all for groups of up to 16; multi-query attention with 32 heads reads the cache twice).
 * The key axis is split into n_splits chunks processed by different workgroups and merged by a
 * second kernel; workspace = mi_attn_decode_workspace_bytes() bytes of fp32 scratch.
 * Algorithmic HBM bytes: 2 * sum_b ctx_len[b] * n_kv_heads * head_dim * e  (K and V read once).
 * ------------------------------------------------------------------------------------------ */
typedef struct mi_decode_args {
    const void* q;
    void* k_cache;
    void* v_cache;
    void* o;
    const int32_t* ctx_len;        /* device, [batch] */
    const void* k_new;             /* [batch, n_kv_heads, head_dim] or NULL */
    const void* v_new;
    const void* rotary_cos;        /* [rotary_table_rows, head_dim] ([.., head_dim / 2] fp32 when interleaved) or NULL */
    const void* rotary_sin;
    const int64_t* position_ids;   /* device, [batch]; required with rotary */
    int64_t rotary_table_rows;
    int32_t batch;
    int32_t max_ctx;
    int32_t n_q_heads;
    int32_t n_kv_heads;
    int32_t head_dim;
    int32_t dtype;
    int64_t cache_stride_batch, cache_stride_token, cache_stride_head;
    float softmax_scale;
    int32_t n_splits;              /* 0 = let the library choose */
    void* workspace;
    size_t workspace_bytes;
    void* stream;
    /* element strides between the sequences of q / k_new / v_new (their [heads, head_dim] part stays contiguous);
     * 0 = packed ([batch, heads, head_dim] contiguous).  Lets q, k and v be column slices of one fused projection. */
    int64_t q_stride_batch, k_new_stride_batch, v_new_stride_batch;
    int32_t rotary_interleaved;    /* fused rotary: 0 = rotate-half, 1 = interleaved pairs with fp32 tables */
} mi_decode_args;

size_t mi_attn_decode_workspace_bytes(int32_t batch, int32_t n_q_heads, int32_t head_dim, int32_t max_ctx);
int mi_attn_decode(const mi_decode_args* args);

/* mi_attn_decode for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, kernels and results
 * as mi_attn_decode, except that `workspace` / `workspace_bytes` are ignored: the per-split partial results go to
 * a static device array inside the library (mi_attn_decode_static_scratch_bytes() bytes, 8 MiB, held by every GPU
 * the library runs on until the process ends).  The call allocates and frees nothing.  It returns MI_E_WORKSPACE
 * when batch * n_q_heads * n_splits * (head_dim + 2) * 4 bytes exceed the array (n_splits as chosen by the library
 * or given, at most 32).  All calls on one GPU share that GPU's array: calls that may overlap on one GPU (different
 * streams, different threads) race and must be serialised by the caller; nothing in the array has to be cleared
 * between calls (every slot a call reads was written by the same call). */
size_t mi_attn_decode_static_scratch_bytes(void);
int mi_attn_decode_static(const mi_decode_args* args);

#ifdef __cplusplus
}
#endif
#endif /* MI355_LAYER_H */
