/*
 * sa2 — sliding-window 2-simplicial attention for AMD MI355X (gfx950), C ABI.
 *
 * This header is the drop-in boundary of the library.  Each entry point replaces
 * one device launch (or launch group) that the reference issues from
 * simplicial_attention/triton_two_simplicial_attention.py; the file:line of the
 * replaced call is given with every function.  No C++ or framework types cross
 * this boundary: plain pointers, sizes, strides and an opaque hipStream_t.
 *
 * Conventions
 *   - Every activation is (batch, seq, heads, dim_head) with an innermost stride
 *     of one element; the three outer strides are passed in elements.  This is
 *     the layout "[b, s, k, h]" of the reference kernels
 *     (triton_two_simplicial_attention.py:60-66).
 *   - lse and delta are contiguous fp32 (batch, heads, seq), the layout of the
 *     reference's M and D buffers (triton_two_simplicial_attention.py:66,740,825).
 *   - Keys/values carry kv_heads heads; query head h reads kv head h / (heads /
 *     kv_heads), the "(h g)" order of triton_two_simplicial_attention.py:1033-1034.
 *     Gradients of keys/values are written with kv_heads heads (already summed
 *     over the group).
 *   - Attended set of query i:  i-w1 < j <= i  and  i-w2 < k <= i
 *     (triton_two_simplicial_attention.py:191-193).  Only causal = 1 is defined.
 *   - seq_len is arbitrary: rows past the end are masked in-kernel, so the caller
 *     does not need the zero padding of triton_two_simplicial_attention.py:1042-1046.
 *   - All calls are asynchronous on the given stream, allocate nothing and may be
 *     issued from any host thread.  Buffers are owned by the caller, and the library
 *     keeps no device state - except sa2_bwd_noalloc, whose scratch is a fixed
 *     device array inside the library (see there).  The device is the caller's
 *     current HIP device.
 *   - Return value: SA2_OK or an sa2_status; sa2_last_error() gives a
 *     thread-local message for the last failure on the calling thread.
 */
#ifndef SA2_H
#define SA2_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 101: saved->t is kept in blocks of 32 rows (sa2_saved_t_bytes), the workspace rules of sa2_bwd_workspace_bytes*
 * cover the split key slabs, sa2_bwd checks every size before its first launch
 * 102: dim_head 256 (its kernels keep no forward partials: the sa2_saved_*_bytes queries return 0 and a non-NULL
 * `saved` is refused) */
#define SA2_VERSION 102

typedef enum sa2_status {
    SA2_OK = 0,
    SA2_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    SA2_ERR_BAD_SHAPE = 2,      /* non-positive size, heads % kv_heads != 0, window < 1 */
    SA2_ERR_UNSUPPORTED = 3,    /* dim_head, dtype or causal flag the kernels do not cover */
    SA2_ERR_ALIGNMENT = 4,      /* pointer or stride breaks the 16-byte row alignment */
    SA2_ERR_LAUNCH = 5          /* hipGetLastError() after a launch was not hipSuccess */
} sa2_status;

typedef enum sa2_dtype { SA2_BF16 = 0 } sa2_dtype;

/* Problem geometry shared by every entry point. */
typedef struct sa2_problem {
    int32_t batch;
    int32_t seq_len;
    int32_t heads;      /* query heads */
    int32_t kv_heads;   /* key/value heads, divides heads */
    int32_t dim_head;   /* 32, 64, 128 or 256 */
    int32_t w1;         /* window of the first key/value set  (reference default 512) */
    int32_t w2;         /* window of the second key/value set (reference default 32), any value >= 1 */
    int32_t causal;     /* must be 1 */
    float   scale;      /* softmax scale, dim_head^-0.5 in the reference (:735) */
    int32_t dtype;      /* sa2_dtype of the activations */
} sa2_problem;

/* A (batch, seq, heads, dim_head) activation: base pointer and element strides. */
typedef struct sa2_tensor {
    void   *ptr;
    int64_t stride_b;
    int64_t stride_n;
    int64_t stride_h;
} sa2_tensor;

/* Optional by-products of the forward that the backward can reuse instead of
 * recomputing them (the reference keeps only q, k, v, out and lse for its backward,
 * triton_two_simplicial_attention.py:800-805, and recomputes everything else):
 *   t  bf16 [batch][heads][w2][ceil(seq_len/32)] blocks of [32 rows][dim_head], the 16-byte pieces of a block in the
 *      order the forward's lanes hold them (opaque to the caller):  T[b,h,d,i,:] = sum_j 2^(x_ij - m) v1[j,:]
 *      for the offset d = i - k, x = scaled logit * log2(e)
 *   m  fp32 [batch][heads][w2][seq_len]:            the reference m of that sum
 * With them dV2[k] = sum_d dO[k+d] * T[d,k+d] * 2^(m - lse*log2e) needs no contraction
 * in the backward.  Sizes: sa2_saved_t_bytes(), sa2_saved_m_bytes().  t 16-byte aligned.
 * dim_head 256 keeps no partials: both sizes are 0 and its calls take saved = NULL. */
typedef struct sa2_saved {
    void  *t;
    float *m;
} sa2_saved;

int64_t sa2_saved_t_bytes(const sa2_problem *prob);   /* -1 if the problem is invalid, 0 if its kernels keep no partials */
int64_t sa2_saved_m_bytes(const sa2_problem *prob);

/* Library version (SA2_VERSION of the build). */
int sa2_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *sa2_last_error(void);

/* 1 if the kernels cover this configuration (dim_head 32, 64, 128 or 256, any w1 >= 1 and w2 >= 1, bf16),
 * else 0.  Replaces the silent limits of the reference (HEAD_DIM fixed to 64, w2 <= 32:
 * triton_two_simplicial_attention.py:51,291,508,586). */
int sa2_supported(int32_t dim_head, int32_t w1, int32_t w2, int32_t dtype);

/* Forward.  Replaces the launch of two_simplicial_attn_fwd_kernel
 * (triton_two_simplicial_attention.py:749-798; kernel :58-228).
 * Writes out (same layout as q) and lse[b,h,n] = log sum exp of the scaled logits.
 * out_residual may be NULL; if given (same shape/dtype as out) it receives
 * bf16(out_fp32 - out), so that out + out_residual carries the fp32 accumulator to
 * about 16 mantissa bits.  The backward uses it to form delta without the rounding
 * error of the bf16 output (the reference forms delta from the rounded output, :282).
 * saved may be NULL; if given, its buffers are filled (see sa2_saved). */
int sa2_fwd(const sa2_problem *prob,
            const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
            const sa2_tensor *v1, const sa2_tensor *v2,
            const sa2_tensor *out, const sa2_tensor *out_residual, float *lse,
            const sa2_saved *saved, void *hip_stream);

/* delta[b,h,n] = sum_d (out + out_residual) * dout; out_residual may be NULL.
 * Replaces backward_preprocess_do_o_dot
 * (triton_two_simplicial_attention.py:834-849; kernel :230-286). */
int sa2_bwd_delta(const sa2_problem *prob, const sa2_tensor *out, const sa2_tensor *out_residual,
                  const sa2_tensor *dout, float *delta, void *hip_stream);

/* Bytes of device workspace the backward needs for this problem; -1 if the problem is invalid.
 * The reference has no counterpart: its five fp32 gradient buffers of
 * triton_two_simplicial_attention.py:853-857 play the same role.  The workspace holds the fp32
 * partial rows of dK2 and dV2 (one block per 32-row query tile; dK2 rows first, the dV2 rows
 * behind them are not needed when the call is given the forward's saved partials, sa2_saved) and,
 * once those are spent, for small grids the two fp32 partial results of dK1/dV1 per key slab.
 * sa2_bwd_workspace_bytes_with_saved() is the size that suffices when saved partials are given. */
int64_t sa2_bwd_workspace_bytes(const sa2_problem *prob);
int64_t sa2_bwd_workspace_bytes_with_saved(const sa2_problem *prob);

/* dQ, dK2, dV2.  Replaces both passes of two_simplicial_attn_bwd_kv2q_kernel
 * (triton_two_simplicial_attention.py:938-1004; kernel :515-712; dq :697-699,709;
 * dk2/dv2 :680-683, :695, :702-707).  One kernel owns the query rows (dQ complete,
 * dK2/dV2 as partial rows in the workspace), a second one sums the partial rows and
 * the query heads of a group.  No atomics; results are bitwise reproducible.
 * saved may be NULL; if it holds what sa2_fwd wrote for these inputs, dV2 is formed from it
 * instead of from a recomputation of the attention weights. */
int sa2_bwd_dq_dkv2(const sa2_problem *prob,
                    const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                    const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout,
                    const float *lse, const float *delta, const sa2_saved *saved,
                    const sa2_tensor *dq, const sa2_tensor *dk2, const sa2_tensor *dv2,
                    void *workspace, int64_t workspace_bytes, void *hip_stream);

/* dK1, dV1 (first key/value set, window w1).  Replaces two_simplicial_attn_bwd_kv1_kernel
 * (triton_two_simplicial_attention.py:868-934; kernel :298-503). */
int sa2_bwd_dkv1(const sa2_problem *prob,
                 const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                 const sa2_tensor *v1, const sa2_tensor *v2, const sa2_tensor *dout,
                 const float *lse, const float *delta,
                 const sa2_tensor *dk1, const sa2_tensor *dv1, void *hip_stream);

/* Whole backward: delta, dQ, dK1/dV1, dK2/dV2 in stream order.  Replaces the body
 * of SlidingTwoSimplicialAttention.backward (triton_two_simplicial_attention.py:808-1006).
 * delta_ws is a caller-owned fp32 (batch, heads, seq) buffer, workspace a caller-owned
 * buffer of at least sa2_bwd_workspace_bytes() bytes; out_residual and saved may be
 * NULL (see sa2_fwd).  Gradients are
 * written in the activation dtype and need no prior zeroing. */
int sa2_bwd(const sa2_problem *prob,
            const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
            const sa2_tensor *v1, const sa2_tensor *v2,
            const sa2_tensor *out, const sa2_tensor *out_residual, const sa2_tensor *dout,
            const float *lse, const sa2_saved *saved, float *delta_ws,
            const sa2_tensor *dq, const sa2_tensor *dk1, const sa2_tensor *dk2,
            const sa2_tensor *dv1, const sa2_tensor *dv2,
            void *workspace, int64_t workspace_bytes, void *hip_stream);

/* Whole backward for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): sa2_bwd without the delta_ws and workspace arguments.
 * No counterpart in the reference.  The delta rows and the dK2/dV2 partial rows live in a
 * device array of SA2_NOALLOC_SCRATCH_BYTES that is part of the library image (each GPU the
 * library runs on holds one copy until the process ends); the call allocates and frees nothing.
 * Problems that need more than that (sa2_bwd_noalloc_scratch_bytes() says how much) are refused
 * with SA2_ERR_UNSUPPORTED: use sa2_bwd with caller-owned buffers.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race; calls
 * in stream order on one stream do not.  The array keeps the previous call's contents; nothing
 * needs clearing because every element a kernel reads is written earlier in the same call.
 * Results are bit-identical to sa2_bwd's. */
#define SA2_NOALLOC_SCRATCH_BYTES (64ll << 20)
int64_t sa2_bwd_noalloc_scratch_bytes(const sa2_problem *prob);   /* -1 if the problem is invalid */
int sa2_bwd_noalloc(const sa2_problem *prob,
                    const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                    const sa2_tensor *v1, const sa2_tensor *v2,
                    const sa2_tensor *out, const sa2_tensor *out_residual, const sa2_tensor *dout,
                    const float *lse, const sa2_saved *saved,
                    const sa2_tensor *dq, const sa2_tensor *dk1, const sa2_tensor *dk2,
                    const sa2_tensor *dv1, const sa2_tensor *dv2, void *hip_stream);

/* ---- module pre-processing around the attention core (first of the "next" rows) ----
 *
 * Fused split + per-head RMSNorm of the qkv projection.  Replaces, for
 * number_key_value_sets = 2 and head_first_dim = False, the split / unflatten / chunk /
 * five RMSNorm calls of HigherOrderAttention.forward (simplicial_mha.py:116-127): reads
 * the projection output qkv[b, n, :] (bf16, channels q (head, d) | k (head, set, d) |
 * v (head, set, d), row_stride elements between tokens) once and writes the five
 * (batch, seq, heads, dim_head) tensors the attention entry points take.
 * w_* are bf16 [dim_head] RMSNorm weights (NULL: ones); y = x * rsqrt(mean(x^2) + eps) * w
 * in fp32, rounded once.  rstd (fp32 [batch*seq][heads + 4*kv_heads]) is kept for the
 * backward.  prob->w1/w2/scale are not used. */
int sa2_qkv_norm_fwd(const sa2_problem *prob, const void *qkv, int64_t row_stride,
                     const void *w_q, const void *w_k1, const void *w_k2, const void *w_v1, const void *w_v2,
                     float eps,
                     const sa2_tensor *q, const sa2_tensor *k1, const sa2_tensor *k2,
                     const sa2_tensor *v1, const sa2_tensor *v2, float *rstd, void *hip_stream);

/* Bytes of workspace sa2_qkv_norm_bwd needs (partial weight gradients); -1 if invalid. */
int64_t sa2_qkv_norm_bwd_workspace_bytes(const sa2_problem *prob);

/* Backward of sa2_qkv_norm_fwd: dqkv (bf16, layout of qkv) from the gradients of the five
 * outputs, and dw (fp32 [5][dim_head], order q, k1, k2, v1, v2; written, not accumulated).
 * The autograd of the reference's five RMSNorm modules plus the backward of split /
 * chunk (simplicial_mha.py:116-127).  Bitwise reproducible (no atomics). */
int sa2_qkv_norm_bwd(const sa2_problem *prob, const void *qkv, int64_t row_stride,
                     const void *w_q, const void *w_k1, const void *w_k2, const void *w_v1, const void *w_v2,
                     const sa2_tensor *dq, const sa2_tensor *dk1, const sa2_tensor *dk2,
                     const sa2_tensor *dv1, const sa2_tensor *dv2, const float *rstd,
                     void *dqkv, float *dw, void *workspace, int64_t workspace_bytes, void *hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* SA2_H */
