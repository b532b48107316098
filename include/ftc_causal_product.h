/*
 * C ABI of the MI355X (gfx950) causal linear-attention product.
 *
 * This is the drop-in boundary for the native functions that
 * fast_transformers/causal_product/__init__.py:9-17 binds as
 * causal_dot_product / causal_dot_backward (CPU: causal_product_cpu.cpp:82-87,
 * 133-141, 212-225; CUDA: causal_product_cuda.cu:1273-1276, 1438-1444,
 * 1471-1483).  Plain pointers and sizes only: no torch types cross it.
 *
 * Conventions
 *  - Tensors are 4-d views (N, H, L, X) described by ftc_tensor4: a device
 *    pointer, a dtype code and sizes/strides in ELEMENTS.  The innermost
 *    stride must be 1 (the reference CUDA path asserts the same,
 *    causal_product_cuda.cu:774-777); N/H/L strides are free and 64-bit.
 *  - Outputs are caller-allocated and fully overwritten.  They need not be
 *    zero-filled (the reference wrapper zero-fills, __init__.py:41,59-61, but
 *    its CPU kernels overwrite as well, causal_product_cpu.cpp:38-40,70).
 *  - Q, K, V share one dtype: FTC_F32 or FTC_BF16.  The forward output and the
 *    upstream gradient are FTC_F32 (the reference allocates the product with
 *    the default dtype, __init__.py:41); dQ, dK, dV have the input dtype
 *    (__init__.py:59-61).  Accumulation is always fp32.
 *  - Every entry point returns 0 on success or a negative ftc_status; the
 *    message of the last failure on the calling thread is ftc_last_error().
 *    No exception crosses the boundary.
 *  - Work is enqueued on `stream` (a hipStream_t; NULL = the default stream)
 *    of the device that owns the pointers and returns without synchronising.
 *  - The library allocates nothing.  Scratch memory comes in through
 *    `workspace`: device memory of at least the number of bytes the matching
 *    *_workspace_bytes call returns, 256-byte aligned, private to the call
 *    until the enqueued work has finished.  Its first
 *    FTC_WORKSPACE_CONTROL_BYTES bytes are a control block (segment tickets
 *    and ready flags): they must be zero before the first call that uses the
 *    buffer and every call leaves them zero again, so one buffer can serve
 *    any sequence of calls, of any shapes, one at a time.  The rest needs no
 *    initialisation.  Word 2 of the control block is an error word: it stays
 *    zero unless a wavefront gave up waiting for another one (which a correct
 *    launch never does); a caller may read it after synchronising.
 */
#ifndef FTC_CAUSAL_PRODUCT_H
#define FTC_CAUSAL_PRODUCT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FTC_WORKSPACE_CONTROL_BYTES 65536
/* size of the built-in scratch array of ftc_causal_dot_product_static (per GPU) */
#define FTC_STATIC_SCRATCH_BYTES (48u << 20)

enum ftc_dtype { FTC_F32 = 0, FTC_BF16 = 1 };

enum ftc_status {
    FTC_OK = 0,
    FTC_ERR_INVALID = -1,     /* null pointer, shape or dtype mismatch, inner stride != 1 */
    FTC_ERR_UNSUPPORTED = -2, /* a size outside what the kernels cover */
    FTC_ERR_WORKSPACE = -3,   /* workspace missing or too small */
    FTC_ERR_HIP = -4          /* a HIP runtime call failed; see ftc_last_error() */
};

typedef struct ftc_tensor4 {
    void *ptr;         /* device pointer to element (0,0,0,0) */
    int32_t dtype;     /* enum ftc_dtype */
    int64_t size[4];   /* N, H, L, X */
    int64_t stride[4]; /* in elements; stride[3] must be 1 */
} ftc_tensor4;

/* Library/ABI version: major * 1000 + minor. */
int ftc_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *ftc_last_error(void);

/*
 * Name of the kernel that the last launch made from this thread used ("" before the first):
 * which of the library's scan kernels the planner chose for the sizes at hand.  For
 * measurement and profiling; no counterpart in the reference.
 */
const char *ftc_last_kernel(void);

/*
 * The library reads its FTC_* environment variables (tuning aids for measurements: they force
 * a kernel or a segment length; none is needed in normal use) once, when it is first used.
 * This call reads them again.  Call it with no work in flight, and repeat the workspace
 * queries afterwards: another route may need another workspace.  No counterpart in the
 * reference.
 */
int ftc_tuning_reload(void);

/*
 * What ftc_causal_dot_product (backward == 0) or ftc_causal_dot_backward (backward != 0,
 * all three gradients, dense outputs) would launch for tensors of these shapes, element
 * types and strides: one line of text per launch (kernel, state size, chains, segments, cuts,
 * workspace), written to `text` (at most text_bytes - 1 characters).  Nothing is launched and
 * no GPU is needed; the data pointers are not read and may be NULL.  Returns what the real
 * call would return for these arguments, workspace checks aside.  For tests of the planner
 * and for tuning; no counterpart in the reference.
 */
int ftc_causal_dot_plan(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                        const ftc_tensor4 *values, int backward, char *text, size_t text_bytes);

/*
 * Clears the control block of a workspace (a fill kernel enqueued on `stream`; no memset, so
 * it may be captured in a graph).  No counterpart in the reference.  A workspace needs this
 * once before its first use unless it was allocated zero-filled, and again after a call whose
 * work was cut short (error word non-zero, see above): a control block that is not zero makes
 * every later call on that workspace stop early.
 */
int ftc_workspace_reset(void *workspace, size_t workspace_bytes, void *stream);

/* Scratch bytes ftc_causal_dot_product needs for these sizes (>= 0), or a negative ftc_status. */
int64_t ftc_causal_dot_product_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t E,
                                               int64_t M, int32_t dtype);

/*
 * product[n,h,l,:] = sum_{j<=l} (queries[n,h,l,:] . keys[n,h,j,:]) values[n,h,j,:]
 * Replaces causal_dot_product(queries, keys, values, product)
 * (causal_product_cpu.cpp:82-124, causal_product_cuda.cu:1273-1285).
 * queries, keys: (N,H,L,E); values, product: (N,H,L,M).  Any E and M for fp32 tensors, like
 * the reference's fallback kernels (causal_product_cuda.cu:1243-1269): beyond 512 the call
 * runs piece by piece of the columns and needs the workspace of the query above; bf16
 * tensors: E, M <= 512 (FTC_ERR_UNSUPPORTED beyond).
 */
int ftc_causal_dot_product(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                           const ftc_tensor4 *values, const ftc_tensor4 *product,
                           void *workspace, size_t workspace_bytes, void *stream);

/*
 * ftc_causal_dot_product for callers that cannot allocate device memory or hand in a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same arguments and result as
 * ftc_causal_dot_product, without the workspace: the scratch memory is an array of
 * FTC_STATIC_SCRATCH_BYTES that is part of the library's device code (each GPU the library
 * runs on holds one until the process ends; the HIP runtime places it when the first call
 * on a device loads that part of the library's device code, so make one call before
 * starting a graph capture).  The call itself allocates and frees nothing and enqueues
 * kernels only.  Sizes whose scratch need
 * (ftc_causal_dot_product_workspace_bytes) exceeds the array are refused with
 * FTC_ERR_WORKSPACE -- except that widths which would otherwise run on zero-padded copies
 * in the workspace then run without them, on the slower shape-agnostic kernel, if the
 * array holds what that needs.  All calls on one GPU share that GPU's array: two calls whose work
 * overlaps in time on one GPU (different streams, different threads) race; calls on one
 * stream are safe.
 */
int ftc_causal_dot_product_static(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                  const ftc_tensor4 *values, const ftc_tensor4 *product,
                                  void *stream);

/*
 * The product with the running state handed in and out, for processing a sequence in
 * pieces and for passing a prompt's state on to step-wise decoding:
 *   S_l = initial_state + sum_{j<=l} keys[n,h,j,:] values[n,h,j,:]^T        (E x M per chain)
 *   product[n,h,l,:] = S_l^T queries[n,h,l,:] ;  final_state = S_{L-1}
 * The state is the S_i of the reference's step-wise module
 * (recurrent/attention/self_attention/linear_attention.py:63-90: "Si = Si + einsum(K, V)",
 * then the read-out), which the reference can only reach one position at a time; its
 * batched native op (causal_product_cpu.cpp:82-124) starts from zero and drops the state.
 * initial_state, final_state: (N,H,E,M), FTC_F32, unit stride along M; either may be NULL
 * (start from zero / do not return the state); they must not overlap.  Needs L >= 1 when
 * final_state is given.  Workspace: ftc_causal_dot_product_workspace_bytes.
 */
int ftc_causal_dot_product_state(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                 const ftc_tensor4 *values, const ftc_tensor4 *initial_state,
                                 const ftc_tensor4 *product, const ftc_tensor4 *final_state,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* Scratch bytes ftc_causal_dot_backward needs (>= 0), or a negative ftc_status. */
int64_t ftc_causal_dot_backward_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t E,
                                                int64_t M, int32_t dtype);

/*
 * Gradients of the product with respect to queries, keys and values given
 * grad_out = d loss / d product.  Replaces causal_dot_backward(queries, keys,
 * values, grad_out, grad_queries, grad_keys, grad_values)
 * (causal_product_cpu.cpp:133-209, causal_product_cuda.cu:1438-1467).
 * The reference always computes all three gradients; here a gradient that is not wanted
 * may be passed as NULL and is then skipped.
 */
int ftc_causal_dot_backward(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                            const ftc_tensor4 *values, const ftc_tensor4 *grad_out,
                            const ftc_tensor4 *grad_queries, const ftc_tensor4 *grad_keys,
                            const ftc_tensor4 *grad_values, void *workspace,
                            size_t workspace_bytes, void *stream);

/*
 * Scratch bytes ftc_causal_linear_attention needs (>= 0), FTC_ERR_UNSUPPORTED when no fused
 * kernel covers these sizes, or another negative ftc_status.
 */
int64_t ftc_causal_linear_attention_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t E,
                                                    int64_t M, int32_t dtype);

/*
 * Causally masked linear attention with the feature map elu(x) + 1, in one pass over the
 * rows.  Replaces the body of CausalLinearAttention.forward
 * (attention/causal_linear_attention.py:71-104) for the default feature map
 * (feature_maps/base.py:71-73): the two feature-map passes (:75-76), the key-length mask
 * (:83), cumsum + einsum for the normaliser (:95), causal_linear with its layout copies
 * (:19-24, :98-102) and the final scale (:104):
 *
 *   phi(x) = x > 0 ? x + 1 : exp(x)
 *   Kf[n,h,j,:] = phi(keys[n,h,j,:]) if j < key_lengths[n] else 0
 *   out[n,h,l,:] = sum_{j<=l} (phi(queries[n,h,l,:]) . Kf[n,h,j,:]) values[n,h,j,:]
 *                  / (phi(queries[n,h,l,:]) . sum_{j<=l} Kf[n,h,j,:] + eps)
 *
 * queries, keys: (N,H,L,E) raw projections (before the feature map); values, out:
 * (N,H,L,M); all FTC_F32, any N/H/L strides with 16-byte aligned rows (the module's
 * (N,L,H,X) tensors are passed as permuted views).  key_lengths: N int64 values on the
 * device, or NULL when every key counts.  (For training see
 * ftc_causal_linear_attention_forward and ..._backward below.)  Sizes: E, M in {32, 64};
 * anything else returns FTC_ERR_UNSUPPORTED and the caller composes the result from
 * ftc_causal_dot_product as before.
 */
int ftc_causal_linear_attention(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                const ftc_tensor4 *values, const int64_t *key_lengths, float eps,
                                const ftc_tensor4 *out, void *workspace, size_t workspace_bytes,
                                void *stream);

/*
 * The same forward, for training: it also writes, when `denominators` is not NULL, the
 * denominators of the formula above (eps included), one float per position, which the
 * backward below needs: (N,H,L,1), FTC_F32, unit stride along L.  Workspace:
 * ftc_causal_linear_attention_workspace_bytes.  The reference keeps the corresponding tensor
 * (Z, attention/causal_linear_attention.py:95) alive through autograd.
 */
int ftc_causal_linear_attention_forward(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                        const ftc_tensor4 *values, const int64_t *key_lengths,
                                        float eps, const ftc_tensor4 *out,
                                        const ftc_tensor4 *denominators, void *workspace,
                                        size_t workspace_bytes, void *stream);

/*
 * Scratch bytes ftc_causal_linear_attention_backward needs (>= 0), FTC_ERR_UNSUPPORTED when the
 * sizes are not covered, or another negative ftc_status.
 */
int64_t ftc_causal_linear_attention_backward_workspace_bytes(int64_t N, int64_t H, int64_t L,
                                                             int64_t E, int64_t M, int32_t dtype);

/*
 * Gradients of ftc_causal_linear_attention_forward with respect to the raw queries, keys and
 * values, given grad_out = d loss / d out.  Replaces what autograd does in the reference for
 * CausalLinearAttention.forward (attention/causal_linear_attention.py:71-104): the backward
 * of the two feature-map passes, of the key-length mask, of cumsum and einsum for the
 * normaliser, of the final scale, and causal_dot_backward twice.  With Qf, Kf as above,
 * gz_l = grad_out_l / den_l and dd_l = -(grad_out_l . out_l) / den_l:
 *
 *   dQf_l = sum_{j<=l} (gz_l . v_j) Kf_j + dd_l sum_{j<=l} Kf_j
 *   dKf_j = sum_{l>=j} (v_j . gz_l) Qf_l + sum_{l>=j} dd_l Qf_l
 *   grad_values_j = sum_{l>=j} (Kf_j . Qf_l) gz_l
 *   grad_queries = dQf phi'(queries);  grad_keys_j = dKf_j phi'(keys_j) if j < key_lengths[n] else 0
 *   phi'(x) = x > 0 ? 1 : exp(x)
 *
 * out, denominators: what the forward wrote.  All tensors FTC_F32 with 16-byte aligned rows;
 * a gradient that is not wanted may be passed as NULL.  Sizes: E, M in {32, 64}.  The launch
 * sequence: one element-wise pass (feature maps, gz, dd into the workspace), the three scans
 * of ftc_causal_dot_backward on them, and a prefix-sum pass over grad_queries and grad_keys.
 */
int ftc_causal_linear_attention_backward(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                         const ftc_tensor4 *values, const int64_t *key_lengths,
                                         const ftc_tensor4 *out, const ftc_tensor4 *denominators,
                                         const ftc_tensor4 *grad_out, const ftc_tensor4 *grad_queries,
                                         const ftc_tensor4 *grad_keys, const ftc_tensor4 *grad_values,
                                         void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FTC_CAUSAL_PRODUCT_H */
