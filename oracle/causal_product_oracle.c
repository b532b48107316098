/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's causal
 * linear-attention product, used as the parity checker for the HIP kernels and
 * as the reported CPU baseline.  Nothing in the shipped package may call it.
 *
 * Algorithm restated from the reference's CPU extension:
 *   fast_transformers/causal_product/causal_product_cpu.cpp:16-26   rank-1 update   (vvt_dot)
 *   fast_transformers/causal_product/causal_product_cpu.cpp:35-51   vector x matrix (vm_dot)
 *   fast_transformers/causal_product/causal_product_cpu.cpp:60-73   matrix x vector (vmt_dot)
 *   fast_transformers/causal_product/causal_product_cpu.cpp:82-124  forward
 *   fast_transformers/causal_product/causal_product_cpu.cpp:133-209 backward
 *
 * Per (n, h) chain, sequentially over l (position l sees key l: update, then read):
 *   forward : S += k_l v_l^T ;  out_l = S^T q_l
 *   backward: pass 1 (l ascending)  S += k_l v_l^T ; dQ_l = S g_l
 *             pass 2 (l descending) R += q_l g_l^T ; dK_l = R v_l ; dV_l = R^T k_l
 * The (n, h) chains are distributed over OpenMP threads exactly as the
 * reference does (collapse(2), one private E x M state per chain).
 *
 * Summation order inside one position follows the reference: the E x M state
 * is row-major, out_l accumulates over e ascending, dQ_l/dK_l accumulate over
 * m ascending.  The file is compiled twice: REAL=float (the checker, built with
 * the reference's flags -O2 -fopenmp -ffast-math) and REAL=double (error
 * yardstick, built without -ffast-math).
 *
 * Pinned by tests/test_oracle.py: against the reference's own compiled CPU
 * extension (oracle/_ref, when built), against the dense closed form
 * tril(Q K^T) V and its autograd gradients in float64 (the check the
 * reference's tests use), against brute-force triple loops on tiny inputs, and
 * against invariants (E = 1 reduces to a cumulative sum, causality, time
 * reversal between the forward and the dV pass).
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef REAL
#define REAL float
#endif

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#ifndef SUFFIX
#define SUFFIX f32
#endif
#define FN(name) CAT(CAT(name, _), SUFFIX)

/* A 4-d view: element (n, h, l, x) lives at p[n*sn + h*sh + l*sl + x*sx]. */
typedef struct {
    REAL *p;
    int64_t sn, sh, sl, sx;
} view4;

static inline REAL *row(const view4 *t, int n, int h, int l) {
    return t->p + (int64_t)n * t->sn + (int64_t)h * t->sh + (int64_t)l * t->sl;
}

/* state[a][b] += x[a] * y[b]           (reference: vvt_dot, cpp:16-26) */
static inline void rank1_add(const REAL *x, int64_t xs, const REAL *y, int64_t ys,
                             REAL *state, int A, int B) {
    for (int a = 0; a < A; a++) {
        const REAL xa = x[a * xs];
        REAL *srow = state + (size_t)a * B;
        for (int b = 0; b < B; b++) srow[b] += xa * y[b * ys];
    }
}

/* out[b] = sum_a x[a] * state[a][b]    (reference: vm_dot, cpp:35-51; zero, then a ascending) */
static inline void vec_mat(const REAL *x, int64_t xs, const REAL *state,
                           REAL *out, int64_t os, int A, int B, REAL *tmp) {
    for (int b = 0; b < B; b++) tmp[b] = 0;
    for (int a = 0; a < A; a++) {
        const REAL xa = x[a * xs];
        const REAL *srow = state + (size_t)a * B;
        for (int b = 0; b < B; b++) tmp[b] += xa * srow[b];
    }
    for (int b = 0; b < B; b++) out[b * os] = tmp[b];
}

/* out[a] = sum_b state[a][b] * y[b]    (reference: vmt_dot, cpp:60-73; b ascending) */
static inline void mat_vec(const REAL *y, int64_t ys, const REAL *state,
                           REAL *out, int64_t os, int A, int B) {
    for (int a = 0; a < A; a++) {
        const REAL *srow = state + (size_t)a * B;
        REAL s = 0;
        for (int b = 0; b < B; b++) s += srow[b] * y[b * ys];
        out[a * os] = s;
    }
}

/* Strides are in elements.  q,k: (N,H,L,E); v,out: (N,H,L,M). */
int FN(oracle_causal_dot_product)(
    const REAL *q, const int64_t *q_stride, const REAL *k, const int64_t *k_stride,
    const REAL *v, const int64_t *v_stride, REAL *out, const int64_t *o_stride,
    int N, int H, int L, int E, int M) {
    const view4 Q = {(REAL *)q, q_stride[0], q_stride[1], q_stride[2], q_stride[3]};
    const view4 K = {(REAL *)k, k_stride[0], k_stride[1], k_stride[2], k_stride[3]};
    const view4 V = {(REAL *)v, v_stride[0], v_stride[1], v_stride[2], v_stride[3]};
    const view4 O = {out, o_stride[0], o_stride[1], o_stride[2], o_stride[3]};
    int failed = 0;

    /* reference cpp:101-123 */
#pragma omp parallel for collapse(2)
    for (int n = 0; n < N; n++) {
        for (int h = 0; h < H; h++) {
            REAL *S = (REAL *)calloc((size_t)E * M + M, sizeof(REAL));
            if (!S) {
#pragma omp atomic write
                failed = 1;
                continue;
            }
            REAL *tmp = S + (size_t)E * M;
            for (int l = 0; l < L; l++) {
                rank1_add(row(&K, n, h, l), K.sx, row(&V, n, h, l), V.sx, S, E, M);
                vec_mat(row(&Q, n, h, l), Q.sx, S, row(&O, n, h, l), O.sx, E, M, tmp);
            }
            free(S);
        }
    }
    return failed ? -1 : 0;
}

/*
 * The forward with the running state handed in and out: S starts from s0 (contiguous
 * (N,H,E,M), or NULL for zeros) and is copied to s_out (or NULL) after the last position.
 * The state and its update are the Si of the reference's step-wise module
 * (fast_transformers/recurrent/attention/self_attention/linear_attention.py:63-66,79-80:
 * "Si = Si + einsum('nhd,nhm->nhdm', K, value)", read out at :86 without the normaliser);
 * the loop is the forward's above.  Pinned by tests/test_oracle.py: two pieces with the
 * state handed over equal one pass of the (pinned) forward, the final state equals the
 * dense K^T V, and a non-zero s0 adds Q s0 to every row.
 */
int FN(oracle_causal_dot_product_state)(
    const REAL *q, const int64_t *q_stride, const REAL *k, const int64_t *k_stride,
    const REAL *v, const int64_t *v_stride, const REAL *s0, REAL *out, const int64_t *o_stride,
    REAL *s_out, int N, int H, int L, int E, int M) {
    const view4 Q = {(REAL *)q, q_stride[0], q_stride[1], q_stride[2], q_stride[3]};
    const view4 K = {(REAL *)k, k_stride[0], k_stride[1], k_stride[2], k_stride[3]};
    const view4 V = {(REAL *)v, v_stride[0], v_stride[1], v_stride[2], v_stride[3]};
    const view4 O = {out, o_stride[0], o_stride[1], o_stride[2], o_stride[3]};
    int failed = 0;
#pragma omp parallel for collapse(2)
    for (int n = 0; n < N; n++) {
        for (int h = 0; h < H; h++) {
            REAL *S = (REAL *)calloc((size_t)E * M + M, sizeof(REAL));
            if (!S) {
#pragma omp atomic write
                failed = 1;
                continue;
            }
            REAL *tmp = S + (size_t)E * M;
            const size_t chain = ((size_t)n * H + h) * E * M;
            if (s0) memcpy(S, s0 + chain, (size_t)E * M * sizeof(REAL));
            for (int l = 0; l < L; l++) {
                rank1_add(row(&K, n, h, l), K.sx, row(&V, n, h, l), V.sx, S, E, M);
                vec_mat(row(&Q, n, h, l), Q.sx, S, row(&O, n, h, l), O.sx, E, M, tmp);
            }
            if (s_out) memcpy(s_out + chain, S, (size_t)E * M * sizeof(REAL));
            free(S);
        }
    }
    return failed ? -1 : 0;
}

/* g: (N,H,L,M); dq,dk: (N,H,L,E); dv: (N,H,L,M). */
int FN(oracle_causal_dot_backward)(
    const REAL *q, const int64_t *q_stride, const REAL *k, const int64_t *k_stride,
    const REAL *v, const int64_t *v_stride, const REAL *g, const int64_t *g_stride,
    REAL *dq, const int64_t *dq_stride, REAL *dk, const int64_t *dk_stride,
    REAL *dv, const int64_t *dv_stride, int N, int H, int L, int E, int M) {
    const view4 Q = {(REAL *)q, q_stride[0], q_stride[1], q_stride[2], q_stride[3]};
    const view4 K = {(REAL *)k, k_stride[0], k_stride[1], k_stride[2], k_stride[3]};
    const view4 V = {(REAL *)v, v_stride[0], v_stride[1], v_stride[2], v_stride[3]};
    const view4 G = {(REAL *)g, g_stride[0], g_stride[1], g_stride[2], g_stride[3]};
    const view4 DQ = {dq, dq_stride[0], dq_stride[1], dq_stride[2], dq_stride[3]};
    const view4 DK = {dk, dk_stride[0], dk_stride[1], dk_stride[2], dk_stride[3]};
    const view4 DV = {dv, dv_stride[0], dv_stride[1], dv_stride[2], dv_stride[3]};
    int failed = 0;

    /* reference cpp:158-208 */
#pragma omp parallel for collapse(2)
    for (int n = 0; n < N; n++) {
        for (int h = 0; h < H; h++) {
            REAL *S = (REAL *)calloc((size_t)E * M + M, sizeof(REAL));
            if (!S) {
#pragma omp atomic write
                failed = 1;
                continue;
            }
            REAL *tmp = S + (size_t)E * M;
            /* pass 1, cpp:165-180: rebuild the forward state, dQ_l = S g_l */
            for (int l = 0; l < L; l++) {
                rank1_add(row(&K, n, h, l), K.sx, row(&V, n, h, l), V.sx, S, E, M);
                mat_vec(row(&G, n, h, l), G.sx, S, row(&DQ, n, h, l), DQ.sx, E, M);
            }
            /* pass 2, cpp:183-206: reverse state R = sum_{j>=l} q_j g_j^T */
            memset(S, 0, (size_t)E * M * sizeof(REAL));
            for (int l = L - 1; l >= 0; l--) {
                rank1_add(row(&Q, n, h, l), Q.sx, row(&G, n, h, l), G.sx, S, E, M);
                mat_vec(row(&V, n, h, l), V.sx, S, row(&DK, n, h, l), DK.sx, E, M);
                vec_mat(row(&K, n, h, l), K.sx, S, row(&DV, n, h, l), DV.sx, E, M, tmp);
            }
            free(S);
        }
    }
    return failed ? -1 : 0;
}
