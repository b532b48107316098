// Backward of causally masked linear attention with the feature map elu(x) + 1: the element-wise
// and prefix-sum kernels around the three gradient scans (ftc_api.hip:
// ftc_causal_linear_attention_backward puts them together).
//
// Forward (fast_transformers/attention/causal_linear_attention.py:71-104 with
// feature_maps/base.py:71-73), per chain, Qf = phi(q), Kf_j = phi(k_j) [j < key_len]:
//
//   den_l = Qf_l . sum_{j <= l} Kf_j + eps ;  out_l = (sum_{j <= l} (Qf_l . Kf_j) v_j) / den_l
//
// With g the gradient of the loss with respect to out, gz_l = g_l / den_l and
// dd_l = -(g_l . out_l) / den_l (the gradient with respect to den_l):
//
//   dQf_l = sum_{j <= l} (gz_l . v_j) Kf_j  +  dd_l sum_{j <= l} Kf_j
//   dKf_j = sum_{l >= j} (v_j . gz_l) Qf_l  +  sum_{l >= j} dd_l Qf_l
//   dv_j  = sum_{l >= j} (Kf_j . Qf_l) gz_l
//   dq = dQf phi'(q) ;  dk_j = dKf_j phi'(k_j) [j < key_len] ;  phi'(x) = x > 0 ? 1 : exp(x)
//
// The first sums are the three scans of the plain backward on (Qf, Kf, v, gz).  The second
// ones are prefix sums along the chain of rows weighted by a scalar.  The two large kernels here
// give a workgroup one segment of 128 positions of one chain: attn_bwd_prep_kernel also leaves
// the segment's totals, attn_bwd_totals_kernel turns those into the sums over the segments
// before and after each one, and attn_bwd_finish_kernel, one more pass over dq and dk, adds the
// prefix sums (those of the other segments, then of the other threads' runs, then its own run)
// and multiplies by phi'.  Qf and Kf are recomputed there from q and k, which phi' needs anyway.
#include "ftc_common.h"

namespace ftc {
namespace {

constexpr int kRun = 4;                    // consecutive positions per thread of the finish kernel
constexpr int kGroups = 32;                // ... whose workgroup has this many groups of 16 lanes
constexpr int kSegment = kGroups * kRun;   // positions per workgroup

__device__ __forceinline__ float phi(float x) {
    return x > 0.f ? x + 1.f : __builtin_amdgcn_exp2f(x * 1.44269502f);
}
__device__ __forceinline__ float phi_prime(float x) {
    return x > 0.f ? 1.f : __builtin_amdgcn_exp2f(x * 1.44269502f);
}
__device__ __forceinline__ float4 phi(float4 x) { return make_float4(phi(x.x), phi(x.y), phi(x.z), phi(x.w)); }
__device__ __forceinline__ float4 phi_prime(float4 x) {
    return make_float4(phi_prime(x.x), phi_prime(x.y), phi_prime(x.z), phi_prime(x.w));
}
__device__ __forceinline__ float4 operator+(float4 a, float4 b) {
    return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w);
}
__device__ __forceinline__ float4 operator*(float4 a, float4 b) {
    return make_float4(a.x * b.x, a.y * b.y, a.z * b.z, a.w * b.w);
}
__device__ __forceinline__ float4 operator*(float s, float4 a) {
    return make_float4(s * a.x, s * a.y, s * a.z, s * a.w);
}
__device__ __forceinline__ float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }

struct Rows {  // rows of `width` floats at ptr[n sn + h sh + l sl + column]
    const float *ptr;
    int64_t sn, sh, sl;
};
struct RowsOut {
    float *ptr;
    int64_t sn, sh, sl;
};

// One workgroup per (chain, segment); 16 lanes per position, lane c of a group takes columns
// 4 c .. 4 c + 3, and the 16 groups walk the segment 16 positions at a time.
//   Qf, Kf (dense rows of E floats), gz (dense rows of M floats), dd (one float per position)
//   sums[(chain nseg + seg) 2 E + e]     = sum_{l in segment} Kf[l][e]
//   sums[(chain nseg + seg) 2 E + E + e] = sum_{l in segment} dd[l] Qf[l][e]
__global__ __launch_bounds__(256) void attn_bwd_prep_kernel(
    Rows q, Rows k, Rows g, Rows out, Rows den, const int64_t *__restrict__ key_len, int H, int L,
    int E, int M, int nseg, float *__restrict__ Qf, float *__restrict__ Kf, float *__restrict__ gz,
    float *__restrict__ dd, float *__restrict__ sums) {
    __shared__ float4 part[2][16][16];
    // (the heads of one batch entry and segment in neighbouring workgroups: with heads
    // interleaved in memory their rows lie side by side)
    const int h = blockIdx.x % H, seg = (blockIdx.x / H) % nseg, n = blockIdx.x / (H * nseg);
    const int64_t chain = (int64_t)n * H + h;
    const int r = threadIdx.x >> 4, c = threadIdx.x & 15;
    const int len = key_len ? (int)min<int64_t>(key_len[n], L) : L;
    const bool has_e = 4 * c < E, has_m = 4 * c < M;
    const int ce = has_e ? 4 * c : 0, cm = has_m ? 4 * c : 0;
    float4 sk = zero4(), sq = zero4();
#pragma unroll 4
    for (int p = 0; p < kSegment / 16; p++) {
        const int l = seg * kSegment + p * 16 + r;
        const bool live = l < L;
        const int lc = live ? l : L - 1;
        const int64_t pos = chain * L + lc;
        const float4 x = *(const float4 *)(q.ptr + n * q.sn + h * q.sh + lc * q.sl + ce);
        const float4 y = *(const float4 *)(k.ptr + n * k.sn + h * k.sh + lc * k.sl + ce);
        const float4 gg = *(const float4 *)(g.ptr + n * g.sn + h * g.sh + lc * g.sl + cm);
        const float4 o = *(const float4 *)(out.ptr + n * out.sn + h * out.sh + lc * out.sl + cm);
        const float z = 1.0f / den.ptr[n * den.sn + h * den.sh + lc * den.sl];
        float dot = has_m ? (gg.x * o.x + gg.y * o.y) + (gg.z * o.z + gg.w * o.w) : 0.f;
        // sum over the 16 lanes of the position
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 16);
        const float d = -dot * z;
        const float4 xf = phi(x), yf = lc < len ? phi(y) : zero4();
        if (live) {
            if (has_e) {
                *(float4 *)(Qf + pos * E + ce) = xf;
                *(float4 *)(Kf + pos * E + ce) = yf;
                sk = sk + yf;
                sq = sq + d * xf;
            }
            if (has_m) *(float4 *)(gz + pos * M + cm) = z * gg;
            if (c == 0) dd[pos] = d;
        }
    }
    part[0][r][c] = sk;
    part[1][r][c] = sq;
    __syncthreads();
    if (threadIdx.x < 32) {  // 16 lanes per kind of sum, the groups added in a fixed order
        const int which = threadIdx.x >> 4;
        float4 t = part[which][0][c];
        for (int i = 1; i < 16; i++) t = t + part[which][i][c];
        if (has_e) *(float4 *)(sums + ((chain * nseg + seg) * 2 + which) * E + ce) = t;
    }
}

// The segments' totals -> what the segments before (Kf) and after (dd Qf) each one add up to,
// in place, each sum in the fixed order that a walk along the chain would take (ascending for
// the first kind, descending for the second).  One workgroup per chain, one lane per kind and
// column; eight totals are in flight at a time.
__global__ __launch_bounds__(128) void attn_bwd_totals_kernel(float *__restrict__ sums, int E, int nseg) {
    const int which = threadIdx.x >> 6, col = threadIdx.x & 63;
    if (col >= E) return;
    float *s = sums + ((int64_t)blockIdx.x * nseg * 2 + which) * E + col;
    const int64_t step = 2 * (int64_t)E;
    float run = 0.f;
    for (int i0 = 0; i0 < nseg; i0 += 8) {
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = which == 0 ? i0 + j : nseg - 1 - (i0 + j);
            x[j] = i0 + j < nseg ? s[i * step] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int i = which == 0 ? i0 + j : nseg - 1 - (i0 + j);
            if (i0 + j < nseg) s[i * step] = run;
            run += x[j];
        }
    }
}

// One workgroup of 32 groups per (chain, segment); 16 lanes per position as above, and group r takes the
// run of kRun consecutive positions seg kSegment + r kRun ...  dq and dk hold the scans'
// results on entry:
//   dq[l] = (dq[l] + dd[l] sum_{j <= l} Kf[j]) phi'(q[l])
//   dk[j] = (dk[j] + sum_{l >= j} dd[l] Qf[l]) phi'(k[j]) [j < key_len]
__global__ __launch_bounds__(16 * kGroups) void attn_bwd_finish_kernel(
    Rows q, Rows k, const int64_t *__restrict__ key_len, const float *__restrict__ dd,
    const float *__restrict__ sums, int H, int L, int E, int nseg, RowsOut dq, RowsOut dk) {
    __shared__ float4 total[2][kGroups][16];
    // (the heads of one batch entry and segment in neighbouring workgroups: with heads
    // interleaved in memory their rows lie side by side)
    const int h = blockIdx.x % H, seg = (blockIdx.x / H) % nseg, n = blockIdx.x / (H * nseg);
    const int64_t chain = (int64_t)n * H + h;
    const int r = threadIdx.x >> 4, c = threadIdx.x & 15;
    const int len = key_len ? (int)min<int64_t>(key_len[n], L) : L;
    const bool has_e = 4 * c < E;
    const int ce = has_e ? 4 * c : 0;
    const int first = seg * kSegment + r * kRun;
    const float *qrow = q.ptr + n * q.sn + h * q.sh + ce;
    const float *krow = k.ptr + n * k.sn + h * k.sh + ce;

    float4 kf[kRun], qd[kRun], pq[kRun], pk[kRun];
    float d[kRun];
#pragma unroll
    for (int i = 0; i < kRun; i++) {
        const int l = first + i;
        const bool live = l < L;
        const int lc = live ? l : L - 1;
        const float4 x = *(const float4 *)(qrow + lc * q.sl);
        const float4 y = *(const float4 *)(krow + lc * k.sl);
        d[i] = dd[chain * L + lc];
        pq[i] = phi_prime(x);
        pk[i] = phi_prime(y);
        kf[i] = live && l < len ? phi(y) : zero4();
        qd[i] = live ? d[i] * phi(x) : zero4();
    }
    // within the run: sums up to and including each position, and from each position on
#pragma unroll
    for (int i = 1; i < kRun; i++) kf[i] = kf[i] + kf[i - 1];
#pragma unroll
    for (int i = kRun - 2; i >= 0; i--) qd[i] = qd[i] + qd[i + 1];
    total[0][r][c] = kf[kRun - 1];
    total[1][r][c] = qd[0];
    // what the segments before (for dq) and after (for dk) this one add (attn_bwd_totals_kernel)
    const float *s = sums + ((chain * nseg + seg) * 2) * E + ce;
    float4 ck = *(const float4 *)s, cq = *(const float4 *)(s + E);
    __syncthreads();
    // and the runs before and after this one in the segment
    for (int i = 0; i < r; i++) ck = ck + total[0][i][c];
    for (int i = kGroups - 1; i > r; i--) cq = cq + total[1][i][c];
    if (!has_e) return;
    if (dq.ptr) {
        float *row = dq.ptr + n * dq.sn + h * dq.sh + ce;
        float4 have[kRun];
#pragma unroll
        for (int i = 0; i < kRun; i++)
            if (first + i < L) have[i] = *(const float4 *)(row + (first + i) * dq.sl);
#pragma unroll
        for (int i = 0; i < kRun; i++)
            if (first + i < L)
                *(float4 *)(row + (first + i) * dq.sl) = (have[i] + d[i] * (ck + kf[i])) * pq[i];
    }
    if (dk.ptr) {
        float *row = dk.ptr + n * dk.sn + h * dk.sh + ce;
        float4 have[kRun];
#pragma unroll
        for (int i = 0; i < kRun; i++)
            if (first + i < L) have[i] = *(const float4 *)(row + (first + i) * dk.sl);
#pragma unroll
        for (int i = 0; i < kRun; i++)
            if (first + i < L)
                *(float4 *)(row + (first + i) * dk.sl) =
                    first + i < len ? (have[i] + (cq + qd[i])) * pk[i] : zero4();
    }
}

Rows rows_of(const Operand &t) { return Rows{(const float *)t.ptr, t.stride_n, t.stride_h, t.stride_l}; }
RowsOut rows_of(const OperandOut &t) { return RowsOut{(float *)t.ptr, t.stride_n, t.stride_h, t.stride_l}; }

}  // namespace

int64_t attention_backward_segments(int64_t L) { return (L + kSegment - 1) / kSegment; }

void launch_attention_backward_prep(const Operand &q, const Operand &k, const Operand &g,
                                    const Operand &out, const Operand &den, const int64_t *key_len,
                                    int64_t N, int64_t H, int64_t L, int E, int M, float *Qf,
                                    float *Kf, float *gz, float *dd, float *sums,
                                    hipStream_t stream) {
    const int nseg = (int)attention_backward_segments(L);
    hipLaunchKernelGGL(attn_bwd_prep_kernel, dim3((unsigned)(N * H * nseg)), dim3(256), 0, stream,
                       rows_of(q), rows_of(k), rows_of(g), rows_of(out), rows_of(den), key_len, (int)H,
                       (int)L, E, M, nseg, Qf, Kf, gz, dd, sums);
}

void launch_attention_backward_finish(const Operand &q, const Operand &k, const int64_t *key_len,
                                      const float *dd, float *sums, int64_t N, int64_t H,
                                      int64_t L, int E, const OperandOut &dq, const OperandOut &dk,
                                      hipStream_t stream) {
    const int nseg = (int)attention_backward_segments(L);
    hipLaunchKernelGGL(attn_bwd_totals_kernel, dim3((unsigned)(N * H)), dim3(128), 0, stream, sums, E, nseg);
    hipLaunchKernelGGL(attn_bwd_finish_kernel, dim3((unsigned)(N * H * nseg)), dim3(16 * kGroups), 0, stream,
                       rows_of(q), rows_of(k), key_len, dd, (const float *)sums, (int)H, (int)L, E, nseg,
                       rows_of(dq), rows_of(dk));
}

}  // namespace ftc
