// Shared declarations of the gfx950 causal-product library (internal; the public
// surface is include/ftc_causal_product.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ftc_causal_product.h"

namespace ftc {

// One operand of a scan: rows of `width` contiguous elements addressed by
// (chain = n*H + h, position l).  Strides in elements.
struct Operand {
    const void *ptr;
    int64_t stride_n, stride_h, stride_l;
    int32_t dtype;  // ftc_dtype
    int32_t width;  // elements per row
};

struct OperandOut {
    void *ptr;
    int64_t stride_n, stride_h, stride_l;
    int32_t dtype;
    int32_t width;
};

// A D x F fp32 state per chain: element (n, h, d, f) at ptr[n*stride_n + h*stride_h +
// d*stride_d + f].  ptr == nullptr: absent.
struct StateRef {
    float *ptr;
    int64_t stride_n, stride_h, stride_d;
};

inline Operand as_operand(const ftc_tensor4 *t) {
    return Operand{t->ptr, t->stride[0], t->stride[1], t->stride[2], t->dtype, (int32_t)t->size[3]};
}
inline OperandOut as_operand_out(const ftc_tensor4 *t) {
    return OperandOut{t->ptr, t->stride[0], t->stride[1], t->stride[2], t->dtype,
                      (int32_t)t->size[3]};
}

// Records the message returned by ftc_last_error() and returns `code`.
int fail(int code, const char *fmt, ...);
// Records which kernel the last launch on this thread used (ftc_last_kernel()).
void note_kernel(const char *name);
// The FTC_* environment variables (tuning aids for measurements; none is needed in normal
// use), read once when the library is first used and again only by ftc_tuning_reload():
// -1 stands for "not set".
struct Tuning {
    int split, pad, wg, tp, tp_segs, tpx, tpx_segs, seg_chunks, group, dma, tph;
    double tp_ratio;  // < 0: not set
    const char *stamp_ptr;
    uint64_t generation;  // counts the reloads: memoised plans are dropped when it changes
};
const Tuning &tuning();

// Plan-only mode of the calling thread (ftc_causal_dot_plan): the scan functions describe the
// launch they would make, one line each, instead of making it, and touch no GPU.
bool plan_only();
void note_plan(const char *fmt, ...);

// bf16 <-> fp32 with round-to-nearest-even (finite inputs; NaN stays NaN).
__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float load_as_f32(const void *base, int32_t dtype, int64_t idx) {
    return dtype == FTC_F32 ? ((const float *)base)[idx]
                            : bf16_to_f32(((const uint16_t *)base)[idx]);
}
__device__ __forceinline__ void store_from_f32(void *base, int32_t dtype, int64_t idx, float x) {
    if (dtype == FTC_F32)
        ((float *)base)[idx] = x;
    else
        ((uint16_t *)base)[idx] = f32_to_bf16(x);
}

// ---------------------------------------------------------------------------
// Generic scan (any D, F <= 512, any L): ftc_generic.hip
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (reverse: j >= l)
//
// a, b: rows of D elements; v, out: rows of F elements.
// ---------------------------------------------------------------------------
constexpr int kGenericMaxDim = 512;

int64_t generic_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F);

int generic_scan(const Operand &a, const Operand &b, const Operand &v, const OperandOut &out,
                 int64_t N, int64_t H, int64_t L, bool reverse, const StateRef &initial,
                 const StateRef &final_, void *workspace, size_t workspace_bytes,
                 hipStream_t stream);

// ---------------------------------------------------------------------------
// MFMA scan: ftc_mfma.hip + ftc_mfma_kernel.h.  One wavefront keeps a D x F state with
// (D, F) in {32, 64, 96, 128} x multiples of 32 and D * F <= 4096; wider outputs are cut into
// column slices of such widths, each slice a scan of its own over the same a and b rows.
// Rows must be 16-byte aligned; all-fp32 operands or the bf16 combinations of a forward /
// backward call.
// ---------------------------------------------------------------------------
struct ScanDesc {
    Operand a, b, v;
    OperandOut out;
    bool reverse;
    StateRef initial;  // optional: the state the scan starts from (read)
    StateRef final_;   // optional: where the state after the last position goes (written)
};
constexpr int kMfmaMaxScans = 4;   // scans per launch
constexpr int kMfmaMaxSlices = 16;  // column slices per scan

// Widths of the column slices that cover F output columns for state rows of width D;
// returns their number (0: this shape does not go to the MFMA path).
int mfma_slice_widths(int64_t D, int64_t F, int (&widths)[kMfmaMaxSlices]);
// Whether the MFMA kernels can read (or write) rows of this width where they lie: 16-byte
// aligned, at most 65536 elements apart.
bool mfma_operand_in_place(const void *ptr, int64_t stride_n, int64_t stride_h, int64_t stride_l,
                           int dtype, int width, int64_t L);
// Column slice [col0, col0 + width) of a scan: same a and b rows, offset v and out rows.
ScanDesc mfma_slice(const ScanDesc &scan, int col0, int width);
bool mfma_scan_supported(const ScanDesc &scan, int64_t L);
// true when two supported scans can share a launch (same widths, same element types)
bool mfma_scan_same_launch(const ScanDesc &x, const ScanDesc &y);
// Workspace for `nscans` scans of one (D, F) run side by side in one launch.
int64_t mfma_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                                  int nscans);
// The chain-parallel kernel: all-fp32 scans of one shape whose state has 16 to 128 rows and
// columns, widths multiples of 4 (also widths that mfma_scan_supported
// does not list).  True when mfma_scan would run these scans, side by side, on that kernel;
// its workspace (part of mfma_scan_workspace_bytes where both apply).
// `forced`: these scans are parts of scans that the caller has split by state rows because
// only this kernel can take them (any multiple of 4 will do, at any size).
bool mfma_tp_takes(const ScanDesc *scans, int nscans, int64_t N, int64_t H, int64_t L,
                   bool forced = false);
int64_t mfma_tp_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F, int nscans,
                                bool forced = false);
// The fused attention form of a forward scan: a and b go through the feature map
// elu(x) + 1, rows of b at or beyond key_lengths[n] count as zero, and every output row is
// divided by (phi(a_l) . sum_{j <= l} phi(b_j) + eps).
struct FusedAttention {
    const int64_t *key_lengths;  // N values on the device, or nullptr (every key counts)
    float eps;
    // optional: where the denominators (phi(a_l) . sum_{j <= l} phi(b_j) + eps) go, one float
    // per position at denominators[n den_sn + h den_sh + l] (the backward needs them)
    float *denominators = nullptr;
    int64_t den_sn = 0, den_sh = 0;
};
bool fused_attention_supported(const ScanDesc &scan, int64_t L);
int64_t fused_attention_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F);
// Runs scans[0..nscans) (all of the same row widths) in one launch.  `fused`: a single
// forward scan in its fused attention form.  `may_chain_parallel` = false keeps the launch
// off the chain-parallel kernel (column slices of a scan that it has declined as a whole).
int mfma_scan(const ScanDesc *scans, int nscans, int64_t N, int64_t H, int64_t L,
              void *workspace, size_t workspace_bytes, hipStream_t stream,
              const FusedAttention *fused = nullptr, bool may_chain_parallel = true,
              bool forced = false);

// Backward of the fused attention (ftc_attention.hip): the kernels around the three scans.
// prep: Qf = phi(q), Kf = phi(k) [l < key_len] (dense rows of E floats), gz = g / den (dense rows
// of M floats), dd = -(g . out) / den (one float per position), and per (chain, segment of
// positions) the totals of Kf and of dd Qf (`sums`: 2 E floats each).  finish: dq and dk, which
// hold the scans' results, get the prefix sums that the denominator contributes and phi'.
int64_t attention_backward_segments(int64_t L);
void launch_attention_backward_prep(const Operand &q, const Operand &k, const Operand &g,
                                    const Operand &out, const Operand &den, const int64_t *key_len,
                                    int64_t N, int64_t H, int64_t L, int E, int M, float *Qf,
                                    float *Kf, float *gz, float *dd, float *sums,
                                    hipStream_t stream);
void launch_attention_backward_finish(const Operand &q, const Operand &k, const int64_t *key_len,
                                      const float *dd, float *sums, int64_t N, int64_t H,
                                      int64_t L, int E, const OperandOut &dq, const OperandOut &dk,
                                      hipStream_t stream);

// Fill every row of `out` with zeros (used for empty contractions).
int zero_rows(const OperandOut &out, int64_t N, int64_t H, int64_t L, hipStream_t stream);

}  // namespace ftc
