// Generic causal scan for gfx950: any row widths D, F in [1, 512], any L, fp32 or
// bf16 rows, fp32 state.  This is the shape-agnostic path (the reference covers
// the same ground with its atomicAdd fallback kernels,
// causal_product_cuda.cu:1204-1434); the MFMA kernels take the common shapes.
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (reverse: j >= l)
//
// One workgroup of 256 lanes owns (chain, L-segment, 64-column slice of F).  Lane
// (g = wave, f = lane in wave) keeps rows [g*DREG, (g+1)*DREG) of column f of the
// D x F state in registers, so a rank-1 update and the read-out of one position
// cost 2*DREG FMAs per lane with the a/b rows read as wave-uniform LDS broadcasts.
// The four partial read-outs of a column (one per wave) are summed through LDS once
// per block of TB positions.
//
// L is split into segments so that short batches still fill 256 CUs: pass 1 writes
// every segment's own state sum, pass 2 turns them into exclusive prefixes (suffixes
// when reversed), pass 3 replays each segment from its prefix and writes the rows.
// With one segment only pass 3 runs.
#include <algorithm>

#include "ftc_common.h"

namespace ftc {
namespace {

constexpr int kThreads = 256;
constexpr int kSlice = 64;  // columns of F per workgroup

struct GenericArgs {
    Operand a, b, v;
    OperandOut out;
    float *states;  // [chain][segment][D][F]
    int64_t L;
    int32_t H, D, F;
    int32_t seg_len, nseg, nslice;
    int32_t reverse;
    int32_t state_only;  // 1: write the segment's state sum; 0: write output rows
    StateRef initial;    // optional state before the first position (single segment: read here)
    StateRef final_;     // optional state after the last position
};

__device__ __forceinline__ int64_t row_offset(int64_t sn, int64_t sh, int64_t sl, int n, int h,
                                              int64_t l) {
    return (int64_t)n * sn + (int64_t)h * sh + l * sl;
}

template <int DREG>
__global__ __launch_bounds__(kThreads) void generic_scan_kernel(GenericArgs p) {
    constexpr int DP = 4 * DREG;            // padded D held by the workgroup
    constexpr int TB = DREG >= 128 ? 8 : 16;  // positions staged per block
    __shared__ float a_s[TB][DP];
    __shared__ float b_s[TB][DP];
    __shared__ float v_s[TB][kSlice];
    __shared__ float part[TB][4][kSlice];

    const int tid = threadIdx.x;
    const int f_local = tid & 63;
    const int g = tid >> 6;

    int64_t wg = blockIdx.x;
    const int slice = (int)(wg % p.nslice);
    wg /= p.nslice;
    const int seg = (int)(wg % p.nseg);
    const int64_t chain = wg / p.nseg;
    const int n = (int)(chain / p.H), h = (int)(chain % p.H);
    const int f0 = slice * kSlice;
    const bool f_ok = f0 + f_local < p.F;

    const int64_t lo = (int64_t)seg * p.seg_len;
    const int64_t hi = min(p.L, lo + (int64_t)p.seg_len);

    float S[DREG];
    float *my_state = p.states ? p.states + ((chain * p.nseg + seg) * (int64_t)p.D) * p.F : nullptr;
    if (!p.state_only && p.nseg > 1) {
#pragma unroll
        for (int i = 0; i < DREG; i++) {
            const int d = g * DREG + i;
            S[i] = (d < p.D && f_ok) ? my_state[(int64_t)d * p.F + f0 + f_local] : 0.f;
        }
    } else if (!p.state_only && p.initial.ptr) {
        // single segment: start from the caller's state
        const float *s0 = p.initial.ptr + (int64_t)n * p.initial.stride_n +
                          (int64_t)h * p.initial.stride_h;
#pragma unroll
        for (int i = 0; i < DREG; i++) {
            const int d = g * DREG + i;
            S[i] = (d < p.D && f_ok) ? s0[(int64_t)d * p.initial.stride_d + f0 + f_local] : 0.f;
        }
    } else {
#pragma unroll
        for (int i = 0; i < DREG; i++) S[i] = 0.f;
    }

    const int64_t a_base = row_offset(p.a.stride_n, p.a.stride_h, 0, n, h, 0);
    const int64_t b_base = row_offset(p.b.stride_n, p.b.stride_h, 0, n, h, 0);
    const int64_t v_base = row_offset(p.v.stride_n, p.v.stride_h, 0, n, h, 0);
    const int64_t o_base = row_offset(p.out.stride_n, p.out.stride_h, 0, n, h, 0);

    const int nblocks = (int)((hi - lo + TB - 1) / TB);
    for (int blk = 0; blk < nblocks; blk++) {
        int64_t p0, p1;
        if (!p.reverse) {
            p0 = lo + (int64_t)blk * TB;
            p1 = min(hi, p0 + TB);
        } else {
            p1 = hi - (int64_t)blk * TB;
            p0 = max(lo, p1 - TB);
        }
        const int nb = (int)(p1 - p0);

        // stage b (always), a (unless only the state is wanted) and the v slice
        for (int idx = tid; idx < TB * DP; idx += kThreads) {
            const int t = idx / DP, d = idx % DP;
            const bool ok = t < nb && d < p.D;
            b_s[t][d] = ok ? load_as_f32(p.b.ptr, p.b.dtype, b_base + (p0 + t) * p.b.stride_l + d)
                           : 0.f;
            if (!p.state_only)
                a_s[t][d] = ok ? load_as_f32(p.a.ptr, p.a.dtype,
                                             a_base + (p0 + t) * p.a.stride_l + d)
                               : 0.f;
        }
        for (int idx = tid; idx < TB * kSlice; idx += kThreads) {
            const int t = idx / kSlice, f = idx % kSlice;
            v_s[t][f] = (t < nb && f0 + f < p.F)
                            ? load_as_f32(p.v.ptr, p.v.dtype,
                                          v_base + (p0 + t) * p.v.stride_l + f0 + f)
                            : 0.f;
        }
        __syncthreads();

        for (int tt = 0; tt < nb; tt++) {
            const int t = p.reverse ? nb - 1 - tt : tt;
            const float cv = v_s[t][f_local];
            const float4 *bp = reinterpret_cast<const float4 *>(&b_s[t][g * DREG]);
            if (p.state_only) {
#pragma unroll
                for (int i = 0; i < DREG; i += 4) {
                    const float4 bb = bp[i / 4];
                    S[i + 0] = fmaf(bb.x, cv, S[i + 0]);
                    S[i + 1] = fmaf(bb.y, cv, S[i + 1]);
                    S[i + 2] = fmaf(bb.z, cv, S[i + 2]);
                    S[i + 3] = fmaf(bb.w, cv, S[i + 3]);
                }
            } else {
                const float4 *ap = reinterpret_cast<const float4 *>(&a_s[t][g * DREG]);
                float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
                for (int i = 0; i < DREG; i += 4) {
                    const float4 bb = bp[i / 4];
                    const float4 aa = ap[i / 4];
                    S[i + 0] = fmaf(bb.x, cv, S[i + 0]);
                    S[i + 1] = fmaf(bb.y, cv, S[i + 1]);
                    S[i + 2] = fmaf(bb.z, cv, S[i + 2]);
                    S[i + 3] = fmaf(bb.w, cv, S[i + 3]);
                    acc0 = fmaf(aa.x, S[i + 0], acc0);
                    acc1 = fmaf(aa.y, S[i + 1], acc1);
                    acc0 = fmaf(aa.z, S[i + 2], acc0);
                    acc1 = fmaf(aa.w, S[i + 3], acc1);
                }
                part[t][g][f_local] = acc0 + acc1;
            }
        }
        __syncthreads();

        if (!p.state_only) {
            for (int idx = tid; idx < nb * kSlice; idx += kThreads) {
                const int t = idx / kSlice, f = idx % kSlice;
                if (f0 + f < p.F) {
                    const float s = (part[t][0][f] + part[t][1][f]) + (part[t][2][f] + part[t][3][f]);
                    store_from_f32(p.out.ptr, p.out.dtype,
                                   o_base + (p0 + t) * p.out.stride_l + f0 + f, s);
                }
            }
            // part/a_s/b_s are rewritten only after the next staging barrier, but the
            // staging loop itself overwrites a_s/b_s/v_s: order it after the reads above.
            __syncthreads();
        }
    }

    if (p.state_only) {
#pragma unroll
        for (int i = 0; i < DREG; i++) {
            const int d = g * DREG + i;
            if (d < p.D && f_ok) my_state[(int64_t)d * p.F + f0 + f_local] = S[i];
        }
    } else if (p.final_.ptr && seg == (p.reverse ? 0 : p.nseg - 1)) {
        // the segment walked last ends on the state after the whole sequence
        float *so = p.final_.ptr + (int64_t)n * p.final_.stride_n + (int64_t)h * p.final_.stride_h;
#pragma unroll
        for (int i = 0; i < DREG; i++) {
            const int d = g * DREG + i;
            if (d < p.D && f_ok) so[(int64_t)d * p.final_.stride_d + f0 + f_local] = S[i];
        }
    }
}

// In place: states[chain][s] <- sum of states[chain][s'] over s' < s (s' > s when reversed).
// The running sum starts from the caller's initial state when there is one.
__global__ __launch_bounds__(kThreads) void generic_state_scan_kernel(float *states, int nseg,
                                                                      int64_t elems, int reverse,
                                                                      StateRef initial, int H,
                                                                      int F) {
    const int64_t blocks_per_chain = (elems + kThreads - 1) / kThreads;
    const int64_t chain = blockIdx.x / blocks_per_chain;
    const int64_t e = (blockIdx.x % blocks_per_chain) * kThreads + threadIdx.x;
    if (e >= elems) return;
    float *base = states + chain * nseg * elems + e;
    float run = 0.f;
    if (initial.ptr)
        run = initial.ptr[(chain / H) * initial.stride_n + (chain % H) * initial.stride_h +
                          (e / F) * initial.stride_d + e % F];
    for (int i = 0; i < nseg; i++) {
        const int s = reverse ? nseg - 1 - i : i;
        const float x = base[(int64_t)s * elems];
        base[(int64_t)s * elems] = run;
        run += x;
    }
}

__global__ __launch_bounds__(kThreads) void zero_rows_kernel(OperandOut out, int64_t H, int64_t L,
                                                             int64_t total) {
    for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < total;
         i += (int64_t)gridDim.x * kThreads) {
        const int x = (int)(i % out.width);
        int64_t r = i / out.width;
        const int64_t l = r % L;
        r /= L;
        const int64_t h = r % H, n = r / H;
        store_from_f32(out.ptr, out.dtype,
                       n * out.stride_n + h * out.stride_h + l * out.stride_l + x, 0.f);
    }
}

struct GenericPlan {
    int nslice, nseg, seg_len;
    int64_t workspace_bytes;
};

GenericPlan make_plan(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F) {
    GenericPlan pl;
    pl.nslice = (int)((F + kSlice - 1) / kSlice);
    const int64_t chains = N * H;
    const int64_t base_wgs = std::max<int64_t>(1, chains * pl.nslice);
    // aim for >= 1024 workgroups (4 per CU) while keeping segments >= 128 positions
    int64_t want = (1024 + base_wgs - 1) / base_wgs;
    int64_t max_seg = std::max<int64_t>(1, L / 128);
    int64_t nseg = std::max<int64_t>(1, std::min(want, max_seg));
    int64_t seg_len = (L + nseg - 1) / nseg;
    seg_len = (seg_len + 15) / 16 * 16;
    nseg = std::max<int64_t>(1, (L + seg_len - 1) / seg_len);
    pl.nseg = (int)nseg;
    pl.seg_len = (int)seg_len;
    // the segment states live behind the workspace's control block, which this path never
    // touches (the MFMA path keeps its tickets and flags there and expects them zero)
    pl.workspace_bytes =
        nseg > 1 ? FTC_WORKSPACE_CONTROL_BYTES + chains * nseg * D * F * (int64_t)sizeof(float) : 0;
    return pl;
}

template <int DREG>
void launch(const GenericArgs &args, int64_t wgs, hipStream_t stream) {
    hipLaunchKernelGGL(generic_scan_kernel<DREG>, dim3((unsigned)wgs), dim3(kThreads), 0, stream,
                       args);
}

void launch_by_width(const GenericArgs &args, int64_t wgs, hipStream_t stream) {
    const int D = args.D;
    if (D <= 32)
        launch<8>(args, wgs, stream);
    else if (D <= 64)
        launch<16>(args, wgs, stream);
    else if (D <= 128)
        launch<32>(args, wgs, stream);
    else if (D <= 256)
        launch<64>(args, wgs, stream);
    else
        launch<128>(args, wgs, stream);
}

}  // namespace

int zero_rows(const OperandOut &out, int64_t N, int64_t H, int64_t L, hipStream_t stream) {
    const int64_t total = N * H * L * out.width;
    if (total == 0) return FTC_OK;
    if (plan_only()) {
        note_plan("zero_rows_kernel: %lld values", (long long)total);
        return FTC_OK;
    }
    const int64_t wgs = std::min<int64_t>((total + kThreads - 1) / kThreads, 65536);
    hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)wgs), dim3(kThreads), 0, stream, out, H, L,
                       total);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(FTC_ERR_HIP, "zero fill launch failed: %s", hipGetErrorString(err));
    return FTC_OK;
}

int64_t generic_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F) {
    return make_plan(N, H, L, D, F).workspace_bytes;
}

int generic_scan(const Operand &a, const Operand &b, const Operand &v, const OperandOut &out,
                 int64_t N, int64_t H, int64_t L, bool reverse, const StateRef &initial,
                 const StateRef &final_, void *workspace, size_t workspace_bytes,
                 hipStream_t stream) {
    note_kernel("generic_scan_kernel");
    const int64_t D = a.width, F = v.width;
    if (D < 1 || F < 1 || D > kGenericMaxDim || F > kGenericMaxDim)
        return fail(FTC_ERR_UNSUPPORTED, "row widths must be in [1, %d] (got %lld and %lld)",
                    kGenericMaxDim, (long long)D, (long long)F);
    if (b.width != D || out.width != F) return fail(FTC_ERR_INVALID, "operand widths disagree");
    const GenericPlan pl = make_plan(N, H, L, D, F);
    if (plan_only()) {
        note_plan("generic_scan_kernel: state %lld x %lld, %s, workspace %lld bytes", (long long)D,
                  (long long)F, reverse ? "reverse" : "forward", (long long)pl.workspace_bytes);
        return FTC_OK;
    }
    if (pl.workspace_bytes > 0 && (!workspace || workspace_bytes < (size_t)pl.workspace_bytes))
        return fail(FTC_ERR_WORKSPACE, "workspace of %lld bytes needed, %zu given",
                    (long long)pl.workspace_bytes, workspace_bytes);
    const int64_t chains = N * H;
    const int64_t wgs = chains * pl.nseg * pl.nslice;
    if (wgs > 0x7fffffffLL) return fail(FTC_ERR_UNSUPPORTED, "too many workgroups");

    GenericArgs args;
    args.a = a;
    args.b = b;
    args.v = v;
    args.out = out;
    args.states =
        pl.nseg > 1 ? (float *)((char *)workspace + FTC_WORKSPACE_CONTROL_BYTES) : nullptr;
    args.L = L;
    args.H = (int32_t)H;
    args.D = (int32_t)D;
    args.F = (int32_t)F;
    args.seg_len = pl.seg_len;
    args.nseg = pl.nseg;
    args.nslice = pl.nslice;
    args.reverse = reverse ? 1 : 0;
    args.initial = initial;
    args.final_ = final_;

    if (pl.nseg > 1) {
        args.state_only = 1;
        launch_by_width(args, wgs, stream);
        const int64_t elems = D * F;
        const int64_t scan_wgs = (elems + kThreads - 1) / kThreads * chains;
        if (scan_wgs > 0x7fffffffLL) return fail(FTC_ERR_UNSUPPORTED, "too many workgroups");
        hipLaunchKernelGGL(generic_state_scan_kernel, dim3((unsigned)scan_wgs), dim3(kThreads), 0,
                           stream, args.states, pl.nseg, elems, args.reverse, initial, (int)H,
                           (int)F);
    }
    args.state_only = 0;
    launch_by_width(args, wgs, stream);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(FTC_ERR_HIP, "generic scan launch failed: %s", hipGetErrorString(err));
    return FTC_OK;
}

}  // namespace ftc
