// C ABI entry points (include/ftc_causal_product.h): argument checking and dispatch.
//
// The four result tensors are all instances of one scan primitive under a change of
// operand roles (the reference's CUDA path uses the same identity,
// causal_product_cuda.cu:1119-1187):
//
//   product = scan_fwd(a=Q, b=K, v=V)      state E x M
//   dQ      = scan_fwd(a=G, b=V, v=K)      state M x E
//   dK      = scan_rev(a=V, b=G, v=Q)      state M x E
//   dV      = scan_rev(a=K, b=Q, v=G)      state E x M
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <mutex>

#include "ftc_common.h"

// Scratch memory of ftc_causal_dot_product_static: one array per GPU, part of the loaded
// code object (zero when it is loaded).  Host code never uses this name as an address; it
// asks the runtime for the array's device address once per device (scratch_of_device).
static __device__ __align__(256) unsigned char scratch[FTC_STATIC_SCRATCH_BYTES];

namespace ftc {

static thread_local char g_error[512] = "";

static thread_local const char *g_kernel = "";
void note_kernel(const char *name) { g_kernel = name; }
static thread_local bool g_plan_only = false;
static thread_local char g_plan[16384] = "";
bool plan_only() { return g_plan_only; }

// ---- tuning aids from the environment, read once -------------------------------------------
static Tuning g_tuning;
static std::atomic<int> g_tuning_state{0};  // 0: not read, 1: being read, 2: ready
static void read_tuning(Tuning &t) {
    auto num = [](const char *name) -> int {
        const char *env = getenv(name);
        return env && *env ? atoi(env) : -1;
    };
    t.split = num("FTC_SPLIT"), t.pad = num("FTC_PAD"), t.wg = num("FTC_WG"), t.tp = num("FTC_TP");
    t.tp_segs = num("FTC_TP_SEGS"), t.tpx = num("FTC_TPX"), t.tpx_segs = num("FTC_TPX_SEGS");
    t.seg_chunks = num("FTC_SEG_CHUNKS"), t.group = num("FTC_GROUP"), t.dma = num("FTC_DMA");
    t.tph = num("FTC_TPH");
    const char *ratio = getenv("FTC_TP_RATIO");
    t.tp_ratio = ratio && *ratio ? atof(ratio) : -1.0;
    t.stamp_ptr = getenv("FTC_STAMP_PTR");
}
const Tuning &tuning() {
    if (g_tuning_state.load(std::memory_order_acquire) != 2) {
        int expected = 0;
        if (g_tuning_state.compare_exchange_strong(expected, 1)) {
            read_tuning(g_tuning);
            g_tuning.generation = 1;
            g_tuning_state.store(2, std::memory_order_release);
        } else {
            while (g_tuning_state.load(std::memory_order_acquire) != 2) {
            }
        }
    }
    return g_tuning;
}
void note_plan(const char *fmt, ...) {
    const size_t used = strlen(g_plan);
    if (used + 2 >= sizeof(g_plan)) return;
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_plan + used, sizeof(g_plan) - used - 1, fmt, ap);
    va_end(ap);
    strcat(g_plan, "\n");
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

namespace {

struct Dims {
    int64_t N, H, L, E, M;
};

int check_tensor(const ftc_tensor4 *t, const char *name, int64_t N, int64_t H, int64_t L,
                 int64_t X, int dtype_a, int dtype_b) {
    if (!t) return fail(FTC_ERR_INVALID, "%s is null", name);
    if (t->dtype != dtype_a && t->dtype != dtype_b)
        return fail(FTC_ERR_INVALID, "%s has dtype code %d, which this argument does not accept",
                    name, (int)t->dtype);
    if (t->size[0] != N || t->size[1] != H || t->size[2] != L || t->size[3] != X)
        return fail(FTC_ERR_INVALID, "%s has shape (%lld,%lld,%lld,%lld), expected (%lld,%lld,%lld,%lld)",
                    name, (long long)t->size[0], (long long)t->size[1], (long long)t->size[2],
                    (long long)t->size[3], (long long)N, (long long)H, (long long)L, (long long)X);
    if (N * H * L * X > 0) {
        if (!t->ptr) return fail(FTC_ERR_INVALID, "%s has a null data pointer", name);
        if (X > 1 && t->stride[3] != 1)
            return fail(FTC_ERR_INVALID, "%s must be contiguous in its last dimension (stride %lld)",
                        name, (long long)t->stride[3]);
    }
    return FTC_OK;
}

int read_dims(const ftc_tensor4 *q, const ftc_tensor4 *v, Dims *d) {
    if (!q || !v) return fail(FTC_ERR_INVALID, "queries or values is null");
    d->N = q->size[0];
    d->H = q->size[1];
    d->L = q->size[2];
    d->E = q->size[3];
    d->M = v->size[3];
    if (d->N < 0 || d->H < 0 || d->L < 0 || d->E < 0 || d->M < 0)
        return fail(FTC_ERR_INVALID, "negative size");
    if (q->dtype != FTC_F32 && q->dtype != FTC_BF16)
        return fail(FTC_ERR_INVALID, "queries dtype code %d is neither FTC_F32 nor FTC_BF16",
                    (int)q->dtype);
    if (d->L > 0x7fffffffLL || d->N * d->H > 0x7fffffffLL)
        return fail(FTC_ERR_UNSUPPORTED, "L and N*H must fit in 31 bits");
    return FTC_OK;
}

// ---- odd widths on the matrix cores: dense zero-padded copies --------------------------
//
// A scan whose rows are not 32, 64, 96 or 128 (a, b) and a multiple of 32 (v, out) values
// wide, or whose rows are misaligned or too far apart, is run on zero-padded dense copies
// of its operands when the workspace has room for them: padding columns of a and b add
// nothing to any dot product, padding columns of v produce output columns that are dropped
// when the result is copied back.  Two extra passes over the rows, but the matrix-core
// kernels are several times faster than the generic one.

// Rows of a strided operand of width w <-> rows of a dense buffer of width wp (a multiple of
// 32), chain after chain, Lp >= L dense rows per chain (more than L for a state whose rows
// are padded as well; those rows are not touched here).  A lane moves one 16-byte group of
// the dense row (T: uint32_t for fp32, uint16_t for bf16 elements); blockIdx.y walks the chains.
template <typename T, bool PAD>
__global__ __launch_bounds__(256) void pad_rows_kernel(T *strided, int64_t sn, int64_t sh, int64_t sl,
                                                       int64_t H, int64_t L, int64_t Lp, int64_t chains,
                                                       int w, int wp, T *dense) {
    constexpr int PER = 16 / sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(PER)));
    const uint32_t groups = (uint32_t)wp / PER;
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    if (j >= (uint32_t)L * groups) return;
    const uint32_t l = j / groups, c0 = (j % groups) * PER;
    for (int64_t chain = blockIdx.y; chain < chains; chain += gridDim.y) {
        T *row = strided + (chain / H) * sn + (chain % H) * sh + (int64_t)l * sl;
        Vec *slot = (Vec *)(dense + (chain * Lp + l) * wp + c0);
        if (PAD) {
            Vec x;
#pragma unroll
            for (int e = 0; e < PER; e++) x[e] = (int)(c0 + e) < w ? row[c0 + e] : (T)0;
            *slot = x;
        } else {
            const Vec x = *slot;
#pragma unroll
            for (int e = 0; e < PER; e++)
                if ((int)(c0 + e) < w) row[c0 + e] = x[e];
        }
    }
}

template <bool PAD>
void launch_pad_rows(void *strided, int64_t sn, int64_t sh, int64_t sl, int64_t N, int64_t H,
                     int64_t L, int w, int wp, int esz, void *dense, hipStream_t stream,
                     int64_t Lp = 0) {
    if (Lp == 0) Lp = L;
    const int per = 16 / esz;
    const dim3 grid((unsigned)((L * (wp / per) + 255) / 256), (unsigned)std::min<int64_t>(N * H, 65535));
    if (esz == 4)
        hipLaunchKernelGGL((pad_rows_kernel<uint32_t, PAD>), grid, dim3(256), 0, stream,
                           (uint32_t *)strided, sn, sh, sl, H, L, Lp, N * H, w, wp, (uint32_t *)dense);
    else
        hipLaunchKernelGGL((pad_rows_kernel<uint16_t, PAD>), grid, dim3(256), 0, stream,
                           (uint16_t *)strided, sn, sh, sl, H, L, Lp, N * H, w, wp, (uint16_t *)dense);
}

// The same between bf16 rows of the caller and fp32 dense rows (bf16 operands of a scan that
// only the fp32 kernels take: exact on the way in, rounded to nearest even on the way out).
template <bool PAD>
__global__ __launch_bounds__(256) void pad_rows_bf16_kernel(uint16_t *strided, int64_t sn, int64_t sh,
                                                            int64_t sl, int64_t H, int64_t L,
                                                            int64_t chains, int w, int wp, float *dense) {
    const uint32_t groups = (uint32_t)wp / 4;
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    if (j >= (uint32_t)L * groups) return;
    const uint32_t l = j / groups, c0 = (j % groups) * 4;
    for (int64_t chain = blockIdx.y; chain < chains; chain += gridDim.y) {
        uint16_t *row = strided + (chain / H) * sn + (chain % H) * sh + (int64_t)l * sl;
        float *slot = dense + (chain * L + l) * wp + c0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (PAD) slot[e] = (int)(c0 + e) < w ? bf16_to_f32(row[c0 + e]) : 0.f;
            else if ((int)(c0 + e) < w) row[c0 + e] = f32_to_bf16(slot[e]);
        }
    }
}
template <bool PAD>
void launch_pad_rows_bf16(void *strided, int64_t sn, int64_t sh, int64_t sl, int64_t N, int64_t H,
                          int64_t L, int w, int wp, void *dense, hipStream_t stream) {
    const dim3 grid((unsigned)((L * (wp / 4) + 255) / 256), (unsigned)std::min<int64_t>(N * H, 65535));
    hipLaunchKernelGGL((pad_rows_bf16_kernel<PAD>), grid, dim3(256), 0, stream, (uint16_t *)strided, sn,
                       sh, sl, H, L, N * H, w, wp, (float *)dense);
}

// (measured down to 512 rows: E = 25, M = 33, one chain of 512 positions, forward + backward
// 0.10 ms on the copies against 0.30 ms on the VALU kernel)
constexpr int64_t kPadMinRows = 512;
int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
__global__ void zero_words_kernel(uint32_t *p, uint32_t words);

// ---- states of 129 .. 512 rows: several scans over a split of the rows --------------------
//
// out_l = sum_d a[l, d] (sum_{j <= l} b[j, d] v[j, :]) is a sum over d: a scan whose a and b
// are wider than the 128 columns that the chain-parallel kernel takes is run as up to four
// scans, on columns 0 .. 127, 128 .. 255 and so on, all but the first one into a buffer in the
// workspace that is then added to the first one's rows (add_rows_kernel).  fp32 rows, widths
// multiples of 4.
bool split_widths(int64_t D, int64_t F) {
    if (tuning().split == 0) return false;  // tuning aid
    return D > 128 && D <= 512 && F >= 4 && F <= 512 && D % 4 == 0 && F % 4 == 0;
}

// rows of a strided fp32 tensor of width w (a multiple of 4, rows 16-byte aligned) += rows of a
// dense one, chain after chain; blockIdx.y walks the chains
__global__ __launch_bounds__(256) void add_rows_kernel(float *strided, int64_t sn, int64_t sh,
                                                       int64_t sl, int64_t H, int64_t L,
                                                       int64_t chains, int w, const float *dense) {
    typedef float Vec __attribute__((ext_vector_type(4)));
    const uint32_t groups = (uint32_t)w / 4;
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    if (j >= (uint32_t)L * groups) return;
    const uint32_t l = j / groups, c0 = (j % groups) * 4;
    for (int64_t chain = blockIdx.y; chain < chains; chain += gridDim.y) {
        Vec *row = (Vec *)(strided + (chain / H) * sn + (chain % H) * sh + (int64_t)l * sl + c0);
        *row += *(const Vec *)(dense + (chain * L + l) * w + c0);
    }
}

// the same for rows of any width and alignment, one value at a time
__global__ __launch_bounds__(256) void add_rows_any_kernel(float *strided, int64_t sn, int64_t sh,
                                                           int64_t sl, int64_t H, int64_t L,
                                                           int64_t chains, int w, const float *dense) {
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    if (j >= (uint32_t)L * (uint32_t)w) return;
    const uint32_t l = j / (uint32_t)w, c = j % (uint32_t)w;
    for (int64_t chain = blockIdx.y; chain < chains; chain += gridDim.y)
        strided[(chain / H) * sn + (chain % H) * sh + (int64_t)l * sl + c] += dense[(chain * L + l) * w + c];
}

// workspace of the launches of a split (the largest need among them) and of the buffers that
// take the later parts' results of up to kMfmaMaxScans scans
int64_t split_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                                   int64_t *launch_bytes) {
    int64_t ws = FTC_WORKSPACE_CONTROL_BYTES;
    for (int k = 1; k <= kMfmaMaxScans; k++) {
        ws = std::max(ws, mfma_tp_workspace_bytes(N, H, L, 128, F, k, true));
        if (D % 128) ws = std::max(ws, mfma_tp_workspace_bytes(N, H, L, D % 128, F, k, true));
    }
    ws = round_up(ws, 256);
    if (launch_bytes) *launch_bytes = ws;
    return ws + kMfmaMaxScans * round_up(N * H * L * F * 4, 256);
}

int run_scans(const ScanDesc *scans, int n, int64_t N, int64_t H, int64_t L, void *workspace,
              size_t workspace_bytes, hipStream_t stream, bool may_pad);

// Runs scans[0 .. n) of one shape (split_widths) as described above.  *done = false (nothing
// launched) when the chain-parallel kernel does not take the parts or the workspace has no room.
int split_scans(const ScanDesc *scans, int n, int64_t N, int64_t H, int64_t L, void *workspace,
                size_t workspace_bytes, hipStream_t stream, bool *done) {
    *done = false;
    const int D = scans[0].a.width, F = scans[0].v.width;
    const int64_t rows = N * H * L, tmp_bytes = round_up(rows * F * 4, 256);
    int64_t ws_launch = 0;
    split_scan_workspace_bytes(N, H, L, D, F, &ws_launch);
    const int64_t need = ws_launch + n * tmp_bytes;
    // part p: columns 128 p .. of a and b, rows 128 p .. of the states
    const int nparts = (D + 127) / 128;
    auto part = [&](int p, ScanDesc (&ps)[kMfmaMaxScans]) {
        const int w = std::min(128, D - 128 * p);
        for (int i = 0; i < n; i++) {
            ps[i] = scans[i];
            ps[i].a.width = ps[i].b.width = w;
            ps[i].a.ptr = (const char *)scans[i].a.ptr + 128 * p * 4;
            ps[i].b.ptr = (const char *)scans[i].b.ptr + 128 * p * 4;
            if (ps[i].initial.ptr) ps[i].initial.ptr += 128 * p * ps[i].initial.stride_d;
            if (ps[i].final_.ptr) ps[i].final_.ptr += 128 * p * ps[i].final_.stride_d;
            if (p > 0)
                ps[i].out = OperandOut{(char *)workspace + ws_launch + i * tmp_bytes, H * L * (int64_t)F,
                                       L * (int64_t)F, (int64_t)F, FTC_F32, (int32_t)F};
        }
    };
    ScanDesc ps[kMfmaMaxScans];
    for (int p = 0; p < nparts; p++) {
        part(p, ps);
        if (!mfma_tp_takes(ps, n, N, H, L, true)) return FTC_OK;
    }
    if (!plan_only() && (!workspace || (int64_t)workspace_bytes < need || (uintptr_t)workspace % 256 != 0))
        return FTC_OK;
    for (int p = 0; p < nparts; p++) {
        part(p, ps);
        const int rc = mfma_scan(ps, n, N, H, L, workspace, (size_t)ws_launch, stream, nullptr, true, true);
        if (rc) return rc;
        if (p == 0) continue;
        if (plan_only()) {
            note_plan("add_rows_kernel: %d result%s of part %d added to the first part's, workspace %lld bytes",
                      n, n == 1 ? "" : "s", p + 1, (long long)need);
            continue;
        }
        const dim3 grid((unsigned)((L * (F / 4) + 255) / 256), (unsigned)std::min<int64_t>(N * H, 65535));
        for (int i = 0; i < n; i++)
            hipLaunchKernelGGL(add_rows_kernel, grid, dim3(256), 0, stream, (float *)scans[i].out.ptr,
                               scans[i].out.stride_n, scans[i].out.stride_h, scans[i].out.stride_l, H, L,
                               N * H, F, (const float *)ps[i].out.ptr);
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) return fail(FTC_ERR_HIP, "add launch failed: %s", hipGetErrorString(err));
    }
    *done = true;
    return FTC_OK;
}
// padded widths of a D x F scan (0: the matrix-core kernels take no such state)
// (129 .. 512: for the split above; multiples of 32 like the output widths, so that a tensor
// that is state rows in one scan and output columns in another needs one copy)
int padded_rows(int64_t D) { return D <= 512 ? (int)round_up(D, 32) : 0; }
// whether the matrix-core kernels take a padded D x F state
bool padded_shape_ok(int64_t Dp, int64_t Fp) {
    int widths[kMfmaMaxSlices];
    return Fp <= 512 && (split_widths(Dp, Fp) || (Dp <= 128 && mfma_slice_widths(Dp, Fp, widths) > 0));
}

int64_t scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                             bool with_pad = true, bool bf16 = false);

// workspace of the padded route of one scan: the scan's own, then dense copies of all four
// operands (fp32 sizes: an upper bound)
// (`bf16`: rows of a state beyond 128 rows are copied whatever their widths, to convert them)
int64_t padded_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                                    bool bf16 = false) {
    const int64_t Dp = padded_rows(D), Fp = round_up(F, 32), rows = N * H * L;
    const bool copies = Dp != D || Fp != F || (bf16 && Dp > 128);
    if (Dp == 0 || !copies || rows < kPadMinRows || !padded_shape_ok(Dp, Fp)) return 0;
    return std::max<int64_t>(round_up(scan_workspace_bytes(N, H, L, Dp, Fp), 256),
                             FTC_WORKSPACE_CONTROL_BYTES) +
           2 * round_up(rows * Dp * 4, 256) + 2 * round_up(rows * Fp * 4, 256) +
           2 * round_up(N * H * Dp * Fp * 4, 256);  // (the states handed in and out)
}

int run_scans(const ScanDesc *scans, int n, int64_t N, int64_t H, int64_t L, void *workspace,
              size_t workspace_bytes, hipStream_t stream, bool may_pad);

// The scans of a call that the matrix-core kernels do not take as they are, run on padded
// copies: `take[i]` says which.  An operand that several scans read is copied once; an
// operand whose rows are fine where they lie is used in place.  Returns with *done = false
// (nothing launched) when the workspace has no room.
int padded_scans(const ScanDesc *scans, int n, const bool *take, int64_t N, int64_t H, int64_t L,
                 void *workspace, size_t workspace_bytes, hipStream_t stream, bool *done) {
    *done = false;
    const int64_t rows = N * H * L;
    auto esz = [](int dtype) { return dtype == FTC_F32 ? 4 : 2; };
    struct Copy {
        const void *ptr;  // the caller's tensor
        int64_t sn, sh, sl;
        int dtype, width, padded;
        bool is_output;
        char *dense;
        int dense_dtype;  // FTC_F32 for a bf16 tensor of a scan that only the fp32 kernels take
    };
    Copy copies[4 * kMfmaMaxScans];
    int ncopies = 0;
    ScanDesc work[kMfmaMaxScans];
    int nwork = 0;
    int64_t ws_scan = 0;
    auto copy_of = [&](const void *ptr, int64_t sn, int64_t sh, int64_t sl, int dtype, int width,
                       int padded, bool is_output, int dense_dtype) -> int {
        for (int i = 0; i < ncopies; i++)
            if (copies[i].ptr == ptr && copies[i].sn == sn && copies[i].sh == sh &&
                copies[i].sl == sl && copies[i].width == width && copies[i].padded == padded &&
                copies[i].dense_dtype == dense_dtype && !copies[i].is_output && !is_output)
                return i;
        copies[ncopies] = Copy{ptr, sn, sh, sl, dtype, width, padded, is_output, nullptr, dense_dtype};
        return ncopies++;
    };
    // the states handed in and out, padded the same way (rows and columns)
    struct StateCopy {
        StateRef ref;
        int D, F, Dp, Fp, scan;
        bool is_output;
        char *dense;
    };
    StateCopy states[2 * kMfmaMaxScans];
    int nstates = 0;
    int which[kMfmaMaxScans][4];
    for (int i = 0; i < n; i++) {
        if (!take[i]) continue;
        const ScanDesc &sc = scans[i];
        const int Dp = padded_rows(sc.a.width), Fp = (int)round_up(sc.v.width, 32);
        if (Dp != sc.a.width || Fp != sc.v.width) {
            if (sc.initial.ptr)
                states[nstates++] = StateCopy{sc.initial, sc.a.width, sc.v.width, Dp, Fp, nwork, false, nullptr};
            if (sc.final_.ptr)
                states[nstates++] = StateCopy{sc.final_, sc.a.width, sc.v.width, Dp, Fp, nwork, true, nullptr};
        }
        ws_scan = std::max(ws_scan, round_up(scan_workspace_bytes(N, H, L, Dp, Fp), 256));
        // states beyond 128 rows run on the fp32 kernels only: bf16 tensors of such a scan are
        // converted on the way
        const bool to_f32 = Dp > 128;
        const Operand *in[3] = {&sc.a, &sc.b, &sc.v};
        const int target[3] = {Dp, Dp, Fp};
        for (int k = 0; k < 3; k++) {
            const Operand &o = *in[k];
            const int dd = to_f32 ? FTC_F32 : o.dtype;
            which[nwork][k] = o.width == target[k] && dd == o.dtype &&
                                      mfma_operand_in_place(o.ptr, o.stride_n, o.stride_h, o.stride_l,
                                                            o.dtype, o.width, L)
                                  ? -1
                                  : copy_of(o.ptr, o.stride_n, o.stride_h, o.stride_l, o.dtype, o.width,
                                            target[k], false, dd);
        }
        const OperandOut &o = sc.out;
        const int dd = to_f32 ? FTC_F32 : o.dtype;
        which[nwork][3] = o.width == Fp && dd == o.dtype &&
                                  mfma_operand_in_place(o.ptr, o.stride_n, o.stride_h, o.stride_l, o.dtype,
                                                        o.width, L)
                              ? -1
                              : copy_of(o.ptr, o.stride_n, o.stride_h, o.stride_l, o.dtype, o.width, Fp, true, dd);
        work[nwork++] = sc;
    }
    // the copies never lie on the control block, which every call must leave zeroed
    ws_scan = std::max<int64_t>(ws_scan, FTC_WORKSPACE_CONTROL_BYTES);
    int64_t need = ws_scan;
    for (int i = 0; i < ncopies; i++) need += round_up(rows * copies[i].padded * esz(copies[i].dense_dtype), 256);
    for (int i = 0; i < nstates; i++) {
        if (N * H * states[i].Dp * states[i].Fp >= 0x7fffffffLL) return FTC_OK;  // (fill kernel: 32-bit count)
        need += round_up(N * H * states[i].Dp * states[i].Fp * 4, 256);
    }
    if (!plan_only() && (!workspace || (int64_t)workspace_bytes < need || (uintptr_t)workspace % 256 != 0))
        return FTC_OK;
    char *base = (char *)workspace + ws_scan;
    for (int i = 0; i < ncopies; i++) {
        copies[i].dense = base;
        base += round_up(rows * copies[i].padded * esz(copies[i].dense_dtype), 256);
    }
    for (int i = 0; i < nstates; i++) {
        StateCopy &st = states[i];
        st.dense = base;
        base += round_up(N * H * st.Dp * st.Fp * 4, 256);
        const StateRef dense_ref{(float *)st.dense, H * (int64_t)st.Dp * st.Fp, (int64_t)st.Dp * st.Fp,
                                 (int64_t)st.Fp};
        (st.is_output ? work[st.scan].final_ : work[st.scan].initial) = dense_ref;
    }
    for (int s = 0; s < nwork; s++) {
        Operand *in[3] = {&work[s].a, &work[s].b, &work[s].v};
        for (int k = 0; k < 3; k++)
            if (which[s][k] >= 0) {
                const Copy &c = copies[which[s][k]];
                const int64_t w = c.padded;
                *in[k] = Operand{c.dense, H * L * w, L * w, w, c.dense_dtype, (int32_t)w};
            }
        if (which[s][3] >= 0) {
            const Copy &c = copies[which[s][3]];
            const int64_t w = c.padded;
            work[s].out = OperandOut{c.dense, H * L * w, L * w, w, c.dense_dtype, (int32_t)w};
        }
    }
    int nin = 0, nout = 0;
    for (int i = 0; i < ncopies; i++) (copies[i].is_output ? nout : nin)++;
    if (plan_only()) {
        note_plan("pad_rows_kernel: %d operand%s copied into zero-padded rows, %d result%s copied "
                  "back, workspace %lld bytes", nin, nin == 1 ? "" : "s", nout, nout == 1 ? "" : "s",
                  (long long)need);
    } else {
        for (int i = 0; i < ncopies; i++) {
            if (copies[i].is_output) continue;
            if (copies[i].dense_dtype != copies[i].dtype)
                launch_pad_rows_bf16<true>((void *)copies[i].ptr, copies[i].sn, copies[i].sh, copies[i].sl,
                                           N, H, L, copies[i].width, copies[i].padded, copies[i].dense,
                                           stream);
            else
                launch_pad_rows<true>((void *)copies[i].ptr, copies[i].sn, copies[i].sh, copies[i].sl,
                                      N, H, L, copies[i].width, copies[i].padded,
                                      esz(copies[i].dtype), copies[i].dense, stream);
        }
        for (int i = 0; i < nstates; i++) {
            const StateCopy &st = states[i];
            if (st.is_output) continue;
            // zeros first (the rows beyond D are not written by the copy), then the D x F part
            hipLaunchKernelGGL(zero_words_kernel, dim3(256), dim3(256), 0, stream, (uint32_t *)st.dense,
                               (uint32_t)(N * H * st.Dp * st.Fp));
            launch_pad_rows<true>((void *)st.ref.ptr, st.ref.stride_n, st.ref.stride_h, st.ref.stride_d,
                                  N, H, st.D, st.F, st.Fp, 4, st.dense, stream, st.Dp);
        }
    }
    int rc = run_scans(work, nwork, N, H, L, workspace, (size_t)ws_scan, stream, false);
    if (rc) return rc;
    if (!plan_only()) {
        for (int i = 0; i < ncopies; i++) {
            if (!copies[i].is_output) continue;
            if (copies[i].dense_dtype != copies[i].dtype)
                launch_pad_rows_bf16<false>((void *)copies[i].ptr, copies[i].sn, copies[i].sh,
                                            copies[i].sl, N, H, L, copies[i].width, copies[i].padded,
                                            copies[i].dense, stream);
            else
                launch_pad_rows<false>((void *)copies[i].ptr, copies[i].sn, copies[i].sh, copies[i].sl,
                                       N, H, L, copies[i].width, copies[i].padded,
                                       esz(copies[i].dtype), copies[i].dense, stream);
        }
        for (int i = 0; i < nstates; i++) {
            const StateCopy &st = states[i];
            if (st.is_output)
                launch_pad_rows<false>((void *)st.ref.ptr, st.ref.stride_n, st.ref.stride_h,
                                       st.ref.stride_d, N, H, st.D, st.F, st.Fp, 4, st.dense, stream,
                                       st.Dp);
        }
        hipError_t err = hipGetLastError();
        if (err != hipSuccess)
            return fail(FTC_ERR_HIP, "padding launch failed: %s", hipGetErrorString(err));
    }
    *done = true;
    return FTC_OK;
}

// ---- rows of more than 512 values: column slices and row parts of at most 512 ---------------
//
// Output columns are independent of each other, and out_l = sum_d a[l, d] (...) is a sum over d:
// a scan whose v rows are wider than 512 is run slice by slice of the columns, one whose a and
// b rows are wider than 512 part by part of those columns, all parts but the first into a
// buffer in the workspace that is then added to the first one's rows.  Every piece is a scan
// of at most 512 x 512 and goes through run_scans like any other.  fp32 rows only.
constexpr int64_t kWidestRows = kGenericMaxDim;
bool wide_shape(int64_t D, int64_t F) { return D > kWidestRows || F > kWidestRows; }
// the pieces: equal widths (multiples of 4 of a and b, of 32 of v and out), the last one shorter
int64_t wide_part_width(int64_t W, int64_t multiple) {
    const int64_t parts = (W + kWidestRows - 1) / kWidestRows;
    return std::min<int64_t>(kWidestRows, round_up((W + parts - 1) / parts, multiple));
}
// workspace of a wide scan: that of its largest piece, then the buffer of the later row parts
int64_t wide_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                                  int64_t *piece_bytes) {
    const int64_t dw = wide_part_width(D, 4), fw = wide_part_width(F, 32);
    int64_t ws = FTC_WORKSPACE_CONTROL_BYTES;
    for (int64_t d : {dw, D % dw})
        for (int64_t f : {fw, F % fw})
            if (d > 0 && f > 0) ws = std::max(ws, scan_workspace_bytes(N, H, L, d, f));
    ws = round_up(ws, 256);
    if (piece_bytes) *piece_bytes = ws;
    return ws + (D > dw ? round_up(N * H * L * fw * 4, 256) : 0);
}

int wide_scan(const ScanDesc &scan, int64_t N, int64_t H, int64_t L, void *workspace,
              size_t workspace_bytes, hipStream_t stream) {
    const int64_t D = scan.a.width, F = scan.v.width;
    if (scan.a.dtype != FTC_F32 || scan.b.dtype != FTC_F32 || scan.v.dtype != FTC_F32 ||
        scan.out.dtype != FTC_F32)
        return fail(FTC_ERR_UNSUPPORTED, "rows of more than %d values must be fp32", (int)kWidestRows);
    const int64_t dw = wide_part_width(D, 4), fw = wide_part_width(F, 32);
    int64_t ws_piece = 0;
    const int64_t need = wide_scan_workspace_bytes(N, H, L, D, F, &ws_piece);
    if (!plan_only() && (!workspace || (int64_t)workspace_bytes < need || (uintptr_t)workspace % 256 != 0))
        return fail(FTC_ERR_WORKSPACE, "workspace of %lld bytes (256-byte aligned) needed, %zu given",
                    (long long)need, workspace_bytes);
    float *later = (float *)((char *)workspace + ws_piece);
    for (int64_t col = 0; col < F; col += fw) {
        const int64_t f = std::min(fw, F - col);
        for (int64_t row = 0; row < D; row += dw) {
            const int64_t d = std::min(dw, D - row);
            ScanDesc piece = scan;
            piece.a.ptr = (const float *)scan.a.ptr + row, piece.a.width = (int32_t)d;
            piece.b.ptr = (const float *)scan.b.ptr + row, piece.b.width = (int32_t)d;
            piece.v.ptr = (const float *)scan.v.ptr + col, piece.v.width = (int32_t)f;
            piece.out.ptr = (float *)scan.out.ptr + col, piece.out.width = (int32_t)f;
            if (piece.initial.ptr) piece.initial.ptr += row * piece.initial.stride_d + col;
            if (piece.final_.ptr) piece.final_.ptr += row * piece.final_.stride_d + col;
            if (row > 0) piece.out = OperandOut{later, H * L * f, L * f, f, FTC_F32, (int32_t)f};
            const int rc = run_scans(&piece, 1, N, H, L, workspace, (size_t)ws_piece, stream, true);
            if (rc) return rc;
            if (row == 0) continue;
            if (plan_only()) {
                note_plan("add_rows_kernel: rows %lld .. of the state, columns %lld ..: result added to "
                          "the first part's, workspace %lld bytes", (long long)row, (long long)col,
                          (long long)need);
                continue;
            }
            float *first = (float *)scan.out.ptr + col;
            const unsigned chains_y = (unsigned)std::min<int64_t>(N * H, 65535);
            const bool quads = f % 4 == 0 && (uintptr_t)first % 16 == 0 && scan.out.stride_n % 4 == 0 &&
                               scan.out.stride_h % 4 == 0 && scan.out.stride_l % 4 == 0;
            if (L * f >= 0x7fffffffLL) return fail(FTC_ERR_UNSUPPORTED, "L x M beyond 31 bits");
            if (quads)
                hipLaunchKernelGGL(add_rows_kernel, dim3((unsigned)((L * (f / 4) + 255) / 256), chains_y),
                                   dim3(256), 0, stream, first, scan.out.stride_n, scan.out.stride_h,
                                   scan.out.stride_l, H, L, N * H, (int)f, (const float *)later);
            else
                hipLaunchKernelGGL(add_rows_any_kernel, dim3((unsigned)((L * f + 255) / 256), chains_y),
                                   dim3(256), 0, stream, first, scan.out.stride_n, scan.out.stride_h,
                                   scan.out.stride_l, H, L, N * H, (int)f, (const float *)later);
            const hipError_t err = hipGetLastError();
            if (err != hipSuccess) return fail(FTC_ERR_HIP, "add launch failed: %s", hipGetErrorString(err));
        }
    }
    return FTC_OK;
}

// whether a scan that the matrix-core kernels do not take as it is may go the padded way
bool pad_eligible(const ScanDesc &sc, int64_t rows) {
    const int Dp = padded_rows(sc.a.width);
    if (Dp == 0 || rows < kPadMinRows) return false;
    if (tuning().pad == 0) return false;  // tuning aid
    return padded_shape_ok(Dp, round_up(sc.v.width, 32));
}

// Runs a list of independent scans.  A scan whose shape the MFMA kernels cover is cut into
// column slices; consecutive slices (of any of the scans) that share widths and element
// types go out in one launch.  Everything else takes the generic path.
int run_scans(const ScanDesc *scans, int n, int64_t N, int64_t H, int64_t L, void *workspace,
              size_t workspace_bytes, hipStream_t stream, bool may_pad = true) {
    // which scans the matrix-core kernels take as they are
    bool native[kMfmaMaxScans], padded[kMfmaMaxScans], taken[kMfmaMaxScans] = {};
    bool any_padded = false;
    if (n > kMfmaMaxScans) return fail(FTC_ERR_INVALID, "too many scans");
    // The scans of one shape go to the chain-parallel kernel together where it takes them
    // (whole scans: a column slice made below is never offered to it).
    bool offered[kMfmaMaxScans] = {};
    for (int i = 0; i < n; i++) {
        if (!wide_shape(scans[i].a.width, scans[i].v.width)) continue;
        const int rc = wide_scan(scans[i], N, H, L, workspace, workspace_bytes, stream);
        if (rc) return rc;
        offered[i] = taken[i] = true;
    }
    for (int i = 0; i < n; i++) {
        if (offered[i]) continue;
        ScanDesc group[kMfmaMaxScans];
        int members[kMfmaMaxScans], ngroup = 0;
        for (int j = i; j < n; j++)
            if (!offered[j] && scans[j].a.width == scans[i].a.width && scans[j].v.width == scans[i].v.width)
                offered[j] = true, members[ngroup] = j, group[ngroup++] = scans[j];
        if (split_widths(group[0].a.width, group[0].v.width)) {
            bool done = false;
            const int rc = split_scans(group, ngroup, N, H, L, workspace, workspace_bytes, stream, &done);
            if (rc) return rc;
            for (int k = 0; k < ngroup && done; k++) taken[members[k]] = true;
            continue;
        }
        if (!mfma_tp_takes(group, ngroup, N, H, L)) continue;
        const int rc = mfma_scan(group, ngroup, N, H, L, workspace, workspace_bytes, stream);
        if (rc) return rc;
        for (int k = 0; k < ngroup; k++) taken[members[k]] = true;
    }
    for (int i = 0; i < n; i++) {
        native[i] = padded[i] = false;
        if (taken[i]) continue;
        int widths[kMfmaMaxSlices];
        int nslices = mfma_slice_widths(scans[i].a.width, scans[i].v.width, widths);
        for (int j = 0, col = 0; j < nslices; col += widths[j], j++)
            if (!mfma_scan_supported(mfma_slice(scans[i], col, widths[j]), L)) nslices = 0;
        native[i] = nslices > 0;
        padded[i] = !native[i] && may_pad && pad_eligible(scans[i], N * H * L);
        any_padded = any_padded || padded[i];
    }
    if (any_padded) {
        bool done = false;
        const int rc = padded_scans(scans, n, padded, N, H, L, workspace, workspace_bytes, stream, &done);
        if (rc) return rc;
        if (!done)
            for (int i = 0; i < n; i++) padded[i] = false;
    }
    ScanDesc batch[kMfmaMaxScans];
    int nbatch = 0;
    auto flush = [&]() -> int {
        if (nbatch == 0) return FTC_OK;
        const int rc = mfma_scan(batch, nbatch, N, H, L, workspace, workspace_bytes, stream, nullptr,
                                 false);
        nbatch = 0;
        return rc;
    };
    for (int i = 0; i < n; i++) {
        if (padded[i] || taken[i]) continue;
        if (!native[i]) {
            int rc = flush();
            if (rc) return rc;
            rc = generic_scan(scans[i].a, scans[i].b, scans[i].v, scans[i].out, N, H, L,
                              scans[i].reverse, scans[i].initial, scans[i].final_, workspace,
                              workspace_bytes, stream);
            if (rc) return rc;
            continue;
        }
        int widths[kMfmaMaxSlices];
        const int nslices = mfma_slice_widths(scans[i].a.width, scans[i].v.width, widths);
        for (int j = 0, col = 0; j < nslices; col += widths[j], j++) {
            const ScanDesc slice = mfma_slice(scans[i], col, widths[j]);
            if (nbatch == kMfmaMaxScans || (nbatch > 0 && !mfma_scan_same_launch(batch[0], slice))) {
                const int rc = flush();
                if (rc) return rc;
            }
            batch[nbatch++] = slice;
        }
    }
    return flush();
}

// Upper bound over every way run_scans may slice and group scans of these widths.
// `with_pad` = false leaves out the padded copies and the buffers of split scans: what a call
// needs at the least (without them such a scan runs on the generic kernel).
int64_t scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F, bool with_pad,
                             bool bf16) {
    if (wide_shape(D, F)) return wide_scan_workspace_bytes(N, H, L, D, F, nullptr);
    int64_t need = generic_scan_workspace_bytes(N, H, L, D, F);
    int widths[kMfmaMaxSlices];
    const int nslices = mfma_slice_widths(D, F, widths);
    for (int j = 0; j < nslices; j++)
        for (int k = 1; k <= kMfmaMaxScans; k++)
            need = std::max(need, mfma_scan_workspace_bytes(N, H, L, D, widths[j], k));
    if (nslices == 0 && with_pad)
        need = std::max(need, padded_scan_workspace_bytes(N, H, L, D, F, bf16));
    for (int k = 1; k <= kMfmaMaxScans; k++)
        need = std::max(need, mfma_tp_workspace_bytes(N, H, L, D, F, k));
    if (with_pad && split_widths(D, F))
        need = std::max(need, split_scan_workspace_bytes(N, H, L, D, F, nullptr));
    return need;
}

// Zeroes `words` 32-bit words (a fill kernel, so that a caller may capture the call in a
// HIP graph, where memset nodes are best avoided).
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t *p, uint32_t words) {
    for (uint32_t i = blockIdx.x * 256u + threadIdx.x; i < words; i += gridDim.x * 256u) p[i] = 0u;
}

// Device address of `scratch` on the current device, looked up on the first call per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];

int scratch_of_device(void **ptr) {
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) return fail(FTC_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(err));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(FTC_ERR_UNSUPPORTED, "device ordinal %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !p)
            return fail(FTC_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev,
                        hipGetErrorString(err));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return FTC_OK;
}

}  // namespace
}  // namespace ftc

using namespace ftc;

extern "C" {

int ftc_version(void) { return 1000; }

int ftc_tuning_reload(void) {
    tuning();  // (makes sure the first read is over)
    Tuning t;
    read_tuning(t);
    t.generation = g_tuning.generation + 1;
    g_tuning = t;
    return FTC_OK;
}

const char *ftc_last_error(void) { return g_error; }

const char *ftc_last_kernel(void) { return g_kernel; }

int64_t ftc_causal_dot_product_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t E,
                                               int64_t M, int32_t dtype) {
    if (N < 0 || H < 0 || L < 0 || E < 0 || M < 0) return fail(FTC_ERR_INVALID, "negative size");
    if (dtype != FTC_F32 && dtype != FTC_BF16) return fail(FTC_ERR_INVALID, "unknown dtype");
    if (N * H * L == 0 || M == 0 || E == 0) return 0;
    if ((E > kGenericMaxDim || M > kGenericMaxDim) && dtype != FTC_F32)
        return fail(FTC_ERR_UNSUPPORTED, "rows of more than %d values must be fp32", kGenericMaxDim);
    return scan_workspace_bytes(N, H, L, E, M, true, dtype == FTC_BF16);
}

int ftc_causal_dot_product(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                           const ftc_tensor4 *values, const ftc_tensor4 *product,
                           void *workspace, size_t workspace_bytes, void *stream) {
    Dims d;
    int rc = read_dims(queries, values, &d);
    if (rc) return rc;
    const int dt = queries->dtype;
    if ((rc = check_tensor(queries, "queries", d.N, d.H, d.L, d.E, dt, dt))) return rc;
    if ((rc = check_tensor(keys, "keys", d.N, d.H, d.L, d.E, dt, dt))) return rc;
    if ((rc = check_tensor(values, "values", d.N, d.H, d.L, d.M, dt, dt))) return rc;
    if ((rc = check_tensor(product, "product", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if (d.N * d.H * d.L * d.M == 0) return FTC_OK;
    hipStream_t s = (hipStream_t)stream;
    if (d.E == 0)  // an empty contraction: every product row is zero
        return zero_rows(as_operand_out(product), d.N, d.H, d.L, s);
    const ScanDesc fwd = {as_operand(queries), as_operand(keys), as_operand(values),
                          as_operand_out(product), false};
    return run_scans(&fwd, 1, d.N, d.H, d.L, workspace, workspace_bytes, s);
}

int ftc_workspace_reset(void *workspace, size_t workspace_bytes, void *stream) {
    if (!workspace || workspace_bytes < (size_t)FTC_WORKSPACE_CONTROL_BYTES)
        return fail(FTC_ERR_WORKSPACE, "a workspace has at least %d bytes",
                    (int)FTC_WORKSPACE_CONTROL_BYTES);
    hipLaunchKernelGGL(zero_words_kernel, dim3(16), dim3(256), 0, (hipStream_t)stream,
                       (uint32_t *)workspace, (uint32_t)(FTC_WORKSPACE_CONTROL_BYTES / 4));
    const hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(FTC_ERR_HIP, "workspace reset launch failed: %s", hipGetErrorString(err));
    return FTC_OK;
}

int ftc_causal_dot_product_static(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                  const ftc_tensor4 *values, const ftc_tensor4 *product,
                                  void *stream) {
    Dims d;
    int rc = read_dims(queries, values, &d);
    if (rc) return rc;
    int64_t need = 0;
    if (d.N * d.H * d.L * d.M > 0 && d.E > 0) {
        need = ftc_causal_dot_product_workspace_bytes(d.N, d.H, d.L, d.E, d.M, queries->dtype);
        if (need < 0) return (int)need;
        // widths that would run on padded copies do without them when the array has no room
        if (need > (int64_t)FTC_STATIC_SCRATCH_BYTES)
            need = scan_workspace_bytes(d.N, d.H, d.L, d.E, d.M, false);
    }
    if (need > (int64_t)FTC_STATIC_SCRATCH_BYTES)
        return fail(FTC_ERR_WORKSPACE,
                    "ftc_causal_dot_product_static: these sizes need %lld bytes of scratch, the "
                    "built-in array holds %lld; use ftc_causal_dot_product with a workspace",
                    (long long)need, (long long)FTC_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (need > 0) {
        if ((rc = scratch_of_device(&ws))) return rc;
        // The array keeps what the last call left.  The states behind the control block are
        // written before they are read; the control block must start at zero, and although
        // every completed call leaves it so, it is cleared here as well so that a call that
        // was cut short cannot spoil the next one.
        hipLaunchKernelGGL(zero_words_kernel, dim3(16), dim3(256), 0, (hipStream_t)stream,
                           (uint32_t *)ws, (uint32_t)(FTC_WORKSPACE_CONTROL_BYTES / 4));
    }
    return ftc_causal_dot_product(queries, keys, values, product, ws, (size_t)need, stream);
}

int ftc_causal_dot_product_state(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                 const ftc_tensor4 *values, const ftc_tensor4 *initial_state,
                                 const ftc_tensor4 *product, const ftc_tensor4 *final_state,
                                 void *workspace, size_t workspace_bytes, void *stream) {
    Dims d;
    int rc = read_dims(queries, values, &d);
    if (rc) return rc;
    const int dt = queries->dtype;
    if ((rc = check_tensor(queries, "queries", d.N, d.H, d.L, d.E, dt, dt))) return rc;
    if ((rc = check_tensor(keys, "keys", d.N, d.H, d.L, d.E, dt, dt))) return rc;
    if ((rc = check_tensor(values, "values", d.N, d.H, d.L, d.M, dt, dt))) return rc;
    if ((rc = check_tensor(product, "product", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if (initial_state && (rc = check_tensor(initial_state, "initial_state", d.N, d.H, d.E, d.M,
                                            FTC_F32, FTC_F32)))
        return rc;
    if (final_state &&
        (rc = check_tensor(final_state, "final_state", d.N, d.H, d.E, d.M, FTC_F32, FTC_F32)))
        return rc;
    hipStream_t s = (hipStream_t)stream;
    auto state_ref = [](const ftc_tensor4 *t) {
        StateRef r = {nullptr, 0, 0, 0};
        if (t) r = StateRef{(float *)t->ptr, t->stride[0], t->stride[1], t->stride[2]};
        return r;
    };
    if (d.N * d.H * d.L * d.M == 0 || d.E == 0) {
        // no position adds to a state; a state of E x M values with nothing to go through
        // is not handed over
        if (final_state && d.N * d.H * d.E * d.M > 0)
            return fail(FTC_ERR_UNSUPPORTED, "a state hand-over needs at least one position");
        if (d.N * d.H * d.L * d.M > 0) return zero_rows(as_operand_out(product), d.N, d.H, d.L, s);
        return FTC_OK;
    }
    ScanDesc fwd = {as_operand(queries), as_operand(keys), as_operand(values),
                    as_operand_out(product), false, state_ref(initial_state),
                    state_ref(final_state)};
    return run_scans(&fwd, 1, d.N, d.H, d.L, workspace, workspace_bytes, s);
}

int64_t ftc_causal_dot_backward_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t E,
                                                int64_t M, int32_t dtype) {
    if (N < 0 || H < 0 || L < 0 || E < 0 || M < 0) return fail(FTC_ERR_INVALID, "negative size");
    if (dtype != FTC_F32 && dtype != FTC_BF16) return fail(FTC_ERR_INVALID, "unknown dtype");
    if (N * H * L == 0 || M == 0 || E == 0) return 0;
    if ((E > kGenericMaxDim || M > kGenericMaxDim) && dtype != FTC_F32)
        return fail(FTC_ERR_UNSUPPORTED, "rows of more than %d values must be fp32", kGenericMaxDim);
    const bool bf16 = dtype == FTC_BF16;
    int64_t need = std::max(scan_workspace_bytes(N, H, L, E, M, true, bf16),
                            scan_workspace_bytes(N, H, L, M, E, true, bf16));
    // the padded route of the three scans together: Q, K, dQ, dK and V, G, dV as dense rows
    if (padded_scan_workspace_bytes(N, H, L, E, M, bf16) > 0 ||
        padded_scan_workspace_bytes(N, H, L, M, E, bf16) > 0) {
        int64_t ws = 0;
        if (padded_rows(E)) ws = std::max(ws, scan_workspace_bytes(N, H, L, padded_rows(E), round_up(M, 32)));
        if (padded_rows(M)) ws = std::max(ws, scan_workspace_bytes(N, H, L, padded_rows(M), round_up(E, 32)));
        int64_t copies = 4 * round_up(N * H * L * round_up(E, 32) * 4, 256) +
                         3 * round_up(N * H * L * round_up(M, 32) * 4, 256);
        // bf16 rows whose two state shapes lie on either side of 128 rows: the scans of the
        // wide one run on fp32 copies, the others on bf16 ones, so the tensors that both
        // read (queries and keys, at most the values as well) are copied once for each
        if (bf16)
            copies += 2 * round_up(N * H * L * round_up(E, 32) * 2, 256) +
                      round_up(N * H * L * round_up(M, 32) * 2, 256);
        need = std::max(need, std::max<int64_t>(round_up(ws, 256), FTC_WORKSPACE_CONTROL_BYTES) + copies);
    }
    return need;
}

int ftc_causal_dot_backward(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                            const ftc_tensor4 *values, const ftc_tensor4 *grad_out,
                            const ftc_tensor4 *grad_queries, const ftc_tensor4 *grad_keys,
                            const ftc_tensor4 *grad_values, void *workspace,
                            size_t workspace_bytes, void *stream) {
    Dims d;
    int rc = read_dims(queries, values, &d);
    if (rc) return rc;
    const int dt = queries->dtype;
    if ((rc = check_tensor(queries, "queries", d.N, d.H, d.L, d.E, dt, dt))) return rc;
    if ((rc = check_tensor(keys, "keys", d.N, d.H, d.L, d.E, dt, dt))) return rc;
    if ((rc = check_tensor(values, "values", d.N, d.H, d.L, d.M, dt, dt))) return rc;
    if ((rc = check_tensor(grad_out, "grad_out", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    // a gradient that is not wanted may be passed as NULL
    if (grad_queries &&
        (rc = check_tensor(grad_queries, "grad_queries", d.N, d.H, d.L, d.E, dt, dt)))
        return rc;
    if (grad_keys && (rc = check_tensor(grad_keys, "grad_keys", d.N, d.H, d.L, d.E, dt, dt)))
        return rc;
    if (grad_values && (rc = check_tensor(grad_values, "grad_values", d.N, d.H, d.L, d.M, dt, dt)))
        return rc;
    if (d.N * d.H * d.L == 0 || d.E == 0 || d.M == 0) {
        // A zero row width: whichever gradient is non-empty is a sum over an empty index set.
        const ftc_tensor4 *outs[3] = {grad_queries, grad_keys, grad_values};
        for (const ftc_tensor4 *t : outs) {
            if (!t) continue;
            if (t->size[0] * t->size[1] * t->size[2] * t->size[3] == 0) continue;
            if ((rc = zero_rows(as_operand_out(t), d.N, d.H, d.L, (hipStream_t)stream))) return rc;
        }
        return FTC_OK;
    }
    hipStream_t s = (hipStream_t)stream;
    const Operand Q = as_operand(queries), K = as_operand(keys), V = as_operand(values),
                  G = as_operand(grad_out);
    ScanDesc scans[3];
    int n = 0;
    if (grad_queries)  // dQ: state M x E, walks up
        scans[n++] = ScanDesc{G, V, K, as_operand_out(grad_queries), false};
    if (grad_keys)  // dK: state M x E, walks down
        scans[n++] = ScanDesc{V, G, Q, as_operand_out(grad_keys), true};
    if (grad_values)  // dV: state E x M, walks down
        scans[n++] = ScanDesc{K, Q, G, as_operand_out(grad_values), true};
    return run_scans(scans, n, d.N, d.H, d.L, workspace, workspace_bytes, s);
}

int ftc_causal_dot_plan(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                        const ftc_tensor4 *values, int backward, char *text, size_t text_bytes) {
    if (!queries || !keys || !values || !text || text_bytes == 0)
        return fail(FTC_ERR_INVALID, "null argument");
    // data pointers are never read here: absent ones are replaced by a placeholder so that
    // the checks of the real entry points apply unchanged
    uintptr_t placeholder = 0;  // (distinct ones: tensors are told apart by their pointers)
    auto with_ptr = [&](ftc_tensor4 t) {
        placeholder += 4096;
        if (!t.ptr) t.ptr = (void *)placeholder;
        return t;
    };
    const ftc_tensor4 q = with_ptr(*queries), k = with_ptr(*keys), v = with_ptr(*values);
    auto dense = [&](int64_t width, int dtype) {
        ftc_tensor4 t;
        placeholder += 4096;
        t.ptr = (void *)placeholder;
        t.dtype = dtype;
        t.size[0] = q.size[0], t.size[1] = q.size[1], t.size[2] = q.size[2], t.size[3] = width;
        t.stride[3] = 1, t.stride[2] = width, t.stride[1] = t.stride[2] * t.size[2];
        t.stride[0] = t.stride[1] * t.size[1];
        return t;
    };
    const ftc_tensor4 out = dense(v.size[3], FTC_F32);
    g_plan[0] = 0;
    g_plan_only = true;
    int rc;
    if (!backward) {
        rc = ftc_causal_dot_product(&q, &k, &v, &out, nullptr, 0, nullptr);
    } else {
        const ftc_tensor4 gq = dense(q.size[3], q.dtype), gk = dense(k.size[3], k.dtype),
                          gv = dense(v.size[3], v.dtype);
        rc = ftc_causal_dot_backward(&q, &k, &v, &out, &gq, &gk, &gv, nullptr, 0, nullptr);
    }
    g_plan_only = false;
    snprintf(text, text_bytes, "%s", g_plan);
    return rc;
}

int64_t ftc_causal_linear_attention_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t E,
                                                    int64_t M, int32_t dtype) {
    if (N < 0 || H < 0 || L < 0 || E < 0 || M < 0) return fail(FTC_ERR_INVALID, "negative size");
    if (dtype != FTC_F32 && dtype != FTC_BF16) return fail(FTC_ERR_INVALID, "unknown dtype");
    if (dtype != FTC_F32 || !(E == 32 || E == 64) || !(M == 32 || M == 64))
        return fail(FTC_ERR_UNSUPPORTED,
                    "the fused attention kernel takes fp32 rows with E, M in {32, 64}");
    if (N * H * L == 0) return 0;
    return fused_attention_workspace_bytes(N, H, L, E, M);
}

static int check_denominators(const ftc_tensor4 *den, const Dims &d) {
    if (den->dtype != FTC_F32) return fail(FTC_ERR_INVALID, "denominators must be float32");
    if (den->size[0] != d.N || den->size[1] != d.H || den->size[2] != d.L || den->size[3] != 1)
        return fail(FTC_ERR_INVALID, "denominators must have shape (N, H, L, 1)");
    if (d.N * d.H * d.L > 0 && !den->ptr) return fail(FTC_ERR_INVALID, "denominators has a null data pointer");
    return FTC_OK;
}

int ftc_causal_linear_attention_forward(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                        const ftc_tensor4 *values, const int64_t *key_lengths,
                                        float eps, const ftc_tensor4 *out,
                                        const ftc_tensor4 *denominators, void *workspace,
                                        size_t workspace_bytes, void *stream) {
    Dims d;
    int rc = read_dims(queries, values, &d);
    if (rc) return rc;
    if ((rc = check_tensor(queries, "queries", d.N, d.H, d.L, d.E, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(keys, "keys", d.N, d.H, d.L, d.E, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(values, "values", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(out, "out", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if (denominators && (rc = check_denominators(denominators, d))) return rc;
    if (!(eps == eps)) return fail(FTC_ERR_INVALID, "eps is not a number");
    if (!(d.E == 32 || d.E == 64) || !(d.M == 32 || d.M == 64))
        return fail(FTC_ERR_UNSUPPORTED,
                    "the fused attention kernel takes fp32 rows with E, M in {32, 64}");
    if (d.N * d.H * d.L == 0) return FTC_OK;
    const ScanDesc fwd = {as_operand(queries), as_operand(keys), as_operand(values),
                          as_operand_out(out), false};
    if (!fused_attention_supported(fwd, d.L))
        return fail(FTC_ERR_UNSUPPORTED,
                    "the fused attention kernel needs 16-byte aligned rows that do not overlap");
    FusedAttention fused;
    fused.key_lengths = key_lengths, fused.eps = eps;
    if (denominators) {
        if (denominators->stride[2] != 1)
            return fail(FTC_ERR_INVALID, "denominators must be contiguous along L");
        fused.denominators = (float *)denominators->ptr;
        fused.den_sn = denominators->stride[0], fused.den_sh = denominators->stride[1];
    }
    return mfma_scan(&fwd, 1, d.N, d.H, d.L, workspace, workspace_bytes, (hipStream_t)stream,
                     &fused);
}

int ftc_causal_linear_attention(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                const ftc_tensor4 *values, const int64_t *key_lengths, float eps,
                                const ftc_tensor4 *out, void *workspace, size_t workspace_bytes,
                                void *stream) {
    return ftc_causal_linear_attention_forward(queries, keys, values, key_lengths, eps, out, nullptr,
                                               workspace, workspace_bytes, stream);
}

// workspace of the backward: [scans][Qf][Kf][gz][dd][segment sums]
static int64_t attention_backward_layout(int64_t N, int64_t H, int64_t L, int64_t E, int64_t M,
                                         int64_t (&offset)[6]) {
    const int64_t positions = N * H * L;
    int64_t at = std::max<int64_t>(
        round_up(std::max(scan_workspace_bytes(N, H, L, E, M, false), scan_workspace_bytes(N, H, L, M, E, false)), 256),
        FTC_WORKSPACE_CONTROL_BYTES);
    offset[0] = 0;
    offset[1] = at, at += round_up(positions * E * 4, 256);   // Qf
    offset[2] = at, at += round_up(positions * E * 4, 256);   // Kf
    offset[3] = at, at += round_up(positions * M * 4, 256);   // gz
    offset[4] = at, at += round_up(positions * 4, 256);       // dd
    offset[5] = at, at += round_up(N * H * attention_backward_segments(L) * 2 * E * 4, 256);
    return at;
}

int64_t ftc_causal_linear_attention_backward_workspace_bytes(int64_t N, int64_t H, int64_t L,
                                                             int64_t E, int64_t M, int32_t dtype) {
    if (N < 0 || H < 0 || L < 0 || E < 0 || M < 0) return fail(FTC_ERR_INVALID, "negative size");
    if (dtype != FTC_F32 || !(E == 32 || E == 64) || !(M == 32 || M == 64))
        return fail(FTC_ERR_UNSUPPORTED,
                    "the fused attention backward takes fp32 rows with E, M in {32, 64}");
    if (N * H * L == 0) return 0;
    int64_t offset[6];
    return attention_backward_layout(N, H, L, E, M, offset);
}

int ftc_causal_linear_attention_backward(const ftc_tensor4 *queries, const ftc_tensor4 *keys,
                                         const ftc_tensor4 *values, const int64_t *key_lengths,
                                         const ftc_tensor4 *out, const ftc_tensor4 *denominators,
                                         const ftc_tensor4 *grad_out, const ftc_tensor4 *grad_queries,
                                         const ftc_tensor4 *grad_keys, const ftc_tensor4 *grad_values,
                                         void *workspace, size_t workspace_bytes, void *stream) {
    Dims d;
    int rc = read_dims(queries, values, &d);
    if (rc) return rc;
    if ((rc = check_tensor(queries, "queries", d.N, d.H, d.L, d.E, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(keys, "keys", d.N, d.H, d.L, d.E, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(values, "values", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(out, "out", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if ((rc = check_tensor(grad_out, "grad_out", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32))) return rc;
    if (!denominators) return fail(FTC_ERR_INVALID, "denominators is null");
    if ((rc = check_denominators(denominators, d))) return rc;
    if (grad_queries && (rc = check_tensor(grad_queries, "grad_queries", d.N, d.H, d.L, d.E, FTC_F32, FTC_F32)))
        return rc;
    if (grad_keys && (rc = check_tensor(grad_keys, "grad_keys", d.N, d.H, d.L, d.E, FTC_F32, FTC_F32)))
        return rc;
    if (grad_values && (rc = check_tensor(grad_values, "grad_values", d.N, d.H, d.L, d.M, FTC_F32, FTC_F32)))
        return rc;
    if (!(d.E == 32 || d.E == 64) || !(d.M == 32 || d.M == 64))
        return fail(FTC_ERR_UNSUPPORTED,
                    "the fused attention backward takes fp32 rows with E, M in {32, 64}");
    if (d.N * d.H * d.L == 0) return FTC_OK;
    for (const ftc_tensor4 *t : {queries, keys, values, out, grad_out, grad_queries, grad_keys})
        if (t && ((uintptr_t)t->ptr % 16 || t->stride[0] % 4 || t->stride[1] % 4 || t->stride[2] % 4))
            return fail(FTC_ERR_UNSUPPORTED, "the fused attention backward needs 16-byte aligned rows");
    int64_t offset[6];
    const int64_t need = attention_backward_layout(d.N, d.H, d.L, d.E, d.M, offset);
    if (!workspace || (int64_t)workspace_bytes < need || (uintptr_t)workspace % 256 != 0)
        return fail(FTC_ERR_WORKSPACE, "workspace of %lld bytes (256-byte aligned) needed, %zu given",
                    (long long)need, workspace_bytes);
    hipStream_t s = (hipStream_t)stream;
    char *base = (char *)workspace;
    float *Qf = (float *)(base + offset[1]), *Kf = (float *)(base + offset[2]);
    float *gz = (float *)(base + offset[3]), *dd = (float *)(base + offset[4]);
    float *sums = (float *)(base + offset[5]);
    Operand den{denominators->ptr, denominators->stride[0], denominators->stride[1],
                denominators->stride[2], FTC_F32, 1};
    launch_attention_backward_prep(as_operand(queries), as_operand(keys), as_operand(grad_out),
                                   as_operand(out), den, key_lengths, d.N, d.H, d.L, (int)d.E, (int)d.M,
                                   Qf, Kf, gz, dd, sums, s);
    // the plain backward's three scans on (Qf, Kf, v, gz)
    auto dense = [&](float *p, int64_t w) {
        return Operand{p, d.H * d.L * w, d.L * w, w, FTC_F32, (int32_t)w};
    };
    const Operand qf = dense(Qf, d.E), kf = dense(Kf, d.E), gzo = dense(gz, d.M), v = as_operand(values);
    ScanDesc scans[3];
    int n = 0;
    if (grad_queries) scans[n++] = ScanDesc{gzo, v, kf, as_operand_out(grad_queries), false};
    if (grad_keys) scans[n++] = ScanDesc{v, gzo, qf, as_operand_out(grad_keys), true};
    if (grad_values) scans[n++] = ScanDesc{kf, qf, gzo, as_operand_out(grad_values), true};
    if (n > 0 && (rc = run_scans(scans, n, d.N, d.H, d.L, workspace, (size_t)offset[1], s))) return rc;
    if (grad_queries || grad_keys) {
        const OperandOut none{nullptr, 0, 0, 0, FTC_F32, (int32_t)d.E};
        launch_attention_backward_finish(as_operand(queries), as_operand(keys), key_lengths, dd, sums,
                                         d.N, d.H, d.L, (int)d.E,
                                         grad_queries ? as_operand_out(grad_queries) : none,
                                         grad_keys ? as_operand_out(grad_keys) : none, s);
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return fail(FTC_ERR_HIP, "attention backward launch failed: %s", hipGetErrorString(err));
    note_kernel("attention backward: prep, three scans, prefix sums");
    return FTC_OK;
}

}  // extern "C"
