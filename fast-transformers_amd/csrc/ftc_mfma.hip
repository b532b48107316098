// MFMA causal scan for gfx950, fp32 rows, (D, F) in {(64,64), (32,128), (128,32)}.
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (REV: j >= l)
//
// One wavefront owns one (chain, L-segment) and walks it in chunks of 32 positions with
// the whole D x F state in its accumulator registers.  Per chunk (i, j index positions of
// the chunk; every product on v_mfma_f32_32x32x16_bf16, written in the transposed
// orientation so that chained operands are already in registers):
//
//   (1)  Pt[j][i]  = sum_d b[j][d] a[i][d]            then masked to j <= i (REV: j >= i)
//   (2a) Ot[f][i]  = sum_j vt[f][j] Pt[j][i]           Pt goes from accumulator to B operand
//   (2b) Ot[f][i] += sum_d S[d][f] a[i][d]             S goes from accumulator to A operand
//   (3)  S[d][f]  += sum_j b[j][d] v[j][f]
//
// fp32 fidelity on bf16 matrix cores: every fp32 value x is cut into three bf16 pieces
// hi + mid + lo == x exactly (three 8-bit slices of the 24-bit significand), and a product
// is the sum of the six piece products of order <= 2 (hi*hi, hi*mid, mid*hi, hi*lo, mid*mid,
// lo*hi), each exact in the fp32 accumulator.  What is dropped is below 2^-23 of the product,
// the size of one fp32 rounding.
//
// Register chaining: a 32x32 accumulator holds, in lane (col = lane % 32, g = lane / 32),
// rows 8*(r/4) + 4*g + (r%4) for r = 0..15.  Registers 8h..8h+7 are therefore 8 values
// of the contraction index for k-step h, provided the other operand uses the same order:
// k-slot (g, t) of a 16-wide k-step carries logical index 8*(t/4) + 4*g + (t%4).
//
// No LDS: every operand fragment is loaded from global memory directly in the register
// layout its MFMA wants.  Row-major fragments (a, and b for (1)) are two 16-byte loads per
// k-step; position-major fragments (b for (3), v) are 4-byte loads in which the 32 lanes
// of a half-wave read 32 consecutive floats of one row, so every load instruction still
// covers whole 128-byte lines.  b is read in both layouts; the second read hits L1/L2.
// (An earlier version transposed b and v through LDS: bank conflicts took 79 % of its LDS
// cycles and the write -> wait -> read round trip per chunk could not be hidden with the
// one wavefront per SIMD that the register budget allows.)
//
// One launch per scan.  A wavefront first sums its segment's own state (reading b and v
// only), publishes it, obtains the state that precedes its segment from the published
// sums of the segments before it (two levels, fixed order), and then replays its segment.
// The wavefronts launched for a chain take its segments in the order in which they start
// running, so a wavefront only ever waits for wavefronts that are already running; every
// wait is bounded and raises an error word instead of spinning forever.
//
// Rows are fetched with raw buffer loads whose descriptor ends at the segment's last row:
// positions outside the segment read as zero and stores to them are dropped, so tails need
// no branches.
#include <algorithm>
#include <cstdlib>

#include "ftc_common.h"

namespace ftc {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) float gfloat;
typedef __attribute__((address_space(1))) uint32_t gu32;

constexpr int kChunk = 32;
constexpr int kWave = 64;
constexpr uint32_t kRsrcFlags = 0x00020000u;  // raw buffer, 32-bit data format
constexpr int kSpinLimit = 1 << 20;           // bounded wait (about a second in total)

// The workspace starts with a control block of fixed size: a header and one flag word per
// wavefront.  It must be zero before the first use and every launch leaves it zero, so
// later calls of any shape can reuse it.  The state slots behind it need no initialisation.
constexpr int kHdrDone = 1, kHdrError = 2;
constexpr int kHdrWords = 64;
constexpr int kControlBytes = FTC_WORKSPACE_CONTROL_BYTES;
// words: [header][one flag per wavefront][one ticket counter per chain]
constexpr int kMaxWaves = ((kControlBytes / 4) - kHdrWords) / 2;
constexpr uint32_t kFlagEmpty = 0, kFlagSum = 1, kFlagTotal = 2;
constexpr int kCoherentAux = 16;  // sc1: the access is performed at agent scope

struct Frag {
    uint32_t w[4];  // 8 bf16, k-slot t in the low (t even) / high (t odd) half of w[t/2]
};

__device__ __forceinline__ f32x16 mfma(const Frag &a, const Frag &b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// (upper 16 bits of x1) : (upper 16 bits of x0)
__device__ __forceinline__ uint32_t pack_hi16(float x0, float x1) {
    return __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), 0x07060302u);
}
__device__ __forceinline__ float drop_hi_piece(float x) {
    return x - __uint_as_float(__float_as_uint(x) & 0xffff0000u);
}

// Cut two fp32 values into NS bf16 pieces each; out[p] packs piece p of (x0, x1).
template <int NS>
__device__ __forceinline__ void split_pair(float x0, float x1, uint32_t (&out)[NS]) {
#pragma unroll
    for (int p = 0; p < NS; p++) {
        out[p] = pack_hi16(x0, x1);
        if (p + 1 < NS) {
            x0 = drop_hi_piece(x0);
            x1 = drop_hi_piece(x1);
        }
    }
}

// Eight fp32 values (k-slots 0..7) -> NS fragments.
template <int NS>
__device__ __forceinline__ void split8(const float (&x)[8], Frag (&f)[NS]) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
        uint32_t o[NS];
        split_pair<NS>(x[2 * q], x[2 * q + 1], o);
#pragma unroll
        for (int p = 0; p < NS; p++) f[p].w[q] = o[p];
    }
}

// acc += A * B over the piece products of order <= NS - 1, smallest first.
template <int NS>
__device__ __forceinline__ f32x16 mfma_split(const Frag (&a)[NS], const Frag (&b)[NS], f32x16 acc) {
#pragma unroll
    for (int order = NS - 1; order >= 0; order--) {
#pragma unroll
        for (int pa = 0; pa <= order; pa++) acc = mfma(a[pa], b[order - pa], acc);
    }
    return acc;
}

__device__ __forceinline__ float4 buffer_load4(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset) {
    const u32x4 r = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0);
    return make_float4(__uint_as_float(r.x), __uint_as_float(r.y), __uint_as_float(r.z),
                       __uint_as_float(r.w));
}
__device__ __forceinline__ float buffer_load1(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 0));
}
__device__ __forceinline__ void buffer_store4(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset,
                                              float x, float y, float z, float w) {
    const u32x4 r = {__float_as_uint(x), __float_as_uint(y), __float_as_uint(z), __float_as_uint(w)};
    __builtin_amdgcn_raw_buffer_store_b128(r, rsrc, byte_offset, 0, 0);
}

// States travel between wavefronts (possibly on different XCDs, whose L2s are not coherent
// with each other) through buffer accesses flagged sc1, which are performed at agent scope
// themselves.  That keeps cache-wide write-back / invalidate operations out of the kernel:
// the writer only has to wait for its stores to be acknowledged before it raises the flag.
__device__ __forceinline__ void wait_for_stores() {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// One scan of a launch.  A launch runs up to kMaxScans independent scans of the same
// (D, F, N, H, L) side by side (the three gradients of a backward call), so that their
// launch gaps and wait times overlap.
struct ScanOperands {
    const float *a, *b, *v;
    float *out;
    int64_t a_sn, a_sh, a_sl;
    int64_t b_sn, b_sh, b_sl;
    int64_t v_sn, v_sh, v_sl;
    int64_t o_sn, o_sh, o_sl;
    int32_t rev;  // 0: j <= l, walk up; 1: j >= l, walk down
    int32_t pad;
};
constexpr int kMaxScans = 3;

struct ScanArgs {
    ScanOperands scan[kMaxScans];
    int64_t L;
    int32_t H, seg_len, nseg;
    int32_t waves_per_scan;
    int32_t total_waves;  // nscans * waves_per_scan
    int32_t group;        // steps per group of the two-level state sum
};

template <int D, int F, int NS>
__global__ __launch_bounds__(kWave) void scan_mfma_kernel(uint32_t *__restrict__ ws_ptr,
                                                          ScanArgs p) {
    constexpr int DT = D / 32, FT = F / 32;  // state tiles
    constexpr int KD = D / 16;               // k-steps over d
    constexpr int kStateElems = D * F;

    const int lane = threadIdx.x;
    const int ln = lane & 31, g = lane >> 5;

    gu32 *hdr = (gu32 *)ws_ptr;
    gu32 *flags = hdr + kHdrWords;
    gfloat *sums = (gfloat *)(hdr + kControlBytes / 4);

    // ---- which segment: the wavefronts launched for a chain take that chain's steps in
    // the order in which they start running, so a step only ever waits for steps that are
    // already running ----
    // chains of all scans are numbered consecutively: global chain = scan * chains + chain
    const uint32_t scan_id = blockIdx.x / (uint32_t)p.waves_per_scan;
    const ScanOperands &op = p.scan[scan_id];
    const bool REV = op.rev != 0;
    const float *a_ptr = op.a, *b_ptr = op.b, *v_ptr = op.v;
    float *out_ptr = op.out;
    uint32_t ticket = 0;
    if (p.nseg > 1) {
        const uint32_t my_chain = blockIdx.x / (uint32_t)p.nseg;
        uint32_t order = 0;
        if (lane == 0)
            order = __hip_atomic_fetch_add(flags + kMaxWaves + my_chain, 1u, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
        order = __builtin_amdgcn_readfirstlane(order);
        ticket = my_chain * (uint32_t)p.nseg + order;
        if (order >= (uint32_t)p.nseg) {
            // the control block was not zero when the launch started: refuse to run on it
            if (lane == 0)
                __hip_atomic_store(hdr + kHdrError, 2u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    } else {
        ticket = blockIdx.x;
    }
    const int64_t chain = (ticket - scan_id * (uint32_t)p.waves_per_scan) / (uint32_t)p.nseg;
    const int step = (int)(ticket % (uint32_t)p.nseg);      // position in dependency order
    const int seg = REV ? p.nseg - 1 - step : step;
    const int n = (int)(chain / p.H), h = (int)(chain % p.H);
    const int64_t lo = (int64_t)seg * p.seg_len;
    const int64_t hi = min(p.L, lo + (int64_t)p.seg_len);
    const int rows = (int)(hi - lo);
    const int nchunks = (rows + kChunk - 1) / kChunk;

    // descriptors based at the segment's first row and ending with its last row
    const float *a_seg = a_ptr + (int64_t)n * op.a_sn + (int64_t)h * op.a_sh + lo * op.a_sl;
    const float *b_seg = b_ptr + (int64_t)n * op.b_sn + (int64_t)h * op.b_sh + lo * op.b_sl;
    const float *v_seg = v_ptr + (int64_t)n * op.v_sn + (int64_t)h * op.v_sh + lo * op.v_sl;
    float *o_seg = out_ptr + (int64_t)n * op.o_sn + (int64_t)h * op.o_sh + lo * op.o_sl;
    const uint32_t a_sl4 = (uint32_t)op.a_sl * 4u, b_sl4 = (uint32_t)op.b_sl * 4u,
                   v_sl4 = (uint32_t)op.v_sl * 4u, o_sl4 = (uint32_t)op.o_sl * 4u;
    const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)a_seg, 0, (rows - 1) * a_sl4 + D * 4, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t b_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)b_seg, 0, (rows - 1) * b_sl4 + D * 4, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)v_seg, 0, (rows - 1) * v_sl4 + F * 4, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)o_seg, 0, (rows - 1) * o_sl4 + F * 4, kRsrcFlags);

    // per-lane byte offsets inside a chunk
    //  row-major fragments: lane (row = ln, g) reads 4 floats at column 16*ks + 4*g (+8)
    //  position-major fragments: lane (col = ln, g), k-slot t of k-step hh is row
    //  16*hh + 8*(t/4) + 4*g + (t%4)
    const uint32_t a_lane = ln * a_sl4 + 16u * g;
    const uint32_t b_lane = ln * b_sl4 + 16u * g;
    // position-major operands pass through LDS as fp32 rows: 16-byte global loads (lane =
    // (row within the load, 4 columns)), 16-byte LDS writes, 4-byte LDS reads by column
    constexpr int kBtLoads = D / 8, kVtLoads = F / 8;            // loads per 32-row tile
    constexpr int kBtRows = 64 / (D / 4), kVtRows = 64 / (F / 4);  // rows per load
    const uint32_t bt_lane = (uint32_t)(lane / (D / 4)) * b_sl4 + 16u * (lane % (D / 4));
    const uint32_t vt_lane = (uint32_t)(lane / (F / 4)) * v_sl4 + 16u * (lane % (F / 4));
    const uint32_t o_lane = ln * o_sl4 + 16u * g;

    // first row of chunk c relative to the segment (REV walks down from the end and its
    // last chunk may start before the segment: those rows read as zero)
    auto chunk_row0 = [&](int c) -> int { return REV ? rows - kChunk * (c + 1) : kChunk * c; };
    // pass 1 walks the chunks downwards; "chunk -1" must lie outside the descriptor
    auto pass1_row0 = [&](int c) -> int { return c < 0 ? -2 * kChunk : chunk_row0(c); };

    // raw fp32 of the chunk being fetched
    float4 a_raw[KD][2];   // a rows, B operand of (1) and (2b)
    float4 b_raw[KD][2];   // b rows, A operand of (1)
    float4 bt_raw[kBtLoads];  // b rows on their way to LDS (A operand of (3))
    float4 vt_raw[kVtLoads];  // v rows on their way to LDS (A operand of (2a), B of (3))
    __shared__ __align__(16) float bt_lds[2][kChunk * D];
    __shared__ __align__(16) float vt_lds[2][kChunk * F];

    auto fetch_rows = [&](__amdgpu_buffer_rsrc_t rs, uint32_t lane_off, uint32_t sl4, int row0,
                          float4 (&raw)[KD][2]) {
        const uint32_t off = lane_off + (uint32_t)row0 * sl4;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            raw[ks][0] = buffer_load4(rs, off + 64u * ks);
            raw[ks][1] = buffer_load4(rs, off + 64u * ks + 32u);
        }
    };
    auto fetch_bt_into = [&](int row0, float4 (&raw)[kBtLoads]) {
        const uint32_t off = bt_lane + (uint32_t)row0 * b_sl4;
#pragma unroll
        for (int i = 0; i < kBtLoads; i++)
            raw[i] = buffer_load4(b_rs, off + (uint32_t)(i * kBtRows) * b_sl4);
    };
    auto fetch_vt_into = [&](int row0, float4 (&raw)[kVtLoads]) {
        const uint32_t off = vt_lane + (uint32_t)row0 * v_sl4;
#pragma unroll
        for (int i = 0; i < kVtLoads; i++)
            raw[i] = buffer_load4(v_rs, off + (uint32_t)(i * kVtRows) * v_sl4);
    };
    // fetched rows -> LDS tile `buf` (row-major, 32 x width floats)
    auto stash_bt_from = [&](int buf, const float4 (&raw)[kBtLoads]) {
#pragma unroll
        for (int i = 0; i < kBtLoads; i++)
            *(float4 *)&bt_lds[buf][(i * kBtRows + lane / (D / 4)) * D + 4 * (lane % (D / 4))] =
                raw[i];
    };
    auto stash_vt_from = [&](int buf, const float4 (&raw)[kVtLoads]) {
#pragma unroll
        for (int i = 0; i < kVtLoads; i++)
            *(float4 *)&vt_lds[buf][(i * kVtRows + lane / (F / 4)) * F + 4 * (lane % (F / 4))] =
                raw[i];
    };
    auto fetch_bt = [&](int row0) { fetch_bt_into(row0, bt_raw); };
    auto fetch_vt = [&](int row0) { fetch_vt_into(row0, vt_raw); };
    auto stash_bt = [&](int buf) { stash_bt_from(buf, bt_raw); };
    auto stash_vt = [&](int buf) { stash_vt_from(buf, vt_raw); };
    // LDS tile -> the NS fragments of k-step hh for the 32 columns of tile `tile`:
    // lane (col = ln, g), k-slot t is row 16*hh + 8*(t/4) + 4*g + (t%4)
    auto frag_from_lds = [&](const float *tile_base, int width, int tile, int hh,
                             Frag (&frag)[NS]) {
        float x[8];
#pragma unroll
        for (int t = 0; t < 8; t++)
            x[t] = tile_base[(16 * hh + 8 * (t / 4) + 4 * g + (t % 4)) * width + 32 * tile + ln];
        split8<NS>(x, frag);
    };
    auto split_rows = [&](const float4 (&raw)[KD][2], Frag (&frag)[KD][NS]) {
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            const float x[8] = {raw[ks][0].x, raw[ks][0].y, raw[ks][0].z, raw[ks][0].w,
                                raw[ks][1].x, raw[ks][1].y, raw[ks][1].z, raw[ks][1].w};
            split8<NS>(x, frag[ks]);
        }
    };

    f32x16 S[DT][FT];
    // (3) S += b^T v
    auto update_state = [&](const Frag (&bt_frag)[DT][2][NS], const Frag (&v_frag)[FT][2][NS]) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
                    S[dt][ft] = mfma_split<NS>(bt_frag[dt][hh], v_frag[ft][hh], S[dt][ft]);
    };

#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int r = 0; r < 16; r++) S[dt][ft][r] = 0.f;

    if (p.nseg > 1) {
        // Segments of a chain form groups of p.group consecutive steps.  The state before
        // step s is (sum of the totals of the groups before its group) + (sum of the sums
        // of the steps before it in its group), always added in ascending order, so the
        // result does not depend on timing.  Every step but the last of its group publishes
        // its own sum; the last step of every group but the last publishes the group total.
        const int G = p.group;
        const int grp = step / G;
        const int grp_first = grp * G;
        const int grp_last = min(grp_first + G, p.nseg) - 1;
        const bool is_last_of_group = step == grp_last;
        const bool need_own_sum = step + 1 < p.nseg;  // the very last step has no reader
        const __amdgpu_buffer_rsrc_t st_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)sums, 0, (uint32_t)(2 * p.total_waves) * (uint32_t)(kStateElems * 4),
            kRsrcFlags);
        const uint32_t lane16 = 16u * lane;
        auto slot_offset = [&](uint32_t slot) -> uint32_t { return slot * (kStateElems * 4); };
        auto publish_state = [&](uint32_t slot, const f32x16 (&T)[DT][FT], uint32_t flag_value) {
            const uint32_t base = slot_offset(slot) + lane16;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        const u32x4 w = {__float_as_uint(T[dt][ft][4 * q4 + 0]),
                                         __float_as_uint(T[dt][ft][4 * q4 + 1]),
                                         __float_as_uint(T[dt][ft][4 * q4 + 2]),
                                         __float_as_uint(T[dt][ft][4 * q4 + 3])};
                        __builtin_amdgcn_raw_buffer_store_b128(
                            w, st_rs, base + (uint32_t)(((dt * FT + ft) * 4 + q4) * kWave * 16), 0,
                            kCoherentAux);
                    }
            wait_for_stores();
            if (lane == 0)
                __hip_atomic_store(flags + ticket, flag_value, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        };
        auto add_state = [&](uint32_t slot, f32x16 (&T)[DT][FT]) {
            const uint32_t base = slot_offset(slot) + lane16;
            // all loads of a state are in flight together, then added in a fixed order
            u32x4 w[DT * FT * 4];
#pragma unroll
            for (int i = 0; i < DT * FT * 4; i++)
                w[i] = __builtin_amdgcn_raw_buffer_load_b128(
                    st_rs, base + (uint32_t)(i * kWave * 16), 0, kCoherentAux);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        const u32x4 x = w[(dt * FT + ft) * 4 + q4];
                        T[dt][ft][4 * q4 + 0] += __uint_as_float(x.x);
                        T[dt][ft][4 * q4 + 1] += __uint_as_float(x.y);
                        T[dt][ft][4 * q4 + 2] += __uint_as_float(x.z);
                        T[dt][ft][4 * q4 + 3] += __uint_as_float(x.w);
                    }
        };
        int spins = 0;
        bool failed = false;
        // wait until `count` wavefronts, tickets first, first + stride, ..., show `bit`
        auto wait_flags = [&](uint32_t first, uint32_t stride, int count, uint32_t bit) {
            const bool mine = lane < count;
            const gu32 *f = flags + first + stride * (uint32_t)lane;
            while (!failed) {
                const uint32_t x =
                    mine ? __hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : bit;
                if (__builtin_amdgcn_ballot_w64((x & bit) == 0) == 0) break;
                if (++spins > kSpinLimit) failed = true;
                __builtin_amdgcn_s_sleep(4);
            }
        };

        // ---- pass 1: the segment's own state sum, walked against the direction of pass 2
        // so that pass 2 starts on the rows read last ----
        if (need_own_sum) {
            // rows are requested two chunks ahead (pass 1 has registers to spare and its
            // chunks are short compared with the memory latency)
            float4 bt_raw2[kBtLoads], vt_raw2[kVtLoads];
            auto sum_chunk = [&](int buf) {
                Frag bt_frag[DT][2][NS], v_frag[FT][2][NS];
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int hh = 0; hh < 2; hh++)
                        frag_from_lds(bt_lds[buf], D, dt, hh, bt_frag[dt][hh]);
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
#pragma unroll
                    for (int hh = 0; hh < 2; hh++)
                        frag_from_lds(vt_lds[buf], F, ft, hh, v_frag[ft][hh]);
                update_state(bt_frag, v_frag);
            };
            fetch_bt_into(pass1_row0(nchunks - 1), bt_raw);
            fetch_vt_into(pass1_row0(nchunks - 1), vt_raw);
            fetch_bt_into(pass1_row0(nchunks - 2), bt_raw2);
            fetch_vt_into(pass1_row0(nchunks - 2), vt_raw2);
            for (int c = nchunks - 1; c >= 0; c -= 2) {
                stash_bt_from(0, bt_raw);
                stash_vt_from(0, vt_raw);
                fetch_bt_into(pass1_row0(c - 2), bt_raw);
                fetch_vt_into(pass1_row0(c - 2), vt_raw);
                sum_chunk(0);
                if (c == 0) break;
                stash_bt_from(1, bt_raw2);
                stash_vt_from(1, vt_raw2);
                fetch_bt_into(pass1_row0(c - 3), bt_raw2);
                fetch_vt_into(pass1_row0(c - 3), vt_raw2);
                sum_chunk(1);
            }
            if (!is_last_of_group) publish_state(ticket, S, kFlagSum);
        }
        // start fetching the first chunk of pass 2 before waiting
        fetch_rows(a_rs, a_lane, a_sl4, chunk_row0(0), a_raw);
        fetch_rows(b_rs, b_lane, b_sl4, chunk_row0(0), b_raw);
        fetch_vt(chunk_row0(0));
        fetch_bt(chunk_row0(0));

        // ---- sums of the earlier steps of this group ----
        f32x16 X[DT][FT];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++)
#pragma unroll
                for (int r = 0; r < 16; r++) X[dt][ft][r] = 0.f;
        const int in_group = step - grp_first;
        const uint32_t chain_ticket0 = ticket - (uint32_t)step;
        if (in_group > 0) {
            wait_flags(chain_ticket0 + grp_first, 1, in_group, kFlagSum);
            if (!failed)
                for (int i = 0; i < in_group; i++) add_state(chain_ticket0 + grp_first + i, X);
        }
        if (is_last_of_group && need_own_sum && !failed) {
            // group total = sums of the group in ascending order (own sum last)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int ft = 0; ft < FT; ft++) S[dt][ft] = X[dt][ft] + S[dt][ft];
            publish_state((uint32_t)p.total_waves + ticket, S, kFlagTotal);
        }
        // ---- totals of the earlier groups, then the in-group part on top ----
        if (grp > 0 && !failed) {
            wait_flags(chain_ticket0 + (uint32_t)(G - 1), (uint32_t)G, grp, kFlagTotal);
            if (!failed) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int ft = 0; ft < FT; ft++) {
                        S[dt][ft] = X[dt][ft];
#pragma unroll
                        for (int r = 0; r < 16; r++) X[dt][ft][r] = 0.f;
                    }
                for (int gq = 0; gq < grp; gq++)
                    add_state((uint32_t)p.total_waves + chain_ticket0 + (uint32_t)(gq * G + G - 1),
                              X);
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int ft = 0; ft < FT; ft++) X[dt][ft] = X[dt][ft] + S[dt][ft];
            }
        }
        if (failed && lane == 0)
            __hip_atomic_store(hdr + kHdrError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++) S[dt][ft] = X[dt][ft];
    } else {
        fetch_rows(a_rs, a_lane, a_sl4, chunk_row0(0), a_raw);
        fetch_rows(b_rs, b_lane, b_sl4, chunk_row0(0), b_raw);
        fetch_vt(chunk_row0(0));
        fetch_bt(chunk_row0(0));
    }

    // ---- pass 2: outputs ----
    for (int c = 0; c < nchunks; c++) {
        const int row0 = chunk_row0(c);
        // rows of the chunk after the last one are outside the descriptor and read as zero,
        // so the prefetch needs no branch
        const int next0 = chunk_row0(c + 1);

        // each operand is cut into pieces as soon as it is needed and its raw registers
        // are refilled with the next chunk right away
        Frag a_frag[KD][NS], b_frag[KD][NS];
        split_rows(a_raw, a_frag);
        split_rows(b_raw, b_frag);
        fetch_rows(a_rs, a_lane, a_sl4, next0, a_raw);
        fetch_rows(b_rs, b_lane, b_sl4, next0, b_raw);

        // (1) Pt = b a^T
        f32x16 P;
#pragma unroll
        for (int r = 0; r < 16; r++) P[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) P = mfma_split<NS>(b_frag[ks], a_frag[ks], P);
        // causal mask inside the chunk: row j = 8*(r/4) + 4*g + r%4, column i = ln
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int j = 8 * (r / 4) + 4 * g + (r % 4);
            const bool keep = REV ? (j >= ln) : (j <= ln);
            P[r] = keep ? P[r] : 0.f;
        }
        Frag p_frag[2][NS];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            const float x[8] = {P[8 * hh + 0], P[8 * hh + 1], P[8 * hh + 2], P[8 * hh + 3],
                                P[8 * hh + 4], P[8 * hh + 5], P[8 * hh + 6], P[8 * hh + 7]};
            split8<NS>(x, p_frag[hh]);
        }

        // this chunk's position-major rows go to LDS, the next chunk's are requested
        const int buf = c & 1;
        stash_vt(buf);
        stash_bt(buf);
        fetch_vt(next0);
        fetch_bt(next0);
        Frag v_frag[FT][2][NS];  // A operand of (2a), B operand of (3)
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++) frag_from_lds(vt_lds[buf], F, ft, hh, v_frag[ft][hh]);

        // (2b) + (2a) per output tile, then store
        const uint32_t o_off = o_lane + (uint32_t)row0 * o_sl4;
#pragma unroll
        for (int ft = 0; ft < FT; ft++) {
            f32x16 O;
#pragma unroll
            for (int r = 0; r < 16; r++) O[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KD; ks++) {
                const int o8 = 8 * (ks % 2);
                const float x[8] = {S[ks / 2][ft][o8 + 0], S[ks / 2][ft][o8 + 1],
                                    S[ks / 2][ft][o8 + 2], S[ks / 2][ft][o8 + 3],
                                    S[ks / 2][ft][o8 + 4], S[ks / 2][ft][o8 + 5],
                                    S[ks / 2][ft][o8 + 6], S[ks / 2][ft][o8 + 7]};
                Frag s_frag[NS];
                split8<NS>(x, s_frag);
                O = mfma_split<NS>(s_frag, a_frag[ks], O);
            }
#pragma unroll
            for (int hh = 0; hh < 2; hh++) O = mfma_split<NS>(v_frag[ft][hh], p_frag[hh], O);
            // lane (i = ln, g) holds f = 32*ft + 8*q + 4*g + 0..3 in registers 4q..4q+3
#pragma unroll
            for (int q = 0; q < 4; q++)
                buffer_store4(o_rs, o_off + 128u * ft + 32u * q, O[4 * q + 0], O[4 * q + 1],
                              O[4 * q + 2], O[4 * q + 3]);
        }

        Frag bt_frag[DT][2][NS];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++) frag_from_lds(bt_lds[buf], D, dt, hh, bt_frag[dt][hh]);
        update_state(bt_frag, v_frag);
    }

    // ---- the last wavefront to finish leaves the workspace zeroed for the next launch ----
    if (p.nseg > 1) {
        uint32_t done = 0;
        if (lane == 0)
            done = __hip_atomic_fetch_add(hdr + kHdrDone, 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
        done = __builtin_amdgcn_readfirstlane(done);
        if (done == (uint32_t)p.total_waves - 1) {
            for (int i = lane; i < p.total_waves; i += kWave)
                __hip_atomic_store(flags + i, kFlagEmpty, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            for (int i = lane; i < p.total_waves / p.nseg; i += kWave)
                __hip_atomic_store(flags + kMaxWaves + i, 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0)
                __hip_atomic_store(hdr + kHdrDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

struct MfmaPlan {
    int nseg, seg_len;
    int64_t waves, workspace_bytes;
};

MfmaPlan make_plan(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F, int nscans) {
    MfmaPlan pl;
    const int64_t chains = std::max<int64_t>(1, N * H);
    const int64_t total_chunks = (L + kChunk - 1) / kChunk;
    // One wavefront per SIMD is resident (LDS footprint): 1024 slots.  Pick the segment
    // length (in chunks) that minimises an estimate of the makespan: rounds of resident
    // wavefronts times the work of one wavefront (pass 1 costs about half of pass 2, the
    // exchange of segment sums about three chunks).
    int64_t best_c = total_chunks;
    double best_cost = (double)total_chunks * (double)((chains * nscans + 1023) / 1024);
    for (int64_t c = 1; c < total_chunks && c <= 4096; c++) {
        const int64_t nseg = (total_chunks + c - 1) / c;
        const int64_t waves = chains * nseg;
        if (waves * nscans > kMaxWaves || nseg > 4096) continue;  // <= 64 groups of 64 steps
        const double rounds = (double)((waves * nscans + 1023) / 1024);
        const double per_wave = nseg > 1 ? c * 1.5 + 3.0 : (double)c;
        const double cost = rounds * per_wave;
        if (cost < best_cost - 1e-9) {
            best_cost = cost;
            best_c = c;
        }
    }
    // tuning aid: FTC_SEG_CHUNKS=<n> forces segments of n chunks
    if (const char *env = getenv("FTC_SEG_CHUNKS")) {
        const int64_t forced = atoll(env);
        if (forced >= 1 && forced <= total_chunks) {
            const int64_t nseg = (total_chunks + forced - 1) / forced;
            if (chains * nseg * nscans <= kMaxWaves && nseg <= 4096) best_c = forced;
        }
    }
    pl.seg_len = (int)(best_c * kChunk);
    pl.nseg = (int)((L + pl.seg_len - 1) / pl.seg_len);
    pl.waves = chains * pl.nseg;
    pl.workspace_bytes = 0;
    if (pl.nseg > 1)
        pl.workspace_bytes =
            kControlBytes + 2 * nscans * pl.waves * D * F * (int64_t)sizeof(float);
    return pl;
}

template <int D, int F>
void launch(void *workspace, const ScanArgs &args, hipStream_t stream) {
    hipLaunchKernelGGL((scan_mfma_kernel<D, F, 3>), dim3((unsigned)args.total_waves), dim3(kWave),
                       0, stream, (uint32_t *)workspace, args);
}

bool aligned16(const void *ptr, int64_t s0, int64_t s1, int64_t s2) {
    return ((uintptr_t)ptr % 16 == 0) && s0 % 4 == 0 && s1 % 4 == 0 && s2 % 4 == 0;
}

// rows must not overlap (the descriptor's end marks the first row outside the segment) and
// row strides must keep a segment's byte extent inside a 32-bit buffer descriptor
bool stride_ok(int64_t stride_l, int width) { return stride_l >= width && stride_l <= (1 << 16); }

}  // namespace

bool mfma_scan_supported(const ScanDesc &sd, int64_t L) {
    const Operand &a = sd.a, &b = sd.b, &v = sd.v;
    const OperandOut &out = sd.out;
    const int D = a.width, F = v.width;
    const bool shape_ok = (D == 64 && F == 64) || (D == 32 && F == 128) || (D == 128 && F == 32);
    if (!shape_ok) return false;
    if (a.dtype != FTC_F32 || b.dtype != FTC_F32 || v.dtype != FTC_F32 || out.dtype != FTC_F32)
        return false;
    if (L > 1 && !(stride_ok(a.stride_l, D) && stride_ok(b.stride_l, D) &&
                   stride_ok(v.stride_l, F) && stride_ok(out.stride_l, F)))
        return false;
    return aligned16(a.ptr, a.stride_n, a.stride_h, a.stride_l) &&
           aligned16(b.ptr, b.stride_n, b.stride_h, b.stride_l) &&
           aligned16(v.ptr, v.stride_n, v.stride_h, v.stride_l) &&
           aligned16(out.ptr, out.stride_n, out.stride_h, out.stride_l);
}

int64_t mfma_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                                  int nscans) {
    const MfmaPlan pl = make_plan(N, H, L, D, F, nscans);
    return pl.workspace_bytes;
}

int mfma_scan(const ScanDesc *scans, int nscans, int64_t N, int64_t H, int64_t L,
              void *workspace, size_t workspace_bytes, hipStream_t stream) {
    if (nscans < 1 || nscans > kMaxScans) return fail(FTC_ERR_INVALID, "bad scan count");
    const int D = scans[0].a.width, F = scans[0].v.width;
    const MfmaPlan pl = make_plan(N, H, L, D, F, nscans);
    if (pl.workspace_bytes > 0 && (!workspace || workspace_bytes < (size_t)pl.workspace_bytes))
        return fail(FTC_ERR_WORKSPACE, "workspace of %lld bytes needed, %zu given",
                    (long long)pl.workspace_bytes, workspace_bytes);
    if (pl.workspace_bytes > 0 && (uintptr_t)workspace % 256 != 0)
        return fail(FTC_ERR_WORKSPACE, "workspace must be 256-byte aligned");

    ScanArgs args;
    int64_t max_stride = 0;
    for (int i = 0; i < kMaxScans; i++) {
        const ScanDesc &sd = scans[i < nscans ? i : 0];
        ScanOperands &o = args.scan[i];
        o.a = (const float *)sd.a.ptr, o.b = (const float *)sd.b.ptr, o.v = (const float *)sd.v.ptr;
        o.out = (float *)sd.out.ptr;
        o.a_sn = sd.a.stride_n, o.a_sh = sd.a.stride_h, o.a_sl = sd.a.stride_l;
        o.b_sn = sd.b.stride_n, o.b_sh = sd.b.stride_h, o.b_sl = sd.b.stride_l;
        o.v_sn = sd.v.stride_n, o.v_sh = sd.v.stride_h, o.v_sl = sd.v.stride_l;
        o.o_sn = sd.out.stride_n, o.o_sh = sd.out.stride_h, o.o_sl = sd.out.stride_l;
        o.rev = sd.reverse ? 1 : 0;
        o.pad = 0;
        max_stride = std::max(max_stride, std::max(std::max(sd.a.stride_l, sd.b.stride_l),
                                                   std::max(sd.v.stride_l, sd.out.stride_l)));
    }
    // buffer descriptors address a segment with 32-bit byte offsets
    if ((int64_t)(pl.seg_len + 2 * kChunk) * max_stride * 4 >= 0x7fffffffLL)
        return fail(FTC_ERR_UNSUPPORTED, "segment too long for 32-bit offsets");
    args.L = L;
    args.H = (int32_t)H;
    args.seg_len = pl.seg_len;
    args.nseg = pl.nseg;
    args.waves_per_scan = (int32_t)pl.waves;
    args.total_waves = (int32_t)(pl.waves * nscans);
    // short chains: one level (every step adds the sums of all steps before it); long
    // chains: groups of about sqrt(nseg) steps
    args.group = pl.nseg;
    if (pl.nseg > 16) {
        args.group = 1;
        while (args.group * args.group < pl.nseg) args.group++;
    }

    if (D == 64 && F == 64)
        launch<64, 64>(workspace, args, stream);
    else if (D == 32 && F == 128)
        launch<32, 128>(workspace, args, stream);
    else
        launch<128, 32>(workspace, args, stream);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(FTC_ERR_HIP, "MFMA scan launch failed: %s", hipGetErrorString(err));
    return FTC_OK;
}

}  // namespace ftc
