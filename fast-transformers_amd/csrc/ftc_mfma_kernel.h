// MFMA causal scan for gfx950, state shapes D x F with D, F multiples of 32 and
// D * F <= 4096; every operand is fp32 or bf16 rows (chosen per operand at compile time),
// the state and all sums are fp32.
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
// Operand paths of scan_mfma_kernel (this file; ftc_mfma_dma_kernel.h feeds everything
// through LDS instead): row-major fragments (a, and b for (1)) are two 16-byte global loads
// per k-step, straight into the register layout the MFMA wants.  Position-major fragments
// (b for (3), v) are fetched as whole rows with 16-byte loads, parked in a double-buffered
// LDS tile in their own element type, and read back by column with element-wide reads
// (consecutive lanes, consecutive banks).  b is read in both layouts; the second read hits
// L1/L2.
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
#pragma once
#include "ftc_common.h"

namespace ftc {
namespace mfma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t lds_u32x4 __attribute__((ext_vector_type(4), may_alias));
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
// x minus the bf16 that sits in the low (even) or high (odd) half of `pair`, exactly: one
// v_dot2c_f32_bf16 with a (-1, 0) or (0, -1) selector instead of a mask and a subtraction.
// The selectors live in scalar registers behind an asm so that they are not folded into an
// inline constant (which this instruction would read as a 32-bit pattern).
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t minus_one_even() {
    uint32_t s;
    asm("s_mov_b32 %0, 0xbf80" : "=s"(s));
    return s;
}
__device__ __forceinline__ uint32_t minus_one_odd() {
    uint32_t s;
    asm("s_mov_b32 %0, 0xbf800000" : "=s"(s));
    return s;
}
__device__ __forceinline__ float minus_piece(float x, uint32_t pair, uint32_t selector) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pair),
                                           __builtin_bit_cast(bf16x2, selector), x, false);
}

// Cut two fp32 values into NS bf16 pieces each (by truncation, so the pieces add up to the
// value exactly); out[p] packs piece p of (x0, x1).
template <int NS>
__device__ __forceinline__ void split_pair(float x0, float x1, uint32_t (&out)[NS]) {
#pragma unroll
    for (int p = 0; p < NS; p++) {
        out[p] = pack_hi16(x0, x1);
        if (p + 1 < NS) {
            x0 = minus_piece(x0, out[p], minus_one_even());
            x1 = minus_piece(x1, out[p], minus_one_odd());
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

// acc += A * B over the piece products of order <= 2, smallest first (an operand that was
// bf16 to begin with has a single piece).
template <int NA, int NB>
__device__ __forceinline__ f32x16 mfma_split(const Frag (&a)[NA], const Frag (&b)[NB], f32x16 acc) {
#pragma unroll
    for (int order = 2; order >= 0; order--) {
#pragma unroll
        for (int pa = 0; pa < NA; pa++) {
            const int pb = order - pa;
            if (pb >= 0 && pb < NB) acc = mfma(a[pa], b[pb], acc);
        }
    }
    return acc;
}

// Element types of the operands.
struct bf16_t {
    uint16_t bits;
};
template <typename T>
struct Elem;
template <>
struct Elem<float> {
    static constexpr int kBytes = 4, kPieces = 3;
};
template <>
struct Elem<bf16_t> {
    static constexpr int kBytes = 2, kPieces = 1;
};

// Four consecutive elements of a row as they come out of one load.
template <typename T>
struct Quad;
template <>
struct Quad<float> {
    float4 v;
};
template <>
struct Quad<bf16_t> {
    uint2 v;  // 4 bf16
};

__device__ __forceinline__ float4 buffer_load4(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset) {
    const u32x4 r = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0);
    return make_float4(__uint_as_float(r.x), __uint_as_float(r.y), __uint_as_float(r.z),
                       __uint_as_float(r.w));
}
__device__ __forceinline__ float buffer_load1(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset) {
    return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 0));
}
__device__ __forceinline__ void buffer_load_quad(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset,
                                                 Quad<float> &q) {
    q.v = buffer_load4(rsrc, byte_offset);
}
__device__ __forceinline__ void buffer_load_quad(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset,
                                                 Quad<bf16_t> &q) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 r = __builtin_amdgcn_raw_buffer_load_b64(rsrc, byte_offset, 0, 0);
    q.v = make_uint2(r.x, r.y);
}
// two quads (k-slots 0..3 and 4..7) -> fragments
__device__ __forceinline__ void quads_to_frags(const Quad<float> &lo, const Quad<float> &hi,
                                               Frag (&f)[3]) {
    const float x[8] = {lo.v.x, lo.v.y, lo.v.z, lo.v.w, hi.v.x, hi.v.y, hi.v.z, hi.v.w};
    split8<3>(x, f);
}
__device__ __forceinline__ void quads_to_frags(const Quad<bf16_t> &lo, const Quad<bf16_t> &hi,
                                               Frag (&f)[1]) {
    f[0] = Frag{{lo.v.x, lo.v.y, hi.v.x, hi.v.y}};
}
// eight values of one column of an LDS tile (rows given) -> fragments
__device__ __forceinline__ void column_to_frags(const float *tile, const int (&idx)[8],
                                                Frag (&f)[3]) {
    float x[8];
#pragma unroll
    for (int t = 0; t < 8; t++) x[t] = tile[idx[t]];
    split8<3>(x, f);
}
__device__ __forceinline__ void column_to_frags(const bf16_t *tile, const int (&idx)[8],
                                                Frag (&f)[1]) {
#pragma unroll
    for (int q = 0; q < 4; q++)
        f[0].w[q] = (uint32_t)tile[idx[2 * q]].bits | ((uint32_t)tile[idx[2 * q + 1]].bits << 16);
}
// four consecutive columns of one output row
__device__ __forceinline__ void buffer_store_out(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset,
                                                 float x, float y, float z, float w, float *) {
    const u32x4 r = {__float_as_uint(x), __float_as_uint(y), __float_as_uint(z), __float_as_uint(w)};
    __builtin_amdgcn_raw_buffer_store_b128(r, rsrc, byte_offset, 0, 0);
}
// (as a conversion of a pair, so that it becomes one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}
__device__ __forceinline__ void buffer_store_out(__amdgpu_buffer_rsrc_t rsrc, uint32_t byte_offset,
                                                 float x, float y, float z, float w, bf16_t *) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 r = {pack_bf16_rne(x, y), pack_bf16_rne(z, w)};
    __builtin_amdgcn_raw_buffer_store_b64(r, rsrc, byte_offset, 0, 0);
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

// Exchange of segment states between the wavefronts of a chain.
//
// Segments of a chain form groups of `group` consecutive steps (steps are numbered in
// dependency order).  The state before step s is (sum of the totals of the groups before
// its group) + (sum of the sums of the steps before it in its group), always added in
// ascending order, so the result does not depend on timing.  Every step but the last of its
// group publishes its own sum; the last step of every group but the last publishes the
// group total.  States travel as sc1 buffer accesses; flags as agent-scope atomics; every
// wait is bounded.
template <int DT, int FT>
struct StateExchange {
    static constexpr int kStateBytes = DT * FT * 16 * kWave * 4;
    gu32 *flags;
    __amdgpu_buffer_rsrc_t st_rs;
    uint32_t total_slots, ticket, chain_ticket0;
    int step, nseg, G, grp, grp_first, lane;
    bool is_last_of_group, need_own_sum, failed;
    int spins;

    // `slots`: 2 * total_slots states; `ticket`: this wavefront's slot, its chain's step-0
    // slot being ticket - step
    __device__ __forceinline__ StateExchange(gu32 *flags_, gfloat *slots, uint32_t total_slots_,
                                             uint32_t ticket_, int step_, int nseg_, int group,
                                             int lane_)
        : flags(flags_), total_slots(total_slots_), ticket(ticket_),
          chain_ticket0(ticket_ - (uint32_t)step_), step(step_), nseg(nseg_), G(group),
          lane(lane_), failed(false), spins(0) {
        st_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)slots, 0, (2u * total_slots) * (uint32_t)kStateBytes, kRsrcFlags);
        grp = step / G;
        grp_first = grp * G;
        const int grp_last = min(grp_first + G, nseg) - 1;
        is_last_of_group = step == grp_last;
        need_own_sum = step + 1 < nseg;  // the very last step has no reader
    }

    __device__ __forceinline__ void publish_state(uint32_t slot, const f32x16 (&T)[DT][FT],
                                                  uint32_t flag_value) {
        const uint32_t base = slot * (uint32_t)kStateBytes + 16u * lane;
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
    }

    __device__ __forceinline__ void add_state(uint32_t slot, f32x16 (&T)[DT][FT]) {
        const uint32_t base = slot * (uint32_t)kStateBytes + 16u * lane;
        // all loads of a state are in flight together, then added in a fixed order
        u32x4 w[DT * FT * 4];
#pragma unroll
        for (int i = 0; i < DT * FT * 4; i++)
            w[i] = __builtin_amdgcn_raw_buffer_load_b128(st_rs, base + (uint32_t)(i * kWave * 16),
                                                         0, kCoherentAux);
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
    }

    // wait until `count` wavefronts, slots first, first + stride, ..., show `bit`
    __device__ __forceinline__ void wait_flags(uint32_t first, uint32_t stride, int count,
                                               uint32_t bit) {
        const bool mine = lane < count;
        const gu32 *f = flags + first + stride * (uint32_t)lane;
        while (!failed) {
            const uint32_t x =
                mine ? __hip_atomic_load(f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : bit;
            if (__builtin_amdgcn_ballot_w64((x & bit) == 0) == 0) break;
            if (++spins > kSpinLimit) failed = true;
            __builtin_amdgcn_s_sleep(4);
        }
        // the states behind these flags are read with plain buffer loads: keep the compiler
        // from moving any of them above the wait
        asm volatile("" ::: "memory");
    }

    // after pass 1: make this step's own sum visible to the later steps of its group
    __device__ __forceinline__ void publish_sum(const f32x16 (&S)[DT][FT]) {
        if (need_own_sum && !is_last_of_group) publish_state(ticket, S, kFlagSum);
    }

    // X <- state before this step (S = this step's own sum, left untouched)
    __device__ __forceinline__ void gather(const f32x16 (&S)[DT][FT], f32x16 (&X)[DT][FT]) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++)
#pragma unroll
                for (int r = 0; r < 16; r++) X[dt][ft][r] = 0.f;
        // ---- sums of the earlier steps of this group ----
        const int in_group = step - grp_first;
        if (in_group > 0) {
            wait_flags(chain_ticket0 + grp_first, 1, in_group, kFlagSum);
            if (!failed)
                for (int i = 0; i < in_group; i++) add_state(chain_ticket0 + grp_first + i, X);
        }
        if (is_last_of_group && need_own_sum && !failed) {
            // group total = sums of the group in ascending order (own sum last)
            f32x16 T[DT][FT];
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int ft = 0; ft < FT; ft++) T[dt][ft] = X[dt][ft] + S[dt][ft];
            publish_state(total_slots + ticket, T, kFlagTotal);
        }
        // ---- totals of the earlier groups, then the in-group part on top ----
        if (grp > 0 && !failed) {
            wait_flags(chain_ticket0 + (uint32_t)(G - 1), (uint32_t)G, grp, kFlagTotal);
            if (!failed) {
                f32x16 T[DT][FT];
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int ft = 0; ft < FT; ft++) {
                        T[dt][ft] = X[dt][ft];
#pragma unroll
                        for (int r = 0; r < 16; r++) X[dt][ft][r] = 0.f;
                    }
                for (int gq = 0; gq < grp; gq++)
                    add_state(total_slots + chain_ticket0 + (uint32_t)(gq * G + G - 1), X);
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int ft = 0; ft < FT; ft++) X[dt][ft] = X[dt][ft] + T[dt][ft];
            }
        }
    }
};

// One scan of a launch.  A launch runs up to kMaxScans independent scans of the same
// (D, F, N, H, L) side by side (the three gradients of a backward call, the column slices
// of a wide output), so that their launch gaps and wait times overlap.
// element types of a scan's rows as ScanOperands::pad carries them: bits set for bf16 rows
constexpr int kRowsBf16A = 1, kRowsBf16B = 2, kRowsBf16V = 4, kRowsBf16Out = 8;

struct ScanOperands {
    const void *a, *b, *v;
    void *out;
    int64_t a_sn, a_sh, a_sl;
    int64_t b_sn, b_sh, b_sl;
    int64_t v_sn, v_sh, v_sl;
    int64_t o_sn, o_sh, o_sl;
    int32_t rev;  // 0: j <= l, walk up; 1: j >= l, walk down
    int32_t pad;  // kRowsBf16* bits (read by the kernel that takes rows of either type scan by scan)
    // optional D x F fp32 states per chain (null: none): the state the scan starts from and
    // the state after its last position; strides in elements, unit stride along F
    const float *s0;
    float *s_out;
    int64_t s0_sn, s0_sh, s0_sd;
    int64_t so_sn, so_sh, so_sd;
};

// The caller's state in accumulator layout: register r of tile (dt, ft) in lane (ln, g) is
// element (d = 32*dt + 8*(r/4) + 4*g + r%4, f = 32*ft + ln), so the 32 lanes of a half-wave
// touch 128 consecutive bytes.
template <int DT, int FT>
__device__ __forceinline__ void add_caller_state(const float *base, int64_t row_stride, int ln,
                                                 int g, f32x16 (&S)[DT][FT]) {
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int d = 32 * dt + 8 * (r / 4) + 4 * g + (r % 4);
                S[dt][ft][r] += base[(int64_t)d * row_stride + 32 * ft + ln];
            }
}
template <int DT, int FT>
__device__ __forceinline__ void store_caller_state(float *base, int64_t row_stride, int ln, int g,
                                                   const f32x16 (&S)[DT][FT]) {
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int d = 32 * dt + 8 * (r / 4) + 4 * g + (r % 4);
                base[(int64_t)d * row_stride + 32 * ft + ln] = S[dt][ft][r];
            }
}
constexpr int kMaxScans = kMfmaMaxScans;

constexpr int kMaxTpSegments = 16;
// chunks that the chain-parallel kernel requests ahead (measured on cfg2: 6 and 8 are slower)
#ifndef FTC_TP_AHEAD
#define FTC_TP_AHEAD 4
#endif
constexpr int kTpAhead = FTC_TP_AHEAD;

struct ScanArgs {
    ScanOperands scan[kMaxScans];
    int64_t L;
    int32_t H, seg_len, nseg;
    int32_t waves_per_scan;
    int32_t total_waves;  // nscans * waves_per_scan
    int32_t group;        // steps per group of the two-level state sum
    // fused attention form of the workgroup kernel only (ftc_wg_kernel.h, NORM)
    float eps;               // added to the denominator
    const int64_t *key_len;  // keys per batch entry, N values on the device; nullptr: all L
    // chain-parallel kernel only (ftc_tp_kernel.h): segment s of a chain is chunks
    // tp_start[s] .. tp_start[s + 1] - 1 (starts are multiples of kTpAhead)
    int32_t tp_start[kMaxTpSegments + 1];
    // ... or, with an exchange of segment sums (tp_exchange != 0), nseg segments of
    // tp_seg_chunks chunks (a multiple of kTpAhead), taken in the order of arrival
    int32_t tp_exchange, tp_seg_chunks;
    // widths of the rows as they lie in memory (a, b: tp_d <= 128; v, out: tp_f <= 128, both
    // multiples of 4) and the number of 64-column blocks of v and out, one workgroup each
    int32_t tp_d, tp_f, tp_fblocks;
};

// Which (scan, chain, L-segment) a wavefront works on.
//
// Workgroups are dispatched round-robin over the 8 XCDs.  Blocks are numbered so that
// wavefront w of every scan of the launch lands on the same XCD at about the same time
// (groups of 8 consecutive blocks per scan): scans that read the same rows find each other's
// lines in that XCD's L2.  Chains of all scans are numbered consecutively
// (scan * chains + chain), and the wavefronts launched for a chain take that chain's steps in
// the order in which they start running (a ticket per chain), so a step only ever waits for
// steps that are already running.
struct Segment {
    uint32_t scan_id, chain_slot0;  // chain_slot0: slot of step 0 of this chain
    uint32_t ticket;                // this wavefront's flag / state slot
    int step, seg;                  // position in dependency order, position along L
    int n, h;
    int64_t lo;                     // first row of the segment
    int rows, nchunks;
    bool rev;
};

// First half: block number -> scan and chain, and the request for a ticket (answer pending
// in `order`, valid in lane 0).
__device__ __forceinline__ void segment_request(const ScanArgs &p, gu32 *flags, int lane,
                                                Segment &s, uint32_t &order) {
    const uint32_t wps = (uint32_t)p.waves_per_scan;
    const uint32_t nscans = (uint32_t)p.total_waves / wps;
    const uint32_t full = (wps / 8u) * 8u;
    uint32_t wave_in_scan;
    if (blockIdx.x < full * nscans) {
        const uint32_t grp = blockIdx.x / (8u * nscans), r = blockIdx.x % (8u * nscans);
        s.scan_id = r / 8u;
        wave_in_scan = grp * 8u + r % 8u;
    } else {
        const uint32_t t = blockIdx.x - full * nscans;
        s.scan_id = t / (wps - full);
        wave_in_scan = full + t % (wps - full);
    }
    const uint32_t vblock = s.scan_id * wps + wave_in_scan;  // block id in scan-major order
    const uint32_t my_chain = vblock / (uint32_t)p.nseg;
    s.chain_slot0 = my_chain * (uint32_t)p.nseg;
    s.rev = p.scan[s.scan_id].rev != 0;
    order = vblock - s.chain_slot0;  // a single segment per chain needs no ticket
    if (p.nseg > 1 && lane == 0)
        order = __hip_atomic_fetch_add(flags + kMaxWaves + my_chain, 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
}

// Second half: waits for the ticket.  Returns false when the control block was not zero at
// the start of the launch (the wavefront must then stop; the error word says so).
__device__ __forceinline__ bool segment_locate(const ScanArgs &p, gu32 *hdr, int lane,
                                               uint32_t order, Segment &s) {
    order = __builtin_amdgcn_readfirstlane(order);
    if (order >= (uint32_t)p.nseg) {
        if (lane == 0)
            __hip_atomic_store(hdr + kHdrError, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return false;
    }
    s.ticket = s.chain_slot0 + order;
    s.step = (int)order;
    s.seg = s.rev ? p.nseg - 1 - s.step : s.step;
    const int64_t chain =
        (s.chain_slot0 - s.scan_id * (uint32_t)p.waves_per_scan) / (uint32_t)p.nseg;
    s.n = (int)(chain / p.H);
    s.h = (int)(chain % p.H);
    s.lo = (int64_t)s.seg * p.seg_len;
    const int64_t hi = min(p.L, s.lo + (int64_t)p.seg_len);
    s.rows = (int)(hi - s.lo);
    s.nchunks = (s.rows + kChunk - 1) / kChunk;
    return true;
}

// The last wavefront of a launch to get here leaves the control block zeroed for the next
// launch (flags, ticket counters, the counter used here).
__device__ __forceinline__ void release_control_block(const ScanArgs &p, gu32 *hdr, gu32 *flags,
                                                      int lane) {
    if (p.nseg <= 1) return;
    uint32_t done = 0;
    if (lane == 0)
        done = __hip_atomic_fetch_add(hdr + kHdrDone, 1u, __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT);
    done = __builtin_amdgcn_readfirstlane(done);
    if (done != (uint32_t)p.total_waves - 1) return;
    for (int i = lane; i < p.total_waves; i += kWave)
        __hip_atomic_store(flags + i, kFlagEmpty, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (int i = lane; i < p.total_waves / p.nseg; i += kWave)
        __hip_atomic_store(flags + kMaxWaves + i, 0u, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    if (lane == 0)
        __hip_atomic_store(hdr + kHdrDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// TA, TB, TV, TO: element types (float or bf16_t) of the a, b, v rows and of the output rows.
template <int D, int F, typename TA, typename TB, typename TV, typename TO>
__global__ __launch_bounds__(kWave) void scan_mfma_kernel(uint32_t *__restrict__ ws_ptr,
                                                          ScanArgs p) {
    constexpr int NSA = Elem<TA>::kPieces, NSB = Elem<TB>::kPieces, NSV = Elem<TV>::kPieces;
    constexpr int NS = 3;  // pieces of the fp32 intermediates (P and the state)
    constexpr int BA = Elem<TA>::kBytes, BB = Elem<TB>::kBytes, BV = Elem<TV>::kBytes,
                  BO = Elem<TO>::kBytes;
    constexpr int DT = D / 32, FT = F / 32;  // state tiles
    constexpr int KD = D / 16;               // k-steps over d
    constexpr int kStateElems = D * F;

    const int lane = threadIdx.x;
    const int ln = lane & 31, g = lane >> 5;

    gu32 *hdr = (gu32 *)ws_ptr;
    gu32 *flags = hdr + kHdrWords;
    gfloat *sums = (gfloat *)(hdr + kControlBytes / 4);

    Segment sg;
    uint32_t order;
    segment_request(p, flags, lane, sg, order);
    if (!segment_locate(p, hdr, lane, order, sg)) return;
    const ScanOperands &op = p.scan[sg.scan_id];
    const bool REV = sg.rev;
    const char *a_ptr = (const char *)op.a, *b_ptr = (const char *)op.b,
               *v_ptr = (const char *)op.v;
    char *out_ptr = (char *)op.out;
    const uint32_t ticket = sg.ticket;
    const int step = sg.step, n = sg.n, h = sg.h, rows = sg.rows, nchunks = sg.nchunks;
    const int64_t lo = sg.lo;

    // descriptors based at the segment's first row and ending with its last row
    const char *a_seg = a_ptr + ((int64_t)n * op.a_sn + (int64_t)h * op.a_sh + lo * op.a_sl) * BA;
    const char *b_seg = b_ptr + ((int64_t)n * op.b_sn + (int64_t)h * op.b_sh + lo * op.b_sl) * BB;
    const char *v_seg = v_ptr + ((int64_t)n * op.v_sn + (int64_t)h * op.v_sh + lo * op.v_sl) * BV;
    char *o_seg = out_ptr + ((int64_t)n * op.o_sn + (int64_t)h * op.o_sh + lo * op.o_sl) * BO;
    // row strides in bytes
    const uint32_t a_slb = (uint32_t)op.a_sl * BA, b_slb = (uint32_t)op.b_sl * BB,
                   v_slb = (uint32_t)op.v_sl * BV, o_slb = (uint32_t)op.o_sl * BO;
    const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)a_seg, 0, (rows - 1) * a_slb + D * BA, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t b_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)b_seg, 0, (rows - 1) * b_slb + D * BB, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)v_seg, 0, (rows - 1) * v_slb + F * BV, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)o_seg, 0, (rows - 1) * o_slb + F * BO, kRsrcFlags);

    // per-lane byte offsets inside a chunk
    //  row-major fragments: lane (row = ln, g) reads columns 16*ks + 4*g + 0..3 and + 8
    //  position-major fragments: lane (col = ln, g), k-slot t of k-step hh is row
    //  16*hh + 8*(t/4) + 4*g + (t%4)
    const uint32_t a_lane = ln * a_slb + 4u * BA * g;
    const uint32_t b_lane = ln * b_slb + 4u * BB * g;
    // position-major operands pass through LDS in their own element type: 16-byte global
    // loads (lane = (row within the load, 16 bytes of it)), 16-byte LDS writes, element-wide
    // LDS reads by column
    // (rows of 96 values do not divide the wavefront: the lanes left over after the last whole
    // row of a load, and rows past the chunk in the last load, neither fetch nor store)
    constexpr int kBtLanes = D * BB / 16, kVtLanes = F * BV / 16;      // lanes per row
    constexpr int kBtRows = kWave / kBtLanes, kVtRows = kWave / kVtLanes;  // rows per load
    constexpr int kBtLoads = (kChunk + kBtRows - 1) / kBtRows,
                  kVtLoads = (kChunk + kVtRows - 1) / kVtRows;
    const uint32_t bt_lane = (uint32_t)(lane / kBtLanes) * b_slb + 16u * (lane % kBtLanes);
    const uint32_t vt_lane = (uint32_t)(lane / kVtLanes) * v_slb + 16u * (lane % kVtLanes);
    constexpr uint32_t kNoRow = 0x80000000u;  // an offset outside every descriptor: reads zero
    auto bt_row = [&](int i) -> int {
        return lane < kBtRows * kBtLanes ? i * kBtRows + lane / kBtLanes : kChunk;
    };
    auto vt_row = [&](int i) -> int {
        return lane < kVtRows * kVtLanes ? i * kVtRows + lane / kVtLanes : kChunk;
    };
    const uint32_t o_lane = ln * o_slb + 4u * BO * g;

    // first row of chunk c relative to the segment (REV walks down from the end and its
    // last chunk may start before the segment: those rows read as zero)
    auto chunk_row0 = [&](int c) -> int { return REV ? rows - kChunk * (c + 1) : kChunk * c; };
    // pass 1 walks the chunks downwards; "chunk -1" must lie outside the descriptor
    auto pass1_row0 = [&](int c) -> int { return c < 0 ? -2 * kChunk : chunk_row0(c); };

    // raw rows of the chunk being fetched
    Quad<TA> a_raw[KD][2];  // a rows, B operand of (1) and (2b)
    Quad<TB> b_raw[KD][2];  // b rows, A operand of (1)
    u32x4 bt_raw[kBtLoads];  // b rows on their way to LDS (A operand of (3))
    u32x4 vt_raw[kVtLoads];  // v rows on their way to LDS (A operand of (2a), B of (3))
    __shared__ __align__(16) TB bt_lds[2][kChunk * D];
    __shared__ __align__(16) TV vt_lds[2][kChunk * F];

    auto fetch_a = [&](int row0) {
        const uint32_t off = a_lane + (uint32_t)row0 * a_slb;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            buffer_load_quad(a_rs, off + 16u * BA * ks, a_raw[ks][0]);
            buffer_load_quad(a_rs, off + 16u * BA * ks + 8u * BA, a_raw[ks][1]);
        }
    };
    auto fetch_b = [&](int row0) {
        const uint32_t off = b_lane + (uint32_t)row0 * b_slb;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            buffer_load_quad(b_rs, off + 16u * BB * ks, b_raw[ks][0]);
            buffer_load_quad(b_rs, off + 16u * BB * ks + 8u * BB, b_raw[ks][1]);
        }
    };
    auto fetch_bt_into = [&](int row0, u32x4 (&raw)[kBtLoads]) {
        const uint32_t off = bt_lane + (uint32_t)row0 * b_slb;
#pragma unroll
        for (int i = 0; i < kBtLoads; i++)
            raw[i] = __builtin_amdgcn_raw_buffer_load_b128(
                b_rs, bt_row(i) < kChunk ? off + (uint32_t)(i * kBtRows) * b_slb : kNoRow, 0, 0);
    };
    auto fetch_vt_into = [&](int row0, u32x4 (&raw)[kVtLoads]) {
        const uint32_t off = vt_lane + (uint32_t)row0 * v_slb;
#pragma unroll
        for (int i = 0; i < kVtLoads; i++)
            raw[i] = __builtin_amdgcn_raw_buffer_load_b128(
                v_rs, vt_row(i) < kChunk ? off + (uint32_t)(i * kVtRows) * v_slb : kNoRow, 0, 0);
    };
    // fetched rows -> LDS tile `buf` (row-major, 32 rows)
    auto stash_bt_from = [&](int buf, const u32x4 (&raw)[kBtLoads]) {
        char *tile = (char *)bt_lds[buf];
#pragma unroll
        for (int i = 0; i < kBtLoads; i++)
            if (bt_row(i) < kChunk)
                *(lds_u32x4 *)(tile + bt_row(i) * (D * BB) + 16 * (lane % kBtLanes)) = raw[i];
    };
    auto stash_vt_from = [&](int buf, const u32x4 (&raw)[kVtLoads]) {
        char *tile = (char *)vt_lds[buf];
#pragma unroll
        for (int i = 0; i < kVtLoads; i++)
            if (vt_row(i) < kChunk)
                *(lds_u32x4 *)(tile + vt_row(i) * (F * BV) + 16 * (lane % kVtLanes)) = raw[i];
    };
    auto fetch_bt = [&](int row0) { fetch_bt_into(row0, bt_raw); };
    auto fetch_vt = [&](int row0) { fetch_vt_into(row0, vt_raw); };
    auto stash_bt = [&](int buf) { stash_bt_from(buf, bt_raw); };
    auto stash_vt = [&](int buf) { stash_vt_from(buf, vt_raw); };
    // LDS tile -> the fragments of k-step hh for the 32 columns of tile `tile`
    auto bt_frags = [&](int buf, int tile, int hh, Frag (&frag)[NSB]) {
        int idx[8];
#pragma unroll
        for (int t = 0; t < 8; t++)
            idx[t] = (16 * hh + 8 * (t / 4) + 4 * g + (t % 4)) * D + 32 * tile + ln;
        column_to_frags(bt_lds[buf], idx, frag);
    };
    auto vt_frags = [&](int buf, int tile, int hh, Frag (&frag)[NSV]) {
        int idx[8];
#pragma unroll
        for (int t = 0; t < 8; t++)
            idx[t] = (16 * hh + 8 * (t / 4) + 4 * g + (t % 4)) * F + 32 * tile + ln;
        column_to_frags(vt_lds[buf], idx, frag);
    };

    f32x16 S[DT][FT];
    // (3) S += b^T v
    auto update_state = [&](const Frag (&bt_frag)[DT][2][NSB], const Frag (&v_frag)[FT][2][NSV]) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
                    S[dt][ft] = mfma_split<NSB, NSV>(bt_frag[dt][hh], v_frag[ft][hh], S[dt][ft]);
    };

#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int r = 0; r < 16; r++) S[dt][ft][r] = 0.f;

    if (p.nseg > 1) {
        StateExchange<DT, FT> xch(flags, sums, (uint32_t)p.total_waves, ticket, step, p.nseg,
                                  p.group, lane);

        // ---- pass 1: the segment's own state sum, walked against the direction of pass 2
        // so that pass 2 starts on the rows read last ----
        if (xch.need_own_sum) {
            // rows are requested two chunks ahead (pass 1 has registers to spare and its
            // chunks are short compared with the memory latency)
            u32x4 bt_raw2[kBtLoads], vt_raw2[kVtLoads];
            auto sum_chunk = [&](int buf) {
                Frag bt_frag[DT][2][NSB], v_frag[FT][2][NSV];
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) bt_frags(buf, dt, hh, bt_frag[dt][hh]);
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) vt_frags(buf, ft, hh, v_frag[ft][hh]);
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
            xch.publish_sum(S);
        }
        // start fetching the first chunk of pass 2 before waiting
        fetch_a(chunk_row0(0));
        fetch_b(chunk_row0(0));
        fetch_vt(chunk_row0(0));
        fetch_bt(chunk_row0(0));

        f32x16 X[DT][FT];
        xch.gather(S, X);
        if (xch.failed && lane == 0)
            __hip_atomic_store(hdr + kHdrError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++) S[dt][ft] = X[dt][ft];
    } else {
        fetch_a(chunk_row0(0));
        fetch_b(chunk_row0(0));
        fetch_vt(chunk_row0(0));
        fetch_bt(chunk_row0(0));
    }
    // every segment starts from (the caller's initial state) + (the sums of the segments
    // before it)
    if (op.s0)
        add_caller_state<DT, FT>(op.s0 + (int64_t)n * op.s0_sn + (int64_t)h * op.s0_sh, op.s0_sd,
                                 ln, g, S);

    // ---- pass 2: outputs ----
    for (int c = 0; c < nchunks; c++) {
        const int row0 = chunk_row0(c);
        // rows of the chunk after the last one are outside the descriptor and read as zero,
        // so the prefetch needs no branch
        const int next0 = chunk_row0(c + 1);

        // each operand is cut into pieces as soon as it is needed and its raw registers
        // are refilled with the next chunk right away
        Frag a_frag[KD][NSA], b_frag[KD][NSB];
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            quads_to_frags(a_raw[ks][0], a_raw[ks][1], a_frag[ks]);
            quads_to_frags(b_raw[ks][0], b_raw[ks][1], b_frag[ks]);
        }
        fetch_a(next0);
        fetch_b(next0);

        // (1) Pt = b a^T
        f32x16 P;
#pragma unroll
        for (int r = 0; r < 16; r++) P[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) P = mfma_split<NSB, NSA>(b_frag[ks], a_frag[ks], P);
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
        Frag v_frag[FT][2][NSV];  // A operand of (2a), B operand of (3)
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++) vt_frags(buf, ft, hh, v_frag[ft][hh]);

        // (2b) + (2a): the output tiles advance side by side so that their MFMA chains are
        // independent of each other, then store
        const uint32_t o_off = o_lane + (uint32_t)row0 * o_slb;
        f32x16 O[FT];
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int r = 0; r < 16; r++) O[ft][r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
#pragma unroll
            for (int ft = 0; ft < FT; ft++) {
                const int o8 = 8 * (ks % 2);
                const float x[8] = {S[ks / 2][ft][o8 + 0], S[ks / 2][ft][o8 + 1],
                                    S[ks / 2][ft][o8 + 2], S[ks / 2][ft][o8 + 3],
                                    S[ks / 2][ft][o8 + 4], S[ks / 2][ft][o8 + 5],
                                    S[ks / 2][ft][o8 + 6], S[ks / 2][ft][o8 + 7]};
                Frag s_frag[NS];
                split8<NS>(x, s_frag);
                O[ft] = mfma_split<NS, NSA>(s_frag, a_frag[ks], O[ft]);
            }
        }
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++)
                O[ft] = mfma_split<NSV, NS>(v_frag[ft][hh], p_frag[hh], O[ft]);
        // lane (i = ln, g) holds f = 32*ft + 8*q + 4*g + 0..3 in registers 4q..4q+3
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                buffer_store_out(o_rs, o_off + (uint32_t)(BO * (32 * ft + 8 * q)), O[ft][4 * q + 0],
                                 O[ft][4 * q + 1], O[ft][4 * q + 2], O[ft][4 * q + 3],
                                 (TO *)nullptr);

        Frag bt_frag[DT][2][NSB];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++) bt_frags(buf, dt, hh, bt_frag[dt][hh]);
        update_state(bt_frag, v_frag);
    }

    // the segment walked last ends on the state after the whole sequence
    if (op.s_out && step == p.nseg - 1)
        store_caller_state<DT, FT>(op.s_out + (int64_t)n * op.so_sn + (int64_t)h * op.so_sh,
                                   op.so_sd, ln, g, S);
    release_control_block(p, hdr, flags, lane);
}

// Host-side launcher of one element-type combination; D, F picked at run time.
template <typename TA, typename TB, typename TV, typename TO>
void launch_scan(int D, int F, void *workspace, const ScanArgs &args, hipStream_t stream) {
    const dim3 grid((unsigned)args.total_waves), block(kWave);
#define FTC_LAUNCH(DD, FF)                                                                      \
    hipLaunchKernelGGL((scan_mfma_kernel<DD, FF, TA, TB, TV, TO>), grid, block, 0, stream,      \
                       (uint32_t *)workspace, args)
    if (D == 64 && F == 64) FTC_LAUNCH(64, 64);
    else if (D == 32 && F == 128) FTC_LAUNCH(32, 128);
    else if (D == 128 && F == 32) FTC_LAUNCH(128, 32);
    else if (D == 32 && F == 32) FTC_LAUNCH(32, 32);
    else if (D == 32 && F == 64) FTC_LAUNCH(32, 64);
    else if (D == 96 && F == 32) FTC_LAUNCH(96, 32);
    else FTC_LAUNCH(64, 32);
#undef FTC_LAUNCH
}

// One function per element-type combination, each compiled in its own file.
void launch_scan_ffff(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);
void launch_scan_bbbf(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);
void launch_scan_fbbb(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);
void launch_scan_bfbb(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);
void launch_scan_bbfb(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);

}  // namespace mfma
}  // namespace ftc
