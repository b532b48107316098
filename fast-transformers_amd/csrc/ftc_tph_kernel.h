// Chain-parallel form of the MFMA causal scan for gfx950 on the fp16 matrix path: fp32 rows
// (or, in the MIX form of the kernel, any operand in bf16: such rows are widened as they arrive
// and rounded to nearest even as they leave; their low pieces are zero), states of up to
// 64 x 64 per workgroup (output columns beyond 64 have a workgroup of their own, widths that do
// not fill the block are clipped).
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (REV: j >= l)
//
// Division of labour, chunking, LDS tiles, swizzles, segments and the exchange of segment
// sums are those of ftc_tp_kernel.h (one workgroup walks one chain; four consumer wavefronts
// hold the state as slabs of 16 columns and share the chunk product Pt through LDS; producer
// wavefronts -- eight here, one quad of every operand per lane and position -- fetch rows
// four chunks ahead and cut them into piece tiles).  What differs is the arithmetic that
// stands for an fp32 product:
//
//  * Every fp32 value x is scaled by a power of two and cut into TWO fp16 pieces, both rounded
//    to nearest: hi = fp16(x s), lo = fp16(x s - hi).  hi + lo carries 22 significand bits of
//    x s as long as |x s| >= 2^-3 (below that the absolute error stays under 2^-25), and
//    |x s| < 2^16 must hold.  A product is the sum of THREE piece products (lo hi, hi lo,
//    hi hi; lo lo is below 2^-22 of the product) on v_mfma_f32_16x16x32_f16, each exact in the
//    fp32 accumulator: half the matrix instructions, two thirds of the LDS traffic and about
//    a third of the vector instructions of three bf16 pieces, with results as close to
//    float64 as those (the reference's own fp32 order is further away than either).
//  * The scales.  Rows are scaled chunk by chunk by powers of two, 2^(4 - e) with 2^e a
//    ceiling above every magnitude concerned: for b and v, whose products add up in the
//    state, every value of that operand met so far in the walk (a ceiling that only rises);
//    for a, the values of the chunk alone.  Scaled values therefore stay below 16, values
//    down to 2^-7 of the ceiling keep 22 bits, and the error of smaller ones is below 2^-29 of
//    the ceiling -- for b and v the way the reference's running fp32 state treats small
//    contributions, for a within the 32 rows of a chunk.  The ceilings come about without a
//    pass of their own: while they cut position k of the walk, the producers look at the rows
//    of position k + 1, which they already hold in registers, and enter what they find in
//    that position's slot in LDS with atomic maxima (for b and v only when a value reaches the
//    running ceiling: rare after the first chunks; for a one word per wavefront and
//    position); after the
//    workgroup barrier all twelve wavefronts read the slot.  All of them thus know the same
//    three exponents for every position, and they depend on the rows alone: however a chain
//    is cut into segments, the results are the same bit for bit (as long as the state stays
//    below 2^14 units, s = 0; beyond that the chunk where s rises depends on the cut, and
//    results agree to the rounding of the state's pieces, 2^-22).
//  * The state is kept in the units of the scaled rows (2^(e_b + e_v - 8)); when a ceiling
//    rises it is rescaled (exactly).  It is cut into pieces with one more power of two,
//    2^-s, chosen so that no element leaves fp16's range: every third chunk s rises if an
//    element of the state exceeds 2^(14 + s) (a chunk adds at most 2^13: three more chunks
//    stay below 2^14 + 3 x 2^13 < 65504).  As long as s = 0, the rule, the cut is plain
//    (one packed conversion per pair for the high pieces).  The chunk product needs no scale:
//    |Pt| <= 64 * 16 * 16 = 2^14.
//  * Ot = (S^T a^T) 2^s + v^T Pt is summed in the units of the chunk and leaves the
//    accumulator through one v_ldexp_f32 per value.
#pragma once
#include <type_traits>

#include "ftc_tp_kernel.h"

namespace ftc {
namespace mfma {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ f32x4 mfma16h(const Frag &a, const Frag &b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// Four fp32 values times a power of two -> packed fp16 pieces (x0, x2 in the low halves), all
// rounded to nearest even.  v_fma_mix{lo,hi}_f16 computes fma(x, s, c) in fp32 (exact here:
// x s is exact, and so is the remainder of a rounding) and rounds once to fp16; the third
// operand is the fp16 hi piece, read from the half that op_sel names and negated.  The two
// pairs are cut in turn, so that no instruction reads (or completes) a half-written register
// right after the instruction that wrote it: that costs a wait state each time.
__device__ __forceinline__ void cut_quad_f16(float x0, float x1, float x2, float x3, float s,
                                             uint32_t &h01, uint32_t &h23, uint32_t &l01,
                                             uint32_t &l23) {
    asm("v_fma_mixlo_f16 %0, %4, %8, 0\n\t"
        "v_fma_mixlo_f16 %1, %6, %8, 0\n\t"
        "v_fma_mixhi_f16 %0, %5, %8, 0\n\t"
        "v_fma_mixhi_f16 %1, %7, %8, 0\n\t"
        "v_fma_mixlo_f16 %2, %4, %8, -%0 op_sel:[0,0,0] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixlo_f16 %3, %6, %8, -%1 op_sel:[0,0,0] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %2, %5, %8, -%0 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %3, %7, %8, -%1 op_sel:[0,0,1] op_sel_hi:[0,0,1]"
        : "=&v"(h01), "=&v"(h23), "=&v"(l01), "=&v"(l23)
        : "v"(x0), "v"(x1), "v"(x2), "v"(x3), "v"(s));
}
// the same without a scale: one packed conversion per pair for the hi pieces
__device__ __forceinline__ void cut_quad_f16_unscaled(float x0, float x1, float x2, float x3,
                                                      uint32_t &h01, uint32_t &h23, uint32_t &l01,
                                                      uint32_t &l23) {
    asm("v_cvt_pk_f16_f32 %0, %4, %5\n\t"
        "v_cvt_pk_f16_f32 %1, %6, %7\n\t"
        "v_fma_mixlo_f16 %2, %4, 1.0, -%0 op_sel:[0,0,0] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixlo_f16 %3, %6, 1.0, -%1 op_sel:[0,0,0] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %2, %5, 1.0, -%0 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\t"
        "v_fma_mixhi_f16 %3, %7, 1.0, -%1 op_sel:[0,0,1] op_sel_hi:[0,0,1]"
        : "=&v"(h01), "=&v"(h23), "=&v"(l01), "=&v"(l23)
        : "v"(x0), "v"(x1), "v"(x2), "v"(x3));
}
// Four consecutive fp32 values of a row -> 8 bytes of each of the two piece tiles.
__device__ __forceinline__ void cut_quad_to_lds(const u32x4 raw, float s, lds_char *tile,
                                                int piece_bytes, int addr) {
    uint32_t h0, l0, h1, l1;
    cut_quad_f16(__uint_as_float(raw.x), __uint_as_float(raw.y), __uint_as_float(raw.z),
                 __uint_as_float(raw.w), s, h0, h1, l0, l1);
    const u32x2 wh = {h0, h1}, wl = {l0, l1};
    *(lds_vec2 *)(tile + addr) = wh;
    *(lds_vec2 *)(tile + piece_bytes + addr) = wl;
}
__device__ __forceinline__ float max_abs4(const u32x4 raw, float m) {
    m = fmaxf(fmaxf(fabsf(__uint_as_float(raw.x)), fabsf(__uint_as_float(raw.y))), m);
    return fmaxf(fmaxf(fabsf(__uint_as_float(raw.z)), fabsf(__uint_as_float(raw.w))), m);
}

// Exponents travel as E = e + 128 with e clamped to -100 .. 120 (E = 28 .. 248), where 2^e is
// the ceiling: every value met so far is below it.
constexpr uint32_t kExpFloor = 28, kExpCeil = 248;
__device__ __forceinline__ float pow2_field(int field) {  // 2^(field - 127), field clamped
    return __uint_as_float((uint32_t)max(1, min(254, field)) << 23);
}
// wave-uniform integer maxima and minima on the scalar unit (written out: the compiler would
// merge them into three-operand vector instructions)
__device__ __forceinline__ uint32_t scalar_max(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("s_max_u32 %0, %1, %2" : "=s"(r) : "s"(a), "s"(b) : "scc");
    return r;
}
__device__ __forceinline__ uint32_t scalar_min(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("s_min_u32 %0, %1, %2" : "=s"(r) : "s"(a), "s"(b) : "scc");
    return r;
}
// the ceiling exponent of a non-negative float, given as its bits in a scalar register (inf and
// NaN: the largest)
__device__ __forceinline__ uint32_t ceiling_of(uint32_t bits) {
    const uint32_t be = (bits >> 23) & 0xffu;  // the value is below 2^(be - 126)
    return scalar_max(kExpFloor, scalar_min(kExpCeil, be + 2u));
}
// The largest of a non-negative float over the wavefront (wave-uniform): four steps inside
// the rows of 16 lanes on the data-parallel path, then one lane of every row.
// (non-negative floats order like their bit patterns: an integer maximum needs no
// canonicalising copy of the lane it reads across, and folds into one instruction)
template <int CTRL>
__device__ __forceinline__ uint32_t max_with_dpp(uint32_t x) {
    return max(x, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true));
}
// ... over each row of 16 lanes (every lane of a row gets the row's maximum)
__device__ __forceinline__ uint32_t row_max_bits(float m) {
    uint32_t b = __float_as_uint(m);
    b = max_with_dpp<0xb1>(b);   // quad_perm [1, 0, 3, 2]
    b = max_with_dpp<0x4e>(b);   // quad_perm [2, 3, 0, 1]
    b = max_with_dpp<0x141>(b);  // row_half_mirror
    b = max_with_dpp<0x140>(b);  // row_mirror
    return b;
}
__device__ __forceinline__ uint32_t wave_max(float m) {  // (the bits of the largest value)
    const uint32_t b = row_max_bits(m);
    return scalar_max(scalar_max((uint32_t)__builtin_amdgcn_readlane((int)b, 0),
                                 (uint32_t)__builtin_amdgcn_readlane((int)b, 16)),
                      scalar_max((uint32_t)__builtin_amdgcn_readlane((int)b, 32),
                                 (uint32_t)__builtin_amdgcn_readlane((int)b, 48)));
}

// The running ceilings of a, b and v as one wavefront knows them (wave-uniform).
struct Ceilings {
    uint32_t Ea, Eb, Ev;
    __device__ __forceinline__ float scale_a() const { return pow2_field(259 - (int)Ea); }
    __device__ __forceinline__ float scale_b() const { return pow2_field(259 - (int)Eb); }
    __device__ __forceinline__ float scale_v() const { return pow2_field(259 - (int)Ev); }
    // exponent of the state's units, and of a chunk's output units (a x state)
    __device__ __forceinline__ int state_exp() const { return (int)(Eb + Ev) - 264; }
    __device__ __forceinline__ int out_exp() const { return (int)(Ea + Eb + Ev) - 396; }
};
typedef __attribute__((address_space(3))) uint32_t lds_u32_t;
// The slot of a position is that of its LDS buffer: words (a, b, v, unused).  The words of b
// and v hold ceilings that only ever rise (a stale one is harmless: it is below the running
// ceiling that every wavefront carries).  The word of a holds the ceiling of the rows of that
// one position, tagged with the position's number in the upper 24 bits, so that what the
// slot held three positions ago is always smaller and needs no clearing.
__device__ __forceinline__ void read_slot(const lds_u32_t *slots, int k, Ceilings &c) {
    const u32x4 s = *(const lds_vec4 *)(slots + 4 * k);
    c.Ea = max(kExpFloor, (uint32_t)__builtin_amdgcn_readfirstlane(s.x) & 0xffu);
    c.Eb = max(c.Eb, (uint32_t)__builtin_amdgcn_readfirstlane(s.y));
    c.Ev = max(c.Ev, (uint32_t)__builtin_amdgcn_readfirstlane(s.z));
}
// Lane maxima of the rows of position `pos` (slot k) against the ceilings of the position
// before it.  a: every row of 16 lanes enters the ceiling of its own values (one lane per row:
// four atomics on one word per wavefront, no trip through scalar registers).  b, v: whoever
// finds a value at or above the running ceiling raises the slot.
__device__ __forceinline__ void raise_slot(lds_u32_t *slots, int k, int pos, const Ceilings &c,
                                           float ma, float mb, float mv, int lane) {
    lds_u32_t *const s = slots + 4 * k;
    const uint32_t ea = ceiling_of(wave_max(ma));
    if (lane == 0)
        __hip_atomic_fetch_max(s + 0, ((uint32_t)(pos + 1) << 8) | ea, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    const bool over = mb >= pow2_field((int)c.Eb - 1) || mv >= pow2_field((int)c.Ev - 1);
    if (__builtin_amdgcn_ballot_w64(over) != 0) {
        const uint32_t eb = ceiling_of(wave_max(mb)), ev = ceiling_of(wave_max(mv));
        if (lane == 0) {
            if (eb > c.Eb) __hip_atomic_fetch_max(s + 1, eb, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (ev > c.Ev) __hip_atomic_fetch_max(s + 2, ev, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
}

// four bf16 values in two words -> the same values as fp32 bit patterns
__device__ __forceinline__ u32x4 widen_bf16_quad(const u32x4 r) {
    return u32x4{r.x << 16, r.x & 0xffff0000u, r.y << 16, r.y & 0xffff0000u};
}

// KS: groups of 32 rows of the state (1: a state of up to 32 rows, which skips the matrix
// instructions and fragment reads of the empty half).  MIX: rows of either element type, as
// ScanOperands::pad says scan by scan (false: all rows fp32).
template <int KS, bool MIX>
__global__ __launch_bounds__(768, 3) void scan_tph_kernel(uint32_t *__restrict__ ws_ptr, ScanArgs p) {
    constexpr int D = 64, F = 64;              // one block of state rows and of output columns
    constexpr int T = 512;                     // producer lanes (eight wavefronts)
    constexpr int PF = kTpAhead;               // chunks requested ahead
    constexpr int RBA = D * 2, RBV = F * 2;    // bytes per row of an fp16 piece tile
    constexpr int kTileA = kChunk * RBA, kTileV = kChunk * RBV;
    constexpr int kOffB = 2 * kTileA, kOffV = 4 * kTileA;
    constexpr int kBufBytes = 4 * kTileA + 2 * kTileV;
    constexpr int kTileP = kChunk * 64;        // Pt pieces: 32 rows (i) of 32 j
    constexpr int QA = D / 4, QV = F / 4;
    constexpr int LA = kChunk * QA / T, LV = kChunk * QV / T;
    static_assert(kChunk == 32 && T % QA == 0 && T % QV == 0, "shape");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool producer = wave >= 4;
    const int w = wave & 3;  // (consumers)

    __shared__ __align__(16) char pieces_mem[3 * kBufBytes];
    __shared__ __align__(16) char pt_mem[3 * 2 * kTileP];
    __shared__ __align__(16) uint32_t slot_mem[16];
    lds_char *const unit_pc = (lds_char *)pieces_mem;
    lds_char *const pt_pc = (lds_char *)pt_mem;
    lds_u32_t *const slots = (lds_u32_t *)slot_mem;

    // ---- which chain (as in scan_tp_kernel) ----
    const uint32_t nseg = (uint32_t)p.nseg;
    const uint32_t chains = (uint32_t)p.waves_per_scan / nseg;
    const uint32_t per_chain = (uint32_t)p.total_waves / chains;  // scans x segments
    const uint32_t full = (chains / 8u) * 8u;
    uint32_t which, chain;
    if (blockIdx.x < full * per_chain) {
        const uint32_t grp = blockIdx.x / (8u * per_chain), r = blockIdx.x % (8u * per_chain);
        which = r / 8u;
        chain = grp * 8u + r % 8u;
    } else {
        const uint32_t t = blockIdx.x - full * per_chain;
        which = t / (chains - full);
        chain = full + t % (chains - full);
    }
    const uint32_t virt = which / nseg;
    const uint32_t scan_id = virt / (uint32_t)p.tp_fblocks;
    const int fb = (int)(virt % (uint32_t)p.tp_fblocks);
    const int Dw = p.tp_d;                      // state rows: a and b are this wide
    const int fw = min(F, p.tp_f - F * fb);     // output columns of this block
    const ScanOperands &op = p.scan[scan_id];
    const bool REV = op.rev != 0;
    const int n = (int)(chain / (uint32_t)p.H), h = (int)(chain % (uint32_t)p.H);
    const int rows = (int)p.L;
    const int total_chunks = (rows + kChunk - 1) / kChunk;
    const bool exchange = p.tp_exchange != 0 && nseg > 1;
    gu32 *const hdr = (gu32 *)ws_ptr;
    gu32 *const flags = hdr + kHdrWords;
    const uint32_t chain_id = virt * chains + chain;  // over all scans of the launch
    int seg = (int)(which % nseg);
    __shared__ uint32_t order_sh;
    if (exchange) {
        if (tid == 0)
            order_sh = __hip_atomic_fetch_add(flags + kMaxWaves + chain_id, 1u, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        seg = (int)__builtin_amdgcn_readfirstlane(order_sh);
        if ((uint32_t)seg >= nseg) {  // the control block was not zero when the launch began
            if (tid == 0)
                __hip_atomic_store(hdr + kHdrError, 2u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }
    const int c0 = exchange ? seg * p.tp_seg_chunks : p.tp_start[seg];
    const int nchunks = min(total_chunks, exchange ? c0 + p.tp_seg_chunks : p.tp_start[seg + 1]);
    // the chunks walked for their state alone: so0 .. so0 + n1 - 1 (n1 a multiple of PF)
    const int so0 = exchange ? c0 : 0;
    const int n1 = exchange ? (seg + 1 < (int)nseg ? nchunks - c0 : 0) : c0;
    const int nwalk = n1 + (nchunks - c0);  // (position nwalk: a chunk of zeros)
    auto so_chunk = [&](int v) -> int { return exchange ? so0 + n1 - 1 - v : so0 + v; };
    auto walk_chunk = [&](int v) -> int { return v < n1 ? so_chunk(v) : c0 + (v - n1); };
    constexpr uint32_t kNoRow = 0x80000000u;  // an offset outside every descriptor
    auto chunk_row0 = [&](int c) -> int { return REV ? rows - kChunk * (c + 1) : kChunk * c; };
    if (tid < 16) slot_mem[tid] = 0;
    Ceilings ce{kExpFloor, kExpFloor, kExpFloor};
    // Position k of the walk goes through LDS buffer (B0 + k) % 3 (pieces, Pt and slot), with B0
    // such that the first chunk of the walk proper has buffer 0: the consumers' loop over
    // those chunks is unrolled three times and addresses LDS with immediate offsets.
    const int B0 = (3 - n1 % 3) % 3;
    auto next_buf = [](int b) -> int { return b == 2 ? 0 : b + 1; };
#ifdef FTC_TIMELINE
    // tuning aid: 32 time stamps per workgroup behind the pointer that the host passes in
    // p.key_len (FTC_STAMP_PTR), written by lane 0 of consumer 0 (0 .. 15) and of producer 0
    // (16 .. 31) in the fifth chunk of the walk proper
    typedef __attribute__((address_space(1))) uint64_t gu64;
    const bool stamp_on = p.key_len != nullptr && w == 0 && lane == 0;
    gu64 *const stamp_base = (gu64 *)p.key_len + blockIdx.x * 32 + (producer ? 16 : 0);
    // ... and behind those, 64 stamps per workgroup: consumer 0 after the barrier of every chunk
    gu64 *const chunk_stamps = (gu64 *)p.key_len + gridDim.x * 32 + blockIdx.x * 64;
#endif
    FTC_STAMP(14);  // workgroup under way
#ifdef FTC_TIMELINE
    if (stamp_on && !producer) chunk_stamps[0] = __builtin_amdgcn_s_memrealtime();
    if (stamp_on && !producer) stamp_base[12] = __builtin_amdgcn_s_memtime();
#endif

    if (producer) {
        // =========================== producers ===========================
        const int ptid = (wave - 4) * 64 + lane;
        const bool a_bf = MIX && (op.pad & kRowsBf16A), b_bf = MIX && (op.pad & kRowsBf16B),
                   v_bf = MIX && (op.pad & kRowsBf16V);
        const uint32_t a_es = a_bf ? 2 : 4, b_es = b_bf ? 2 : 4, v_es = v_bf ? 2 : 4;  // bytes
        const uint32_t a_slb = (uint32_t)op.a_sl * a_es, b_slb = (uint32_t)op.b_sl * b_es,
                       v_slb = (uint32_t)op.v_sl * v_es;
        const char *a_seg = (const char *)op.a + ((int64_t)n * op.a_sn + (int64_t)h * op.a_sh) * a_es;
        const char *b_seg = (const char *)op.b + ((int64_t)n * op.b_sn + (int64_t)h * op.b_sh) * b_es;
        const char *v_seg = (const char *)op.v +
                            ((int64_t)n * op.v_sn + (int64_t)h * op.v_sh + F * fb) * v_es;
        const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)a_seg, 0, (rows - 1) * a_slb + Dw * a_es, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t b_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)b_seg, 0, (rows - 1) * b_slb + Dw * b_es, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)v_seg, 0, (rows - 1) * v_slb + fw * v_es, kRsrcFlags);
        // One quad (four columns of one row) of every operand per lane and position.  Widths
        // that do not fill the block: a lane whose four columns lie beyond the width asks
        // outside the descriptor and cuts zeros (widths are multiples of 4).
        static_assert(LA == 1 && LV == 1 && QA == QV, "one quad per lane");
        const int prow = ptid / QA, pc4 = ptid % QA;
        const bool ab_in = 4 * pc4 < Dw;
        const bool v_in = 4 * pc4 < fw;
        const uint32_t a_goff = (uint32_t)prow * a_slb + 4u * a_es * pc4,
                       b_goff = (uint32_t)prow * b_slb + 4u * b_es * pc4,
                       v_goff = (uint32_t)prow * v_slb + 4u * v_es * pc4;
        const int a_waddr = TpSwizzle<RBA>::addr(prow, 8 * pc4),
                  b_waddr = TpSwizzle<RBA>::addr(prow, 2 * b_tile_column(4 * pc4)),
                  v_waddr = TpSwizzle<RBV>::addr(prow, 8 * pc4);
        struct Raw {  // (bf16 rows: the quad in the first two words)
            u32x4 a, b, v;
        };
        Raw raw[PF];
        // (MIX: the same two 8-byte requests whatever the type -- no branch around a request,
        // which would end the run of requests in flight; the second one of a bf16 quad asks
        // outside the descriptor)
        auto load_quad = [&](const __amdgpu_buffer_rsrc_t rs, uint32_t off, bool bf) -> u32x4 {
            if (!MIX) return __builtin_amdgcn_raw_buffer_load_b128(rs, off, 0, 0);
            const u32x2 lo = __builtin_amdgcn_raw_buffer_load_b64(rs, off, 0, 0);
            const u32x2 hi = __builtin_amdgcn_raw_buffer_load_b64(rs, bf ? kNoRow : off + 8u, 0, 0);
            return u32x4{lo.x, lo.y, hi.x, hi.y};
        };
        // (bf16 quads are widened in place, once, when the look-ahead first touches them: one
        // position later the cut finds fp32 bit patterns whatever the rows held)
        auto widen = [&](u32x4 &r, bool bf) {
            if (MIX && bf) r = widen_bf16_quad(r);
        };
        // Every request is made every time, whether its rows exist or not (a chunk walked for
        // its state alone needs no rows of a; positions past the end of the walk have no
        // rows): a request outside the descriptor costs no memory traffic and reads as zero,
        // and with a fixed number of requests per chunk the compiler can wait for the oldest
        // ones only.
        auto fetch = [&](Raw &r, int v) {  // v: position of the walk
            const int row0 = v < nwalk ? chunk_row0(walk_chunk(v)) : -2 * kChunk;
            const int row0_x = v >= n1 ? row0 : -2 * kChunk;
            // (the sums wrap: a chunk that starts before the first row has its later rows in place)
            r.a = load_quad(a_rs, ab_in ? a_goff + (uint32_t)row0_x * a_slb : kNoRow, a_bf);
            r.b = load_quad(b_rs, ab_in ? b_goff + (uint32_t)row0 * b_slb : kNoRow, b_bf);
            r.v = load_quad(v_rs, v_in ? v_goff + (uint32_t)row0 * v_slb : kNoRow, v_bf);
        };
        // the largest magnitudes of the rows of a position against the ceilings (rows that
        // were not asked for read as zeros); k: that position's slot
        auto look_ahead = [&](Raw &r, int k, int pos) {
            widen(r.a, a_bf), widen(r.b, b_bf), widen(r.v, v_bf);
            raise_slot(slots, k, pos, ce, max_abs4(r.a, 0.f), max_abs4(r.b, 0.f), max_abs4(r.v, 0.f), lane);
        };
        // A position of the walk goes to its LDS buffer through register set (position % PF).
        // The first n1 positions only feed the state: no piece of a.
        auto cut = [&](const Raw &r, int buf, bool own) {
            lds_char *const pc = unit_pc + buf * kBufBytes;
            if (own) cut_quad_to_lds(r.a, ce.scale_a(), pc, kTileA, a_waddr);
            cut_quad_to_lds(r.b, ce.scale_b(), pc + kOffB, kTileA, b_waddr);
            cut_quad_to_lds(r.v, ce.scale_v(), pc + kOffV, kTileV, v_waddr);
            if (!own) asm volatile("" ::"v"(r.a));
        };
#pragma unroll
        for (int j = 0; j < PF; j++) fetch(raw[j], j);
        wg_barrier();  // the slots are zero
        look_ahead(raw[0], B0, 0);
        wg_barrier();  // the slot of position 0 is complete
        // Barrier number k (k = 0: before the consumers' first position; k >= 1: in the
        // middle of position k - 1) finds position k cut and the slot of position k + 1
        // complete.  The last one finds a chunk of zeros.
        int buf = B0;
        auto step = [&](int v, int j, bool own) {
            if (own && v == n1 + 4) FTC_STAMP(0);
            read_slot(slots, buf, ce);
            look_ahead(raw[(j + 1) % PF], next_buf(buf), v + 1);
            if (own && v == n1 + 4) FTC_STAMP(1);
            cut(raw[j], buf, own);
            if (own && v == n1 + 4) FTC_STAMP(2);
            fetch(raw[j], v + PF);
            buf = buf == 2 ? 0 : buf + 1;
            if (own && v == n1 + 4) FTC_STAMP(3);
            wg_barrier();
            __builtin_amdgcn_sched_barrier(0);  // one chunk at a time, in this order
            if (own && v == n1 + 4) FTC_STAMP(4);
        };
        for (int v = 0; v < n1; v += PF) {
#pragma unroll
            for (int j = 0; j < PF; j++) step(v + j, j, false);
        }
        // (whole trips in the loop, the rest after it)
        int v = n1;
        for (; v + PF <= nwalk + 1; v += PF) {
#pragma unroll
            for (int j = 0; j < PF; j++) step(v + j, j, true);
        }
#pragma unroll
        for (int j = 0; j < PF - 1; j++) {
            if (v + j > nwalk) return;
            read_slot(slots, buf, ce);
            look_ahead(raw[(j + 1) % PF], next_buf(buf), v + j + 1);
            cut(raw[j], buf, true);
            buf = buf == 2 ? 0 : buf + 1;
            wg_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }

    // =========================== consumers ===========================
    const int ln = lane & 15, g = lane >> 4;
    const bool o_bf = MIX && (op.pad & kRowsBf16Out);
    const uint32_t o_es = o_bf ? 2 : 4;  // bytes
    const uint32_t o_slb = (uint32_t)op.o_sl * o_es;
    char *o_seg = (char *)op.out + ((int64_t)n * op.o_sn + (int64_t)h * op.o_sh + F * fb) * o_es;
    const __amdgpu_buffer_rsrc_t o_rs =
        __builtin_amdgcn_make_buffer_rsrc((void *)o_seg, 0, (rows - 1) * o_slb + fw * o_es, kRsrcFlags);
    // Pt quadrant of this wavefront (see scan_tp_kernel)
    const int jh = w == 0 ? 0 : w == 1 ? 1 : ((w == 2) == REV ? 1 : 0);
    const int ih = w == 0 ? 0 : w == 1 ? 1 : 1 - jh;
    int a_addr[2][2], b_addr[2][2];  // [local i tile][ks], [ks][u]
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
        for (int x = 0; x < 2; x++)
            a_addr[x][ks] = TpSwizzle<RBA>::addr(16 * (x ^ ih) + ln, 2 * (32 * ks + 8 * g));
#pragma unroll
        for (int u = 0; u < 2; u++)
            b_addr[ks][u] = kOffB + TpSwizzle<RBA>::addr(
                                        16 * jh + ln, 2 * b_tile_column(32 * ks + 8 * g + 4 * u));
    }
    int bt_addr[4][2], vt_addr[2];
#pragma unroll
    for (int u2 = 0; u2 < 2; u2++) {
        const int row = 8 * g + (ln >> 2) + 4 * u2;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
            bt_addr[dt][u2] = kOffB + TpSwizzle<RBA>::addr(
                row, 2 * b_tile_column(32 * (dt / 2) + 4 * (dt % 2) + 8 * (ln & 3)));
        vt_addr[u2] = kOffV + TpSwizzle<RBV>::addr(row, 2 * (16 * w + 4 * (ln & 3)));
    }
    const int pt_waddr = TpSwizzle<64>::addr(16 * ih + ln, 2 * (16 * jh + 4 * g));
    int pt_raddr[2];
#pragma unroll
    for (int x = 0; x < 2; x++) pt_raddr[x] = TpSwizzle<64>::addr(16 * (x ^ ih) + ln, 16 * g);
    uint32_t keep[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int j = 16 * jh + 4 * g + r, i = 16 * ih + ln;
        keep[r] = (REV ? (j >= i) : (j <= i)) ? 0xffffffffu : 0u;
        asm volatile("" : "+v"(keep[r]));
    }
    uint32_t o_lane[2];
#pragma unroll
    for (int x = 0; x < 2; x++)
        o_lane[x] = (uint32_t)(16 * (x ^ ih) + ln) * o_slb + o_es * (16 * w + 4 * g);
    const bool o_in = 16 * w + 4 * g < fw;  // (columns beyond the width are not stored)

    constexpr int NT = 2 * KS;  // state tiles of 16 rows
    f32x4 S[4];                 // the slab, in units of 2^Ucur
#pragma unroll
    for (int dt = 0; dt < 4; dt++) S[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    int Ucur = 0;
    constexpr int kPa[3] = {1, 0, 0}, kPb[3] = {0, 1, 0};  // piece products, smallest first
    auto state_row = [&](int dt, int r) -> int { return 32 * (dt / 2) + 8 * g + 4 * (dt % 2) + r; };
    const bool st_in = 16 * w + ln < fw;
    auto scale_state = [&](int e) {  // S <- S 2^e
#pragma unroll
        for (int dt = 0; dt < NT; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++) S[dt][r] = __builtin_amdgcn_ldexpf(S[dt][r], e);
    };
    auto add_caller_state = [&]() {  // in units of 2^Ucur
        const float *base =
            op.s0 + (int64_t)n * op.s0_sn + (int64_t)h * op.s0_sh + F * fb + 16 * w + ln;
#pragma unroll
        for (int dt = 0; dt < NT; dt++) {
            float x[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int d = state_row(dt, r);
                const bool in = st_in && d < Dw;
                x[r] = *(in ? base + (int64_t)d * op.s0_sd : op.s0);
                x[r] = in ? __builtin_amdgcn_ldexpf(x[r], -Ucur) : 0.f;
            }
            S[dt] += f32x4{x[0], x[1], x[2], x[3]};
        }
    };

    Frag af[2][2][2], bfr[2][2], bt[4][2], vf[2];
    // row-major fragment number i of a chunk (12: b for the quadrant first, then a)
    auto rm_frag = [&](const lds_char *pc, int i) {
        const int k = i % 2, ks = (i / 2) % 2, x = i / 4;
        if (ks >= KS) return;
        if (x == 0)
            bfr[ks][k] = lds_frag8x2(pc + k * kTileA + b_addr[ks][0], pc + k * kTileA + b_addr[ks][1]);
        else
            af[x - 1][ks][k] = lds_frag16(pc + k * kTileA + a_addr[x - 1][ks]);
    };
    // position-major fragment number i of a chunk (10: v first, then b^T tile by tile)
    auto tr_frag_into = [&](Frag (&btx)[4][2], Frag (&vfx)[2], const lds_char *pc, int i) {
        if (i >= 2 && (i - 2) / 4 >= KS) return;  // tiles 2, 3: rows 32 .. 63
        if (i < 2)
            vfx[i] = lds_frag_tr(pc + i * kTileV + vt_addr[0], pc + i * kTileV + vt_addr[1]);
        else {
            const int dt = (i - 2) / 2, k = (i - 2) % 2;
            btx[dt][k] = lds_frag_tr(pc + k * kTileA + bt_addr[dt][0], pc + k * kTileA + bt_addr[dt][1]);
        }
    };
    int buf = B0;  // LDS buffer of the chunk at hand
    wg_barrier();  // the slots are zero
    wg_barrier();  // the slot of position 0 is complete
    wg_barrier();  // barrier 0: position 0 is cut
    read_slot(slots, B0, ce);
    Ucur = ce.state_exp();
    if (op.s0 && !exchange) add_caller_state();
    if (n1 > 0) {
        // ---- the first n1 positions of the walk: state update only ----
        // The loop is skewed by one position: while the matrix instructions of position k - 1
        // run, the fragments of position k arrive in the other set of registers.
        int U_prev = Ucur;                 // units of the fragments about to be multiplied
        Frag bt2[4][2] = {}, vf2[2] = {};  // (the first round multiplies zeros)
        for (int c = 0; c < n1; c += PF) {
#pragma unroll
            for (int j = 0; j < PF; j++) {
                const lds_char *pc = unit_pc + buf * kBufBytes;
                read_slot(slots, buf, ce);  // the ceilings of position c + j
                if (U_prev != Ucur) {       // the ceilings rose: the state shrinks
                    scale_state(Ucur - U_prev);
                    Ucur = U_prev;
                }
#pragma unroll
                for (int i = 0; i < 12; i++) {
                    const bool rows_exist = (i % 4) / 2 < KS;
                    if (j % 2 == 0) {
                        if (rows_exist) S[i % 4] = mfma16h(bt2[i % 4][kPa[i / 4]], vf2[kPb[i / 4]], S[i % 4]);
                        if (i < 10) tr_frag_into(bt, vf, pc, i);
                    } else {
                        if (rows_exist) S[i % 4] = mfma16h(bt[i % 4][kPa[i / 4]], vf[kPb[i / 4]], S[i % 4]);
                        if (i < 10) tr_frag_into(bt2, vf2, pc, i);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                U_prev = ce.state_exp();
                buf = next_buf(buf);
                wg_barrier();
#ifdef FTC_TIMELINE
                if (stamp_on && c + j < 30) chunk_stamps[32 + c + j] = __builtin_amdgcn_s_memrealtime();
#endif
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // the last of these positions (n1 is even: its fragments are in the second set)
        if (U_prev != Ucur) {
            scale_state(Ucur - U_prev);
            Ucur = U_prev;
        }
#pragma unroll
        for (int i = 0; i < 12; i++) {
            if ((i % 4) / 2 < KS) S[i % 4] = mfma16h(bt2[i % 4][kPa[i / 4]], vf2[kPb[i / 4]], S[i % 4]);
            rm_frag(unit_pc + buf * kBufBytes, i);  // our own first chunk is cut
            __builtin_amdgcn_sched_barrier(0);
        }
        read_slot(slots, buf, ce);  // the ceilings of our own first chunk
    } else {
#pragma unroll
        for (int i = 0; i < 12; i++) rm_frag(unit_pc, i);
    }
    if (exchange) {
        // ---- the sum of this segment's rows goes out, the state before the segment comes in ----
        const uint32_t total_units = (uint32_t)p.total_waves;
        gfloat *const sums = (gfloat *)(hdr + kControlBytes / 4);
        StateExchange<1, 1> xch(flags, sums, 4u * total_units,
                                (uint32_t)w * total_units + chain_id * nseg + (uint32_t)seg, seg,
                                (int)nseg, p.group, lane);
        f32x16 Sx[1][1], X[1][1];
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                Sx[0][0][4 * dt + r] = dt < NT ? __builtin_amdgcn_ldexpf(S[dt][r], Ucur) : 0.f;
        if (n1 > 0) xch.publish_sum(Sx);
        xch.gather(Sx, X);
        if (xch.failed && lane == 0)
            __hip_atomic_store(hdr + kHdrError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // the units of the first chunk of the second pass (its ceilings are already known)
        Ucur = ce.state_exp();
#pragma unroll
        for (int dt = 0; dt < NT; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++) S[dt][r] = __builtin_amdgcn_ldexpf(X[0][0][4 * dt + r], -Ucur);
        if (op.s0) add_caller_state();
    }
    // ---- the walk proper ----
    // `ce` holds the ceilings of the chunk at hand, Ucur the units of S.  dU <= 0: the
    // state's units rise by -dU with this chunk (S is rescaled once all of it has been cut).
    int dU = Ucur - ce.state_exp();
    int s = 0;  // S is cut as S 2^(dU - s)
    auto lane_max_state = [&]() -> float {
        float m = 0.f;
#pragma unroll
        for (int dt = 0; dt < NT; dt++)
            m = fmaxf(fmaxf(fmaxf(fabsf(S[dt][0]), fabsf(S[dt][1])), fmaxf(fabsf(S[dt][2]), fabsf(S[dt][3]))), m);
        return m;
    };
    {
        if (dU != 0) {
            scale_state(dU);
            Ucur -= dU;
            dU = 0;
        }
        const float m = lane_max_state();
        while (s < 100 && __builtin_amdgcn_ballot_w64(m > pow2_field(127 + 14 + s)) != 0) s++;
    }
    float kappa = pow2_field(127 + dU - s);  // scale of the cut of S
    bool plain_cut = dU - s == 0;            // ... which is one as a rule: a cheaper cut
    int s_cut = s;                            // ... and the s that went into it
    float mS = 0.f;                           // largest |S| seen while cutting
    Frag sf[2][2];
    // tile 2 ks + u of S_w -> words 2 u, 2 u + 1 of the fragments of k-step ks
    // (`track`: also note the largest magnitude.  One state in three is looked at, the one
    // cut for the chunks in LDS buffer 0: s then rises when an element exceeds 2^(14 + s)
    // units, three more chunks add at most 3 x 2^13, and 2^14 + 3 x 2^13 is below what fp16
    // holds.)
    auto cut_s = [&](int ks, int u, bool track) {
        const f32x4 x = S[2 * ks + u];
        if (track)
            mS = fmaxf(fmaxf(fmaxf(fabsf(x[0]), fabsf(x[1])), fmaxf(fabsf(x[2]), fabsf(x[3]))), mS);
        if (plain_cut)
            cut_quad_f16_unscaled(x[0], x[1], x[2], x[3], sf[ks][0].w[2 * u], sf[ks][0].w[2 * u + 1],
                                  sf[ks][1].w[2 * u], sf[ks][1].w[2 * u + 1]);
        else
            cut_quad_f16(x[0], x[1], x[2], x[3], kappa, sf[ks][0].w[2 * u], sf[ks][0].w[2 * u + 1],
                         sf[ks][1].w[2 * u], sf[ks][1].w[2 * u + 1]);
    };
    cut_s(0, 0, true);
    cut_s(0, 1, true);

    // Ot_w of the chunk before in the units of that chunk (exponent Xo), and where its rows
    // go (before the first chunk: nowhere)
    f32x4 O[2];
#pragma unroll
    for (int x = 0; x < 2; x++) O[x] = f32x4{0.f, 0.f, 0.f, 0.f};
    int Xo = 0;
    uint32_t o_off = 0x80000000u;
    auto store_rows = [&](int x) {
        const float y0 = __builtin_amdgcn_ldexpf(O[x][0], Xo), y1 = __builtin_amdgcn_ldexpf(O[x][1], Xo),
                    y2 = __builtin_amdgcn_ldexpf(O[x][2], Xo), y3 = __builtin_amdgcn_ldexpf(O[x][3], Xo);
        const uint32_t at = o_in ? o_off + o_lane[x] : kNoRow;
        if (!MIX) {
            buffer_store_out(o_rs, at, y0, y1, y2, y3, (float *)nullptr);
        } else if (o_bf) {  // (a branch that the whole launch takes one way: no request hangs on it)
            const u32x2 packed = {pack_bf16_rne(y0, y1), pack_bf16_rne(y2, y3)};
            __builtin_amdgcn_raw_buffer_store_b64(packed, o_rs, at, 0, 0);
        } else {
            buffer_store_out(o_rs, at, y0, y1, y2, y3, (float *)nullptr);
        }
    };
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    // One chunk, in LDS buffer B (a compile-time number, so that every LDS access of the body
    // has its buffer in the instruction's immediate offset).  Sums that end in one place are
    // chained through one accumulator, with other matrix instructions in between: Ot_w =
    // (S_w^T a^T) 2^s + v_w^T Pt needs no addition at all while s = 0, which is the rule.
    auto chunk_body = [&](int c, auto buffer_number) {
        constexpr int B = decltype(buffer_number)::value, BN = (B + 1) % 3;
        const lds_char *pc = unit_pc + B * kBufBytes;
        const lds_char *pn = unit_pc + BN * kBufBytes;
        lds_char *const ptc = pt_pc + B * (2 * kTileP);
        Frag pf[2][2];
        f32x4 P;  // (cleared by the first matrix instruction of its sum)
        if (c == c0 + 4) FTC_STAMP(0);
        __builtin_amdgcn_sched_barrier(0);
        // phase 1: (1) the quadrant in turn with (2b) Ot_w = S_w^T a^T for rows 0 .. 31 of
        // the state; underneath: the rows of the chunk before go out, tiles 2, 3 of S_w are
        // cut into pieces, the position-major reads
#pragma unroll
        for (int i = 0; i < 6; i++) {
            const int m = i % 3, ks = i / 3, x = i % 2, mo = i / 2;
            if (i == 0) store_rows(0);
            if (i == 1) store_rows(1);
            if (ks < KS) P = mfma16h(bfr[ks][kPa[m]], af[0][ks][kPb[m]], i == 0 ? zero : P);
            O[x] = mfma16h(sf[0][kPa[mo]], af[x][0][kPb[mo]], mo == 0 ? zero : O[x]);
            if ((i == 1 || i == 3) && KS > 1) cut_s(1, i / 2, B == 0);
            tr_frag_into(bt, vf, pc, i);
            if (i < 4) tr_frag_into(bt, vf, pc, 6 + i);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (c == c0 + 4) FTC_STAMP(1);
        // all of S is cut: it takes the units of this chunk, and s follows its size
        if (dU != 0) {
            scale_state(dU);
            mS = __builtin_amdgcn_ldexpf(mS, dU);
            s = max(0, s + dU);
            Ucur -= dU;
        }
        if (B == 0) {
            while (s < 100 && __builtin_amdgcn_ballot_w64(mS > pow2_field(127 + 14 + s)) != 0) s++;
            mS = 0.f;
        }
        if (c == c0 + 4) FTC_STAMP(2);
        __builtin_amdgcn_sched_barrier(0);
        // phase 2: (2b) for rows 32 .. 63 in turn with (3) S_w += b^T v_w for tiles 0 and 1;
        // underneath: the quadrant is masked, cut and handed to the others
#pragma unroll
        for (int i = 0; i < 6; i++) {
            const int x = i % 2, m = i / 2;
            if (KS > 1) O[x] = mfma16h(sf[1][kPa[m]], af[x][1][kPb[m]], O[x]);
            S[i % 2] = mfma16h(bt[i % 2][kPa[m]], vf[kPb[m]], S[i % 2]);
            if (i == 1) {
                uint32_t h0, l0, h1, l1;
                cut_quad_f16_unscaled(__uint_as_float(__float_as_uint(P[0]) & keep[0]),
                                      __uint_as_float(__float_as_uint(P[1]) & keep[1]),
                                      __uint_as_float(__float_as_uint(P[2]) & keep[2]),
                                      __uint_as_float(__float_as_uint(P[3]) & keep[3]), h0, h1, l0, l1);
                const u32x2 wh = {h0, h1}, wl = {l0, l1};
                *(lds_vec2 *)(ptc + pt_waddr) = wh;
                *(lds_vec2 *)(ptc + kTileP + pt_waddr) = wl;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (c == c0 + 4) FTC_STAMP(4);
        wg_barrier();
        if (c == c0 + 4) FTC_STAMP(5);
#ifdef FTC_TIMELINE
        if (stamp_on && c - c0 < 30) chunk_stamps[c - c0 + 1] = __builtin_amdgcn_s_memrealtime();
#endif
        // All of Pt is in LDS, the next chunk is cut and its slot complete.
        // phase 3: (3) for tiles 2 and 3, then (2a) Ot_w += v_w^T Pt; underneath: the next
        // chunk's row-major fragments are requested and tiles 0, 1 of S_w cut into pieces
#pragma unroll
        for (int x = 0; x < 2; x++)
#pragma unroll
            for (int k = 0; k < 2; k++) pf[x][k] = lds_frag16(ptc + k * kTileP + pt_raddr[x]);
        const int Xc = ce.out_exp();
        const u32x4 slot_next = *(const lds_vec4 *)(slots + 4 * BN);
        if (s_cut != 0) {  // (rare: the state has grown beyond 2^14 units)
            const float r_cut = pow2_field(127 + s_cut);
            O[0] *= r_cut;
            O[1] *= r_cut;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 6; i++) {
            const int m = i / 2;
            if (KS > 1) S[2 + i % 2] = mfma16h(bt[2 + i % 2][kPa[m]], vf[kPb[m]], S[2 + i % 2]);
            rm_frag(pn, 2 * i);
            rm_frag(pn, 2 * i + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        // the ceilings of the next chunk
        ce.Ea = max(kExpFloor, (uint32_t)__builtin_amdgcn_readfirstlane(slot_next.x) & 0xffu);
        ce.Eb = max(ce.Eb, (uint32_t)__builtin_amdgcn_readfirstlane(slot_next.y));
        ce.Ev = max(ce.Ev, (uint32_t)__builtin_amdgcn_readfirstlane(slot_next.z));
        dU = Ucur - ce.state_exp();
        kappa = pow2_field(127 + dU - s);
        plain_cut = dU - s == 0;
        s_cut = s;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 6; i++) {
            const int x = i % 2, m = i / 2;
            O[x] = mfma16h(vf[kPa[m]], pf[x][kPb[m]], O[x]);
            if (i == 1 || i == 3) cut_s(0, i / 2, BN == 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        o_off = (uint32_t)chunk_row0(c) * o_slb;
        Xo = Xc;
        if (c == c0 + 4) FTC_STAMP(6);
    };
    {
        int c = c0;
        for (; c + 3 <= nchunks; c += 3) {
            chunk_body(c, std::integral_constant<int, 0>());
            chunk_body(c + 1, std::integral_constant<int, 1>());
            chunk_body(c + 2, std::integral_constant<int, 2>());
        }
        if (c < nchunks) chunk_body(c++, std::integral_constant<int, 0>());
        if (c < nchunks) chunk_body(c++, std::integral_constant<int, 1>());
    }
    store_rows(0);
    store_rows(1);
    FTC_STAMP(15);  // last rows on their way
#ifdef FTC_TIMELINE
    if (stamp_on) stamp_base[13] = __builtin_amdgcn_s_memtime();
#endif
    if (op.s_out && seg == (int)nseg - 1) {
        float *base =
            op.s_out + (int64_t)n * op.so_sn + (int64_t)h * op.so_sh + F * fb + 16 * w + ln;
#pragma unroll
        for (int dt = 0; dt < NT; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int d = state_row(dt, r);
                if (st_in && d < Dw) base[(int64_t)d * op.so_sd] = __builtin_amdgcn_ldexpf(S[dt][r], Ucur);
            }
    }
    // the last consumer of the launch leaves the control block zeroed
    if (exchange) {
        const uint32_t total_units = (uint32_t)p.total_waves;
        uint32_t done = 0;
        if (lane == 0)
            done = __hip_atomic_fetch_add(hdr + kHdrDone, 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
        done = __builtin_amdgcn_readfirstlane(done);
        if (done == 4u * total_units - 1) {
            for (uint32_t i = lane; i < 4u * total_units; i += kWave)
                __hip_atomic_store(flags + i, kFlagEmpty, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            for (uint32_t i = lane; i < total_units / nseg; i += kWave)
                __hip_atomic_store(flags + kMaxWaves + i, 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0)
                __hip_atomic_store(hdr + kHdrDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace mfma
}  // namespace ftc
