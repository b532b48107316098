// Workgroup form of the MFMA causal scan for gfx950, all-fp32 rows.
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (REV: j >= l)
//
// Same mathematics, piece split, chunking and state exchange as ftc_mfma_kernel.h.  What
// differs is who does what.  A workgroup has eight wavefronts: four that only feed the matrix
// cores ("consumers", wavefronts 0..3) and four that only fetch rows and cut them into bf16
// pieces ("producers", wavefronts 4..7).  The hardware places wavefronts i and i + 4 of a
// workgroup on the same SIMD, so every SIMD holds one consumer and one producer and the
// vector ALU work of cutting runs under the other wavefront's matrix instructions.
//
//  * A unit of work is one (chain, L-segment).  A unit belongs to NW = F / 32 consumers and
//    NW producers; a workgroup carries NS = 4 / NW units side by side (two for F = 64).
//    Consumer w of a unit owns the output columns 32 w .. 32 w + 31: its slab of the D x F
//    state (D / 2 registers), its columns of v and of the output.
//  * The producers of a unit fetch the rows of a chunk with 16-byte loads, cut every fp32
//    value into its three bf16 pieces (exact, see ftc_mfma_kernel.h) and write the pieces as
//    three row-major bf16 tiles per operand into LDS, one chunk ahead of the consumers
//    (two buffers, one workgroup barrier per chunk).
//  * Consumers read fragments whose contraction index runs along a row (a; b for
//    Pt = b a^T) with 16-byte LDS reads, and fragments whose contraction index runs along
//    the chunk (b^T and v for the state update, v^T for Ot += v^T Pt) with
//    ds_read_b64_tr_b16, which hands every lane four values of one column: within 16 lanes,
//    lane i receives element i % 4 of the 8 bytes addressed by lanes i / 4, 4 + i / 4,
//    8 + i / 4 and 12 + i / 4.
//
// Register layouts of a consumer (32x32x16 MFMA; lane = (ln = lane % 32, g = lane / 32)):
//  * k-slot t of lane group g in a k-step of 16 carries contraction index 8 g + t when the
//    index runs along a row (natural order), and chunk position 8 (t / 4) + 4 g + t % 4 when
//    it runs along the chunk (the order in which Pt leaves the accumulator).
//  * State tile dt: register r of lane (ln, g) is S[d][f] with f = 32 w + ln and
//    d = 32 dt + 16 (r / 8) + 8 g + r % 8, so that registers 8 k .. 8 k + 7 are the A operand
//    of k-step 2 dt + k in natural order.  The b^T fragments of the state update are read
//    in the matching column order.
//
// All units of a workgroup pass the same barriers, so every loop runs for the largest chunk
// count among them; a unit that has run out of chunks (or does not exist: the last
// workgroup of a scan may have fewer units) only keeps time.
//
// NORM = true is causally masked linear attention in one pass over the rows
// (fast_transformers/attention/causal_linear_attention.py:71-104 with the feature map of
// feature_maps/base.py:71-73):
//
//   out[c, l, :] = sum_{j <= l} (phi(a_l) . phi'(b_j)) v_j  /  (phi(a_l) . sum_{j <= l} phi'(b_j) + eps)
//   phi(x) = x > 0 ? x + 1 : exp(x)   (= elu(x) + 1);   phi'(b_j) = phi(b_j) if j < key_len[n] else 0
//
//  * The producers apply phi to the rows of a and b as they cut them, and zero the rows of b
//    at or beyond the key length (and beyond the end of the segment, where phi(0) = 1 would
//    otherwise enter).
//  * The denominator is the same scan with a column of ones for values.  A unit gets one
//    more consumer (w = F / 32) whose "values" are a constant tile in LDS: column 0 one,
//    columns 1 .. 31 zero.  Its state is sum phi'(b_j) (in column 0), and row 0 of its Ot is
//    the denominator of the chunk's 32 positions, which it leaves in LDS before the
//    barrier that ends the chunk.  The other consumers hold their Ot across that barrier,
//    divide, and store.  With F = 64 a unit takes three of the four consumers of a
//    workgroup and the fourth idles (one unit per workgroup); with F = 32 there are two
//    units of two consumers each.
#pragma once
#include "ftc_mfma_dma_kernel.h"

namespace ftc {
namespace mfma {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// XOR swizzle of a bf16 piece tile with rows of RB bytes (64, 128 or 256): 16-byte slot p of
// row r sits at slot p ^ key(r).  The keys make three access patterns free of bank
// conflicts: 16-byte reads of one slot column over 16 consecutive rows (row-major
// fragments), the transposing reads (4 consecutive rows x 64 bytes per 32 lanes), and
// the producers' 8-byte writes of whole rows.
template <int RB>
struct PieceSwizzle {
    static constexpr int kSlots = RB / 16;
    __device__ static __forceinline__ int key(int r) {
        if (RB == 64) return (r >> 2) & 3;
        if (RB == 128) return (((r >> 1) & 1) << 2) | ((r >> 2) & 3);
        return ((r & 3) << 2) | ((r >> 2) & 3);
    }
    // byte address inside the tile of logical byte `off` of row `row`
    __device__ static __forceinline__ int addr(int row, int off) {
        return (row * kSlots + ((off >> 4) ^ key(row))) * 16 + (off & 15);
    }
};

__device__ __forceinline__ Frag lds_frag16(const lds_char *p) {
    const u32x4 r = *(const lds_vec4 *)p;
    return Frag{{r.x, r.y, r.z, r.w}};
}
// k-slots 0..3 from the transposing read at p0, 4..7 from the one at p1
__device__ __forceinline__ Frag lds_frag_tr(const lds_char *p0, const lds_char *p1) {
    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                                   (lds_s16x4 *)p0));
    const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                                   (lds_s16x4 *)p1));
    return Frag{{lo.x, lo.y, hi.x, hi.y}};
}

// Tuning aid: with -DFTC_TIMELINE the first consumer of every unit records when it passes the
// marked points (s_memrealtime ticks) behind the state slots of the workspace, 16 words per
// unit; the host side then reserves that room.
#ifdef FTC_TIMELINE
#define FTC_STAMP(i)                                                                  \
    do {                                                                              \
        if (stamp_on) stamp_base[(i)] = __builtin_amdgcn_s_memrealtime();             \
    } while (0)
#else
#define FTC_STAMP(i) \
    do {             \
    } while (0)
#endif

// Workgroup barrier that waits for this wavefront's LDS traffic only: rows requested from
// memory for a later chunk stay in flight across it (__syncthreads would wait for them).
__device__ __forceinline__ void wg_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// split_pair<3> for a wavefront that also feeds the matrix cores.  v_dot2c_f32_bf16, which
// split_pair uses to subtract a piece, does not issue while a matrix instruction of the same
// wavefront is in flight (measured: each one adds its full 2.5 ns to a 14 ns MFMA), whereas
// v_and_b32, v_sub_f32 and v_perm_b32 do (six of them cost 2.7 ns together).  Here the
// remainder is x - (x & 0xffff0000): one more instruction per value and piece, all hidden.
__device__ __forceinline__ void split_pair_under_mfma(float x0, float x1, uint32_t (&out)[3]) {
#pragma unroll
    for (int p = 0; p < 3; p++) {
        out[p] = pack_hi16(x0, x1);
        if (p + 1 < 3) {
            x0 = x0 - __uint_as_float(__float_as_uint(x0) & 0xffff0000u);
            x1 = x1 - __uint_as_float(__float_as_uint(x1) & 0xffff0000u);
        }
    }
}

// elu(x) + 1 = x + 1 for x > 0, exp(x) otherwise (NaN stays NaN, as in the reference's
// elu(x) + 1).  For x <= 0 the exponent x log2(e) is rounded once, which costs at most
// |x| 2^-24 ln 2 of relative accuracy -- in absolute terms never more than
// 2^-24 ln 2 max_x |x| e^x = 1.6e-8, a fraction of the rounding of a feature near one.
__device__ __forceinline__ float feature_phi(float x) {
    return x > 0.f ? x + 1.f : __builtin_amdgcn_exp2f(x * 1.44269502f);
}
// the feature map on four values of a row
__device__ __forceinline__ u32x4 feature_quad(const u32x4 raw) {
    u32x4 r;
    r.x = __float_as_uint(feature_phi(__uint_as_float(raw.x)));
    r.y = __float_as_uint(feature_phi(__uint_as_float(raw.y)));
    r.z = __float_as_uint(feature_phi(__uint_as_float(raw.z)));
    r.w = __float_as_uint(feature_phi(__uint_as_float(raw.w)));
    return r;
}

// Four consecutive fp32 values of a row -> 8 bytes of each of the three piece tiles.
__device__ __forceinline__ void split_quad_to_lds(const u32x4 raw, lds_char *tile, int piece_bytes,
                                                  int addr) {
    uint32_t lo[3], hi[3];
    split_pair_under_mfma(__uint_as_float(raw.x), __uint_as_float(raw.y), lo);
    split_pair_under_mfma(__uint_as_float(raw.z), __uint_as_float(raw.w), hi);
#pragma unroll
    for (int pc = 0; pc < 3; pc++) {
        const u32x2 w = {lo[pc], hi[pc]};
        *(lds_vec2 *)(tile + pc * piece_bytes + addr) = w;
    }
}

// The caller's state <-> the slab registers of a consumer (layout in the file header).
template <int DT>
__device__ __forceinline__ void wg_add_caller_state(const float *base, int64_t row_stride, int f,
                                                    int g, f32x16 (&S)[DT]) {
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int d = 32 * dt + 16 * (r / 8) + 8 * g + (r % 8);
            S[dt][r] += base[(int64_t)d * row_stride + f];
        }
}
template <int DT>
__device__ __forceinline__ void wg_store_caller_state(float *base, int64_t row_stride, int f, int g,
                                                      const f32x16 (&S)[DT]) {
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int d = 32 * dt + 16 * (r / 8) + 8 * g + (r % 8);
            base[(int64_t)d * row_stride + f] = S[dt][r];
        }
}

// Which unit a (workgroup, slot) pair works on.  In ScanArgs the counts are per unit here:
// waves_per_scan / total_waves count units, and the flag words and state slots of consumer w
// of the unit with ticket t are those of "ticket" w * total_waves + t.
//
// Workgroups are dispatched round-robin over the 8 XCDs.  They are numbered so that
// workgroup i of every scan of the launch lands on the same XCD at about the same time
// (groups of 8 consecutive workgroups per scan).  Returns false for a slot past the last
// unit of its scan.
template <int NS>
__device__ __forceinline__ bool unit_request(const ScanArgs &p, gu32 *flags, int slot,
                                             bool take_ticket, Segment &s, uint32_t &order) {
    const uint32_t ups = (uint32_t)p.waves_per_scan;  // units per scan
    const uint32_t bps = (ups + NS - 1) / NS;         // workgroups per scan
    const uint32_t nscans = (uint32_t)p.total_waves / ups;
    const uint32_t full = (bps / 8u) * 8u;
    uint32_t block_in_scan;
    if (blockIdx.x < full * nscans) {
        const uint32_t grp = blockIdx.x / (8u * nscans), r = blockIdx.x % (8u * nscans);
        s.scan_id = r / 8u;
        block_in_scan = grp * 8u + r % 8u;
    } else {
        const uint32_t t = blockIdx.x - full * nscans;
        s.scan_id = t / (bps - full);
        block_in_scan = full + t % (bps - full);
    }
    const uint32_t unit_in_scan = block_in_scan * NS + (uint32_t)slot;
    order = 0;
    s.chain_slot0 = 0;
    s.rev = false;
    if (unit_in_scan >= ups) return false;
    const uint32_t vunit = s.scan_id * ups + unit_in_scan;  // unit id in scan-major order
    const uint32_t my_chain = vunit / (uint32_t)p.nseg;
    s.chain_slot0 = my_chain * (uint32_t)p.nseg;
    s.rev = p.scan[s.scan_id].rev != 0;
    order = vunit - s.chain_slot0;  // a single segment per chain needs no ticket
    if (p.nseg > 1 && take_ticket)
        order = __hip_atomic_fetch_add(flags + kMaxWaves + my_chain, 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

template <int D, int F, bool NORM>
__global__ __launch_bounds__(512, 2) void scan_wg_kernel(uint32_t *__restrict__ ws_ptr,
                                                         ScanArgs p) {
    constexpr int NWV = F / 32;               // consumers of a unit that own value columns
    constexpr int NW = NWV + (NORM ? 1 : 0);  // consumers per unit
    constexpr int NS = 4 / NW;                // units per workgroup
    constexpr int NP = 4 / NS;                // producers per unit
    constexpr int T = 64 * NP;                // producer lanes per unit
    constexpr int kOnesTile = kChunk * 64;    // bytes of a piece tile of the constant values
    constexpr int PF = NORM ? 4 : 2;          // chunks requested ahead by the producers
    constexpr int DT = D / 32;          // state tiles per slab
    constexpr int KD = D / 16;          // k-steps over d
    constexpr int RBA = D * 2, RBV = F * 2;             // bytes per row of a bf16 piece tile
    constexpr int kTileA = kChunk * RBA, kTileV = kChunk * RBV;  // bytes per piece tile
    constexpr int kOffB = 3 * kTileA, kOffV = 6 * kTileA;        // operand offsets in a buffer
    constexpr int kBufBytes = 6 * kTileA + 3 * kTileV;           // pieces of one chunk
    constexpr int kUnitBytes = 2 * kBufBytes;                    // two buffers
    constexpr int QA = D / 4, QV = F / 4;               // 16-byte fp32 quads per row
    constexpr int LA = kChunk * QA / T, LV = kChunk * QV / T;  // quads per producer lane
    static_assert(NS >= 1 && NS * NP == 4 && kChunk * QA % T == 0 && kChunk * QV % T == 0, "shape");
    static_assert(PF % 2 == 0, "register set and LDS buffer of a chunk follow from its parity");
    static_assert(T % QA == 0, "a lane's quads of a and b share their columns");
    static_assert(NS * kUnitBytes + (NORM ? 3 * kOnesTile + 1024 : 0) <= 160 * 1024 - 256, "LDS");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool producer = wave >= 4;
    // consumer: unit and slab; producer: unit and index among the unit's producers
    const int slot = (wave & 3) / (producer ? NP : NW);
    const int w = (wave & 3) % (producer ? NP : NW);
    const bool in_use = slot < NS;     // false: a consumer left over (three consumers per unit)
    const bool is_den = NORM && w == NWV;  // the consumer that carries the denominator
    const int ln = lane & 31, g = lane >> 5;

    gu32 *hdr = (gu32 *)ws_ptr;
    gu32 *flags = hdr + kHdrWords;
    gfloat *sums = (gfloat *)(hdr + kControlBytes / 4);

    __shared__ __align__(16) char pieces_mem[NS * kUnitBytes];
    __shared__ uint32_t order_sh[4];
    __shared__ int count_sh[4][2];
    __shared__ __align__(16) char ones_mem[NORM ? 3 * kOnesTile : 16];
    __shared__ float den_sh[NORM ? NS : 1][2][kChunk];
    lds_char *const unit_pc = (lds_char *)pieces_mem + (in_use ? slot : 0) * kUnitBytes;
    if constexpr (NORM) {
        for (int i = tid; i < 3 * kOnesTile / 4; i += 512) ((uint32_t *)ones_mem)[i] = 0u;
    }

    // ---- which unit: one ticket per unit, taken by lane 0 of its first consumer ----
    Segment sg;
    bool valid;
    {
        uint32_t order;
        const bool leader = in_use && !producer && w == 0 && lane == 0;
        valid = unit_request<NS>(p, flags, slot, leader, sg, order) && in_use;
        if (leader) order_sh[slot] = order;
        __syncthreads();
        order = order_sh[slot];
        if (valid) valid = segment_locate(p, hdr, leader ? 0 : 1, order, sg);
        if constexpr (NORM) {
            // column 0 of piece 0 of the constant values is one (bf16 0x3f80)
            if (tid < kChunk)
                *(uint16_t *)(ones_mem + PieceSwizzle<64>::addr(tid, 0)) = (uint16_t)0x3f80;
        }
    }
    // Every lane of a wavefront holds the same answer; saying so keeps the segment's
    // descriptors and loop bounds in scalar registers (a descriptor the compiler cannot prove
    // uniform costs a loop over its distinct values around every load and store).
    valid = __builtin_amdgcn_readfirstlane((int)valid) != 0;
    const ScanOperands &op = p.scan[valid ? sg.scan_id : 0];
    const bool REV = valid && sg.rev;
    const int step = valid ? sg.step : 0, n = valid ? sg.n : 0, h = valid ? sg.h : 0;
    const int rows = valid ? sg.rows : 1, nchunks = valid ? sg.nchunks : 0;
    const int64_t lo = valid ? sg.lo : 0;
    const uint32_t total_units = (uint32_t)p.total_waves;
    const bool exchange = valid && p.nseg > 1;
    const bool need_own_sum = exchange && step + 1 < p.nseg;
    // chunk counts of the two passes, largest over the units of the workgroup
    const int n1 = need_own_sum ? nchunks : 0, n2 = nchunks;
    if (in_use && !producer && w == 0 && lane == 0) {
        count_sh[slot][0] = n1;
        count_sh[slot][1] = n2;
    }
    __syncthreads();
    int n1max = 0, n2max = 0;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        n1max = max(n1max, count_sh[s][0]);
        n2max = max(n2max, count_sh[s][1]);
    }

    n1max = __builtin_amdgcn_readfirstlane(n1max);
    n2max = __builtin_amdgcn_readfirstlane(n2max);
#ifdef FTC_TIMELINE
    // stamps 0 .. 4 and 8 .. 15: first consumer of the unit; 5 .. 7: its first producer
    typedef __attribute__((address_space(1))) uint64_t gu64;
    const bool stamp_on = valid && p.nseg > 1 && w == 0 && lane == 0;
    gu64 *const stamp_base =
        (gu64 *)((__attribute__((address_space(1))) char *)ws_ptr + kControlBytes +
                 (int64_t)2 * p.total_waves * (D * 32 * NW * 4)) + (valid ? sg.ticket : 0) * 16;
#endif
    auto chunk_row0 = [&](int c) -> int { return REV ? rows - kChunk * (c + 1) : kChunk * c; };

    if (producer) {
        // =========================== producers ===========================
        const bool active = in_use;
        const int ptid = w * 64 + lane;
        // NORM: rows of b at or beyond this limit (counted from the start of the segment) are
        // zeroed: the key length of the batch entry and the end of the segment
        int b_limit = 0;
        if constexpr (NORM) {
            if (valid) {
                const int64_t len = p.key_len ? p.key_len[n] : p.L;
                b_limit = (int)max((int64_t)0, min((int64_t)rows, len - lo));
            }
        }
        const int prow = ptid / QA;  // row of quad 0 of this lane; quad q: prow + q * (T / QA)
        const uint32_t a_slb = (uint32_t)op.a_sl * 4, b_slb = (uint32_t)op.b_sl * 4,
                       v_slb = (uint32_t)op.v_sl * 4;
        const char *a_seg =
            (const char *)op.a + ((int64_t)n * op.a_sn + (int64_t)h * op.a_sh + lo * op.a_sl) * 4;
        const char *b_seg =
            (const char *)op.b + ((int64_t)n * op.b_sn + (int64_t)h * op.b_sh + lo * op.b_sl) * 4;
        const char *v_seg =
            (const char *)op.v + ((int64_t)n * op.v_sn + (int64_t)h * op.v_sh + lo * op.v_sl) * 4;
        // an absent unit gets empty descriptors: every load returns zeros
        const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)a_seg, 0, valid ? (rows - 1) * a_slb + D * 4 : 0, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t b_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)b_seg, 0, valid ? (rows - 1) * b_slb + D * 4 : 0, kRsrcFlags);
        const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(
            (void *)v_seg, 0, valid ? (rows - 1) * v_slb + F * 4 : 0, kRsrcFlags);
        // quad q of a lane is 16-byte unit q * T + ptid of the chunk's tile
        uint32_t a_goff[LA], b_goff[LA], v_goff[LV];  // byte offset inside a chunk (global)
        int a_waddr[LA], v_waddr[LV];                 // byte address inside a piece tile (LDS)
#pragma unroll
        for (int q = 0; q < LA; q++) {
            const int u = q * T + ptid, row = u / QA, c4 = u % QA;
            a_goff[q] = (uint32_t)row * a_slb + 16u * c4;
            b_goff[q] = (uint32_t)row * b_slb + 16u * c4;
            a_waddr[q] = PieceSwizzle<RBA>::addr(row, 8 * c4);
        }
#pragma unroll
        for (int q = 0; q < LV; q++) {
            const int u = q * T + ptid, row = u / QV, c4 = u % QV;
            v_goff[q] = (uint32_t)row * v_slb + 16u * c4;
            v_waddr[q] = PieceSwizzle<RBV>::addr(row, 8 * c4);
        }
        // Rows are requested PF chunks ahead of the cut, into PF sets of registers that take
        // turns, so that a request has several chunks' time to be served.  (With one unit per
        // workgroup the requests in flight are all that keeps the memory system busy.)
        struct Raw {
            u32x4 a[LA], b[LA], v[LV];
            int row0;
        };
        Raw raw[PF];
        auto fetch = [&](Raw &r, int row0, bool with_a) {
            if (!active) return;
            r.row0 = row0;
#pragma unroll
            for (int q = 0; q < LA; q++) {
                if (with_a)
                    r.a[q] = __builtin_amdgcn_raw_buffer_load_b128(
                        a_rs, a_goff[q] + (uint32_t)row0 * a_slb, 0, 0);
                r.b[q] = __builtin_amdgcn_raw_buffer_load_b128(
                    b_rs, b_goff[q] + (uint32_t)row0 * b_slb, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < LV; q++)
                r.v[q] = __builtin_amdgcn_raw_buffer_load_b128(
                    v_rs, v_goff[q] + (uint32_t)row0 * v_slb, 0, 0);
        };
        auto cut = [&](const Raw &r, int buf, bool with_a) {
            if (!active) return;
            lds_char *const pc = unit_pc + buf * kBufBytes;
            // NORM: every row of the chunk lies below the limit for rows of b (scalar test)
            const bool whole = NORM && r.row0 >= 0 && r.row0 + kChunk <= b_limit;
#pragma unroll
            for (int q = 0; q < LA; q++) {
                if constexpr (NORM) {
                    if (with_a) split_quad_to_lds(feature_quad(r.a[q]), pc, kTileA, a_waddr[q]);
                    u32x4 bq = feature_quad(r.b[q]);
                    if (!whole) {  // a chunk that the key length or the end of the segment cuts
                        if ((uint32_t)(r.row0 + prow + q * (T / QA)) >= (uint32_t)b_limit)
                            bq = u32x4{0u, 0u, 0u, 0u};
                    }
                    split_quad_to_lds(bq, pc + kOffB, kTileA, a_waddr[q]);
                } else {
                    if (with_a) split_quad_to_lds(r.a[q], pc, kTileA, a_waddr[q]);
                    split_quad_to_lds(r.b[q], pc + kOffB, kTileA, a_waddr[q]);
                }
            }
#pragma unroll
            for (int q = 0; q < LV; q++) split_quad_to_lds(r.v[q], pc + kOffV, kTileV, v_waddr[q]);
        };
        // rows of a chunk that does not exist lie outside the descriptor and read as zero
        auto pass1_row0 = [&](int i) -> int { return i < n1 ? chunk_row0(n1 - 1 - i) : -2 * kChunk; };
        auto pass2_row0 = [&](int c) -> int { return c < n2 ? chunk_row0(c) : -2 * kChunk; };
        // One pass over nmax chunks: chunk i of the walk goes to LDS buffer i % 2 through
        // register set i % PF; one barrier before the first chunk and one per chunk.
        auto run_pass = [&](int nmax, auto row0_of, bool with_a) {
#pragma unroll
            for (int j = 0; j < PF; j++) fetch(raw[j], row0_of(j), with_a);
            cut(raw[0], 0, with_a);
            fetch(raw[0], row0_of(PF), with_a);
            wg_barrier();
            // Whole trips in the loop, the rest after it: a way out of the middle of the loop
            // would join the paths at the loop's head, and the compiler would then wait for
            // every request at the head instead of counting.
            int c = 0;
            for (; c + PF <= nmax; c += PF) {
#pragma unroll
                for (int j = 0; j < PF; j++) {
                    if (with_a && c + j == 4) FTC_STAMP(5);  // pass 2, fifth chunk
                    // Made every time, also past the last chunk (requests outside the
                    // descriptor cost no traffic and return zeros): with a fixed number of
                    // requests per chunk the compiler waits for the oldest only
                    // (s_waitcnt vmcnt(n), n younger requests) instead of for all of them.
                    cut(raw[(j + 1) % PF], (j + 1) & 1, with_a);
                    fetch(raw[(j + 1) % PF], row0_of(c + j + 1 + PF), with_a);
                    if (with_a && c + j == 4) FTC_STAMP(6);
                    wg_barrier();
                    __builtin_amdgcn_sched_barrier(0);  // one chunk at a time, in this order
                    if (with_a && c + j == 4) FTC_STAMP(7);
                }
            }
#pragma unroll
            for (int j = 0; j < PF - 1; j++) {
                if (c + j >= nmax) return;
                cut(raw[(j + 1) % PF], (j + 1) & 1, with_a);
                wg_barrier();
            }
        };
        // pass 1 walks against the direction of pass 2
        if (n1max > 0) run_pass(n1max, pass1_row0, false);
        run_pass(n2max, pass2_row0, true);
        return;
    }

    // =========================== consumers ===========================
    FTC_STAMP(0);
    const uint32_t vticket = (uint32_t)w * total_units + (valid ? sg.ticket : 0);
    const uint32_t o_slb = (uint32_t)op.o_sl * 4;
    char *o_seg = (char *)op.out + ((int64_t)n * op.o_sn + (int64_t)h * op.o_sh + lo * op.o_sl) * 4;
    const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)o_seg, 0, valid ? (rows - 1) * o_slb + F * 4 : 0, kRsrcFlags);
    const uint32_t o_lane = ln * o_slb + 4u * (32 * w + 4 * g);

    // row-major fragments of a and b: lane (row = ln, g), k-step ks: columns 16 ks + 8 g + 0..7
    int row_addr[KD];
#pragma unroll
    for (int ks = 0; ks < KD; ks++) row_addr[ks] = PieceSwizzle<RBA>::addr(ln, 32 * ks + 16 * g);
    // transposing reads: lane = 16 G + s supplies 8 bytes of row 8 u + 4 (G / 2) + s / 4 (+ 16 hh)
    //  b^T, tile dt: columns 32 dt + 16 (G % 2) + 8 (x % 2) + 4 (x / 2) + 0..3, x = s % 4
    //  v (this consumer's slab): columns 32 w + 16 (G % 2) + 4 x + 0..3
    // (rows 16 .. 31 of a tile have the swizzle keys of rows 0 .. 15)
    // The values of the denominator's consumer are the constant tile: other base, other
    // tile and half-tile strides (vts, vhs), rows of 64 bytes.
    int bt_addr[DT][2], vt_addr[2];
    const int vts = is_den ? kOnesTile : kTileV, vhs = is_den ? 16 * 64 : 16 * RBV;
    {
        const int G = lane >> 4, s = lane & 15, x = s & 3;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int row = 8 * u + 4 * (G / 2) + s / 4;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
                bt_addr[dt][u] = kOffB + PieceSwizzle<RBA>::addr(
                    row, 2 * (32 * dt + 16 * (G % 2) + 8 * (x % 2) + 4 * (x / 2)));
            vt_addr[u] = is_den ? PieceSwizzle<64>::addr(row, 2 * (16 * (G % 2) + 4 * x))
                                : PieceSwizzle<RBV>::addr(row, 2 * (32 * w + 16 * (G % 2) + 4 * x));
        }
    }
    auto v_tiles = [&](const lds_char *pc) -> const lds_char * {
        return is_den ? (const lds_char *)ones_mem : pc + kOffV;
    };
    // causal mask inside a chunk as bit masks (all ones: keep): accumulator register r of
    // lane (i = ln, g) holds row j = 8 (r / 4) + 4 g + r % 4 of Pt
    uint32_t keep[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int j = 8 * (r / 4) + 4 * g + (r % 4);
        keep[r] = (REV ? (j >= ln) : (j <= ln)) ? 0xffffffffu : 0u;
        asm volatile("" : "+v"(keep[r]));
    }
    f32x16 S[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) S[dt][r] = 0.f;
    // position-major fragments of the chunk in buffer pc: v (this slab's columns), b^T
    auto v_frags = [&](const lds_char *pc, Frag (&f)[2][3]) {
        const lds_char *const vpc = v_tiles(pc);
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int k = 0; k < 3; k++)
                f[hh][k] = lds_frag_tr(vpc + k * vts + hh * vhs + vt_addr[0],
                                       vpc + k * vts + hh * vhs + vt_addr[1]);
    };
    auto bt_frags = [&](const lds_char *pc, Frag (&f)[2][DT][3]) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int k = 0; k < 3; k++)
                    f[hh][dt][k] = lds_frag_tr(pc + k * kTileA + hh * 16 * RBA + bt_addr[dt][0],
                                               pc + k * kTileA + hh * 16 * RBA + bt_addr[dt][1]);
    };
    // (3) S += b^T v
    auto update_state = [&](const Frag (&bt)[2][DT][3], const Frag (&v_frag)[2][3]) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) S[dt] = mfma_split<3, 3>(bt[hh][dt], v_frag[hh], S[dt]);
    };

    // the slab of a consumer is a state of DT x 1 tiles for the exchange
    f32x16 Sx[DT][1];
    StateExchange<DT, 1> xch(flags, sums, (uint32_t)NW * total_units, vticket, step, p.nseg,
                             p.group, lane);
    // ---- pass 1: the segment's own state sum ----
    if (n1max > 0) {
        wg_barrier();
        for (int i = 0; i < n1max; i++) {
            const lds_char *pc = unit_pc + (i & 1) * kBufBytes;
            Frag v_frag[2][3], bt[2][DT][3];
            if (i < n1) {
                v_frags(pc, v_frag);
                bt_frags(pc, bt);
            }
            // the fragments are in registers: the producers may refill this buffer while the
            // matrix cores add the chunk to the state
            wg_barrier();
            if (i < n1) update_state(bt, v_frag);
        }
        if (need_own_sum) {
#pragma unroll
            for (int dt = 0; dt < DT; dt++) Sx[dt][0] = S[dt];
            xch.publish_sum(Sx);
        }
    }
    FTC_STAMP(1);
    if (exchange) {
        f32x16 X[DT][1];
#pragma unroll
        for (int dt = 0; dt < DT; dt++) Sx[dt][0] = S[dt];
        xch.gather(Sx, X);
        if (xch.failed && lane == 0)
            __hip_atomic_store(hdr + kHdrError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) S[dt] = X[dt][0];
    }
    if (!NORM && valid && op.s0)
        wg_add_caller_state<DT>(op.s0 + (int64_t)n * op.s0_sn + (int64_t)h * op.s0_sh, op.s0_sd,
                                32 * w + ln, g, S);

    // ---- pass 2: outputs ----
    // A consumer is the only wavefront with matrix work on its SIMD, and a wavefront issues in
    // order: its own vector ALU work (cutting S and Pt) and its LDS reads overlap with its
    // matrix instructions only when they alternate in the instruction stream.  The body of a
    // chunk is therefore written out in that order, one matrix instruction and what goes
    // under it at a time, with scheduling barriers that keep the compiler from regrouping it:
    //
    //   cut S(0) | (1)[0] + cut S(1) | (2b)[0] + reads | (1)[1] + cut S(2) | (2b)[1] + reads | ...
    //   | (3) + mask and cut Pt | (2a) | store
    //
    // (1)[ks], (2b)[ks]: the six matrix instructions of k-step ks of Pt = b a^T and of
    // Ot = S^T a^T; "reads": the transposing reads of v and b^T for (3) and (2a).
    constexpr int kPa[6] = {0, 1, 2, 0, 1, 0}, kPb[6] = {2, 1, 0, 1, 0, 0};  // piece products
    constexpr int kTrFrags = 6 + 6 * DT;  // position-major fragments of a chunk
    constexpr int kM3 = 12 * DT;          // matrix instructions of (3)
    FTC_STAMP(2);
    wg_barrier();
    FTC_STAMP(3);
    f32x16 O_held;  // NORM: Ot of a chunk, kept across the barrier behind which its denominator is
    for (int c = 0; c < n2max; c++) {
        if (c < n2) {
            const lds_char *pc = unit_pc + (c & 1) * kBufBytes;
            const lds_char *const vpc = v_tiles(pc);
            Frag af[KD][3], bf[KD][3], v_frag[2][3], bt[2][DT][3], sf[2][3], p_frag[2][3];
            f32x16 P, O;
#pragma unroll
            for (int ks = 0; ks < KD; ks++)
#pragma unroll
                for (int k = 0; k < 3; k++) {
                    af[ks][k] = lds_frag16(pc + k * kTileA + row_addr[ks]);
                    bf[ks][k] = lds_frag16(pc + kOffB + k * kTileA + row_addr[ks]);
                }
            // pair q of k-step ks of S -> sf[ks % 2]
            auto cut_s = [&](int ks, int q) {
                uint32_t o[3];
                split_pair_under_mfma(S[ks / 2][8 * (ks % 2) + 2 * q],
                                      S[ks / 2][8 * (ks % 2) + 2 * q + 1], o);
#pragma unroll
                for (int k = 0; k < 3; k++) sf[ks % 2][k].w[q] = o[k];
            };
            // position-major fragment number i in the order in which (3) and (2a) use them
            auto tr_frag = [&](int i) {
                const int hh = i / (3 + 3 * DT), j = i % (3 + 3 * DT);
                if (j < 3)
                    v_frag[hh][j] = lds_frag_tr(vpc + j * vts + hh * vhs + vt_addr[0],
                                                vpc + j * vts + hh * vhs + vt_addr[1]);
                else {
                    const int dt = (j - 3) / 3, k = (j - 3) % 3;
                    bt[hh][dt][k] = lds_frag_tr(pc + k * kTileA + hh * 16 * RBA + bt_addr[dt][0],
                                                pc + k * kTileA + hh * 16 * RBA + bt_addr[dt][1]);
                }
            };
#pragma unroll
            for (int r = 0; r < 16; r++) P[r] = 0.f, O[r] = 0.f;
#pragma unroll
            for (int q = 0; q < 4; q++) cut_s(0, q);
            __builtin_amdgcn_sched_barrier(0);
            int tr_next = 0;
#pragma unroll
            for (int ks = 0; ks < KD; ks++) {
#pragma unroll
                for (int i = 0; i < 6; i++) {  // (1)[ks], with S(ks + 1) cut underneath
                    P = mfma(bf[ks][kPa[i]], af[ks][kPb[i]], P);
                    if (ks + 1 < KD && i < 4) cut_s(ks + 1, i);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int i = 0; i < 6; i++) {  // (2b)[ks], with the transposing reads underneath
                    O = mfma(sf[ks % 2][kPa[i]], af[ks][kPb[i]], O);
                    if (tr_next < kTrFrags) tr_frag(tr_next++);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            // (3) S += b^T v, with the masking and cutting of Pt underneath
#pragma unroll
            for (int i = 0; i < kM3; i++) {
                const int hh = i / (6 * DT), dt = (i / 6) % DT, m = i % 6;
                S[dt] = mfma(bt[hh][dt][kPa[m]], v_frag[hh][kPb[m]], S[dt]);
#pragma unroll
                for (int u = 0; u < 8; u++)
                    if ((u * kM3) / 8 == i) {  // pair u of Pt: registers 2 u, 2 u + 1
                        uint32_t o[3];
                        split_pair_under_mfma(
                            __uint_as_float(__float_as_uint(P[2 * u]) & keep[2 * u]),
                            __uint_as_float(__float_as_uint(P[2 * u + 1]) & keep[2 * u + 1]), o);
#pragma unroll
                        for (int k = 0; k < 3; k++) p_frag[u / 4][k].w[u % 4] = o[k];
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
            // (2a) Ot += v^T Pt
#pragma unroll
            for (int hh = 0; hh < 2; hh++)
#pragma unroll
                for (int m = 0; m < 6; m++) O = mfma(v_frag[hh][kPa[m]], p_frag[hh][kPb[m]], O);
            // lane (i = ln, g) holds f = 32 w + 8 q + 4 g + 0..3 in registers 4 q .. 4 q + 3
            if constexpr (NORM) {
                if (is_den) {
                    if (g == 0) {
                        const float den = O[0] + p.eps;
                        den_sh[slot][c & 1][ln] = den;
                        // (the caller's copy of the denominators, for the backward)
                        const int row = chunk_row0(c) + ln;
                        if (op.s_out && row < rows)
                            op.s_out[(int64_t)n * op.so_sn + (int64_t)h * op.so_sh + lo + row] = den;
                    }
                } else {
                    O_held = O;
                }
            } else {
                const uint32_t o_off = o_lane + (uint32_t)chunk_row0(c) * o_slb;
#pragma unroll
                for (int q = 0; q < 4; q++)
                    buffer_store4(o_rs, o_off + (uint32_t)(4 * 8 * q), O[4 * q + 0], O[4 * q + 1],
                                  O[4 * q + 2], O[4 * q + 3]);
            }
        }
        wg_barrier();
        if constexpr (NORM) {
            if (c < n2 && !is_den) {
                const float z = 1.0f / den_sh[slot][c & 1][ln];
                const uint32_t o_off = o_lane + (uint32_t)chunk_row0(c) * o_slb;
#pragma unroll
                for (int q = 0; q < 4; q++)
                    buffer_store4(o_rs, o_off + (uint32_t)(4 * 8 * q), O_held[4 * q + 0] * z,
                                  O_held[4 * q + 1] * z, O_held[4 * q + 2] * z,
                                  O_held[4 * q + 3] * z);
            }
        }
        if (c < 8) FTC_STAMP(8 + c);
    }
    FTC_STAMP(4);
    if (!valid) return;
    if (!NORM && op.s_out && step == p.nseg - 1)
        wg_store_caller_state<DT>(op.s_out + (int64_t)n * op.so_sn + (int64_t)h * op.so_sh,
                                  op.so_sd, 32 * w + ln, g, S);

    // the last consumer of the launch leaves the control block zeroed
    if (p.nseg > 1) {
        uint32_t done = 0;
        if (lane == 0)
            done = __hip_atomic_fetch_add(hdr + kHdrDone, 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
        done = __builtin_amdgcn_readfirstlane(done);
        if (done == (uint32_t)NW * total_units - 1) {
            for (uint32_t i = lane; i < (uint32_t)NW * total_units; i += kWave)
                __hip_atomic_store(flags + i, kFlagEmpty, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            for (uint32_t i = lane; i < total_units / (uint32_t)p.nseg; i += kWave)
                __hip_atomic_store(flags + kMaxWaves + i, 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0)
                __hip_atomic_store(hdr + kHdrDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// units (chain segments) per workgroup for output rows of F values
// `norm`: the fused attention form of the kernel (NORM = true)
inline int scan_wg_units_per_block(int F, bool norm) { return 4 / (F / 32 + (norm ? 1 : 0)); }
void launch_scan_wg_ffff(int D, int F, bool norm, void *ws, const ScanArgs &args,
                         hipStream_t stream);
bool scan_wg_covers(int D, int F);
bool scan_wg_norm_covers(int D, int F);
// chain-parallel form (ftc_tp_kernel.h): one workgroup per chain of a 64 x 64 all-fp32 scan
void launch_scan_tp(void *ws, const ScanArgs &args, hipStream_t stream);
// the same on the fp16 matrix path (ftc_tph_kernel.h): states of up to 64 rows
// `mixed`: some rows are bf16 (ScanOperands::pad of every scan says which)
void launch_scan_tph(void *ws, const ScanArgs &args, bool mixed, hipStream_t stream);

}  // namespace mfma
}  // namespace ftc
