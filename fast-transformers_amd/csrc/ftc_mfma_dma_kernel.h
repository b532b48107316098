// MFMA causal scan for gfx950, variant for state rows of at most 64 values: the rows of a
// chunk travel from global memory straight into LDS (buffer loads with the LDS modifier), so
// the prefetch of the next chunk occupies no registers and every row is fetched once.
//
// Same algorithm, products, piece split and state exchange as ftc_mfma_kernel.h; only the
// way operands reach their fragments differs:
//
//  * Each operand has an LDS tile of 32 rows.  A load instruction moves 64 x 16 bytes and
//    puts lane L's 16 bytes at tile + 16 * L, so the tile layout is chosen through the
//    global addresses the lanes ask for: slot (row r, position p) holds piece p ^ s(r) of
//    row r.  With that XOR swizzle both access patterns are free of bank conflicts: the
//    16-byte reads of row-major fragments (16 consecutive rows, one logical piece) and the
//    element-wide reads of position-major fragments (32 consecutive columns, one row).
//  * a and v are read once per chunk and live on as fragments, so one tile each suffices:
//    the next chunk is requested as soon as the fragments are cut.  b is read row-major at
//    the start of a chunk and by column at its end, so it alternates between two tiles.
//  * Rows outside the segment's descriptor arrive as zeros, as with register loads.
#pragma once
#include "ftc_mfma_kernel.h"

namespace ftc {
namespace mfma {

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef __attribute__((address_space(3))) uint16_t lds_u16;
typedef __attribute__((address_space(3))) float lds_f32;
typedef uint32_t u32x4_a __attribute__((ext_vector_type(4), may_alias));
typedef uint32_t u32x2_a __attribute__((ext_vector_type(2), may_alias));
typedef __attribute__((address_space(3))) u32x4_a lds_vec4;
typedef __attribute__((address_space(3))) u32x2_a lds_vec2;

// XOR swizzle of a tile whose rows have RB bytes (a power of two, 64..512).
template <int RB>
struct Swizzle {
    static constexpr int kPieces = RB / 16;                      // 16-byte pieces per row
    static constexpr int kXor = kPieces < 16 ? kPieces : 16;     // pieces the XOR permutes
    static constexpr int kRowsPerBankRow = 16 / kXor;            // rows per 256 bytes of LDS
    __device__ static __forceinline__ int key(int row) {
        return (row / kRowsPerBankRow) & (kXor - 1);
    }
    // byte address inside the tile of logical byte `off` of row `row`
    __device__ static __forceinline__ int addr(int row, int off) {
        return (row * kPieces + ((off >> 4) ^ key(row))) * 16 + (off & 15);
    }
    // 16-byte slot j of the tile holds this logical piece of this row
    __device__ static __forceinline__ void slot(int j, int &row, int &piece) {
        row = j / kPieces;
        piece = (j % kPieces) ^ key(row);
    }
};

// Requests for one tile: kLoads instructions, lane offsets prepared once.
template <int RB>
struct TileRequest {
    static constexpr int kLoads = kChunk * RB / (kWave * 16);
    uint32_t lane_off[kLoads];
    __device__ __forceinline__ void prepare(int lane, uint32_t row_stride_bytes) {
#pragma unroll
        for (int i = 0; i < kLoads; i++) {
            int row, piece;
            Swizzle<RB>::slot(i * kWave + lane, row, piece);
            lane_off[i] = (uint32_t)row * row_stride_bytes + 16u * (uint32_t)piece;
        }
    }
    // rows row0 .. row0 + 31 of the segment -> tile
    __device__ __forceinline__ void issue(__amdgpu_buffer_rsrc_t rsrc, lds_char *tile, int row0,
                                          uint32_t row_stride_bytes) const {
        const uint32_t base = (uint32_t)row0 * row_stride_bytes;
        // every read of the tile's previous contents has delivered its data
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < kLoads; i++)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void *)(tile + i * kWave * 16), 16,
                                                     lane_off[i] + base, 0, 0, 0);
    }
};

// four consecutive elements of a tile row as a Quad
__device__ __forceinline__ void lds_read_quad(const lds_char *p, Quad<float> &q) {
    const u32x4 r = *(const lds_vec4 *)p;
    q.v = make_float4(__uint_as_float(r.x), __uint_as_float(r.y), __uint_as_float(r.z),
                      __uint_as_float(r.w));
}
__device__ __forceinline__ void lds_read_quad(const lds_char *p, Quad<bf16_t> &q) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 r = *(const lds_vec2 *)p;
    q.v = make_uint2(r.x, r.y);
}
// eight elements of one tile column (byte addresses given), cut into fragments
__device__ __forceinline__ void lds_column_to_frags(const lds_char *tile, const int (&addr)[8],
                                                    int extra, Frag (&f)[3], float *) {
    float x[8];
#pragma unroll
    for (int t = 0; t < 8; t++) x[t] = *(const lds_f32 *)(tile + addr[t] + extra);
    split8<3>(x, f);
}
__device__ __forceinline__ void lds_column_to_frags(const lds_char *tile, const int (&addr)[8],
                                                    int extra, Frag (&f)[1], bf16_t *) {
    uint32_t x[8];
#pragma unroll
    for (int t = 0; t < 8; t++) x[t] = *(const lds_u16 *)(tile + addr[t] + extra);
#pragma unroll
    for (int q = 0; q < 4; q++) f[0].w[q] = x[2 * q] | (x[2 * q + 1] << 16);
}

template <int D, int F, typename TA, typename TB, typename TV, typename TO>
__global__ __launch_bounds__(kWave) void scan_dma_kernel(uint32_t *__restrict__ ws_ptr,
                                                         ScanArgs p) {
    constexpr int NSA = Elem<TA>::kPieces, NSB = Elem<TB>::kPieces, NSV = Elem<TV>::kPieces;
    constexpr int NS = 3;  // pieces of the fp32 intermediates (P and the state)
    constexpr int BA = Elem<TA>::kBytes, BB = Elem<TB>::kBytes, BV = Elem<TV>::kBytes,
                  BO = Elem<TO>::kBytes;
    constexpr int DT = D / 32, FT = F / 32;  // state tiles
    constexpr int KD = D / 16;               // k-steps over d
    constexpr int RBA = D * BA, RBB = D * BB, RBV = F * BV;  // row bytes

    const int lane = threadIdx.x;
    const int ln = lane & 31, g = lane >> 5;

    gu32 *hdr = (gu32 *)ws_ptr;
    gu32 *flags = hdr + kHdrWords;
    gfloat *sums = (gfloat *)(hdr + kControlBytes / 4);

    // the ticket is asked for here and looked at only after the per-lane address tables,
    // which do not depend on it, have been set up
    Segment sg;
    uint32_t order;
    segment_request(p, flags, lane, sg, order);
    const ScanOperands &op = p.scan[sg.scan_id];
    const bool REV = sg.rev;
    const uint32_t a_slb = (uint32_t)op.a_sl * BA, b_slb = (uint32_t)op.b_sl * BB,
                   v_slb = (uint32_t)op.v_sl * BV, o_slb = (uint32_t)op.o_sl * BO;
    TileRequest<RBA> a_req;
    TileRequest<RBB> b_req;
    TileRequest<RBV> v_req;
    a_req.prepare(lane, a_slb);
    b_req.prepare(lane, b_slb);
    v_req.prepare(lane, v_slb);

    // per-lane tile addresses
    //  row-major fragments: lane (row = ln, g), k-step ks: elements 16*ks + 4*g + 0..3, + 8
    int a_row_addr[KD][2], b_row_addr[KD][2];
#pragma unroll
    for (int ks = 0; ks < KD; ks++)
#pragma unroll
        for (int w = 0; w < 2; w++) {
            a_row_addr[ks][w] = Swizzle<RBA>::addr(ln, (16 * ks + 4 * g + 8 * w) * BA);
            b_row_addr[ks][w] = Swizzle<RBB>::addr(ln, (16 * ks + 4 * g + 8 * w) * BB);
        }
    //  position-major fragments: lane (col = 32*tile + ln, g), k-slot t of k-step hh is row
    //  16*hh + 8*(t/4) + 4*g + (t%4); the swizzle key does not depend on hh
    int b_col_addr[DT][8], v_col_addr[FT][8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const int row = 8 * (t / 4) + 4 * g + (t % 4);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
            b_col_addr[dt][t] = Swizzle<RBB>::addr(row, (32 * dt + ln) * BB);
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
            v_col_addr[ft][t] = Swizzle<RBV>::addr(row, (32 * ft + ln) * BV);
    }
    // causal mask inside a chunk as bit masks (all ones: keep): accumulator register r of
    // lane (i = ln, g) holds row j = 8*(r/4) + 4*g + r%4 of Pt
    uint32_t keep[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int j = 8 * (r / 4) + 4 * g + (r % 4);
        keep[r] = (REV ? (j >= ln) : (j <= ln)) ? 0xffffffffu : 0u;
        // kept in a vector register: as 16 lane masks in scalar registers they would push
        // other scalars out
        asm volatile("" : "+v"(keep[r]));
    }

    if (!segment_locate(p, hdr, lane, order, sg)) return;
    const uint32_t ticket = sg.ticket;
    const int step = sg.step, n = sg.n, h = sg.h, rows = sg.rows, nchunks = sg.nchunks;
    const int64_t lo = sg.lo;

    const char *a_seg =
        (const char *)op.a + ((int64_t)n * op.a_sn + (int64_t)h * op.a_sh + lo * op.a_sl) * BA;
    const char *b_seg =
        (const char *)op.b + ((int64_t)n * op.b_sn + (int64_t)h * op.b_sh + lo * op.b_sl) * BB;
    const char *v_seg =
        (const char *)op.v + ((int64_t)n * op.v_sn + (int64_t)h * op.v_sh + lo * op.v_sl) * BV;
    char *o_seg = (char *)op.out + ((int64_t)n * op.o_sn + (int64_t)h * op.o_sh + lo * op.o_sl) * BO;
    const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)a_seg, 0, (rows - 1) * a_slb + RBA, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t b_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)b_seg, 0, (rows - 1) * b_slb + RBB, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)v_seg, 0, (rows - 1) * v_slb + RBV, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)o_seg, 0, (rows - 1) * o_slb + F * BO, kRsrcFlags);
    const uint32_t o_lane = ln * o_slb + 4u * BO * g;

    auto chunk_row0 = [&](int c) -> int { return REV ? rows - kChunk * (c + 1) : kChunk * c; };
    auto pass1_row0 = [&](int c) -> int { return c < 0 ? -2 * kChunk : chunk_row0(c); };

    // ---- LDS tiles (separate arrays: the compiler then waits per tile, not for all) ----
    __shared__ __align__(16) char a_tile_mem[kChunk * RBA];
    __shared__ __align__(16) char b_tile0_mem[kChunk * RBB];
    __shared__ __align__(16) char b_tile1_mem[kChunk * RBB];
    __shared__ __align__(16) char v_tile_mem[kChunk * RBV];
    // pass 1 alternates v between v_tile and a second tile: a's, when it is large enough
    constexpr bool kVinA = RBA >= RBV;
    constexpr bool kVSecond = kVinA || (kChunk * (RBA + 2 * RBB + 2 * RBV) <= 40960);
    __shared__ __align__(16) char v_tile_extra_mem[(kVSecond && !kVinA) ? kChunk * RBV : 16];
    lds_char *const a_tile = (lds_char *)a_tile_mem, *const b_tile0 = (lds_char *)b_tile0_mem,
                    *const b_tile1 = (lds_char *)b_tile1_mem, *const v_tile = (lds_char *)v_tile_mem;
    lds_char *const v_second = kVinA ? a_tile : (lds_char *)v_tile_extra_mem;

    auto bt_frags = [&](const lds_char *tile, int dt, int hh, Frag (&frag)[NSB]) {
        lds_column_to_frags(tile, b_col_addr[dt], hh * 16 * RBB, frag, (TB *)nullptr);
    };
    auto vt_frags = [&](const lds_char *tile, int ft, int hh, Frag (&frag)[NSV]) {
        lds_column_to_frags(tile, v_col_addr[ft], hh * 16 * RBV, frag, (TV *)nullptr);
    };

    f32x16 S[DT][FT];
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

    StateExchange<DT, FT> xch(flags, sums, (uint32_t)p.total_waves, ticket, step, p.nseg, p.group,
                              lane);
    if (p.nseg > 1) {
        // ---- pass 1: the segment's own state sum, walked against the direction of pass 2.
        // Every tile is refilled with the chunk two steps on as soon as it has been read. ----
        if (xch.need_own_sum) {
            auto sum_chunk = [&](lds_char *b_tile, lds_char *vt, int c) {
                Frag bt_frag[DT][2][NSB], v_frag[FT][2][NSV];
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) bt_frags(b_tile, dt, hh, bt_frag[dt][hh]);
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) vt_frags(vt, ft, hh, v_frag[ft][hh]);
                b_req.issue(b_rs, b_tile, pass1_row0(c - 2), b_slb);
                if (kVSecond) v_req.issue(v_rs, vt, pass1_row0(c - 2), v_slb);
                else v_req.issue(v_rs, vt, pass1_row0(c - 1), v_slb);
                update_state(bt_frag, v_frag);
            };
            b_req.issue(b_rs, b_tile0, pass1_row0(nchunks - 1), b_slb);
            v_req.issue(v_rs, v_tile, pass1_row0(nchunks - 1), v_slb);
            b_req.issue(b_rs, b_tile1, pass1_row0(nchunks - 2), b_slb);
            if (kVSecond) v_req.issue(v_rs, v_second, pass1_row0(nchunks - 2), v_slb);
            for (int c = nchunks - 1; c >= 0; c -= 2) {
                sum_chunk(b_tile0, v_tile, c);
                if (c == 0) break;
                sum_chunk(b_tile1, kVSecond ? v_second : v_tile, c - 1);
            }
            xch.publish_sum(S);
        }
    }
    // ---- first chunks of pass 2 (requested before waiting for the other wavefronts) ----
    a_req.issue(a_rs, a_tile, chunk_row0(0), a_slb);
    b_req.issue(b_rs, b_tile0, chunk_row0(0), b_slb);
    v_req.issue(v_rs, v_tile, chunk_row0(0), v_slb);
    b_req.issue(b_rs, b_tile1, chunk_row0(1), b_slb);
    if (p.nseg > 1) {
        f32x16 X[DT][FT];
        xch.gather(S, X);
        if (xch.failed && lane == 0)
            __hip_atomic_store(hdr + kHdrError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++) S[dt][ft] = X[dt][ft];
    }
    // every segment starts from (the caller's initial state) + (the sums of the segments
    // before it)
    if (op.s0)
        add_caller_state<DT, FT>(op.s0 + (int64_t)n * op.s0_sn + (int64_t)h * op.s0_sh, op.s0_sd,
                                 ln, g, S);

    // ---- pass 2: outputs.  b alternates between its two tiles, hence the chunk pairs. ----
    // row-major fragments of a chunk's a and b rows; a's tile is free afterwards
    Frag a_frag[KD][NSA], b_frag[KD][NSB];
    auto row_frags = [&](lds_char *b_tile) {
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            Quad<TA> a0, a1;
            lds_read_quad(a_tile + a_row_addr[ks][0], a0);
            lds_read_quad(a_tile + a_row_addr[ks][1], a1);
            quads_to_frags(a0, a1, a_frag[ks]);
            Quad<TB> b0, b1;
            lds_read_quad(b_tile + b_row_addr[ks][0], b0);
            lds_read_quad(b_tile + b_row_addr[ks][1], b1);
            quads_to_frags(b0, b1, b_frag[ks]);
        }
    };
    row_frags(b_tile0);
    a_req.issue(a_rs, a_tile, chunk_row0(1), a_slb);

    // On entry a_frag, b_frag hold chunk c; on exit they hold chunk c + 1, cut while the
    // matrix cores are busy with the state update.
    auto output_chunk = [&](int c, lds_char *b_tile, lds_char *b_next) {
        const int row0 = chunk_row0(c);
        Frag a_cur[KD][NSA];
#pragma unroll
        for (int ks = 0; ks < KD; ks++)
#pragma unroll
            for (int pc = 0; pc < NSA; pc++) a_cur[ks][pc] = a_frag[ks][pc];

        // (1) Pt = b a^T
        f32x16 P;
#pragma unroll
        for (int r = 0; r < 16; r++) P[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) P = mfma_split<NSB, NSA>(b_frag[ks], a_cur[ks], P);
#pragma unroll
        for (int r = 0; r < 16; r++) P[r] = __uint_as_float(__float_as_uint(P[r]) & keep[r]);
        Frag p_frag[2][NS];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            const float x[8] = {P[8 * hh + 0], P[8 * hh + 1], P[8 * hh + 2], P[8 * hh + 3],
                                P[8 * hh + 4], P[8 * hh + 5], P[8 * hh + 6], P[8 * hh + 7]};
            split8<NS>(x, p_frag[hh]);
        }

        // v by column; its tile is then free for the next chunk
        Frag v_frag[FT][2][NSV];
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++) vt_frags(v_tile, ft, hh, v_frag[ft][hh]);
        v_req.issue(v_rs, v_tile, chunk_row0(c + 1), v_slb);

        // (2b) + (2a), output tiles side by side, then store
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
                O[ft] = mfma_split<NS, NSA>(s_frag, a_cur[ks], O[ft]);
            }
        }
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++)
                O[ft] = mfma_split<NSV, NS>(v_frag[ft][hh], p_frag[hh], O[ft]);
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                buffer_store_out(o_rs, o_off + (uint32_t)(BO * (32 * ft + 8 * q)), O[ft][4 * q + 0],
                                 O[ft][4 * q + 1], O[ft][4 * q + 2], O[ft][4 * q + 3],
                                 (TO *)nullptr);

        // (3): b by column; this b tile then takes the chunk after next
        Frag bt_frag[DT][2][NSB];
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++) bt_frags(b_tile, dt, hh, bt_frag[dt][hh]);
        b_req.issue(b_rs, b_tile, chunk_row0(c + 2), b_slb);
        row_frags(b_next);
        a_req.issue(a_rs, a_tile, chunk_row0(c + 2), a_slb);
        update_state(bt_frag, v_frag);
    };
    for (int c = 0; c < nchunks; c += 2) {
        output_chunk(c, b_tile0, b_tile1);
        if (c + 1 < nchunks) output_chunk(c + 1, b_tile1, b_tile0);
    }
    // the segment walked last ends on the state after the whole sequence
    if (op.s_out && step == p.nseg - 1)
        store_caller_state<DT, FT>(op.s_out + (int64_t)n * op.so_sn + (int64_t)h * op.so_sh,
                                   op.so_sd, ln, g, S);
    // nothing may still be on its way into LDS when the wavefront ends
    wait_for_stores();

    release_control_block(p, hdr, flags, lane);
}

// Host-side launcher of one element-type combination; (D, F) with D <= 64.
template <typename TA, typename TB, typename TV, typename TO>
void launch_scan_dma(int D, int F, void *workspace, const ScanArgs &args, hipStream_t stream) {
    const dim3 grid((unsigned)args.total_waves), block(kWave);
#define FTC_LAUNCH(DD, FF)                                                                      \
    hipLaunchKernelGGL((scan_dma_kernel<DD, FF, TA, TB, TV, TO>), grid, block, 0, stream,       \
                       (uint32_t *)workspace, args)
    if (D == 64 && F == 64) FTC_LAUNCH(64, 64);
    else if (D == 32 && F == 128) FTC_LAUNCH(32, 128);
    else if (D == 32 && F == 32) FTC_LAUNCH(32, 32);
    else if (D == 32 && F == 64) FTC_LAUNCH(32, 64);
    else FTC_LAUNCH(64, 32);
#undef FTC_LAUNCH
}

// Instantiated for all-fp32 scans (ftc_mfma_dma_ffff.hip); with bf16 rows, which need no
// piece split, the register-fed kernel measured as fast or faster.
void launch_scan_dma_ffff(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);

}  // namespace mfma
}  // namespace ftc
