// Workgroup form of the MFMA causal scan for gfx950, all-fp32 rows.
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (REV: j >= l)
//
// Same mathematics, piece split, chunking and state exchange as ftc_mfma_kernel.h, but a
// (chain, L-segment) belongs to a workgroup of NW = F / 32 wavefronts instead of a single
// one.  Wavefront w owns the 32 output columns 32w .. 32w+31: its slab of the D x F state
// (D x 32, D / 2 accumulator registers), its columns of v and of the output.  What all
// wavefronts need -- the a and b rows of a chunk -- is fetched from memory once, cut into
// bf16 pieces once, and shared through LDS:
//
//  * The lanes of the workgroup together fetch the chunk's rows with 16-byte loads,
//    cut every fp32 value into its three bf16 pieces and write the pieces as three
//    row-major bf16 tiles per operand (XOR-swizzled 16-byte slots).
//  * Fragments whose contraction index runs along a row (a; b for Pt = b a^T) are 16-byte
//    LDS reads.  Fragments whose contraction index runs along the chunk (b^T and v for the
//    state update, v^T for Ot += v^T Pt) are read with ds_read_b64_tr_b16, which hands every
//    lane four values of one column: within 16 lanes, lane i receives element i % 4 of the
//    8 bytes addressed by lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4.
//  * With one state slab per wavefront a wavefront needs at most 256 registers, so two
//    workgroups share a SIMD and one's matrix work overlaps the other's piece cutting.
//
// Register layouts (32x32x16 MFMA; lane = (ln = lane % 32, g = lane / 32)):
//  * k-slot t of lane group g in a k-step of 16 carries contraction index 8 g + t when the
//    index runs along a row (natural order), and chunk position 8 (t / 4) + 4 g + t % 4 when
//    it runs along the chunk (the order in which Pt leaves the accumulator).
//  * State tile dt: register r of lane (ln, g) is S[d][f] with f = 32 w + ln and
//    d = 32 dt + 16 (r / 8) + 8 g + r % 8, so that registers 8 k .. 8 k + 7 are the A operand
//    of k-step 2 dt + k in natural order.  The b^T fragments of the state update are read
//    in the matching column order.
#pragma once
#include "ftc_mfma_dma_kernel.h"

namespace ftc {
namespace mfma {

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

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

// Workgroup barrier that waits for this wavefront's LDS traffic only: rows requested from
// memory for the next chunk stay in flight across it (__syncthreads would wait for them).
__device__ __forceinline__ void wg_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Four consecutive fp32 values of a row -> 8 bytes of each of the three piece tiles.
__device__ __forceinline__ void split_quad_to_lds(const u32x4 raw, lds_char *tile, int piece_bytes,
                                                  int addr) {
    uint32_t lo[3], hi[3];
    split_pair<3>(__uint_as_float(raw.x), __uint_as_float(raw.y), lo);
    split_pair<3>(__uint_as_float(raw.z), __uint_as_float(raw.w), hi);
#pragma unroll
    for (int pc = 0; pc < 3; pc++) {
        const u32x2 w = {lo[pc], hi[pc]};
        *(lds_vec2 *)(tile + pc * piece_bytes + addr) = w;
    }
}

// The caller's state <-> the slab registers of wavefront w (layout in the file header).
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

// In ScanArgs the counts are per workgroup here: waves_per_scan / total_waves count
// workgroups, and the flag words and state slots of wavefront w of workgroup t are those of
// "ticket" w * total_waves + t.
template <int D, int F>
__global__ __launch_bounds__(64 * (F / 32), 2) void scan_wg_kernel(uint32_t *__restrict__ ws_ptr,
                                                                   ScanArgs p) {
    constexpr int NW = F / 32;          // wavefronts per workgroup
    constexpr int T = 64 * NW;          // lanes per workgroup
    constexpr int DT = D / 32;          // state tiles per slab
    constexpr int KD = D / 16;          // k-steps over d
    constexpr int RBA = D * 2, RBV = F * 2;             // bytes per row of a bf16 piece tile
    constexpr int kTileA = kChunk * RBA, kTileV = kChunk * RBV;  // bytes per piece tile
    constexpr int QA = D / 4, QV = F / 4;               // 16-byte fp32 quads per row
    constexpr int LA = kChunk * QA / T, LV = kChunk * QV / T;  // quads per lane and chunk
    static_assert(kChunk * QA % T == 0 && kChunk * QV % T == 0, "tile does not divide over lanes");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ln = lane & 31, g = lane >> 5;

    gu32 *hdr = (gu32 *)ws_ptr;
    gu32 *flags = hdr + kHdrWords;
    gfloat *sums = (gfloat *)(hdr + kControlBytes / 4);

    __shared__ __align__(16) char a_mem[3 * kTileA];
    __shared__ __align__(16) char b_mem[3 * kTileA];
    __shared__ __align__(16) char v_mem[3 * kTileV];
    __shared__ uint32_t order_sh;
    lds_char *const a_pc = (lds_char *)a_mem, *const b_pc = (lds_char *)b_mem,
                    *const v_pc = (lds_char *)v_mem;

    // ---- which segment: one ticket per workgroup ----
    Segment sg;
    {
        uint32_t order;
        segment_request(p, flags, wave == 0 ? lane : 1, sg, order);
        if (tid == 0) order_sh = order;
        __syncthreads();
        order = order_sh;
        if (!segment_locate(p, hdr, tid, order, sg)) return;
    }
    const ScanOperands &op = p.scan[sg.scan_id];
    const bool REV = sg.rev;
    const int step = sg.step, n = sg.n, h = sg.h, rows = sg.rows, nchunks = sg.nchunks;
    const int64_t lo = sg.lo;
    const uint32_t total_wgs = (uint32_t)p.total_waves;
    const uint32_t vticket = (uint32_t)wave * total_wgs + sg.ticket;

    const uint32_t a_slb = (uint32_t)op.a_sl * 4, b_slb = (uint32_t)op.b_sl * 4,
                   v_slb = (uint32_t)op.v_sl * 4, o_slb = (uint32_t)op.o_sl * 4;
    const char *a_seg =
        (const char *)op.a + ((int64_t)n * op.a_sn + (int64_t)h * op.a_sh + lo * op.a_sl) * 4;
    const char *b_seg =
        (const char *)op.b + ((int64_t)n * op.b_sn + (int64_t)h * op.b_sh + lo * op.b_sl) * 4;
    const char *v_seg =
        (const char *)op.v + ((int64_t)n * op.v_sn + (int64_t)h * op.v_sh + lo * op.v_sl) * 4;
    char *o_seg = (char *)op.out + ((int64_t)n * op.o_sn + (int64_t)h * op.o_sh + lo * op.o_sl) * 4;
    const __amdgpu_buffer_rsrc_t a_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)a_seg, 0, (rows - 1) * a_slb + D * 4, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t b_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)b_seg, 0, (rows - 1) * b_slb + D * 4, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t v_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)v_seg, 0, (rows - 1) * v_slb + F * 4, kRsrcFlags);
    const __amdgpu_buffer_rsrc_t o_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)o_seg, 0, (rows - 1) * o_slb + F * 4, kRsrcFlags);

    // ---- per-lane addresses ----
    // fetch + cut: quad q of a lane is 16-byte unit q * T + tid of the chunk's tile
    uint32_t a_goff[LA], b_goff[LA], v_goff[LV];  // byte offset inside a chunk (global)
    int a_waddr[LA], v_waddr[LV];                 // byte address inside a piece tile (LDS)
#pragma unroll
    for (int q = 0; q < LA; q++) {
        const int u = q * T + tid, row = u / QA, c4 = u % QA;
        a_goff[q] = (uint32_t)row * a_slb + 16u * c4;
        b_goff[q] = (uint32_t)row * b_slb + 16u * c4;
        a_waddr[q] = Swizzle<RBA>::addr(row, 8 * c4);
    }
#pragma unroll
    for (int q = 0; q < LV; q++) {
        const int u = q * T + tid, row = u / QV, c4 = u % QV;
        v_goff[q] = (uint32_t)row * v_slb + 16u * c4;
        v_waddr[q] = Swizzle<RBV>::addr(row, 8 * c4);
    }
    // row-major fragments of a and b: lane (row = ln, g), k-step ks: columns 16 ks + 8 g + 0..7
    int row_addr[KD];
#pragma unroll
    for (int ks = 0; ks < KD; ks++) row_addr[ks] = Swizzle<RBA>::addr(ln, 32 * ks + 16 * g);
    // transposing reads: lane = 16 G + s supplies 8 bytes of row 8 u + 4 (G / 2) + s / 4 (+ 16 hh)
    //  b^T, tile dt: columns 32 dt + 16 (G % 2) + 8 (x % 2) + 4 (x / 2) + 0..3, x = s % 4
    //  v (this wavefront's slab): columns 32 w + 16 (G % 2) + 4 x + 0..3
    int bt_addr[DT][2], vt_addr[2];
    {
        const int G = lane >> 4, s = lane & 15, x = s & 3;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int row = 8 * u + 4 * (G / 2) + s / 4;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
                bt_addr[dt][u] = Swizzle<RBA>::addr(
                    row, 2 * (32 * dt + 16 * (G % 2) + 8 * (x % 2) + 4 * (x / 2)));
            vt_addr[u] = Swizzle<RBV>::addr(row, 2 * (32 * wave + 16 * (G % 2) + 4 * x));
        }
    }
    // rows 16 .. 31 of a tile have the swizzle keys of rows 0 .. 15
    static_assert(Swizzle<RBA>::kRowsPerBankRow * Swizzle<RBA>::kXor == 16 &&
                      Swizzle<RBV>::kRowsPerBankRow * Swizzle<RBV>::kXor == 16,
                  "swizzle period");
    // causal mask inside a chunk: accumulator register r of lane (i = ln, g) holds row
    // j = 8 (r / 4) + 4 g + r % 4 of Pt
    uint32_t keep[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int j = 8 * (r / 4) + 4 * g + (r % 4);
        keep[r] = (REV ? (j >= ln) : (j <= ln)) ? 0xffffffffu : 0u;
        asm volatile("" : "+v"(keep[r]));
    }
    const uint32_t o_lane = ln * o_slb + 4u * (32 * wave + 4 * g);

    auto chunk_row0 = [&](int c) -> int { return REV ? rows - kChunk * (c + 1) : kChunk * c; };
    auto pass1_row0 = [&](int c) -> int { return c < 0 ? -2 * kChunk : chunk_row0(c); };

    // raw rows on their way from memory
    u32x4 a_raw[LA], b_raw[LA], v_raw[LV];
    auto fetch_b = [&](int row0) {
#pragma unroll
        for (int q = 0; q < LA; q++)
            b_raw[q] = __builtin_amdgcn_raw_buffer_load_b128(
                b_rs, b_goff[q] + (uint32_t)row0 * b_slb, 0, 0);
    };
    auto fetch_v = [&](int row0) {
#pragma unroll
        for (int q = 0; q < LV; q++)
            v_raw[q] = __builtin_amdgcn_raw_buffer_load_b128(
                v_rs, v_goff[q] + (uint32_t)row0 * v_slb, 0, 0);
    };
    auto fetch_a = [&](int row0) {
#pragma unroll
        for (int q = 0; q < LA; q++)
            a_raw[q] = __builtin_amdgcn_raw_buffer_load_b128(
                a_rs, a_goff[q] + (uint32_t)row0 * a_slb, 0, 0);
    };
    auto cut_b = [&]() {
#pragma unroll
        for (int q = 0; q < LA; q++) split_quad_to_lds(b_raw[q], b_pc, kTileA, a_waddr[q]);
    };
    auto cut_a = [&]() {
#pragma unroll
        for (int q = 0; q < LA; q++) split_quad_to_lds(a_raw[q], a_pc, kTileA, a_waddr[q]);
    };
    auto cut_v = [&]() {
#pragma unroll
        for (int q = 0; q < LV; q++) split_quad_to_lds(v_raw[q], v_pc, kTileV, v_waddr[q]);
    };
    auto v_frags = [&](int hh, Frag (&f)[3]) {
#pragma unroll
        for (int pc = 0; pc < 3; pc++)
            f[pc] = lds_frag_tr(v_pc + pc * kTileV + hh * 16 * RBV + vt_addr[0],
                                v_pc + pc * kTileV + hh * 16 * RBV + vt_addr[1]);
    };
    auto bt_frags = [&](int dt, int hh, Frag (&f)[3]) {
#pragma unroll
        for (int pc = 0; pc < 3; pc++)
            f[pc] = lds_frag_tr(b_pc + pc * kTileA + hh * 16 * RBA + bt_addr[dt][0],
                                b_pc + pc * kTileA + hh * 16 * RBA + bt_addr[dt][1]);
    };

    f32x16 S[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) S[dt][r] = 0.f;
    // (3) S += b^T v for the chunk whose pieces are in LDS
    auto update_state = [&](const Frag (&v_frag)[2][3]) {
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                Frag bt[3];
                bt_frags(dt, hh, bt);
                S[dt] = mfma_split<3, 3>(bt, v_frag[hh], S[dt]);
            }
    };

    // the slab of a wavefront is a state of DT x 1 tiles for the exchange
    f32x16 Sx[DT][1];
    StateExchange<DT, 1> xch(flags, sums, (uint32_t)NW * total_wgs, vticket, step, p.nseg, p.group,
                             lane);
    if (p.nseg > 1) {
        // ---- pass 1: the segment's own state sum, walked against the direction of pass 2 ----
        if (xch.need_own_sum) {
            fetch_b(pass1_row0(nchunks - 1));
            fetch_v(pass1_row0(nchunks - 1));
            for (int c = nchunks - 1; c >= 0; c--) {
                cut_b();
                cut_v();
                fetch_b(pass1_row0(c - 1));
                fetch_v(pass1_row0(c - 1));
                wg_barrier();
                Frag v_frag[2][3];
                v_frags(0, v_frag[0]);
                v_frags(1, v_frag[1]);
                update_state(v_frag);
                wg_barrier();
            }
#pragma unroll
            for (int dt = 0; dt < DT; dt++) Sx[dt][0] = S[dt];
            xch.publish_sum(Sx);
        }
    }
    // ---- first chunk of pass 2 (requested before waiting for the other workgroups) ----
    fetch_a(chunk_row0(0));
    fetch_b(chunk_row0(0));
    fetch_v(chunk_row0(0));
    if (p.nseg > 1) {
        f32x16 X[DT][1];
#pragma unroll
        for (int dt = 0; dt < DT; dt++) Sx[dt][0] = S[dt];
        xch.gather(Sx, X);
        if (xch.failed && lane == 0)
            __hip_atomic_store(hdr + kHdrError, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int dt = 0; dt < DT; dt++) S[dt] = X[dt][0];
    }
    if (op.s0)
        wg_add_caller_state<DT>(op.s0 + (int64_t)n * op.s0_sn + (int64_t)h * op.s0_sh, op.s0_sd,
                                32 * wave + ln, g, S);

    // ---- pass 2: outputs ----
    for (int c = 0; c < nchunks; c++) {
        const int row0 = chunk_row0(c);
        cut_a();
        cut_b();
        cut_v();
        // rows of the chunk after the last one are outside the descriptors and read as zero
        fetch_a(chunk_row0(c + 1));
        fetch_b(chunk_row0(c + 1));
        fetch_v(chunk_row0(c + 1));
        wg_barrier();

        // (1) Pt = b a^T (every wavefront needs all of it)
        f32x16 P;
#pragma unroll
        for (int r = 0; r < 16; r++) P[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            Frag af[3], bf[3];
#pragma unroll
            for (int pc = 0; pc < 3; pc++) {
                af[pc] = lds_frag16(a_pc + pc * kTileA + row_addr[ks]);
                bf[pc] = lds_frag16(b_pc + pc * kTileA + row_addr[ks]);
            }
            P = mfma_split<3, 3>(bf, af, P);
        }
        // (2b) Ot = S^T a^T while Pt is on its way
        f32x16 O;
#pragma unroll
        for (int r = 0; r < 16; r++) O[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KD; ks++) {
            const int o8 = 8 * (ks % 2);
            const float x[8] = {S[ks / 2][o8 + 0], S[ks / 2][o8 + 1], S[ks / 2][o8 + 2],
                                S[ks / 2][o8 + 3], S[ks / 2][o8 + 4], S[ks / 2][o8 + 5],
                                S[ks / 2][o8 + 6], S[ks / 2][o8 + 7]};
            Frag s_frag[3], af[3];
            split8<3>(x, s_frag);
#pragma unroll
            for (int pc = 0; pc < 3; pc++) af[pc] = lds_frag16(a_pc + pc * kTileA + row_addr[ks]);
            O = mfma_split<3, 3>(s_frag, af, O);
        }
        // mask and cut Pt
#pragma unroll
        for (int r = 0; r < 16; r++) P[r] = __uint_as_float(__float_as_uint(P[r]) & keep[r]);
        Frag p_frag[2][3];
#pragma unroll
        for (int hh = 0; hh < 2; hh++) {
            const float x[8] = {P[8 * hh + 0], P[8 * hh + 1], P[8 * hh + 2], P[8 * hh + 3],
                                P[8 * hh + 4], P[8 * hh + 5], P[8 * hh + 6], P[8 * hh + 7]};
            split8<3>(x, p_frag[hh]);
        }
        // (2a) Ot += v^T Pt
        Frag v_frag[2][3];
        v_frags(0, v_frag[0]);
        v_frags(1, v_frag[1]);
#pragma unroll
        for (int hh = 0; hh < 2; hh++) O = mfma_split<3, 3>(v_frag[hh], p_frag[hh], O);
        // lane (i = ln, g) holds f = 32 w + 8 q + 4 g + 0..3 in registers 4 q .. 4 q + 3
        const uint32_t o_off = o_lane + (uint32_t)row0 * o_slb;
#pragma unroll
        for (int q = 0; q < 4; q++)
            buffer_store4(o_rs, o_off + (uint32_t)(4 * 8 * q), O[4 * q + 0], O[4 * q + 1],
                          O[4 * q + 2], O[4 * q + 3]);
        // (3) S += b^T v
        update_state(v_frag);
        wg_barrier();
    }
    if (op.s_out && step == p.nseg - 1)
        wg_store_caller_state<DT>(op.s_out + (int64_t)n * op.so_sn + (int64_t)h * op.so_sh,
                                  op.so_sd, 32 * wave + ln, g, S);

    // the last wavefront of the launch leaves the control block zeroed
    if (p.nseg > 1) {
        uint32_t done = 0;
        if (lane == 0)
            done = __hip_atomic_fetch_add(hdr + kHdrDone, 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
        done = __builtin_amdgcn_readfirstlane(done);
        if (done == (uint32_t)NW * total_wgs - 1) {
            for (uint32_t i = lane; i < (uint32_t)NW * total_wgs; i += kWave)
                __hip_atomic_store(flags + i, kFlagEmpty, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            for (uint32_t i = lane; i < total_wgs / (uint32_t)p.nseg; i += kWave)
                __hip_atomic_store(flags + kMaxWaves + i, 0u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            if (lane == 0)
                __hip_atomic_store(hdr + kHdrDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// (D, F) with D in {32, 64} and F in {32, 64, 128}
void launch_scan_wg_ffff(int D, int F, void *ws, const ScanArgs &args, hipStream_t stream);
bool scan_wg_covers(int D, int F);

}  // namespace mfma
}  // namespace ftc
