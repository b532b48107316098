// Host side of the MFMA scan (kernel: ftc_mfma_kernel.h): which scans qualify, how L is cut
// into segments, workspace size, and the launch.
#include <algorithm>
#include <cstdint>
#include <cstdlib>

#include "ftc_wg_kernel.h"

namespace ftc {
using namespace mfma;
namespace {

struct MfmaPlan {
    int nseg, seg_len;
    int64_t waves, workspace_bytes;
};

// all-fp32 scans of these widths run as workgroups of F / 32 wavefronts (ftc_wg_kernel.h)
bool use_wg_kernel(int64_t D, int64_t F, int nscans, int64_t L, bool all_f32) {
    if (!all_f32 || !scan_wg_covers((int)D, (int)F)) return false;
    if (tuning().wg >= 0) return tuning().wg != 0;  // tuning aid
    // Measured: a single scan over long chains (the forward) is 2-7 % faster in workgroup
    // form (cfg3 forward 331 us against 349, N=8, H=16, L=4096: 164 against 177); launches of
    // three scans and short chains are faster with one wavefront per segment.
    return nscans == 1 && L >= 128 * kChunk && D == 64 && F == 64;
}

// Row widths that the chain-parallel kernel takes (ftc_tp_kernel.h): states of 16 x 16 to
// 128 x 128, walked in blocks of 64 rows, with one workgroup per block of 64 output columns;
// widths that are multiples of 4 (a lane's 16 bytes lie wholly inside a row or wholly outside).
// (`forced`: a part of a scan that the caller has split because only this kernel takes it;
// then any multiple of 4 will do)
bool tp_widths(int64_t D, int64_t F, bool forced = false) {
    const int64_t least = forced ? 4 : 16;
    return D >= least && D <= 128 && F >= least && F <= 512 && D % 4 == 0 && F % 4 == 0;
}
int64_t tp_fblocks(int64_t F) { return (F + 63) / 64; }

// whether the kernels that split L take fp32 rows of these widths (as column slices, if need be)
bool mfma_scan_supported_widths(int64_t D, int64_t F) {
    int widths[kMfmaMaxSlices];
    return mfma_slice_widths(D, F, widths) > 0;
}

// all-fp32 scans can run one workgroup per chain (and block of 64 output columns) with no
// split of L (ftc_tp_kernel.h).  `units`: chains x scans x column blocks; `wide`: a state
// other than 64 x 64, for which the kernels that split L are half as fast as for 64 x 64;
// `others`: one of those kernels takes this shape (else the choice is the VALU kernel).
// Returns the number of segments per chain (0: another kernel takes the launch).
int tp_kernel_segments(int64_t units, int64_t L, bool wide, bool others, bool long_chains = false,
                       bool cut_long = false, int64_t most_units = 512, int64_t brief_chunks = 0) {
    // a chain is walked by one workgroup from end to end: beyond 256 chunks the split of L
    // of the other kernels is faster, and its segment sums also keep the rounding of a long
    // running state in check (`long_chains`: the caller knows better, see tp_plan_compute)
    if (L > (long_chains ? 1024 : 256) * kChunk) return 0;
    // One workgroup per CU at a time.  A workgroup that takes a whole chain reads every row
    // once; with fewer chains than CUs a chain is cut into up to four segments whose
    // workgroups each rebuild the state before their segment by themselves (a state-only
    // chunk costs a bit more than half of a full one), as long as that fills at least half the GPU.
    const int64_t total_chunks = (L + kChunk - 1) / kChunk;
    int nseg = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(4, 256 / units), total_chunks));
    if (tuning().tp_segs >= 0) nseg = std::max(1, std::min(tuning().tp_segs, 16));  // tuning aid
    if (tuning().tp >= 0) return tuning().tp != 0 ? nseg : 0;                       // tuning aid
    // Measured (forward, us, N=10 H=8): cfg2 (L=1000) 30 against 42 for the kernels that split
    // L and exchange states; L=3000: 75 against 84; L=4096: 100 against 108; L=8192: 201
    // against 201 -- cut chains pay off while the chunks that a workgroup walks for its
    // state alone are few.
    if (nseg > 1 && total_chunks > 128) {
        if (!wide && !long_chains) return 0;
        if (!wide) nseg = 1;
        // (`cut_long`: shapes that never exchange keep their cuts: 32 x 128, 64 chains, L=8192,
        // forward: 190 us in two segments against 219 whole and 206 on the kernels that split L)
        if (!cut_long) nseg = 1;
    }
    // (wide states: the other kernels run them as column slices that each repeat the chunk
    // product, and lose at any number of rounds; on a quarter of the CUs they still win, N=1,
    // H=8, L=2048, 128 x 128 forward: 52 against 91 us.  The VALU kernel loses always.)
    // (chains of up to `brief_chunks` chunks at any number, see tp_plan_compute)
    const bool brief = total_chunks <= brief_chunks;
    if (wide) return !others || brief || units * nseg >= 128 ? nseg : 0;
    // Beyond `most_units` workgroups the other kernels win again (short chains: there every
    // chain has its own wavefront, all resident at once, and nothing is split either).
    return (brief || units * nseg >= (long_chains ? 112 : 128)) && units <= most_units ? nseg : 0;
}

// Where to cut a chain of `chunks` chunks into (at most) `nseg` segments for the
// chain-parallel kernel.  The workgroup of a segment first rebuilds the state before its
// segment from the chunks in front of it (measured: 0.55 to 0.6 of the time of a chunk that
// also produces rows -- 0.75 against 1.3 us on the fp16-piece kernel with every workgroup
// streaming rows), so later segments are made shorter until all workgroups finish together:
// the starts (multiples of kTpAhead chunks, what the producers request ahead) that minimise the
// longest workgroup.  Returns the number of segments; start[0 .. n] filled (start[n] = chunks).
int tp_segment_starts(int64_t chunks, int nseg, int32_t *start) {
    const int groups = (int)((chunks + kTpAhead - 1) / kTpAhead);
    nseg = std::max(1, std::min(std::min(nseg, groups), kMaxTpSegments));
    double kStateOnly = 0.6;
    if (tuning().tp_ratio >= 0) kStateOnly = tuning().tp_ratio;  // tuning aid
    // best[s][g]: smallest achievable longest time of segments s .. nseg-1 when segment s
    // starts at group g (dynamic programme from the last segment back)
    constexpr int kMaxGroups = 64;  // 256 chunks
    if (groups > kMaxGroups || nseg == 1) {
        start[0] = 0, start[1] = (int32_t)chunks;
        return 1;
    }
    double best[kMaxTpSegments + 1][kMaxGroups + 1];
    int next[kMaxTpSegments + 1][kMaxGroups + 1];
    for (int s = 0; s <= nseg; s++)
        for (int g = 0; g <= groups; g++) best[s][g] = 1e30, next[s][g] = groups;
    best[nseg][groups] = 0.0;
    for (int s = nseg - 1; s >= 0; s--)
        for (int g = s; g < groups; g++)
            for (int e = g + 1; e <= groups - (nseg - 1 - s); e++) {
                const double t = std::max(kStateOnly * g + (e - g), best[s + 1][e]);
                if (t < best[s][g]) best[s][g] = t, next[s][g] = e;
            }
    int g = 0;
    for (int s = 0; s < nseg; s++) {
        start[s] = kTpAhead * g;
        g = next[s][g];
    }
    start[nseg] = (int32_t)chunks;
    return nseg;
}

// Longer chains on few CUs: the chain-parallel kernel with an exchange of segment sums.  A
// chain is cut into as many equal segments as fill the GPU (one workgroup each); a workgroup
// walks its own chunks twice, first for their state alone.  Returns the number of chunks per
// segment (0: not this way) and the number of segments in *nseg.
int tp_exchange_segments(int64_t units, int64_t L, bool wide, int *nseg, bool keep_two = false) {
    const int64_t total_chunks = (L + kChunk - 1) / kChunk;
    *nseg = 0;
    if (tuning().tpx == 0) return 0;  // tuning aid
    // Up to 64 chunks the cut chains without an exchange are as fast (cfg2: 30 us either way)
    // and need no workspace -- unless the chains are so few that four or more segments of each
    // fit one round of workgroups: those win from 24 chunks on, also against the kernels that
    // split L (64 x 64 forward, us, this way / before: 16 chains, L=2048: 28 / 44, L=1024:
    // 21 / 28; 8 chains, L=2048: 23 / 31; 32 chains, L=2048: 34 / 42; backward of 8 chains,
    // L=2048: 31 / 38, of 4: 26 / 37; 128 x 128 forward, 16 chains, L=2048: 50 / 81).
    const bool force = tuning().tpx_segs >= 2;  // tuning aid: also where the rules below say no
    const bool brief = total_chunks <= 64;
    // (not for one or two workgroups' worth of chains, 22 against 21 us, and from 33 on only
    // from 48 chunks: backward of 16 chains, L=1024: 34 against 26 cut in five without an exchange)
    if (!force && (units < 1 || total_chunks < 24)) return 0;
    if (!force && brief && (units < 3 || units > 64 || (units > 32 && total_chunks < 48))) return 0;
    // (more workgroups than CUs: only where chains are too long to walk whole)
    if (!force && units > 128 && total_chunks <= 256) return 0;
    int64_t want = 256 / units;
    // the number of segments with the shortest estimated time, rounds x (a segment walked
    // twice + the exchange and the start, in chunks' time)
    // (wide states: twelve chunks' time for those -- with six, 128 x 128 backward of 16 chains,
    // L=4096, went into three rounds of 16-chunk segments, 202 us, where two segments take 185)
    auto shortest = [&](double twice, double fixed) {
        double best = 1e30;
        for (int64_t n = std::max<int64_t>(2, (total_chunks + 255) / 256); n <= 64; n++) {
            const int64_t c = ((total_chunks + n - 1) / n + kTpAhead - 1) / kTpAhead * kTpAhead;
            const int64_t rounds = (units * ((total_chunks + c - 1) / c) + 255) / 256;
            const double t = (double)rounds * (twice * (double)c + fixed);
            if (t < best - 1e-9) best = t, want = n;
        }
    };
    if (wide) {
        // workgroups that do not fill whole rounds of 256 (the first walk at 0.4 of the cost)
        if (units * want != 256) shortest(1.4, 12.0);
    } else if (want < 2 || (total_chunks + want - 1) / want > 256) {
        // 64 x 64 with no single round of segments of at most 256 chunks: a few rounds still
        // beat the kernels that split L while those have no more than a wavefront or two per
        // SIMD to run (backward, ms, this way with the segments chosen here / split L:
        // N*H = 16, L=65536: 0.71 / 0.79; 32, L=32768: 0.72 / 0.82; 64, L=16384: 0.80 / 0.91;
        // 128, L=16384: 1.36 / 1.56; but 256, L=16384: 2.70 / 2.60.  Ten segments at N*H = 16
        // against 8: 0.83, 11: 0.82, 16: 0.79 -- the last round wants to be full).
        if (!force && units > 384) return 0;
        shortest(1.0, 40.0);
    }
    // Two segments of up to 64 chunks lose to chains cut in two without an exchange, whose
    // first workgroup walks its part once (forward, 96 chains, L=4096: 117 against 100 us; 128
    // chains: 145 against 128; backward of 32 chains: 110 against 95); with three segments the
    // exchange wins again (backward of 24 chains: 83 against 86; forward of 64: 73 against 88).
    // Wider states the same (64 x 128 forward, 64 chains, L=4096: 116 against 104; 128 x 128
    // backward of 16 chains: 204 against 186).
    // (`keep_two`: the caller compares with other kernels, not with cut chains)
    if (!force && !keep_two && want == 2 && total_chunks <= 128) return 0;
    // segments of at least four chunks (one or two chains, L=4096: 32 segments 21.5 us, 16: 25.1)
    want = std::min<int64_t>(want, total_chunks / 4);
    if (tuning().tpx_segs >= 0) want = std::max(1, tuning().tpx_segs);  // tuning aid
    if (want < 2) return 0;
    const int64_t seg_chunks = ((total_chunks + want - 1) / want + kTpAhead - 1) / kTpAhead * kTpAhead;
    const int64_t n = (total_chunks + seg_chunks - 1) / seg_chunks;
    // a workgroup walks at most 256 chunks with one running state (rounding), a chain has
    // at most 64 x 64 steps (flags of a group are watched by one wavefront), and every
    // consumer of every segment has a flag word
    if (n < 2 || seg_chunks > 256 || n > 4096 || 4 * units * n > kMaxWaves) return 0;
    *nseg = (int)n;
    return (int)seg_chunks;
}

// The chain-parallel kernel's plan for `nscans` scans of a D x F state over chains x L rows:
// *seg_chunks > 0: an exchange with *nseg segments of that many chunks; else *nseg > 0: chains
// cut into *nseg segments that need no exchange; both 0: another kernel takes the launch.
// `mixed`: rows with bf16 among them (the fp16-piece form of the kernel takes those; the plans
// are those of fp32 rows where the kernel is used at all).
// `mixed`: kMixedRows: rows with bf16 among them; kMixedGradValues: a single scan of bf16 a and b
// whose values are fp32 (the dV scan of a bf16 backward)
constexpr int kMixedRows = 1, kMixedGradValues = 2;
void tp_plan_compute(int64_t D, int64_t F, int64_t chains, int nscans, int64_t L, int *nseg,
                     int *seg_chunks, bool forced, int mixed) {
    *nseg = *seg_chunks = 0;
    if (!tp_widths(D, F, forced)) return;
    const bool wide = D != 64 || F != 64 || forced;
    const bool others = !forced && mfma_scan_supported_widths(D, F);
    const int64_t units = chains * nscans * tp_fblocks(F);
    // A single scan over bf16 rows: the kernels that split L multiply such rows as they are,
    // one matrix instruction per product, and win while this kernel has workgroups for fewer
    // than half of the CUs (forward, 64 x 64, L=1000, N*H = 80: 32 against 36 us, 96: 33
    // against 36, 112: 38 against 36, 128: 42 against 37, 192: 53 against 42) or would need
    // an exchange (N*H = 128, L=4096: 114 against 132 us; L=8192: 208 against 241; without one,
    // N*H = 192, L=4096: 160 against 140).  The three scans of a backward call are faster
    // here for up to 128 chains (L=1000, N*H = 80: 50 against 101 us).
    const bool lone_mixed = mixed && nscans == 1 && others;
    if (lone_mixed && units < 112) return;
    // (N*H = 128, L=1024: 35 against 38 us; L=2048: 61 against 54)
    if (lone_mixed && units < 192 && L > 48 * kChunk) return;
    // Shapes of the other kernels with 32 rows or columns (a workgroup here has half of its
    // matrix work or half of its consumers to spare for them): measured at N=8, H=16, L=4096,
    // forward + backward, 32 x 128 0.62 against 0.80 ms and 128 x 32 0.76 against 0.78 on whole
    // chains, but 32 x 32 0.34 against 0.28, and with an exchange (N=4, H=16, L=16384)
    // 128 x 32 1.73 against 1.58 and 32 x 128 1.70 against 1.59: those stay where they were.
    const bool narrow = others && (D <= 32 || F <= 32);
    // Chains too short for an exchange (fewer than 24 chunks) run here on any number of
    // workgroups: the kernels that split L pay more for their exchange than a workgroup for
    // walking the chain (64 x 64 forward, 8 chains, L=640: 19 against 27 us; 128 x 128 backward, 4
    // chains, L=512: 29 against 62).  A single scan on the bf16-piece kernel, and its scans with
    // half of the consumers idle, only up to 8 chunks (128 x 128 forward, 2 chains, L=256: 16
    // against 17, L=512: 22 against 17; 128 x 32 forward, 8 chains, L=512: 27 against 20).
    const int64_t brief_chunks = D <= 64 || (F > 32 && nscans >= 2) ? 23 : 8;
    if (narrow && D <= 32 && F <= 32) return;
    // A single scan over bf16 rows in blocks of 64 output columns reads a and b once per block:
    // beyond two rounds of workgroups, or one for a state of 32 rows, the kernels that split L
    // win (64 x 128, 512 chains, L=512: 92 against 58 us, L=2048: 309 against 272; 256 chains:
    // 149 against 175.  32 x 128, 256 chains, L=1024: 75 against 58; 128 chains: 40 against 40)
    if (lone_mixed && units > (narrow ? 256 : 512)) return;
    // ... and so do thousands of chains of one or two chunks with a state of at most 64 x 64,
    // where a workgroup's start costs more than its chunks (8192 chains, L=64: 32 x 128 1.17
    // against 0.60 ms, 20 x 20 0.63 against 0.46 on padded copies), and 32-wide shapes on more
    // than two rounds of workgroups, as for 64 x 64.
    // (four rounds for a state of 32 rows on chains of 32 chunks or more: 32 x 128 forward, 384
    // chains, L=1024: 113 against 174 us; 512 chains, L=2048: 277 against 344; 1024 chains: 293 / 279)
    if (narrow && units > (D <= 32 && L >= 32 * kChunk ? 1024 : 512) && tuning().tp < 0) return;
    // ... and 32-wide shapes on few workgroups: a workgroup of this kernel walks its chunks at
    // 1.1 to 1.7 us each whatever else the GPU does, the kernels that split L spread them over
    // all CUs (forward, us, this kernel / those: 32 x 128, 32 chains, L=4096: 83 / 62; 16 chains:
    // 78 / 54; 64 chains, 128 workgroups: 94 / 106.  128 x 32, 32 chains, L=4096: 152 / 69; 64
    // chains: 170 / 103; 128 chains: 227 / 204, L=2048: 107 / 101; 256 chains: 317 / 383).  Short
    // chains stay (32 x 128, 32 chains, L=1024: 29 / 39; 128 x 32, 64 chains, L=512: 32 / 36),
    // and 64 x 32 on the fp16-piece kernel needs 128 workgroups like 32 x 64 (128 chains,
    // L=2048: 51 / 57, L=8192: 210 / 229; 64 chains, L=1024: 28 / 32, L=2048: 47 / 41).
    if (narrow && tuning().tp < 0) {
        const int64_t total_chunks = (L + kChunk - 1) / kChunk;
        // a single scan on the bf16-piece kernel with half of its consumers without columns
        const bool lone_slab = F <= 32 && D > 64 && nscans == 1;
        int64_t least = 64, brief = lone_slab ? 16 : 32;
        // (the kernels that split L run 96 columns as slices: 32 x 96, 16 chains, L=2048: 44 / 73)
        if (D <= 32 && F == 96) least = 32, brief = 64;
        if (total_chunks > brief_chunks && units < (lone_slab ? 256 : 128) &&
            !(units >= least && total_chunks <= brief))
            return;
    }
    if (!forced && D <= 64 && F <= 64 && units > 512 && L <= 2 * kChunk) return;
    // fp32 64 x 64 chains of 257 to 1024 chunks on 112 workgroups or more are walked whole: a
    // running fp32 state of that length is what the reference keeps too (L=32768 against float64:
    // scale errors 1.8e-6 forward and 3e-6 backward where the reference's own order has 1.1e-6 and
    // 4e-6), and a workgroup per chain and scan reads every row once where an exchange reads it
    // twice and the kernels that split L more often (us, whole / before: forward, 256 chains,
    // L=16384: 883 / 1061; 128 chains: 485 / 537; backward of 64 chains: 559 / 704; of 256: 2082
    // / 2626; of 256 at L=32768: 4134 / 5290; of 36 chains, 108 workgroups: 466 / 419).
    // The same for the other states that the fp16-piece kernel takes, from 192 workgroups on, 128
    // beyond 512 chunks (64 x 128 forward, 128 chains, L=16384: 662 against 1049 us; 64 chains,
    // L=32768: 910 against 1083, L=16384: 458 against 452; 48 x 80, 64 chains, L=16384: 470 / 405).  Not for the bf16-piece kernel: 128 x 128 walked whole at L=12000 is outside the
    // element-wise bound 2.8 times as often as the reference's own order, where twice is the bar.
    // (32-wide states included: 32 x 128 forward, 128 chains, L=16384: 553 against 756; 64 x 32
    // backward, 256 chains, L=12000: 1404 against 1825)
    // ... and the three scans of a backward call over bf16 rows, whose results are rounded to
    // bf16 anyway, from 192 workgroups on (64 chains, L=16384: 634 against 783 us; 256 chains:
    // 1783 against 2430; 43 chains: 512 against 483)
    const bool mixed_backward = mixed == kMixedRows && nscans == 3;
    const bool walk_long = (!mixed || mixed_backward) && D <= 64 && L > 256 * kChunk &&
                           L <= 1024 * kChunk &&
                           units >= (mixed_backward ? 192 : !wide ? 112 : L > 512 * kChunk ? 128 : 192);
    if (!narrow && !walk_long) *seg_chunks = tp_exchange_segments(units, L, wide, nseg, lone_mixed);
    if (lone_mixed && units < 256 && *seg_chunks > 0) {
        *nseg = *seg_chunks = 0;
        return;
    }
    // ... and so do the three scans of a backward call over bf16 rows where the exchange would
    // have two segments per chain or more than one round of workgroups (32 chains, L=8192: 232
    // against 201 us, L=16384: 448 against 364; 16 chains, five segments each: 109 against 168
    // and 194 against 227)
    if (mixed == kMixedRows && nscans == 3 && *seg_chunks > 0 && units * 3 > 256) {
        *nseg = *seg_chunks = 0;
        return;
    }
    // The dV scan of a bf16 backward with a state of at most 32 rows and a workgroup for every
    // CU is walked whole however long the chain: what the kernels that split L read twice there
    // is the fp32 gradient, the widest operand by far (N=4, H=32, L=16384, 32 x 128: 0.485
    // against 0.629 ms; the forward of the same shape, whose wide operand is the fp32 result
    // that either kernel writes once, loses: 0.656 against 0.495).  bf16 results make the
    // rounding of a long running fp32 state a non-issue.
    const bool long_chains = walk_long || (mixed == kMixedGradValues && D <= 32 && units == 256);
    // The three scans of a backward call over bf16 rows stay here for up to six rounds of
    // workgroups: the kernels that split L, good at many fp32 chains, multiply bf16 rows as they
    // are but re-read them in a first pass (backward, us, this kernel / those: 256 chains, L=1024:
    // 116 / 172; 512 chains, L=2048: 471 / 593; 768 chains, L=512: 227 / 196, L=2048: 701 / 732).
    // fp32 rows, 64 x 64: any number of chains of 16 chunks or more (the fp16-piece kernel walks
    // them faster than the kernels that split L stream them: backward, 256 chains, L=4096: 528
    // against 694 us; 768 chains, L=2048: 784 against 1013; forward, 1536 chains, L=1024: 309
    // against 376); from 8 chunks on three rounds of workgroups for a single scan and nine for
    // the three of a backward call (L=256: backward of 384 chains 71 against 82, of 768 chains
    // 136 against 146, of 2048 chains 327 against 295; forward of 768 chains 50 against 50, of
    // 1024 chains 65 against 56), two below that (256 chains, L=128: 31 against 27)
    const int64_t chunks = (L + kChunk - 1) / kChunk;
    const int64_t most_units = mixed == kMixedRows && nscans == 3 ? 1536
                               : mixed              ? 512
                               : chunks >= 16       ? INT64_MAX
                               : chunks >= 8        ? (nscans == 3 ? 2304 : 768)
                                                    : 512;
    if (*seg_chunks == 0)
        *nseg = tp_kernel_segments(units, L, wide, others, long_chains, narrow, most_units, brief_chunks);
}

// workspace of the exchange: control block, then two state slots (own sum, group total) of
// D x 16 floats (D rounded up to whole blocks of 64 rows) per consumer, four consumers per segment
int64_t tp_exchange_workspace_bytes(int64_t units, int nseg, int64_t D) {
    return kControlBytes + 2 * 4 * units * nseg * (int64_t)((D + 63) / 64 * 64 * 16 * 4);
}

// `wg`: the plan is for workgroups of F / 32 wavefronts (each has its own flag words);
// `norm`: for their fused attention form, with one more wavefront and state slab per unit
MfmaPlan make_plan_compute(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F, int nscans,
                           bool wg, bool norm) {
    MfmaPlan pl;
    const int64_t flags_per_unit = wg ? F / 32 + (norm ? 1 : 0) : 1;
    const int64_t chains = std::max<int64_t>(1, N * H);
    const int64_t total_chunks = (L + kChunk - 1) / kChunk;
    // Resident at a time: 1024 wavefronts (one per SIMD: register footprint), or one workgroup
    // per CU with 4 / (F / 32) segments each.  Pick the segment
    // length (in chunks) that minimises an estimate of the makespan: rounds of resident
    // wavefronts times the work of one wavefront (pass 1 costs about half of pass 2, the
    // exchange of segment sums about three chunks).
    const int64_t slots = wg ? 256 * scan_wg_units_per_block((int)F, norm) : 1024;
    int64_t best_c = total_chunks;
    double best_cost = (double)total_chunks * (double)((chains * nscans + slots - 1) / slots);
    for (int64_t c = 1; c < total_chunks && c <= 4096; c++) {
        const int64_t nseg = (total_chunks + c - 1) / c;
        const int64_t waves = chains * nseg;
        if (waves * nscans * flags_per_unit > kMaxWaves || nseg > 4096) continue;  // <= 64 groups of 64 steps
        const double rounds = (double)((waves * nscans + slots - 1) / slots);
        // (the exchange: a step reads the sums of its group and the totals of the groups before
        // it one after the other, about a chunk and a half's time each beyond the first four;
        // bf16 forward, 32 chains, L=1024: segments of 1 / 2 / 4 / 8 chunks 34 / 23 / 23 / 29 us)
        double reads = (double)(nseg - 1);
        if (nseg > 5) {
            int64_t g = 1;
            while (g * g < nseg) g++;
            reads = (double)((g - 1) + ((nseg + g - 1) / g - 1));
        }
        // (states of up to 64 x 64 only: on wider ones a chunk takes longer and the reads weigh
        // less -- 128 x 32, 8 chains, L=4096: segments of 4 chunks 51 us, of 8 chunks 69)
        const double look_back = D <= 64 && F <= 64 ? 1.6 * std::max(0.0, reads - 4.0) : 0.0;
        const double per_wave = nseg > 1 ? c * 1.5 + 3.0 + look_back : (double)c;
        const double cost = rounds * per_wave;
        if (cost < best_cost - 1e-9) {
            best_cost = cost;
            best_c = c;
        }
    }
    // tuning aid: FTC_SEG_CHUNKS=<n> forces segments of n chunks
    if (tuning().seg_chunks >= 0) {
        const int64_t forced = tuning().seg_chunks;
        if (forced >= 1 && forced <= total_chunks) {
            const int64_t nseg = (total_chunks + forced - 1) / forced;
            if (chains * nseg * nscans * flags_per_unit <= kMaxWaves && nseg <= 4096) best_c = forced;
        }
    }
    pl.seg_len = (int)(best_c * kChunk);
    pl.nseg = (int)((L + pl.seg_len - 1) / pl.seg_len);
    pl.waves = chains * pl.nseg;
    pl.workspace_bytes = 0;
    if (pl.nseg > 1)
        pl.workspace_bytes = kControlBytes + 2 * nscans * pl.waves * D * (F + (norm ? 32 : 0)) *
                                                 (int64_t)sizeof(float);
#ifdef FTC_TIMELINE
    pl.workspace_bytes += nscans * pl.waves * 128;  // time stamps (ftc_wg_kernel.h)
#endif
    return pl;
}

// Plans depend on the sizes alone and a caller repeats the same sizes call after call (the
// segment search walks up to 4096 candidates for a long sequence): the last plans of every
// thread are kept, keyed by their arguments and by the generation of the tuning variables.
template <typename Value>
struct PlanMemo {
    static constexpr int kEntries = 32;
    struct Entry {
        int64_t key[8];
        uint64_t generation;
        Value value;
    };
    Entry entry[kEntries] = {};
    template <typename Compute>
    Value get(const int64_t (&key)[8], Compute compute) {
        uint64_t h = 1469598103934665603ull;
        for (int64_t k : key) h = (h ^ (uint64_t)k) * 1099511628211ull;
        Entry &e = entry[h % kEntries];
        const uint64_t generation = tuning().generation;
        bool hit = e.generation == generation;
        for (int i = 0; i < 8 && hit; i++) hit = e.key[i] == key[i];
        if (!hit) {
            e.value = compute();
            for (int i = 0; i < 8; i++) e.key[i] = key[i];
            e.generation = generation;
        }
        return e.value;
    }
};
struct TpPlan {
    int nseg, seg_chunks;
};
void tp_plan(int64_t D, int64_t F, int64_t chains, int nscans, int64_t L, int *nseg, int *seg_chunks,
             bool forced = false, int mixed = 0) {
    static thread_local PlanMemo<TpPlan> memo;
    const int64_t key[8] = {D, F, chains, nscans, L, forced ? 1 : 0, mixed, 0};
    const TpPlan pl = memo.get(key, [&]() {
        TpPlan p;
        tp_plan_compute(D, F, chains, nscans, L, &p.nseg, &p.seg_chunks, forced, mixed);
        return p;
    });
    *nseg = pl.nseg, *seg_chunks = pl.seg_chunks;
}
MfmaPlan make_plan(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F, int nscans, bool wg,
                   bool norm = false) {
    static thread_local PlanMemo<MfmaPlan> memo;
    const int64_t key[8] = {N, H, L, D, F, nscans, wg ? 1 : 0, norm ? 1 : 0};
    return memo.get(key, [&]() { return make_plan_compute(N, H, L, D, F, nscans, wg, norm); });
}

// every row must start on a 16-byte boundary (16-byte loads and stores)
bool aligned16(const void *ptr, int64_t s0, int64_t s1, int64_t s2, int dtype) {
    const int per16 = dtype == FTC_F32 ? 4 : 8;
    return ((uintptr_t)ptr % 16 == 0) && s0 % per16 == 0 && s1 % per16 == 0 && s2 % per16 == 0;
}

// what the chain-parallel kernel asks of rows: fp32 rows on 16-byte boundaries, bf16 rows (which
// it reads and writes four values at a time) on 8-byte boundaries
bool aligned_quads(const void *ptr, int64_t s0, int64_t s1, int64_t s2, int dtype) {
    if (dtype == FTC_F32) return aligned16(ptr, s0, s1, s2, dtype);
    return ((uintptr_t)ptr % 8 == 0) && s0 % 4 == 0 && s1 % 4 == 0 && s2 % 4 == 0;
}

// element-type combinations with a compiled kernel: (a, b, v, out)
enum Combo { kNone = 0, kFFFF, kBBBF, kFBBB, kBFBB, kBBFB };
Combo combo_of(const ScanDesc &sd) {
    const int a = sd.a.dtype, b = sd.b.dtype, v = sd.v.dtype, o = sd.out.dtype;
    const int F32 = FTC_F32, B16 = FTC_BF16;
    if (a == F32 && b == F32 && v == F32 && o == F32) return kFFFF;  // every fp32 scan
    if (a == B16 && b == B16 && v == B16 && o == F32) return kBBBF;  // bf16 forward
    if (a == F32 && b == B16 && v == B16 && o == B16) return kFBBB;  // bf16 dQ (a = grad_out)
    if (a == B16 && b == F32 && v == B16 && o == B16) return kBFBB;  // bf16 dK (b = grad_out)
    if (a == B16 && b == B16 && v == F32 && o == B16) return kBBFB;  // bf16 dV (v = grad_out)
    return kNone;
}

// chain-parallel scans of states of up to 64 rows run on the fp16 matrix path
// (ftc_tph_kernel.h: two scaled fp16 pieces per value), wider ones on three bf16 pieces
bool tph_takes_rows(int64_t D) {
    return D <= 64 && tuning().tph != 0;  // (FTC_TPH=0: tuning aid)
}

// rows must not overlap (the descriptor's end marks the first row outside the segment) and
// row strides must keep a segment's byte extent inside a 32-bit buffer descriptor
bool stride_ok(int64_t stride_l, int width) { return stride_l >= width && stride_l <= (1 << 16); }

}  // namespace

int mfma_slice_widths(int64_t D, int64_t F, int (&widths)[kMfmaMaxSlices]) {
    // the widest state a wavefront holds is 4096 values
    const int widest = D == 32 ? 128 : D == 64 ? 64 : (D == 96 || D == 128) ? 32 : 0;
    if (widest == 0 || F < 32 || F % 32 != 0) return 0;
    int n = 0;
    for (int64_t left = F; left > 0;) {
        int w = widest;
        while (w > left) w /= 2;
        if (n == kMfmaMaxSlices) return 0;
        widths[n++] = w;
        left -= w;
    }
    return n;
}

ScanDesc mfma_slice(const ScanDesc &scan, int col0, int width) {
    ScanDesc s = scan;
    const int vb = scan.v.dtype == FTC_F32 ? 4 : 2, ob = scan.out.dtype == FTC_F32 ? 4 : 2;
    s.v.ptr = (const char *)scan.v.ptr + (int64_t)col0 * vb;
    s.v.width = width;
    s.out.ptr = (char *)scan.out.ptr + (int64_t)col0 * ob;
    s.out.width = width;
    if (s.initial.ptr) s.initial.ptr += col0;
    if (s.final_.ptr) s.final_.ptr += col0;
    return s;
}

bool mfma_scan_same_launch(const ScanDesc &x, const ScanDesc &y) {
    return combo_of(x) == combo_of(y) && x.a.width == y.a.width && x.v.width == y.v.width;
}

bool mfma_operand_in_place(const void *ptr, int64_t stride_n, int64_t stride_h, int64_t stride_l,
                           int dtype, int width, int64_t L) {
    return (L <= 1 || stride_ok(stride_l, width)) && aligned16(ptr, stride_n, stride_h, stride_l, dtype);
}

bool mfma_scan_supported(const ScanDesc &sd, int64_t L) {
    const Operand &a = sd.a, &b = sd.b, &v = sd.v;
    const OperandOut &out = sd.out;
    const int D = a.width, F = v.width;
    const bool shape_ok = (D == 64 && F == 64) || (D == 32 && F == 128) || (D == 128 && F == 32) ||
                          (D == 32 && F == 32) || (D == 32 && F == 64) || (D == 64 && F == 32) ||
                          (D == 96 && F == 32);
    if (!shape_ok) return false;
    if (combo_of(sd) == kNone) return false;
    if (L > 1 && !(stride_ok(a.stride_l, D) && stride_ok(b.stride_l, D) &&
                   stride_ok(v.stride_l, F) && stride_ok(out.stride_l, F)))
        return false;
    return aligned16(a.ptr, a.stride_n, a.stride_h, a.stride_l, a.dtype) &&
           aligned16(b.ptr, b.stride_n, b.stride_h, b.stride_l, b.dtype) &&
           aligned16(v.ptr, v.stride_n, v.stride_h, v.stride_l, v.dtype) &&
           aligned16(out.ptr, out.stride_n, out.stride_h, out.stride_l, out.dtype);
}

int64_t mfma_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F,
                                  int nscans) {
    // whichever kernel the element types will select
    int64_t bytes = std::max(make_plan(N, H, L, D, F, nscans, false).workspace_bytes,
                             make_plan(N, H, L, D, F, nscans, true).workspace_bytes);
    return std::max(bytes, mfma_tp_workspace_bytes(N, H, L, D, F, nscans));
}

int64_t mfma_tp_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F, int nscans,
                                bool forced) {
    int nseg = 0, seg_chunks = 0;
    const int64_t chains = std::max<int64_t>(1, N * H);
    tp_plan(D, F, chains, nscans, L, &nseg, &seg_chunks, forced);
    return seg_chunks > 0 ? tp_exchange_workspace_bytes(chains * nscans * tp_fblocks(F), nseg, D) : 0;
}

bool mfma_tp_takes(const ScanDesc *scans, int nscans, int64_t N, int64_t H, int64_t L, bool forced) {
    const int D = scans[0].a.width, F = scans[0].v.width;
    if (nscans < 1 || nscans > kMaxScans || !tp_widths(D, F, forced)) return false;
    int64_t widest_stride = 0;
    int mixed = nscans == 1 && combo_of(scans[0]) == kBBFB ? kMixedGradValues : 0;
    for (int i = 0; i < nscans; i++) {
        const ScanDesc &sd = scans[i];
        const Combo combo = combo_of(sd);
        if (combo != kFFFF && mixed == 0) mixed = kMixedRows;
        // rows with bf16 among them: the fp16-piece form of the kernel only
        if (combo == kNone || (combo != kFFFF && !tph_takes_rows(D))) return false;
        if (sd.a.width != D || sd.v.width != F) return false;
        if (L > 1 && !(stride_ok(sd.a.stride_l, D) && stride_ok(sd.b.stride_l, D) &&
                       stride_ok(sd.v.stride_l, F) && stride_ok(sd.out.stride_l, F)))
            return false;
        if (!(aligned_quads(sd.a.ptr, sd.a.stride_n, sd.a.stride_h, sd.a.stride_l, sd.a.dtype) &&
              aligned_quads(sd.b.ptr, sd.b.stride_n, sd.b.stride_h, sd.b.stride_l, sd.b.dtype) &&
              aligned_quads(sd.v.ptr, sd.v.stride_n, sd.v.stride_h, sd.v.stride_l, sd.v.dtype) &&
              aligned_quads(sd.out.ptr, sd.out.stride_n, sd.out.stride_h, sd.out.stride_l, sd.out.dtype)))
            return false;
        widest_stride = std::max(widest_stride, std::max(std::max(sd.a.stride_l, sd.b.stride_l),
                                                         std::max(sd.v.stride_l, sd.out.stride_l)));
    }
    // the chain-parallel kernel addresses a whole chain through one 32-bit descriptor
    if ((L + 2 * kChunk) * std::max<int64_t>(widest_stride, std::max(D, F)) * 4 >= 0x7fffffffLL)
        return false;
    int nseg = 0, seg_chunks = 0;
    tp_plan(D, F, std::max<int64_t>(1, N * H), nscans, L, &nseg, &seg_chunks, forced, mixed);
    return nseg > 0;
}

bool fused_attention_supported(const ScanDesc &sd, int64_t L) {
    return combo_of(sd) == kFFFF && !sd.reverse && !sd.initial.ptr && !sd.final_.ptr &&
           scan_wg_norm_covers(sd.a.width, sd.v.width) && mfma_scan_supported(sd, L);
}

int64_t fused_attention_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F) {
    return make_plan(N, H, L, D, F, 1, true, true).workspace_bytes;
}

int mfma_scan(const ScanDesc *scans, int nscans, int64_t N, int64_t H, int64_t L,
              void *workspace, size_t workspace_bytes, hipStream_t stream,
              const FusedAttention *fused, bool may_chain_parallel, bool forced) {
    if (nscans < 1 || nscans > kMaxScans) return fail(FTC_ERR_INVALID, "bad scan count");
    const int D = scans[0].a.width, F = scans[0].v.width;
    const Combo combo = combo_of(scans[0]);
    if (fused && (nscans != 1 || !fused_attention_supported(scans[0], L)))
        return fail(FTC_ERR_UNSUPPORTED, "no fused attention kernel for this shape or layout");
    const bool tp_shape = !fused && may_chain_parallel && mfma_tp_takes(scans, nscans, N, H, L, forced);
    const int64_t chains = std::max<int64_t>(1, N * H);
    const int64_t fblocks = tp_shape ? tp_fblocks(F) : 1;
    int tpx_nseg = 0, tpx_seg_chunks = 0, tp_nseg = 0;
    if (tp_shape) {
        int any_bf16 = nscans == 1 && combo == kBBFB ? kMixedGradValues : 0;
        for (int i = 0; i < nscans; i++)
            if (combo_of(scans[i]) != kFFFF && any_bf16 == 0) any_bf16 = kMixedRows;
        tp_plan(D, F, chains, nscans, L, &tpx_nseg, &tpx_seg_chunks, forced, any_bf16);
        if (tpx_seg_chunks == 0) tp_nseg = tpx_nseg, tpx_nseg = 0;
    }
    const bool tp = tp_nseg > 0 || tpx_seg_chunks > 0;
    if (!tp && !mfma_scan_supported(scans[0], L))
        return fail(FTC_ERR_UNSUPPORTED, "no MFMA kernel takes a %d x %d state here", D, F);
    const bool wg = fused || use_wg_kernel(D, F, nscans, L, combo == kFFFF);
    MfmaPlan pl = make_plan(N, H, L, D, F, nscans, wg, fused != nullptr);
    int32_t tp_start[kMaxTpSegments + 1] = {0};
    if (tpx_seg_chunks > 0) {  // one workgroup per chain segment, segment sums exchanged
        pl.nseg = tpx_nseg;
        pl.seg_len = tpx_seg_chunks * kChunk;
        pl.waves = chains * pl.nseg;
        pl.workspace_bytes = tp_exchange_workspace_bytes(chains * nscans * fblocks, pl.nseg, D);
    } else if (tp) {  // one workgroup per chain segment, nothing to exchange
        pl.nseg = tp_segment_starts((L + kChunk - 1) / kChunk, tp_nseg, tp_start);
        pl.seg_len = (int)L;
        pl.waves = chains * pl.nseg;
        pl.workspace_bytes = 0;
    }
    if (!plan_only()) {
        if (pl.workspace_bytes > 0 && (!workspace || workspace_bytes < (size_t)pl.workspace_bytes))
            return fail(FTC_ERR_WORKSPACE, "workspace of %lld bytes needed, %zu given",
                        (long long)pl.workspace_bytes, workspace_bytes);
        if (pl.workspace_bytes > 0 && (uintptr_t)workspace % 256 != 0)
            return fail(FTC_ERR_WORKSPACE, "workspace must be 256-byte aligned");
    }

    ScanArgs args;
    int64_t max_stride = 0;
    for (int i = 0; i < kMaxScans; i++) {
        const ScanDesc &sd = scans[i < nscans ? i : 0];
        ScanOperands &o = args.scan[i];
        o.a = sd.a.ptr, o.b = sd.b.ptr, o.v = sd.v.ptr;
        o.out = sd.out.ptr;
        // With a single position the row stride addresses nothing, but the kernels still
        // step over the 31 absent rows of the chunk with it: those must fall outside the
        // one-row descriptor, so a stride below the row width is replaced by the width.
        auto row_stride = [L](int64_t stride_l, int width) {
            return L == 1 ? std::max<int64_t>(stride_l, width) : stride_l;
        };
        o.a_sn = sd.a.stride_n, o.a_sh = sd.a.stride_h, o.a_sl = row_stride(sd.a.stride_l, D);
        o.b_sn = sd.b.stride_n, o.b_sh = sd.b.stride_h, o.b_sl = row_stride(sd.b.stride_l, D);
        o.v_sn = sd.v.stride_n, o.v_sh = sd.v.stride_h, o.v_sl = row_stride(sd.v.stride_l, F);
        o.o_sn = sd.out.stride_n, o.o_sh = sd.out.stride_h, o.o_sl = row_stride(sd.out.stride_l, F);
        o.rev = sd.reverse ? 1 : 0;
        // (element types of the rows, for the kernel that takes them scan by scan)
        o.pad = (sd.a.dtype == FTC_BF16 ? kRowsBf16A : 0) | (sd.b.dtype == FTC_BF16 ? kRowsBf16B : 0) |
                (sd.v.dtype == FTC_BF16 ? kRowsBf16V : 0) | (sd.out.dtype == FTC_BF16 ? kRowsBf16Out : 0);
        o.s0 = sd.initial.ptr;
        o.s0_sn = sd.initial.stride_n, o.s0_sh = sd.initial.stride_h, o.s0_sd = sd.initial.stride_d;
        o.s_out = sd.final_.ptr;
        o.so_sn = sd.final_.stride_n, o.so_sh = sd.final_.stride_h, o.so_sd = sd.final_.stride_d;
        if (fused && fused->denominators)  // (the fused form has no state to hand out)
            o.s_out = fused->denominators, o.so_sn = fused->den_sn, o.so_sh = fused->den_sh, o.so_sd = 0;
        max_stride = std::max(max_stride, std::max(std::max(sd.a.stride_l, sd.b.stride_l),
                                                   std::max(sd.v.stride_l, sd.out.stride_l)));
    }
    // buffer descriptors address a segment with 32-bit byte offsets
    if ((int64_t)((tp ? L : (int64_t)pl.seg_len) + 2 * kChunk) * max_stride * 4 >= 0x7fffffffLL)
        return fail(FTC_ERR_UNSUPPORTED, "segment too long for 32-bit offsets");
    args.L = L;
    args.eps = fused ? fused->eps : 0.f;
    args.key_len = fused ? fused->key_lengths : nullptr;
#ifdef FTC_TIMELINE
    if (tp)  // tuning aid: where the chain-parallel kernel writes its time stamps
        if (const char *env = getenv("FTC_STAMP_PTR"))  // (a build for measurements only)
            args.key_len = (const int64_t *)(uintptr_t)strtoull(env, nullptr, 0);
#endif
    args.H = (int32_t)H;
    args.seg_len = pl.seg_len;
    for (int i = 0; i <= kMaxTpSegments; i++) args.tp_start[i] = tp_start[i];
    args.tp_exchange = tpx_seg_chunks > 0 ? 1 : 0;
    args.tp_seg_chunks = tpx_seg_chunks;
    args.nseg = pl.nseg;
    args.waves_per_scan = (int32_t)pl.waves;
    args.total_waves = (int32_t)(pl.waves * nscans * fblocks);
    args.tp_d = D, args.tp_f = F, args.tp_fblocks = (int32_t)fblocks;
    // very short chains: one level (every step adds the sums of all steps before it);
    // otherwise groups of about sqrt(nseg) steps, which moves fewer states per step
    args.group = pl.nseg;
    if (pl.nseg > 5) {
        args.group = 1;
        while (args.group * args.group < pl.nseg) args.group++;
    }
    // tuning aid: FTC_GROUP=<n> forces groups of n steps
    if (tuning().group >= 0) args.group = std::max(1, tuning().group);
    // a wavefront watches one flag per lane: at most 64 steps per group and 64 groups
    args.group = std::min(args.group, 64);
    while ((pl.nseg + args.group - 1) / args.group > 64) args.group++;

    const bool half_pieces = tp && tph_takes_rows(D);
    bool mixed = false;  // rows with bf16 among them
    for (int i = 0; i < nscans; i++) {
        mixed = mixed || combo_of(scans[i]) != kFFFF;
        if ((!half_pieces && combo_of(scans[i]) != combo) || scans[i].a.width != D || scans[i].v.width != F)
            return fail(FTC_ERR_INVALID, "scans of one launch must share widths and dtypes");
    }
    // fp32 states of up to 64 rows: the kernel that feeds its fragments from LDS tiles
    bool dma = D <= 64 && combo == kFFFF;
    if (tuning().dma >= 0) dma = dma && tuning().dma != 0;  // tuning aid
    note_kernel(tp ? (half_pieces ? (tpx_seg_chunks > 0 ? "scan_tph_kernel (exchange)" : "scan_tph_kernel")
                                  : (tpx_seg_chunks > 0 ? "scan_tp_kernel (exchange)" : "scan_tp_kernel"))
                : wg ? (fused ? "scan_wg_kernel<NORM>" : "scan_wg_kernel")
                : dma ? "scan_dma_kernel" : "scan_mfma_kernel");
    if (plan_only()) {
        char cuts[160] = "";
        if (tp && tpx_seg_chunks == 0)
            for (int i = 0, at = 0; i <= pl.nseg && at < 140; i++)
                at += snprintf(cuts + at, sizeof(cuts) - at, "%s%d", i ? "," : ", cuts at chunks ",
                               (int)args.tp_start[i]);
        note_plan("%s: %d scan%s (%s), state %d x %d, %lld chains, %d segment%s of %d rows%s, "
                  "%lld workgroups or wavefronts, workspace %lld bytes",
                  ftc_last_kernel(), nscans, nscans == 1 ? "" : "s",
                  scans[0].reverse ? "first one reverse" : "first one forward", D, F,
                  (long long)chains, (int)pl.nseg, pl.nseg == 1 ? "" : "s", (int)pl.seg_len, cuts,
                  (long long)args.total_waves, (long long)pl.workspace_bytes);
        return FTC_OK;
    }
    if (tp) {
        if (half_pieces)
            launch_scan_tph(workspace, args, mixed, stream);
        else
            launch_scan_tp(workspace, args, stream);
    } else if (wg) {
        launch_scan_wg_ffff(D, F, fused != nullptr, workspace, args, stream);
    } else if (dma) {
        launch_scan_dma_ffff(D, F, workspace, args, stream);
    } else switch (combo) {
        case kFFFF: launch_scan_ffff(D, F, workspace, args, stream); break;
        case kBBBF: launch_scan_bbbf(D, F, workspace, args, stream); break;
        case kFBBB: launch_scan_fbbb(D, F, workspace, args, stream); break;
        case kBFBB: launch_scan_bfbb(D, F, workspace, args, stream); break;
        case kBBFB: launch_scan_bbfb(D, F, workspace, args, stream); break;
        default: return fail(FTC_ERR_UNSUPPORTED, "no MFMA kernel for this dtype combination");
    }
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(FTC_ERR_HIP, "MFMA scan launch failed: %s", hipGetErrorString(err));
    return FTC_OK;
}

}  // namespace ftc
