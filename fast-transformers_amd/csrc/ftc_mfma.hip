// MFMA causal scan for gfx950, fp32 rows, row widths D, F in {32, 64, 128} (D*F <= 4096).
//
//   out[c, l, f] = sum_{j <= l} (a[c,l,:] . b[c,j,:]) * v[c,j,f]      (REV: j >= l)
//
// One wavefront owns one (chain, L-segment) and walks it in chunks of 32 positions with
// the whole D x F state in its accumulator registers; wavefronts never synchronise with
// each other.  Per chunk (i, j index positions of the chunk, all products on
// v_mfma_f32_32x32x16_bf16, written in the transposed orientation so that every chained
// operand is already in registers):
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
// Register-chaining: a 32x32 accumulator holds, in lane (col = lane % 32, g = lane / 32),
// rows 8*(r/4) + 4*g + (r%4) for r = 0..15.  Registers 8h..8h+7 are therefore 8 values
// of the contraction index for k-step h, provided the other operand uses the same order:
// k-slot (g, t) of a 16-wide k-step carries logical index 8*(t/4) + 4*g + (t%4).  LDS
// tiles are stored with that order inside every 16-block (blocks of 4 swapped: 0,2,1,3),
// so one ds_read_b128 yields a fragment.
#include <algorithm>

#include "ftc_common.h"

namespace ftc {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// LDS is written as 8-byte and read as 16-byte words of the same bf16 data
typedef uint32_t lds_u32x2 __attribute__((ext_vector_type(2), may_alias));
typedef uint32_t lds_u32x4 __attribute__((ext_vector_type(4), may_alias));

constexpr int kChunk = 32;
constexpr int kWave = 64;

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

// position of logical index x inside its 16-block for x a multiple of 4
__device__ __forceinline__ int perm4(int x) {
    // blocks of four: 0,1,2,3 -> 0,2,1,3
    const int blk = (x >> 2) & 3;
    const int swapped = ((blk & 1) << 1) | (blk >> 1);
    return (x & ~15) | (swapped << 2);
}

struct MfmaArgs {
    const float *a, *b, *v;
    float *out;
    float *states;  // [chain][segment][D*F], accumulator-register order
    int64_t a_sn, a_sh, a_sl;
    int64_t b_sn, b_sh, b_sl;
    int64_t v_sn, v_sh, v_sl;
    int64_t o_sn, o_sh, o_sl;
    int64_t L;
    int32_t H, seg_len, nseg;
    int32_t state_only;
};

template <int D, int F, int NS>
struct Lds {
    // per row: NS planes of the row's bf16 values, then 16 bytes of padding (keeps the
    // row pitch at 4 (mod 8) dwords so that ds_read_b128 by 8 consecutive rows is
    // conflict free)
    static constexpr int kRowB = NS * D * 2 + 16;        // B_s[j][plane][pos(d)]
    static constexpr int kRowT = NS * kChunk * 2 + 16;   // Bt_s[d][plane][pos(j)], Vt_s[f][..]
    static constexpr int kOffB = 0;
    static constexpr int kOffBt = kOffB + kChunk * kRowB;
    static constexpr int kOffVt = kOffBt + D * kRowT;
    static constexpr int kBytes = kOffVt + F * kRowT;
};

template <int D, int F, int NS, bool REV>
__global__ __launch_bounds__(kWave) void scan_mfma_kernel(MfmaArgs p) {
    using Lay = Lds<D, F, NS>;
    constexpr int DT = D / 32, FT = F / 32;  // state tiles
    constexpr int KD = D / 16;               // k-steps over d
    constexpr int BLK_B = (kChunk / 4) * (D / 4) / kWave;  // 4x4 blocks of b per lane
    constexpr int BLK_V = (kChunk / 4) * (F / 4) / kWave;
    __shared__ __align__(16) unsigned char lds[Lay::kBytes];

    const int lane = threadIdx.x;
    const int ln = lane & 31, g = lane >> 5;

    const int64_t wg = blockIdx.x;
    const int seg = (int)(wg % p.nseg);
    const int64_t chain = wg / p.nseg;
    const int n = (int)(chain / p.H), h = (int)(chain % p.H);
    const int64_t lo = (int64_t)seg * p.seg_len;
    const int64_t hi = min(p.L, lo + (int64_t)p.seg_len);
    const bool full = !p.state_only;

    const float *a_base = p.a + (int64_t)n * p.a_sn + (int64_t)h * p.a_sh;
    const float *b_base = p.b + (int64_t)n * p.b_sn + (int64_t)h * p.b_sh;
    const float *v_base = p.v + (int64_t)n * p.v_sn + (int64_t)h * p.v_sh;
    float *o_base = p.out + (int64_t)n * p.o_sn + (int64_t)h * p.o_sh;
    float *my_state = p.states ? p.states + (chain * p.nseg + seg) * (int64_t)(D * F) : nullptr;

    f32x16 S[DT][FT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int ft = 0; ft < FT; ft++) {
            if (full && p.nseg > 1) {
#pragma unroll
                for (int r = 0; r < 16; r++)
                    S[dt][ft][r] = my_state[((dt * FT + ft) * 16 + r) * kWave + lane];
            } else {
#pragma unroll
                for (int r = 0; r < 16; r++) S[dt][ft][r] = 0.f;
            }
        }

    // raw fp32 of the chunk being staged
    float4 a_raw[KD][2];
    float4 b_raw[BLK_B][4];
    float4 v_raw[BLK_V][4];
    const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);

    auto chunk_start = [&](int c) -> int64_t {
        return REV ? hi - (int64_t)kChunk * (c + 1) : lo + (int64_t)kChunk * c;
    };
    auto load_chunk = [&](int64_t t0) {
        if (full) {
            const int64_t t = t0 + ln;
            const bool ok = t >= lo && t < hi;
            const float *row = a_base + t * p.a_sl;
#pragma unroll
            for (int ks = 0; ks < KD; ks++) {
                a_raw[ks][0] = ok ? *(const float4 *)(row + 16 * ks + 4 * g) : zero4;
                a_raw[ks][1] = ok ? *(const float4 *)(row + 16 * ks + 8 + 4 * g) : zero4;
            }
        }
#pragma unroll
        for (int u = 0; u < BLK_B; u++) {
            const int id = lane + kWave * u;
            const int jb = id / (D / 4), dq = id % (D / 4);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int64_t tok = t0 + 4 * jb + t;
                const bool ok = tok >= lo && tok < hi;
                b_raw[u][t] = ok ? *(const float4 *)(b_base + tok * p.b_sl + 4 * dq) : zero4;
            }
        }
#pragma unroll
        for (int u = 0; u < BLK_V; u++) {
            const int id = lane + kWave * u;
            const int jb = id / (F / 4), fq = id % (F / 4);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int64_t tok = t0 + 4 * jb + t;
                const bool ok = tok >= lo && tok < hi;
                v_raw[u][t] = ok ? *(const float4 *)(v_base + tok * p.v_sl + 4 * fq) : zero4;
            }
        }
    };

    const int nchunks = (int)((hi - lo + kChunk - 1) / kChunk);
    if (nchunks > 0) load_chunk(chunk_start(0));

    for (int c = 0; c < nchunks; c++) {
        const int64_t t0 = chunk_start(c);

        // ---- stage b (row and transposed layouts) and v (transposed) as bf16 pieces ----
#pragma unroll
        for (int u = 0; u < BLK_B; u++) {
            const int id = lane + kWave * u;
            const int jb = id / (D / 4), dq = id % (D / 4);
            const float xs[4][4] = {
                {b_raw[u][0].x, b_raw[u][0].y, b_raw[u][0].z, b_raw[u][0].w},
                {b_raw[u][1].x, b_raw[u][1].y, b_raw[u][1].z, b_raw[u][1].w},
                {b_raw[u][2].x, b_raw[u][2].y, b_raw[u][2].z, b_raw[u][2].w},
                {b_raw[u][3].x, b_raw[u][3].y, b_raw[u][3].z, b_raw[u][3].w}};
            // pieces packed along d (for B_s rows) ...
            uint32_t row_lo[4][NS], row_hi[4][NS];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                split_pair<NS>(xs[t][0], xs[t][1], row_lo[t]);
                split_pair<NS>(xs[t][2], xs[t][3], row_hi[t]);
            }
            if (full) {
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int pl = 0; pl < NS; pl++) {
                        unsigned char *dst = lds + Lay::kOffB + (4 * jb + t) * Lay::kRowB +
                                             pl * D * 2 + perm4(4 * dq) * 2;
                        *(lds_u32x2 *)dst = lds_u32x2{row_lo[t][pl], row_hi[t][pl]};
                    }
            }
            // ... and along j (for Bt_s rows): same pieces, regrouped by 16-bit halves
#pragma unroll
            for (int cdx = 0; cdx < 4; cdx++)
#pragma unroll
                for (int pl = 0; pl < NS; pl++) {
                    uint32_t w0, w1;
                    const uint32_t s0 = (cdx < 2) ? row_lo[0][pl] : row_hi[0][pl];
                    const uint32_t s1 = (cdx < 2) ? row_lo[1][pl] : row_hi[1][pl];
                    const uint32_t s2 = (cdx < 2) ? row_lo[2][pl] : row_hi[2][pl];
                    const uint32_t s3 = (cdx < 2) ? row_lo[3][pl] : row_hi[3][pl];
                    if ((cdx & 1) == 0) {  // low halves
                        w0 = __builtin_amdgcn_perm(s1, s0, 0x05040100u);
                        w1 = __builtin_amdgcn_perm(s3, s2, 0x05040100u);
                    } else {  // high halves
                        w0 = __builtin_amdgcn_perm(s1, s0, 0x07060302u);
                        w1 = __builtin_amdgcn_perm(s3, s2, 0x07060302u);
                    }
                    unsigned char *dst = lds + Lay::kOffBt + (4 * dq + cdx) * Lay::kRowT +
                                         pl * kChunk * 2 + perm4(4 * jb) * 2;
                    *(lds_u32x2 *)dst = lds_u32x2{w0, w1};
                }
        }
#pragma unroll
        for (int u = 0; u < BLK_V; u++) {
            const int id = lane + kWave * u;
            const int jb = id / (F / 4), fq = id % (F / 4);
            const float xs[4][4] = {
                {v_raw[u][0].x, v_raw[u][0].y, v_raw[u][0].z, v_raw[u][0].w},
                {v_raw[u][1].x, v_raw[u][1].y, v_raw[u][1].z, v_raw[u][1].w},
                {v_raw[u][2].x, v_raw[u][2].y, v_raw[u][2].z, v_raw[u][2].w},
                {v_raw[u][3].x, v_raw[u][3].y, v_raw[u][3].z, v_raw[u][3].w}};
#pragma unroll
            for (int cdx = 0; cdx < 4; cdx++) {
                uint32_t o01[NS], o23[NS];
                split_pair<NS>(xs[0][cdx], xs[1][cdx], o01);
                split_pair<NS>(xs[2][cdx], xs[3][cdx], o23);
#pragma unroll
                for (int pl = 0; pl < NS; pl++) {
                    unsigned char *dst = lds + Lay::kOffVt + (4 * fq + cdx) * Lay::kRowT +
                                         pl * kChunk * 2 + perm4(4 * jb) * 2;
                    *(lds_u32x2 *)dst = lds_u32x2{o01[pl], o23[pl]};
                }
            }
        }

        // ---- a: straight into B-operand fragments ----
        Frag a_frag[KD][NS];
        if (full) {
#pragma unroll
            for (int ks = 0; ks < KD; ks++) {
                const float x[8] = {a_raw[ks][0].x, a_raw[ks][0].y, a_raw[ks][0].z, a_raw[ks][0].w,
                                    a_raw[ks][1].x, a_raw[ks][1].y, a_raw[ks][1].z, a_raw[ks][1].w};
                split8<NS>(x, a_frag[ks]);
            }
        }

        // raw registers are free again: fetch the next chunk while this one is computed
        if (c + 1 < nchunks) load_chunk(chunk_start(c + 1));

        // single wavefront: LDS writes above are ordered before the reads below
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // fragments of vt: A operand of (2a) and B operand of (3)
        Frag v_frag[FT][2][NS];
#pragma unroll
        for (int ft = 0; ft < FT; ft++)
#pragma unroll
            for (int hh = 0; hh < 2; hh++)
#pragma unroll
                for (int pl = 0; pl < NS; pl++) {
                    const unsigned char *src = lds + Lay::kOffVt + (32 * ft + ln) * Lay::kRowT +
                                               pl * kChunk * 2 + (16 * hh + 8 * g) * 2;
                    const lds_u32x4 q = *(const lds_u32x4 *)src;
                    v_frag[ft][hh][pl] = Frag{{q.x, q.y, q.z, q.w}};
                }

        if (full) {
            // (1) Pt = b a^T
            f32x16 P;
#pragma unroll
            for (int r = 0; r < 16; r++) P[r] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KD; ks++) {
                Frag bA[NS];
#pragma unroll
                for (int pl = 0; pl < NS; pl++) {
                    const unsigned char *src = lds + Lay::kOffB + ln * Lay::kRowB + pl * D * 2 +
                                               (16 * ks + 8 * g) * 2;
                    const lds_u32x4 q = *(const lds_u32x4 *)src;
                    bA[pl] = Frag{{q.x, q.y, q.z, q.w}};
                }
                P = mfma_split<NS>(bA, a_frag[ks], P);
            }
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

            // (2a) + (2b) per output tile, then store
            const int64_t tok = t0 + ln;
            const bool row_ok = tok >= lo && tok < hi;
#pragma unroll
            for (int ft = 0; ft < FT; ft++) {
                f32x16 O;
#pragma unroll
                for (int r = 0; r < 16; r++) O[r] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KD; ks++) {
                    const float x[8] = {S[ks / 2][ft][8 * (ks % 2) + 0], S[ks / 2][ft][8 * (ks % 2) + 1],
                                        S[ks / 2][ft][8 * (ks % 2) + 2], S[ks / 2][ft][8 * (ks % 2) + 3],
                                        S[ks / 2][ft][8 * (ks % 2) + 4], S[ks / 2][ft][8 * (ks % 2) + 5],
                                        S[ks / 2][ft][8 * (ks % 2) + 6], S[ks / 2][ft][8 * (ks % 2) + 7]};
                    Frag s_frag[NS];
                    split8<NS>(x, s_frag);
                    O = mfma_split<NS>(s_frag, a_frag[ks], O);
                }
#pragma unroll
                for (int hh = 0; hh < 2; hh++) O = mfma_split<NS>(v_frag[ft][hh], p_frag[hh], O);
                if (row_ok) {
                    float *orow = o_base + tok * p.o_sl + 32 * ft + 4 * g;
#pragma unroll
                    for (int q = 0; q < 4; q++)
                        *(float4 *)(orow + 8 * q) =
                            make_float4(O[4 * q + 0], O[4 * q + 1], O[4 * q + 2], O[4 * q + 3]);
                }
            }
        }

        // (3) S += b^T v
#pragma unroll
        for (int hh = 0; hh < 2; hh++)
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                Frag btA[NS];
#pragma unroll
                for (int pl = 0; pl < NS; pl++) {
                    const unsigned char *src = lds + Lay::kOffBt + (32 * dt + ln) * Lay::kRowT +
                                               pl * kChunk * 2 + (16 * hh + 8 * g) * 2;
                    const lds_u32x4 q = *(const lds_u32x4 *)src;
                    btA[pl] = Frag{{q.x, q.y, q.z, q.w}};
                }
#pragma unroll
                for (int ft = 0; ft < FT; ft++)
                    S[dt][ft] = mfma_split<NS>(btA, v_frag[ft][hh], S[dt][ft]);
            }

        // the next iteration overwrites the LDS tiles read above
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }

    if (p.state_only) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int ft = 0; ft < FT; ft++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    my_state[((dt * FT + ft) * 16 + r) * kWave + lane] = S[dt][ft][r];
    }
}

// In place: states[chain][s] <- sum over s' < s (s' > s when reversed); any element order.
__global__ __launch_bounds__(256) void state_scan_kernel(float *states, int nseg, int64_t elems,
                                                         int reverse) {
    const int64_t blocks_per_chain = (elems + 255) / 256;
    const int64_t chain = blockIdx.x / blocks_per_chain;
    const int64_t e = (blockIdx.x % blocks_per_chain) * 256 + threadIdx.x;
    if (e >= elems) return;
    float *base = states + chain * nseg * elems + e;
    float run = 0.f;
    for (int i = 0; i < nseg; i++) {
        const int s = reverse ? nseg - 1 - i : i;
        const float x = base[(int64_t)s * elems];
        base[(int64_t)s * elems] = run;
        run += x;
    }
}

struct MfmaPlan {
    int nseg, seg_len;
    int64_t workspace_bytes;
};

MfmaPlan make_plan(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F) {
    MfmaPlan pl;
    const int64_t chains = std::max<int64_t>(1, N * H);
    // one wavefront per SIMD is what the LDS footprint allows: aim for ~2 waves of work
    // per SIMD (2048 wavefronts) with segments of at least 4 chunks
    int64_t want = (2048 + chains - 1) / chains;
    int64_t max_seg = std::max<int64_t>(1, L / (4 * kChunk));
    int64_t nseg = std::max<int64_t>(1, std::min(want, max_seg));
    int64_t seg_len = (L + nseg - 1) / nseg;
    seg_len = (seg_len + kChunk - 1) / kChunk * kChunk;
    nseg = std::max<int64_t>(1, (L + seg_len - 1) / seg_len);
    pl.nseg = (int)nseg;
    pl.seg_len = (int)seg_len;
    pl.workspace_bytes = nseg > 1 ? chains * nseg * D * F * (int64_t)sizeof(float) : 0;
    return pl;
}

template <int D, int F>
void launch(const MfmaArgs &args, int64_t wgs, bool reverse, hipStream_t stream) {
    if (reverse)
        hipLaunchKernelGGL((scan_mfma_kernel<D, F, 3, true>), dim3((unsigned)wgs), dim3(kWave), 0,
                           stream, args);
    else
        hipLaunchKernelGGL((scan_mfma_kernel<D, F, 3, false>), dim3((unsigned)wgs), dim3(kWave), 0,
                           stream, args);
}

bool aligned16(const void *ptr, int64_t s0, int64_t s1, int64_t s2) {
    return ((uintptr_t)ptr % 16 == 0) && s0 % 4 == 0 && s1 % 4 == 0 && s2 % 4 == 0;
}

}  // namespace

bool mfma_scan_supported(const Operand &a, const Operand &b, const Operand &v,
                         const OperandOut &out) {
    const int D = a.width, F = v.width;
    const bool shape_ok = (D == 64 && F == 64) || (D == 32 && F == 128) || (D == 128 && F == 32);
    if (!shape_ok) return false;
    if (a.dtype != FTC_F32 || b.dtype != FTC_F32 || v.dtype != FTC_F32 || out.dtype != FTC_F32)
        return false;
    return aligned16(a.ptr, a.stride_n, a.stride_h, a.stride_l) &&
           aligned16(b.ptr, b.stride_n, b.stride_h, b.stride_l) &&
           aligned16(v.ptr, v.stride_n, v.stride_h, v.stride_l) &&
           aligned16(out.ptr, out.stride_n, out.stride_h, out.stride_l);
}

int64_t mfma_scan_workspace_bytes(int64_t N, int64_t H, int64_t L, int64_t D, int64_t F) {
    return make_plan(N, H, L, D, F).workspace_bytes;
}

int mfma_scan(const Operand &a, const Operand &b, const Operand &v, const OperandOut &out,
              int64_t N, int64_t H, int64_t L, bool reverse, void *workspace,
              size_t workspace_bytes, hipStream_t stream) {
    const int D = a.width, F = v.width;
    const MfmaPlan pl = make_plan(N, H, L, D, F);
    if (pl.workspace_bytes > 0 && (!workspace || workspace_bytes < (size_t)pl.workspace_bytes))
        return fail(FTC_ERR_WORKSPACE, "workspace of %lld bytes needed, %zu given",
                    (long long)pl.workspace_bytes, workspace_bytes);
    const int64_t chains = N * H;
    const int64_t wgs = chains * pl.nseg;
    if (wgs > 0x7fffffffLL) return fail(FTC_ERR_UNSUPPORTED, "too many workgroups");

    MfmaArgs args;
    args.a = (const float *)a.ptr;
    args.b = (const float *)b.ptr;
    args.v = (const float *)v.ptr;
    args.out = (float *)out.ptr;
    args.states = pl.nseg > 1 ? (float *)workspace : nullptr;
    args.a_sn = a.stride_n, args.a_sh = a.stride_h, args.a_sl = a.stride_l;
    args.b_sn = b.stride_n, args.b_sh = b.stride_h, args.b_sl = b.stride_l;
    args.v_sn = v.stride_n, args.v_sh = v.stride_h, args.v_sl = v.stride_l;
    args.o_sn = out.stride_n, args.o_sh = out.stride_h, args.o_sl = out.stride_l;
    args.L = L;
    args.H = (int32_t)H;
    args.seg_len = pl.seg_len;
    args.nseg = pl.nseg;

    auto run = [&](const MfmaArgs &x) {
        if (D == 64 && F == 64) launch<64, 64>(x, wgs, reverse, stream);
        else if (D == 32 && F == 128) launch<32, 128>(x, wgs, reverse, stream);
        else launch<128, 32>(x, wgs, reverse, stream);
    };
    if (pl.nseg > 1) {
        args.state_only = 1;
        run(args);
        const int64_t elems = (int64_t)D * F;
        const int64_t scan_wgs = (elems + 255) / 256 * chains;
        hipLaunchKernelGGL(state_scan_kernel, dim3((unsigned)scan_wgs), dim3(256), 0, stream,
                           args.states, pl.nseg, elems, reverse ? 1 : 0);
    }
    args.state_only = 0;
    run(args);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess)
        return fail(FTC_ERR_HIP, "MFMA scan launch failed: %s", hipGetErrorString(err));
    return FTC_OK;
}

}  // namespace ftc
