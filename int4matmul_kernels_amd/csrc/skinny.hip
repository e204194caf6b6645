// Few-row products for gfx950, two kernels.  skinny_kernel (described first): 2 .. 96 rows of states (32 per
// workgroup) against a dense int4 / int3 / int2 or 16:32 sparse int4 weight matrix, HBM-bound like the
// matvec (every packed word is read once and used for all rows).  wide_rows_kernel (further down): 17 .. 256
// rows, whose waves share one staged copy of the states and dequantise each weight.  skinny_rows() at the
// end picks one by shape.  The reference has no such path: it sends M >= 2 to its
// 64-row matmul tiles (int4matmul.cpp:27) and M == 1 with B > 1 to one matvec
// per batch element, re-reading the weights each time (matvec_kernel.cu:346).
//
// The rows are multiplied on the matrix core: v_mfma_f32_16x16x32_f16 takes 16
// rows of states as its 16 x 32 operand (rows >= R are zero; 17 .. 32 rows take
// two such tiles) and, as its 32 x 16 operand, 8 consecutive k of one column per
// lane -- which is exactly one packed int4 word; the four lane groups of a wave
// hold the four packed rows of a 32-row block.  A word becomes that operand
// without converting a single code: mask-and-OR of the word (and of the word
// shifted by 8) gives the half2 pairs {1024 + q0, 1024 + q4}, {64 + q1, 64 + q5},
// {1024 + q2, 1024 + q6}, {64 + q3, 64 + q7}; the states are stored to LDS in the
// same k order 0,4,1,5,2,6,3,7.  (int2 / int3: the chunk's 16 / 24 bits, pairs
// {1024 + q_even, 256 or 128 + q_odd} in natural order.)
// The offsets are removed once per quantisation group in fp32 together with
// scale and zero:
//     y[m, n] += s[n] * (acc[m, n] - sum_k off_k x[m, k] - z[n] * sum_k x[m, k])
// which is the exact value of sum_k x (q - z) s (the per-weight fp16 roundings of
// the reference's decode are not reproduced, as in the matvec).
//
// A workgroup owns a strip of 16 * CW columns (lane j of a wave holds the words
// of CW adjacent columns: CW * 64 contiguous bytes per packed row and wave) and
// its W waves split K; each wave stages the states of its own K range through
// a private LDS buffer, 64 k at a time, and the partial tiles are summed
// through LDS at the end; narrow matrices with a long K are also split along K across workgroups.
//
// 16:32 sparse int4 takes the same kernel.  Every lane group loads the block's
// mask word and both words of kept codes (the four groups of a wave ask for the
// same addresses); group h skips the codes of the rows before its eight with a
// population count of the lower mask bits, and expands its codes to their rows
// with the v_perm selectors of a 256-entry table in LDS (indexed by the mask
// byte), in the int4 k order.  No magic numbers here: the bytes 0x1q (bit 4: "this
// row is kept") become the halves 0x001q, i.e. the fp16 denormals (16 + q) 2^-24,
// which the matrix core multiplies exactly; a second MFMA on the same operand
// masked to 0x0010 gives 16 * 2^-24 * (sum of the kept rows' states), and
//     y[m, n] += s[n] * (2^24 (accA - accM) - z[n] * 2^20 accM).
#include "common.h"

#include <algorithm>
#include <atomic>
#include <type_traits>

namespace i4 {

// magic numbers (div_magic) of the divisors of the balanced launch's range arithmetic: K / 64, the group's units, q, q + 1
struct BalancedMagics { uint32_t units, group_units, share_lo, share_hi; };

struct SkinnyArgs {
    h16* outs;
    const uint32_t* matrix;
    const uint32_t* mask;   // 16:32 sparse only
    const h16* x;
    const h16* scales;
    const h16* zeros;
    int R, K, S;
    int group_units;        // group size / 64
    int units_per_wave;
    int accumulate;         // 1: outs = fp16(fp32(outs) + product) (matvec semantics); 0: overwrite
    // split-K across workgroups (gridDim.z > 1; narrow matrices with a long K): each workgroup takes
    // `units_per_split` units, stores its fp32 partial tile to `part` and counts itself in; the last one
    // to arrive adds the partials up in split order and writes the strip
    int units_per_split;
    float* part;
    int* counters;
    int block_rows;         // wide kernel: rows of states per workgroup (blockIdx.y), a multiple of 16
    // balanced launch of the few-row kernel (more strips than CUs): 256 workgroups share the strips' units
    // evenly, workgroup i takes [i q + i r / 256, (i + 1) q + (i + 1) r / 256) of strips x units, strip-major
    int bal_q, bal_r;
    BalancedMagics bal_magics;
    // launch with a fifth column per lane: the first `wide_wgs` workgroups take 80 columns, the others 64
    int wide_wgs;
};

constexpr int SK_PITCH = 144;                   // bytes between rows of a staged unit (128 + 16: conflict-free)
constexpr int SK_XBUF = 32 * SK_PITCH;          // one staged unit: 32 rows x 64 k
constexpr int SK_WAVE_LDS = 2 * SK_XBUF + 256;  // two unit buffers + the group sums of 32 rows

template <int CW> struct Words;
template <> struct Words<4> { typedef u32x4 type; };
template <> struct Words<2> { typedef u32x2 type; };
template <> struct Words<1> { typedef uint32_t type; };

template <int CW>
__device__ __forceinline__ uint32_t word_of(const typename Words<CW>::type& v, int c) {
    if constexpr (CW == 1) return v;
    else return v[c];
}


// Per format: the k order of the 8 halves of an operand chunk, the offsets the
// magic-number decode leaves on the low / high half of operand register e, and
// the packed rows of a 32-row block.
//   int4: order 0,4,1,5,2,6,3,7; registers 0, 2 carry 1024 + q, registers 1, 3 carry 64 + q
//   int2: natural order, {1024 + q_even, 256 + q_odd};  int3: natural order, {1024 + q_even, 128 + q_odd}
template <int BITS, bool SPARSE = false> struct SkFmt;
template <> struct SkFmt<4, true> {
    static constexpr int ROWS = 2, LOADS = 6;            // per block: two words of codes and the mask word
    __device__ static constexpr int order(int e) { return (e >> 1) + 4 * (e & 1); }
    __device__ static constexpr uint32_t offs(int) { return 0u; }
};
template <> struct SkFmt<4> {
    static constexpr int ROWS = 4, LOADS = 2;            // packed rows per block, loads per lane and unit
    __device__ static constexpr int order(int e) { return (e >> 1) + 4 * (e & 1); }
    __device__ static constexpr uint32_t offs(int e) { return (e & 1) ? 0x54005400u : 0x64006400u; }
};
template <> struct SkFmt<2> {
    static constexpr int ROWS = 2, LOADS = 2;
    __device__ static constexpr int order(int e) { return e; }
    __device__ static constexpr uint32_t offs(int) { return 0x5C006400u; }
};
template <> struct SkFmt<3> {
    static constexpr int ROWS = 3, LOADS = 4;
    __device__ static constexpr int order(int e) { return e; }
    __device__ static constexpr uint32_t offs(int) { return 0x58006400u; }
};

// The 8 codes of one chunk (`f`: BITS bits apart, LSB first, garbage above) -> MFMA
// operand of magic numbers; m0/g0 (and m1/g1 for int4) are the format's mask and
// magic constants held in VGPRs.
template <int BITS>
__device__ __forceinline__ h16x8 magic_operand(uint32_t f, uint32_t m0, uint32_t m1, uint32_t g0, uint32_t g1) {
    u32x4 r;
    if constexpr (BITS == 4) {
        const uint32_t f8 = f >> 8;
        r = u32x4{(f & m0) | g0, (f & m1) | g1, (f8 & m0) | g0, (f8 & m1) | g1};
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t u = f >> (2 * BITS * e);
            r[e] = (__builtin_amdgcn_perm(u, u, 0x01000100u) & m0) | g0;       // low 16 bits in both halves
        }
    }
    return bitcast<h16x8>(r);
}

// 16:32: `v` = the chunk's kept codes as consecutive nibbles, `sel` = the selectors of its mask byte
__device__ __forceinline__ u32x4 sparse_operand(uint32_t v, const u32x4& sel, uint32_t nib, uint32_t flag) {
    const uint32_t even = (v & nib) | flag, odd = ((v >> 4) & nib) | flag;
    return u32x4{__builtin_amdgcn_perm(odd, even, sel.x), __builtin_amdgcn_perm(odd, even, sel.y),
                 __builtin_amdgcn_perm(odd, even, sel.z), __builtin_amdgcn_perm(odd, even, sel.w)};
}

__device__ __forceinline__ h16x8 exact_operand_sparse(uint32_t v, uint32_t m8, h16 sc, h16 ze) {
    h16 row[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const bool kept = (m8 >> r) & 1u;
        row[r] = kept ? dequant_code<4>(v & 15u, sc, ze) : (h16)0.0f;
        v >>= kept ? 4 : 0;
    }
    h16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = row[SkFmt<4, true>::order(e)];
    return o;
}

// The chunk's 8 fp16 weights themselves, in the operand's k order, in either quantisation mode
// (the mode belongs to the lane's column and group), bit-exact with dequant_code and without a
// branch: from the magic-number pairs, P = the codes (offsets removed, exact) or +-2^e,
//     A = P + N (one rounding),  w = fma(A, B, C) (one rounding)
// with (N, B, C) = (-z, s, -0) for a linear group -- fp16(q - z), then fp16(. * s); adding -0
// changes no bit -- and (-0, -s, z) for an exponent group, the reference's single-rounded fma.
template <int BITS>
__device__ __forceinline__ h16x8 exact_operand(uint32_t f, uint32_t m0, uint32_t m1, uint32_t g0, uint32_t g1,
                                               h16 sc, h16 ze) {
    const u32x4 h = bitcast<u32x4>(magic_operand<BITS>(f, m0, m1, g0, g1));
    const bool expo = !(sc >= (h16)0.0f);
    const h16x2 minus0 = as_h2(0x80008000u), s2 = {sc, sc}, z2 = {ze, ze};
    const h16x2 N = expo ? minus0 : -z2, B = expo ? -s2 : s2, C = expo ? z2 : minus0;
    u32x4 r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t offs = SkFmt<BITS>::offs(e);                    // {2^a, 2^b} as halves
        const h16x2 q = as_h2(h[e]) - as_h2(offs);                     // exact
        // the same offsets as integers, for the packed multiply: 2^(exponent field - 15)
        const uint32_t ints = off2(1u << (((offs >> 10) & 31u) - 15u), 1u << (((offs >> 26) & 31u) - 15u));
        const h16x2 P = expo ? as_h2(expo_operand<BITS>(h[e], ints)) : q;
        r[e] = as_u32(__builtin_elementwise_fma(P + N, B, C));
    }
    return bitcast<h16x8>(r);
}

// Balanced launch: workgroup i of 256 takes the range [i q + i r / 256, (i + 1) q + (i + 1) r / 256) of
// strips x units (strip-major; q, r = quotient and remainder of the total by 256).  The range is at least one
// strip and less than two strips long, so it touches at most three strips: three segments, segment k on strip
// strip0 + k.  The workgroup's waves are dealt to the segments in proportion to their units (at least one each).
// For one wave: its segment (`mine`), the segment's units [lo, hi) within its strip, the segment's first wave
// and number of waves; for the workgroup's copy of scales and zeros in LDS: the first group of each segment
// and where each segment's groups start (goff3: all groups).
struct BalancedShare { int strip0, mine, lo, hi, wave0, waves, glo0, glo1, glo2, goff1, goff2, goff3; };
// (A dozen quotients stand between a wave's start and its first loads: they are taken with the divisors' magic
// numbers, which the host passes -- magic_div, csrc/common.h.)
// a / b for 0 <= a < 2^22 through the float reciprocal, for a divisor without a magic number at hand
__device__ __forceinline__ int small_div(int a, int b, float inv_b) {
    int q = (int)((float)a * inv_b);
    int r = a - q * b;
    if (r < 0) { --q; r += b; }
    if (r >= b) ++q;
    return q;
}
__device__ __forceinline__ BalancedShare balanced_share(int q, int r, const BalancedMagics& mg, int i, int units, int group_units,
                                                        int nwaves, int wave) {
    BalancedShare b{};
    const int lo = i * q + ((i * r) >> 8), hi = (i + 1) * q + (((i + 1) * r) >> 8);           // (/ 256 workgroups)
    const int share = hi - lo;
    const uint32_t share_magic = share == q ? mg.share_lo : mg.share_hi;
    b.strip0 = magic_div(lo, units, mg.units);
    int seg_lo[3], seg_n[3], seg_w[3], dealt = 0;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        const int s0 = (b.strip0 + k) * units;
        const int from = max(lo, s0), to = min(hi, s0 + units);
        seg_lo[k] = from - s0;
        seg_n[k] = max(0, to - from);
        seg_w[k] = seg_n[k] > 0 ? max(1, magic_div(seg_n[k] * nwaves + share / 2, share, share_magic)) : 0;
        dealt += seg_w[k];
    }
    // the rounding may deal a wave or two too many or too few: take from the segment with the fewest units per
    // wave, give to the one with the most (the pick's units and waves are kept by value: no indexed registers)
#pragma unroll
    for (int it = 0; it < 3; ++it) {
        if (dealt > nwaves) {
            int k = -1, kn = 0, kw = 1;
#pragma unroll
            for (int c = 0; c < 3; ++c)
                if (seg_w[c] > 1 && (k < 0 || seg_n[c] * kw < kn * seg_w[c])) { k = c; kn = seg_n[c]; kw = seg_w[c]; }
#pragma unroll
            for (int c = 0; c < 3; ++c) if (c == k) --seg_w[c];
            --dealt;
        } else if (dealt < nwaves) {
            int k = -1, kn = 0, kw = 1;
#pragma unroll
            for (int c = 0; c < 3; ++c)
                if (seg_n[c] > 0 && (k < 0 || seg_n[c] * kw > kn * seg_w[c])) { k = c; kn = seg_n[c]; kw = seg_w[c]; }
#pragma unroll
            for (int c = 0; c < 3; ++c) if (c == k) ++seg_w[c];
            ++dealt;
        }
    }
    int w0 = 0;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        if (wave >= w0 && wave < w0 + seg_w[k]) { b.mine = k; b.wave0 = w0; b.waves = seg_w[k]; b.lo = seg_lo[k]; b.hi = seg_lo[k] + seg_n[k]; }
        w0 += seg_w[k];
    }
    const int g0 = magic_div(seg_lo[0], group_units, mg.group_units), g1 = magic_div(seg_lo[1], group_units, mg.group_units),
              g2 = magic_div(seg_lo[2], group_units, mg.group_units);
    b.glo0 = g0; b.glo1 = g1; b.glo2 = g2;
    b.goff1 = seg_n[0] > 0 ? magic_div(seg_lo[0] + seg_n[0] - 1, group_units, mg.group_units) + 1 - g0 : 0;
    b.goff2 = b.goff1 + (seg_n[1] > 0 ? magic_div(seg_lo[1] + seg_n[1] - 1, group_units, mg.group_units) + 1 - g1 : 0);
    b.goff3 = b.goff2 + (seg_n[2] > 0 ? magic_div(seg_lo[2] + seg_n[2] - 1, group_units, mg.group_units) + 1 - g2 : 0);
    return b;
}

// CW: columns per lane; RT: row groups of 8 that can hold real rows (R <= 8 RT);
// MT: 16-row MFMA tiles; PF: units of packed weights in flight per wave
// BAL: the workgroups share the work evenly instead of taking a strip each (more strips than CUs): a workgroup's
// range of (strip, unit) touches two or three strips, its waves are dealt to them in proportion, every wave works
// on one strip, and a strip that two workgroups share is summed through the hand-over below.
// XC = 1: a fifth column per lane (CW = 4 only, dense formats): the workgroup's columns are four or five slivers of
// 16, the lane's four adjacent columns in the first four and column j of the fifth (a.wide_wgs workgroups have one)
template <int BITS, int CW, int RT, bool SPARSE, bool BAL = false, int XC = 0>
__global__ __launch_bounds__(512) void skinny_kernel(const uint32_t* pre_matrix, const h16* pre_x, const h16* pre_scales, const h16* pre_zeros,
                                                   int pre_S, int pre_K, int pre_group_units, int pre_units, SkinnyArgs a) {
    // (what the first loads depend on, once more in front of the record: the first dwords of a kernel's arguments
    // reach a wave in registers at its start, a record's fields are fetched by the wave itself)
    a.matrix = pre_matrix; a.x = pre_x; a.scales = pre_scales; a.zeros = pre_zeros; a.S = pre_S; a.K = pre_K;
    a.group_units = pre_group_units; a.units_per_wave = pre_units;
    using F = SkFmt<BITS, SPARSE>;
    constexpr int NL = F::LOADS;
    constexpr int PF = (BITS == 3 && CW == 4) || (SPARSE && CW == 4) ? 2 : 4, MT = RT == 4 ? 2 : 1;
    constexpr int PFX = RT == 4 ? 2 : 4;            // units of states in flight per wave
    constexpr int CT = CW + XC;                     // columns per lane in all
    constexpr int STRIP = 16 * CT;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    typedef typename Words<CW>::type words_t;
    const int t = threadIdx.x, lane = t & 63, nwaves = blockDim.x >> 6;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);   // scalar: the unit loop runs on SGPRs
    const int j = lane & 15, h = lane >> 4;
    const int units = a.K / 64;
    // the wave's strip, the part of the strip's units that its workgroup (BAL: its segment of the workgroup's
    // range) covers, and the wave's own units in it
    int strip = blockIdx.x, split_lo, split_hi, u0, u1;
    int seg_wave0 = 0, seg_waves = nwaves;                      // the waves that work on the same strip
    BalancedShare bs{};
    if constexpr (BAL) {
        bs = balanced_share(a.bal_q, a.bal_r, a.bal_magics, blockIdx.x, units, a.group_units, nwaves, wave);
        strip = bs.strip0 + bs.mine;
        split_lo = bs.lo;
        split_hi = bs.hi;
        seg_wave0 = bs.wave0;
        seg_waves = bs.waves;
        const int upw = small_div(split_hi - split_lo + seg_waves - 1, seg_waves, 1.f / (float)seg_waves);
        u0 = min(split_hi, split_lo + (wave - seg_wave0) * upw);
        u1 = min(split_hi, u0 + upw);
    } else {
        split_lo = blockIdx.z * a.units_per_split;
        split_hi = min(units, split_lo + a.units_per_split);
        u0 = min(split_hi, split_lo + wave * a.units_per_wave);
        u1 = min(split_hi, u0 + a.units_per_wave);
    }
    // first column of the workgroup, of the lane's CW adjacent columns, and the lane's column in the fifth sliver
    // (a workgroup without one re-reads its first sliver there and does not write the result)
    const bool has_extra = XC != 0 && (int)blockIdx.x < a.wide_wgs;
    const int colbase = XC != 0 ? (has_extra ? 80 * (int)blockIdx.x : 80 * a.wide_wgs + 64 * ((int)blockIdx.x - a.wide_wgs))
                                : strip * STRIP;
    const int col0 = colbase + CW * j;
    const int colx = has_extra ? colbase + 16 * CW + j : colbase + j;
    // more than 32 rows: blockIdx.y takes rows 32 y .. 32 y + 31 (each block reads the strip's weights again)
    const int row0 = blockIdx.y * 32;
    const int R = min(32, a.R - row0);

    // The strip's scales and zeros ([groups][STRIP] halves each) are copied to LDS
    // once: the loop then never waits on a global load other than its prefetched
    // weights and states.  Exponent-mode scales (negative or NaN) anywhere in the
    // strip switch the whole workgroup to the exact per-weight decode.  (The copy
    // runs after the first loads have been issued, under their latency.)
    // (of the groups that the workgroup's share of K touches: group_lo onwards)
    const int group_lo = split_lo / a.group_units;
    const int groups = (split_hi + a.group_units - 1) / a.group_units - group_lo;
    // (BAL: the copies of the workgroup's segments one after the other; this wave's starts at group sz_goff)
    const int sz_groups = BAL ? bs.goff3 : groups, sz_goff = BAL ? (bs.mine == 0 ? 0 : bs.mine == 1 ? bs.goff1 : bs.goff2) : 0;
    // (16:32: the selector table is allocated statically: its LDS address is a compile-time constant)
    __shared__ __attribute__((aligned(16))) u32x4 lut_table[SPARSE ? 256 : 1];
    const char* lut = reinterpret_cast<const char*>(lut_table);
    if constexpr (SPARSE) {
        // for mask byte b, pair e = (row e, row e + 4): byte 0 picks the code byte of row e out of
        // {even nibbles, odd nibbles} by its rank among the kept rows, byte 2 that of row e + 4;
        // 0x0C yields 0.  Stored under the nibble-swapped byte (see the lookup).
        for (int b = t; b < 256; b += blockDim.x) {
            uint32_t selb[8];
            int rank = 0;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const bool k = (b >> r) & 1;
                selb[r] = k ? (uint32_t)((rank & 1) * 4 + (rank >> 1)) : 0x0Cu;
                rank += k;
            }
            u32x4 e;
#pragma unroll
            for (int q = 0; q < 4; ++q) e[q] = selb[q] | (0x0Cu << 8) | (selb[q + 4] << 16) | (0x0Cu << 24);
            lut_table[((b & 15) << 4) | (b >> 4)] = e;
        }
    }
    uint32_t* sz = reinterpret_cast<uint32_t*>(lds + nwaves * SK_WAVE_LDS + 16);      // scales, then zeros
    auto scan_scales = [&]() __attribute__((always_inline)) -> bool {
        int* flag = reinterpret_cast<int*>(lds + nwaves * SK_WAVE_LDS);
        if (t == 0) *flag = 0;
        __syncthreads();
        bool bad = false;
        const int n = sz_groups * (STRIP / 2);
        for (int i = t; i < n; i += blockDim.x) {
            const int g = i / (STRIP / 2), c = i % (STRIP / 2);
            int64_t at;
            if constexpr (BAL) {
                // (sums rather than selections among the three segments' values: the compiler turns a selection
                // among fields into an indexed load, which puts the whole record into scratch memory)
                const int k1 = g >= bs.goff1 ? 1 : 0, k2 = g >= bs.goff2 ? 1 : 0;
                const int first = bs.glo0 + k1 * (bs.glo1 - bs.glo0) + k2 * (bs.glo2 - bs.glo1);
                const int off = k1 * bs.goff1 + k2 * (bs.goff2 - bs.goff1);
                at = (int64_t)(first + g - off) * a.S + (bs.strip0 + k1 + k2) * STRIP + 2 * c;
            } else {
                at = (int64_t)(group_lo + g) * a.S + colbase + ((XC != 0 && !has_extra && c >= 8 * CW) ? 2 * c - 16 * CW : 2 * c);
            }
            const uint32_t two = *reinterpret_cast<const uint32_t*>(a.scales + at);
            bad |= !(as_h2(two).x >= (h16)0.0f) || !(as_h2(two).y >= (h16)0.0f);
            sz[i] = two;
            sz[n + i] = *reinterpret_cast<const uint32_t*>(a.zeros + at);
        }
        if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0) *flag = 1;
        __syncthreads();
        return *flag != 0;
    };
    bool general = false;

    char* my = lds + wave * SK_WAVE_LDS;
    float* sums = reinterpret_cast<float*>(my + 2 * SK_XBUF);   // [0..31] sum x, [32..63] sum off x

    // accumulators: acc = raw products of the current group, y = finished groups
    // (register e of tile mt is row 16 mt + 4 h + e, column j)
    // (16:32: accm = the same for the "kept" flags)
    f32x4 acc[CT][MT], accm[SPARSE ? CW : 1][MT], y[CT][MT];
#pragma unroll
    for (int c = 0; c < CT; ++c)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            acc[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            y[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (SPARSE || c == 0) accm[SPARSE ? c : 0][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }

    if (u0 >= u1) general = scan_scales();          // idle waves still take part in its barriers
    if (u0 < u1) {
        // ---- loaders
        // weights of unit u, CW words per load.  Lane group h needs chunk h (8 codes) of
        // each of the unit's two 32-row blocks:
        //   int4: packed row 4 blk + h;  int2: row 2 blk + h / 2, its low or high half;
        //   int3: bits 24 h .. 24 h + 23 of the block's 96-bit stream = rows {0,0,1,1}[h] and the
        //         next one, shifted right by {0, 24, 16, 40}[h]
        const int wrow = BITS == 4 ? h : (BITS == 2 ? (h >> 1) : (h >> 1));
        const int wshift = BITS == 4 ? 0 : (BITS == 2 ? 16 * (h & 1) : (h == 0 ? 0 : h == 1 ? 24 : h == 2 ? 16 : 40));
        //   16:32: every lane group loads both words of kept codes and the mask word of the block
        //          (w[3 blk], w[3 blk + 1], w[3 blk + 2])
        const uint32_t* wbase = a.matrix + (int64_t)(SPARSE ? 0 : wrow) * a.S + col0;
        const uint32_t* mbase = SPARSE ? a.mask + col0 : nullptr;
        const uint32_t* xbase = a.matrix + (int64_t)wrow * a.S + colx;
        auto load_w = [&](words_t w[NL], uint32_t wx[NL], int u) {
            const uint32_t* p = wbase + (int64_t)u * (2 * F::ROWS) * a.S;
            if constexpr (SPARSE) {
                const uint32_t* pm = mbase + (int64_t)u * 2 * a.S;
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    w[3 * blk] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p + (int64_t)(2 * blk) * a.S));
                    w[3 * blk + 1] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p + (int64_t)(2 * blk + 1) * a.S));
                    w[3 * blk + 2] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(pm + (int64_t)blk * a.S));
                }
            } else {
#pragma unroll
                for (int i = 0; i < NL; ++i) {
                    const int row = BITS == 3 ? 3 * (i >> 1) + (i & 1) : F::ROWS * i;       // relative to the lane's first row
                    w[i] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p + (int64_t)row * a.S));
                    if constexpr (XC != 0)
                        wx[i] = __builtin_nontemporal_load(xbase + ((int64_t)u * (2 * F::ROWS) + row) * a.S);
                }
            }
        };
        // 16:32: mask bits of the rows before the lane group's eight; selector that replicates mask byte h
        const uint32_t below = SPARSE ? (1u << (8 * h)) - 1u : 0u, rep_h = 0x01010101u * h;
        // the 8 codes of chunk h of block blk, column c
        auto chunk_bits = [&](const words_t w[NL], const uint32_t wx[NL], int blk, int c) -> uint32_t {
            auto word = [&](int idx) -> uint32_t { return c < CW ? word_of<CW>(w[idx], c < CW ? c : 0) : wx[idx]; };
            if constexpr (BITS == 3)
                return (uint32_t)((((uint64_t)word(2 * blk + 1) << 32) | word(2 * blk)) >> wshift);
            else
                return word(blk) >> wshift;
        };
        // states of unit u (8 RT rows x 128 bytes): 8 / RT lanes per row, RT 16-byte chunks
        // each; the rows of the LDS buffers beyond 8 RT stay zero
        constexpr int LPR = 8 / RT;                                   // lanes per row
        const int xm = lane / LPR, xpart = lane % LPR;
        const bool xreal = xm < R;
        const h16* xsrc = a.x + (int64_t)(row0 + min(xm, R - 1)) * a.K + xpart * (8 * RT);
        auto load_x = [&](u32x4 xr[RT], int u) {
#pragma unroll
            for (int i = 0; i < RT; ++i)
                xr[i] = xreal ? *reinterpret_cast<const u32x4*>(xsrc + u * 64 + i * 8) : u32x4{0, 0, 0, 0};
        };
        // store a loaded unit to LDS buffer p and return its per-row sums (all lanes of a row get them)
        auto stage_x = [&](const u32x4 xr[RT], int p, float& sx, float& so) {
            const uint32_t ONES = 0x3C003C00u;
            sx = 0.f; so = 0.f;
#pragma unroll
            for (int i = 0; i < RT; ++i) {
                const u32x4 v = xr[i];
                // the k order inside the chunk that the operand decode produces (int4: 0,4,1,5,2,6,3,7)
                u32x4 q = v;
                if constexpr (BITS == 4)
                    q = u32x4{__builtin_amdgcn_perm(v[2], v[0], 0x05040100u), __builtin_amdgcn_perm(v[2], v[0], 0x07060302u),
                              __builtin_amdgcn_perm(v[3], v[1], 0x05040100u), __builtin_amdgcn_perm(v[3], v[1], 0x07060302u)};
                if constexpr (!SPARSE) {                 // (16:32 has no offsets to remove)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        sx = dot2(q[e], ONES, sx);
                        so = dot2(q[e], F::offs(e), so);
                    }
                }
                *reinterpret_cast<u32x4*>(my + p * SK_XBUF + xm * SK_PITCH + (xpart * RT + i) * 16) = q;
            }
            if constexpr (!SPARSE) {
                // the other lanes of the row: lane ^ 1, lane ^ 2, lane ^ 4 as far as the row extends
                sx += dpp_f32<0xB1>(sx);
                so += dpp_f32<0xB1>(so);
                if constexpr (LPR >= 4) { sx += dpp_f32<0x4E>(sx); so += dpp_f32<0x4E>(so); }
                if constexpr (LPR >= 8) { sx += dpp_f32<0x141>(sx); so += dpp_f32<0x141>(so); }
            }
        };
        // rows that never receive states must read as zero
        for (int i = lane; i < 2 * SK_XBUF / 16; i += 64) *reinterpret_cast<u32x4*>(my + i * 16) = u32x4{0, 0, 0, 0};

        words_t w[PF][NL];
        uint32_t wx[PF][NL];                // (XC: the fifth column's words)
        u32x4 xr[PFX][RT];
        const uint32_t m0 = in_vgpr(BITS == 4 ? 0x000F000Fu : BITS == 2 ? 0x000C0003u : 0x00380007u);
        const uint32_t g0 = in_vgpr(BITS == 4 ? 0x64006400u : BITS == 2 ? 0x5C006400u : 0x58006400u);
        const uint32_t m1 = BITS == 4 ? in_vgpr(0x00F000F0u) : 0u, g1 = BITS == 4 ? in_vgpr(0x54005400u) : 0u;
        const uint32_t sp_nib = SPARSE ? in_vgpr(0x0F0F0F0Fu) : 0u, sp_flag = SPARSE ? in_vgpr(0x10101010u) : 0u;
        const uint32_t sp_kept = SPARSE ? in_vgpr(0x00100010u) : 0u, sp_idx = SPARSE ? in_vgpr(0x00000FF0u) : 0u;
        float gS = 0.f, gO = 0.f;           // sums of the current group so far (row lane / 2)
        float nS, nO;                       // sums of the unit staged last (the next to be multiplied)
        // scale / zero of the lane's CW columns for group gi, from the LDS copy
        h16 sc[CT], ze[CT];
#pragma unroll
        for (int c = 0; c < CT; ++c) { sc[c] = (h16)0.f; ze[c] = (h16)0.f; }
        auto load_sz = [&](int gi) {
            const h16* ps = reinterpret_cast<const h16*>(sz) + (sz_goff + gi - group_lo) * STRIP + CW * j;
            const h16* pz = ps + sz_groups * STRIP;
            if constexpr (CW == 4) {
                const u32x2 s2 = *reinterpret_cast<const u32x2*>(ps), z2 = *reinterpret_cast<const u32x2*>(pz);
                sc[0] = as_h2(s2.x).x; sc[1] = as_h2(s2.x).y; sc[2] = as_h2(s2.y).x; sc[3] = as_h2(s2.y).y;
                ze[0] = as_h2(z2.x).x; ze[1] = as_h2(z2.x).y; ze[2] = as_h2(z2.y).x; ze[3] = as_h2(z2.y).y;
            } else if constexpr (CW == 2) {
                const uint32_t s1 = *reinterpret_cast<const uint32_t*>(ps), z1 = *reinterpret_cast<const uint32_t*>(pz);
                sc[0] = as_h2(s1).x; sc[1] = as_h2(s1).y; ze[0] = as_h2(z1).x; ze[1] = as_h2(z1).y;
            } else {
                sc[0] = ps[0]; ze[0] = pz[0];
            }
            if constexpr (XC != 0) { sc[CW] = ps[16 * CW + j - CW * j]; ze[CW] = pz[16 * CW + j - CW * j]; }
        };

#pragma unroll
        for (int f = 0; f < PF; ++f) load_w(w[f], wx[f], min(u0 + f, u1 - 1));
        load_x(xr[0], u0);
        general = scan_scales();
        stage_x(xr[0], 0, nS, nO);
        // set f holds unit u0 + f (f >= 1) and, for f = 0, unit u0 + PFX
#pragma unroll
        for (int f = 1; f <= PFX; ++f) load_x(xr[f % PFX], min(u0 + f, u1 - 1));

        // p: parity of the LDS buffer that holds unit u; xn: the register set with the states of unit u + 1.
        // The decode mode is a compile-time tag: one loop body per mode, no branches inside.
        auto step = [&](auto mode, int u, int p, words_t w[NL], uint32_t wx[NL], u32x4 xn[RT]) {
            constexpr bool general = decltype(mode)::value;
            if constexpr (general) {
                if (u == u0 || u % a.group_units == 0) load_sz(u / a.group_units);
            }
            gS += nS; gO += nO;
            // 2 blocks of 32 k: lane group h multiplies chunk h (8 k) of the block
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                h16x8 xa[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    xa[mt] = *reinterpret_cast<const h16x8*>(my + p * SK_XBUF + (j + 16 * mt) * SK_PITCH + (i * 4 + h) * 16);
#pragma unroll
                for (int c = 0; c < CT; ++c) {
                    if constexpr (SPARSE) {
                        const uint32_t m = word_of<CW>(w[3 * i + 2], c);
                        const uint64_t st = ((uint64_t)word_of<CW>(w[3 * i + 1], c) << 32) | word_of<CW>(w[3 * i], c);
                        // the codes of the rows before this chunk are skipped, 4 bits each (a full
                        // skip of 64 bits only happens when no row of the chunk is kept)
                        const uint32_t v = (uint32_t)(st >> ((uint32_t)__builtin_popcount(m & below) << 2));
                        const uint32_t mb4 = __builtin_amdgcn_perm(m, m, rep_h);           // mask byte h, four times
                        if constexpr (general) {
                            const h16x8 wb = exact_operand_sparse(v, mb4 & 0xFFu, sc[c], ze[c]);
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt)
                                acc[c][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], wb, acc[c][mt], 0, 0, 0);
                        } else {
                            // (table entries sit under the nibble-swapped byte = bits 4 .. 11 of mb4)
                            const u32x4 sel = *reinterpret_cast<const u32x4*>(lut + (mb4 & sp_idx));
                            const u32x4 b = sparse_operand(v, sel, sp_nib, sp_flag);
                            const u32x4 bm = u32x4{b.x & sp_kept, b.y & sp_kept, b.z & sp_kept, b.w & sp_kept};
#pragma unroll
                            for (int mt = 0; mt < MT; ++mt) {
                                acc[c][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], bitcast<h16x8>(b), acc[c][mt], 0, 0, 0);
                                accm[c][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], bitcast<h16x8>(bm), accm[c][mt], 0, 0, 0);
                            }
                        }
                    } else {
                        const uint32_t f = chunk_bits(w, wx, i, c);
                        const h16x8 wb = general ? exact_operand<BITS>(f, m0, m1, g0, g1, sc[c], ze[c])
                                                 : magic_operand<BITS>(f, m0, m1, g0, g1);
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            acc[c][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], wb, acc[c][mt], 0, 0, 0);
                    }
                }
            }
            // refill this register set PF units ahead; move the next unit's states to LDS
            load_w(w, wx, min(u + PF, u1 - 1));
            stage_x(xn, p ^ 1, nS, nO);
            load_x(xn, min(u + 1 + PFX, u1 - 1));
            // group complete (or this wave's range ends): fold it into y
            if ((u + 1) % a.group_units == 0 || u + 1 == u1) {
                if constexpr (SPARSE && !general) {
                    load_sz(u / a.group_units);
#pragma unroll
                    for (int c = 0; c < CW; ++c) {
                        // y += s (A - z M) with A = 2^24 (acc - accm), M = 2^20 accm
                        const float ka = (float)sc[c] * 16777216.f;
                        const float km = -(ka + (float)sc[c] * (float)ze[c] * 1048576.f);
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                y[c][mt][e] = __builtin_fmaf(ka, acc[c][mt][e], __builtin_fmaf(km, accm[c][mt][e], y[c][mt][e]));
                            acc[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                            accm[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                        }
                    }
                } else {
                if (xpart == 0) { sums[xm] = gS; sums[32 + xm] = gO; }
                if constexpr (!general) load_sz(u / a.group_units);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    const f32x4 s4 = *reinterpret_cast<const f32x4*>(&sums[16 * mt + 4 * h]);
                    const f32x4 o4 = *reinterpret_cast<const f32x4*>(&sums[32 + 16 * mt + 4 * h]);
#pragma unroll
                    for (int c = 0; c < CT; ++c) {
                        const float sf = general ? 1.f : (float)sc[c];
                        const float z = general ? 0.f : (float)ze[c];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float off = general ? 0.f : o4[e] + z * s4[e];
                            y[c][mt][e] += sf * (acc[c][mt][e] - off);
                        }
                        acc[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                    }
                }
                }
                gS = 0.f; gO = 0.f;
            }
        };
        auto run = [&](auto mode) {
            constexpr int UN = PF > PFX ? PF : PFX;      // register sets rotate with periods PF and PFX
            for (int u = u0; u < u1; u += UN) {
#pragma unroll
                for (int f = 0; f < UN; ++f) {
                    if (f > 0 && u + f >= u1) break;
                    step(mode, u + f, f & 1, w[f % PF], wx[f % PF], xr[(f + 1) % PFX]);
                }
            }
        };
        if (general) run(std::integral_constant<bool, true>{});
        else run(std::integral_constant<bool, false>{});
    }

    // ---- sum the waves' partial tiles through LDS (tile: [16 MT rows][16 CW columns] fp32)
    __syncthreads();
    constexpr int TILE = MT * 16 * STRIP;
    float* red = reinterpret_cast<float*>(lds);
    auto tile_at = [&](float* base, int mt, int e) { return base + ((mt * 16 + 4 * h + e) * 16 + j) * CT; };
    if constexpr (BAL) {
        // every wave leaves its tile; the first wave of each segment adds up its segment's, in wave order
        float* dst = red + wave * TILE;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int c = 0; c < CT; ++c) tile_at(dst, mt, e)[c] = y[c][mt][e];
        __syncthreads();
        if (wave != seg_wave0) return;
        for (int w = seg_wave0 + 1; w < seg_wave0 + seg_waves; ++w) {
            float* src = red + w * TILE;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int c = 0; c < CT; ++c) y[c][mt][e] += tile_at(src, mt, e)[c];
        }
    }
    for (int s = BAL ? 0 : (nwaves >> 1); s >= 1; s >>= 1) {
        if (wave >= s && wave < 2 * s) {
            float* dst = red + (wave - s) * TILE;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int c = 0; c < CT; ++c) tile_at(dst, mt, e)[c] = y[c][mt][e];
        }
        __syncthreads();
        if (wave < s) {
            float* src = red + wave * TILE;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int c = 0; c < CT; ++c) y[c][mt][e] += tile_at(src, mt, e)[c];
        }
        __syncthreads();
    }
    if (BAL || wave == 0) {
        // (BAL: a strip shared by two workgroups -- never more: a workgroup's range is at least a strip long)
        const bool shared = BAL ? (split_lo > 0 || split_hi < units) : gridDim.z > 1;
        if (shared) {
            // hand-over between the workgroups of a strip: write-through stores of the partial tile
            // (value v of lane l at (v * 64 + l) * 4), a device-scope counter, and whoever finds all
            // the others counted reads every partial back in split order -- one summation order
            // whoever is last -- and goes on to write the strip.  One wave: no barrier involved.
            constexpr int NV = CW * MT * 4, THROUGH = 17;                 // sc0 | sc1: straight to memory
            const int tile = BAL ? strip : blockIdx.y * gridDim.x + blockIdx.x, ks = BAL ? 2 : gridDim.z;
            const int my_split = BAL ? (split_lo > 0 ? 1 : 0) : blockIdx.z;
            char* const slots = reinterpret_cast<char*>(a.part) + (int64_t)tile * ks * (NV * 256);
            const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
                slots + (int64_t)my_split * (NV * 256), 0, NV * 256, 0x00020000);
#pragma unroll
            for (int c = 0; c < CW; ++c)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float v = y[c][mt][e];       // (a bit_cast straight from the vector element reads element 0)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), mine,
                                                              (((c * MT + mt) * 4 + e) * 64 + lane) * 4, 0, THROUGH);
                    }
            // (the fences keep the compiler from moving the counter update ahead of the stores, or the
            // loads below ahead of it; the hardware side is the wait for the stores' acknowledgement)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_s_waitcnt(0);
            int arrived = 0;
            if (lane == 0) arrived = __hip_atomic_fetch_add(a.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            arrived = __builtin_amdgcn_readfirstlane(arrived);
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (arrived != ks - 1) return;
            if (lane == 0) __hip_atomic_store(a.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int c = 0; c < CW; ++c)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) y[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int sp = 0; sp < ks; ++sp) {
                const __amdgpu_buffer_rsrc_t theirs = __builtin_amdgcn_make_buffer_rsrc(
                    slots + (int64_t)sp * (NV * 256), 0, NV * 256, 0x00020000);
#pragma unroll
                for (int c = 0; c < CW; ++c)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            y[c][mt][e] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                theirs, (((c * MT + mt) * 4 + e) * 64 + lane) * 4, 0, THROUGH));
            }
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = mt * 16 + 4 * h + e;
                if (m < R) {
                    h16* o = a.outs + (int64_t)(row0 + m) * a.S + col0;
#pragma unroll
                    for (int c = 0; c < CW; ++c) {
                        float v = y[c][mt][e];
                        if (a.accumulate) v += (float)o[c];
                        o[c] = (h16)v;
                    }
                    if (XC != 0 && has_extra) {
                        h16* ox = a.outs + (int64_t)(row0 + m) * a.S + colx;
                        float v = y[CT - 1][mt][e];
                        if (a.accumulate) v += (float)ox[0];
                        ox[0] = (h16)v;
                    }
                }
            }
    }
}

// ---- 17 ... 512 rows, every format: the eight waves of a workgroup share one staged copy of the states.
// In the kernel above every wave stages the states of its own units, so a workgroup of 64 columns reads
// all R x K states: with R = 64 that is four times the packed weights it reads.  Here the waves stand side
// by side along the columns (32 each, 256 per workgroup), all walk the same units, and each unit's states
// (16 MT rows x 128 bytes) are moved to LDS once per workgroup, by all 512 threads, a unit ahead of the
// MFMAs: one barrier per unit.  Thread t stages chunk t % 8 (8 k) of row t / 8.  With this many rows the
// kernel is bound by its vector instructions, and folding scale and zero into the accumulators once per
// group (3 operations per accumulator element, plus the row sums at the staging) costs more of them than
// dequantising each weight: the operand is the reference's fp16(fp16(q - z) s), three packed operations
// per pair of weights on top of the magic-number decode, and the accumulators hold the product itself.
// K is split across workgroups (blockIdx.z) with the hand-over above, one counter per wave.
template <int BITS, int MT, bool SPARSE = false>
__global__ __launch_bounds__(512) void wide_rows_kernel(const uint32_t* pre_matrix, const h16* pre_x, const h16* pre_scales, const h16* pre_zeros,
                                                   int pre_S, int pre_K, int pre_group_units, int pre_units, SkinnyArgs a) {
    // (what the first loads depend on, once more in front of the record: the first dwords of a kernel's arguments
    // reach a wave in registers at its start, a record's fields are fetched by the wave itself)
    a.matrix = pre_matrix; a.x = pre_x; a.scales = pre_scales; a.zeros = pre_zeros; a.S = pre_S; a.K = pre_K;
    a.group_units = pre_group_units; a.units_per_split = pre_units;
    using F = SkFmt<BITS, SPARSE>;
    // (units of weights in flight per wave: four; two in the tall 16:32 blocks, whose registers are short)
    constexpr int CW = 2, NL = F::LOADS, PF = (SPARSE && MT > 4) ? 2 : 4, ROWS = 16 * MT, STRIP = 16 * CW, WSTRIP = 8 * STRIP;
    constexpr int XBUF = ROWS * SK_PITCH;
    extern __shared__ __attribute__((aligned(16))) char lds[];
    typedef typename Words<CW>::type words_t;
    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int j = lane & 15, h = lane >> 4;
    const int col0 = blockIdx.x * WSTRIP + wave * STRIP + CW * j;
    const int units = a.K / 64;
    const int u0 = blockIdx.z * a.units_per_split, u1 = min(units, u0 + a.units_per_split);
    const int row0 = blockIdx.y * a.block_rows;
    const int R = min(a.block_rows, a.R - row0);
    const int group_lo = u0 / a.group_units;
    const int groups = (u1 + a.group_units - 1) / a.group_units - group_lo;

    // (16:32: the selector table of the kernel above, same layout)
    __shared__ __attribute__((aligned(16))) u32x4 lut_table[SPARSE ? 256 : 1];
    const char* lut = reinterpret_cast<const char*>(lut_table);
    if constexpr (SPARSE) {
        for (int b = t; b < 256; b += 512) {
            uint32_t selb[8];
            int rank = 0;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const bool k = (b >> r) & 1;
                selb[r] = k ? (uint32_t)((rank & 1) * 4 + (rank >> 1)) : 0x0Cu;
                rank += k;
            }
            u32x4 e;
#pragma unroll
            for (int q = 0; q < 4; ++q) e[q] = selb[q] | (0x0Cu << 8) | (selb[q + 4] << 16) | (0x0Cu << 24);
            lut_table[((b & 15) << 4) | (b >> 4)] = e;
        }
    }
    // LDS: two unit buffers, a flag, the strip's scales and zeros
    char* const xb = lds;
    int* const flag = reinterpret_cast<int*>(lds + 2 * XBUF);
    uint32_t* const sz = reinterpret_cast<uint32_t*>(lds + 2 * XBUF + 16);
    auto scan_scales = [&]() -> bool {
        if (t == 0) *flag = 0;
        __syncthreads();
        bool bad = false;
        const int n = groups * (WSTRIP / 2);
        for (int i = t; i < n; i += 512) {
            const int g = i / (WSTRIP / 2), c = i % (WSTRIP / 2);
            const int64_t at = (int64_t)(group_lo + g) * a.S + blockIdx.x * WSTRIP + 2 * c;
            const uint32_t two = *reinterpret_cast<const uint32_t*>(a.scales + at);
            bad |= !(as_h2(two).x >= (h16)0.0f) || !(as_h2(two).y >= (h16)0.0f);
            sz[i] = two;
            sz[n + i] = *reinterpret_cast<const uint32_t*>(a.zeros + at);
        }
        if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0) *flag = 1;
        __syncthreads();
        return *flag != 0;
    };

    f32x4 acc[CW][MT];
#pragma unroll
    for (int c = 0; c < CW; ++c)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // weights of unit u: as in the kernel above (lane group h: chunk h of each of the unit's two blocks)
    const int wrow = BITS == 4 ? h : (h >> 1);
    const int wshift = BITS == 4 ? 0 : (BITS == 2 ? 16 * (h & 1) : (h == 0 ? 0 : h == 1 ? 24 : h == 2 ? 16 : 40));
    const uint32_t* wbase = a.matrix + (int64_t)(SPARSE ? 0 : wrow) * a.S + col0;
    const uint32_t* mbase = SPARSE ? a.mask + col0 : nullptr;
    auto load_w = [&](words_t w[NL], int u) {
        const uint32_t* p = wbase + (int64_t)u * (2 * F::ROWS) * a.S;
        if constexpr (SPARSE) {          // every lane group: both words of kept codes and the mask word of each block
            const uint32_t* pm = mbase + (int64_t)u * 2 * a.S;
#pragma unroll
            for (int blk = 0; blk < 2; ++blk) {
                w[3 * blk] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p + (int64_t)(2 * blk) * a.S));
                w[3 * blk + 1] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p + (int64_t)(2 * blk + 1) * a.S));
                w[3 * blk + 2] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(pm + (int64_t)blk * a.S));
            }
        } else {
#pragma unroll
            for (int i = 0; i < NL; ++i) {
                const int row = BITS == 3 ? 3 * (i >> 1) + (i & 1) : F::ROWS * i;
                w[i] = __builtin_nontemporal_load(reinterpret_cast<const words_t*>(p + (int64_t)row * a.S));
            }
        }
    };
    auto chunk_bits = [&](const words_t w[NL], int blk, int c) -> uint32_t {
        if constexpr (BITS == 3)
            return (uint32_t)((((uint64_t)word_of<CW>(w[2 * blk + 1], c) << 32) | word_of<CW>(w[2 * blk], c)) >> wshift);
        else
            return word_of<CW>(w[blk], c) >> wshift;
    };
    // states: thread t moves chunk t % 8 of row t / 8 (and of row t / 8 + 64 in blocks of more than 64 rows)
    constexpr int XP = (ROWS + 63) / 64;
    struct XRegs { u32x4 v[XP]; };
    const int xrow = t >> 3, xchunk = t & 7;
    const h16* xsrc[XP];
#pragma unroll
    for (int q = 0; q < XP; ++q) xsrc[q] = a.x + (int64_t)(row0 + min(xrow + 64 * q, R - 1)) * a.K + xchunk * 8;
    // (every thread loads -- rows beyond R re-read row R - 1, their products are never written: a load
    // under a branch would make the compiler wait for all loads in flight at every use of one)
    auto load_x = [&](int u) -> XRegs {
        XRegs r;
#pragma unroll
        for (int q = 0; q < XP; ++q) r.v[q] = *reinterpret_cast<const u32x4*>(xsrc[q] + u * 64);
        return r;
    };
    auto stage_x = [&](const XRegs& x, int p) {
#pragma unroll
        for (int k = 0; k < XP; ++k) {
            const u32x4 v = x.v[k];
            u32x4 q = v;
            if constexpr (BITS == 4)         // the k order inside the chunk that the operand decode produces
                q = u32x4{__builtin_amdgcn_perm(v[2], v[0], 0x05040100u), __builtin_amdgcn_perm(v[2], v[0], 0x07060302u),
                          __builtin_amdgcn_perm(v[3], v[1], 0x05040100u), __builtin_amdgcn_perm(v[3], v[1], 0x07060302u)};
            if (xrow + 64 * k < ROWS) *reinterpret_cast<u32x4*>(xb + p * XBUF + (xrow + 64 * k) * SK_PITCH + xchunk * 16) = q;
        }
    };

    words_t w[PF][NL];
    XRegs xr[PF];
    const uint32_t m0 = in_vgpr(BITS == 4 ? 0x000F000Fu : BITS == 2 ? 0x000C0003u : 0x00380007u);
    const uint32_t g0 = in_vgpr(BITS == 4 ? 0x64006400u : BITS == 2 ? 0x5C006400u : 0x58006400u);
    const uint32_t m1 = BITS == 4 ? in_vgpr(0x00F000F0u) : 0u, g1 = BITS == 4 ? in_vgpr(0x54005400u) : 0u;
    h16 sc[CW], ze[CW];
    h16x2 s2[CW], c2[CW];               // {s, s} and {z, z} of the lane's columns
#pragma unroll
    for (int c = 0; c < CW; ++c) { sc[c] = (h16)0.f; ze[c] = (h16)0.f; s2[c] = h16x2{(h16)0.f, (h16)0.f}; c2[c] = s2[c]; }
    auto load_sz = [&](int gi) {
        const h16* ps = reinterpret_cast<const h16*>(sz) + (gi - group_lo) * WSTRIP + wave * STRIP + CW * j;
        const h16* pz = ps + groups * WSTRIP;
        const uint32_t s1 = *reinterpret_cast<const uint32_t*>(ps), z1 = *reinterpret_cast<const uint32_t*>(pz);
        sc[0] = as_h2(s1).x; sc[1] = as_h2(s1).y; ze[0] = as_h2(z1).x; ze[1] = as_h2(z1).y;
#pragma unroll
        for (int c = 0; c < CW; ++c) {
            s2[c] = h16x2{sc[c], sc[c]};
            c2[c] = h16x2{ze[c], ze[c]};
        }
    };
    // 16:32: the expanded chunk (halves 0x001q for a kept row, 0 for a dropped one; see the kernel above)
    // ORed with 1024 is 1040 + q; minus 1040 the code, exactly, or -16; then the same two roundings, and
    // the dropped rows are multiplied by 0 -- bit 4 of the half, the "kept" flag, times 0x3C0 is fp16 1.0
    const uint32_t below = SPARSE ? (1u << (8 * h)) - 1u : 0u, rep_h = 0x01010101u * h;
    const uint32_t sp_nib = SPARSE ? in_vgpr(0x0F0F0F0Fu) : 0u, sp_flag = SPARSE ? in_vgpr(0x10101010u) : 0u;
    const uint32_t sp_kept = SPARSE ? in_vgpr(0x00100010u) : 0u, sp_idx = SPARSE ? in_vgpr(0x00000FF0u) : 0u;
    auto sparse_chunk = [&](const words_t w[NL], int blk, int c, uint32_t& v, uint32_t& mb4) {
        const uint32_t m = word_of<CW>(w[3 * blk + 2], c);
        const uint64_t st = ((uint64_t)word_of<CW>(w[3 * blk + 1], c) << 32) | word_of<CW>(w[3 * blk], c);
        v = (uint32_t)(st >> ((uint32_t)__builtin_popcount(m & below) << 2));
        mb4 = __builtin_amdgcn_perm(m, m, rep_h);           // mask byte h, four times
    };
    auto sparse_scaled_operand = [&](uint32_t v, uint32_t mb4, int c) -> h16x8 {
        const u32x4 sel = *reinterpret_cast<const u32x4*>(lut + (mb4 & sp_idx));
        u32x4 r = sparse_operand(v, sel, sp_nib, sp_flag);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const h16x2 kept = as_h2((r[e] & sp_kept) * 0x3C0u);
            const h16x2 q = as_h2(r[e] | 0x64006400u) - as_h2(0x64106410u);
            r[e] = bitcast<uint32_t>(((q - c2[c]) * kept) * s2[c]);
        }
        return bitcast<h16x8>(r);
    };
    // the chunk's magic numbers minus their offsets are the codes, exactly; then the reference's own
    // two roundings: fp16(fp16(q - z) s) (matmul.cuh:115-125)
    auto scaled_operand = [&](uint32_t f, int c) -> h16x8 {
        u32x4 r = bitcast<u32x4>(magic_operand<BITS>(f, m0, m1, g0, g1));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const h16x2 q = as_h2(r[e]) - as_h2(F::offs(e));
            r[e] = bitcast<uint32_t>((q - c2[c]) * s2[c]);
        }
        return bitcast<h16x8>(r);
    };

    // set f holds the weights of unit u0 + f; xr[f] the states of unit u0 + 1 + f (unit u0 goes to LDS at once)
#pragma unroll
    for (int f = 0; f < PF; ++f) load_w(w[f], min(u0 + f, u1 - 1));
    {
        const XRegs first = load_x(u0);
#pragma unroll
        for (int f = 0; f < PF; ++f) xr[f] = load_x(min(u0 + 1 + f, u1 - 1));
        const bool general = scan_scales();
        stage_x(first, 0);
        __syncthreads();

        // p: the LDS buffer that holds unit u; xn: the states of unit u + 1
        auto step = [&](auto mode, int u, int p, words_t wu[NL], XRegs& xn) {
            constexpr bool general = decltype(mode)::value;
            if (u == u0 || u % a.group_units == 0) load_sz(u / a.group_units);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                h16x8 xa[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    xa[mt] = *reinterpret_cast<const h16x8*>(xb + p * XBUF + (j + 16 * mt) * SK_PITCH + (i * 4 + h) * 16);
#pragma unroll
                for (int c = 0; c < CW; ++c) {
                    h16x8 wb;
                    if constexpr (SPARSE) {
                        uint32_t v, mb4;
                        sparse_chunk(wu, i, c, v, mb4);
                        wb = general ? exact_operand_sparse(v, mb4 & 0xFFu, sc[c], ze[c]) : sparse_scaled_operand(v, mb4, c);
                    } else {
                        const uint32_t f = chunk_bits(wu, i, c);
                        wb = general ? exact_operand<BITS>(f, m0, m1, g0, g1, sc[c], ze[c]) : scaled_operand(f, c);
                    }
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[c][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[mt], wb, acc[c][mt], 0, 0, 0);
                }
            }
            load_w(wu, min(u + PF, u1 - 1));
            if (u + 1 < u1) stage_x(xn, p ^ 1);
            xn = load_x(min(u + 1 + PF, u1 - 1));
            __syncthreads();
        };
        auto run = [&](auto mode) {
            int u = u0;
            for (; u + PF <= u1; u += PF) {               // (whole rounds without early exits, as above)
#pragma unroll
                for (int f = 0; f < PF; ++f) step(mode, u + f, f & 1, w[f], xr[f]);
            }
#pragma unroll
            for (int f = 0; f < PF - 1; ++f) {
                if (u + f >= u1) break;
                step(mode, u + f, f & 1, w[f], xr[f]);
            }
        };
        if (general) run(std::integral_constant<bool, true>{});
        else run(std::integral_constant<bool, false>{});
    }

    if (gridDim.z > 1) {
        // hand-over between the workgroups of a strip (see the kernel above): every wave stores its part of
        // the workgroup's partial tile, one counter per strip and row block
        constexpr int NV = CW * MT * 4, THROUGH = 17;
        const int tile = blockIdx.y * gridDim.x + blockIdx.x, ks = gridDim.z;
        char* const slots = reinterpret_cast<char*>(a.part) + ((int64_t)(tile * ks) * 8 + wave) * (NV * 256);
        const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
            slots + (int64_t)blockIdx.z * (8 * NV * 256), 0, NV * 256, 0x00020000);
#pragma unroll
        for (int c = 0; c < CW; ++c)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = acc[c][mt][e];
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), mine,
                                                          (((c * MT + mt) * 4 + e) * 64 + lane) * 4, 0, THROUGH);
                }
        __builtin_amdgcn_s_waitcnt(0);                 // every store of this thread has been acknowledged
        __syncthreads();
        if (t == 0) *flag = __hip_atomic_fetch_add(a.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*flag != ks - 1) return;
        if (t == 0) __hip_atomic_store(a.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int c = 0; c < CW; ++c)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[c][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int sp = 0; sp < ks; ++sp) {
            const __amdgpu_buffer_rsrc_t theirs = __builtin_amdgcn_make_buffer_rsrc(
                slots + (int64_t)sp * (8 * NV * 256), 0, NV * 256, 0x00020000);
#pragma unroll
            for (int c = 0; c < CW; ++c)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[c][mt][e] += __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                            theirs, (((c * MT + mt) * 4 + e) * 64 + lane) * 4, 0, THROUGH));
        }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = mt * 16 + 4 * h + e;
            if (m < R) {
                h16* o = a.outs + (int64_t)(row0 + m) * a.S + col0;
#pragma unroll
                for (int c = 0; c < CW; ++c) {
                    float v = acc[c][mt][e];
                    if (a.accumulate) v += (float)o[c];
                    o[c] = (h16)v;
                }
            }
        }
}

// Plan of the wide kernel: row blocks of 16 ... 64 rows, 256-column strips, K split over about as many
// workgroups as there are CUs (at least 8 units each; one counter per strip and row block: at most 1024).
struct WidePlan { bool use; int mt, row_blocks, block_rows, ksplit, units_per_split; size_t part_bytes; };
// LDS of the wide kernel: two unit buffers of states, a flag, the selector table's alignment slack, and the
// strip's scales and zeros for the workgroup's share of K (1 KB per quantisation group)
static size_t wide_lds_bytes(int block_rows, int64_t groups) {
    return 2 * (size_t)block_rows * SK_PITCH + 1024 + 16 + (size_t)groups * 256 * 4;
}
static int64_t wide_groups(int64_t units, int64_t units_per_split, int64_t ksplit, int64_t group_units) {
    int64_t groups = (units + group_units - 1) / group_units;
    if (ksplit > 1) groups = std::min(groups, (units_per_split + group_units - 1) / group_units + 1);
    return groups;
}
constexpr size_t WIDE_LDS_LIMIT = 150 * 1024;

// `group_units`: 64-row units per quantisation group (K / 64 and more: a single group)
// Whether the few-row kernel above runs 33 ... 96 rows (two or three row blocks per strip) as one round of 128 ... 256
// workgroups, or through its own split-K on a narrow output (the same conditions as unsplit_cw / plan_skinny_split).
static bool skinny_one_round(int64_t R, int64_t S, bool sparse) {
    const int64_t blocks = (R + 31) / 32;
    if (S % 64 == 0 && S / 32 * blocks < 192) return true;
    for (const int c : {4, 2, 1}) {
        if (sparse && c == 4) continue;
        const int64_t wgs = S / (16 * c) * blocks;
        if (S % (16 * c) == 0 && wgs >= 128 && wgs <= 256) return true;
    }
    return false;
}

static WidePlan plan_wide(int64_t R, int64_t K, int64_t S, bool sparse, int64_t group_units) {
    WidePlan p{false, 0, 0, 0, 1, 0, 0};
    // (knob: 1 = never, n >= 2 = from n rows on whatever the shape)
    const int64_t knob = tuning(TUNE_NO_WIDE), min_rows = knob >= 2 ? knob : 17;
    if (R < min_rows || R > SK_WIDE_MAX_ROWS || S % 256 != 0 || K % 64 != 0 || knob == 1) return p;
    // Row blocks of up to 64 rows, or of up to 128 (16:32: with two units of weights in flight per wave instead
    // of four, for the registers): every row block decodes the strip's weights again, so two blocks of 64 rows
    // cost nearly twice one block of 128 --
    // unless halving the number of workgroups means splitting K more than about six ways to fill the GPU, or
    // into shares of less than 20 units, where the hand-over of the partial tiles (twice as large, twice as
    // many) takes the gain back (measured: K=5120, S=20480, 128 rows 70 -> 52 us, int3 76 -> 58; K=8192,
    // S=28672, 128 rows 127 -> 95 us; K=28672, S=8192, 192 rows 172 -> 132 us; K=S=8192, 128 rows, 8 splits
    // instead of 4: 41 -> 46 us; K=2048, S=16384, 128 rows, shares of 8 units: 25 -> 30 us; 16:32, K=5120,
    // S=20480: 96 rows 92 -> 51 us, 128 rows 79 (256-row tiles) -> 60 us)
    const int64_t units = K / 64, forced = tuning(TUNE_MM_SPLIT);
    int64_t wgs = 0, ks = 1;
    auto shape = [&](int64_t tallest) {
        p.row_blocks = (int)((R + tallest - 1) / tallest);
        p.block_rows = (int)(((R + p.row_blocks - 1) / p.row_blocks + 15) / 16 * 16);
        p.mt = p.block_rows / 16;
        if (p.mt == 5) p.mt = 6;                      // (instantiated: 1, 2, 3, 4, 6, 8 tiles of 16 rows)
        if (p.mt == 7) p.mt = 8;
        p.block_rows = p.mt * 16;
        wgs = S / 256 * p.row_blocks;
        // (one workgroup per CU: as many splits as keep the grid within one round of 256 -- a grid a little
        // larger than that runs a second round -- and four when even the unsplit grid leaves a third of the
        // CUs idle)
        ks = 256 / wgs;
        if (ks <= 1 && wgs > 128 && wgs < 256) ks = 4;
        ks = std::max<int64_t>(1, std::min<int64_t>(ks, units / 8));
        if (forced >= 1) ks = std::min<int64_t>(forced, std::max<int64_t>(1, units / 4));
        if (wgs > 1024) ks = 1;
        // (a long share of K with small groups: more splits, within one round of workgroups, until the share's
        // scales and zeros fit the LDS)
        const size_t room = WIDE_LDS_LIMIT - (sparse ? 4096 : 0);
        while (wgs * (ks + 1) <= 256 && ks < units / 8 &&
               wide_lds_bytes(p.block_rows, wide_groups(units, (units + ks - 1) / ks, ks, group_units)) > room)
            ++ks;
    };
    shape(128);
    if (R <= 64 || ks > 6 || (ks > 1 && units / ks < 20)) shape(64);
    // (49 ... 64 rows on a narrow output: two blocks of 32 rows with half the splits instead of one block of 64 --
    // K=11008, S=4096: 28.7 -> 23.0 us; K=14336, S=4096: 31.3 -> 26.9; from 5120 columns on the single block wins on a long K)
    if (!sparse && R > 48 && R <= 64 && S <= 4096 && forced < 1) shape(32);
    // 65 ... 512 rows of a dense format against 1024 ... 32768 columns: block height
    // (up to 128, 96, 64 or 48 rows) and split by a cost model fitted to 4 900 timed launches (int4, K = 2048 ...
    // 28672, S = 4096 ... 8192, 72 ... 512 rows; its pick is within 0.3 % of the best measured candidate on average,
    // 6.6 % at worst -- on 1 800 more launches at S = 2048 and 3072 with up to 16 splits, not used in the fit: 0.3 / 3.8 %
    // (and it is used from 1024 columns on: K=8192, S=1280, 104 rows 27.8 -> 21.9 us);
    // on 1 900 more at S = 11008 ... 28672, where it serves up to 192 rows: 0.3 / 10 %, the
    // rules above 6.7 / 70 %: K=2048, S=28672, 128 rows 50 -> 30 us --,
    // where the rules above were 8 % off on K <= 8192 and up to 73 % -- e.g. K=2048, S=8192, 416 rows: seven blocks
    // of 64 rows split four ways, 49 us, against 28 us unsplit; int3, int2 and other group sizes rank alike):
    // a workgroup takes a[row tiles] us per 64-row unit of its share plus 3.9 us; a split costs 0.8 us per way
    // and 1.9 us per row tile, less 4.2; workgroups run in rounds of 256, the last one charged 3.5 us x its fill.
    // (16:32, fitted apart to 2 300 launches at S = 4096 ... 8192: 1.12 / 1.20 / 1.32 / 1.54 us per unit, 4.2 us per
    // workgroup, a split 0.9 us per way + 1.7 per row tile - 3.7, the last round 5.3 us x its fill; the pick is within
    // 0.1 % of the best candidate on average, 2.8 % at worst, where the rules above were 5 % / 27 % off -- K=4096,
    // S=8192, 160 rows 50 -> 39 us; K=14336, S=8192, 128 rows 82 -> 69)
    struct WideCost { double per_unit[9], workgroup, split, per_way, per_tile, last_round; };
    static const WideCost dense_cost = {{0, 0, 0, 0.617, 0.707, 0, 0.912, 0, 1.059}, 3.92, -4.164, 0.798, 1.915, 3.544};
    static const WideCost sparse_cost = {{0, 0, 0, 1.12, 1.203, 0, 1.32, 0, 1.537}, 4.17, -3.744, 0.921, 1.701, 5.284};
    if (R > 64 && S >= (sparse ? 4096 : 1024) && S <= (sparse ? 8192 : 32768) && forced < 1) {
        const WideCost& wc = sparse ? sparse_cost : dense_cost;
        const size_t room = WIDE_LDS_LIMIT - (sparse ? 4096 : 0);
        double best = 1e30;
        int64_t best_tall = 0, best_ks = 1;
        for (const int64_t tallest : {128, 96, 64, 48}) {
            shape(tallest);
            const int64_t tiles = wgs;
            for (int64_t k = 1; k <= 16 && (k == 1 || units / k >= 8) && tiles * k <= 1024; ++k) {
                const int64_t share = (units + k - 1) / k, rounds = (tiles * k + 255) / 256, last = tiles * k - (rounds - 1) * 256;
                if (wide_lds_bytes(p.block_rows, wide_groups(units, share, (units + share - 1) / share, group_units)) > room) continue;
                const double t = rounds * (wc.per_unit[p.mt] * share + wc.workgroup) +
                                 (k > 1 ? wc.split + wc.per_way * k + wc.per_tile * p.mt : 0.0) +
                                 (rounds > 1 ? wc.last_round * last / 256.0 : 0.0);
                if (t < best) { best = t; best_tall = tallest; best_ks = k; }
            }
        }
        if (best_tall != 0) { shape(best_tall); ks = best_ks; }
    }
    p.units_per_split = (int)((units + ks - 1) / ks);
    p.ksplit = (int)((units + p.units_per_split - 1) / p.units_per_split);
    if (wide_lds_bytes(p.block_rows, wide_groups(units, p.units_per_split, p.ksplit, group_units)) >
        WIDE_LDS_LIMIT - (sparse ? 4096 : 0))
        return p;
    // measured against the kernel above (K = 2048 ... 20480, S = 1024 ... 28672): with 17 ... 32 rows it
    // needs 32 ... 96 strips and long shares of K, with 33 ... 64 rows matrices of 32 M weights and more
    // and from 129 rows on the tile kernels win on wide outputs (beyond 14336 columns; from 193 rows beyond
    // 10240, from 257 rows beyond 8192 -- K=8192, S=10240, 192 rows: 52 against 64 us; K=4096, S=14336, 192
    // rows: 42.5 against 49, 256 rows: 52 against 50)
    // (16:32, whose decode costs more here and in the tile kernels alike: 17 ... 32 rows from 64 M weights
    // on, 33 ... 64 rows from 32 M, 65 ... 128 rows always, up to 256 rows for outputs of at most 8192 columns
    // -- K=S=8192, 192 rows: 59 against 71 us --, beyond that of at most 4096)
    if (knob < 2 && forced < 1) {
        if (sparse) {
            if (R <= 32 && K * S < (1ll << 26)) return p;
            // (33 ... 64 rows: the kernel above while its two row blocks per strip make one round of workgroups -- outputs
            // of at most 4096 columns -- up to K = 8192: K=S=4096, 40 / 64 rows 16.3 / 16.3 against 20.9 / 23.4 us; K=8192,
            // S=4096 25.3 / 24.8 against 27.5 / 31.1; beyond that only on a short K: K=4096, S=5120 28.3 / 29.3 against
            // 22.5 / 24.8; K=5120, S=6144 33.5 / 33.9 against 23.3 / 26.7)
            if (R > 32 && R <= 64 &&
                (skinny_one_round(R, S, true) ? (K <= 8192 || S < 3072) : (K < 4096 && K * S < (1ll << 25))))
                return p;
            // (the padded 256-row tiles win on very wide outputs against two row blocks)
            if (R > 96 && R <= 128 && S > 16384 && p.row_blocks > 1) return p;
            if (R > 128 && (S > 8192 || (R > 256 && S > 4096))) return p;
        } else {
            // (24 ... 31 strips only on a long K: K=14336, S=6144, 20 / 32 rows 24.5 / 24.5 against 29.6 / 32.3 us for the
            // kernel above; K=8192, S=6144 18.9 / 19.0 against 18.7 / 19.5)
            if (R <= 32 && (wgs < (units >= 160 ? 24 : 32) || wgs > 96 || p.units_per_split < 16)) return p;
            // (one round of 129 ... 256 strips of 64 columns: the kernel above up to K = 6144 -- K=4096, S=14336, 20 / 32
            // rows 16.3 / 17.7 against 18.4 / 18.3 us; K=5120, S=16384 19.4 / 21.8 against 22.7 / 22.8; K=8192, S=12288
            // 25.8 / 27.1 against 25.1 / 25.1)
            if (R <= 32 && S % 64 == 0 && S / 64 > 128 && S / 64 <= 256 && K <= 6144) return p;
            // (33 ... 64 rows are two row blocks of the kernel above: where its strips can be cut to give one round of
            // 128 ... 256 workgroups -- or its own split-K serves a narrow output -- it wins up to K = 5120, on outputs
            // of at most 4096 columns up to K = 8192 and below 3072 columns always: K=S=4096, 40 / 64 rows 13.0 / 13.2
            // against 16.1 / 18.7 us; K=5120, S=8192 18.5 / 18.9 against 19.4 / 22.3; K=8192, S=4096 19.5 / 19.6 against
            // 22.3 / 26.6; K=8192, S=6144 24.7 / 25.0 against 21.9 / 25.4; K=14336, S=5120 36.9 against 27.6 / 31.3)
            if (R > 32 && R <= 64 &&
                (skinny_one_round(R, S, false) ? (K <= 5120 || (K <= 8192 && S <= 4096) || S < 3072) : K * S < (1ll << 25)))
                return p;
            // (with the plan from the cost model, up to 192 rows on any width it covers: K=4096, S=20480, 160 rows 50 us
            // against 71 for the tiles, K=8192, S=20480, 192 rows 97 against 114, K=2048, S=20480 29 against 40)
            // (193 ... 256 rows: on a K of at most 4096 as well -- K=4096, S=20480, 256 rows 64 against 74 us; K=8192: 122
            // against 114)
            if (R > 128 && S > 8192 && S > (R <= 192 ? 32768 : R <= 256 ? (K <= 4096 ? 32768 : 10240) : 8192)) return p;
        }
    }
    p.part_bytes = p.ksplit > 1 ? (size_t)wgs * 8 * p.ksplit * (2 * p.mt * 4 * 256) : 0;
    p.use = true;
    return p;
}

template <int BITS, bool SPARSE = false>
static bool launch_wide(SkinnyArgs a, const WidePlan& p, hipStream_t st) {
    const size_t lds = wide_lds_bytes(p.block_rows, wide_groups(a.K / 64, p.units_per_split, p.ksplit, a.group_units));
    if (lds > WIDE_LDS_LIMIT - (SPARSE ? 4096 : 0)) return false;
    a.block_rows = p.block_rows;
    a.units_per_split = p.units_per_split;
    const dim3 grid((unsigned)(a.S / 256), (unsigned)p.row_blocks, (unsigned)p.ksplit), block(512);
    if (noting("wide_rows_kernel<bits=%d,%s,row_tiles=%d> strips=%u row_blocks=%u ksplit=%u", BITS, SPARSE ? "16:32" : "dense", p.mt,
               grid.x, grid.y, grid.z))
        return true;
    auto go = [&](auto kernel, int slot) {
        static std::atomic<uint64_t> done[6];
        int dev = 0;
        hipGetDevice(&dev);
        const uint64_t bit = 1ull << (dev & 63);
        if (!(done[slot].load(std::memory_order_relaxed) & bit)) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
            done[slot].fetch_or(bit, std::memory_order_relaxed);
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, st, a.matrix, a.x, a.scales, a.zeros, a.S, a.K, a.group_units, a.units_per_split, a);
    };
    if (p.mt == 1) go(wide_rows_kernel<BITS, 1, SPARSE>, 0);
    else if (p.mt == 2) go(wide_rows_kernel<BITS, 2, SPARSE>, 1);
    else if (p.mt == 3) go(wide_rows_kernel<BITS, 3, SPARSE>, 2);
    else if (p.mt == 4) go(wide_rows_kernel<BITS, 4, SPARSE>, 3);
    else if (p.mt == 6) go(wide_rows_kernel<BITS, 6, SPARSE>, 4);
    else go(wide_rows_kernel<BITS, 8, SPARSE>, 5);
    return true;
}

template <int BITS, int CW, bool SPARSE>
static bool launch_skinny(const SkinnyArgs& a, int waves, int ksplit, hipStream_t st) {
    const int strips = a.S / (16 * CW);
    const int rt = ((a.R > 32 ? 32 : a.R) + 7) / 8;
    int groups = (a.K / 64 + a.group_units - 1) / a.group_units;
    if (ksplit > 1) groups = std::min(groups, (a.units_per_split + a.group_units - 1) / a.group_units + 1);
    size_t lds = (size_t)waves * SK_WAVE_LDS + 16 + (size_t)groups * 16 * CW * 4;
    const size_t red = (size_t)(waves / 2) * (rt <= 2 ? 1 : 2) * 16 * 16 * CW * 4;
    if (red > lds) lds = red;
    if (lds > 150 * 1024 - (SPARSE ? 4096 : 0)) return false;      // (16:32: 4 KB of static LDS for the selector table)
    const dim3 grid(strips, (a.R + 31) / 32, ksplit), block(waves * 64);
    if (noting("skinny_kernel<bits=%d,%s,columns_per_lane=%d,row_tiles=%d> strips=%d row_blocks=%u ksplit=%d waves=%d", BITS,
               SPARSE ? "16:32" : "dense", CW, rt <= 1 ? 1 : (rt <= 2 ? 2 : 4), strips, grid.y, ksplit, waves))
        return true;
    auto go = [&](auto kernel, int slot) {
        // more than 64 KB of dynamic LDS has to be requested once per kernel and device
        static std::atomic<uint64_t> done[3];
        int dev = 0;
        hipGetDevice(&dev);
        const uint64_t bit = 1ull << (dev & 63);
        if (!(done[slot].load(std::memory_order_relaxed) & bit)) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                150 * 1024);
            done[slot].fetch_or(bit, std::memory_order_relaxed);
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, st, a.matrix, a.x, a.scales, a.zeros, a.S, a.K, a.group_units, a.units_per_wave, a);
    };
    if (rt <= 1) go(skinny_kernel<BITS, CW, 1, SPARSE>, 0);
    else if (rt <= 2) go(skinny_kernel<BITS, CW, 2, SPARSE>, 1);
    else go(skinny_kernel<BITS, CW, 4, SPARSE>, 2);
    return true;
}

// The balanced launch: 64-column strips, eight waves, `wgs` workgroups that share strips x units evenly.
// Partial tiles of the strips that two workgroups share: two slots per strip in `part`, one counter per strip.
constexpr int SK_BAL_WGS = 256;
static_assert(SK_BAL_WGS == 1 << 8, "balanced_share divides by it with a shift");
static size_t skinny_balanced_part_bytes(int64_t S) { return (size_t)(S / 64) * 2 * (4 * 2 * 4 * 256); }
// Where it pays (8 and 16 rows, K = 3072 ... 14336, us, a workgroup per strip / shared): int4 K=5120, S=20480 19.1 / 16.6,
// K=8192, S=18432 27.4 / 21.0, K=3072, S=20480 13.8 / 12.9; 16:32 K=5120, S=20480 29.5 / 24.5, K=8192, S=18432 43.5 / 31.0;
// beyond a quarter more strips than CUs only on a long K, where a workgroup per strip means eight waves each and two
// rounds (K=12288, S=28672 48.5 / 39.8, K=10240, S=24576 39.0 / 30.9; K=8192, S=22016 28.7 / 29.3 and K=4096, S=28672
// 17.2 / 18.0 do not gain).  17 ... 32 rows, whose accumulators fill the register file, lose (K=2048, S=20480 14.8 / 15.9).
static bool balanced_shape(int64_t R, int64_t K, int64_t S) {
    const int64_t strips = S / 64, units = K / 64;
    if (R < 2 || R > 16 || S % 64 != 0 || strips <= SK_BAL_WGS || strips >= 2 * SK_BAL_WGS || strips * units >= (1ll << 22)) return false;
    return units >= (strips <= SK_BAL_WGS * 5 / 4 ? 48 : 160);
}
template <int BITS, bool SPARSE>
static bool launch_skinny_balanced(SkinnyArgs a, hipStream_t st) {
    constexpr int CW = 4, WAVES = 8;
    const int strips = a.S / 64, units = a.K / 64;
    const int rt = (a.R + 7) / 8;
    const int64_t total = (int64_t)strips * units;
    a.bal_q = (int)(total / SK_BAL_WGS);
    a.bal_r = (int)(total % SK_BAL_WGS);
    a.bal_magics = {div_magic((uint32_t)units), div_magic((uint32_t)a.group_units), div_magic((uint32_t)a.bal_q), div_magic((uint32_t)a.bal_q + 1u)};
    // scales in LDS: a workgroup's range is less than two strips long and touches at most three
    const int groups = 2 * ((units + a.group_units - 1) / a.group_units) + 3;
    size_t lds = (size_t)WAVES * SK_WAVE_LDS + 16 + (size_t)groups * 16 * CW * 4;
    const size_t red = (size_t)WAVES * 16 * 16 * CW * 4;
    if (red > lds) lds = red;
    if (lds > 150 * 1024 - (SPARSE ? 4096 : 0)) return false;
    const dim3 grid(SK_BAL_WGS, 1, 1), block(WAVES * 64);
    if (noting("skinny_kernel<bits=%d,%s,columns_per_lane=%d,row_tiles=%d,balanced> strips=%d row_blocks=1 workgroups=%d waves=%d",
               BITS, SPARSE ? "16:32" : "dense", CW, rt <= 1 ? 1 : 2, strips, SK_BAL_WGS, WAVES))
        return true;
    auto go = [&](auto kernel) {
        static std::atomic<uint64_t> done;
        int dev = 0;
        hipGetDevice(&dev);
        const uint64_t bit = 1ull << (dev & 63);
        if (!(done.load(std::memory_order_relaxed) & bit)) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                150 * 1024);
            done.fetch_or(bit, std::memory_order_relaxed);
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, st, a.matrix, a.x, a.scales, a.zeros, a.S, a.K, a.group_units, a.units_per_wave, a);
    };
    if (rt <= 1) go(skinny_kernel<BITS, CW, 1, SPARSE, true>);
    else go(skinny_kernel<BITS, CW, 2, SPARSE, true>);            // (up to 16 rows: balanced_shape)
    return true;
}

// Between 256 and 320 strips of 64 columns: 256 workgroups of four or five slivers of 16 columns each, so that
// every CU has one workgroup and none a second (dense formats, up to 16 rows).
// int3 and int2 (8 and 16 rows, us, a workgroup per strip / shared strips / slivers): K=5120, S=20480 int3 22.5 / 19.3 / 17.8,
// int2 21.2 / 18.2 / 16.6; K=8192, S=18432 int3 32.4 / 24.1 / 24.2; K=14336, S=19200 int3 56.2 / 44.8 / 38.8, int2 53.0 / 41.3 /
// 34.6.  int4, whose words carry a third more bytes per unit, does better with shared strips (K=5120, S=20480 18.5 with
// slivers), and so does 16:32, which has no registers for a fifth column.
static bool sliver_shape(int bits, int64_t R, int64_t K, int64_t S, bool sparse) {
    const int64_t slivers = S / 16;
    return !sparse && bits != 4 && R >= 2 && R <= 16 && S % 64 == 0 && slivers > 4 * SK_BAL_WGS && slivers <= 5 * SK_BAL_WGS &&
           K / 64 >= 48;
}
template <int BITS>
static bool launch_skinny_slivers(SkinnyArgs a, hipStream_t st) {
    constexpr int CW = 4, CT = 5, WAVES = 8;
    const int rt = (a.R + 7) / 8;
    a.wide_wgs = a.S / 16 - 4 * SK_BAL_WGS;
    a.units_per_split = a.K / 64;
    a.units_per_wave = (a.units_per_split + WAVES - 1) / WAVES;
    const int groups = (a.K / 64 + a.group_units - 1) / a.group_units;
    size_t lds = (size_t)WAVES * SK_WAVE_LDS + 16 + (size_t)groups * 16 * CT * 4;
    const size_t red = (size_t)(WAVES / 2) * 16 * 16 * CT * 4;
    if (red > lds) lds = red;
    if (lds > 150 * 1024) return false;
    const dim3 grid(SK_BAL_WGS, 1, 1), block(WAVES * 64);
    if (noting("skinny_kernel<bits=%d,dense,columns_per_lane=4+1,row_tiles=%d> strips=%d (%d of 80 columns, the others of 64) "
               "row_blocks=1 ksplit=1 waves=%d", BITS, rt <= 1 ? 1 : 2, SK_BAL_WGS, a.wide_wgs, WAVES))
        return true;
    auto go = [&](auto kernel) {
        static std::atomic<uint64_t> done;
        int dev = 0;
        hipGetDevice(&dev);
        const uint64_t bit = 1ull << (dev & 63);
        if (!(done.load(std::memory_order_relaxed) & bit)) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                150 * 1024);
            done.fetch_or(bit, std::memory_order_relaxed);
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, st, a.matrix, a.x, a.scales, a.zeros, a.S, a.K, a.group_units, a.units_per_wave, a);
    };
    if (rt <= 1) go(skinny_kernel<BITS, CW, 1, false, false, 1>);
    else go(skinny_kernel<BITS, CW, 2, false, false, 1>);
    return true;
}

template <int BITS, bool SPARSE = false>
static bool launch_skinny_cw(const SkinnyArgs& a, int cw, int waves, int ksplit, hipStream_t st) {
    if (cw == 4) return launch_skinny<BITS, 4, SPARSE>(a, waves, ksplit, st);
    if (cw == 2) return launch_skinny<BITS, 2, SPARSE>(a, waves, ksplit, st);
    return launch_skinny<BITS, 1, SPARSE>(a, waves, ksplit, st);
}

// Columns per lane of the unsplit kernel: the widest strips (64, 32 or 16 columns) that still give at
// least 256 workgroups, else at least 128 (narrow strips use half a cache line per packed row).
static int unsplit_cw(int64_t R, int64_t S, bool sparse) {
    int cw = 1;
    // (more than 32 rows run as two or three row blocks per strip, each a workgroup: the widest strips -- within what
    // the format's registers allow -- that give one round of 128 ... 256 workgroups, where there are such: K=2048,
    // S=8192, 40 rows in 256 workgroups of 64 columns instead of 512 of 32)
    if (R > 32) {
        const int64_t blocks = (R + 31) / 32;
        int64_t best = 0;
        for (const int c : {4, 2, 1}) {
            if (sparse && c == 4) continue;
            const int64_t wgs = S / (16 * c) * blocks;
            if (S % (16 * c) == 0 && wgs >= 128 && wgs <= 256 && wgs > best) { best = wgs; cw = c; }
        }
        if (best != 0) return cw;
    }
    // (64-column strips as soon as they give more than half a round of workgroups: 129 ... 255 of them finish in one
    // round where twice as many 32-column strips need two -- up to 16 rows, us: K=8192, S=12288 21.5 -> 17.4; K=14336,
    // S=14336 38.3 -> 25.5; K=4096, S=10240 12.9 -> 11.9; 16:32, K=8192, S=12288 32.8 -> 26.0)
    const int prefer[4][2] = {{4, 129}, {2, 256}, {4, 128}, {2, 128}};       // {columns per lane, workgroups}
    for (const auto& c : prefer)
        if (S % (16 * c[0]) == 0 && S / (16 * c[0]) >= c[1]) { cw = c[0]; break; }
    // (16:32 with more than 16 rows: four columns per lane would not fit the register file)
    if (sparse && R > 16 && cw == 4) cw = 2;
    return cw;
}

// Split-K plan of the few-row kernel: when even 32-column strips would give fewer than 192 workgroups,
// 64-column strips with as many workgroups per strip as come closest to one per CU, each with at least
// six units per wave -- if that makes at least as many workgroups as the unsplit choice of narrower
// strips (with more than 16 rows, where wide strips matter more: half as many).  `part_bytes`: room for
// the partial tiles (0: no split).
struct SkinnySplit { int cw, ksplit; size_t tiles, part_bytes; };
static SkinnySplit plan_skinny_split(int64_t R, int64_t K, int64_t S, bool sparse) {
    SkinnySplit p{0, 1, 0, 0};
    if (S % 64 != 0 || R < 2 || R > 96) return p;
    const int64_t row_blocks = (R + 31) / 32, units = K / 64;
    if (S / 32 * row_blocks >= 192) return p;
    const int cw = sparse && R > 16 ? 2 : 4;
    const int64_t wgs = S / (16 * cw) * row_blocks;
    int64_t ks = std::min<int64_t>(256 / wgs, units / (8 * 6));
    if ((R > 16 ? 2 : 1) * wgs * ks < S / (16 * unsplit_cw(R, S, sparse)) * row_blocks) ks = 1;
    const int64_t forced = tuning(TUNE_MM_SPLIT);
    if (forced >= 1) ks = std::min<int64_t>(forced, std::max<int64_t>(1, units / 16));
    if (ks < 2 || wgs > 1024) return p;
    p.cw = cw;
    p.ksplit = (int)ks;
    p.tiles = (size_t)wgs;
    p.part_bytes = (size_t)wgs * ks * (cw * 2 * 4 * 256);       // up to 32 rows x 16 cw columns of fp32 per partial
    return p;
}

size_t skinny_workspace_bytes(int64_t R, int64_t K, int64_t S, bool sparse) {
    const SkinnySplit p = plan_skinny_split(R, K, S, sparse);
    // (the split of the wide kernel can depend on the group size: room for whichever needs most)
    size_t wide = 0;
    for (const int64_t group_units : {1, 2, 3, 4, 6, 8, 16, 0x7FFFFFF}) {
        const WidePlan w = plan_wide(R, K, S, sparse, group_units);
        if (w.use) wide = std::max(wide, w.part_bytes);
    }
    const size_t balanced = balanced_shape(R, K, S) ? skinny_balanced_part_bytes(S) : 0;
    return std::max(std::max<size_t>(p.ksplit > 1 ? p.part_bytes : 0, wide), balanced);
}

// Product of 2 <= R <= 96 rows with a dense or (sparse_mask != nullptr) 16:32 sparse int4 matrix; beyond that
// the tile kernels are faster.  Returns false when the shape is not one this kernel takes (the caller then
// uses the general kernels).
bool skinny_rows(int bits, h16* outs, const uint32_t* matrix, const h16* x, const h16* scales, const h16* zeros,
                 int64_t R, int64_t K, int64_t S, int64_t group_size, bool accumulate, hipStream_t st,
                 const uint32_t* sparse_mask, void* workspace, size_t workspace_bytes) {
    if (R < 2 || R > SK_WIDE_MAX_ROWS || S % 16 != 0 || K % 64 != 0 || K > (1 << 30) || S > (1 << 28)) return false;
    if (sparse_mask && bits != 4) return false;
    SkinnyArgs a;
    a.outs = outs; a.matrix = matrix; a.mask = sparse_mask; a.x = x; a.scales = scales; a.zeros = zeros;
    a.R = (int)R; a.K = (int)K; a.S = (int)S;
    const int64_t gu = group_size / 64;
    a.group_units = (int)(gu > 0x7FFFFFF ? 0x7FFFFFF : gu);
    a.accumulate = accumulate ? 1 : 0;
    a.block_rows = 32;
    a.part = nullptr;
    a.counters = nullptr;
    a.bal_q = 0; a.bal_r = 0;
    a.wide_wgs = 0;
    // 33 rows and more, dense: the kernel whose waves share the staged states
    {
        const WidePlan wp = plan_wide(R, K, S, sparse_mask != nullptr, a.group_units);
        const WorkspaceParts ws = workspace_parts(workspace, workspace_bytes);
        if (wp.use && (wp.ksplit == 1 || (ws.counters != nullptr && ws.scratch_bytes >= wp.part_bytes))) {
            a.units_per_wave = 0;
            a.counters = reinterpret_cast<int*>(ws.counters);
            a.part = reinterpret_cast<float*>(ws.scratch);
            const bool ok = sparse_mask ? launch_wide<4, true>(a, wp, st)
                          : bits == 4 ? launch_wide<4>(a, wp, st) : bits == 3 ? launch_wide<3>(a, wp, st) : launch_wide<2>(a, wp, st);
            if (ok) return true;
        }
    }
    if (R > 96) return false;
    // four waves split K when there are more workgroups than CUs (three of them fit a CU) and K
    // is short (each wave should walk a dozen units or more), eight otherwise -- also at exactly one
    // workgroup per CU, where eight waves keep twice the bytes in flight (K=5120, S=16384, 8 rows:
    // 14.6 -> 12.0 us; K=S=8192: 16.5 -> 12.3 us; 320 and 448 strips: 17.7 against 22.2, 27 against 32)
    int cw = unsplit_cw(R, S, sparse_mask != nullptr);
    {   // (tuning: columns per lane of the few-row kernel where the shape allows them)
        const int64_t forced_cw = tuning(TUNE_MV_LK);
        if ((forced_cw == 1 || forced_cw == 2 || (forced_cw == 4 && !(sparse_mask && R > 16))) && S % (16 * forced_cw) == 0)
            cw = (int)forced_cw;
    }
    const int units = (int)(K / 64);
    int waves = (int)tuning(TUNE_MV_WAVES);
    if (waves != 2 && waves != 4 && waves != 8) waves = S / (16 * cw) > 256 && units < 160 ? 4 : 8;
    while (waves > 1 && units < 2 * waves) waves >>= 1;
    auto launch = [&](int cw_, int waves_, int ksplit_) {
        a.units_per_wave = (a.units_per_split + waves_ - 1) / waves_;
        if (sparse_mask) return launch_skinny_cw<4, true>(a, cw_, waves_, ksplit_, st);
        if (bits == 4) return launch_skinny_cw<4>(a, cw_, waves_, ksplit_, st);
        if (bits == 3) return launch_skinny_cw<3>(a, cw_, waves_, ksplit_, st);
        return launch_skinny_cw<2>(a, cw_, waves_, ksplit_, st);
    };
    // split-K across workgroups where the plan asks for it and the scratch half of the workspace has room
    // for the partial tiles (per-strip counters: last page of the half that is kept zero)
    a.part = nullptr;
    a.counters = nullptr;
    const SkinnySplit sp = plan_skinny_split(R, K, S, sparse_mask != nullptr);
    const WorkspaceParts ws = workspace_parts(workspace, workspace_bytes);
    if (sp.ksplit > 1 && ws.counters != nullptr && ws.scratch_bytes >= sp.part_bytes) {
        a.units_per_split = (units + sp.ksplit - 1) / sp.ksplit;
        a.counters = reinterpret_cast<int*>(ws.counters);
        a.part = reinterpret_cast<float*>(ws.scratch);
        const int ksplit = (units + a.units_per_split - 1) / a.units_per_split;          // no empty split
        if (launch(sp.cw, 8, ksplit)) return true;
    }
    a.units_per_split = units;
    // a quarter more 64-column strips than CUs at most: a workgroup per CU, of 64 or 80 columns
    if (tuning(TUNE_NO_BALANCE) == 0 && tuning(TUNE_MV_LK) == 0 && sliver_shape(bits, R, K, S, sparse_mask != nullptr)) {
        const bool ok = bits == 3 ? launch_skinny_slivers<3>(a, st) : launch_skinny_slivers<2>(a, st);
        if (ok) return true;
    }
    // more 64-column strips than CUs, fewer than twice as many: one workgroup per CU, the strips' units shared evenly
    // (16:32 with more than 16 rows has no 64-column strips)
    if (cw == 4 && tuning(TUNE_NO_BALANCE) == 0 && balanced_shape(R, K, S) && ws.counters != nullptr &&
        ws.scratch_bytes >= skinny_balanced_part_bytes(S)) {
        a.counters = reinterpret_cast<int*>(ws.counters);
        a.part = reinterpret_cast<float*>(ws.scratch);
        a.units_per_wave = 0;
        const bool ok = sparse_mask ? launch_skinny_balanced<4, true>(a, st)
                      : bits == 4 ? launch_skinny_balanced<4, false>(a, st)
                      : bits == 3 ? launch_skinny_balanced<3, false>(a, st) : launch_skinny_balanced<2, false>(a, st);
        if (ok) return true;
        a.counters = nullptr;
        a.part = nullptr;
    }
    return launch(cw, waves, 1);
}

}  // namespace i4
