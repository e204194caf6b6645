// Quantized matrix-vector product for gfx950: outs = fp16(fp32(outs) + x @ W).
//
// Bandwidth-bound streaming kernel.  The packed matrix is [rows, S] with the
// column index contiguous, so lanes own columns: a lane reads 16 bytes = the
// packed words of 4 adjacent columns of one packed row.  K is cut into 64-row
// "units" (the granularity of quantisation groups).  A wavefront is LK lane
// groups of 64/LK lanes; each lane group streams its own units, so one load
// instruction fetches LK contiguous segments of (64/LK)*16 bytes.  A workgroup
// owns a strip of (64/LK)*4 columns and a range of units; grid.y cuts K further.
//
// The states x of the workgroup's K range are staged once in LDS, already
// permuted into the half2 pairs the decode produces, together with per-unit
// sums; every lane of a lane group reads the same LDS address (a broadcast).
//
// Arithmetic (int4 / int2): codes are never converted one by one.  A mask and
// an OR turn two fields of a word into a half2 whose lanes are 2^e + q ("magic"
// exponents chosen so that the field lands on the units of the mantissa),
// v_dot2_f32_f16 multiplies the pair by the matching pair of states into an fp32
// accumulator, and the constant part sum_k 2^e_k x_k is removed once per unit.
// Per (unit, column):  y += s * (sum_k x_k q_k - z * sum_k x_k), the exact value
// of sum_k x_k (q_k - z) s; the two fp16 roundings the reference applies to each
// weight are not reproduced here (the dequantise helper is the bit-exact one).
// Columns whose scale is negative (exponent quantisation) are left out of the
// fast loop and handled by a second, general loop that only runs if any exist.
//
// Partial sums meet in LDS; across workgroups they meet in 8-byte slots of the
// workspace {fp32 partial, flag}: a workgroup publishes its slots with
// device-scope write-through stores and leaves; the workgroup with the highest
// index of the strip polls the slots, adds them in a fixed order
// (deterministic), adds the prior contents of outs, writes fp16 and clears the
// slots.  No cache-wide fence and no read-modify-write atomics are used.
#include "common.h"

#include <algorithm>
#include <mutex>

namespace i4 {

constexpr int MV_MAX_WAVES = 8;
constexpr int MV_MAX_SPLITS = 32;          // slots per column in the workspace
constexpr int MV_MAX_UNITS_WG = 224;      // LDS staging: up to 264 B per unit, 64 KB in all

struct MatvecArgs {
    h16* outs;
    const uint32_t* matrix;
    const uint32_t* mask;
    const h16* x;
    const h16* scales;
    const h16* zeros;
    uint64_t* slots;        // [splits - 1][S] hand-over slots {partial sum, flag}
    int K, S;
    int units_total;        // K / 64
    int units_per_wg;
    int group_units;        // group size in units (>= 1); huge for a single group
    uint32_t group_magic;   // div_magic(group_units)
    int splits;             // == gridDim.y
    uint32_t* sticky;       // hand-over error word of the workspace (non-zero: poisoned)
    int spin_limit;         // polls before a reader gives up
    int rows;               // several rows of states in one pass (NR = 4 kernels): how many (2 .. 4), K apart in x, S apart in outs
    int accumulate;         // ... and whether they add onto outs (the matvec entry) or overwrite it (the matmul entry)
};

// ------------------------------------------------------------------ formats
template <int BITS, bool SPARSE> struct Fmt;
// ROWS / MROWS: packed weight / mask rows per unit; XS: bytes of staged states per unit
template <> struct Fmt<4, false> { static constexpr int ROWS = 8, MROWS = 0, XS = 128; static constexpr bool FAST = true; };
template <> struct Fmt<3, false> { static constexpr int ROWS = 6, MROWS = 0, XS = 160; static constexpr bool FAST = true; };
template <> struct Fmt<2, false> { static constexpr int ROWS = 4, MROWS = 0, XS = 128; static constexpr bool FAST = true; };
template <> struct Fmt<4, true>  { static constexpr int ROWS = 4, MROWS = 2, XS = 128; static constexpr bool FAST = true; };

template <int BITS, bool SPARSE>
struct Unit {
    u32x4 w[Fmt<BITS, SPARSE>::ROWS];
    u32x4 m[Fmt<BITS, SPARSE>::MROWS == 0 ? 1 : Fmt<BITS, SPARSE>::MROWS];
    u32x2 sc, ze;            // fp16 scales / zeros of the lane's 4 columns
};

template <int BITS, bool SPARSE>
__device__ __forceinline__ void load_unit(Unit<BITS, SPARSE>& u, const MatvecArgs& a, int unit, int col) {
    constexpr int ROWS = Fmt<BITS, SPARSE>::ROWS, MROWS = Fmt<BITS, SPARSE>::MROWS;
    const int64_t S = a.S;
    // scale / zero first: loads return in order, so the unit is complete when its last weight
    // row arrives instead of two small requests to other pages later
    const int64_t gofs = (int64_t)magic_div(unit, a.group_units, a.group_magic) * S + col;
    u.sc = *reinterpret_cast<const u32x2*>(a.scales + gofs);
    u.ze = *reinterpret_cast<const u32x2*>(a.zeros + gofs);
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t* p = a.matrix + (int64_t)unit * ROWS * S + col;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) u.w[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + r * S));
    if constexpr (MROWS > 0) {
        const uint32_t* q = a.mask + (int64_t)unit * MROWS * S + col;
#pragma unroll
        for (int r = 0; r < MROWS; ++r) u.m[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q + r * S));
    }
}

// (mask and magic are held in registers, in_vgpr: one v_and_or_b32)
__device__ __forceinline__ uint32_t and_or(uint32_t w, uint32_t mask, uint32_t magic) {
    return (w & mask) | magic;
}

// operand of the matrix core for one pair: {2^a + q, 2^b + q'} (linear mode, offsets removed
// later) or {+-2^e, +-2^e'} (exponent mode, nothing to remove); `offsets` = {2^a, 2^b} as integers
template <int BITS, bool EXPO>
__device__ __forceinline__ uint32_t operand(uint32_t w, uint32_t mask, uint32_t magic, uint32_t offsets) {
    const uint32_t h = and_or(w, mask, magic);
    if constexpr (EXPO) return expo_operand<BITS>(h, offsets);
    else return h;
}

// ---- fast paths.  xp points at the unit's staged states (LDS).
//
// The multiply-accumulate itself runs on the matrix core, which is otherwise
// idle in a matvec and executes beside the VALU: v_mfma_f32_4x4x4_16B_f16 is 16
// independent 4x4x4 products, block b = lanes 4b..4b+3; lane 4b+j supplies
// column j of B (4 consecutive k) and lane 4b+i row i of A.  Every lane passes
// the same four states as its A row and its own four weights as its B column,
// so each of the lane's 4 result registers holds its column's dot product.
typedef _Float16 h16x4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mma4(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, f32x4 c) {
    const u32x2 a = {a0, a1}, b = {b0, b1};
    return __builtin_amdgcn_mfma_f32_4x4x4f16(bitcast<h16x4v>(a), bitcast<h16x4v>(b), c, 0, 0, 0);
}

// int4: word bits: code j at 4j.  Pairs (j, j+4) sit at equal offsets in the two
// halves of the word; offsets 0 and 4 are inside the fp16 mantissa, so
//   (w & 0x000F000F) | 0x64006400 = {1024 + q0, 1024 + q4}
//   (w & 0x00F000F0) | 0x54005400 = {  64 + q1,   64 + q5}
// and the same two masks on w >> 8 give (q2,q6) and (q3,q7).  Staged states per
// packed row: {x0,x4},{x1,x5},{x2,x6},{x3,x7}.  off_k = 1024 (k even), 64 (k odd).
// MV_NCOL of the lane's 4 columns are accumulated side by side (independent MFMA
// chains); fewer chains need fewer accumulator registers at the price of
// re-reading the staged states.
#ifndef MV_NCOL
#define MV_NCOL 2
#endif
template <bool EXPO = false>
__device__ __forceinline__ void unit_fast(const Unit<4, false>& u, const h16* xp, f32x4 acc[4]) {
    const uint32_t M0 = in_vgpr(0x000F000Fu), M1 = in_vgpr(0x00F000F0u);
    const uint32_t G0 = in_vgpr(0x64006400u), G1 = in_vgpr(0x54005400u);
    constexpr uint32_t O0 = off2(1024, 1024), O1 = off2(64, 64);
#pragma unroll
    for (int c0 = 0; c0 < 4; c0 += MV_NCOL) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const u32x4 p = *reinterpret_cast<const u32x4*>(xp + r * 8);
#pragma unroll
            for (int c = c0; c < c0 + MV_NCOL; ++c) {
                const uint32_t w = u.w[r][c], w8 = w >> 8;
                acc[c] = mma4(p.x, p.y, operand<4, EXPO>(w, M0, G0, O0), operand<4, EXPO>(w, M1, G1, O1), acc[c]);
                acc[c] = mma4(p.z, p.w, operand<4, EXPO>(w8, M0, G0, O0), operand<4, EXPO>(w8, M1, G1, O1), acc[c]);
            }
        }
    }
}

// int2: word bits: code j at 2j, 16 codes.  Pairs (j, j+8) share an offset;
// offsets 0,2,4,6,8 fit the mantissa (magic 2^(10-o)); codes 5,6,7 / 13,14,15
// come down to offsets 0,2,4 after a shift by 10.  Staged states per packed row:
// {x_j, x_{j+8}} for j = 0..7.  off_k by k mod 8: 1024,256,64,16,4,1024,256,64.
template <bool EXPO = false>
__device__ __forceinline__ void unit_fast(const Unit<2, false>& u, const h16* xp, f32x4 acc[4]) {
    constexpr uint32_t O0 = off2(1024, 1024), O1 = off2(256, 256), O2 = off2(64, 64), O3 = off2(16, 16), O4 = off2(4, 4);
    const uint32_t M0 = in_vgpr(0x00030003u), M1 = in_vgpr(0x000C000Cu), M2 = in_vgpr(0x00300030u),
                   M3 = in_vgpr(0x00C000C0u), M4 = in_vgpr(0x03000300u);
    const uint32_t G0 = in_vgpr(0x64006400u), G1 = in_vgpr(0x5C005C00u), G2 = in_vgpr(0x54005400u),
                   G3 = in_vgpr(0x4C004C00u), G4 = in_vgpr(0x44004400u);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const u32x4 pa = *reinterpret_cast<const u32x4*>(xp + r * 16);
        const u32x4 pb = *reinterpret_cast<const u32x4*>(xp + r * 16 + 8);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w = u.w[r][c], w10 = w >> 10;
            acc[c] = mma4(pa.x, pa.y, operand<2, EXPO>(w, M0, G0, O0), operand<2, EXPO>(w, M1, G1, O1), acc[c]);
            acc[c] = mma4(pa.z, pa.w, operand<2, EXPO>(w, M2, G2, O2), operand<2, EXPO>(w, M3, G3, O3), acc[c]);
            acc[c] = mma4(pb.x, pb.y, operand<2, EXPO>(w, M4, G4, O4), operand<2, EXPO>(w10, M0, G0, O0), acc[c]);
            acc[c] = mma4(pb.z, pb.w, operand<2, EXPO>(w10, M1, G1, O1), operand<2, EXPO>(w10, M2, G2, O2), acc[c]);
        }
    }
}

// int3: every 32 codes of a column are a 96-bit stream over three words, code j
// at stream bit 3j.  A 32-bit window of the stream that starts at bit 3c-1 has
// codes c, c+1, c+2 at offsets 1, 4, 7 of its low half and codes c+5, c+6, c+7
// at offsets 0, 3, 6 of its high half: three mask-and-OR operations turn it into
// three half2 pairs.  Windows at c = 0, 8, 16, 24 (one shift or funnel shift
// each) cover 24 codes; the pairs (4,11), (12,19), (20,27) come from windows at
// bits 12, 36, 60 (offsets 0 and 5), codes 3 and 28 from plain shifts.  The
// states are staged in exactly this pair order, so 26 VALU operations and 9
// MFMAs process 32 weights.  I3_LO/I3_HI list the code index in the low / high
// half of pair p (-1: unused, its state is staged as zero); I3_OFF is the magic
// offset 2^e each code is read with.
__device__ constexpr int I3_LO[18] = {0, 1, 2, 8, 9, 10, 16, 17, 18, 24, 25, 26, 4, 12, 20, 3, 28, -1};
__device__ constexpr int I3_HI[18] = {5, 6, 7, 13, 14, 15, 21, 22, 23, 29, 30, 31, 11, 19, 27, -1, -1, -1};
__device__ constexpr float I3_OFF[32] = {512, 64, 8, 1024, 1024, 1024, 128, 16, 512, 64, 8, 32, 1024, 1024, 128, 16,
                                         512, 64, 8, 32, 1024, 1024, 128, 16, 512, 64, 8, 32, 1024, 1024, 128, 16};

template <bool EXPO = false>
__device__ __forceinline__ void unit_fast(const Unit<3, false>& u, const h16* xp, f32x4 acc[4]) {
    constexpr uint32_t OA1 = off2(512, 1024), OA2 = off2(64, 128), OA3 = off2(8, 16), OL = off2(1024, 32), OS = off2(1024, 1024);
    const uint32_t MA1 = in_vgpr(0x0007000Eu), GA1 = in_vgpr(0x64006000u);   // {512 + c, 1024 + c5}
    const uint32_t MA2 = in_vgpr(0x00380070u), GA2 = in_vgpr(0x58005400u);   // {64 + c1, 128 + c6}
    const uint32_t MA3 = in_vgpr(0x01C00380u), GA3 = in_vgpr(0x4C004800u);   // {8 + c2, 16 + c7}
    const uint32_t ML = in_vgpr(0x00E00007u), GL = in_vgpr(0x50006400u);     // {1024 + lo, 32 + hi}
    const uint32_t MS = in_vgpr(0x00000007u), GS = in_vgpr(0x64006400u);     // {1024 + lo, 1024}
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {
        const uint32_t* xw = reinterpret_cast<const uint32_t*>(xp) + hb * 20;
        const u32x4 p0 = *reinterpret_cast<const u32x4*>(xw), p1 = *reinterpret_cast<const u32x4*>(xw + 4),
                    p2 = *reinterpret_cast<const u32x4*>(xw + 8), p3 = *reinterpret_cast<const u32x4*>(xw + 12);
        const u32x2 p4 = *reinterpret_cast<const u32x2*>(xw + 16);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w0 = u.w[3 * hb][c], w1 = u.w[3 * hb + 1][c], w2 = u.w[3 * hb + 2][c];
            const uint32_t a0 = w0 << 1, a1 = __builtin_amdgcn_alignbit(w1, w0, 23),
                           a2 = __builtin_amdgcn_alignbit(w2, w1, 15), a3 = w2 >> 7;
            const uint32_t l0 = __builtin_amdgcn_alignbit(w1, w0, 12), l1 = __builtin_amdgcn_alignbit(w2, w1, 4),
                           l2 = __builtin_amdgcn_alignbit(w2, w1, 28);
            const uint32_t s3 = w0 >> 9, s28 = w2 >> 20;
            f32x4 r = acc[c];
            r = mma4(p0.x, p0.y, operand<3, EXPO>(a0, MA1, GA1, OA1), operand<3, EXPO>(a0, MA2, GA2, OA2), r);
            r = mma4(p0.z, p0.w, operand<3, EXPO>(a0, MA3, GA3, OA3), operand<3, EXPO>(a1, MA1, GA1, OA1), r);
            r = mma4(p1.x, p1.y, operand<3, EXPO>(a1, MA2, GA2, OA2), operand<3, EXPO>(a1, MA3, GA3, OA3), r);
            r = mma4(p1.z, p1.w, operand<3, EXPO>(a2, MA1, GA1, OA1), operand<3, EXPO>(a2, MA2, GA2, OA2), r);
            r = mma4(p2.x, p2.y, operand<3, EXPO>(a2, MA3, GA3, OA3), operand<3, EXPO>(a3, MA1, GA1, OA1), r);
            r = mma4(p2.z, p2.w, operand<3, EXPO>(a3, MA2, GA2, OA2), operand<3, EXPO>(a3, MA3, GA3, OA3), r);
            r = mma4(p3.x, p3.y, operand<3, EXPO>(l0, ML, GL, OL), operand<3, EXPO>(l1, ML, GL, OL), r);
            r = mma4(p3.z, p3.w, operand<3, EXPO>(l2, ML, GL, OL), operand<3, EXPO>(s3, MS, GS, OS), r);
            const uint32_t last = operand<3, EXPO>(s28, MS, GS, OS);
            r = mma4(p4.x, p4.y, last, last, r);          // second pair is unused: its states are zero
            acc[c] = r;
        }
    }
}

// byte selector of v_perm_b32(hi_src, lo_src, sel) that builds the half2 {state a, state b}
// from the natural-order dwords holding them; -1 selects zero
__host__ __device__ constexpr uint32_t pair_selector(int a, int b) {
    const uint32_t lo = a < 0 ? 0x0C0Cu : (uint32_t)(((a & 1) * 2 + 1) << 8 | ((a & 1) * 2));
    const uint32_t hi = b < 0 ? 0x0C0Cu : (uint32_t)((4 + (b & 1) * 2 + 1) << 8 | (4 + (b & 1) * 2));
    return hi << 16 | lo;
}

// 16:32 sparse int4.  Per (32-row block, column): a mask word and 16 kept codes
// packed in 64 bits.  Two dot products are needed per column: A = sum over kept
// rows of x*q and M = sum over kept rows of x (dropped rows contribute exactly 0).
// The kept codes are first expanded to their rows.  The mask is taken a byte at
// a time: the next eight nibbles of the code stream are split into eight bytes
// (even / odd nibbles of one word, each with bit 4 set as a "kept" flag), and a
// 256-entry table in LDS holds, for every mask byte, the four v_perm selectors
// that route the right byte (or zero) into the 16-bit halves of the pairs
// (row j, row j+4) of that byte's eight rows.  The halves {0x001q, 0x001q'} go to
// the MFMA as they are: as fp16 they are the denormals (16 + q) * 2^-24, which
// the matrix unit multiplies exactly (it does not flush them).  Masking the same
// halves with 0x0010 gives 16 * 2^-24 per kept row for the second dot product:
//     accA = 2^-24 (A + 16 M),   accM = 2^-20 M.
// The mask byte is first replicated into all four bytes of a register: its
// population count is then the stream's shift in bits (4 per kept code), and its
// bits 4..11 are the table offset (entries are stored under the nibble-swapped byte).
// Staged states per unit: for each block 16 dwords {x_j, x_j+4}, ordered as the
// dense int4 path.

// EXPO: the exponent quantisation of the same rows.  A kept row's half 0x001q becomes +-2^(q & 7) -- the code's low
// three bits added to the exponent field of 1.0 (the "kept" flag times 0x3C0 is fp16 1.0), its top bit the sign --
// and a dropped row's stays 0: accA = sum over kept rows of x * +-2^e, exactly; accM as before.
__device__ __forceinline__ uint32_t sparse_expo_halves(uint32_t h, uint32_t kept) {
    const uint32_t t = h << 10;
    const uint32_t magnitude = __umul24(kept, 0x3C0u) + (t & 0x1C001C00u);
    return ((t << 2) & 0x80008000u) | magnitude;
}
template <bool EXPO = false>
__device__ __forceinline__ void unit_fast_sparse(const Unit<4, true>& u, const h16* xp, const char* lut,
                                                 f32x4 accA[4], f32x4 accM[4]) {
    const uint32_t NIB = in_vgpr(0x0F0F0F0Fu), FLAG = in_vgpr(0x10101010u), KEPT = in_vgpr(0x00100010u);
    const uint32_t IDX = in_vgpr(0x00000FF0u);
    const uint32_t* xw = reinterpret_cast<const uint32_t*>(xp);
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t m = u.m[hb][c];
            uint64_t stream = (uint64_t)u.w[2 * hb][c] | ((uint64_t)u.w[2 * hb + 1][c] << 32);
            f32x4 ra = accA[c], rm = accM[c];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // ---- rows 8i .. 8i+7
                const uint32_t mb4 = __builtin_amdgcn_perm(m, m, 0x01010101u * i);      // mask byte i, four times
                const u32x4 sel = *reinterpret_cast<const u32x4*>(lut + (mb4 & IDX));
                const uint32_t chunk = (uint32_t)stream;
                const uint32_t even = and_or(chunk, NIB, FLAG), odd = and_or(chunk >> 4, NIB, FLAG);
                stream >>= __builtin_popcount(mb4);
                const u32x4 px = *reinterpret_cast<const u32x4*>(xw + hb * 16 + i * 4);
                uint32_t b0 = __builtin_amdgcn_perm(odd, even, sel.x);
                uint32_t b1 = __builtin_amdgcn_perm(odd, even, sel.y);
                uint32_t b2 = __builtin_amdgcn_perm(odd, even, sel.z);
                uint32_t b3 = __builtin_amdgcn_perm(odd, even, sel.w);
                const uint32_t k0 = b0 & KEPT, k1 = b1 & KEPT, k2 = b2 & KEPT, k3 = b3 & KEPT;
                if constexpr (EXPO) {
                    b0 = sparse_expo_halves(b0, k0); b1 = sparse_expo_halves(b1, k1);
                    b2 = sparse_expo_halves(b2, k2); b3 = sparse_expo_halves(b3, k3);
                }
                ra = mma4(px.x, px.y, b0, b1, ra);
                rm = mma4(px.x, px.y, k0, k1, rm);
                ra = mma4(px.z, px.w, b2, b3, ra);
                rm = mma4(px.z, px.w, k2, k3, rm);
            }
            accA[c] = ra;
            accM[c] = rm;
        }
    }
}
__device__ __forceinline__ void unit_fast(const Unit<4, true>&, const h16*, f32x4[4]) {}

template <int BITS>
__device__ __forceinline__ float fast_offset(int k) {      // magic offset of row k of a unit
    if constexpr (BITS == 4) return (k & 1) ? 64.f : 1024.f;
    const int j = k & 7;
    return (float)(1024 >> (2 * (j < 5 ? j : j - 5)));
}

// ---- general path: any format, either quantisation mode.  Deliberately compact
// (rolled loops, few registers): it serves the formats without a fast path and
// the rare exponent-mode columns.  The 32 codes of a block are consumed from a
// bit stream held in four registers.  States are read in natural order from
// global memory.  acc[c] = sum over kept k of x_k * value(q_k), xs[c] = sum over
// kept k of x_k.
template <int BITS, bool SPARSE>
__device__ __forceinline__ void unit_generic(const Unit<BITS, SPARSE>& u, const h16* __restrict__ xg,
                                             const bool expo[4], float acc[4], float xs[4]) {
    constexpr int WPB = SPARSE ? 2 : BITS;           // packed words per 32-row block
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        float ac = 0.f, xc = 0.f;
#pragma unroll
        for (int hb = 0; hb < 2; ++hb) {
            uint32_t s[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < WPB; ++i) s[i] = u.w[hb * WPB + i][c];
            uint32_t keep = 0xFFFFFFFFu;
            if constexpr (SPARSE) keep = u.m[hb][c];
#pragma unroll 2
            for (int t = 0; t < 32; ++t) {
                const uint32_t code = s[0] & ((1u << BITS) - 1u);
                const bool k = keep & 1u;
                keep >>= 1;
                const uint32_t sh = SPARSE ? (k ? 4u : 0u) : (uint32_t)BITS;
                s[0] = __builtin_amdgcn_alignbit(s[1], s[0], sh);
                s[1] = __builtin_amdgcn_alignbit(s[2], s[1], sh);
                s[2] = __builtin_amdgcn_alignbit(s[3], s[2], sh);
                s[3] >>= sh;
                const float xv = (float)xg[hb * 32 + t];
                const float val = code_value<BITS>(code, expo[c]);
                ac += k ? xv * val : 0.f;
                xc += k ? xv : 0.f;
            }
        }
        acc[c] = ac;
        xs[c] = xc;
    }
}

__device__ __forceinline__ void unpack_params(const u32x2 sc2, const u32x2 ze2, float sc[4], float ze[4],
                                              bool expo[4]) {
    const h16x2 s01 = as_h2(sc2.x), s23 = as_h2(sc2.y), z01 = as_h2(ze2.x), z23 = as_h2(ze2.y);
    sc[0] = (float)s01.x; sc[1] = (float)s01.y; sc[2] = (float)s23.x; sc[3] = (float)s23.y;
    ze[0] = (float)z01.x; ze[1] = (float)z01.y; ze[2] = (float)z23.x; ze[3] = (float)z23.y;
#pragma unroll
    for (int c = 0; c < 4; ++c) expo[c] = !(sc[c] >= 0.f);     // NaN takes the exponent branch
}

// sum over an aligned group of 4 / 8 lanes (valid in every lane of the group)
__device__ __forceinline__ float sum4(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    return v;
}
__device__ __forceinline__ float sum8(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    return v;
}

// ---- cross-workgroup hand-over.  A slot is 8 bytes {fp32 partial sum, flag};
// it is written with one device-scope (write-through) 64-bit store and read
// with device-scope loads, so no cache-wide fence is needed and a writer never
// waits.  flag == SLOT_FULL marks a slot as written; the reader clears it.
constexpr uint32_t SLOT_FULL = 0x600DF00Du;
constexpr int MV_SPIN_LIMIT = 1 << 22;            // polls before a reader gives up

__device__ __forceinline__ void slot_store(uint64_t* p, float v, uint32_t flag) {
    const uint64_t bits = (uint64_t)bitcast<uint32_t>(v) | ((uint64_t)flag << 32);
    __hip_atomic_store(p, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint64_t slot_load(const uint64_t* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// PF: keep the next unit's loads in flight while the current one is processed
// (more registers); without it a lane group loads and processes one unit at a
// time and relies on the other resident waves to cover the latency.
//
// NR = 2, 4: up to two / four rows of states in one pass over the weights (dense formats).  The 4x4x4 MFMA
// computes a 4 x 4 block per four lanes; with one row of states every lane passes the same four
// states as its row of A and three of the four result registers repeat the first.  Here lane
// 4b + i passes row i's states, and register i of a lane is row i's dot product for the lane's
// column: the same instructions and the same weight traffic give four rows of outputs (NR = 2:
// lanes 4b + i and 4b + i + 2 pass row i, two registers are used).  Staged states, unit sums, the
// reduction area and the hand-over slots (slot row = split * NR + row) are kept per row.
template <int BITS, bool SPARSE, int LK, bool PF, int NR = 1>
__global__ __launch_bounds__(MV_MAX_WAVES * WAVE)
void matvec_kernel(const uint32_t* pre_matrix, const h16* pre_scales, const h16* pre_zeros, const h16* pre_x, int pre_S,
                   int pre_units_per_wg, int pre_group_units, int pre_units_total, uint32_t pre_group_magic, MatvecArgs a) {
    // (the arguments that the first loads depend on, once more in front of the record: the first dwords of a kernel's
    // arguments can be handed to a wave in registers at its start, a record's fields are fetched by the wave itself)
    a.matrix = pre_matrix; a.scales = pre_scales; a.zeros = pre_zeros; a.x = pre_x; a.S = pre_S;
    a.units_per_wg = pre_units_per_wg; a.group_units = pre_group_units; a.units_total = pre_units_total; a.group_magic = pre_group_magic;
    constexpr bool FAST = Fmt<BITS, SPARSE>::FAST;
    static_assert(NR == 1 || ((NR == 2 || NR == 4) && FAST && !SPARSE), "several rows: dense formats only");
    constexpr int LC = WAVE / LK;                 // column lanes per lane group
    constexpr int COLS = LC * 4;                  // columns per strip

    // staged states (64 halves per unit) then per-unit {sum x, sum off*x}; the
    // same memory is reused for the final reduction
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // 16:32 only: the table of v_perm selectors per mask byte, statically allocated so that
    // its LDS address is a compile-time constant (a table read then needs no address add)
    __shared__ __attribute__((aligned(16))) u32x4 lut[SPARSE ? 256 : 1];
    h16* xs = reinterpret_cast<h16*>(smem);
    float* sums = reinterpret_cast<float*>(smem + (size_t)a.units_per_wg * NR * Fmt<BITS, SPARSE>::XS);
    float* red = reinterpret_cast<float*>(smem);

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, nwaves = blockDim.x >> 6;
    const int cl = lane % LC, kl = lane / LC;
    const int strip = blockIdx.x, split = blockIdx.y;
    const int col = strip * COLS + cl * 4;
    const bool col_ok = col < a.S;

    const int wg_u0 = split * a.units_per_wg;
    const int wg_u1 = min(wg_u0 + a.units_per_wg, a.units_total);
    const int ng = nwaves * LK, grp = wave * LK + kl;

    // ---- issue order matters: loads return in order, so the (small) loads of
    // the states go first and the weight loads follow; the staging below then
    // only waits for the states while the weights are still in flight.
    // A staging item is what one thread permutes: one packed row's worth of
    // states for int4 / int2 (8 / 16 halves), one 32-row cell for int3 and 16:32.
    constexpr int ITEM_H = SPARSE ? 32 : (BITS == 4 ? 8 : (BITS == 2 ? 16 : 32));   // halves per item
    constexpr int IPU = 64 / ITEM_H;                                  // items per unit
    constexpr int ITEM_V = ITEM_H / 8;                                // 16-byte loads per item
    // (NR rows: item r belongs to unit-row block r / IPU = unit * NR + row, whose staged states and sums
    // lie side by side; rows beyond a.rows are staged as zeros)
    const int nitems = FAST ? (wg_u1 - wg_u0) * IPU * NR : 0;
    const int nitems8 = (nitems + 7) & ~7;
    const h16* xg = a.x + wg_u0 * 64;
    u32x4 xv[ITEM_V];
#pragma unroll
    for (int i = 0; i < ITEM_V; ++i) xv[i] = u32x4{0, 0, 0, 0};
    auto load_x = [&](int r) {
        if (r < nitems) {
            if constexpr (NR == 1) {
#pragma unroll
                for (int i = 0; i < ITEM_V; ++i) xv[i] = *reinterpret_cast<const u32x4*>(xg + r * ITEM_H + i * 8);
            } else {
                const int block = r / IPU, row = block % NR, item = (block / NR) * IPU + r % IPU;
#pragma unroll
                for (int i = 0; i < ITEM_V; ++i)
                    xv[i] = row < a.rows ? *reinterpret_cast<const u32x4*>(xg + (int64_t)row * a.K + item * ITEM_H + i * 8)
                                         : u32x4{0, 0, 0, 0};
            }
        }
    };
    if constexpr (FAST) load_x(t);

    Unit<BITS, SPARSE> ua, ub;
    int u = wg_u0 + grp;
    const bool work = col_ok && u < wg_u1;
    const bool work_b = PF && work && u + ng < wg_u1;
    if (work) load_unit(ua, a, u, col);
    if constexpr (PF) {
        if (work_b) load_unit(ub, a, u + ng, col);
    }

    if constexpr (SPARSE) {
        // selector table: for mask byte b, pair j = (row j, row j+4): byte 0 picks the code of
        // row j from the pool {even nibbles, odd nibbles}, byte 2 that of row j+4; 0x0C yields 0
        for (int b = t; b < 256; b += blockDim.x) {
            uint32_t selb[8];
            int rank = 0;
#pragma unroll
            for (int p8 = 0; p8 < 8; ++p8) {
                const bool k = (b >> p8) & 1;
                selb[p8] = k ? (uint32_t)((rank & 1) * 4 + (rank >> 1)) : 0x0Cu;
                rank += k;
            }
            u32x4 e;
#pragma unroll
            for (int j = 0; j < 4; ++j) e[j] = selb[j] | (0x0Cu << 8) | (selb[j + 4] << 16) | (0x0Cu << 24);
            lut[((b & 15) << 4) | (b >> 4)] = e;                    // stored under the nibble-swapped byte
        }
    }
    if constexpr (FAST) {
        for (int r = t; r < nitems8; r += blockDim.x) {
            if (r != t) load_x(r);
            float s = 0.f, o = 0.f;
            if (r < nitems) {
                if constexpr (SPARSE) {                                            // one 32-row block
                    uint32_t d[16];                                                // d[j] = {x_2j, x_2j+1}
#pragma unroll
                    for (int i = 0; i < 4; ++i) { d[4 * i] = xv[i].x; d[4 * i + 1] = xv[i].y; d[4 * i + 2] = xv[i].z; d[4 * i + 3] = xv[i].w; }
                    uint32_t* dstA = reinterpret_cast<uint32_t*>(xs) + r * 16;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {                                  // rows 8i..8i+7: {x_j, x_j+4}
                        u32x4 p;
                        p.x = __builtin_amdgcn_perm(d[4 * i + 2], d[4 * i], 0x05040100u);
                        p.y = __builtin_amdgcn_perm(d[4 * i + 2], d[4 * i], 0x07060302u);
                        p.z = __builtin_amdgcn_perm(d[4 * i + 3], d[4 * i + 1], 0x05040100u);
                        p.w = __builtin_amdgcn_perm(d[4 * i + 3], d[4 * i + 1], 0x07060302u);
                        *reinterpret_cast<u32x4*>(dstA + 4 * i) = p;
                    }
                    // (no magic offsets in this format: the per-unit sums stay 0)
                } else if constexpr (BITS == 4) {
                    const u32x4 v = xv[0];                                         // x0x1 x2x3 x4x5 x6x7
                    u32x4 p;
                    p.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);            // {x0, x4}
                    p.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);            // {x1, x5}
                    p.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);            // {x2, x6}
                    p.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);            // {x3, x7}
                    *reinterpret_cast<u32x4*>(xs + r * 8) = p;
                    const float e = lo_f32(v.x) + lo_f32(v.y) + lo_f32(v.z) + lo_f32(v.w);
                    const float d = hi_f32(v.x) + hi_f32(v.y) + hi_f32(v.z) + hi_f32(v.w);
                    s = e + d;
                    o = 1024.f * e + 64.f * d;
                } else if constexpr (BITS == 2) {
                    const u32x4 va = xv[0], vb = xv[1];
                    u32x4 pa, pb;
                    pa.x = __builtin_amdgcn_perm(vb.x, va.x, 0x05040100u);         // {x0, x8}
                    pa.y = __builtin_amdgcn_perm(vb.x, va.x, 0x07060302u);         // {x1, x9}
                    pa.z = __builtin_amdgcn_perm(vb.y, va.y, 0x05040100u);
                    pa.w = __builtin_amdgcn_perm(vb.y, va.y, 0x07060302u);
                    pb.x = __builtin_amdgcn_perm(vb.z, va.z, 0x05040100u);
                    pb.y = __builtin_amdgcn_perm(vb.z, va.z, 0x07060302u);
                    pb.z = __builtin_amdgcn_perm(vb.w, va.w, 0x05040100u);
                    pb.w = __builtin_amdgcn_perm(vb.w, va.w, 0x07060302u);
                    *reinterpret_cast<u32x4*>(xs + r * 16) = pa;
                    *reinterpret_cast<u32x4*>(xs + r * 16 + 8) = pb;
                    const uint32_t w[8] = {va.x, va.y, va.z, va.w, vb.x, vb.y, vb.z, vb.w};
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float lo = lo_f32(w[j]), hi = hi_f32(w[j]);
                        s += lo + hi;
                        o += lo * fast_offset<2>(2 * j) + hi * fast_offset<2>(2 * j + 1);
                    }
                } else {                                                           // int3: one 32-row cell
                    uint32_t d[16];                                                // d[j] = {x_2j, x_2j+1}
#pragma unroll
                    for (int i = 0; i < 4; ++i) { d[4 * i] = xv[i].x; d[4 * i + 1] = xv[i].y; d[4 * i + 2] = xv[i].z; d[4 * i + 3] = xv[i].w; }
                    uint32_t q[20];
#pragma unroll
                    for (int k = 0; k < 18; ++k) {
                        const int lo = I3_LO[k], hi = I3_HI[k];
                        q[k] = __builtin_amdgcn_perm(d[hi < 0 ? 0 : hi / 2], d[lo < 0 ? 0 : lo / 2], pair_selector(lo, hi));
                    }
                    q[18] = q[19] = 0u;
                    uint32_t* dst = reinterpret_cast<uint32_t*>(xs) + r * 20;
#pragma unroll
                    for (int k = 0; k < 20; k += 4) *reinterpret_cast<u32x4*>(dst + k) = u32x4{q[k], q[k + 1], q[k + 2], q[k + 3]};
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const float lo = lo_f32(d[j]), hi = hi_f32(d[j]);
                        s += lo + hi;
                        o += lo * I3_OFF[2 * j] + hi * I3_OFF[2 * j + 1];
                    }
                }
            }
            // sum the items of a unit (aligned groups of IPU lanes)
            if constexpr (IPU == 8) { s = sum8(s); o = sum8(o); }
            else if constexpr (IPU == 4) { s = sum4(s); o = sum4(o); }
            else { s += dpp_f32<0xB1>(s); o += dpp_f32<0xB1>(o); }
            if ((r % IPU) == 0 && r < nitems) {    // first item of a unit publishes its sums
                sums[(r / IPU) * 2] = s;
                sums[(r / IPU) * 2 + 1] = o;
            }
        }
        __syncthreads();
    }

    float y[4] = {0.f, 0.f, 0.f, 0.f};
    float yr[NR == 1 ? 1 : 4][NR == 1 ? 1 : NR] = {};       // NR rows: yr[column][row] instead of y
    bool need_general = false;

    auto finish_unit = [&](const Unit<BITS, SPARSE>& un, int unit) {
        float sc[4], ze[4];
        bool expo[4];
        unpack_params(un.sc, un.ze, sc, ze, expo);
        if constexpr (FAST && SPARSE) {
            f32x4 accA[4], accM[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) { accA[c] = f32x4{0.f, 0.f, 0.f, 0.f}; accM[c] = f32x4{0.f, 0.f, 0.f, 0.f}; }
            const int lu = unit - wg_u0;
            unit_fast_sparse(un, xs + lu * (Fmt<BITS, SPARSE>::XS / 2), reinterpret_cast<const char*>(lut), accA, accM);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float sl = fmaxf(sc[c], 0.f);
                // A = 2^24 (accA - accM), M = 2^20 accM
                y[c] += sl * (16777216.f * (accA[c][0] - accM[c][0]) - ze[c] * (1048576.f * accM[c][0]));
                need_general |= expo[c];
            }
        } else if constexpr (FAST) {
            f32x4 acc[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
            const int lu = unit - wg_u0;
            if constexpr (NR == 1) {
                unit_fast(un, xs + lu * (Fmt<BITS, SPARSE>::XS / 2), acc);
                const float xsum = sums[lu * 2], xoff = sums[lu * 2 + 1];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    // exponent-mode columns (scale < 0 or NaN) contribute nothing here
                    const float sl = fmaxf(sc[c], 0.f);
                    y[c] += sl * ((acc[c][0] - xoff) - ze[c] * xsum);
                    need_general |= expo[c];
                }
            } else {
                unit_fast(un, xs + (lu * NR + (lane & (NR - 1))) * (Fmt<BITS, SPARSE>::XS / 2), acc);
                float xsum[NR], xoff[NR];
#pragma unroll
                for (int r = 0; r < NR; ++r) { xsum[r] = sums[(lu * NR + r) * 2]; xoff[r] = sums[(lu * NR + r) * 2 + 1]; }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float sl = fmaxf(sc[c], 0.f);
#pragma unroll
                    for (int r = 0; r < NR; ++r) yr[c][r] += sl * ((acc[c][r] - xoff[r]) - ze[c] * xsum[r]);
                    need_general |= expo[c];
                }
            }
        } else {
            float acc[4], xsv[4];
            unit_generic<BITS, SPARSE>(un, a.x + unit * 64, expo, acc, xsv);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float lin = sc[c] * (acc[c] - ze[c] * xsv[c]);
                const float ex = ze[c] * xsv[c] - sc[c] * acc[c];
                y[c] += expo[c] ? ex : lin;
            }
        }
    };

    if (work) {
        if constexpr (PF) {
            // ua and ub are both in flight on entry
            bool has_b = work_b;
            for (;;) {
                finish_unit(ua, u);
                if (!has_b) break;
                const int u2 = u + 2 * ng, u3 = u + 3 * ng;
                const bool has_a = u2 < wg_u1;
                if (has_a) load_unit(ua, a, u2, col);
                finish_unit(ub, u + ng);
                if (!has_a) break;
                has_b = u3 < wg_u1;
                if (has_b) load_unit(ub, a, u3, col);
                u = u2;
            }
        } else {
            for (;;) {
                finish_unit(ua, u);
                u += ng;
                if (u >= wg_u1) break;
                load_unit(ua, a, u, col);
            }
        }
    }

    if constexpr (FAST) {
        // exponent-mode columns: a second pass over the units that have any (the group's scales
        // are looked at first; most units are skipped).  Dense formats run the same operands
        // through the exponent decode -- no offsets to remove, y += z * sum(x) - s * sum(x * +-2^e);
        // 16:32 likewise, with the sum over the kept rows from its second accumulator.
        if (__builtin_amdgcn_ballot_w64(need_general) != 0 && work) {
            for (int v = wg_u0 + grp; v < wg_u1; v += ng) {
                const u32x2 sc2 = *reinterpret_cast<const u32x2*>(a.scales + (int64_t)magic_div(v, a.group_units, a.group_magic) * a.S + col);
                const h16x2 s01 = as_h2(sc2.x), s23 = as_h2(sc2.y);
                const bool any = !(s01.x >= (h16)0.f) | !(s01.y >= (h16)0.f) | !(s23.x >= (h16)0.f) | !(s23.y >= (h16)0.f);
                if (__builtin_amdgcn_ballot_w64(any) == 0) continue;
                load_unit(ua, a, v, col);
                float sc[4], ze[4];
                bool expo[4];
                unpack_params(ua.sc, ua.ze, sc, ze, expo);
                if constexpr (!SPARSE) {
                    f32x4 acc[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) acc[c] = f32x4{0.f, 0.f, 0.f, 0.f};
                    const int lu = v - wg_u0;
                    if constexpr (NR == 1) {
                        unit_fast<true>(ua, xs + lu * (Fmt<BITS, SPARSE>::XS / 2), acc);
                        const float xsum = sums[lu * 2];
#pragma unroll
                        for (int c = 0; c < 4; ++c) y[c] += expo[c] ? ze[c] * xsum - sc[c] * acc[c][0] : 0.f;
                    } else {
                        unit_fast<true>(ua, xs + (lu * NR + (lane & (NR - 1))) * (Fmt<BITS, SPARSE>::XS / 2), acc);
#pragma unroll
                        for (int r = 0; r < NR; ++r) {
                            const float xsum = sums[(lu * NR + r) * 2];
#pragma unroll
                            for (int c = 0; c < 4; ++c) yr[c][r] += expo[c] ? ze[c] * xsum - sc[c] * acc[c][r] : 0.f;
                        }
                    }
                } else {
                    // 16:32: the same expansion of the kept codes, their halves turned into +-2^e; M = 2^20 accM
                    f32x4 accA[4], accM[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) { accA[c] = f32x4{0.f, 0.f, 0.f, 0.f}; accM[c] = f32x4{0.f, 0.f, 0.f, 0.f}; }
                    unit_fast_sparse<true>(ua, xs + (v - wg_u0) * (Fmt<BITS, SPARSE>::XS / 2), reinterpret_cast<const char*>(lut), accA, accM);
#pragma unroll
                    for (int c = 0; c < 4; ++c) y[c] += expo[c] ? ze[c] * (1048576.f * accM[c][0]) - sc[c] * accA[c][0] : 0.f;
                }
            }
        }
    }

    if constexpr (NR > 1) {
        // ---- the same reduction and hand-over per row: a plane of the reduction area and a slot row per row
        __syncthreads();
        const int plane = (int)blockDim.x * 4;
#pragma unroll
        for (int r = 0; r < NR; ++r)
            *reinterpret_cast<f32x4*>(&red[r * plane + (wave * 64 + lane) * 4]) = f32x4{yr[0][r], yr[1][r], yr[2][r], yr[3][r]};
        __syncthreads();
        constexpr int MAXC = COLS / WAVE;
        const uint32_t poisoned = a.splits > 1 && split == a.splits - 1
                                      ? __hip_atomic_load(a.sticky, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
        for (int r = 0; r < a.rows; ++r) {
#pragma unroll
            for (int i = 0; i < MAXC; ++i) {
                const int j = t + i * (int)blockDim.x;
                const int ocol = strip * COLS + j;
                if (j >= COLS || ocol >= a.S) continue;
                float total = 0.f;
                for (int w = 0; w < nwaves; ++w)
#pragma unroll
                    for (int k = 0; k < LK; ++k) total += red[r * plane + (w * 64 + k * LC) * 4 + j];
                h16* const out = a.outs + (int64_t)r * a.S + ocol;
                const float prior = a.accumulate ? (float)*out : 0.f;
                if (a.splits == 1) {
                    *out = (h16)(prior + total);
                } else if (split != a.splits - 1) {
                    slot_store(&a.slots[((int64_t)split * NR + r) * a.S + ocol], total, SLOT_FULL);
                } else {
                    float sum = prior;
                    bool ok = poisoned == 0;
                    for (int sp = 0; sp < a.splits - 1; ++sp) {
                        uint64_t* p = &a.slots[((int64_t)sp * NR + r) * a.S + ocol];
                        uint64_t v = slot_load(p);
                        int spins = 0;
                        while ((uint32_t)(v >> 32) != SLOT_FULL && spins < a.spin_limit) {
                            __builtin_amdgcn_s_sleep(1);
                            v = slot_load(p);
                            ++spins;
                        }
                        ok &= (uint32_t)(v >> 32) == SLOT_FULL;
                        sum += bitcast<float>((uint32_t)v);
                        slot_store(p, 0.f, 0u);
                    }
                    sum += total;
                    if (!ok) __hip_atomic_store(a.sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    *out = ok ? (h16)sum : (h16)__builtin_nanf("");
                }
            }
        }
        return;
    }

    // ---- workgroup reduction through LDS (the staging area is free now)
    __syncthreads();
    *reinterpret_cast<f32x4*>(&red[(wave * 64 + lane) * 4]) = f32x4{y[0], y[1], y[2], y[3]};
    __syncthreads();
    // each thread finishes the columns j = t, t + blockDim.x, ... of the strip
    // (a workgroup may have fewer threads than the strip has columns)
    constexpr int MAXC = COLS / WAVE;                      // columns per thread with one wave
    float total[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
        const int j = t + i * (int)blockDim.x;
        total[i] = 0.f;
        if (j < COLS) {
            for (int w = 0; w < nwaves; ++w)
#pragma unroll
                for (int k = 0; k < LK; ++k) total[i] += red[(w * 64 + k * LC) * 4 + j];
        }
    }
    auto for_owned = [&](auto&& fn) {
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
            const int j = t + i * (int)blockDim.x;
            const int ocol = strip * COLS + j;
            if (j < COLS && ocol < a.S) fn(i, ocol);
        }
    };
    if (a.splits == 1) {
        for_owned([&](int i, int ocol) { a.outs[ocol] = (h16)((a.accumulate ? (float)a.outs[ocol] : 0.f) + total[i]); });
        return;
    }

    // ---- across workgroups.  Splits 0 .. n-2 publish their partial sums and
    // leave.  Split n-1 has the highest workgroup index of its strip, so by the
    // time it runs every other split has been dispatched: it waits for their
    // slots, adds them in a fixed order (deterministic), clears them for the
    // next call and writes the result.
    if (split != a.splits - 1) {
        for_owned([&](int i, int ocol) { slot_store(&a.slots[(int64_t)split * a.S + ocol], total[i], SLOT_FULL); });
        return;
    }
    // (a hand-over that timed out earlier may have left late slots behind: the workspace stays
    // poisoned -- every result NaN -- until the host zero-fills it again)
    const uint32_t poisoned = __hip_atomic_load(a.sticky, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for_owned([&](int i, int ocol) {
        float sum = a.accumulate ? (float)a.outs[ocol] : 0.f;
        bool ok = poisoned == 0;
        // slots are fetched eight at a time so that their latencies overlap; a
        // slot that is not full yet is polled again on its own
        for (int s0 = 0; s0 < a.splits - 1; s0 += 8) {
            uint64_t v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                v[k] = s0 + k < a.splits - 1 ? slot_load(&a.slots[(int64_t)(s0 + k) * a.S + ocol]) : 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                if (s0 + k >= a.splits - 1) break;
                uint64_t* p = &a.slots[(int64_t)(s0 + k) * a.S + ocol];
                int spins = 0;
                while ((uint32_t)(v[k] >> 32) != SLOT_FULL && spins < a.spin_limit) {
                    __builtin_amdgcn_s_sleep(1);
                    v[k] = slot_load(p);
                    ++spins;
                }
                ok &= (uint32_t)(v[k] >> 32) == SLOT_FULL;
                sum += bitcast<float>((uint32_t)v[k]);
                slot_store(p, 0.f, 0u);
            }
        }
        sum += total[i];
        // a slot that never arrived (which would mean a writer was never run) poisons the
        // output -- and the workspace, since the writer may still fill its slot later --
        // instead of hanging the wave
        if (!ok) __hip_atomic_store(a.sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        a.outs[ocol] = ok ? (h16)sum : (h16)__builtin_nanf("");
    });
}

// LDS of a launch: staged states + per-unit sums (per row), or the reduction area (4 floats per thread and row)
template <int BITS, bool SPARSE>
static size_t matvec_lds_bytes(int units_per_wg, int threads, int nr) {
    return std::max((size_t)units_per_wg * nr * (Fmt<BITS, SPARSE>::XS + 8), (size_t)threads * 16 * nr);
}

// up to four rows of states per pass (dense formats, no prefetch variant needed: the launcher passes its choice)
template <int BITS, int NR>
static void launch_rows(const MatvecArgs& a, int lk, bool pf, dim3 grid, dim3 block, hipStream_t st) {
    const size_t lds = matvec_lds_bytes<BITS, false>(a.units_per_wg, (int)block.x, NR);
#define I4_LAUNCH(LK_, PF_) hipLaunchKernelGGL((matvec_kernel<BITS, false, LK_, PF_, NR>), grid, block, lds, st, a.matrix, a.scales, a.zeros, a.x, a.S, a.units_per_wg, a.group_units, a.units_total, a.group_magic, a)
    if (lk == 1) { if (pf) I4_LAUNCH(1, true); else I4_LAUNCH(1, false); }
    else if (lk == 2) { if (pf) I4_LAUNCH(2, true); else I4_LAUNCH(2, false); }
    else { if (pf) I4_LAUNCH(4, true); else I4_LAUNCH(4, false); }
#undef I4_LAUNCH
}

template <int BITS, bool SPARSE>
static void launch(const MatvecArgs& a, int lk, bool pf, dim3 grid, dim3 block, hipStream_t st) {
    const size_t lds = matvec_lds_bytes<BITS, SPARSE>(a.units_per_wg, (int)block.x, 1);
#define I4_LAUNCH(LK_, PF_) hipLaunchKernelGGL((matvec_kernel<BITS, SPARSE, LK_, PF_>), grid, block, lds, st, a.matrix, a.scales, a.zeros, a.x, a.S, a.units_per_wg, a.group_units, a.units_total, a.group_magic, a)
    if (lk == 1) { if (pf) I4_LAUNCH(1, true); else I4_LAUNCH(1, false); }
    else if (lk == 2) { if (pf) I4_LAUNCH(2, true); else I4_LAUNCH(2, false); }
    else { if (pf) I4_LAUNCH(4, true); else I4_LAUNCH(4, false); }
#undef I4_LAUNCH
}

}  // namespace i4

using namespace i4;

// Launch shape of a matvec: strips of 256 / lk columns, `waves` waves per workgroup, `upwg` units per
// workgroup dealt round-robin to its lane groups; the grid's y dimension (`splits`) covers the rest of K.
struct MatvecShape { int lk, waves, upwg, splits, strips; };
static MatvecShape plan_matvec(int64_t S, int units_total) {
    // Launch shape: strips of 256/lk columns, `waves` waves per workgroup, `upwg`
    // units per workgroup dealt round-robin to its lane groups; the grid's y
    // dimension covers the rest of K.
    // Defaults (measured on MI355X): the narrowest lane-group split that still
    // gives about 160 strips, about 640 workgroups in all (2.5 per CU, all
    // resident at once), 4 waves each.
    int lk = (int)tuning(TUNE_MV_LK), waves = (int)tuning(TUNE_MV_WAVES), upwg = (int)tuning(TUNE_MV_UNITS);
    if (lk != 1 && lk != 2 && lk != 4) {
        lk = 1;
        while (lk < 4 && (S + 256 / lk - 1) / (256 / lk) < 160) lk *= 2;
    }
    const int cols = 256 / lk;
    const int strips = (int)((S + cols - 1) / cols);
    if (waves <= 0) waves = 4;
    if (waves > MV_MAX_WAVES) waves = MV_MAX_WAVES;
    if (upwg <= 0) {
        int want_splits = (640 + strips / 2) / strips;
        if (want_splits < 1) want_splits = 1;
        upwg = (units_total + want_splits - 1) / want_splits;
        if (upwg < 4) upwg = 4;
    }
    if (upwg > units_total) upwg = units_total;
    // The workgroup of a strip's last split sums the strip up once the others have handed
    // their partial sums over.  With equal shares it finishes its own units last (it is
    // dispatched last) and only then starts on the reduction and the hand-over, after the
    // streaming has ended; with about half a share it is through both while the others still
    // stream, and the launch ends with them.  So the other splits take U / (splits - 1/2) units
    // each and the last one the rest (measured on MI355X: 3 - 9 % faster for every format at
    // S = 8192 ... 28672 with 3 - 5 splits) -- unless that costs the lane groups of a launch
    // without prefetch another round.  With more splits the idle share of the last one is
    // missed in the streaming instead (K = 11008, S = 4096, 10 splits: 8 % slower), so they
    // keep equal shares.
    if (tuning(TUNE_MV_UNITS) <= 0) {
        const int s0 = (units_total + upwg - 1) / upwg;
        if (s0 >= 2 && s0 <= 5) {
            const int ng = waves * lk;
            const int w = (2 * units_total + (2 * s0 - 1) - 1) / (2 * s0 - 1);        // ceil(U / (s0 - 1/2))
            const bool prefetching = w >= 3 * ng;
            const bool same_rounds = (w + ng - 1) / ng == (upwg + ng - 1) / ng;
            if (w > upwg && w <= MV_MAX_UNITS_WG && units_total - (s0 - 1) * w >= 1 &&
                (units_total + w - 1) / w == s0 && (prefetching || same_rounds))
                upwg = w;
        }
    }
    int splits = (units_total + upwg - 1) / upwg;
    if (splits > MV_MAX_SPLITS) {                           // bounded slot count: more units each
        upwg = (units_total + MV_MAX_SPLITS - 1) / MV_MAX_SPLITS;
        splits = (units_total + upwg - 1) / upwg;
    }
    if (waves * lk > upwg) waves = (upwg + lk - 1) / lk;    // no idle waves
    return MatvecShape{lk, waves, upwg, splits, strips};
}

// Two to four rows of states (a matmul with that many rows in all, or a matvec with that many batch
// elements), dense formats: the matvec kernel with a row per MFMA result register -- one pass over the
// weights at the matvec's rate.  Returns false when it does not take the shape (the few-row kernels do then):
// the hand-over needs four slot rows per split, the staged states four times the LDS.
bool i4::matvec_rows(int bits, h16* outs, const uint32_t* matrix, const h16* x, const h16* scales, const h16* zeros,
                     int64_t R, int64_t K, int64_t S, int64_t group_size, bool accumulate, hipStream_t st,
                     void* workspace, size_t workspace_bytes) {
    if (R < 2 || R > 4 || K % 64 != 0 || S % 4 != 0) return false;
    // measured against the few-row kernel (S = 11008 ... 32768, warm weights): 10 - 26 % faster up to K = 5120
    // (K=5120, S=20480: 2 / 3 / 4 rows 14.0 / 15.4 / 17.1 against 18.4 / 18.1 / 18.3 us; K=4096, S=11008: 9.5 / 11.1 /
    // 12.3 against 11.3 / 12.5 / 12.4), 3 - 14 % slower from K = 6144 on, where staging four rows of states per
    // workgroup weighs more; below K = 4096 only two rows gain.  Two rows (NR = 2) gain on a longer K as well
    // while K is split at most five ways (K=8192, S=22016: 21.0 against 26.0 us; K=28672, S=8192: 26.6 against
    // 33.3; ten splits, K=14336, S=4096: 15.5 against 13.3)
    // Narrow outputs lose (two rows against the few-row kernel, us: K=4096, S=2048 15.1 / 9.5; K=S=4096 11.7 / 9.4;
    // K=5120, S=6144 11.1 / 10.4; from S = 8192 on 9.3 - 10.0 / 9.6 - 10.6 and better; three and four rows: S = 6144
    // 13 - 16 / 10, S = 8192 12 - 14 / 10, S = 11008 11.5 - 13.5 / 12.8 - 14.7), and at exactly 16384 columns the
    // few-row kernel has one workgroup on every CU and wins for three and four rows (12.0 - 13.8 / 11.5 - 12.7)
    if (S < 8192) return false;
    // (... and up to 16384 columns altogether since the few-row kernel takes such outputs in one round of 64-column
    // strips: K=4096, S=14336, three / four rows 11.4 / 12.6 against 10.3 us)
    if (R > 2 && S <= 16384) return false;
    if (R > 2 && (K > 5120 || K < 4096)) return false;
    const int units_total = (int)(K / 64);
    const MatvecShape ms = plan_matvec(S, units_total);
    const int nr = R <= 2 ? 2 : 4;
    if (ms.splits * nr > MV_MAX_SPLITS || ms.upwg * nr > MV_MAX_UNITS_WG) return false;
    if (R == 2 && K > 5120 && ms.splits > 5) return false;
    const WorkspaceParts ws = workspace_parts(workspace, workspace_bytes);
    if (ms.splits > 1 && ws.slots_bytes < matvec_slots_bytes(S)) return false;
    const bool pf = ms.upwg >= 3 * ms.waves * ms.lk && tuning(TUNE_MV_NOPF) == 0;
    MatvecArgs a;
    a.outs = outs;
    a.matrix = matrix;
    a.mask = nullptr;
    a.x = x;
    a.scales = scales;
    a.zeros = zeros;
    a.slots = (uint64_t*)workspace;
    a.K = (int)K;
    a.S = (int)S;
    a.units_total = units_total;
    a.units_per_wg = ms.upwg;
    a.group_units = (int)(group_size / 64 > 0x7FFFFFF ? 0x7FFFFFF : group_size / 64);
    a.group_magic = div_magic((uint32_t)a.group_units);
    a.splits = ms.splits;
    a.sticky = ms.splits > 1 ? reinterpret_cast<uint32_t*>(ws.counters - 8) : nullptr;
    a.spin_limit = tuning(TUNE_MV_SPIN) > 0 ? (int)tuning(TUNE_MV_SPIN) : MV_SPIN_LIMIT;
    a.rows = (int)R;
    a.accumulate = accumulate ? 1 : 0;
    const dim3 grid(ms.strips, ms.splits, 1), block(ms.waves * WAVE);
    if (noting("matvec_kernel<bits=%d,dense,lane_groups=%d,prefetch=%d,rows=%d> strips=%d splits=%d waves=%d units_per_workgroup=%d rows=%d",
               bits, ms.lk, (int)pf, nr, ms.strips, ms.splits, ms.waves, ms.upwg, (int)R))
        return true;
    if (nr == 2) {
        if (bits == 4) launch_rows<4, 2>(a, ms.lk, pf, grid, block, st);
        else if (bits == 3) launch_rows<3, 2>(a, ms.lk, pf, grid, block, st);
        else launch_rows<2, 2>(a, ms.lk, pf, grid, block, st);
    } else {
        if (bits == 4) launch_rows<4, 4>(a, ms.lk, pf, grid, block, st);
        else if (bits == 3) launch_rows<3, 4>(a, ms.lk, pf, grid, block, st);
        else launch_rows<2, 4>(a, ms.lk, pf, grid, block, st);
    }
    return true;
}

static int matvec_plain(int bits, void* outs, const void* matrix, const void* multiplier, const void* scales, const void* zeros,
                        const void* sparse_mask, int64_t B, int64_t K, int64_t S, int64_t g, bool accumulate, void* workspace,
                        size_t workspace_bytes, hipStream_t st);

// A single row through the matmul entry (which overwrites outs): the matvec kernel serves it at the matvec's
// rate, where a tile kernel would spend a 128-row tile on it (K=5120, S=20480: 79 -> 12 us; K=28672, S=8192:
// 407 -> 27 us).  False when the matvec cannot take the shape with the workspace at hand.
bool i4::matvec_one_row(int bits, h16* outs, const uint32_t* matrix, const uint32_t* sparse_mask, const h16* x, const h16* scales,
                        const h16* zeros, int64_t K, int64_t S, int64_t group_size, hipStream_t st, void* workspace,
                        size_t workspace_bytes, int* rc) {
    if (K % 64 != 0 || S % 4 != 0) return false;
    if (K / 64 > (int64_t)MV_MAX_SPLITS * MV_MAX_UNITS_WG) return false;        // (several launches: the tile kernels take it)
    const MatvecShape ms = plan_matvec(S, (int)(K / 64));
    if (ms.upwg > MV_MAX_UNITS_WG) return false;
    if (ms.splits > 1 && workspace_parts(workspace, workspace_bytes).slots_bytes < matvec_slots_bytes(S)) return false;
    *rc = matvec_plain(bits, outs, matrix, x, scales, zeros, sparse_mask, 1, K, S, group_size, false, workspace, workspace_bytes, st);
    return true;
}

static int matvec_impl(int bits, void* outs, const void* matrix, const void* multiplier,
                       const void* scales, const void* zeros, const void* sparse_mask,
                       const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                       void* stream) {
    int rc = validate_product(bits, outs, matrix, multiplier, scales, zeros, sparse_mask, shape, true);
    if (rc != INT4MM_OK) return rc;
    const int64_t B = shape->batch, K = shape->in_size, S = shape->out_size;
    if (B * shape->seq_len * S == 0) return INT4MM_OK;
    // the documented rule, whichever launch shape the product takes: a workspace of int4mm_workspace_bytes(S)
    if (workspace_parts(workspace, workspace_bytes).slots_bytes < matvec_slots_bytes(S)) return INT4MM_ERR_WORKSPACE;

    const int64_t g = shape->group_size < 0 ? ONE_GROUP : shape->group_size;

    // several batch elements of one row each: one pass over the weights for all of them
    if (B >= 2 && B <= 4 && !sparse_mask && !tuning(TUNE_NO_SKINNY) &&
        matvec_rows(bits, (h16*)outs, (const uint32_t*)matrix, (const h16*)multiplier, (const h16*)scales, (const h16*)zeros,
                    B, K, S, g, true, (hipStream_t)stream, workspace, workspace_bytes))
        return check_launch("matvec");
    if (B >= 2 && B <= SK_WIDE_MAX_ROWS && !tuning(TUNE_NO_SKINNY) &&
        skinny_rows(bits, (h16*)outs, (const uint32_t*)matrix, (const h16*)multiplier, (const h16*)scales,
                    (const h16*)zeros, B, K, S, g, true, (hipStream_t)stream, (const uint32_t*)sparse_mask, workspace, workspace_bytes))
        return check_launch("matvec");

    // more batch elements than the few-row kernels take at once: chunks of up to 512 through them (they add onto outs
    // as the matvec does; 1 100 elements at K=4096, S=4096: three launches instead of 1 100), the plain kernel for what
    // they do not take
    int64_t done = 0;
    if (B > SK_WIDE_MAX_ROWS && !tuning(TUNE_NO_SKINNY)) {
        while (B - done >= 2) {
            const int64_t n = std::min<int64_t>(SK_WIDE_MAX_ROWS, B - done);
            if (!skinny_rows(bits, (h16*)outs + done * S, (const uint32_t*)matrix, (const h16*)multiplier + done * K, (const h16*)scales,
                             (const h16*)zeros, n, K, S, g, true, (hipStream_t)stream, (const uint32_t*)sparse_mask, workspace,
                             workspace_bytes))
                break;
            rc = check_launch("matvec");
            if (rc != INT4MM_OK) return rc;
            done += n;
        }
        if (done == B) return INT4MM_OK;
    }
    return matvec_plain(bits, (h16*)outs + done * S, matrix, (const h16*)multiplier + done * K, scales, zeros, sparse_mask, B - done, K, S, g,
                        true, workspace, workspace_bytes, (hipStream_t)stream);
}

// One launch of the single-row kernel per batch row; `accumulate`: add onto outs (the matvec entry) or
// overwrite it (a single row through the matmul entry).  A launch stages its share of the states in LDS and
// cuts K at most MV_MAX_SPLITS ways, so it covers MV_MAX_SPLITS x MV_MAX_UNITS_WG units of K; a longer K (the
// reference's grid covers any: matvec_kernel.cu:339-347) goes in ranges of that many units, each a whole
// number of quantisation groups, the later ones adding onto the result of the earlier.
static int matvec_plain(int bits, void* outs, const void* matrix, const void* multiplier, const void* scales, const void* zeros,
                        const void* sparse_mask, int64_t B, int64_t K, int64_t S, int64_t g, bool accumulate, void* workspace,
                        size_t workspace_bytes, hipStream_t st) {
    const int64_t units_all = K / 64;
    const int64_t gu = g / 64 > 0x7FFFFFF ? 0x7FFFFFF : g / 64;               // units per quantisation group
    int64_t range_units = (int64_t)MV_MAX_SPLITS * MV_MAX_UNITS_WG;
    if (units_all > range_units) {
        if (gu > range_units && gu < units_all) return INT4MM_ERR_SHAPE;        // (a group longer than a launch covers)
        if (gu <= range_units) range_units = range_units / gu * gu;
    }
    for (int64_t u0 = 0; u0 < units_all; u0 += range_units) {
        const int units_total = (int)std::min(range_units, units_all - u0);
        const MatvecShape ms = plan_matvec(S, units_total);
        const int lk = ms.lk, waves = ms.waves, upwg = ms.upwg, splits = ms.splits, strips = ms.strips;
        if (upwg > MV_MAX_UNITS_WG) return INT4MM_ERR_SHAPE;
        if (splits > 1 && workspace_parts(workspace, workspace_bytes).slots_bytes < matvec_slots_bytes(S))
            return INT4MM_ERR_WORKSPACE;
        // software prefetch only pays when lane groups walk several units
        const bool pf = upwg >= 3 * waves * lk && tuning(TUNE_MV_NOPF) == 0;

        MatvecArgs a;
        // the range's first packed row, mask row and group row (u0 is a multiple of the group size, or 0)
        a.matrix = (const uint32_t*)matrix + (sparse_mask ? u0 * 4 : u0 * 2 * bits) * S;
        a.mask = sparse_mask ? (const uint32_t*)sparse_mask + u0 * 2 * S : nullptr;
        a.scales = (const h16*)scales + (u0 / gu) * S;
        a.zeros = (const h16*)zeros + (u0 / gu) * S;
        a.slots = (uint64_t*)workspace;
        a.K = units_total * 64;
        a.S = (int)S;
        a.units_total = units_total;
        a.units_per_wg = upwg;
        a.group_units = (int)gu;
        a.group_magic = div_magic((uint32_t)a.group_units);
        a.splits = splits;
        a.sticky = splits > 1 ? reinterpret_cast<uint32_t*>(workspace_parts(workspace, workspace_bytes).counters - 8) : nullptr;
        a.spin_limit = tuning(TUNE_MV_SPIN) > 0 ? (int)tuning(TUNE_MV_SPIN) : MV_SPIN_LIMIT;
        a.rows = 1;
        a.accumulate = (accumulate || u0 > 0) ? 1 : 0;

        const dim3 grid(strips, splits, 1), block(waves * WAVE);
        if (noting("matvec_kernel<bits=%d,%s,lane_groups=%d,prefetch=%d> strips=%d splits=%d waves=%d units_per_workgroup=%d batch=%d",
                   bits, sparse_mask ? "16:32" : "dense", lk, (int)pf, strips, splits, waves, upwg, (int)B))
            continue;
        for (int64_t b = 0; b < B; ++b) {                      // one pass over the weights per batch row
            a.outs = (h16*)outs + b * S;
            a.x = (const h16*)multiplier + b * K + u0 * 64;
            if (sparse_mask) launch<4, true>(a, lk, pf, grid, block, st);
            else if (bits == 4) launch<4, false>(a, lk, pf, grid, block, st);
            else if (bits == 3) launch<3, false>(a, lk, pf, grid, block, st);
            else launch<2, false>(a, lk, pf, grid, block, st);
            const int rc = check_launch("matvec");
            if (rc != INT4MM_OK) return rc;
        }
    }
    return INT4MM_OK;
}

extern "C" int int4mm_matvec(int bits, void* outs, const void* matrix, const void* multiplier,
                             const void* scales, const void* zeros, const void* sparse_mask,
                             const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                             void* stream) {
    return matvec_impl(bits, outs, matrix, multiplier, scales, zeros, sparse_mask, shape, workspace, workspace_bytes, stream);
}

// ---- the same product for callers that cannot allocate.  The hand-over slots and split-K
// partials live in a file-scope device array instead of a caller's workspace.  Every device has
// its own copy of the array at its own address, resolved once per device (with that device
// current) and used from then on; host code never passes the array's name to a kernel.
namespace i4 {
constexpr int64_t STATIC_MAX_OUT_SIZE = 32768;
// == int4mm_workspace_bytes(STATIC_MAX_OUT_SIZE): slots for 32 K splits x 32768 columns, the counter
// page, and as much again as scratch for partial tiles
constexpr size_t STATIC_SCRATCH_BYTES = 2 * (4096 + (size_t)STATIC_MAX_OUT_SIZE * 8 * 32 + 4096);
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];   // zero at load; calls leave it zeroed where it must be
constexpr int STATIC_MAX_DEVICES = 64;
static void* g_scratch_ptr[STATIC_MAX_DEVICES];
static std::mutex g_scratch_mu;
}  // namespace i4

// The calling thread's current device's copy of the built-in array (resolved on first use); false if the
// runtime cannot name it.
bool i4::static_scratch(void** ptr, size_t* bytes) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_MAX_DEVICES) return false;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {                        // first call on this device
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) {
            (void)hipGetLastError();
            return false;
        }
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    *bytes = STATIC_SCRATCH_BYTES;
    return true;
}

extern "C" int int4mm_matvec_static(int bits, void* outs, const void* matrix, const void* multiplier,
                                    const void* scales, const void* zeros, const void* sparse_mask,
                                    const int4mm_shape* shape, void* stream) {
    if (shape == nullptr) return INT4MM_ERR_NULL;
    if (shape->out_size > STATIC_MAX_OUT_SIZE) return INT4MM_ERR_WORKSPACE;     // beyond the built-in scratch
    void* ptr;
    size_t bytes;
    if (!static_scratch(&ptr, &bytes)) return INT4MM_ERR_LAUNCH;
    return matvec_impl(bits, outs, matrix, multiplier, scales, zeros, sparse_mask, shape, ptr, bytes, stream);
}
