// Quantized matrix-matrix product for gfx950:
//     outs[m, s] = fp16( sum_k fp32(x[m, k]) * fp32(w16[k, s]) )
// where w16 is the fp16 matrix the reference's unpack step builds (two fp16
// roundings per weight in linear mode, one fused multiply-add in exponent mode).
//
// Two kernels.  matmul_kernel_pipe (further down) is the fast one for shapes
// made of whole tiles; matmul_kernel takes everything else.  Common to both: one
// workgroup owns a tile of outs; per K step the packed weights of the tile are
// read from HBM once, decoded and dequantised to fp16 ONCE by the workgroup and
// stored to LDS in the operand layout of v_mfma_f32_32x32x16_f16: 16-byte chunks
// of 8 consecutive k for one column, chunk (kc, n) at kc*BN + n, which both the
// writes (lanes along n) and the MFMA operand reads (lanes along n) touch
// without bank conflicts.  The states tile is stored row-major with an XOR
// swizzle of the chunk index so that row-contiguous writes and column-of-rows
// operand reads are both conflict-free.  Accumulation is fp32 in the MFMA
// accumulators.
//
// matmul_kernel walks K in steps of 64 with the global loads of step k+1 issued
// before the MFMA phase of step k (register prefetch) and two barriers per step.
//
// Workgroups are renumbered so that the 8 XCDs (each with its own L2) take
// disjoint column ranges of the weight matrix.
#include "common.h"

#include <algorithm>
#include <cmath>
#include <type_traits>

namespace i4 {

constexpr int BK = 64;

// swizzle of the 16-byte chunk index inside a 128-byte row of the states tile
__device__ __forceinline__ int a_swz(int m) { return (m & 7) ^ ((m >> 3) & 1); }

struct MatmulArgs {
    h16* outs;
    const uint32_t* matrix;
    const uint32_t* mask;
    const h16* x;
    const h16* scales;
    const h16* zeros;
    int M, K, S;
    int group_units;        // group size / 64
    int tiles_m, tiles_n;
    int by_columns;         // pipelined kernel: 1 = an XCD walks its range of tile columns row by row
    // split-K (pipelined kernel, grids that would leave most of the GPU idle): `ksplit` workgroups
    // share a tile, each walks 1 / ksplit of the K steps and stores its fp32 partial tile to
    // `part`; the one that arrives last (`counters`, one per tile) adds them up in split order
    int ksplit;
    float* part;
    int* counters;
    // tiles (in grid order) before `split_from` are not split: a grid whose last round would fill
    // at most half of the GPU splits only the tiles of that round
    int split_from;
};

// Raw packed data of one (32-row block, column) cell
template <int BITS, bool SPARSE>
struct Cell {
    uint32_t w[SPARSE ? 2 : BITS];
    uint32_t m;
};

template <int BITS, bool SPARSE>
__device__ __forceinline__ void load_cell(Cell<BITS, SPARSE>& c, const MatmulArgs& a, int blk, int col) {
    constexpr int ROWS = SPARSE ? 2 : BITS;
    const int64_t S = a.S;
    const uint32_t* p = a.matrix + (int64_t)blk * ROWS * S + col;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) c.w[r] = p[r * S];
    c.m = SPARSE ? a.mask[(int64_t)blk * S + col] : 0xFFFFFFFFu;
}

// General cell decode: 32 fp16 weights = 4 chunks of 8, bit-exact with the
// reference decode, any format and either quantisation mode.
template <int BITS, bool SPARSE>
__device__ __forceinline__ void dequant_cell_generic(const Cell<BITS, SPARSE>& c, h16 sc, h16 ze, h16x8 out[4]) {
    uint32_t codes[32];
    if constexpr (SPARSE) {
        uint64_t v = (uint64_t)c.w[0] | ((uint64_t)c.w[1] << 32);
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            const bool k = (c.m >> t) & 1u;
            codes[t] = (uint32_t)v & 0xFu;
            v >>= k ? 4 : 0;
        }
    } else if constexpr (BITS == 3) {
        const uint64_t lo = (uint64_t)c.w[0] | ((uint64_t)c.w[1] << 32);
        const uint64_t hi = (uint64_t)c.w[1] | ((uint64_t)c.w[2] << 32);
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            const int pos = 3 * t;
            codes[t] = pos + 3 <= 64 ? (uint32_t)(lo >> pos) & 7u : (uint32_t)(hi >> (pos - 32)) & 7u;
        }
    } else {
        constexpr int PER = 32 / BITS;
#pragma unroll
        for (int i = 0; i < BITS; ++i) {
            uint32_t v = c.w[i];
#pragma unroll
            for (int j = 0; j < PER; ++j) { codes[i * PER + j] = v & ((1u << BITS) - 1u); v >>= BITS; }
        }
    }
#pragma unroll
    for (int t = 0; t < 32; ++t) {
        h16 w = dequant_code<BITS>(codes[t], sc, ze);
        if (SPARSE && !((c.m >> t) & 1u)) w = (h16)0.0f;
        out[t >> 3][t & 7] = w;
    }
}

// Fast linear-mode decode of one dense int4 word into 8 fp16 weights in natural
// k order, bit-exact: the word's low (high) two bytes are replicated into both
// halves of a register, so that mask-and-OR yields the half2 {1024 + q_even,
// 64 + q_odd}; subtracting {1024, 64} is exact, then the reference's own two
// roundings follow: fp16(q - z), fp16(. * s).
// (mask / magic constants are held in registers, in_vgpr, so that v_and_or_b32 is selected)

__device__ __forceinline__ h16x8 dequant_word_int4(uint32_t u, h16x2 negz, h16x2 s2) {
    const uint32_t MSK = in_vgpr(0x00F0000Fu), MAGIC = in_vgpr(0x54006400u);
    const h16x2 unmagic = {(h16)-1024.0f, (h16)-64.0f};
    const uint32_t lo = __builtin_amdgcn_perm(u, u, 0x01000100u);    // bytes B0 B1 B0 B1
    const uint32_t hi = __builtin_amdgcn_perm(u, u, 0x03020302u);    // bytes B2 B3 B2 B3
    const uint32_t h[4] = {(lo & MSK) | MAGIC, ((lo >> 8) & MSK) | MAGIC,
                           (hi & MSK) | MAGIC, ((hi >> 8) & MSK) | MAGIC};
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        h16x2 q = as_h2(h[i]) + unmagic;       // exact: {q_even, q_odd}
        h16x2 d = q + negz;                    // fp16 subtract, one rounding
        r[i] = as_u32(d * s2);                 // fp16 multiply, one rounding
    }
    return bitcast<h16x8>(r);
}

template <int BITS, bool SPARSE>
__device__ __forceinline__ void dequant_cell(const Cell<BITS, SPARSE>& c, h16 sc, h16 ze, h16x8 out[4]) {
    if constexpr (BITS == 4 && !SPARSE) {
        if (sc >= (h16)0.0f) {
            const h16x2 negz = {-ze, -ze}, s2 = {sc, sc};
#pragma unroll
            for (int i = 0; i < 4; ++i) out[i] = dequant_word_int4(c.w[i], negz, s2);
            return;
        }
    }
    dequant_cell_generic<BITS, SPARSE>(c, sc, ze, out);
}

// T threads; thread t owns column t % BN of the weight tile and CPT of its
// (2 * BN / T) 32-row cells per K step.
template <int BITS, bool SPARSE, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64, 2) void matmul_kernel(MatmulArgs a) {
    constexpr int WAVES_N = BN / WN, WAVES_M = BM / WM;
    constexpr int T = WAVES_M * WAVES_N * 64;
    constexpr int TM = WM / 32, TN = WN / 32;     // MFMA tiles per wave
    constexpr int A_CHUNKS = BM * 8 / T;          // 16-byte chunks of the states tile per thread
    constexpr int CPT = 2 * BN / T;               // weight cells per thread
    static_assert(BM * 8 % T == 0 && (T == BN || T == 2 * BN), "tile/thread mismatch");
    static_assert(CPT == 1 || CPT == 2, "one or two cells per thread");

    __shared__ __attribute__((aligned(16))) h16 As[BM * BK];
    __shared__ __attribute__((aligned(16))) h16 Bs[BK * BN];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

    // XCD-aware renumbering: workgroup i runs on XCD i % 8; give each XCD a
    // contiguous range of column tiles and walk the row tiles fastest.
    int bid = blockIdx.x;
    const int total = a.tiles_m * a.tiles_n;
    {
        const int per_xcd = (total + 7) / 8;
        const int xcd = bid % 8, local = bid / 8;
        const int renum = xcd * per_xcd + local;
        if (total % 8 == 0) bid = renum;
    }
    const int tile_m = bid % a.tiles_m, tile_n = bid / a.tiles_m;
    const int m0 = tile_m * BM, s0 = tile_n * BN;
    const int64_t boff = blockIdx.z;
    const h16* x = a.x + boff * a.M * (int64_t)a.K;
    h16* outs = a.outs + boff * a.M * (int64_t)a.S;

    const int bn = t % BN, bhb0 = (t / BN) * CPT;
    const int bcol = min(s0 + bn, a.S - 1);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    u32x4 areg[A_CHUNKS];
    Cell<BITS, SPARSE> cell[CPT];
    h16 sc, ze;

    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = t + T * i, m = c >> 3, kc = c & 7;
            const int row = min(m0 + m, a.M - 1);
            areg[i] = *reinterpret_cast<const u32x4*>(x + (int64_t)row * a.K + kt * BK + kc * 8);
        }
#pragma unroll
        for (int q = 0; q < CPT; ++q) load_cell<BITS, SPARSE>(cell[q], a, kt * 2 + bhb0 + q, bcol);
        const int64_t gofs = (int64_t)(kt / a.group_units) * a.S + bcol;
        sc = a.scales[gofs];
        ze = a.zeros[gofs];
    };

    const int ktiles = a.K / BK;
    load_tile(0);
    for (int kt = 0; kt < ktiles; ++kt) {
        // registers -> LDS
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = t + T * i, m = c >> 3, kc = c & 7;
            *reinterpret_cast<u32x4*>(&As[m * BK + ((kc ^ a_swz(m)) << 3)]) = areg[i];
        }
#pragma unroll
        for (int q = 0; q < CPT; ++q) {
            h16x8 w[4];
            dequant_cell<BITS, SPARSE>(cell[q], sc, ze, w);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                *reinterpret_cast<h16x8*>(&Bs[(((bhb0 + q) * 4 + e) * BN + bn) * 8]) = w[e];
        }
        __syncthreads();
        if (kt + 1 < ktiles) load_tile(kt + 1);

#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const int kc = 2 * ks + (lane >> 5);
            h16x8 af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = wm0 + i * 32 + (lane & 31);
                af[i] = *reinterpret_cast<const h16x8*>(&As[m * BK + ((kc ^ a_swz(m)) << 3)]);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = wn0 + j * 32 + (lane & 31);
                bf[j] = *reinterpret_cast<const h16x8*>(&Bs[(kc * BN + n) * 8]);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: accumulator register r of lane l is row 8*(r/4) + 4*(l/32) + r%4,
    // column l%32 of its 32x32 tile
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = s0 + wn0 + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < a.M && col < a.S) outs[(int64_t)row * a.S + col] = (h16)acc[i][j][r];
            }
        }
}

// ---- pipelined variant for dense int4: (TM * 64) x (NW * 64) tile, 2 x NW waves
// of (TM * 32) x 64, K steps of 32, three LDS stages of each operand.  With
// NW = 2 (256 x 128 tile, 72 KB of LDS, four waves) two workgroups share a CU
// and fill each other's barrier and latency bubbles.
//  * states go global -> registers three steps ahead and are stored to the LDS
//    stage of step k+2 during step k;
//  * packed weights go global -> registers four steps ahead and are decoded
//    into the LDS stage of step k+2 one word at a time between the MFMAs of
//    step k, so VALU, LDS and the matrix core overlap inside a wave;
//  * MFMA operand fragments are fetched one 16-wide k slice ahead, ACROSS step
//    boundaries: everything a step reads was complete one barrier earlier, so
//    the barrier that closes a step orders buffer reuse only and the MFMA
//    stream never drains while waves wait for each other.
// The steady-state loop body has no branches; a tile that contains exponent-mode
// groups takes a second pipelined loop whose decode serves either mode (dense formats, 256-column
// tiles) or a plain two-stage loop with that decode (the others).
constexpr int PK = 32;            // K per step of the pipelined kernel

// One 16-byte chunk = 8 consecutive k of one column; `bits` holds its 8 codes, LSB first, BITS bits apart (bits
// above 8 * BITS are ignored).  Linear-mode fast decode of such a chunk, bit-exact.  The two codes of a pair
// are brought to the low bits of the two halves of a register; mask-and-OR with
// a magic exponent turns them into {2^a + q_even, 2^b + q_odd}, whose offsets
// are then subtracted exactly before the reference's two roundings.
template <int BITS>
__device__ __forceinline__ h16x8 dequant_chunk_fast(uint32_t bits, h16x2 negz, h16x2 s2) {
    if constexpr (BITS == 4) {
        return dequant_word_int4(bits, negz, s2);
    } else {
        // int2: pair j = bits 4j .. 4j+3 of the 16 code bits, replicated into both halves:
        //       low half keeps bits 0-1 (ulp 1 at 2^10), high half bits 2-3 (ulp 1/4 at 2^8).
        // int3: pair j = bits 6j .. 6j+5: low half bits 0-2 (2^10), high half bits 3-5 (ulp 1/8 at 2^7).
        constexpr uint32_t MSK = BITS == 2 ? 0x000C0003u : 0x00380007u;
        constexpr uint32_t MAGIC = BITS == 2 ? 0x5C006400u : 0x58006400u;
        const h16x2 unmagic = {(h16)-1024.0f, BITS == 2 ? (h16)-256.0f : (h16)-128.0f};
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t u = bits >> (2 * BITS * j);
            const uint32_t v = __builtin_amdgcn_perm(u, u, 0x01000100u);     // low 16 bits in both halves
            h16x2 q = as_h2((v & MSK) | MAGIC) + unmagic;      // exact: {q_even, q_odd}
            h16x2 d = q + negz;                                // fp16 subtract, one rounding
            r[j] = as_u32(d * s2);                             // fp16 multiply, one rounding
        }
        return bitcast<h16x8>(r);
    }
}

// Either mode, chosen per thread (a thread decodes one column, and the mode belongs to a
// (group, column)), without a branch: bit-exact with dequant_code in both.  Shared tail
//     A = P + N (one rounding),  w = fma(A, B, C) (one rounding)
// linear:   P = q, N = -z, B = s, C = -0:  fp16(q - z), then fp16(. * s) -- adding -0 changes nothing
// exponent: P = +-2^e, N = -0, B = -s, C = z:  the reference's single-rounded fma (matmul.cuh:127-136)
// +-2^e comes from the pair's magic-number word {2^a | q_even, 2^b | q_odd << BITS}: a packed
// 16-bit multiply moves both codes to bits 10.. of their halves (the magic bits leave through the
// top), the low BITS - 1 bits are the exponent field's increment over 15, the top bit is the sign.
template <int BITS>
__device__ __forceinline__ h16x2 expo_pair(uint32_t h) {
    return as_h2(expo_operand<BITS>(h, off2(1024u, 1u << (10 - BITS))));
}

template <int BITS>
__device__ __forceinline__ h16x8 dequant_chunk_mixed(uint32_t bits, bool expo, h16x2 negz, h16x2 s2) {
    const h16x2 minus0 = as_h2(0x80008000u);
    const h16x2 N = expo ? minus0 : negz, B = expo ? -s2 : s2, C = expo ? -negz : minus0;
    uint32_t h[4];
    h16x2 unmagic;
    if constexpr (BITS == 4) {
        const uint32_t MSK = in_vgpr(0x00F0000Fu), MAGIC = in_vgpr(0x54006400u);
        unmagic = h16x2{(h16)-1024.0f, (h16)-64.0f};
        const uint32_t lo = __builtin_amdgcn_perm(bits, bits, 0x01000100u);
        const uint32_t hi = __builtin_amdgcn_perm(bits, bits, 0x03020302u);
        h[0] = (lo & MSK) | MAGIC; h[1] = ((lo >> 8) & MSK) | MAGIC;
        h[2] = (hi & MSK) | MAGIC; h[3] = ((hi >> 8) & MSK) | MAGIC;
    } else {
        constexpr uint32_t MSK = BITS == 2 ? 0x000C0003u : 0x00380007u;
        constexpr uint32_t MAGIC = BITS == 2 ? 0x5C006400u : 0x58006400u;
        unmagic = h16x2{(h16)-1024.0f, BITS == 2 ? (h16)-256.0f : (h16)-128.0f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t u = bits >> (2 * BITS * j);
            h[j] = (__builtin_amdgcn_perm(u, u, 0x01000100u) & MSK) | MAGIC;
        }
    }
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const h16x2 q = as_h2(h[j]) + unmagic;             // exact: {q_even, q_odd}
        const h16x2 P = expo ? expo_pair<BITS>(h[j]) : q;
        const h16x2 A = P + N;
        r[j] = as_u32(__builtin_elementwise_fma(A, B, C));
    }
    return bitcast<h16x8>(r);
}

// 16:32 sparse int4.  `v` holds the (up to 8) kept codes of one 8-row chunk as
// consecutive nibbles, `m8` the chunk's mask bits.  A 256-entry table in LDS
// (8 words per mask byte: four words of per-half keep masks, two v_perm
// selectors) spreads the kept codes to their rows: the even / odd nibbles are
// separated into bytes, v_perm picks for every row the byte of its rank, a
// second v_perm widens byte pairs to {0x6400 | q, 0x6400 | q'}.  Dropped rows
// are cleared at the end, so they are exactly zero.
constexpr int SPARSE_LUT_WORDS = 256 * 8;

__device__ __forceinline__ void sparse_lut_entry(uint32_t e, uint32_t out[8]) {
    uint32_t sel[2] = {0, 0}, hm[4] = {0, 0, 0, 0};
    uint32_t rank = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const bool kept = (e >> i) & 1u;
        const uint32_t byte = kept ? ((rank & 1u) ? 4u + (rank >> 1) : (rank >> 1)) : 0x0Cu;
        sel[i >> 2] |= byte << (8 * (i & 3));
        if (kept) { hm[i >> 1] |= 0xFFFFu << (16 * (i & 1)); ++rank; }
    }
    out[0] = hm[0]; out[1] = hm[1]; out[2] = hm[2]; out[3] = hm[3];
    out[4] = sel[0]; out[5] = sel[1]; out[6] = 0; out[7] = 0;
}

__device__ __forceinline__ h16x8 dequant_chunk_sparse_fast(uint32_t v, uint32_t m8, const uint32_t* lut,
                                                           h16x2 negz, h16x2 s2) {
    const u32x4 keep = *reinterpret_cast<const u32x4*>(lut + m8 * 8);
    const u32x2 sel = *reinterpret_cast<const u32x2*>(lut + m8 * 8 + 4);
    const uint32_t even = v & 0x0F0F0F0Fu, odd = (v >> 4) & 0x0F0F0F0Fu;
    const uint32_t c03 = __builtin_amdgcn_perm(odd, even, sel.x);       // codes of rows 0..3, one per byte
    const uint32_t c47 = __builtin_amdgcn_perm(odd, even, sel.y);
    const uint32_t MAGIC = 0x64006400u;
    const uint32_t h[4] = {__builtin_amdgcn_perm(c03, MAGIC, 0x01050104u), __builtin_amdgcn_perm(c03, MAGIC, 0x01070106u),
                           __builtin_amdgcn_perm(c47, MAGIC, 0x01050104u), __builtin_amdgcn_perm(c47, MAGIC, 0x01070106u)};
    const h16x2 unmagic = {(h16)-1024.0f, (h16)-1024.0f};
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        h16x2 q = as_h2(h[i]) + unmagic;       // exact
        h16x2 d = q + negz;                    // fp16 subtract, one rounding
        r[i] = as_u32(d * s2) & keep[i];       // fp16 multiply, one rounding; dropped rows -> +0
    }
    return bitcast<h16x8>(r);
}

// Either mode per thread without a branch (see dequant_chunk_mixed): the rows' codes ride on 1024 in both halves of
// a pair, so the packed multiply that moves them to bits 10.. is by 1024 for both.
__device__ __forceinline__ h16x8 dequant_chunk_sparse_mixed(uint32_t v, uint32_t m8, const uint32_t* lut, bool expo,
                                                            h16x2 negz, h16x2 s2) {
    const u32x4 keep = *reinterpret_cast<const u32x4*>(lut + m8 * 8);
    const u32x2 sel = *reinterpret_cast<const u32x2*>(lut + m8 * 8 + 4);
    const uint32_t even = v & 0x0F0F0F0Fu, odd = (v >> 4) & 0x0F0F0F0Fu;
    const uint32_t c03 = __builtin_amdgcn_perm(odd, even, sel.x);
    const uint32_t c47 = __builtin_amdgcn_perm(odd, even, sel.y);
    const uint32_t MAGIC = 0x64006400u;
    const uint32_t h[4] = {__builtin_amdgcn_perm(c03, MAGIC, 0x01050104u), __builtin_amdgcn_perm(c03, MAGIC, 0x01070106u),
                           __builtin_amdgcn_perm(c47, MAGIC, 0x01050104u), __builtin_amdgcn_perm(c47, MAGIC, 0x01070106u)};
    const h16x2 unmagic = {(h16)-1024.0f, (h16)-1024.0f}, minus0 = as_h2(0x80008000u);
    const h16x2 N = expo ? minus0 : negz, B = expo ? -s2 : s2, C = expo ? -negz : minus0;
    u32x4 r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const h16x2 q = as_h2(h[i]) + unmagic;             // exact
        const h16x2 P = expo ? as_h2(expo_operand<4>(h[i], off2(1024u, 1024u))) : q;
        r[i] = as_u32(__builtin_elementwise_fma(P + N, B, C)) & keep[i];      // dropped rows -> +0
    }
    return bitcast<h16x8>(r);
}


// Per-format constants of the pipelined kernel: packed rows per 32-row block and
// the number of packed words a thread loads per K step for its two chunks.
template <int BITS, bool SPARSE> struct PipeFmt;
template <> struct PipeFmt<4, false> { static constexpr int ROWS = 4, NWORDS = 2; };
template <> struct PipeFmt<3, false> { static constexpr int ROWS = 3, NWORDS = 2; };
template <> struct PipeFmt<2, false> { static constexpr int ROWS = 2, NWORDS = 1; };
template <> struct PipeFmt<4, true> { static constexpr int ROWS = 2, NWORDS = 2; };

constexpr int P_STAGES = 3;

// PING: the waves of the first half ("compute first") run a step as its 16 MFMAs back to back
// and then everything else; the waves of the second half run everything else first and the MFMAs
// last.  A SIMD holds one wave of each kind, so its matrix pipe is fed by one wave at a time while
// the other loads, decodes and stores -- instead of both competing for it and the younger one
// finishing the step alone.
template <int BITS, bool SPARSE, int TM, int NW, bool PING, bool SPLIT>
__device__ __forceinline__ void pipe_tile(const MatmulArgs& a, const int m0, const int s0, const h16* x,
                                          h16* outs, h16* As, h16* Bs, uint32_t* lut, const int tile, const int split,
                                          const int nsplit) {
    constexpr int BM = TM * 64, BN = NW * 64, WM = TM * 32, WN = 64, TN = 2, T = 2 * NW * 64;
    constexpr int A_STAGE = BM * PK, B_STAGE = PK * BN;            // halves per stage
    constexpr int A_ROWS = T / 4;                                  // rows covered by one 16-byte load per thread
    constexpr int A_LOADS = BM / A_ROWS;                           // such loads per thread and step

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / NW) * WM, wn0 = (wave % NW) * WN;

    // states stage: row m at m * 64 bytes, 16-byte chunk c of the row stored at
    // c ^ ((m >> 2) & 3): sixteen consecutive rows read the same logical chunk
    // from sixteen different bank groups.  Thread t moves chunk t % 4 of rows
    // t / 4 + A_ROWS * i through registers (rows >= M re-read row M - 1 and are
    // dropped at the store).  The tile's columns lie inside the matrix
    // (launcher's duty).
    struct AStage { u32x4 v[A_LOADS]; };
    const int a_row = t >> 2, a_chunk = t & 3;
    // every global address is a buffer resource (the tile's rows of states; the whole
    // of the packed matrix, mask, scales, zeros) plus a per-lane 32-bit byte offset that
    // never changes plus a workgroup-uniform 32-bit offset that moves with the K step:
    // buffer loads add the three themselves, no address arithmetic is left to the VALU
    // (the launcher admits only shapes whose tensors stay below 4 GB)
    constexpr int RSRC_FLAGS = 0x00020000;               // raw buffer, 32-bit data format
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<h16*>(x + (int64_t)m0 * a.K), 0, min(a.M - m0, BM) * a.K * 2, RSRC_FLAGS);
    uint32_t a_off[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
        a_off[i] = (uint32_t)((min(a_row + A_ROWS * i, a.M - 1 - m0) * a.K + a_chunk * 8) * 2);
    const int a_dst = a_row * PK + ((a_chunk ^ ((a_row >> 2) & 3)) << 3);       // halves; rows + A_ROWS: same swizzle
    auto load_a = [&](AStage& r, uint32_t step_off) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) r.v[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_off[i], step_off, 0);
    };
    auto write_a = [&](const AStage& r, int stage) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            *reinterpret_cast<u32x4*>(&As[stage * A_STAGE + i * A_ROWS * PK + a_dst]) = r.v[i];
    };

    // weights: thread owns column bn and packed rows 2 bhb, 2 bhb + 1 of every K step.
    // scale / zero travel as the aligned 32-bit word that holds the column's half
    // (sub-dword loads make the compiler wait for every outstanding load); `half_sel`
    // replicates the wanted half into both lanes of a packed register.
    // Thread (bn, bhb) decodes rows 16 bhb .. 16 bhb + 15 of the step's 32-row block:
    // int4 words 2 bhb, 2 bhb + 1; int2 word bhb; int3 words bhb, bhb + 1 (bits
    // 48 bhb .. 48 bhb + 47 of the block's 96-bit stream); 16:32 sparse: both words
    // and the mask word of the block.
    using F = PipeFmt<BITS, SPARSE>;
    constexpr int NWORDS = F::NWORDS;
    const int bn = t % BN, bhb = t / BN;
    const int bcol = s0 + bn;
    struct Stage { uint32_t w[NWORDS]; uint32_t m; uint32_t sc, ze; };
    const uint32_t half_sel = (bcol & 1) ? 0x03020302u : 0x01000100u;
    uint32_t b_off[NWORDS];
#pragma unroll
    for (int i = 0; i < NWORDS; ++i)
        b_off[i] = (uint32_t)((((SPARSE ? 0 : BITS == 4 ? 2 * bhb : bhb) + i) * a.S + bcol) * 4);
    const uint32_t m_off = (uint32_t)(bcol * 4);
    const uint32_t m_step = 4u * a.S;                    // bytes of one row of mask words
    const uint32_t sz_off = (uint32_t)((bcol & ~1) * 2);
    const uint32_t b_step = (uint32_t)(F::ROWS * 4) * a.S;   // bytes of packed weights per K step
    const uint32_t g_step = 2u * a.S;                    // bytes of one row of scales / zeros
    const int k_blocks = a.K / PK, n_groups = (k_blocks + a.group_units * 2 - 1) / (a.group_units * 2);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(a.matrix), 0, (int)(k_blocks * b_step), RSRC_FLAGS);
    const __amdgpu_buffer_rsrc_t m_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint32_t*>(SPARSE ? a.mask : a.matrix), 0, (int)(k_blocks * m_step), RSRC_FLAGS);
    const __amdgpu_buffer_rsrc_t sc_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<h16*>(a.scales), 0, (int)(n_groups * g_step), RSRC_FLAGS);
    const __amdgpu_buffer_rsrc_t ze_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<h16*>(a.zeros), 0, (int)(n_groups * g_step), RSRC_FLAGS);
    // cursor over K steps: byte offsets of the step's packed-weight rows, mask row and scale / zero row
    struct Cursor { uint32_t w, m, sz; int kt, left; };
    auto cursor_at = [&](int kt) {
        const int gu = a.group_units * 2, group = kt / gu;
        return Cursor{kt * b_step, SPARSE ? kt * m_step : 0u, group * g_step, kt, gu - kt % gu};
    };
    auto load_b = [&](Stage& s, const Cursor& c) {
#pragma unroll
        for (int i = 0; i < NWORDS; ++i) s.w[i] = __builtin_amdgcn_raw_buffer_load_b32(w_rsrc, b_off[i], c.w, 0);
        if constexpr (SPARSE) s.m = __builtin_amdgcn_raw_buffer_load_b32(m_rsrc, m_off, c.m, 0);
        s.sc = __builtin_amdgcn_raw_buffer_load_b32(sc_rsrc, sz_off, c.sz, 0);
        s.ze = __builtin_amdgcn_raw_buffer_load_b32(ze_rsrc, sz_off, c.sz, 0);
    };
    auto stage_scale = [&](const Stage& s) { return as_h2(__builtin_amdgcn_perm(s.sc, s.sc, half_sel)); };
    auto stage_negzero = [&](const Stage& s) {
        return as_h2(__builtin_amdgcn_perm(s.ze, s.ze, half_sel) ^ 0x80008000u);
    };
    // the 8 codes of the thread's chunk q (rows 16 bhb + 8 q .. + 7), LSB first
    const int i3_shift = 16 * bhb;
    auto chunk_bits = [&](const Stage& s, int q) -> uint32_t {
        if constexpr (BITS == 4) return s.w[q];
        else if constexpr (BITS == 2) return q ? s.w[0] >> 16 : s.w[0];
        else return (uint32_t)((((uint64_t)s.w[1] << 32) | s.w[0]) >> (i3_shift + 24 * q));
    };
    // 16:32 sparse: mask bits of chunk q and its kept codes as consecutive nibbles.
    // The codes of rows before the chunk are skipped by a right shift of 4 bits
    // each (done in two halves: the total can reach 64).
    auto sparse_chunk = [&](const Stage& s, int q, uint32_t& v, uint32_t& m8) {
        const uint32_t m16 = (s.m >> (16 * bhb)) & 0xFFFFu;
        uint32_t skip = bhb ? __builtin_popcount(s.m & 0xFFFFu) : 0;
        if (q) skip += __builtin_popcount(m16 & 0xFFu);
        m8 = (m16 >> (8 * q)) & 0xFFu;
        const uint64_t st = ((uint64_t)s.w[1] << 32) | s.w[0];
        v = (uint32_t)((st >> (2 * skip)) >> (2 * skip));
    };
    auto write_b_fast = [&](const Stage& s, int stage, int q) {
        h16x8 w;
        if constexpr (SPARSE) {
            uint32_t v, m8;
            sparse_chunk(s, q, v, m8);
            w = dequant_chunk_sparse_fast(v, m8, lut, stage_negzero(s), stage_scale(s));
        } else {
            w = dequant_chunk_fast<BITS>(chunk_bits(s, q), stage_negzero(s), stage_scale(s));
        }
        *reinterpret_cast<h16x8*>(&Bs[stage * B_STAGE + ((bhb * 2 + q) * BN + bn) * 8]) = w;
    };
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // fragment addresses (halves, inside a stage); k slice ks selects chunk 2 ks + lane / 32
    int a_frag[TM], b_frag[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a_frag[i] = (wm0 + i * 32 + (lane & 31)) * PK;
#pragma unroll
    for (int j = 0; j < TN; ++j) b_frag[j] = (wn0 + j * 32 + (lane & 31)) * 8;
    const int a_sw = (lane >> 2) & 3;                 // row offsets are multiples of 32: same swizzle
    auto load_frags = [&](int stage, int ks, h16x8 fa[TM], h16x8 fb[TN]) {
        const int kc = 2 * ks + (lane >> 5);
#pragma unroll
        for (int i = 0; i < TM; ++i)
            fa[i] = *reinterpret_cast<const h16x8*>(&As[stage * A_STAGE + a_frag[i] + ((kc ^ a_sw) << 3)]);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[j] = *reinterpret_cast<const h16x8*>(&Bs[stage * B_STAGE + kc * BN * 8 + b_frag[j]]);
    };
    auto mfma_slice = [&](const h16x8 fa[TM], const h16x8 fb[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    };

    // K steps kt0 .. last of the matrix belong to this workgroup (all of them unless SPLIT)
    const int ksteps = a.K / PK;
    const int per_split = SPLIT ? (ksteps + nsplit - 1) / nsplit : ksteps;
    const int kt0 = SPLIT ? split * per_split : 0;
    const int ktiles = SPLIT ? min(ksteps, kt0 + per_split) - kt0 : ksteps;
    const int last = kt0 + ktiles - 1;

    // Cursors of the loads: weights run four K steps ahead of the MFMAs, states
    // three; both stop at the last step (the surplus loads re-read it, unused).
    Cursor cur = cursor_at(kt0);
    // (selects instead of branches: a branch here would split the scheduling
    // region of the step and invite the compiler to reuse the previous step's
    // scale / zero registers, which makes the step wait for its newest loads)
    // (plain integer arithmetic on purpose: conditions kept as booleans come out as
    // 64-bit lane-mask operations, several scalar instructions each)
    const int gu2 = a.group_units * 2;
    auto advance = [&]() {
        const int more = min(last - cur.kt, 1);                  // 1 until the last step is reached
        const int wrap = cur.left == 1 ? more : 0;
        cur.kt += more;
        cur.w += more * b_step;
        if constexpr (SPARSE) cur.m += more * m_step;
        cur.sz += wrap * g_step;
        cur.left += wrap * gu2 - more;
    };
    uint32_t a_cur = (uint32_t)kt0 * (PK * 2);
    int a_kt = kt0;
    auto advance_a = [&]() {
        const int more = min(last - a_kt, 1);
        a_kt += more;
        a_cur += more * (PK * 2);
    };
    Stage r[3];
    AStage ra[2];
    // the first two steps' operands are requested before the look at the scales below, whose
    // round trip to memory they then share
    load_a(ra[0], a_cur); advance_a();
    load_a(ra[1], a_cur); advance_a();
    load_b(r[0], cur); advance();
    load_b(r[1], cur); advance();

    // Does any (group, column) of this tile use exponent quantisation (scale < 0
    // or NaN)?  One pass over the tile's scales (a few KB); the answer is
    // workgroup-uniform and selects between the pipelined loop, whose decode is
    // the branch-free linear one, and the loops that also serve exponent groups.
    int& any_expo = *reinterpret_cast<int*>(Bs);          // borrowed before the pipeline starts
    __syncthreads();
    if constexpr (SPARSE) {
        if (t < 256) {
            uint32_t e[8];
            sparse_lut_entry(t, e);
            *reinterpret_cast<u32x4*>(lut + t * 8) = u32x4{e[0], e[1], e[2], e[3]};
            *reinterpret_cast<u32x4*>(lut + t * 8 + 4) = u32x4{e[4], e[5], e[6], e[7]};
        }
    }
    if (t == 0) any_expo = 0;
    __syncthreads();
    {
        // the tile's scales are `groups` rows of BN / 2 aligned 32-bit words; the threads share them
        // out and fetch four words each per trip, all in flight together (one round trip to
        // memory instead of one per group)
        bool bad = false;
        const int groups = (ksteps + a.group_units * 2 - 1) / (a.group_units * 2);
        const int total = groups * (BN / 2);
        const uint32_t* tile_scales = reinterpret_cast<const uint32_t*>(a.scales + s0);
        const int64_t row_words = a.S / 2;
        for (int i0 = t; i0 < total; i0 += 4 * T) {
            uint32_t v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int i = min(i0 + k * T, total - 1);
                v[k] = tile_scales[(int64_t)(i / (BN / 2)) * row_words + i % (BN / 2)];
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const h16x2 h = as_h2(v[k]);
                bad |= !(h.x >= (h16)0.0f) | !(h.y >= (h16)0.0f);
            }
        }
        if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0) any_expo = 1;
    }
    __syncthreads();
    const bool tile_has_expo = any_expo != 0;
    __syncthreads();

    if (!tile_has_expo) {
        h16x8 fa[2][TM], fb[2][TN];         // fragments of the current and the next k slice
        // Step kt, u = kt % 6, stage b = kt % 3.  On entry: states and decoded weights
        // of steps kt, kt+1 are complete in stages b, b+1; ra[kt % 2] holds the states
        // and r[(kt+2) % 3] the packed weights of step kt+2, which this step moves
        // into stage b+2; the fragments of slice (kt, 0) are in fa[0] / fb[0].  The
        // step loads states kt+3 and weights kt+4 into the register sets it does not use.
        auto body = [&](int b, AStage& ra_new, const AStage& ra_wr, Stage& r_new, const Stage& r_dec) {
            const int b1 = (b + 1) % P_STAGES, b2 = (b + 2) % P_STAGES;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                if (ks == 0) load_frags(b, 1, fa[1], fb[1]);
                else load_frags(b1, 0, fa[0], fb[0]);
                if (ks == 0) {
                    load_a(ra_new, a_cur);             // step kt + 3
                    load_b(r_new, cur);                // step kt + 4
                    advance_a();
                    advance();
                }
                if (ks == 0) { write_b_fast(r_dec, b2, 0); write_b_fast(r_dec, b2, 1); }
                if (ks == 1) write_a(ra_wr, b2);
                mfma_slice(fa[ks], fb[ks]);
                // scheduling template.  First slice: the next slice's fragment reads, then
                // every MFMA followed by decode instructions of both of the thread's chunks
                // (and one of this step's global loads), the two LDS stores of the decoded
                // chunks last.  Second slice: fragment reads, one MFMA, the LDS stores of the
                // states, the remaining MFMAs -- every store of the step then has most of a
                // slice to complete before the barrier asks for it.
                if (ks == 0) {
                    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN + (SPARSE ? 4 : 0), 0);
#pragma unroll
                    for (int e = 0; e < TM * TN; ++e) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, TM == 4 ? 6 : 12, 0);
                        if (e < A_LOADS + NWORDS + (SPARSE ? 3 : 2)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);
                } else {
                    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x200, A_LOADS, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1, 0);
                }
            }
            // this step's LDS stores are complete; then all waves meet
            __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0) only
            __builtin_amdgcn_s_barrier();
        };
        // the same step in the two orders of PING (phase = 0: MFMAs first; 1: MFMAs last).  Compute-first
        // waves enter with the step's fragments (both slices) in registers and leave with the next step's;
        // the others fetch the step's own fragments at its start.
        auto body_ping = [&](auto phase_tag, int b, AStage& ra_new, const AStage& ra_wr, Stage& r_new, const Stage& r_dec) {
            constexpr int phase = decltype(phase_tag)::value;
            const int b1 = (b + 1) % P_STAGES, b2 = (b + 2) % P_STAGES;
            if constexpr (phase == 0) {
                mfma_slice(fa[0], fb[0]);
                mfma_slice(fa[1], fb[1]);
            }
            load_frags(phase == 0 ? b1 : b, 0, fa[0], fb[0]);
            load_frags(phase == 0 ? b1 : b, 1, fa[1], fb[1]);
            load_a(ra_new, a_cur);             // step kt + 3
            load_b(r_new, cur);                // step kt + 4
            advance_a();
            advance();
            write_b_fast(r_dec, b2, 0);
            write_b_fast(r_dec, b2, 1);
            write_a(ra_wr, b2);
            if constexpr (phase == 1) {
                mfma_slice(fa[0], fb[0]);
                mfma_slice(fa[1], fb[1]);
            }
            // scheduling template: the MFMAs as one cluster with the decode instructions in their
            // shadow (an MFMA occupies the pipe for 32 cycles, the wave issues three or four other
            // instructions meanwhile); fragment reads, global loads and LDS stores outside it
            if constexpr (phase == 0) {
#pragma unroll
                for (int e = 0; e < 2 * TM * TN; ++e) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * (TM + TN) + (SPARSE ? 4 : 0), 0);
                __builtin_amdgcn_sched_group_barrier(0x020, A_LOADS + NWORDS + (SPARSE ? 3 : 2), 0);
                __builtin_amdgcn_sched_group_barrier(0x200, A_LOADS + 2, 0);
            } else {
                __builtin_amdgcn_sched_group_barrier(0x100, 2 * (TM + TN) + (SPARSE ? 4 : 0), 0);
                __builtin_amdgcn_sched_group_barrier(0x020, A_LOADS + NWORDS + (SPARSE ? 3 : 2), 0);
                __builtin_amdgcn_sched_group_barrier(0x200, A_LOADS, 0);
#pragma unroll
                for (int e = 0; e < 2 * TM * TN; ++e) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                }
                __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);
            }
            __builtin_amdgcn_sched_barrier(0);       // nothing of this step moves behind the barrier
            __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0) only
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        };
        write_a(ra[0], 0);
        write_a(ra[1], 1);
        load_a(ra[0], a_cur); advance_a();              // step 2
#pragma unroll
        for (int q = 0; q < 2; ++q) { write_b_fast(r[0], 0, q); write_b_fast(r[1], 1, q); }
        load_b(r[2], cur); advance();                   // step 2
        load_b(r[0], cur); advance();                   // step 3
        __syncthreads();
        load_frags(0, 0, fa[0], fb[0]);
        // LDS stages and weight registers rotate with period 3, state registers with
        // period 2: six steps per trip, unrolled so that all of them are compile-time names
        if constexpr (!PING) {
            for (int kt = 0; kt < ktiles; kt += 6) {
#pragma unroll
                for (int u = 0; u < 6; ++u) {
                    if (u > 0 && kt + u >= ktiles) break;
                    body(u % 3, ra[(u + 1) % 2], ra[u % 2], r[(u + 1) % 3], r[(u + 2) % 3]);
                }
            }
        } else {
            auto run = [&](auto phase_tag) {
                for (int kt = 0; kt < ktiles; kt += 6) {
#pragma unroll
                    for (int u = 0; u < 6; ++u) {
                        if (u > 0 && kt + u >= ktiles) break;
                        body_ping(phase_tag, u % 3, ra[(u + 1) % 2], ra[u % 2], r[(u + 1) % 3], r[(u + 2) % 3]);
                    }
                }
            };
            if (__builtin_amdgcn_readfirstlane(wave) < NW) {
                load_frags(0, 1, fa[1], fb[1]);
                run(std::integral_constant<int, 0>{});
            } else {
                run(std::integral_constant<int, 1>{});
            }
        }
    } else if constexpr (!SPARSE && NW == 4) {
        // A tile with exponent-mode groups: the same three-stage pipeline (in the plain order of a
        // step: fragments, loads, decode between the MFMAs, stores, barrier) with the decode that
        // serves either mode per thread.  (256-column tiles only: in the 128-column kernel, which
        // keeps two workgroups per compute unit, this loop does not fit the registers, and its
        // spills slowed the linear loop down as well.)
        auto write_b_mixed = [&](const Stage& s, int stage, int q) {
            const h16x2 s2 = stage_scale(s);
            const bool expo = !(s2.x >= (h16)0.0f);
            const h16x8 w = dequant_chunk_mixed<BITS>(chunk_bits(s, q), expo, stage_negzero(s), s2);
            *reinterpret_cast<h16x8*>(&Bs[stage * B_STAGE + ((bhb * 2 + q) * BN + bn) * 8]) = w;
        };
        h16x8 fa[2][TM], fb[2][TN];
        auto body_mixed = [&](int b, AStage& ra_new, const AStage& ra_wr, Stage& r_new, const Stage& r_dec) {
            const int b1 = (b + 1) % P_STAGES, b2 = (b + 2) % P_STAGES;
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                if (ks == 0) load_frags(b, 1, fa[1], fb[1]);
                else load_frags(b1, 0, fa[0], fb[0]);
                if (ks == 0) {
                    load_a(ra_new, a_cur);             // step kt + 3
                    load_b(r_new, cur);                // step kt + 4
                    advance_a();
                    advance();
                    write_b_mixed(r_dec, b2, 0);
                    write_b_mixed(r_dec, b2, 1);
                } else {
                    write_a(ra_wr, b2);
                }
                mfma_slice(fa[ks], fb[ks]);
                if (ks == 0) {
                    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
                    for (int e = 0; e < TM * TN; ++e) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, TM == 4 ? 14 : 28, 0);
                        if (e < A_LOADS + NWORDS + 2) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                    }
                    __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);
                } else {
                    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x200, A_LOADS, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1, 0);
                }
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0) only
            __builtin_amdgcn_s_barrier();
        };
        write_a(ra[0], 0);
        write_a(ra[1], 1);
        load_a(ra[0], a_cur); advance_a();              // step 2
#pragma unroll
        for (int q = 0; q < 2; ++q) { write_b_mixed(r[0], 0, q); write_b_mixed(r[1], 1, q); }
        load_b(r[2], cur); advance();                   // step 2
        load_b(r[0], cur); advance();                   // step 3
        __syncthreads();
        load_frags(0, 0, fa[0], fb[0]);
        for (int kt = 0; kt < ktiles; kt += 6) {
#pragma unroll
            for (int u = 0; u < 6; ++u) {
                if (u > 0 && kt + u >= ktiles) break;
                body_mixed(u % 3, ra[(u + 1) % 2], ra[u % 2], r[(u + 1) % 3], r[(u + 2) % 3]);
            }
        }
    } else {
        // A tile with exponent-mode groups, 16:32 and the 128-column tiles (whose registers do not hold a second copy
        // of the pipelined loop): a plain loop over two LDS stages -- the step's operands, requested two steps
        // earlier, are decoded (either mode per thread, without a branch) and stored, the operands of the step
        // after next are requested, one barrier, the step's MFMAs.  (A stage is written again two steps later,
        // and every wave has left its reads of it behind when it arrives at the barrier in between.)
        auto write_b_two_modes = [&](const Stage& s, int stage, int q) {
            const h16x2 s2 = stage_scale(s);
            const bool expo = !(s2.x >= (h16)0.0f);
            h16x8 w;
            if constexpr (SPARSE) {
                uint32_t v, m8;
                sparse_chunk(s, q, v, m8);
                w = dequant_chunk_sparse_mixed(v, m8, lut, expo, stage_negzero(s), s2);
            } else {
                w = dequant_chunk_mixed<BITS>(chunk_bits(s, q), expo, stage_negzero(s), s2);
            }
            *reinterpret_cast<h16x8*>(&Bs[stage * B_STAGE + ((bhb * 2 + q) * BN + bn) * 8]) = w;
        };
        h16x8 fa[TM], fb[TN];
        for (int kt = 0; kt < ktiles; kt += 2) {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                if (u > 0 && kt + u >= ktiles) break;
                write_a(ra[u], u);
                write_b_two_modes(r[u], u, 0);
                write_b_two_modes(r[u], u, 1);
                if (kt + u + 2 < ktiles) {
                    load_a(ra[u], a_cur); advance_a();
                    load_b(r[u], cur); advance();
                }
                __syncthreads();
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    load_frags(u, ks, fa, fb);
                    mfma_slice(fa, fb);
                }
            }
        }
    }
    if (SPLIT && nsplit > 1) {
        // Every workgroup of the tile stores its partial accumulators (16 bytes per lane and
        // store: register group g of thread t at (g * T + t) * 16 -- whole cache lines per wave)
        // and then counts itself in; whoever finds all the others counted adds the partials up
        // in split order (its own included, from memory: the sum has one order whoever is
        // last) and writes the tile.  Stores and loads go straight through to memory
        // (system-scope cache policy), the counter is a device-scope atomic: no cache-wide
        // fence, no waiting.  (Two workgroups per tile: the last one adds the other's partial to
        // its own registers -- a sum of two terms has one value in either order.)
        constexpr int SLOT_BYTES = BM * BN * 4, THROUGH = 17;      // sc0 | sc1
        char* const slots = reinterpret_cast<char*>(a.part) + (int64_t)tile * nsplit * SLOT_BYTES;
        const __amdgpu_buffer_rsrc_t mine = __builtin_amdgcn_make_buffer_rsrc(
            slots + (int64_t)split * SLOT_BYTES, 0, SLOT_BYTES, RSRC_FLAGS);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    __builtin_amdgcn_raw_buffer_store_b128(bitcast<u32x4>(v), mine, (((i * TN + j) * 4 + q) * T + t) * 16, 0, THROUGH);
                }
        __builtin_amdgcn_s_waitcnt(0);                 // every store of this thread has been acknowledged
        int* const flag = reinterpret_cast<int*>(As);
        __syncthreads();
        if (t == 0) *flag = __hip_atomic_fetch_add(a.counters + tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*flag != nsplit - 1) return;
        if (t == 0) __hip_atomic_store(a.counters + tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // clean for the next call
        if (nsplit > 2) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
        }
        for (int sp = nsplit > 2 ? 0 : 1 - split; sp < (nsplit > 2 ? nsplit : 2 - split); ++sp) {
            const __amdgpu_buffer_rsrc_t theirs = __builtin_amdgcn_make_buffer_rsrc(
                slots + (int64_t)sp * SLOT_BYTES, 0, SLOT_BYTES, RSRC_FLAGS);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x4 v = bitcast<f32x4>(__builtin_amdgcn_raw_buffer_load_b128(
                            theirs, (((i * TN + j) * 4 + q) * T + t) * 16, 0, THROUGH));
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] += v[e];
                    }
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = s0 + wn0 + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm0 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (row < a.M) outs[(int64_t)row * a.S + col] = (h16)acc[i][j][r];
            }
        }
}

template <int BITS, bool SPARSE, int NW, int TM, bool PING, bool SPLIT>
__global__ __launch_bounds__(NW * 128, NW == 2 ? 2 : 1) void matmul_kernel_pipe(MatmulArgs a) {
    constexpr int BM = TM * 64, BN = NW * 64;
    __shared__ __attribute__((aligned(16))) h16 As[P_STAGES * BM * PK];
    __shared__ __attribute__((aligned(16))) h16 Bs[P_STAGES * PK * BN];
    __shared__ __attribute__((aligned(16))) uint32_t Lut[SPARSE ? SPARSE_LUT_WORDS : 4];
    // (split-K: the workgroups of a tile are neighbours in the grid, so they run at about the same time;
    // the tiles before `split_from` are whole)
    const int total = a.tiles_m * a.tiles_n;
    int bid = blockIdx.x, split = 0, nsplit = 1, slot = 0;
    if constexpr (SPLIT) {
        const int v = (int)blockIdx.x - a.split_from;
        if (v >= 0) {
            bid = a.split_from + v / a.ksplit;
            split = v % a.ksplit;
            nsplit = a.ksplit;
            slot = (int)blockIdx.z * (total - a.split_from) + v / a.ksplit;       // counter and partial tiles
        }
    }
    int tile_m, tile_n;
    if (total % 8 == 0) {
        // XCD-aware numbering: workgroups are dealt round-robin to the 8 XCDs (each
        // with its own L2), so XCD x takes the contiguous range x * total / 8 ... of tiles
        const int per_xcd = total / 8, l = bid / 8;
        if (a.by_columns) {
            // ... walked one tile row at a time across the XCD's tile columns: the tiles in
            // flight on an XCD then share few rows of states, whose 64 bytes per row and K
            // step outweigh the packed weights' 16 bytes per column (measured: 1-5 % faster
            // than column by column)
            const int cols = per_xcd / a.tiles_m;
            tile_m = l / cols;
            tile_n = (bid % 8) * cols + l % cols;
        } else {
            bid = (bid % 8) * per_xcd + l;
            tile_m = bid % a.tiles_m, tile_n = bid / a.tiles_m;
        }
    } else {
        tile_m = bid % a.tiles_m, tile_n = bid / a.tiles_m;
    }
    const int64_t boff = blockIdx.z;
    pipe_tile<BITS, SPARSE, TM, NW, PING, SPLIT>(a, tile_m * BM, tile_n * BN, a.x + boff * a.M * (int64_t)a.K,
                                          a.outs + boff * a.M * (int64_t)a.S, As, Bs, Lut, slot, split, nsplit);
}

template <int BITS, bool SPARSE, int NW, int TM = 4, bool PING = false>
static void launch_pipe(MatmulArgs a, int64_t B, hipStream_t st) {
    a.tiles_m = (a.M + TM * 64 - 1) / (TM * 64);
    a.tiles_n = a.S / (NW * 64);
    const int total = a.tiles_m * a.tiles_n;
    const dim3 grid(a.split_from + (total - a.split_from) * a.ksplit, 1, (unsigned)B), block(NW * 128);
    a.by_columns = a.tiles_n % 8 == 0;
    if (noting("matmul_kernel_pipe<bits=%d,%s,tile=%dx%d,%s> tiles=%d ksplit=%d split_from=%d workgroups=%u batch=%d", BITS,
               SPARSE ? "16:32" : "dense", TM * 64, NW * 64, PING ? "two-phase" : "plain", total, a.ksplit, a.split_from, grid.x, (int)B))
        return;
    if (a.ksplit > 1) {
        hipLaunchKernelGGL((matmul_kernel_pipe<BITS, SPARSE, NW, TM, PING, true>), grid, block, 0, st, a);
        return;
    }
    hipLaunchKernelGGL((matmul_kernel_pipe<BITS, SPARSE, NW, TM, PING, false>), grid, block, 0, st, a);
}

// ---- split-K plan.  Shapes with at most 128 tiles of 256 x 256 leave more than half of the GPU
// idle; they run as 256 x 128 tiles (16:32: 256 x 256) with `ksplit` workgroups per tile.  The factor
// minimises a cost in K steps fitted to measurements (K = 4096 ... 20480, 32 ... 240 tiles):
// rounds of 256 workgroups x (steps per workgroup + 20 for its prologue and hand-over) + 6 per split.
constexpr int64_t MM_SPLIT_MAX_TILES = 1024;             // counters: one int per tile in 4 KB
constexpr int64_t MM_SPLIT_MAX_BYTES = 192ll << 20;      // cap of the partial tiles
struct SplitPlan { int ksplit; int64_t tiles; int64_t tile_bytes; };
static SplitPlan plan_split(bool sparse, int64_t B, int64_t M, int64_t K, int64_t S) {
    const SplitPlan none{1, 0, 0};
    if (S % (sparse ? 256 : 128) != 0) return none;
    const int64_t m_pad = (M + 255) / 256 * 256, tiles4 = m_pad / 256 * ((S + 255) / 256) * B;
    if (tiles4 > 128) return none;
    SplitPlan p{1, m_pad / 256 * (S / (sparse ? 256 : 128)) * B, sparse ? 256 * 256 * 4 : 256 * 128 * 4};
    if (p.tiles > MM_SPLIT_MAX_TILES) return none;
    const int64_t steps = K / 32, forced = tuning(TUNE_MM_SPLIT);
    // (16:32, whose 256 x 256 tiles run one per CU: a GPU filled to the last CU runs its K steps 39 % slower than a
    // nearly empty one -- the power limit --, three quarters full 15 % slower; fitted to 320 timed launches, K = 2048 ...
    // 14336, 16 ... 128 tiles, 1 ... 8 ways: 64 tiles at K=4096 four ways 79 us, three ways 68; 32 tiles at K=14336 eight
    // ways 125, six ways 106.  Its pick is within 1 % of the best measured factor on average, 10 % at worst; without
    // the term 3 % / 20 %.  The dense formats' 256 x 128 tiles, two workgroups per CU, are within 1.4 % / 11 % as is.)
    auto cost = [&](int64_t ks) -> double {
        const int64_t wgs = p.tiles * ks, rounds = (wgs + 255) / 256;
        const double own = (double)(rounds * ((steps + ks - 1) / ks + 20));
        if (!sparse) return own + (ks > 1 ? 6.0 * ks : 0.0);
        const double fill = wgs >= 256 ? 1.0 : wgs / 256.0;
        return own * (1.0 + 0.39 * std::pow(fill, 3.2)) + (ks > 1 ? 5.0 * ks : 0.0);
    };
    int64_t best = 1;
    for (int64_t ks = 2; ks <= 8; ++ks) {
        if (steps / ks < 8 || p.tiles * ks * p.tile_bytes > MM_SPLIT_MAX_BYTES) break;
        if (forced == ks) { best = ks; break; }
        if (forced == 0 && cost(ks) < cost(best)) best = ks;
    }
    if (best < 2) return none;
    p.ksplit = (int)best;
    return p;
}

// ---- split of the last round.  256 x 256 tiles run one per CU, in rounds of 256; when the last round
// would fill at most half of the GPU, its tiles -- and only they -- are split along K over as many
// workgroups as fit half of the GPU (at least two per tile, at least 32 K steps each).
struct TailPlan { int ksplit; int64_t split_from, tiles; };
static TailPlan plan_tail(int64_t B, int64_t M, int64_t K, int64_t S) {
    const TailPlan none{1, 0, 0};
    if (B != 1 || S % 256 != 0 || tuning(TUNE_MM_TAIL) == 1) return none;
    const int64_t total = (M + 255) / 256 * (S / 256), tail = total % 256;
    if (total <= 256 || tail == 0 || tail > 128) return none;
    // (measured, K = 2048 ... 8192, tails of 16 ... 128 tiles: the split pays while its workgroups fill at most half of
    // the GPU -- two per tile from 64 tiles on, where the second adds the first one's partial tile to its registers
    // and nothing else is read back -- and while a share keeps 32 K steps: K=4096, S=8192, 2304 rows, 32 tiles in
    // the tail: eight ways 197 us, four ways 170; K=2048, S=8192, 2560 rows, 64 tiles: four ways 121, two ways 101,
    // unsplit 107; a tail of 97 ... 128 tiles on K = 2048 is better left whole, 110 against 117)
    if (tail > 96 && K < 3072) return none;
    const int64_t cap = tuning(TUNE_MM_TAIL) >= 2 ? tuning(TUNE_MM_TAIL) : 8;
    const int64_t ks = std::min<int64_t>({std::max<int64_t>(2, 128 / tail), cap, K / 32 / 32});
    if (ks < 2 || tail * ks * (256 * 256 * 4) > MM_SPLIT_MAX_BYTES) return none;
    return TailPlan{(int)ks, total - tail, tail};
}

template <int BITS, bool SPARSE, int BM, int BN, int WM, int WN>
static void launch_tile(MatmulArgs a, int64_t B, hipStream_t st) {
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.S + BN - 1) / BN;
    const dim3 grid(a.tiles_m * a.tiles_n, 1, (unsigned)B), block((BM / WM) * (BN / WN) * 64);
    if (noting("matmul_kernel<bits=%d,%s,tile=%dx%d> tiles=%u batch=%d", BITS, SPARSE ? "16:32" : "dense", BM, BN, grid.x, (int)B)) return;
    hipLaunchKernelGGL((matmul_kernel<BITS, SPARSE, BM, BN, WM, WN>), grid, block, 0, st, a);
}

template <int BITS, bool SPARSE>
static void launch(MatmulArgs a, int64_t B, hipStream_t st, void* workspace, size_t workspace_bytes) {
    // variant 0 = automatic.  Tile-aligned shapes take the pipelined kernel, as
    // 256 x 256 tiles (one eight-wave workgroup per CU) or 256 x 128 tiles (two
    // four-wave workgroups per CU).  Measured on MI355X (K = 4096 ... 20480, S = 5120
    // ... 28672, M = 256 ... 4096): the small tiles win when at most half of the CUs
    // would get a large tile, and in the second round of large tiles while it is at
    // most three eighths full; the large ones everywhere else.  The 16:32 format always takes the large tiles (its decode
    // needs more registers than the four-wave shape leaves).  Everything else:
    // 128 x 256 tiles, and 128 x 128 for narrow outputs or few rows.
    int variant = (int)tuning(TUNE_MM_VARIANT);
    // (M is padded to whole tiles of 256 rows; measured worth it up to half as many rows again
    // -- the general kernel reaches about 60 % of the pipelined one's rate -- and for a single
    // row of tiles from 129 rows on, where the general kernel would need two rows of its 128-row tiles)
    const int64_t m_pad = (a.M + 255) / 256 * 256;
    // (97 ... 128 rows: the general kernel's single row of 128 x 128 tiles cannot split K; the padded
    // pipelined kernel can, and wins when K is long -- 16:32: from K = 1024; dense: from K = 2048 on
    // outputs too narrow to give the general kernel a tile per CU and a half)
    const bool pad_97_128 = a.M > 96 && a.M <= 128 && (SPARSE ? a.K >= 1024 : (a.K >= 2048 && a.S <= 12288));
    // (the kernel addresses with 32-bit byte offsets into buffer resources: 256 rows of states,
    // the whole packed matrix and the whole of scales / zeros have to stay below 2 GB each)
    const int64_t w_bytes = (int64_t)a.K / 32 * PipeFmt<BITS, SPARSE>::ROWS * 4 * a.S;
    const int64_t sz_bytes = ((int64_t)a.K / 64 + a.group_units - 1) / a.group_units * a.S * 2;
    const bool shape_ok = a.K <= (1 << 22) && a.S <= (1 << 27) && w_bytes < (1ll << 31) && sz_bytes < (1ll << 31);
    // (257 ... 341 rows, padded by half and more: still better than the general kernel where split-K makes up
    // for a small grid, and for 16:32 everywhere -- its general decode is slow; measured K >= 2048)
    const bool pad_257_341 = a.M > 256 && a.M < 342 && a.K >= 2048 &&
                             (SPARSE || m_pad / 256 * ((a.S + 255) / 256) * B <= 128);
    const bool m_ok = (m_pad * 2 <= a.M * 3 || (a.M > 128 && a.M <= 256) || pad_97_128 || pad_257_341) && shape_ok;
    // An odd number of 128-row tile rows (257 ... 384 rows, 513 ... 640, ... up to 1152): 128 x 256 tiles (the
    // same kernel with half the rows per wave) instead of 256 x 256 tiles padded by another 128 rows -- when
    // they give the GPU at most one round of at least half (16:32: three quarters) of its CUs; smaller grids
    // are better off with split-K
    const int64_t rows_128 = (a.M + 127) / 128, tiles_128 = rows_128 * (a.S / 256) * B;
    // (dense: also with an even number of rows when the 128 x 256 tiles fill nine sixteenths of the GPU and more --
    // better than half as many 256 x 256 tiles or 256 x 128 tiles with split-K, by 5 - 10 %)
    // (K=S=3072, eleven to thirteen rows of 128: 132 - 156 tiles of 128 x 256 in 49 - 50 us against 56 - 59 for the
    // 256 x 128 tiles that used to serve 1408 ... 1664 rows there)
    const bool odd_rows = rows_128 % 2 == 1 && rows_128 <= (SPARSE ? 9 : 13);
    const bool three_rows = a.M > 256 && shape_ok && a.S % 256 == 0 && tiles_128 <= 256 &&
                            (SPARSE ? odd_rows && tiles_128 >= 192 : tiles_128 >= (odd_rows ? 128 : 144));
    const bool pipe2_ok = !SPARSE && m_ok && a.S % 128 == 0;
    const bool pipe4_ok = m_ok && a.S % 256 == 0;
    if (variant != 1 && variant != 3 && variant != 5 && variant != 6 && variant != 7 && variant != 9) variant = 0;
    if ((variant == 5 && !pipe2_ok) || ((variant == 6 || variant == 9) && !pipe4_ok) ||
        (variant == 7 && !(shape_ok && a.S % 256 == 0))) variant = 0;
    // (a last round of large tiles that fills at most half of the GPU is split along K when the
    // workspace has room for its partial tiles: better than small tiles then)
    const TailPlan tp = plan_tail(B, a.M, a.K, a.S);
    const WorkspaceParts wsp = workspace_parts(workspace, workspace_bytes);
    const bool tail_ok = pipe4_ok && tp.ksplit > 1 && wsp.counters != nullptr &&
                         wsp.scratch_bytes >= (size_t)(tp.tiles * tp.ksplit * (256 * 256 * 4));
    if (variant == 0) {
        const int64_t tiles4 = m_pad / 256 * ((a.S + 255) / 256) * B;
        const int64_t last = tiles4 % 256;
        const bool small_better = tiles4 <= 128 || (!tail_ok && tiles4 > 256 && tiles4 < 512 && last > 0 && last <= 96);
        // (a grid that fills at most half of the GPU with a short K: the pipelined kernel's prologue -- three
        // stages, the scan of the scales -- costs more than its faster steps return; measured K <= 1024)
        // (a long K on a narrow output: 256 x 128 tiles split three ways and more along K, in shares of at least
        // 140 steps, beat one round of unsplit 128 x 256 tiles -- K=20480, S=5120: 769 rows 283 -> 240 us, 1024 rows
        // 279 -> 252 us; K=14336, S=4096, 1280 rows 198 -> 187 us; shorter shares lose: K=S=8192, 1024 rows 147 / 159)
        bool long_k_split = false;
        if (!SPARSE && three_rows && pipe2_ok) {
            const SplitPlan sp = plan_split(false, B, a.M, a.K, a.S);
            long_k_split = sp.ksplit >= 3 && a.K / 32 / sp.ksplit >= 140 && wsp.counters != nullptr &&
                           wsp.scratch_bytes >= (size_t)(sp.tiles * sp.ksplit * sp.tile_bytes);
        }
        // (16:32 with at most 128 padded 256-row tiles: those, split along K, beat the 128-row tiles from K = 4096 on --
        // K=S=8192, 896 rows: 182 -> 163 us; K=8192, S=10240, 640 rows: 178 -> 155; K=16384, S=7168, 800 rows: 346 -> 271;
        // K=4096: 0 - 12 %; at K=2048 the unsplit 128-row tiles still win by 1 - 7 %)
        bool sparse_split = false;
        if (SPARSE && three_rows && pipe4_ok && tiles4 <= 128 && a.K >= 4096) {
            const SplitPlan sp = plan_split(true, B, a.M, a.K, a.S);
            sparse_split = sp.ksplit > 1 && wsp.counters != nullptr && sp.tiles <= 1024 &&
                           wsp.scratch_bytes >= (size_t)(sp.tiles * sp.ksplit * sp.tile_bytes);
        }
        if (!SPARSE && tiles4 <= 128 && a.K <= 1024) variant = 1;
        else if (long_k_split) variant = 5;
        else if (three_rows && !sparse_split) variant = 7;
        else if (pipe4_ok && (SPARSE || !pipe2_ok || !small_better)) variant = 6;
        else if (pipe2_ok) variant = 5;
        else if (a.M > 512 && a.S >= 256) variant = 3;
        else variant = 1;
    }
    // split-K where the plan asks for it and the scratch half of the caller's workspace has room for
    // the partial tiles (the per-tile counters sit in the last page of the half that is kept zero)
    if ((SPARSE && (variant == 6 || variant == 9)) || (!SPARSE && variant == 5)) {
        const SplitPlan sp = plan_split(SPARSE, B, a.M, a.K, a.S);
        const WorkspaceParts ws = workspace_parts(workspace, workspace_bytes);
        if (sp.ksplit > 1 && ws.counters != nullptr && sp.tiles <= 1024 &&
            ws.scratch_bytes >= (size_t)(sp.tiles * sp.ksplit * sp.tile_bytes)) {
            a.ksplit = sp.ksplit;
            a.counters = reinterpret_cast<int*>(ws.counters);
            a.part = reinterpret_cast<float*>(ws.scratch);
        }
    }
    if (a.ksplit == 1 && (variant == 6 || variant == 9) && tail_ok) {
        a.ksplit = tp.ksplit;
        a.split_from = (int)tp.split_from;
        a.counters = reinterpret_cast<int*>(wsp.counters);
        a.part = reinterpret_cast<float*>(wsp.scratch);
    }
    if (variant == 1) launch_tile<BITS, SPARSE, 128, 128, 64, 64>(a, B, st);
    else if (variant == 3) launch_tile<BITS, SPARSE, 128, 256, 128, 64>(a, B, st);
    // (256 x 256: the dense formats run the two halves of the workgroup in opposite phases, 2-3 %
    // faster; the 16:32 decode has no registers to spare for it.  Variant 9 forces the plain order.)
    else if (variant == 7) launch_pipe<BITS, SPARSE, 4, 2>(a, B, st);
    else if (variant == 6 && !SPARSE) launch_pipe<BITS, SPARSE, 4, 4, true>(a, B, st);
    else if (variant == 6 || variant == 9) launch_pipe<BITS, SPARSE, 4>(a, B, st);
    else if constexpr (!SPARSE) launch_pipe<BITS, false, 2>(a, B, st);
}

}  // namespace i4

using namespace i4;

extern "C" int int4mm_matmul(int bits, void* outs, const void* matrix, const void* multiplier,
                             const void* scales, const void* zeros, const void* sparse_mask,
                             const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                             void* stream) {
    int rc = validate_product(bits, outs, matrix, multiplier, scales, zeros, sparse_mask, shape, false);
    if (rc != INT4MM_OK) return rc;
    int64_t B = shape->batch, M = shape->seq_len;
    const int64_t K = shape->in_size, S = shape->out_size;
    if (B * M * S == 0) return INT4MM_OK;
    // Batches are contiguous ([B, M, K] states, [B, M, S] outputs) and every kernel's rows are independent: B
    // products of M rows are one product of B * M rows -- whole tiles instead of B padded ones (K=5120, S=20480: 32
    // batch elements of 20 rows 970 -> 152 us, 5 of 130 rows 258 -> 153).
    if (B > 1 && B * M <= ((int64_t)1 << 31) - 256) { M *= B; B = 1; }
    if (((M + 127) / 128) * ((S + 127) / 128) > 0x7FFFFFFF / 2) return INT4MM_ERR_SHAPE;
    const int64_t g = shape->group_size < 0 ? ONE_GROUP : shape->group_size;

    hipStream_t st = (hipStream_t)stream;
    // 2 .. 96 rows in all (batches are contiguous, so they flatten; on suitable shapes up to 512): the few-row
    // kernels, which read every packed word once for all rows -- unless a tile-kernel variant is forced
    if (B * M == 1 && !tuning(TUNE_NO_SKINNY) && !tuning(TUNE_MM_VARIANT) &&
        matvec_one_row(bits, (h16*)outs, (const uint32_t*)matrix, (const uint32_t*)sparse_mask, (const h16*)multiplier,
                       (const h16*)scales, (const h16*)zeros, K, S, g, st, workspace, workspace_bytes, &rc))
        return rc;
    if (B * M >= 2 && B * M <= 4 && !sparse_mask && !tuning(TUNE_NO_SKINNY) && !tuning(TUNE_MM_VARIANT) &&
        matvec_rows(bits, (h16*)outs, (const uint32_t*)matrix, (const h16*)multiplier, (const h16*)scales, (const h16*)zeros,
                    B * M, K, S, g, false, st, workspace, workspace_bytes))
        return check_launch("matmul");
    if (B * M >= 2 && B * M <= SK_WIDE_MAX_ROWS && !tuning(TUNE_NO_SKINNY) && !tuning(TUNE_MM_VARIANT) &&
        skinny_rows(bits, (h16*)outs, (const uint32_t*)matrix, (const h16*)multiplier, (const h16*)scales,
                    (const h16*)zeros, B * M, K, S, g, false, st, (const uint32_t*)sparse_mask, workspace, workspace_bytes))
        return check_launch("matmul");

    MatmulArgs a;
    a.outs = (h16*)outs;
    a.matrix = (const uint32_t*)matrix;
    a.mask = (const uint32_t*)sparse_mask;
    a.x = (const h16*)multiplier;
    a.scales = (const h16*)scales;
    a.zeros = (const h16*)zeros;
    a.M = (int)M;
    a.K = (int)K;
    a.S = (int)S;
    a.group_units = (int)(g / 64 > 0x7FFFFFF ? 0x7FFFFFF : g / 64);
    a.tiles_m = a.tiles_n = 0;
    a.by_columns = 0;
    a.ksplit = 1;
    a.split_from = 0;
    a.part = nullptr;
    a.counters = nullptr;

    if (sparse_mask) launch<4, true>(a, B, st, workspace, workspace_bytes);
    else if (bits == 4) launch<4, false>(a, B, st, workspace, workspace_bytes);
    else if (bits == 3) launch<3, false>(a, B, st, workspace, workspace_bytes);
    else launch<2, false>(a, B, st, workspace, workspace_bytes);
    return check_launch("matmul");
}

// Workspace with which int4mm_matmul may split K for this shape: what the matvec needs, plus room for
// the partial tiles in the scratch half.  A smaller workspace is not an error: the product then runs unsplit.
extern "C" size_t int4mm_matmul_workspace_bytes(const int4mm_shape* shape, int sparse) {
    if (shape == nullptr) return 0;
    int64_t B = shape->batch, M = shape->seq_len;
    const int64_t K = shape->in_size, S = shape->out_size;
    size_t need = int4mm_workspace_bytes(S);
    if (B <= 0 || M <= 0 || K < 64 || S < 128) return need;
    if (B > 1 && B * M <= ((int64_t)1 << 31) - 256) { M *= B; B = 1; }           // (as int4mm_matmul does)
    // (the matvec entry takes more than 512 batch elements of one row in chunks of up to 512 through the few-row kernels)
    const size_t few_rows = B * M <= SK_WIDE_MAX_ROWS ? skinny_workspace_bytes(B * M, K, S, sparse != 0)
                          : shape->seq_len == 1 ? skinny_workspace_bytes(SK_WIDE_MAX_ROWS, K, S, sparse != 0) : 0;
    if (B * M <= 96) return need + 2 * round_to_page(few_rows);
    const SplitPlan sp = plan_split(sparse != 0, B, M, K, S);
    if (sp.ksplit > 1 || few_rows > 0)
        need += 2 * round_to_page(std::max(few_rows, sp.ksplit > 1 ? (size_t)(sp.tiles * sp.ksplit * sp.tile_bytes) : 0));
    const TailPlan tp = plan_tail(B, M, K, S);
    if (sp.ksplit == 1 && tp.ksplit > 1) need += 2 * round_to_page((size_t)(tp.tiles * tp.ksplit * (256 * 256 * 4)));
    return need;
}
