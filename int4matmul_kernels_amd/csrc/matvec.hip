// Quantized matrix-vector product for gfx950: outs = fp16(fp32(outs) + x @ W).
//
// Bandwidth-bound streaming kernel.  The packed matrix is [rows, S] with the
// column index contiguous, so lanes own columns: a lane reads 16 bytes = the
// packed words of 4 adjacent columns of one packed row, a wavefront reads
// 1 KiB contiguous per row.  K is cut into 64-row "units" (the granularity of
// quantisation groups); a wave walks a run of units, a workgroup's waves walk
// adjacent runs, grid.y cuts K further.  Partial sums meet in LDS, and across
// workgroups through fp32 slots in the workspace with an arrival counter: the
// last workgroup of a column strip adds the slots in a fixed order, adds the
// prior contents of outs and writes fp16 -- one kernel, deterministic.
//
// Arithmetic: the states x are wave-uniform, so they travel through scalar
// registers.  For int4/int2 the codes are never converted one by one: a mask
// and an OR turn two fields of a word into a half2 whose lanes are 2^e + q
// ("magic" exponents chosen so that the field lands on the units of the
// mantissa), v_dot2_f32_f16 multiplies that pair by the matching pair of states
// into an fp32 accumulator, and the constant part sum_k 2^e_k * x_k is removed
// once per unit.  Per (group, column):  y += s * (sum_k x_k q_k - z * sum_k x_k),
// which is the exact value of sum_k x_k (q_k - z) s; the fp16 roundings that the
// reference applies to each weight are not reproduced here (they are in the
// dequantise helper, which is bit-exact).
#include "common.h"

namespace i4 {

constexpr int MV_MAX_WAVES = 16;
constexpr int MV_COLS = 256;          // columns per wave: 64 lanes x 4
constexpr int MV_MAX_SPLITS = 32;

struct MatvecArgs {
    h16* outs;
    const uint32_t* matrix;
    const uint32_t* mask;
    const h16* x;
    const h16* scales;
    const h16* zeros;
    float* partials;        // [splits][S]
    int* counters;          // [strips]
    int K, S;
    int units_total;        // K / 64
    int units_per_wave;
    int group_units;        // group size in units (>= 1); huge for a single group
    int splits;             // == gridDim.y
};

typedef const uint32_t __attribute__((address_space(4))) * const_u32p;

__device__ __forceinline__ const_u32p to_const(const void* p) {
    return (const_u32p)(uintptr_t)p;
}

// ------------------------------------------------------------------ formats
// Packed rows per 64-row unit, and how one unit is held in registers.
template <int BITS, bool SPARSE> struct Fmt;
template <> struct Fmt<4, false> { static constexpr int ROWS = 8, MROWS = 0; };
template <> struct Fmt<3, false> { static constexpr int ROWS = 6, MROWS = 0; };
template <> struct Fmt<2, false> { static constexpr int ROWS = 4, MROWS = 0; };
template <> struct Fmt<4, true>  { static constexpr int ROWS = 4, MROWS = 2; };

template <int BITS, bool SPARSE>
struct Unit {
    u32x4 w[Fmt<BITS, SPARSE>::ROWS];
    u32x4 m[Fmt<BITS, SPARSE>::MROWS == 0 ? 1 : Fmt<BITS, SPARSE>::MROWS];
    u32x2 sc, ze;            // fp16 scales / zeros of the lane's 4 columns
    float xl;                // x[k0 + lane] for the wave-wide sums
};

template <int BITS, bool SPARSE>
__device__ __forceinline__ void load_unit(Unit<BITS, SPARSE>& u, const MatvecArgs& a, int unit,
                                          int col, bool col_ok, int lane) {
    constexpr int ROWS = Fmt<BITS, SPARSE>::ROWS, MROWS = Fmt<BITS, SPARSE>::MROWS;
    const int64_t S = a.S;
    if (col_ok) {
        const uint32_t* p = a.matrix + (int64_t)unit * ROWS * S + col;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) u.w[r] = *reinterpret_cast<const u32x4*>(p + r * S);
        if constexpr (MROWS > 0) {
            const uint32_t* q = a.mask + (int64_t)unit * MROWS * S + col;
#pragma unroll
            for (int r = 0; r < MROWS; ++r) u.m[r] = *reinterpret_cast<const u32x4*>(q + r * S);
        }
        const int64_t gofs = (int64_t)(unit / a.group_units) * S + col;
        u.sc = *reinterpret_cast<const u32x2*>(a.scales + gofs);
        u.ze = *reinterpret_cast<const u32x2*>(a.zeros + gofs);
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) u.w[r] = u32x4{0, 0, 0, 0};
        if constexpr (MROWS > 0) {
#pragma unroll
            for (int r = 0; r < MROWS; ++r) u.m[r] = u32x4{0, 0, 0, 0};
        }
        u.sc = u32x2{0, 0};
        u.ze = u32x2{0, 0};
    }
    u.xl = (float)a.x[unit * 64 + lane];
}

__device__ __forceinline__ uint32_t pack_lo(uint32_t a, uint32_t b) { return (a & 0xFFFFu) | (b << 16); }
__device__ __forceinline__ uint32_t pack_hi(uint32_t a, uint32_t b) { return (a >> 16) | (b & 0xFFFF0000u); }

// Slow, fully general accumulation of one unit (any format, either quantisation
// mode).  acc[c] = sum over kept k of x_k * value(q_k); xs[c] = sum over kept k
// of x_k.
template <int BITS, bool SPARSE>
__device__ __forceinline__ void unit_generic(const Unit<BITS, SPARSE>& u, const_u32p xw,
                                             const bool expo[4], float acc[4], float xs[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) { acc[c] = 0.f; xs[c] = 0.f; }
#pragma unroll
    for (int hb = 0; hb < 2; ++hb) {                 // two 32-row blocks
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint32_t codes[32];
            uint32_t keep = 0xFFFFFFFFu;
            if constexpr (SPARSE) {
                uint64_t v = (uint64_t)u.w[2 * hb][c] | ((uint64_t)u.w[2 * hb + 1][c] << 32);
                keep = u.m[hb][c];
#pragma unroll
                for (int t = 0; t < 32; ++t) {
                    const bool k = (keep >> t) & 1u;
                    codes[t] = (uint32_t)v & 0xFu;
                    v >>= k ? 4 : 0;
                }
            } else if constexpr (BITS == 3) {
                const uint64_t lo = (uint64_t)u.w[3 * hb][c] | ((uint64_t)u.w[3 * hb + 1][c] << 32);
                const uint64_t hi = (uint64_t)u.w[3 * hb + 1][c] | ((uint64_t)u.w[3 * hb + 2][c] << 32);
#pragma unroll
                for (int t = 0; t < 32; ++t) {
                    const int pos = 3 * t;
                    codes[t] = pos + 3 <= 64 ? (uint32_t)(lo >> pos) & 7u
                                             : (uint32_t)(hi >> (pos - 32)) & 7u;
                }
            } else {
                constexpr int PER = 32 / BITS;
#pragma unroll
                for (int i = 0; i < BITS; ++i) {
                    uint32_t v = u.w[BITS * hb + i][c];
#pragma unroll
                    for (int j = 0; j < PER; ++j) { codes[i * PER + j] = v & ((1u << BITS) - 1u); v >>= BITS; }
                }
            }
#pragma unroll
            for (int t = 0; t < 32; ++t) {
                const uint32_t xpair = xw[hb * 16 + t / 2];
                const float xv = (t & 1) ? hi_f32(xpair) : lo_f32(xpair);
                const float val = code_value<BITS>(codes[t], expo[c]);
                const bool k = !SPARSE || ((keep >> t) & 1u);
                acc[c] += k ? xv * val : 0.f;
                if (SPARSE) xs[c] += k ? xv : 0.f;
            }
        }
    }
}

// Fast int4 path.  Word bits: code j at 4j.  Pairs (j, j+4) sit at equal offsets
// in the two halves of the word; offsets 0 and 4 are inside the fp16 mantissa, so
//   (w & 0x000F000F) | 0x64006400 = {1024 + q0, 1024 + q4}
//   (w & 0x00F000F0) | 0x54005400 = {  64 + q1,   64 + q5}
// and the same two masks on w >> 8 give (q2,q6) and (q3,q7).  Returns
// sum_k x_k (q_k + off_k) for the 4 columns, off_k = 1024 (k even) or 64 (k odd).
__device__ __forceinline__ void unit_fast_int4(const Unit<4, false>& u, const_u32p xw, float acc[4]) {
    const uint32_t M0 = 0x000F000Fu, M1 = 0x00F000F0u, G0 = 0x64006400u, G1 = 0x54005400u;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = 0.f;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        const uint32_t x01 = xw[4 * r], x23 = xw[4 * r + 1], x45 = xw[4 * r + 2], x67 = xw[4 * r + 3];
        const uint32_t p04 = pack_lo(x01, x45), p15 = pack_hi(x01, x45);
        const uint32_t p26 = pack_lo(x23, x67), p37 = pack_hi(x23, x67);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w = u.w[r][c], w8 = w >> 8;
            acc[c] = dot2((w & M0) | G0, p04, acc[c]);
            acc[c] = dot2((w & M1) | G1, p15, acc[c]);
            acc[c] = dot2((w8 & M0) | G0, p26, acc[c]);
            acc[c] = dot2((w8 & M1) | G1, p37, acc[c]);
        }
    }
}

// Fast int2 path.  Word bits: code j at 2j, 16 codes.  Pairs (j, j+8) share an
// offset; offsets 0,2,4,6,8 fit the mantissa (magic 2^(10-o)), the remaining
// codes 5,6,7 / 13,14,15 come down to offsets 0,2,4 after a shift by 10.
// off_k by k mod 8: 1024, 256, 64, 16, 4, 1024, 256, 64.
__device__ __forceinline__ void unit_fast_int2(const Unit<2, false>& u, const_u32p xw, float acc[4]) {
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        uint32_t p[8];                                   // p[j] = {x_j, x_{j+8}}
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const uint32_t a = xw[8 * r + j / 2], b = xw[8 * r + 4 + j / 2];
            p[j] = (j & 1) ? pack_hi(a, b) : pack_lo(a, b);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t w = u.w[r][c], w10 = w >> 10;
            acc[c] = dot2((w & 0x00030003u) | 0x64006400u, p[0], acc[c]);
            acc[c] = dot2((w & 0x000C000Cu) | 0x5C005C00u, p[1], acc[c]);
            acc[c] = dot2((w & 0x00300030u) | 0x54005400u, p[2], acc[c]);
            acc[c] = dot2((w & 0x00C000C0u) | 0x4C004C00u, p[3], acc[c]);
            acc[c] = dot2((w & 0x03000300u) | 0x44004400u, p[4], acc[c]);
            acc[c] = dot2((w10 & 0x00030003u) | 0x64006400u, p[5], acc[c]);
            acc[c] = dot2((w10 & 0x000C000Cu) | 0x5C005C00u, p[6], acc[c]);
            acc[c] = dot2((w10 & 0x00300030u) | 0x54005400u, p[7], acc[c]);
        }
    }
}

template <int BITS, bool SPARSE> struct FastPath { static constexpr bool HAS = false; };
template <> struct FastPath<4, false> { static constexpr bool HAS = true; };
template <> struct FastPath<2, false> { static constexpr bool HAS = true; };

// magic offset of row k (k = index inside the unit) on the fast paths
template <int BITS>
__device__ __forceinline__ float fast_offset(int k) {
    if constexpr (BITS == 4) return (k & 1) ? 64.f : 1024.f;
    const int j = k & 7;
    const int o = 2 * (j < 5 ? j : j - 5);
    return (float)(1024 >> o);
}

// One unit: y[c] += contribution of 64 rows to the lane's 4 columns.
template <int BITS, bool SPARSE>
__device__ __forceinline__ void process_unit(const Unit<BITS, SPARSE>& u, const MatvecArgs& a,
                                             int unit, int lane, float y[4]) {
    const_u32p xw = to_const(a.x) + unit * 32;           // 64 halves, wave-uniform
    const h16x2 s01 = as_h2(u.sc.x), s23 = as_h2(u.sc.y);
    const h16x2 z01 = as_h2(u.ze.x), z23 = as_h2(u.ze.y);
    const float sc[4] = {(float)s01.x, (float)s01.y, (float)s23.x, (float)s23.y};
    const float ze[4] = {(float)z01.x, (float)z01.y, (float)z23.x, (float)z23.y};
    const bool expo[4] = {!(sc[0] >= 0.f), !(sc[1] >= 0.f), !(sc[2] >= 0.f), !(sc[3] >= 0.f)};
    const bool any_expo = __builtin_amdgcn_ballot_w64(expo[0] | expo[1] | expo[2] | expo[3]) != 0;

    const float xsum = SPARSE ? 0.f : wave_sum(u.xl);    // sum of the unit's 64 states
    float acc[4], xs[4];
    bool fast = false;
    if constexpr (FastPath<BITS, SPARSE>::HAS) {
        if (!any_expo) {
            fast = true;
            const float off = wave_sum(u.xl * fast_offset<BITS>(lane));
            if constexpr (BITS == 4) unit_fast_int4(u, xw, acc);
            else unit_fast_int2(u, xw, acc);
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[c] -= off;
        }
    }
    if (!fast) unit_generic<BITS, SPARSE>(u, xw, expo, acc, xs);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float xc = SPARSE ? xs[c] : xsum;
        // linear: s * (acc - z * X)      exponent: (-s) * acc + z * X
        const float lin = sc[c] * (acc[c] - ze[c] * xc);
        const float ex = ze[c] * xc - sc[c] * acc[c];
        y[c] += expo[c] ? ex : lin;
    }
}

template <int BITS, bool SPARSE>
__global__ __launch_bounds__(MV_MAX_WAVES * WAVE) void matvec_kernel(MatvecArgs a) {
    __shared__ float red[MV_MAX_WAVES][MV_COLS];
    __shared__ int is_last;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int strip = blockIdx.x, split = blockIdx.y;
    const int col = strip * MV_COLS + lane * 4;
    const bool col_ok = col < a.S;

    const int u_begin = (split * nwaves + wave) * a.units_per_wave;
    const int u_end = min(u_begin + a.units_per_wave, a.units_total);

    float y[4] = {0.f, 0.f, 0.f, 0.f};
    if (u_begin < u_end) {
        Unit<BITS, SPARSE> ua, ub;
        load_unit(ua, a, u_begin, col, col_ok, lane);
        for (int u = u_begin; u < u_end; u += 2) {
            const bool has_b = u + 1 < u_end;
            if (has_b) load_unit(ub, a, u + 1, col, col_ok, lane);
            process_unit(ua, a, u, lane, y);
            if (has_b) {
                if (u + 2 < u_end) load_unit(ua, a, u + 2, col, col_ok, lane);
                process_unit(ub, a, u + 1, lane, y);
            }
        }
    }

    // ---- workgroup reduction through LDS
    *reinterpret_cast<f32x4*>(&red[wave][lane * 4]) = f32x4{y[0], y[1], y[2], y[3]};
    __syncthreads();
    const int t = threadIdx.x;
    float total = 0.f;
    const int ocol = strip * MV_COLS + t;
    const bool owner = t < MV_COLS && ocol < a.S;
    if (owner) {
        for (int w = 0; w < nwaves; ++w) total += red[w][t];
    }
    if (a.splits == 1) {
        if (owner) a.outs[ocol] = (h16)((float)a.outs[ocol] + total);
        return;
    }

    // ---- across workgroups: fp32 slot per split, last arrival finishes
    if (owner) a.partials[(int64_t)split * a.S + ocol] = total;
    __threadfence();
    __syncthreads();
    if (t == 0) {
        const int prev = __hip_atomic_fetch_add(&a.counters[strip], 1, __ATOMIC_ACQ_REL,
                                                __HIP_MEMORY_SCOPE_AGENT);
        is_last = prev == a.splits - 1;
    }
    __syncthreads();
    if (!is_last) return;
    __threadfence();
    if (owner) {
        float sum = 0.f;
        for (int sp = 0; sp < a.splits; ++sp)
            sum += __builtin_nontemporal_load(&a.partials[(int64_t)sp * a.S + ocol]);
        a.outs[ocol] = (h16)((float)a.outs[ocol] + sum);
    }
    if (t == 0) a.counters[strip] = 0;                    // ready for the next call
}

template <int BITS, bool SPARSE>
static void launch(const MatvecArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    hipLaunchKernelGGL((matvec_kernel<BITS, SPARSE>), grid, block, 0, st, a);
}

}  // namespace i4

using namespace i4;

extern "C" int int4mm_matvec(int bits, void* outs, const void* matrix, const void* multiplier,
                             const void* scales, const void* zeros, const void* sparse_mask,
                             const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                             void* stream) {
    int rc = validate_product(bits, outs, matrix, multiplier, scales, zeros, sparse_mask, shape, true);
    if (rc != INT4MM_OK) return rc;
    const int64_t B = shape->batch, K = shape->in_size, S = shape->out_size;
    if (B * shape->seq_len * S == 0) return INT4MM_OK;

    const int units_total = (int)(K / 64);
    const int strips = (int)((S + MV_COLS - 1) / MV_COLS);
    const int64_t g = shape->group_size < 0 ? ONE_GROUP : shape->group_size;

    // Work split: aim for ~16 resident waves on each of the 256 CUs.
    int waves = (int)tuning(TUNE_MV_WAVES), upw = (int)tuning(TUNE_MV_UNITS);
    if (upw <= 0) {
        const int64_t want_waves = 256 * 12;
        int64_t per_strip = (want_waves + strips - 1) / strips;
        upw = (int)((units_total + per_strip - 1) / per_strip);
        if (upw < 1) upw = 1;
    }
    if (waves <= 0) waves = 4;
    if (waves > MV_MAX_WAVES) waves = MV_MAX_WAVES;
    int runs = (units_total + upw - 1) / upw;             // wave-sized runs along K
    if (waves > runs) waves = runs;
    int splits = (runs + waves - 1) / waves;
    if (splits > MV_MAX_SPLITS) {                          // keep the slot count bounded
        splits = MV_MAX_SPLITS;
        upw = (units_total + splits * waves - 1) / (splits * waves);
        runs = (units_total + upw - 1) / upw;
        splits = (runs + waves - 1) / waves;
    }
    if (splits > 1) {
        if (workspace == nullptr || workspace_bytes < int4mm_workspace_bytes(S))
            return INT4MM_ERR_WORKSPACE;
        if (strips * 4 > 4096) return INT4MM_ERR_SHAPE;
    }

    MatvecArgs a;
    a.matrix = (const uint32_t*)matrix;
    a.mask = (const uint32_t*)sparse_mask;
    a.scales = (const h16*)scales;
    a.zeros = (const h16*)zeros;
    a.counters = (int*)workspace;
    a.partials = workspace ? (float*)((char*)workspace + 4096) : nullptr;
    a.K = (int)K;
    a.S = (int)S;
    a.units_total = units_total;
    a.units_per_wave = upw;
    a.group_units = (int)(g / 64 > 0x7FFFFFF ? 0x7FFFFFF : g / 64);
    a.splits = splits;

    const dim3 grid(strips, splits, 1), block(waves * WAVE);
    hipStream_t st = (hipStream_t)stream;
    for (int64_t b = 0; b < B; ++b) {                      // one pass over the weights per batch row
        a.outs = (h16*)outs + b * S;
        a.x = (const h16*)multiplier + b * K;
        if (sparse_mask) launch<4, true>(a, grid, block, st);
        else if (bits == 4) launch<4, false>(a, grid, block, st);
        else if (bits == 3) launch<3, false>(a, grid, block, st);
        else launch<2, false>(a, grid, block, st);
        rc = check_launch("matvec");
        if (rc != INT4MM_OK) return rc;
    }
    return INT4MM_OK;
}
