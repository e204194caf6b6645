// Quantized matrix-matrix product for gfx950:
//     outs[m, s] = fp16( sum_k fp32(x[m, k]) * fp32(w16[k, s]) )
// where w16 is the fp16 matrix the reference's unpack step builds (two fp16
// roundings per weight in linear mode, one fused multiply-add in exponent mode).
//
// One workgroup owns a BM x BN tile of outs and walks K in steps of 64.  Per
// step the packed weights of the tile (64 x BN codes) are read from HBM once,
// decoded and dequantised to fp16 ONCE by the workgroup (2 threads per column,
// one 32-row block each) and stored to LDS in the operand layout of
// v_mfma_f32_32x32x16_f16: 16-byte chunks of 8 consecutive k for one column,
// chunk (kc, n) at kc*BN + n, which both the writes (lanes along n) and the MFMA
// operand reads (lanes along n) touch without bank conflicts.  The states tile
// (BM x 64 fp16) is stored row-major with an XOR swizzle of the chunk index so
// that row-contiguous writes and column-of-rows operand reads are both
// conflict-free.  Accumulation is fp32 in the MFMA accumulators.
#include "common.h"

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
};

// Raw packed data of one (32-row block, column) cell
template <int BITS, bool SPARSE>
struct Cell {
    uint32_t w[SPARSE ? 2 : BITS];
    uint32_t m;
    h16 sc, ze;
};

template <int BITS, bool SPARSE>
__device__ __forceinline__ void load_cell(Cell<BITS, SPARSE>& c, const MatmulArgs& a, int blk, int col) {
    constexpr int ROWS = SPARSE ? 2 : BITS;
    const int64_t S = a.S;
    const uint32_t* p = a.matrix + (int64_t)blk * ROWS * S + col;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) c.w[r] = p[r * S];
    c.m = SPARSE ? a.mask[(int64_t)blk * S + col] : 0xFFFFFFFFu;
    const int64_t gofs = (int64_t)((blk >> 1) / a.group_units) * S + col;
    c.sc = a.scales[gofs];
    c.ze = a.zeros[gofs];
}

// Cell -> 32 fp16 weights = 4 chunks of 8, bit-exact with the reference decode
template <int BITS, bool SPARSE>
__device__ __forceinline__ void dequant_cell(const Cell<BITS, SPARSE>& c, h16x8 out[4]) {
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
        h16 w = dequant_code<BITS>(codes[t], c.sc, c.ze);
        if (SPARSE && !((c.m >> t) & 1u)) w = (h16)0.0f;
        out[t >> 3][t & 7] = w;
    }
}

template <int BITS, bool SPARSE, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(2 * BN) void matmul_kernel(MatmulArgs a) {
    constexpr int T = 2 * BN;                     // threads: two per tile column
    constexpr int WAVES_N = BN / WN, WAVES_M = BM / WM;
    static_assert(WAVES_M * WAVES_N * 64 == T, "wave grid must match the thread count");
    constexpr int TM = WM / 32, TN = WN / 32;     // MFMA tiles per wave
    constexpr int A_CHUNKS = BM * 8 / T;          // 16-byte chunks of the states tile per thread
    static_assert(BM * 8 % T == 0, "states tile must divide among the threads");

    __shared__ __attribute__((aligned(16))) h16 As[BM * BK];
    __shared__ __attribute__((aligned(16))) h16 Bs[BK * BN];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int m0 = blockIdx.y * BM, s0 = blockIdx.x * BN;
    const int64_t boff = blockIdx.z;
    const h16* x = a.x + boff * a.M * (int64_t)a.K;
    h16* outs = a.outs + boff * a.M * (int64_t)a.S;

    // B loader: column n, 32-row block hb of the K step
    const int bn = t % BN, bhb = t / BN;
    const int bcol = min(s0 + bn, a.S - 1);

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    u32x4 areg[A_CHUNKS];
    Cell<BITS, SPARSE> cell;

    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = t + T * i, m = c >> 3, kc = c & 7;
            const int row = min(m0 + m, a.M - 1);
            areg[i] = *reinterpret_cast<const u32x4*>(x + (int64_t)row * a.K + kt * BK + kc * 8);
        }
        load_cell<BITS, SPARSE>(cell, a, kt * 2 + bhb, bcol);
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
        {
            h16x8 w[4];
            dequant_cell<BITS, SPARSE>(cell, w);
#pragma unroll
            for (int q = 0; q < 4; ++q)
                *reinterpret_cast<h16x8*>(&Bs[((bhb * 4 + q) * BN + bn) * 8]) = w[q];
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

template <int BITS, bool SPARSE>
static void launch(const MatmulArgs& a, int64_t B, hipStream_t st) {
    constexpr int BM = 128, BN = 128;
    const dim3 grid((a.S + BN - 1) / BN, (a.M + BM - 1) / BM, (unsigned)B), block(2 * BN);
    hipLaunchKernelGGL((matmul_kernel<BITS, SPARSE, BM, BN, 64, 64>), grid, block, 0, st, a);
}

}  // namespace i4

using namespace i4;

extern "C" int int4mm_matmul(int bits, void* outs, const void* matrix, const void* multiplier,
                             const void* scales, const void* zeros, const void* sparse_mask,
                             const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                             void* stream) {
    (void)workspace; (void)workspace_bytes;
    int rc = validate_product(bits, outs, matrix, multiplier, scales, zeros, sparse_mask, shape, false);
    if (rc != INT4MM_OK) return rc;
    const int64_t B = shape->batch, M = shape->seq_len, K = shape->in_size, S = shape->out_size;
    if (B * M * S == 0) return INT4MM_OK;
    if ((M + 127) / 128 > 65535) return INT4MM_ERR_SHAPE;
    const int64_t g = shape->group_size < 0 ? ONE_GROUP : shape->group_size;

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

    hipStream_t st = (hipStream_t)stream;
    if (sparse_mask) launch<4, true>(a, B, st);
    else if (bits == 4) launch<4, false>(a, B, st);
    else if (bits == 3) launch<3, false>(a, B, st);
    else launch<2, false>(a, B, st);
    return check_launch("matmul");
}
