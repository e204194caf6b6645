// Pack / unpack / dequantise helpers for the packed weight formats.  These are
// integer kernels bound by HBM traffic: one thread owns one (32-row block,
// column) cell, lanes run along the column index so every global access of the
// [rows, S] matrices is coalesced.
#include "common.h"

namespace i4 {

// 32 codes of one column, blocks of 32 rows: the shared decode step.
template <int BITS, bool SPARSE>
__device__ __forceinline__ void decode_block32(const uint32_t* __restrict__ matrix,
                                               const uint32_t* __restrict__ mask, int64_t S,
                                               int64_t blk, int64_t s, uint32_t codes[32],
                                               uint32_t& keep) {
    keep = 0xFFFFFFFFu;
    if constexpr (SPARSE) {
        const uint32_t lo = matrix[(2 * blk) * S + s], hi = matrix[(2 * blk + 1) * S + s];
        uint64_t v = (uint64_t)lo | ((uint64_t)hi << 32);
        keep = mask[blk * S + s];
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            const bool k = (keep >> t) & 1u;
            codes[t] = k ? (uint32_t)(v & 0xF) : 0u;
            v >>= k ? 4 : 0;
        }
    } else if constexpr (BITS == 3) {
        const uint32_t w0 = matrix[(3 * blk) * S + s], w1 = matrix[(3 * blk + 1) * S + s],
                       w2 = matrix[(3 * blk + 2) * S + s];
        const uint64_t lo = (uint64_t)w0 | ((uint64_t)w1 << 32);   // stream bits 0..63
        const uint64_t hi = (uint64_t)w1 | ((uint64_t)w2 << 32);   // stream bits 32..95
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            const int pos = 3 * t;
            codes[t] = pos + 3 <= 64 ? (uint32_t)(lo >> pos) & 7u : (uint32_t)(hi >> (pos - 32)) & 7u;
        }
    } else {
        constexpr int PER = 32 / BITS;
#pragma unroll
        for (int i = 0; i < BITS; ++i) {
            uint32_t v = matrix[(BITS * blk + i) * S + s];
#pragma unroll
            for (int j = 0; j < PER; ++j) {
                codes[i * PER + j] = v & ((1u << BITS) - 1u);
                v >>= BITS;
            }
        }
    }
}

template <int BITS, bool SPARSE>
__global__ __launch_bounds__(256) void unpack_kernel(uint8_t* __restrict__ codes_out,
                                                     uint8_t* __restrict__ keep_out,
                                                     const uint32_t* __restrict__ matrix,
                                                     const uint32_t* __restrict__ mask, int64_t K,
                                                     int64_t S) {
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, blk = blockIdx.y;
    if (s >= S) return;
    uint32_t codes[32], keep;
    decode_block32<BITS, SPARSE>(matrix, mask, S, blk, s, codes, keep);
#pragma unroll
    for (int t = 0; t < 32; ++t) {
        codes_out[(blk * 32 + t) * S + s] = (uint8_t)codes[t];
        if (keep_out) keep_out[(blk * 32 + t) * S + s] = (uint8_t)((keep >> t) & 1u);
    }
}

// The same for four adjacent columns per thread (S a multiple of 4): a row's four codes leave as one 32-bit
// store, a wave's store is 256 contiguous bytes of a row instead of 64 (K = S = 16384, int4: 87 -> 76 us).
template <int BITS, bool SPARSE>
__global__ __launch_bounds__(256) void unpack4_kernel(uint8_t* __restrict__ codes_out,
                                                      uint8_t* __restrict__ keep_out,
                                                      const uint32_t* __restrict__ matrix,
                                                      const uint32_t* __restrict__ mask, int64_t K,
                                                      int64_t S) {
    const int64_t s = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4, blk = blockIdx.y;
    if (s >= S) return;
    uint32_t out[32], kept[32];
#pragma unroll
    for (int t = 0; t < 32; ++t) { out[t] = 0u; kept[t] = 0u; }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        uint32_t codes[32], keep;
        decode_block32<BITS, SPARSE>(matrix, mask, S, blk, s + c, codes, keep);
#pragma unroll
        for (int t = 0; t < 32; ++t) {
            out[t] |= (codes[t] & 0xFFu) << (8 * c);
            kept[t] |= ((keep >> t) & 1u) << (8 * c);
        }
    }
#pragma unroll
    for (int t = 0; t < 32; ++t) {
        *reinterpret_cast<uint32_t*>(codes_out + (blk * 32 + t) * S + s) = out[t];
        if (keep_out) *reinterpret_cast<uint32_t*>(keep_out + (blk * 32 + t) * S + s) = kept[t];
    }
}

template <int BITS, bool SPARSE>
__global__ __launch_bounds__(256) void dequantize_kernel(h16* __restrict__ w_out,
                                                         const uint32_t* __restrict__ matrix,
                                                         const uint32_t* __restrict__ mask,
                                                         const h16* __restrict__ scales,
                                                         const h16* __restrict__ zeros, int64_t K,
                                                         int64_t S, int64_t group_size) {
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, blk = blockIdx.y;
    if (s >= S) return;
    uint32_t codes[32], keep;
    decode_block32<BITS, SPARSE>(matrix, mask, S, blk, s, codes, keep);
    const int64_t gi = (blk * 32) / group_size;      // group_size is a multiple of 64
    const h16 sc = scales[gi * S + s], ze = zeros[gi * S + s];
#pragma unroll
    for (int t = 0; t < 32; ++t) {
        h16 w = dequant_code<BITS>(codes[t], sc, ze);
        if (SPARSE && !((keep >> t) & 1u)) w = (h16)0.0f;
        w_out[(blk * 32 + t) * S + s] = w;
    }
}

// codes uint8 [K, S] -> packed words, LSB-first bitstream of 32 codes per block
template <int BITS>
__global__ __launch_bounds__(256) void dense_pack_kernel(uint32_t* __restrict__ matrix_out,
                                                         const uint8_t* __restrict__ codes_in,
                                                         int64_t K, int64_t S) {
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, blk = blockIdx.y;
    if (s >= S) return;
    uint64_t lo = 0, hi = 0;                          // stream bits 0..63 and 64..127
#pragma unroll
    for (int t = 0; t < 32; ++t) {
        const uint64_t c = codes_in[(blk * 32 + t) * S + s] & ((1u << BITS) - 1u);
        const int pos = BITS * t;
        if (pos < 64) {
            lo |= c << pos;
            if (pos + BITS > 64) hi |= c >> (64 - pos);
        } else {
            hi |= c << (pos - 64);
        }
    }
    const uint32_t w[4] = {(uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32)};
#pragma unroll
    for (int i = 0; i < BITS; ++i) matrix_out[(BITS * blk + i) * S + s] = w[i];
}

// 16:32 packer.  Inputs are in the [S, K] orientation (row = output column): a thread takes four
// consecutive 32-row cells of its column -- the 128 consecutive bytes of a whole cache line of each
// input -- compacts the kept codes eight rows at a time (keep flags gathered by a multiply, code bytes moved to
// the front by v_perm with selectors from a 256-entry table, squeezed to nibbles) and writes three words per cell
// with lanes along the column index.  K = S = 16384: 180 us with one cell per thread and a 32-step loop per cell,
// 174 with whole lines, 165 with this compaction; staging a 64-column tile through LDS so that a wave reads whole
// 256-byte runs changed nothing (173 against 174) -- what remains is the transposition: a wave's 64 lanes read
// lines K bytes apart.
constexpr int SPARSE_PACK_CELLS = 4;
__global__ __launch_bounds__(256) void sparse_pack_kernel(uint32_t* __restrict__ wt_outs,
                                                          uint32_t* __restrict__ msk_outs,
                                                          const uint8_t* __restrict__ wt_in,
                                                          const uint8_t* __restrict__ msk_in,
                                                          int64_t S, int64_t K,
                                                          int* __restrict__ bad_blocks) {
    // compaction table: for a byte of eight keep flags, the v_perm selectors that move the kept rows' code bytes to
    // the front in row order (0 ... 7: that row of the eight; 0x0C: a zero byte)
    __shared__ u32x2 front[256];
    {
        uint32_t sel[2] = {0x0C0C0C0Cu, 0x0C0C0C0Cu};
        int p = 0;
        for (int r = 0; r < 8; ++r)
            if ((threadIdx.x >> r) & 1u) {
                sel[p >> 2] = (sel[p >> 2] & ~(0xFFu << (8 * (p & 3)))) | ((uint32_t)r << (8 * (p & 3)));
                ++p;
            }
        front[threadIdx.x] = u32x2{sel[0], sel[1]};
    }
    __syncthreads();
    const int64_t s = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, blk0 = (int64_t)blockIdx.y * SPARSE_PACK_CELLS;
    if (s >= S) return;
    const int64_t cells = K / 32;
    u32x4 wq[SPARSE_PACK_CELLS][2], mq[SPARSE_PACK_CELLS][2];
#pragma unroll
    for (int i = 0; i < SPARSE_PACK_CELLS; ++i) {
        if (blk0 + i >= cells) break;
        const u32x4* wp = reinterpret_cast<const u32x4*>(wt_in + s * K + (blk0 + i) * 32);
        const u32x4* mp = reinterpret_cast<const u32x4*>(msk_in + s * K + (blk0 + i) * 32);
        wq[i][0] = wp[0]; wq[i][1] = wp[1]; mq[i][0] = mp[0]; mq[i][1] = mp[1];
    }
    // keep flags of four rows (bytes > 0) as four bits: the top bit of every non-zero byte, gathered by a multiply
    auto flags4 = [](uint32_t m) {
        const uint32_t nz = ((((m & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | m) & 0x80808080u) >> 7;
        return ((nz * 0x00204081u) >> 21) & 0xFu;
    };
    // four code bytes (each at most 15) to four nibbles
    auto nibbles4 = [](uint32_t o) {
        const uint32_t n = (o | (o >> 4)) & 0x00FF00FFu;
        return (n | (n >> 8)) & 0xFFFFu;
    };
    int bad = 0;
#pragma unroll
    for (int i = 0; i < SPARSE_PACK_CELLS; ++i) {
        const int64_t blk = blk0 + i;
        if (blk >= cells) break;
        const uint32_t wv[8] = {wq[i][0].x, wq[i][0].y, wq[i][0].z, wq[i][0].w, wq[i][1].x, wq[i][1].y, wq[i][1].z, wq[i][1].w};
        const uint32_t mv[8] = {mq[i][0].x, mq[i][0].y, mq[i][0].z, mq[i][0].w, mq[i][1].x, mq[i][1].y, mq[i][1].z, mq[i][1].w};
        uint32_t bmsk = 0;
        uint64_t v = 0;
        int rank = 0;
#pragma unroll
        for (int g8 = 0; g8 < 4; ++g8) {                            // eight rows at a time
            const uint32_t m8 = flags4(mv[2 * g8]) | (flags4(mv[2 * g8 + 1]) << 4);
            const u32x2 sel = front[m8];
            const uint32_t clo = wv[2 * g8] & 0x0F0F0F0Fu, chi = wv[2 * g8 + 1] & 0x0F0F0F0Fu;
            const uint32_t kept = nibbles4(__builtin_amdgcn_perm(chi, clo, sel.x)) |
                                  (nibbles4(__builtin_amdgcn_perm(chi, clo, sel.y)) << 16);
            bmsk |= m8 << (8 * g8);
            if (rank < 16) v |= (uint64_t)kept << (4 * rank);       // (codes beyond the sixteenth fall off the top)
            rank += __builtin_popcount(m8);
        }
        msk_outs[blk * S + s] = bmsk;
        wt_outs[(2 * blk) * S + s] = (uint32_t)v;
        wt_outs[(2 * blk + 1) * S + s] = (uint32_t)(v >> 32);
        bad += rank != 16;
    }
    if (bad && bad_blocks) atomicAdd(bad_blocks, bad);
}

static dim3 cell_grid(int64_t S, int64_t K) { return dim3((unsigned)((S + 255) / 256), (unsigned)(K / 32)); }

}  // namespace i4

using namespace i4;

extern "C" {

int int4mm_sparse_pack(void* wt_outs, void* msk_outs, const void* wt_in, const void* msk_in,
                       int64_t out_size, int64_t in_size, void* bad_blocks, void* stream) {
    if (out_size < 0 || in_size < 0 || in_size % 32 != 0) return INT4MM_ERR_SHAPE;
    if (in_size / 32 > 65535) return INT4MM_ERR_SHAPE;
    if (out_size == 0 || in_size == 0) return INT4MM_OK;
    if (!wt_outs || !msk_outs || !wt_in || !msk_in) return INT4MM_ERR_NULL;
    if (((uintptr_t)wt_in | (uintptr_t)msk_in) & 15u) return INT4MM_ERR_ALIGN;
    const dim3 grid((unsigned)((out_size + 255) / 256), (unsigned)((in_size / 32 + SPARSE_PACK_CELLS - 1) / SPARSE_PACK_CELLS));
    hipLaunchKernelGGL(sparse_pack_kernel, grid, dim3(256), 0,
                       (hipStream_t)stream, (uint32_t*)wt_outs, (uint32_t*)msk_outs,
                       (const uint8_t*)wt_in, (const uint8_t*)msk_in, out_size, in_size,
                       (int*)bad_blocks);
    return check_launch("sparse_pack");
}

int int4mm_dense_pack(int bits, void* matrix_out, const void* codes_in, int64_t in_size,
                      int64_t out_size, void* stream) {
    if (bits != 4 && bits != 3 && bits != 2) return INT4MM_ERR_BITS;
    if (out_size < 0 || in_size < 0 || in_size % 32 != 0 || in_size / 32 > 65535)
        return INT4MM_ERR_SHAPE;
    if (out_size == 0 || in_size == 0) return INT4MM_OK;
    if (!matrix_out || !codes_in) return INT4MM_ERR_NULL;
    const dim3 grid = cell_grid(out_size, in_size), block(256);
    hipStream_t st = (hipStream_t)stream;
    uint32_t* o = (uint32_t*)matrix_out;
    const uint8_t* c = (const uint8_t*)codes_in;
    if (bits == 4) hipLaunchKernelGGL(dense_pack_kernel<4>, grid, block, 0, st, o, c, in_size, out_size);
    if (bits == 3) hipLaunchKernelGGL(dense_pack_kernel<3>, grid, block, 0, st, o, c, in_size, out_size);
    if (bits == 2) hipLaunchKernelGGL(dense_pack_kernel<2>, grid, block, 0, st, o, c, in_size, out_size);
    return check_launch("dense_pack");
}

int int4mm_unpack(int bits, void* codes_out, void* keep_out, const void* matrix,
                  const void* sparse_mask, int64_t in_size, int64_t out_size, void* stream) {
    if (bits != 4 && bits != 3 && bits != 2) return INT4MM_ERR_BITS;
    if (sparse_mask && bits != 4) return INT4MM_ERR_SPARSE_BITS;
    if (out_size < 0 || in_size < 0 || in_size % 32 != 0 || in_size / 32 > 65535)
        return INT4MM_ERR_SHAPE;
    if (out_size == 0 || in_size == 0) return INT4MM_OK;
    if (!codes_out || !matrix) return INT4MM_ERR_NULL;
    const dim3 grid = cell_grid(out_size, in_size), block(256);
    hipStream_t st = (hipStream_t)stream;
    uint8_t* o = (uint8_t*)codes_out;
    uint8_t* k = (uint8_t*)keep_out;
    const uint32_t* m = (const uint32_t*)matrix;
    const uint32_t* msk = (const uint32_t*)sparse_mask;
    if (out_size % 4 == 0 && (((uintptr_t)codes_out | (uintptr_t)keep_out) & 3u) == 0) {
        const dim3 grid4((unsigned)((out_size / 4 + 255) / 256), grid.y);
        if (msk) hipLaunchKernelGGL((unpack4_kernel<4, true>), grid4, block, 0, st, o, k, m, msk, in_size, out_size);
        else if (bits == 4) hipLaunchKernelGGL((unpack4_kernel<4, false>), grid4, block, 0, st, o, k, m, msk, in_size, out_size);
        else if (bits == 3) hipLaunchKernelGGL((unpack4_kernel<3, false>), grid4, block, 0, st, o, k, m, msk, in_size, out_size);
        else hipLaunchKernelGGL((unpack4_kernel<2, false>), grid4, block, 0, st, o, k, m, msk, in_size, out_size);
        return check_launch("unpack");
    }
    if (msk) hipLaunchKernelGGL((unpack_kernel<4, true>), grid, block, 0, st, o, k, m, msk, in_size, out_size);
    else if (bits == 4) hipLaunchKernelGGL((unpack_kernel<4, false>), grid, block, 0, st, o, k, m, msk, in_size, out_size);
    else if (bits == 3) hipLaunchKernelGGL((unpack_kernel<3, false>), grid, block, 0, st, o, k, m, msk, in_size, out_size);
    else hipLaunchKernelGGL((unpack_kernel<2, false>), grid, block, 0, st, o, k, m, msk, in_size, out_size);
    return check_launch("unpack");
}

int int4mm_dequantize(int bits, void* w_out, const void* matrix, const void* scales,
                      const void* zeros, const void* sparse_mask, int64_t in_size,
                      int64_t out_size, int64_t n_groups, int64_t group_size, void* stream) {
    if (bits != 4 && bits != 3 && bits != 2) return INT4MM_ERR_BITS;
    if (sparse_mask && bits != 4) return INT4MM_ERR_SPARSE_BITS;
    if (out_size < 0 || in_size < 0 || in_size % 64 != 0 || in_size / 32 > 65535 || n_groups <= 0)
        return INT4MM_ERR_SHAPE;
    if (group_size == 0 || (group_size > 0 && group_size % 64 != 0)) return INT4MM_ERR_GROUP;
    const int64_t g = group_size < 0 ? ONE_GROUP : group_size;
    if (n_groups > ((int64_t)1 << 40) || g * n_groups < in_size) return INT4MM_ERR_SHAPE;
    if (out_size == 0 || in_size == 0) return INT4MM_OK;
    if (!w_out || !matrix || !scales || !zeros) return INT4MM_ERR_NULL;
    const dim3 grid = cell_grid(out_size, in_size), block(256);
    hipStream_t st = (hipStream_t)stream;
    h16* o = (h16*)w_out;
    const uint32_t* m = (const uint32_t*)matrix;
    const uint32_t* msk = (const uint32_t*)sparse_mask;
    const h16* sc = (const h16*)scales;
    const h16* ze = (const h16*)zeros;
    if (msk) hipLaunchKernelGGL((dequantize_kernel<4, true>), grid, block, 0, st, o, m, msk, sc, ze, in_size, out_size, g);
    else if (bits == 4) hipLaunchKernelGGL((dequantize_kernel<4, false>), grid, block, 0, st, o, m, msk, sc, ze, in_size, out_size, g);
    else if (bits == 3) hipLaunchKernelGGL((dequantize_kernel<3, false>), grid, block, 0, st, o, m, msk, sc, ze, in_size, out_size, g);
    else hipLaunchKernelGGL((dequantize_kernel<2, false>), grid, block, 0, st, o, m, msk, sc, ze, in_size, out_size, g);
    return check_launch("dequantize");
}

}  // extern "C"
