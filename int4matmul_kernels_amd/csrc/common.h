// Shared device helpers for the gfx950 kernels: fp16 vector types, wave-level
// reductions, the bit-exact dequantisation of one code, and host-side launch
// bookkeeping.  Written for 64-lane wavefronts only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/int4mm.h"

namespace i4 {

typedef _Float16 h16;
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;
constexpr int64_t ONE_GROUP = 0x0FFFFFFF;   // group_size < 0: a single group

template <typename To, typename From>
__device__ __forceinline__ To bitcast(From v) { return __builtin_bit_cast(To, v); }

__device__ __forceinline__ h16x2 as_h2(uint32_t v) { return bitcast<h16x2>(v); }
__device__ __forceinline__ uint32_t as_u32(h16x2 v) { return bitcast<uint32_t>(v); }
__device__ __forceinline__ float lo_f32(uint32_t v) { return (float)as_h2(v).x; }
__device__ __forceinline__ float hi_f32(uint32_t v) { return (float)as_h2(v).y; }

// acc + a.x*b.x + a.y*b.y with an fp32 accumulator (v_dot2_f32_f16)
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), acc, false);
}

// ---- wave-wide sum through DPP: quad swaps, half-row and row mirrors, then the
// four row totals are combined from lanes 0/16/32/48.  Every lane gets the total.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return bitcast<float>(__builtin_amdgcn_update_dpp(0, bitcast<int>(v), CTRL, 0xF, 0xF, true));
}

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_f32<0xB1>(v);    // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);    // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);   // row_half_mirror
    v += dpp_f32<0x140>(v);   // row_mirror
    int b = bitcast<int>(v);
    float r0 = bitcast<float>(__builtin_amdgcn_readlane(b, 0));
    float r1 = bitcast<float>(__builtin_amdgcn_readlane(b, 16));
    float r2 = bitcast<float>(__builtin_amdgcn_readlane(b, 32));
    float r3 = bitcast<float>(__builtin_amdgcn_readlane(b, 48));
    return (r0 + r1) + (r2 + r3);
}

// (w & mask) | magic is one VALU op (v_and_or_b32) only when both constants sit in registers: a VOP3
// instruction of this ISA cannot carry two literals.  Such constants are materialised once through an
// opaque move, and the expression itself is left to the compiler (so that it also tracks the VALU -> MFMA
// operand hazards, which it cannot do through inline assembly).
__device__ __forceinline__ uint32_t in_vgpr(uint32_t literal) {
    uint32_t r;
    asm("v_mov_b32 %0, %1" : "=v"(r) : "s"(literal));
    return r;
}

// a / b for 0 <= a < 2^22, b >= 1 with b's magic number floor(2^32 / b) + 1 (2^32 - 1 for b = 1), which the host passes:
// the high word of the product is the quotient or one off -- eight integer instructions where the compiler's exact
// division by a run-time divisor takes ~35
__host__ __device__ inline uint32_t div_magic(uint32_t b) { return b <= 1 ? 0xFFFFFFFFu : (uint32_t)(0x100000000ull / b) + 1u; }
__host__ __device__ inline int magic_div(int a, int b, uint32_t magic) {
    int q = (int)(uint32_t)(((uint64_t)(uint32_t)a * magic) >> 32);
    if (q * b > a) --q;
    if ((q + 1) * b <= a) ++q;
    return q;
}

// ---- one code -> fp16 weight, the two roundings of the linear mode and the
// single-rounded fused multiply-add of the exponent mode.
template <int BITS>
__device__ __forceinline__ h16 dequant_code(uint32_t q, h16 scale, h16 zero) {
    if (scale >= (h16)0.0f) {
        h16 d = (h16)(float)q - zero;       // fp16 subtract, one rounding
        return d * scale;                    // fp16 multiply, one rounding
    }
    constexpr uint32_t EXP_MSK = (1u << (BITS - 1)) - 1u, SGN = 1u << (BITS - 1);
    int iv = 1 << (q & EXP_MSK);
    if (q & SGN) iv = -iv;
    return __builtin_fmaf16((h16)(float)iv, -scale, zero);
}

// Exponent quantisation on magic-number operands.  A magic-number pair {2^a | q << o, 2^b | q' << o'}
// holds its two codes inside the mantissas, at offsets o, o' with 2^(10 - o) = 2^a the half's magic
// offset; a packed 16-bit multiply by those offsets (`offsets` = 2^a | 2^b << 16, as integers)
// moves both codes to bits 10.. of their halves -- whatever the magic bits turn into lies above
// the code and is masked away.  The code's low BITS - 1 bits are then the exponent field's
// increment over 15 (2^0) and its top bit is the sign: the half becomes +-2^(code's low bits),
// the value the exponent mode multiplies by (matmul.cuh:127-136).
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
template <int BITS>
__device__ __forceinline__ uint32_t expo_operand(uint32_t h, uint32_t offsets) {
    const uint32_t m = bitcast<uint32_t>(bitcast<u16x2>(h) * bitcast<u16x2>(offsets));
    constexpr uint32_t E1 = ((1u << (BITS - 1)) - 1u) << 10, EMASK = E1 | (E1 << 16);
    const uint32_t magnitude = (m & EMASK) + 0x3C003C00u;
    return ((m << (6 - BITS)) & 0x80008000u) | magnitude;
}
__host__ __device__ constexpr uint32_t off2(uint32_t lo, uint32_t hi) { return lo | (hi << 16); }

// value a code stands for before scale/zero are applied: q in linear mode,
// +-2^(low bits) in exponent mode
template <int BITS>
__device__ __forceinline__ float code_value(uint32_t q, bool exponent_mode) {
    constexpr uint32_t EXP_MSK = (1u << (BITS - 1)) - 1u, SGN = 1u << (BITS - 1);
    float lin = (float)q;
    float ex = (float)(1u << (q & EXP_MSK));
    ex = (q & SGN) ? -ex : ex;
    return exponent_mode ? ex : lin;
}

// ---- host side
struct LaunchStatus { int code; hipError_t hip; };

int check_launch(const char* what);           // returns INT4MM_OK or INT4MM_ERR_LAUNCH
int validate_product(int bits, const void* outs, const void* matrix, const void* multiplier,
                     const void* scales, const void* zeros, const void* sparse_mask,
                     const int4mm_shape* sh, bool matvec);
int64_t tuning(int key);                       // see int4mm_tune (values are per host thread)
enum TuneKey { TUNE_MV_WAVES = 0, TUNE_MV_UNITS = 1, TUNE_MV_LK = 2, TUNE_MM_VARIANT = 3, TUNE_MV_NOPF = 4,
               TUNE_NO_SKINNY = 5, TUNE_MM_SPLIT = 6, TUNE_MM_TAIL = 7, TUNE_NO_WIDE = 8, TUNE_NO_BALANCE = 9,
               TUNE_MV_SPIN = 10, TUNE_COUNT = 11 };

// int4mm_describe_launch: while this thread is "noting", a launcher records the kernel and launch
// shape it has chosen instead of launching it.  noting(...) returns true (skip the launch) in that mode.
bool noting(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
bool is_noting();

// few-row product (2 .. 96 rows; sparse_mask != nullptr: 16:32 int4); false = shape not taken, use the general kernels
bool skinny_rows(int bits, _Float16* outs, const uint32_t* matrix, const _Float16* x, const _Float16* scales,
                 const _Float16* zeros, int64_t R, int64_t K, int64_t S, int64_t group_size, bool accumulate,
                 hipStream_t st, const uint32_t* sparse_mask, void* workspace, size_t workspace_bytes);
// two to four rows through the matvec kernel (dense formats; csrc/matvec.hip): false when it does not take the shape
bool matvec_rows(int bits, _Float16* outs, const uint32_t* matrix, const _Float16* x, const _Float16* scales,
                 const _Float16* zeros, int64_t R, int64_t K, int64_t S, int64_t group_size, bool accumulate,
                 hipStream_t st, void* workspace, size_t workspace_bytes);
// a single row through the matmul entry (overwrites outs); *rc is the launch's result when the shape is taken
bool matvec_one_row(int bits, _Float16* outs, const uint32_t* matrix, const uint32_t* sparse_mask, const _Float16* x,
                    const _Float16* scales, const _Float16* zeros, int64_t K, int64_t S, int64_t group_size, hipStream_t st,
                    void* workspace, size_t workspace_bytes, int* rc);
// most rows the few-row path takes (beyond 96: only its kernel with shared staging, for the shapes it serves)
constexpr int SK_WIDE_MAX_ROWS = 512;
// bytes of partial tiles with which the few-row kernel splits K across workgroups (0: no split)
size_t skinny_workspace_bytes(int64_t R, int64_t K, int64_t S, bool sparse);

// Layout of a caller's workspace, a function of its size alone so that calls with different shapes may
// share one buffer.  The lower half (down to a page boundary) is kept zero between calls: the matvec's
// hand-over slots from byte 0 and, in its last page, the arrival counters of the split-K kernels.  The
// upper half is scratch for partial tiles; no call relies on what it holds.
struct WorkspaceParts {
    char* counters;           // one page (nullptr: the workspace has no room for it); the 8 bytes in front of it
                              // are the matvec's hand-over error word (non-zero: a hand-over timed out)
    char* scratch;
    size_t slots_bytes;       // room for the matvec's slots, below the counters
    size_t scratch_bytes;
};
inline WorkspaceParts workspace_parts(void* workspace, size_t bytes) {
    WorkspaceParts p{nullptr, nullptr, 0, 0};
    const size_t kept_zero = (bytes / 2) & ~size_t(4095);
    if (workspace == nullptr || kept_zero < 8192) return p;
    p.counters = static_cast<char*>(workspace) + kept_zero - 4096;
    p.scratch = static_cast<char*>(workspace) + kept_zero;
    p.slots_bytes = kept_zero - 4096;
    p.scratch_bytes = bytes - kept_zero;
    return p;
}
// the matvec's hand-over slots: up to 32 K-splits x out_size (in 256s) x {fp32, flag}
inline size_t matvec_slots_bytes(int64_t out_size) {
    if (out_size < 0) out_size = 0;
    return 4096 + (size_t)((out_size + 255) / 256 * 256) * 8 * 32;
}
// the array built into the library that int4mm_matvec_static uses as its workspace (csrc/matvec.hip): the
// current device's copy and its size; false if the runtime cannot resolve it
bool static_scratch(void** ptr, size_t* bytes);
inline size_t round_to_page(size_t n) { return (n + 4095) & ~size_t(4095); }

}  // namespace i4
