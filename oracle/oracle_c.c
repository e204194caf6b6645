/*
 * Scalar C restatement of the reference's decode loops and products.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/liboracle_c.so and loaded by
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg as a checker
 * and as the "port" CPU baseline.  Nothing in the product links or loads it.
 *
 * It deliberately follows the *loop structure* of the CUDA decoders (shift and
 * consume), whereas oracle/oracle.py states the formats in closed form; the
 * tests require the two to agree, which pins both against a transposed index,
 * a wrong shift or a dropped carry bit.  fp16 arithmetic is done in double and
 * rounded once per reference operation (each of __hsub, __hmul, __hfma is one
 * correctly rounded operation; a double holds their exact result for every
 * operand the formats can produce, except exponent-mode sums whose operands
 * are more than 40 binades apart).
 *
 * Paths cited are relative to the reference checkout.
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>
#include <string.h>

/* ---- software binary16 ------------------------------------------------- */
static double h2d(uint16_t h) {
    int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
    double v;
    if (e == 0)       v = ldexp((double)m, -24);
    else if (e == 31) v = m ? NAN : INFINITY;
    else              v = ldexp((double)(m + 1024), e - 25);
    return s ? -v : v;
}

static uint16_t d2h(double d) {           /* round to nearest even */
    if (isnan(d)) return 0x7E00;
    uint16_t sign = signbit(d) ? 0x8000 : 0;
    double a = fabs(d);
    if (a >= 65520.0) return sign | 0x7C00;
    if (a < ldexp(1.0, -14)) return sign | (uint16_t)nearbyint(ldexp(a, 24));
    int e;
    double f = nearbyint(frexp(a, &e) * 2048.0);    /* [1024, 2048] */
    if (f == 2048.0) { f = 1024.0; e += 1; }
    int E = e - 1 + 15;
    if (E >= 31) return sign | 0x7C00;
    return sign | (uint16_t)(E << 10) | (uint16_t)((int)f - 1024);
}

uint16_t oc_d2h(double d) { return d2h(d); }
double oc_h2d(uint16_t h) { return h2d(h); }

/* ---- dequantize<LINEAR> matmul.cuh:115-125, <EXPONENT_SYM> :127-136,
 *      dynamic switch :414-428 ------------------------------------------- */
static uint16_t dequant_linear(uint32_t v, int bits, uint16_t scale, uint16_t zero) {
    uint32_t q = v & ((1u << bits) - 1u);
    uint16_t d = d2h((double)q - h2d(zero));          /* __hsub(__uint2half_rn(q), zero) */
    return d2h(h2d(d) * h2d(scale));                  /* __hmul(.., scale) */
}

static uint16_t dequant_exponent(uint32_t v, int bits, uint16_t pos_scale, uint16_t zero) {
    uint32_t exp_msk = (1u << (bits - 1)) - 1u, sgn = 1u << (bits - 1);
    int iv = ((v & sgn) ? -1 : 1) * (int)(1u << (v & exp_msk));
    return d2h((double)iv * h2d(pos_scale) + h2d(zero)); /* __hfma */
}

static uint16_t dequant_dynamic(uint32_t v, int bits, uint16_t scale, uint16_t zero) {
    if (h2d(scale) >= 0.0)                              /* __hge(scale, 0) */
        return dequant_linear(v, bits, scale, zero);
    return dequant_exponent(v, bits, scale ^ 0x8000, zero);   /* __hneg(scale) */
}

uint16_t oc_dequant(uint32_t v, int bits, uint16_t scale, uint16_t zero) {
    return dequant_dynamic(v, bits, scale, zero);
}

/* ---- column decoders: one 32-code run of one column --------------------- */
/* power-of-two widths: shift-and-consume, matmul.cuh:256-265 */
static void decode32_pow2(const uint32_t* col, size_t stride, int bits, uint8_t out[32]) {
    int per = 32 / bits, n = 0;
    for (int i = 0; i < bits; ++i) {                /* bits words hold 32 codes */
        uint32_t v = col[(size_t)i * stride];
        for (int j = 0; j < per; ++j) { out[n++] = (uint8_t)(v & ((1u << bits) - 1u)); v >>= bits; }
    }
}

/* int3: the three-word walk of matvec_kernel.cu:53-127 (second statement of
 * the format; matmul.cuh:270-309 is the first) */
static void decode32_int3(const uint32_t* col, size_t stride, uint8_t out[32]) {
    uint32_t v = col[0], v2 = col[stride];
    int n = 0;
    for (int i = 0; i < 10; ++i) { out[n++] = v & 7; v >>= 3; }      /* codes 0..9 */
    v |= (v2 & 1u) << 2;                                              /* code 10: 2 bits + 1 */
    out[n++] = v & 7;
    v = v2 >> 1; v2 = col[2 * stride];
    for (int i = 0; i < 10; ++i) { out[n++] = v & 7; v >>= 3; }      /* codes 11..20 */
    v |= (v2 & 3u) << 1;                                              /* code 21: 1 bit + 2 */
    out[n++] = v & 7;
    v = v2 >> 2;
    for (int i = 0; i < 10; ++i) { out[n++] = v & 7; v >>= 3; }      /* codes 22..31 */
}

/* sparse int4: consume the 64-bit compacted word under the mask,
 * matvec_kernel.cu:135-169; dropped rows are reported through keep[] */
static void decode32_sparse(const uint32_t* wcol, const uint32_t* mcol, size_t stride,
                            uint8_t out[32], uint8_t keep[32]) {
    uint64_t v = (uint64_t)wcol[0] | ((uint64_t)wcol[stride] << 32);
    uint32_t msk = mcol[0];
    for (int t = 0; t < 32; ++t) {
        if (msk & 1u) { out[t] = (uint8_t)(v & 0xF); keep[t] = 1; v >>= 4; }
        else          { out[t] = 0; keep[t] = 0; }
        msk >>= 1;
    }
}

static void decode32(int bits, int sparse, const uint32_t* matrix, const uint32_t* mask,
                     size_t S, size_t blk, size_t s, uint8_t codes[32], uint8_t keep[32]) {
    memset(keep, 1, 32);
    if (sparse)         decode32_sparse(matrix + (2 * blk) * S + s, mask + blk * S + s, S, codes, keep);
    else if (bits == 3) decode32_int3(matrix + (3 * blk) * S + s, S, codes);
    else                decode32_pow2(matrix + ((size_t)bits * blk) * S + s, S, bits, codes);
}

/* codes_out / keep_out: uint8 [K, S] (keep_out may be NULL) */
void oc_unpack(int bits, const uint32_t* matrix, const uint32_t* mask, size_t K, size_t S,
               uint8_t* codes_out, uint8_t* keep_out) {
    uint8_t c[32], k[32];
    for (size_t blk = 0; blk < K / 32; ++blk)
        for (size_t s = 0; s < S; ++s) {
            decode32(bits, mask != NULL, matrix, mask, S, blk, s, c, k);
            for (int t = 0; t < 32; ++t) {
                codes_out[(blk * 32 + t) * S + s] = c[t];
                if (keep_out) keep_out[(blk * 32 + t) * S + s] = k[t];
            }
        }
}

/* fp16 tile the kernels build: w16_out uint16 [K, S]; scales/zeros [G, S];
 * group index uses the dense K index also for the sparse format
 * (matmul_kernel.cu:261-263, matvec_kernel.cu:234,241-242) */
void oc_dequantize(int bits, const uint32_t* matrix, const uint32_t* mask,
                   const uint16_t* scales, const uint16_t* zeros, int64_t group_size,
                   size_t K, size_t S, uint16_t* w16_out) {
    size_t g = group_size < 0 ? 0x0FFFFFFF : (size_t)group_size;
    uint8_t c[32], k[32];
    for (size_t blk = 0; blk < K / 32; ++blk)
        for (size_t s = 0; s < S; ++s) {
            decode32(bits, mask != NULL, matrix, mask, S, blk, s, c, k);
            for (int t = 0; t < 32; ++t) {
                size_t kk = blk * 32 + t, gi = kk / g;
                uint16_t w = dequant_dynamic(c[t], bits, scales[gi * S + s], zeros[gi * S + s]);
                w16_out[kk * S + s] = k[t] ? w : 0;            /* matmul.cuh:398 */
            }
        }
}

/* sparse packer, lane by lane as utils_kernel.cu:29-63: ballot -> mask word,
 * popc rank, shift, add-reduce, two 32-bit halves.  wt_in/msk_in: uint8 [S,K]
 * (height = S, stride = K).  Returns the number of blocks whose popcount is
 * not 16 (the device assert at :41). */
int64_t oc_sparse_pack(uint32_t* wt_outs, uint32_t* msk_outs, const uint8_t* wt_in,
                       const uint8_t* msk_in, size_t height, size_t stride) {
    int64_t bad = 0;
    for (size_t ry = 0; ry < height; ++ry)
        for (size_t bx = 0; bx < stride / 32; ++bx) {
            uint32_t bmsk = 0;
            for (int lane = 0; lane < 32; ++lane)
                if (msk_in[bx * 32 + lane + ry * stride] > 0) bmsk |= 1u << lane;
            msk_outs[ry + bx * height] = bmsk;
            if (__builtin_popcount(bmsk) != 16) ++bad;
            uint64_t sum = 0;
            for (int lane = 0; lane < 32; ++lane) {
                uint32_t pos = (uint32_t)__builtin_popcount(bmsk & ((1u << lane) - 1u));
                uint64_t v = wt_in[bx * 32 + lane + ry * stride];
                v &= 0xF; v <<= 4 * pos; v *= (uint64_t)((bmsk >> lane) & 1u);
                sum += v;
            }
            size_t rx = bx * 32;
            wt_outs[ry + (rx / 16) * height] = (uint32_t)(sum & 0xFFFFFFFFu);
            wt_outs[ry + (rx / 16 + 1) * height] = (uint32_t)((sum >> 32) & 0xFFFFFFFFu);
        }
    return bad;
}

/* Matvec in the reference's arithmetic: per 64-row slab and column, an fp32
 * running sum of float(x_k) * float(w_k) in ascending k
 * (matvec_kernel.cu:29-48,256-258), slabs added in ascending order into an
 * fp32 accumulator seeded with the prior contents of outs (:351,:263), then
 * rounded to fp16 (:381-382).  The GPU reference adds slabs in atomic order,
 * so this is one admissible ordering, not the only one.
 * x: uint16 [K]; outs: uint16 [S] in/out. */
void oc_matvec(int bits, const uint32_t* matrix, const uint32_t* mask, const uint16_t* x,
               const uint16_t* scales, const uint16_t* zeros, int64_t group_size,
               size_t K, size_t S, uint16_t* outs) {
    size_t g = group_size < 0 ? 0x0FFFFFFF : (size_t)group_size;
    uint8_t c[32], k[32];
    for (size_t s = 0; s < S; ++s) {
        float acc = (float)h2d(outs[s]);
        for (size_t slab = 0; slab < K / 64; ++slab) {
            float part[2] = {0.0f, 0.0f};            /* two 32-row halves = two warps */
            for (int hb = 0; hb < 2; ++hb) {
                size_t blk = slab * 2 + hb;
                decode32(bits, mask != NULL, matrix, mask, S, blk, s, c, k);
                size_t gi = (slab * 64) / g;         /* one scale per slab, :234 */
                float m = 0.0f;
                for (int t = 0; t < 32; ++t) {
                    if (!k[t]) continue;
                    uint16_t w = dequant_dynamic(c[t], bits, scales[gi * S + s], zeros[gi * S + s]);
                    m += (float)h2d(x[blk * 32 + t]) * (float)h2d(w);
                }
                part[hb] = m;
            }
            acc += part[0];
            acc += part[1];
        }
        outs[s] = d2h((double)acc);
    }
}
