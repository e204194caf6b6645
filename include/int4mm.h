/*
 * int4mm.h -- C ABI of libint4mm_hip.so: quantized int{4,3,2} x fp16 matvec and
 * matmul for AMD MI355X (gfx950), plus the pack / unpack helpers of the same
 * formats.
 *
 * Plain pointers and sizes only; no torch types.  Every pointer is a DEVICE
 * pointer unless stated otherwise.  `stream` is a hipStream_t passed as void*
 * (NULL = the null stream).  All launches are asynchronous on `stream`; the
 * functions validate their arguments on the host first and return a non-zero
 * INT4MM_ERR_* code without launching anything if a check fails.
 *
 * Citations name the reference interface each entry point replaces
 * (paths relative to the mstnegate/int4matmul_kernels checkout).
 *
 * Dimension names: K = in_size (reduction dim, unpacked weight rows),
 * S = out_size (output columns), R = packed rows of `matrix`,
 * G = rows of scales/zeros, g = group_size.
 *
 * Formats (bit-exact with the reference):
 *   matrix, dense int4/int2 : int32 [K*bits/32, S]; code k of a word at bits
 *                             bits*(k mod 32/bits), LSB first.
 *   matrix, dense int3      : int32 [3K/32, S]; every 32 codes of a column are
 *                             a 96-bit LSB-first stream over 3 rows.
 *   matrix + mask, 16:32    : mask int32 [K/32, S], bit t of [b,s] set <=> row
 *                             32b+t kept; matrix int32 [K/16, S], rows 2b,2b+1 =
 *                             low/high half of the 64-bit word of kept codes in
 *                             ascending row order, 4 bits each.  Dropped rows
 *                             decode to exactly 0.
 *   scales, zeros           : fp16 [G, S], entry (k / g, s), dense k index.
 *                             scale >= 0: w = fp16(fp16(q - z) * s);
 *                             scale <  0: w = fp16_fma(+-2^(q & (2^(bits-1)-1)), -s, z),
 *                             sign = top bit of the code.
 *   multiplier, outs        : fp16 [B, M, K] and [B, M, S], contiguous.
 *
 * Numerics of the products.  "Bit-exact" above is about the formats and the helpers
 * (pack, unpack, dequantize).  int4mm_matmul with 17 or more rows of states multiplies
 * exactly those fp16 weights and accumulates in fp32.  int4mm_matvec and the few-row
 * kernels behind both products (2..16 rows, and up to 96 on some shapes) do not round
 * per weight: they accumulate sum(x * q) and sum(x) in fp32 and apply scale and zero
 * once per group, y += s * (sum(x * q) - z * sum(x)), which is the exact value of
 * sum(x * (q - z) * s) up to fp32 rounding -- closer to the true product than the
 * reference's fp16(fp16(q - z) * s) weights, but not the same bits.  A single row through
 * int4mm_matmul is served by the matvec kernel as well (overwriting outs, as the matmul
 * does): bit for bit int4mm_matvec's result on zeroed outs, as long as the workspace holds
 * the matvec's part (int4mm_workspace_bytes); without it a tile kernel takes the row.  Results are a
 * deterministic function of the inputs and the shape (no atomics on data).
 */
#ifndef INT4MM_H
#define INT4MM_H

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define INT4MM_API __attribute__((visibility("default")))
#else
#define INT4MM_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define INT4MM_OK               0
#define INT4MM_ERR_BITS         1   /* bits not in {4,3,2}          (int4matmul.cpp:35,45)           */
#define INT4MM_ERR_SPARSE_BITS  2   /* 16:32 mask with bits != 4    (matmul.cuh:184-190,328-332)     */
#define INT4MM_ERR_SHAPE        3   /* a size rule below is violated (matmul_kernel.cu:379-416)      */
#define INT4MM_ERR_GROUP        4   /* group_size not a positive multiple of 64 and not negative     */
#define INT4MM_ERR_NULL         5   /* a required pointer is NULL                                     */
#define INT4MM_ERR_WORKSPACE    6   /* workspace missing or smaller than int4mm_workspace_bytes()    */
#define INT4MM_ERR_LAUNCH       7   /* the HIP runtime refused the launch; see int4mm_last_hip_error */
#define INT4MM_ERR_ALIGN        8   /* a pointer is not 16-byte aligned                              */
#define INT4MM_ERR_HANDOVER     9   /* a matvec hand-over timed out on this workspace (see int4mm_workspace_status) */

/* Human-readable text for a code above (host pointer, static storage). */
INT4MM_API const char* int4mm_error_string(int code);
/* hipError_t value of the most recent INT4MM_ERR_LAUNCH on this thread. */
INT4MM_API int int4mm_last_hip_error(void);
/* ABI version of this header; bumped on any signature change. */
INT4MM_API int int4mm_abi_version(void);

/* Benchmark / tuning hook, not part of the drop-in boundary: overrides a launch
 * heuristic for the calling host thread (value 0 restores the default).  key 0 = waves per
 * workgroup of the matvec and few-row kernels, 1 = matvec 64-row units per lane
 * group, 2 = matvec lane groups per wave / few-row kernel columns per lane (1, 2, 4), 3 = matmul kernel variant
 * (5 / 6 / 7 = pipelined 256x128 / 256x256 / 128x256 tiles, 9 = 256x256 without
 * the two-phase order; a forced variant also keeps the product away from the
 * few-row kernels), 4 = matvec: 1 disables prefetch,
 * 5 = 1 disables the few-row (2..512 rows) kernels, 6 = split-K factor of the
 * matmul and few-row kernels (1 = never split, 2..8 = that factor where the
 * shape allows a split at all), 7 = 1: the tiles of a matmul's last, partly
 * filled round are not split, 8 = the few-row kernel whose waves share the
 * staged states: 1 = never, n >= 2 = from n rows on whatever the shape,
 * 9 = 1: few-row products never take the balanced launch (workgroups sharing the strips evenly),
 * 10 = polls after which a matvec hand-over gives up (failure-handling tests). */
INT4MM_API int int4mm_tune(int key, int64_t value);

/* Shape of one product.  matrix_rows = R, n_groups = G (rows of scales/zeros).
 * Rules (violations -> INT4MM_ERR_SHAPE), a strict superset of the reference's
 * asserts at matmul_kernel.cu:379-416,435-439 and matvec_kernel.cu:307-337,356-360:
 *   dense : R * 32 == K * bits         sparse (bits == 4) : R * 16 == K
 *   K % 64 == 0, S % 64 == 0 (README.md:9), B, M >= 1 (B*M*S == 0 returns OK)
 *   group_size < 0 (one group) or group_size % 64 == 0; g * G >= K
 * One requirement the reference does not have:
 *   int4mm_matvec needs a workspace of int4mm_workspace_bytes(S) bytes, whatever launch
 *   shape the product takes (INT4MM_ERR_WORKSPACE without one; it does not fall back).
 * (A K beyond 458752 -- what one launch covers: 32 ranges of 224 units of 64 rows -- runs as
 * several launches, each adding onto the result of the one before.  The only shape refused
 * for its length is a single quantisation group longer than that on a still longer K.)
 */
typedef struct int4mm_shape {
    int64_t batch;        /* B */
    int64_t seq_len;      /* M */
    int64_t in_size;      /* K */
    int64_t out_size;     /* S */
    int64_t matrix_rows;  /* R */
    int64_t n_groups;     /* G */
    int64_t group_size;   /* g, or negative for a single group */
} int4mm_shape;

/* Bytes of device scratch the two products may use for any shape with
 * out_size <= `max_out_size` (partial sums and arrival counters of the split-K
 * finish).  The buffer must be zero-filled once before its first use (e.g. with
 * int4mm_workspace_init); the kernels leave it zeroed where it must be zero.
 * Calls that share one workspace must not overlap in time.  Calls of different
 * shapes may share one: its layout depends on its size alone (the lower half is
 * kept zero -- hand-over slots, arrival counters -- and the upper half is scratch
 * for partial tiles), so always pass the size the buffer was zero-filled with. */
INT4MM_API size_t int4mm_workspace_bytes(int64_t max_out_size);
/* Zero-fills a workspace with a kernel on `stream` (no allocation, no memset node: it may be
 * recorded into a graph).  workspace == NULL with workspace_bytes == 0 means the array built
 * into the library that int4mm_matvec_static works on. */
INT4MM_API int int4mm_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/* Health of a workspace.  The matvec's workgroups hand partial sums over through the workspace;
 * the last workgroup of a column range waits for the others with a bounded number of polls.  If
 * that wait ever runs out (it cannot while the GPU dispatches workgroups in order), the affected
 * outputs are NaN, the workspace is marked, and every later matvec on it returns NaN too -- never a
 * silently wrong number -- until int4mm_workspace_init has zero-filled it again.  This call copies
 * the mark back on `stream`, waits for it and returns INT4MM_ERR_HANDOVER if it is set.
 * workspace == NULL with workspace_bytes == 0 asks about the array built into the library
 * (int4mm_matvec_static), which int4mm_workspace_init(NULL, 0, stream) zero-fills again.  No
 * counterpart in the reference, whose atomics cannot time out (matvec_kernel.cu:263). */
INT4MM_API int int4mm_workspace_status(void* workspace, size_t workspace_bytes, void* stream);

/* Which kernel, tile shape and split would int4mm_matvec (product 0) or int4mm_matmul (product 1)
 * launch for `shape` with a workspace of `workspace_bytes`?  Writes a one-line description into
 * `text` (host memory) using the launcher's own decision code with the launches switched off; it
 * touches no GPU.  For tests that pin the dispatch of the benchmark shapes, and for profiling. */
INT4MM_API int int4mm_describe_launch(int product, int bits, const int4mm_shape* shape, int sparse,
                  size_t workspace_bytes, char* text, size_t text_bytes);

/* Bytes of workspace with which int4mm_matmul may split the K dimension of `shape`
 * over several workgroups per output tile (shapes with so few tiles that most of
 * the GPU would idle, or whose last round of tiles would leave half of it idle; `sparse` != 0 for the 16:32 format), or
 * a few-row product share its column strips out evenly over the workgroups (more strips than compute units) -- also
 * int4mm_matvec with 2 and more batch entries, which takes the few-row kernels (in chunks of up to 512); never less than
 * int4mm_workspace_bytes(shape->out_size).  A smaller workspace is not an error:
 * the product then runs unsplit.  Same zero-fill rule as above.  No counterpart in
 * the reference, whose matmul (matmul_kernel.cu:375-459) uses no scratch. */
INT4MM_API size_t int4mm_matmul_workspace_bytes(const int4mm_shape* shape, int sparse);

/* Matrix-vector product, M == 1 per batch entry:
 *     outs[b,0,:] = fp16( fp32(outs[b,0,:]) + multiplier[b,0,:] @ W )
 * i.e. the result is ADDED onto the prior contents of outs, as the reference's
 * launcher does through its fp32 temporary.
 * Replaces matvec_packed_int<bits> / matvec_int{4,3,2}
 * (matvec_kernel.cu:302-387).  shape->seq_len must be 1 (matvec_kernel.cu:323).
 * sparse_mask == NULL selects the dense format. */
INT4MM_API int int4mm_matvec(int bits, void* outs, const void* matrix, const void* multiplier,
                  const void* scales, const void* zeros, const void* sparse_mask,
                  const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                  void* stream);

/* int4mm_matvec for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without
 * the workspace, same kernels.  Results are bit for bit those of int4mm_matvec on a workspace
 * that allows the same launch plan: always for one row of states; for several batch entries
 * when that workspace has int4mm_matmul_workspace_bytes() and the few-row kernels' partial
 * sums fit the array's scratch half (8.4 MB) -- a smaller workspace, or larger partials, makes
 * one of the two run unsplit, which changes the summation order, not the accuracy class.  The
 * hand-over slots and split-K partials live in a 16.8 MB device array built into the library (each GPU the library
 * runs on holds its copy until the process ends), which covers out_size <= 32768; a wider
 * product returns INT4MM_ERR_WORKSPACE.  The call allocates and frees nothing.  Its first
 * call on a device looks up that device's copy of the array (make it once outside any
 * graph capture).  All calls on one GPU share the array: calls that overlap in time on one
 * GPU (two streams) race, exactly as two int4mm_matvec calls sharing one workspace would.
 * A hand-over that times out marks the array like any workspace: int4mm_workspace_status(NULL,
 * 0, stream) reports it and int4mm_workspace_init(NULL, 0, stream) clears it.
 * No counterpart in the reference, whose matvec allocates an fp32 temporary per call
 * (matvec_kernel.cu:351). */
INT4MM_API int int4mm_matvec_static(int bits, void* outs, const void* matrix, const void* multiplier,
                  const void* scales, const void* zeros, const void* sparse_mask,
                  const int4mm_shape* shape, void* stream);

/* Matrix-matrix product:
 *     outs[b,m,:] = fp16( sum_k fp32(multiplier[b,m,k]) * fp32(W[k,:]) )   (overwrites outs)
 * Replaces matmul_packed_int<bits> / matmul_int{4,3,2}
 * (matmul_kernel.cu:375-463).  Any M >= 1 is accepted. */
INT4MM_API int int4mm_matmul(int bits, void* outs, const void* matrix, const void* multiplier,
                  const void* scales, const void* zeros, const void* sparse_mask,
                  const int4mm_shape* shape, void* workspace, size_t workspace_bytes,
                  void* stream);

/* 16:32 sparse int4 packer.  wt_in / msk_in: uint8 [S, K] (row = output column;
 * msk_in > 0 keeps the row); wt_outs: int32 [K/16, S]; msk_outs: int32 [K/32, S].
 * Requires K % 32 == 0.  Replaces sparse_int4_pack / weight_matrix_packing
 * (utils_kernel.cu:19-119, int4matmul.cpp:50-63).
 * bad_blocks (device int32[1], may be NULL) is incremented once for every
 * (column, 32-row block) whose mask does not keep exactly 16 rows -- the
 * condition the reference asserts on the device (utils_kernel.cu:41). */
INT4MM_API int int4mm_sparse_pack(void* wt_outs, void* msk_outs, const void* wt_in, const void* msk_in,
                       int64_t out_size, int64_t in_size, void* bad_blocks, void* stream);

/* Dense packer for int4/int3/int2: codes uint8 [K, S] (row = k) -> matrix
 * int32 [K*bits/32, S].  The reference packs dense weights with Python loops
 * (kernel_test.py:60-123); this is the on-device equivalent of those loops. */
INT4MM_API int int4mm_dense_pack(int bits, void* matrix_out, const void* codes_in,
                      int64_t in_size, int64_t out_size, void* stream);

/* Unpack to raw codes: codes_out uint8 [K, S]; keep_out uint8 [K, S] or NULL
 * (1 = kept; all ones for dense).  Inverse of the two packers; the decode step
 * of smem_unpack_weights (matmul.cuh:246-405) without the dequantisation. */
INT4MM_API int int4mm_unpack(int bits, void* codes_out, void* keep_out, const void* matrix,
                  const void* sparse_mask, int64_t in_size, int64_t out_size, void* stream);

/* Unpack + dequantise to the fp16 matrix the kernels multiply by:
 * w_out fp16 [K, S], bit-exact with dequantize<> / smem_unpack_weights
 * (matmul.cuh:115-136,246-428), dropped sparse rows = +0.0. */
INT4MM_API int int4mm_dequantize(int bits, void* w_out, const void* matrix, const void* scales,
                      const void* zeros, const void* sparse_mask, int64_t in_size,
                      int64_t out_size, int64_t n_groups, int64_t group_size, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* INT4MM_H */
