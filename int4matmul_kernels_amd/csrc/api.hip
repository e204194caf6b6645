// Host-side plumbing of the C ABI: error text, argument validation shared by
// the two products, tuning knobs and workspace set-up.
#include "common.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

namespace i4 {

static thread_local int g_last_hip_error = 0;
static thread_local int64_t g_tuning[TUNE_COUNT];
static thread_local bool g_noting = false;
static thread_local char g_note[512];

bool is_noting() { return g_noting; }
bool noting(const char* fmt, ...) {
    if (!g_noting) return false;
    const size_t used = strlen(g_note);
    if (used + 2 < sizeof(g_note)) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(g_note + used, sizeof(g_note) - used, fmt, ap);
        va_end(ap);
        strncat(g_note, "; ", sizeof(g_note) - strlen(g_note) - 1);
    }
    return true;
}

int check_launch(const char*) {
    if (g_noting) return INT4MM_OK;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return INT4MM_ERR_LAUNCH;
    }
    return INT4MM_OK;
}

int64_t tuning(int key) { return (key >= 0 && key < TUNE_COUNT) ? g_tuning[key] : 0; }

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Superset of the reference's host asserts (matmul_kernel.cu:379-416,435-439;
// matvec_kernel.cu:307-337,356-360): every one of them is a returned error here.
int validate_product(int bits, const void* outs, const void* matrix, const void* multiplier,
                     const void* scales, const void* zeros, const void* sparse_mask,
                     const int4mm_shape* sh, bool matvec) {
    if (bits != 4 && bits != 3 && bits != 2) return INT4MM_ERR_BITS;
    if (sh == nullptr) return INT4MM_ERR_NULL;
    if (sparse_mask != nullptr && bits != 4) return INT4MM_ERR_SPARSE_BITS;
    const int64_t B = sh->batch, M = sh->seq_len, K = sh->in_size, S = sh->out_size;
    const int64_t R = sh->matrix_rows, G = sh->n_groups, g = sh->group_size;
    if (B < 0 || M < 0 || K <= 0 || S <= 0 || R <= 0 || G <= 0) return INT4MM_ERR_SHAPE;
    if (matvec && M != 1 && B * M * S != 0) return INT4MM_ERR_SHAPE;        // matvec_kernel.cu:323
    if (K % 64 != 0 || S % 64 != 0) return INT4MM_ERR_SHAPE;                 // README.md:9
    if (sparse_mask != nullptr) {
        if (R * 16 != K) return INT4MM_ERR_SHAPE;                            // R*32*2/bits == K
    } else {
        if (R * 32 != K * bits) return INT4MM_ERR_SHAPE;
    }
    if (g == 0 || (g > 0 && g % 64 != 0)) return INT4MM_ERR_GROUP;           // matmul_kernel.cu:383
    const int64_t geff = g < 0 ? ONE_GROUP : g;
    if (G > (int64_t)1 << 40 || geff * G < K) return INT4MM_ERR_SHAPE;       // :413-414
    if (K > ((int64_t)1 << 31) - 64 || S > ((int64_t)1 << 31) - 256 || M > ((int64_t)1 << 31) - 256 ||
        B > 65535)
        return INT4MM_ERR_SHAPE;
    if (B * M * S == 0) return INT4MM_OK;
    if (!outs || !matrix || !multiplier || !scales || !zeros) return INT4MM_ERR_NULL;
    if (!aligned16(outs) || !aligned16(matrix) || !aligned16(multiplier) || !aligned16(scales) ||
        !aligned16(zeros) || !aligned16(sparse_mask))
        return INT4MM_ERR_ALIGN;
    return INT4MM_OK;
}

__global__ void fill_zero_kernel(uint32_t* p, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace i4

using namespace i4;

extern "C" {

const char* int4mm_error_string(int code) {
    switch (code) {
        case INT4MM_OK: return "ok";
        case INT4MM_ERR_BITS: return "unsupported bit width (must be 4, 3 or 2)";
        case INT4MM_ERR_SPARSE_BITS: return "16:32 sparsity is supported for int4 only";
        case INT4MM_ERR_SHAPE: return "tensor shapes are inconsistent or not multiples of 64";
        case INT4MM_ERR_GROUP: return "group_size must be negative or a positive multiple of 64";
        case INT4MM_ERR_NULL: return "a required pointer is null";
        case INT4MM_ERR_WORKSPACE: return "workspace missing or too small";
        case INT4MM_ERR_LAUNCH: return "HIP launch failed";
        case INT4MM_ERR_ALIGN: return "a device pointer is not 16-byte aligned";
        case INT4MM_ERR_HANDOVER: return "a matvec hand-over timed out earlier on this workspace; zero-fill it again";
        default: return "unknown int4mm error";
    }
}

int int4mm_last_hip_error(void) { return g_last_hip_error; }
int int4mm_abi_version(void) { return 1; }

// Benchmark/tuning hook: overrides a launch heuristic for the calling thread (0 restores the default).
// Keys: 0 = matvec waves per workgroup, 1 = matvec units per lane group,
// 2 = matvec lane groups per wave (1, 2 or 4), 3 = matmul kernel variant,
// 4 = matvec: 1 disables the software prefetch, 5 = 1 disables the few-row kernel,
// 6 = matmul split-K factor (1 = never, 2..8 = forced where the shape allows a split),
// 7 = 1: the tiles of a matmul's last, partly filled round are not split,
// 8 = 1: 33 .. 96 rows take the few-row kernel whose waves stage their own states,
// 9 = 1: no balanced few-row launch, 10 = polls before a matvec hand-over gives up.
int int4mm_tune(int key, int64_t value) {
    if (key < 0 || key >= TUNE_COUNT) return INT4MM_ERR_SHAPE;
    g_tuning[key] = value;
    return INT4MM_OK;
}

// the matvec's slots and the counter page in the half that is kept zero; as much again above it
size_t int4mm_workspace_bytes(int64_t max_out_size) {
    return 2 * (matvec_slots_bytes(max_out_size) + 4096);
}

// workspace == NULL: the array built into the library (what int4mm_matvec_static works on); a fill kernel on
// `stream`, no allocation, no memset node
int int4mm_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
    if (workspace == nullptr) {
        if (workspace_bytes != 0) return INT4MM_ERR_NULL;
        if (!static_scratch(&workspace, &workspace_bytes)) return INT4MM_ERR_LAUNCH;
    }
    if (workspace_bytes < 4096) return INT4MM_ERR_WORKSPACE;
    size_t n = workspace_bytes / 4;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (uint32_t*)workspace, n);
    return check_launch("workspace_init");
}


// What would int4mm_matvec (product 0) or int4mm_matmul (product 1) launch for this shape?  Runs the
// launcher's own decision code with the launches switched off; needs no GPU.
int int4mm_describe_launch(int product, int bits, const int4mm_shape* shape, int sparse, size_t workspace_bytes,
                           char* text, size_t text_bytes) {
    if (shape == nullptr || text == nullptr || text_bytes == 0) return INT4MM_ERR_NULL;
    void* fake = reinterpret_cast<void*>(uintptr_t(1) << 20);          // aligned, never dereferenced on the host
    g_note[0] = 0;
    g_noting = true;
    const int rc = (product == 0 ? int4mm_matvec : int4mm_matmul)(bits, fake, fake, fake, fake, fake, sparse ? fake : nullptr, shape,
                                                                  workspace_bytes ? fake : nullptr, workspace_bytes, nullptr);
    g_noting = false;
    snprintf(text, text_bytes, "%s", g_note);
    return rc;
}

// Has a matvec hand-over on this workspace timed out since it was last zero-filled?  (Copies one word
// back on `stream` and waits for it.)  After INT4MM_ERR_HANDOVER every matvec on the workspace returns
// NaN until int4mm_workspace_init has run again.
int int4mm_workspace_status(void* workspace, size_t workspace_bytes, void* stream) {
    if (workspace == nullptr) {                                  // the built-in array of int4mm_matvec_static
        if (workspace_bytes != 0) return INT4MM_ERR_NULL;
        if (!static_scratch(&workspace, &workspace_bytes)) return INT4MM_ERR_LAUNCH;
    }
    const WorkspaceParts p = workspace_parts(workspace, workspace_bytes);
    if (p.counters == nullptr) return INT4MM_ERR_WORKSPACE;
    uint32_t word = 0;
    if (hipMemcpyAsync(&word, p.counters - 8, 4, hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess ||
        hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
        g_last_hip_error = (int)hipGetLastError();
        return INT4MM_ERR_LAUNCH;
    }
    return word ? INT4MM_ERR_HANDOVER : INT4MM_OK;
}

}  // extern "C"
