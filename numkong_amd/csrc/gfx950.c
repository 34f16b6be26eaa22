/**
 *  @brief Host side of the gfx950 backend: operand placement, staging, the reference's error convention.
 *  @file numkong_amd/csrc/gfx950.c
 *
 *  Defines `nk_dots_packed_size_<T>_gfx950`, `nk_dots_pack_<T>_gfx950`, `nk_dots_packed_<T>_gfx950`, the packed
 *  distances and the symmetric kinds on top of them: the backend-suffixed kernels that dispatch_<T>.c binds, in the way the reference names its per-ISA
 *  kernels (include/numkong/dots.h:361-1877). Plain C over the thin HIP ABI of <numkong_amd/hip_abi.h>.
 *
 *  The reference's kernels take caller-owned pointers and return nothing (include/numkong/dots.h:84-98);
 *  so do these. A pointer the GPU can address is used in place; a plain host pointer is staged through
 *  a temporary device buffer that lives for the duration of the call (the one hidden allocation of this
 *  library). Failures follow c/numkong.c:195-216: size 0, pack is a no-op, the product fills C with 0xFF.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "dispatch.h"
#include "numkong_amd/hip_abi.h"

static _Thread_local char nk_amd_error_[256] = "";

static void nk_amd_set_error_(char const *where) {
    char const *detail = nk_hip_last_error();
    snprintf(nk_amd_error_, sizeof(nk_amd_error_), "%s: %s", where, detail && detail[0] ? detail : "failed");
}

char const *nk_amd_last_error(void) { return nk_amd_error_; }

/** Bytes of one row of `k` elements: eight 1-bit or two 4-bit values to a byte, whole bytes (cast/serial.h:519-538). */
static size_t nk_amd_row_bytes_(nk_dtype_t dtype, size_t k) {
    switch (dtype) {
    case nk_u1_k: return (k + 7) / 8;
    case nk_i4_k:
    case nk_u4_k: return (k + 1) / 2;
    case nk_i8_k:
    case nk_u8_k:
    case nk_e4m3_k:
    case nk_e5m2_k:
    case nk_e2m3_k:
    case nk_e3m2_k: return k;
    case nk_f16_k:
    case nk_bf16_k: return k * 2;
    case nk_f32_k: return k * 4;
    case nk_f64_k: return k * 8;
    default: return 0;
    }
}

/** Bytes of one output: f64 for the two wide types, 32 bits for everything else on this path. */
static size_t nk_amd_output_bytes_(nk_dtype_t dtype) { return dtype == nk_f32_k || dtype == nk_f64_k ? 8 : 4; }

static size_t nk_amd_round_up_(size_t x, size_t to) { return (x + to - 1) / to * to; }

/** 0xFF over the m x n outputs only: the reference stub writes n * 8 bytes per row (c/numkong.c:209-216),
 *  which overruns 4-byte outputs; the convention is kept, the overrun is not (`out_bytes` per output). */
static void nk_amd_fill_error_(void *c, int c_kind, size_t m, size_t n, size_t c_stride, size_t out_bytes) {
    if (!c || !m || !n) return;
    if (c_kind == 1) { /* (as 32-bit words: two per f64 output) */
        if (nk_hip_fill_rows_async(c, m, n * out_bytes / 4, c_stride, 0xFFFFFFFFu, NULL) == 0) nk_hip_stream_synchronize(NULL);
        return;
    }
    for (size_t row = 0; row < m; ++row) memset((char *)c + row * c_stride, 0xFF, n * out_bytes);
}

int nk_amd_dots_pack_async(nk_dtype_t dtype, void const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride,
                           void *b_packed, void *stream) {
    return nk_hip_dots_pack_async((int)dtype, b, n, k, b_stride, b_packed, stream);
}

int nk_amd_dots_packed_async(nk_dtype_t dtype, void const *a, void const *b_packed, void *c, nk_size_t m, nk_size_t n,
                             nk_size_t k, nk_size_t a_stride, nk_size_t c_stride, void *stream) {
    return nk_hip_dots_packed_async((int)dtype, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
}

int nk_amd_spatials_packed_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *a, void const *b_packed, void *c,
                                 nk_size_t m, nk_size_t n, nk_size_t k, nk_size_t a_stride, nk_size_t c_stride,
                                 void *stream) {
    int const metric = kind == nk_kernel_angulars_packed_k ? 1 : (kind == nk_kernel_euclideans_packed_k ? 2 : 0);
    return nk_hip_spatials_packed_async((int)dtype, metric, a, b_packed, c, m, n, k, a_stride, c_stride, stream);
}

static nk_size_t nk_amd_packed_size_(nk_dtype_t dtype, nk_size_t n, nk_size_t k) {
    return nk_hip_dots_packed_size((int)dtype, n, k);
}

static void nk_amd_pack_(nk_dtype_t dtype, void const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride,
                         void *b_packed) {
    nk_amd_error_[0] = 0;
    size_t const total = nk_hip_dots_packed_size((int)dtype, n, k);
    if (!total || !b_packed) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_pack: unsupported dtype or dimensions");
        return;
    }
    if (nk_hip_device_count() <= 0) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_pack: no HIP device");
        return;
    }
    int const b_kind = (n && k) ? nk_hip_pointer_kind(b) : 1;
    int const p_kind = nk_hip_pointer_kind(b_packed);
    void *staged_b = NULL, *staged_p = NULL;
    void const *device_b = b;
    void *device_p = b_packed;
    size_t device_b_stride = b_stride;
    int status = 0;

    if (b_kind == 0) {
        size_t const row_bytes = nk_amd_row_bytes_(dtype, k);
        device_b_stride = nk_amd_round_up_(row_bytes, 16);
        status = nk_hip_malloc(&staged_b, n * device_b_stride);
        if (!status) status = nk_hip_memcpy2d_h2d(staged_b, device_b_stride, b, b_stride, row_bytes, n, NULL);
        device_b = staged_b;
    }
    if (!status && p_kind == 0) {
        status = nk_hip_malloc(&staged_p, total);
        device_p = staged_p;
    }
    if (!status) status = nk_hip_dots_pack_async((int)dtype, device_b, n, k, device_b_stride, device_p, NULL);
    if (!status && staged_p) status = nk_hip_memcpy_d2h(b_packed, staged_p, total, NULL);
    if (!status) status = nk_hip_stream_synchronize(NULL);
    if (status) nk_amd_set_error_("nk_dots_pack");
    if (staged_b) nk_hip_free(staged_b);
    if (staged_p) nk_hip_free(staged_p);
}

/** `metric`: 0 dot products, 1 angular distances, 2 euclidean distances; outputs are 4 bytes wide, 8 for f32 and f64 inputs. */
static void nk_amd_packed_(nk_dtype_t dtype, int metric, void const *a, void const *b_packed, void *c, nk_size_t m,
                           nk_size_t n, nk_size_t k, nk_size_t a_stride, nk_size_t c_stride) {
    nk_amd_error_[0] = 0;
    if (!m || !n) return;
    size_t const out_bytes = nk_amd_output_bytes_(dtype);
    size_t const total = nk_hip_dots_packed_size((int)dtype, n, k);
    if (nk_hip_device_count() <= 0) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_packed: no HIP device");
        nk_amd_fill_error_(c, 0, m, n, c_stride, out_bytes);
        return;
    }
    int const c_kind = nk_hip_pointer_kind(c);
    if (!total || !b_packed || !c) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_packed: unsupported dtype or dimensions");
        nk_amd_fill_error_(c, c_kind, m, n, c_stride, out_bytes);
        return;
    }
    int const a_kind = k ? nk_hip_pointer_kind(a) : 1;
    int const p_kind = nk_hip_pointer_kind(b_packed);
    void *staged_a = NULL, *staged_p = NULL, *staged_c = NULL;
    void const *device_a = a, *device_p = b_packed;
    void *device_c = c;
    size_t device_a_stride = a_stride, device_c_stride = c_stride;
    int status = 0;

    if (a_kind == 0) {
        size_t const row_bytes = nk_amd_row_bytes_(dtype, k);
        device_a_stride = nk_amd_round_up_(row_bytes, 16);
        status = nk_hip_malloc(&staged_a, m * device_a_stride);
        if (!status) status = nk_hip_memcpy2d_h2d(staged_a, device_a_stride, a, a_stride, row_bytes, m, NULL);
        device_a = staged_a;
    }
    if (!status && p_kind == 0) {
        status = nk_hip_malloc(&staged_p, total);
        if (!status) status = nk_hip_memcpy_h2d(staged_p, b_packed, total, NULL);
        device_p = staged_p;
    }
    if (!status && c_kind == 0) {
        device_c_stride = nk_amd_round_up_(n * out_bytes, 16);
        status = nk_hip_malloc(&staged_c, m * device_c_stride);
        device_c = staged_c;
    }
    if (!status && metric == 0)
        status = nk_hip_dots_packed_async((int)dtype, device_a, device_p, device_c, m, n, k, device_a_stride,
                                          device_c_stride, NULL);
    if (!status && metric != 0)
        status = nk_hip_spatials_packed_async((int)dtype, metric, device_a, device_p, device_c, m, n, k, device_a_stride,
                                              device_c_stride, NULL);
    if (!status && staged_c) status = nk_hip_memcpy2d_d2h(c, c_stride, staged_c, device_c_stride, n * out_bytes, m, NULL);
    if (!status) status = nk_hip_stream_synchronize(NULL);
    if (status) {
        nk_amd_set_error_("nk_dots_packed");
        nk_amd_fill_error_(c, c_kind, m, n, c_stride, out_bytes);
    }
    if (staged_a) nk_hip_free(staged_a);
    if (staged_p) nk_hip_free(staged_p);
    if (staged_c) nk_hip_free(staged_c);
}

nk_size_t nk_amd_symmetric_workspace_size(nk_dtype_t dtype, nk_size_t vectors_count, nk_size_t depth,
                                          nk_size_t row_start, nk_size_t row_count) {
    return nk_hip_symmetric_workspace_size((int)dtype, vectors_count, depth, row_start, row_count);
}

static int nk_amd_symmetric_metric_(nk_kernel_kind_t kind) {
    switch (kind) {
    case nk_kernel_dots_symmetric_k: return 0;
    case nk_kernel_angulars_symmetric_k: return 1;
    case nk_kernel_euclideans_symmetric_k: return 2;
    default: return -1;
    }
}

int nk_amd_symmetric_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *vectors, nk_size_t vectors_count,
                           nk_size_t depth, nk_size_t stride, void *result, nk_size_t result_stride, nk_size_t row_start,
                           nk_size_t row_count, void *workspace, nk_size_t workspace_bytes, void *stream) {
    return nk_hip_symmetric_async((int)dtype, nk_amd_symmetric_metric_(kind), vectors, vectors_count, depth, stride,
                                  result, result_stride, row_start, row_count, workspace, workspace_bytes, stream);
}

/** 0xFF over the whole n x n result, as the reference's stub does (c/numkong.c:218-227), 4 bytes per output. */
static void nk_amd_fill_symmetric_error_(void *result, int kind, size_t n, size_t result_stride, size_t out_bytes) {
    nk_amd_fill_error_(result, kind, n, n, result_stride, out_bytes);
}

/**
 *  The symmetric kinds: rows [row_start, row_start + row_count) of the upper triangle of the n x n result.
 *  Host operands are staged: the vectors from the window's first 32-row boundary on, and the window of the result
 *  both ways, so that what the kernel does not write (left of the diagonal) comes back as the caller had it.
 */
static void nk_amd_symmetric_(nk_dtype_t dtype, int metric, void const *vectors, nk_size_t n, nk_size_t k,
                              nk_size_t stride, void *result, nk_size_t result_stride, nk_size_t row_start,
                              nk_size_t row_count) {
    nk_amd_error_[0] = 0;
    if (!n || !row_count || row_start >= n) return;
    size_t const out_bytes = nk_amd_output_bytes_(dtype);
    if (nk_hip_device_count() <= 0) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_symmetric: no HIP device");
        nk_amd_fill_symmetric_error_(result, 0, n, result_stride, out_bytes);
        return;
    }
    int const r_kind = nk_hip_pointer_kind(result);
    size_t const workspace_bytes = nk_hip_symmetric_workspace_size((int)dtype, n, k, row_start, row_count);
    if (!workspace_bytes || !result) {
        snprintf(nk_amd_error_, sizeof(nk_amd_error_), "nk_dots_symmetric: unsupported dtype or dimensions");
        nk_amd_fill_symmetric_error_(result, r_kind, n, result_stride, out_bytes);
        return;
    }
    size_t const row_end = row_count < n - row_start ? row_start + row_count : n;
    size_t const first = row_start / 32 * 32; /* vectors and result columns from here on take part */
    int const v_kind = k ? nk_hip_pointer_kind(vectors) : 1;
    void *staged_v = NULL, *staged_r = NULL, *workspace = NULL;
    /* device views, addressed as if they started at vector 0 / result element (0, 0) */
    char const *device_v = (char const *)vectors;
    char *device_r = (char *)result;
    size_t device_stride = stride, device_r_stride = result_stride;
    int status = nk_hip_malloc(&workspace, workspace_bytes);

    if (!status && v_kind == 0) {
        size_t const row_bytes = nk_amd_row_bytes_(dtype, k);
        device_stride = nk_amd_round_up_(row_bytes, 16);
        status = nk_hip_malloc(&staged_v, (n - first) * device_stride);
        if (!status)
            status = nk_hip_memcpy2d_h2d(staged_v, device_stride, (char const *)vectors + first * stride, stride,
                                         row_bytes, n - first, NULL);
        device_v = (char const *)staged_v - first * device_stride;
    }
    char *host_window = (char *)result + row_start * result_stride + first * out_bytes;
    if (!status && r_kind == 0) {
        device_r_stride = nk_amd_round_up_((n - first) * out_bytes, 16);
        status = nk_hip_malloc(&staged_r, (row_end - row_start) * device_r_stride);
        if (!status)
            status = nk_hip_memcpy2d_h2d(staged_r, device_r_stride, host_window, result_stride, (n - first) * out_bytes,
                                         row_end - row_start, NULL);
        device_r = (char *)staged_r - row_start * device_r_stride - first * out_bytes;
    }
    if (!status)
        status = nk_hip_symmetric_async((int)dtype, metric, device_v, n, k, device_stride, device_r, device_r_stride,
                                        row_start, row_count, workspace, workspace_bytes, NULL);
    if (!status && staged_r)
        status = nk_hip_memcpy2d_d2h(host_window, result_stride, staged_r, device_r_stride, (n - first) * out_bytes,
                                     row_end - row_start, NULL);
    if (!status) status = nk_hip_stream_synchronize(NULL);
    else (void)nk_hip_stream_synchronize(NULL);
    if (status) {
        nk_amd_set_error_("nk_dots_symmetric");
        nk_amd_fill_symmetric_error_(result, r_kind, n, result_stride, out_bytes);
    }
    if (staged_v) nk_hip_free(staged_v);
    if (staged_r) nk_hip_free(staged_r);
    if (workspace) nk_hip_free(workspace);
}

#define NK_AMD_DEFINE_BACKEND_DOTS_(T, in_t, out_t)                                                                     \
    nk_size_t nk_dots_packed_size_##T##_gfx950(nk_size_t width, nk_size_t depth) {                                 \
        return nk_amd_packed_size_(nk_##T##_k, width, depth);                                                      \
    }                                                                                                              \
    void nk_dots_pack_##T##_gfx950(in_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,            \
                                   void *b_packed) {                                                               \
        nk_amd_pack_(nk_##T##_k, b, width, depth, b_stride, b_packed);                                             \
    }                                                                                                              \
    void nk_dots_packed_##T##_gfx950(in_t const *a, void const *b_packed, out_t *c, nk_size_t height,              \
                                     nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride) {   \
        nk_amd_packed_(nk_##T##_k, 0, a, b_packed, c, height, width, depth, a_stride, c_stride);                   \
    }                                                                                                              \
    void nk_dots_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,             \
                                        nk_size_t stride, out_t *result, nk_size_t result_stride,                  \
                                        nk_size_t row_start, nk_size_t row_count) {                                \
        nk_amd_symmetric_(nk_##T##_k, 0, vectors, vectors_count, depth, stride, result, result_stride, row_start,  \
                          row_count);                                                                              \
    }

#define NK_AMD_DEFINE_BACKEND_DISTANCES_(T, in_t, r_t)                                                                 \
    void nk_angulars_packed_##T##_gfx950(in_t const *a, void const *b_packed, r_t *c, nk_size_t height,       \
                                         nk_size_t width, nk_size_t depth, nk_size_t a_stride,                     \
                                         nk_size_t c_stride) {                                                     \
        nk_amd_packed_(nk_##T##_k, 1, a, b_packed, c, height, width, depth, a_stride, c_stride);                   \
    }                                                                                                              \
    void nk_euclideans_packed_##T##_gfx950(in_t const *a, void const *b_packed, r_t *c, nk_size_t height,     \
                                           nk_size_t width, nk_size_t depth, nk_size_t a_stride,                   \
                                           nk_size_t c_stride) {                                                   \
        nk_amd_packed_(nk_##T##_k, 2, a, b_packed, c, height, width, depth, a_stride, c_stride);                   \
    }                                                                                                              \
    void nk_angulars_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,         \
                                            nk_size_t stride, r_t *result, nk_size_t result_stride,           \
                                            nk_size_t row_start, nk_size_t row_count) {                            \
        nk_amd_symmetric_(nk_##T##_k, 1, vectors, vectors_count, depth, stride, result, result_stride, row_start,  \
                          row_count);                                                                              \
    }                                                                                                              \
    void nk_euclideans_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,       \
                                              nk_size_t stride, r_t *result, nk_size_t result_stride,         \
                                              nk_size_t row_start, nk_size_t row_count) {                          \
        nk_amd_symmetric_(nk_##T##_k, 2, vectors, vectors_count, depth, stride, result, result_stride, row_start,  \
                          row_count);                                                                              \
    }

NK_AMD_DEFINE_BACKEND_DOTS_(i8, nk_i8_t, nk_i32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(i8, nk_i8_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(u8, nk_u8_t, nk_u32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(u8, nk_u8_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(i4, nk_i4x2_t, nk_i32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(i4, nk_i4x2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(u4, nk_u4x2_t, nk_u32_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(u4, nk_u4x2_t, nk_f32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(u1, nk_u1x8_t, nk_u32_t)
NK_AMD_DEFINE_BACKEND_DOTS_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DEFINE_BACKEND_DOTS_(f64, nk_f64_t, nk_f64_t)
NK_AMD_DEFINE_BACKEND_DISTANCES_(f64, nk_f64_t, nk_f64_t)
