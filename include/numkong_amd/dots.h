/**
 *  @brief Packed batched dot products C[m x n] = A[m x k] * B[n x k]^T on one MI355X (gfx950).
 *  @file include/numkong_amd/dots.h
 *
 *  Drop-in boundary for the packed-dots path of NumKong: every declaration below has the name,
 *  prototype and meaning of the reference symbol cited next to it, so a caller of the reference's
 *  `libnumkong.so` links against `libnumkong_amd.so` unchanged for this path. Everything else the
 *  reference exports (other kernel families, other dtypes) is absent on purpose.
 *
 *  Differences a caller can observe:
 *
 *  - Operands may live in host OR device memory. Device (hipMalloc) and device-addressable pointers are
 *    used in place; plain host pointers are staged through temporary device buffers (correct, but bound
 *    by PCIe). Mixed placements are allowed per pointer.
 *  - The packed image is this library's own format (MFMA operand-fragment order) and, like the
 *    reference's, only valid for the matching `nk_dots_packed_*`. It is a relocatable byte image:
 *    copying `nk_dots_packed_size_T(n, k)` bytes (host<->device included) keeps it valid. It must be
 *    16-byte aligned (any malloc/hipMalloc result is).
 *  - Calls are synchronous as in the reference: C is complete when the call returns.
 *  - On failure (no GPU, launch error, packed image that does not match dtype/n/k) the reference
 *    convention applies: `packed_size` returns 0, `pack` does nothing, `packed` fills the m x n outputs
 *    with 0xFF bytes (NaN / -1 / UINT_MAX). `nk_amd_last_error()` says why.
 *
 *  All strides are in bytes (reference: include/numkong/dots.h:59-71).
 */
#ifndef NUMKONG_AMD_DOTS_H
#define NUMKONG_AMD_DOTS_H

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__) || defined(__clang__)
#define NK_DYNAMIC __attribute__((visibility("default")))
#else
#define NK_DYNAMIC
#endif

/* Scalar types of the signatures (reference: include/numkong/types.h:798-861). The 16-bit and 8-bit float
 * types are raw bit patterns, as in the reference's dynamic-dispatch build (c/dispatch.h:10-12). */
typedef signed char nk_i8_t;
typedef unsigned char nk_u8_t;
typedef signed int nk_i32_t;
typedef unsigned int nk_u32_t;
typedef unsigned long long nk_u64_t;
typedef float nk_f32_t;
typedef double nk_f64_t;
typedef unsigned short nk_f16_t;
typedef unsigned short nk_bf16_t;
typedef unsigned char nk_e4m3_t;
typedef unsigned char nk_e5m2_t;
typedef unsigned char nk_e2m3_t; /* one 6-bit float per byte */
typedef unsigned char nk_e3m2_t;
typedef unsigned char nk_i4x2_t; /* two 4-bit integers per byte, the even dimension in the low nibble */
typedef unsigned char nk_u4x2_t;
typedef unsigned char nk_u1x8_t; /* eight 1-bit values per byte */
typedef nk_u64_t nk_size_t;

/** Element types (reference: include/numkong/types.h:923-952; same numeric codes). */
typedef enum {
    nk_dtype_unknown_k = 0,
    nk_u1_k = 1 << 1,
    nk_i8_k = 1 << 2,
    nk_i32_k = 1 << 4,
    nk_u8_k = 1 << 6,
    nk_u32_k = 1 << 8,
    nk_f64_k = 1 << 10,
    nk_f32_k = 1 << 11,
    nk_f16_k = 1 << 12,
    nk_bf16_k = 1 << 13,
    nk_e4m3_k = 1 << 14,
    nk_e5m2_k = 1 << 15,
    nk_i4_k = 1 << 16,
    nk_u4_k = 1 << 17,
    nk_e2m3_k = 1 << 18,
    nk_e3m2_k = 1 << 19,
} nk_dtype_t;

/** Kernel kinds (reference: include/numkong/capabilities.h:178-253; same codes). The three dots kinds and the
 *  two packed distance kinds, and the three symmetric kinds, resolve to kernels here; every other kind resolves to
 *  the error stub with capability 0. */
typedef enum {
    nk_kernel_unknown_k = 0,
    nk_kernel_dot_k = 'i',
    nk_kernel_dots_packed_size_k = 'P',
    nk_kernel_dots_pack_k = 'Q',
    nk_kernel_dots_packed_k = 'G',
    nk_kernel_dots_symmetric_k = 'y',
    nk_kernel_angulars_packed_k = 'N',
    nk_kernel_euclideans_packed_k = 'E',
    nk_kernel_angulars_symmetric_k = 'n',
    nk_kernel_euclideans_symmetric_k = 'D',
} nk_kernel_kind_t;

/** Capability mask (reference: include/numkong/capabilities.h:258-304). Bit 0 keeps its reference meaning
 *  but has no kernels behind it here; bit 62, unused by the reference, marks the gfx950 GPU backend. */
typedef nk_u64_t nk_capability_t;
#define nk_cap_serial_k ((nk_capability_t)1)
#define nk_cap_any_k    ((nk_capability_t)0xFFFFFFFFFFFFFFFFull)
#define nk_cap_gfx950_k ((nk_capability_t)1 << 62)

/* Punned kernel pointers (reference: include/numkong/capabilities.h:306-389). */
typedef void (*nk_metric_dense_punned_t)(void const *a, void const *b, nk_size_t dimensions, void *result);
typedef nk_size_t (*nk_dots_packed_size_punned_t)(nk_size_t columns, nk_size_t depth);
typedef void (*nk_dots_pack_punned_t)(void const *b, nk_size_t columns, nk_size_t depth, nk_size_t b_stride_bytes,
                                      void *b_packed);
typedef void (*nk_dots_packed_punned_t)(void const *a, void const *b_packed, void *c, nk_size_t rows, nk_size_t columns,
                                        nk_size_t depth, nk_size_t a_stride_bytes, nk_size_t c_stride_bytes);
typedef void (*nk_dots_symmetric_punned_t)(void const *vectors, nk_size_t vectors_count, nk_size_t depth,
                                           nk_size_t stride_bytes, void *result, nk_size_t result_stride_bytes,
                                           nk_size_t row_start, nk_size_t row_count);
typedef void (*nk_kernel_punned_t)(void *);

/* Bytes of the packed image of an (width x depth) B. Reference: include/numkong/dots.h:172-195. */
NK_DYNAMIC nk_size_t nk_dots_packed_size_i8(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_u8(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_bf16(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_f16(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_e4m3(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_e5m2(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_e2m3(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_e3m2(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_i4(nk_size_t width, nk_size_t depth); /* depth in 4-bit values */
NK_DYNAMIC nk_size_t nk_dots_packed_size_u4(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_u1(nk_size_t width, nk_size_t depth); /* depth in bits */
NK_DYNAMIC nk_size_t nk_dots_packed_size_f32(nk_size_t width, nk_size_t depth);
NK_DYNAMIC nk_size_t nk_dots_packed_size_f64(nk_size_t width, nk_size_t depth);

/* Pack row-major B (width rows of depth elements, b_stride bytes apart). Reference: include/numkong/dots.h:203-237. */
NK_DYNAMIC void nk_dots_pack_i8(nk_i8_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride, void *b_packed);
NK_DYNAMIC void nk_dots_pack_u8(nk_u8_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride, void *b_packed);
NK_DYNAMIC void nk_dots_pack_bf16(nk_bf16_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                  void *b_packed);
NK_DYNAMIC void nk_dots_pack_f16(nk_f16_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                 void *b_packed);
NK_DYNAMIC void nk_dots_pack_e4m3(nk_e4m3_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                  void *b_packed);
NK_DYNAMIC void nk_dots_pack_e5m2(nk_e5m2_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                  void *b_packed);
NK_DYNAMIC void nk_dots_pack_e2m3(nk_e2m3_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                  void *b_packed);
NK_DYNAMIC void nk_dots_pack_e3m2(nk_e3m2_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                  void *b_packed);
NK_DYNAMIC void nk_dots_pack_i4(nk_i4x2_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                void *b_packed);
NK_DYNAMIC void nk_dots_pack_u4(nk_u4x2_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                void *b_packed);
NK_DYNAMIC void nk_dots_pack_u1(nk_u1x8_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                void *b_packed);
NK_DYNAMIC void nk_dots_pack_f32(nk_f32_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                 void *b_packed);
NK_DYNAMIC void nk_dots_pack_f64(nk_f64_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,
                                 void *b_packed);

/* C = A * B^T with widened accumulators, C overwritten. Reference: include/numkong/dots.h:248-287. */
NK_DYNAMIC void nk_dots_packed_i8(nk_i8_t const *a, void const *b_packed, nk_i32_t *c, nk_size_t height,
                                  nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_u8(nk_u8_t const *a, void const *b_packed, nk_u32_t *c, nk_size_t height,
                                  nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_bf16(nk_bf16_t const *a, void const *b_packed, nk_f32_t *c, nk_size_t height,
                                    nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_f16(nk_f16_t const *a, void const *b_packed, nk_f32_t *c, nk_size_t height,
                                   nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_e4m3(nk_e4m3_t const *a, void const *b_packed, nk_f32_t *c, nk_size_t height,
                                    nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_e5m2(nk_e5m2_t const *a, void const *b_packed, nk_f32_t *c, nk_size_t height,
                                    nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_e2m3(nk_e2m3_t const *a, void const *b_packed, nk_f32_t *c, nk_size_t height,
                                    nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_e3m2(nk_e3m2_t const *a, void const *b_packed, nk_f32_t *c, nk_size_t height,
                                    nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_i4(nk_i4x2_t const *a, void const *b_packed, nk_i32_t *c, nk_size_t height,
                                  nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_u4(nk_u4x2_t const *a, void const *b_packed, nk_u32_t *c, nk_size_t height,
                                  nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
/* 1-bit values: c[i][j] = popcount(a_i AND b_j). Reference: include/numkong/dots.h:289-296. */
NK_DYNAMIC void nk_dots_packed_u1(nk_u1x8_t const *a, void const *b_packed, nk_u32_t *c, nk_size_t height,
                                  nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);

/* The two wide types: f64 results. f32 products are exact in f64 and summed in f64; f64 uses the reference's
 * compensated sum, and both reproduce its serial kernels bit for bit (include/numkong/dot/serial.h:262-335). */
NK_DYNAMIC void nk_dots_packed_f32(nk_f32_t const *a, void const *b_packed, nk_f64_t *c, nk_size_t height,
                                   nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);
NK_DYNAMIC void nk_dots_packed_f64(nk_f64_t const *a, void const *b_packed, nk_f64_t *c, nk_size_t height,
                                   nk_size_t width, nk_size_t depth, nk_size_t a_stride, nk_size_t c_stride);

/* Distances over the same packed B, in one pass: result[i][j] = angular (1 - cosine) or euclidean distance between
 * row i of A and row j of B, f32 results (f64 for f32 and f64 inputs). Reference: include/numkong/spatials.h:72-300. */
#define NK_AMD_DECLARE_SPATIALS_(T, in_t, r_t)                                                                            \
    NK_DYNAMIC void nk_angulars_packed_##T(in_t const *a, void const *b_packed, r_t *result, nk_size_t rows,     \
                                           nk_size_t cols, nk_size_t depth, nk_size_t a_stride, nk_size_t r_stride);  \
    NK_DYNAMIC void nk_euclideans_packed_##T(in_t const *a, void const *b_packed, r_t *result, nk_size_t rows,   \
                                             nk_size_t cols, nk_size_t depth, nk_size_t a_stride, nk_size_t r_stride);
NK_AMD_DECLARE_SPATIALS_(i8, nk_i8_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(u8, nk_u8_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(i4, nk_i4x2_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(u4, nk_u4x2_t, nk_f32_t)
NK_AMD_DECLARE_SPATIALS_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DECLARE_SPATIALS_(f64, nk_f64_t, nk_f64_t)
#undef NK_AMD_DECLARE_SPATIALS_

/* All pairs of one set of vectors: result[i][j] for i in [row_start, row_start + row_count), j >= i, is the dot
 * product (widened, as above) or the angular / euclidean distance (f32; f64 for f32 and f64 inputs) of vectors i and j; the distance of a vector
 * from itself is exactly 0. Only that upper triangle of the window is written; a caller that wants the full matrix
 * mirrors it (python/distance.c:865-872) and splits the rows among its threads with the window arguments. Reference:
 * include/numkong/dots.h:298-359, include/numkong/spatials.h:76-120, 245-275; include/numkong/dots/serial.h:2361-2435,
 * 2802-2878 for the semantics. */
#define NK_AMD_DECLARE_SYMMETRIC_(T, in_t, out_t, r_t)                                                                    \
    NK_DYNAMIC void nk_dots_symmetric_##T(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,              \
                                          nk_size_t stride, out_t *result, nk_size_t result_stride,                   \
                                          nk_size_t row_start, nk_size_t row_count);                                  \
    NK_DYNAMIC void nk_angulars_symmetric_##T(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,          \
                                              nk_size_t stride, r_t *result, nk_size_t result_stride,            \
                                              nk_size_t row_start, nk_size_t row_count);                              \
    NK_DYNAMIC void nk_euclideans_symmetric_##T(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,        \
                                                nk_size_t stride, r_t *result, nk_size_t result_stride,          \
                                                nk_size_t row_start, nk_size_t row_count);
NK_AMD_DECLARE_SYMMETRIC_(i8, nk_i8_t, nk_i32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(u8, nk_u8_t, nk_u32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(bf16, nk_bf16_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(f16, nk_f16_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(e4m3, nk_e4m3_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(e5m2, nk_e5m2_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(e2m3, nk_e2m3_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(e3m2, nk_e3m2_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(i4, nk_i4x2_t, nk_i32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(u4, nk_u4x2_t, nk_u32_t, nk_f32_t)
NK_AMD_DECLARE_SYMMETRIC_(f32, nk_f32_t, nk_f64_t, nk_f64_t)
NK_AMD_DECLARE_SYMMETRIC_(f64, nk_f64_t, nk_f64_t, nk_f64_t)
#undef NK_AMD_DECLARE_SYMMETRIC_

/* The 1-bit type has the dot-product kinds only (packed above, symmetric here), with their backend-suffixed names;
 * its distance kinds resolve to the error stubs. */
#define NK_AMD_DECLARE_DOTS_ONLY_(T, in_t, out_t)                                                                      \
    NK_DYNAMIC void nk_dots_symmetric_##T(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,              \
                                          nk_size_t stride, out_t *result, nk_size_t result_stride,                   \
                                          nk_size_t row_start, nk_size_t row_count);                                  \
    NK_DYNAMIC nk_size_t nk_dots_packed_size_##T##_gfx950(nk_size_t width, nk_size_t depth);                          \
    NK_DYNAMIC void nk_dots_pack_##T##_gfx950(in_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,    \
                                              void *b_packed);                                                        \
    NK_DYNAMIC void nk_dots_packed_##T##_gfx950(in_t const *a, void const *b_packed, out_t *c, nk_size_t height,      \
                                                nk_size_t width, nk_size_t depth, nk_size_t a_stride,                 \
                                                nk_size_t c_stride);                                                  \
    NK_DYNAMIC void nk_dots_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,     \
                                                   nk_size_t stride, out_t *result, nk_size_t result_stride,          \
                                                   nk_size_t row_start, nk_size_t row_count);
NK_AMD_DECLARE_DOTS_ONLY_(u1, nk_u1x8_t, nk_u32_t)
#undef NK_AMD_DECLARE_DOTS_ONLY_

/* Capability and lookup API. Reference: c/numkong.c:767-768, 831-913. */
NK_DYNAMIC int nk_uses_dynamic_dispatch(void);
NK_DYNAMIC int nk_configure_thread(nk_capability_t capabilities);
NK_DYNAMIC nk_capability_t nk_capabilities(void);
NK_DYNAMIC nk_capability_t nk_capabilities_available(void);
NK_DYNAMIC nk_capability_t nk_capabilities_compiled(void);
NK_DYNAMIC void nk_dispatch_table_update(nk_capability_t capabilities);
NK_DYNAMIC void nk_find_kernel_punned(nk_kernel_kind_t kind, nk_dtype_t dtype, nk_capability_t viable,
                                      nk_kernel_punned_t *kernel_output, nk_capability_t *capability_output);

/** Output element type of a kernel kind for an input type (reference: include/numkong/numkong.h:41-45). */
NK_DYNAMIC nk_dtype_t nk_kernel_output_dtype(nk_kernel_kind_t kind, nk_dtype_t input);

/* The gfx950 kernels by their backend-suffixed names, as the reference exposes `_serial`, `_haswell`, ...
 * (include/numkong/dots.h:361-1877). Same prototypes as the dispatched entry points above. */
#define NK_AMD_DECLARE_BACKEND_(T, in_t, out_t, r_t)                                                                      \
    NK_DYNAMIC nk_size_t nk_dots_packed_size_##T##_gfx950(nk_size_t width, nk_size_t depth);                           \
    NK_DYNAMIC void nk_dots_pack_##T##_gfx950(in_t const *b, nk_size_t width, nk_size_t depth, nk_size_t b_stride,     \
                                              void *b_packed);                                                         \
    NK_DYNAMIC void nk_dots_packed_##T##_gfx950(in_t const *a, void const *b_packed, out_t *c, nk_size_t height,       \
                                                nk_size_t width, nk_size_t depth, nk_size_t a_stride,                  \
                                                nk_size_t c_stride);                                 \
    NK_DYNAMIC void nk_angulars_packed_##T##_gfx950(in_t const *a, void const *b_packed, r_t *c, nk_size_t height,  \
                                                    nk_size_t width, nk_size_t depth, nk_size_t a_stride,                 \
                                                    nk_size_t c_stride);                                                  \
    NK_DYNAMIC void nk_euclideans_packed_##T##_gfx950(in_t const *a, void const *b_packed, r_t *c, nk_size_t height, \
                                                      nk_size_t width, nk_size_t depth, nk_size_t a_stride,               \
                                                      nk_size_t c_stride);                                                \
    NK_DYNAMIC void nk_dots_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,         \
                                                   nk_size_t stride, out_t *result, nk_size_t result_stride,              \
                                                   nk_size_t row_start, nk_size_t row_count);                             \
    NK_DYNAMIC void nk_angulars_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,     \
                                                       nk_size_t stride, r_t *result, nk_size_t result_stride,       \
                                                       nk_size_t row_start, nk_size_t row_count);                         \
    NK_DYNAMIC void nk_euclideans_symmetric_##T##_gfx950(in_t const *vectors, nk_size_t vectors_count, nk_size_t depth,   \
                                                         nk_size_t stride, r_t *result, nk_size_t result_stride,     \
                                                         nk_size_t row_start, nk_size_t row_count);
NK_AMD_DECLARE_BACKEND_(i8, nk_i8_t, nk_i32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(u8, nk_u8_t, nk_u32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(bf16, nk_bf16_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(f16, nk_f16_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(e4m3, nk_e4m3_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(e5m2, nk_e5m2_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(e2m3, nk_e2m3_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(e3m2, nk_e3m2_t, nk_f32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(i4, nk_i4x2_t, nk_i32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(u4, nk_u4x2_t, nk_u32_t, nk_f32_t)
NK_AMD_DECLARE_BACKEND_(f32, nk_f32_t, nk_f64_t, nk_f64_t)
NK_AMD_DECLARE_BACKEND_(f64, nk_f64_t, nk_f64_t, nk_f64_t)
#undef NK_AMD_DECLARE_BACKEND_

/* Additions without a counterpart in the reference. */

/** Text of the last failure on the calling thread ("" if none). The reference has no error channel. */
NK_DYNAMIC char const *nk_amd_last_error(void);

/**
 *  Asynchronous forms for callers that own a HIP stream (`stream` is a `hipStream_t`, NULL = default
 *  stream): device-accessible pointers only, no synchronisation, 0 on success. They exist so that a host
 *  program can queue packing and products behind its own work and time them with its own events; the
 *  synchronous reference-compatible entry points above are these plus staging plus a stream sync.
 */
NK_DYNAMIC int nk_amd_dots_pack_async(nk_dtype_t dtype, void const *b, nk_size_t width, nk_size_t depth,
                                      nk_size_t b_stride, void *b_packed, void *stream);
NK_DYNAMIC int nk_amd_dots_packed_async(nk_dtype_t dtype, void const *a, void const *b_packed, void *c,
                                        nk_size_t height, nk_size_t width, nk_size_t depth, nk_size_t a_stride,
                                        nk_size_t c_stride, void *stream);
/** `kind` is nk_kernel_angulars_packed_k or nk_kernel_euclideans_packed_k. */
NK_DYNAMIC int nk_amd_spatials_packed_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *a, void const *b_packed,
                                            void *c, nk_size_t height, nk_size_t width, nk_size_t depth,
                                            nk_size_t a_stride, nk_size_t c_stride, void *stream);

/**
 *  The symmetric kinds on the caller's stream. They pack the window's vectors first, so they need scratch memory:
 *  `workspace` is device memory, 256-byte aligned, of at least `nk_amd_symmetric_workspace_size` bytes for the same
 *  arguments, and belongs to the call until the stream has run it. `kind` is nk_kernel_dots_symmetric_k,
 *  nk_kernel_angulars_symmetric_k or nk_kernel_euclideans_symmetric_k.
 */
NK_DYNAMIC nk_size_t nk_amd_symmetric_workspace_size(nk_dtype_t dtype, nk_size_t vectors_count, nk_size_t depth,
                                                     nk_size_t row_start, nk_size_t row_count);
NK_DYNAMIC int nk_amd_symmetric_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *vectors,
                                      nk_size_t vectors_count, nk_size_t depth, nk_size_t stride, void *result,
                                      nk_size_t result_stride, nk_size_t row_start, nk_size_t row_count, void *workspace,
                                      nk_size_t workspace_bytes, void *stream);

/**
 *  `nk_amd_symmetric_async` for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 *  loops, harnesses that forbid hipMalloc): no workspace argument, no allocation of any kind inside. It has no
 *  counterpart in the reference. The scratch memory is a fixed array of `nk_amd_symmetric_static_capacity()` bytes
 *  (32 MiB) that the library keeps in the memory of every GPU it runs on; a call that would need more
 *  (`nk_amd_symmetric_workspace_size` says how much) returns non-zero and `nk_hip_last_error()` names both numbers.
 *  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU race, so keep them on one stream.
 */
NK_DYNAMIC nk_size_t nk_amd_symmetric_static_capacity(void);
NK_DYNAMIC int nk_amd_symmetric_static_async(nk_kernel_kind_t kind, nk_dtype_t dtype, void const *vectors,
                                             nk_size_t vectors_count, nk_size_t depth, nk_size_t stride, void *result,
                                             nk_size_t result_stride, nk_size_t row_start, nk_size_t row_count,
                                             void *stream);

#ifdef __cplusplus
}
#endif

#endif // NUMKONG_AMD_DOTS_H
