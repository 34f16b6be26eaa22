/**
 *  @brief Exported entry points of the packed-dots path, dispatched through one global table.
 *  @file numkong_amd/csrc/numkong.c
 *
 *  Counterpart of the reference's c/numkong.c for this path: the table (c/numkong.c:231), the
 *  `nk_dots_packed_size_T` / `nk_dots_pack_T` / `nk_dots_packed_T` trampolines (c/numkong.c:347-364,
 *  instantiated :628-671), the `nk_angulars_packed_T` / `nk_euclideans_packed_T` ones next to them and the three
 *  symmetric kinds, the error stubs (:78-81, :195-227), the capability and lookup API
 *  (:767-768, :831-913) and initialisation when the library is loaded (:916-919).
 */
#include <stdatomic.h>
#include <string.h>

#include "dispatch.h"
#include "numkong_amd/hip_abi.h"

__attribute__((aligned(64))) nk_implementations_t nk_dispatch_table;

static void nk_fill_error_(void *ptr, nk_size_t bytes) { memset(ptr, 0xFF, bytes); }

void nk_error_dense_(void const *a, void const *b, nk_size_t n, void *d) {
    (void)a, (void)b, (void)n;
    nk_fill_error_(d, sizeof(nk_f64_t));
}

nk_size_t nk_error_packed_size_(nk_size_t n, nk_size_t k) {
    (void)n, (void)k;
    return 0;
}

void nk_error_pack_(void const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride, void *b_packed) {
    (void)b, (void)n, (void)k, (void)b_stride, (void)b_packed;
}

/** The stub of a kind this library has no kernel for (with the GPU backend selected, failures are reported by the
 *  backend itself, which knows the width of its outputs): n * 4 bytes per row are poisoned, the width of every output
 *  on this path but the f64 results of f32 and f64 inputs, of which that is the first half of each row. A device
 *  pointer is filled on the device. */
void nk_error_dots_(void const *a, void const *b_packed, void *c, nk_size_t m, nk_size_t n, nk_size_t k,
                    nk_size_t a_stride, nk_size_t c_stride) {
    (void)a, (void)b_packed, (void)k, (void)a_stride;
    if (nk_hip_device_count() > 0 && nk_hip_pointer_kind(c) == 1) {
        if (nk_hip_fill_rows_async(c, m, n, c_stride, 0xFFFFFFFFu, 0) == 0) nk_hip_stream_synchronize(0);
        return;
    }
    for (nk_size_t row = 0; row < m; ++row) nk_fill_error_((char *)c + row * c_stride, n * 4);
}

/** The same for the types with f64 outputs: n * 8 bytes per row, what the reference's stub writes for every type. */
void nk_error_dots_wide_(void const *a, void const *b_packed, void *c, nk_size_t m, nk_size_t n, nk_size_t k,
                         nk_size_t a_stride, nk_size_t c_stride) {
    nk_error_dots_(a, b_packed, c, m, 2 * n, k, a_stride, c_stride);
}

/** The reference's stub poisons the whole n x n result, whatever the window (c/numkong.c:218-227). */
void nk_error_dots_symmetric_(void const *vectors, nk_size_t n_vectors, nk_size_t depth, nk_size_t stride, void *result,
                              nk_size_t result_stride, nk_size_t row_start, nk_size_t row_count) {
    (void)row_start, (void)row_count;
    nk_error_dots_(vectors, 0, result, n_vectors, n_vectors, depth, stride, result_stride);
}

void nk_error_dots_symmetric_wide_(void const *vectors, nk_size_t n_vectors, nk_size_t depth, nk_size_t stride,
                                   void *result, nk_size_t result_stride, nk_size_t row_start, nk_size_t row_count) {
    (void)row_start, (void)row_count;
    nk_error_dots_(vectors, 0, result, n_vectors, 2 * n_vectors, depth, stride, result_stride);
}

#define NK_AMD_DISPATCH_DOTS_(T, in_t, out_t)                                                                   \
    NK_DYNAMIC nk_size_t nk_dots_packed_size_##T(nk_size_t n, nk_size_t k) {                                    \
        return nk_dispatch_table.dots_packed_size_##T(n, k);                                                    \
    }                                                                                                           \
    NK_DYNAMIC void nk_dots_pack_##T(in_t const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride,               \
                                     void *b_packed) {                                                          \
        nk_dispatch_table.dots_pack_##T(b, n, k, b_stride, b_packed);                                           \
    }                                                                                                           \
    NK_DYNAMIC void nk_dots_packed_##T(in_t const *a, void const *b_packed, out_t *c, nk_size_t m, nk_size_t n, \
                                       nk_size_t k, nk_size_t a_stride, nk_size_t c_stride) {                   \
        nk_dispatch_table.dots_packed_##T(a, b_packed, c, m, n, k, a_stride, c_stride);                         \
    }                                                                                                           \
    NK_DYNAMIC void nk_dots_symmetric_##T(in_t const *vectors, nk_size_t n, nk_size_t k, nk_size_t stride,      \
                                          out_t *result, nk_size_t result_stride, nk_size_t row_start,          \
                                          nk_size_t row_count) {                                                \
        nk_dispatch_table.dots_symmetric_##T(vectors, n, k, stride, result, result_stride, row_start, row_count); \
    }

#define NK_AMD_DISPATCH_DISTANCES_(T, in_t, r_t)                                                                   \
    NK_DYNAMIC void nk_angulars_packed_##T(in_t const *a, void const *b_packed, r_t *c, nk_size_t m,       \
                                           nk_size_t n, nk_size_t k, nk_size_t a_stride, nk_size_t c_stride) {  \
        nk_dispatch_table.angulars_packed_##T(a, b_packed, c, m, n, k, a_stride, c_stride);                     \
    }                                                                                                           \
    NK_DYNAMIC void nk_euclideans_packed_##T(in_t const *a, void const *b_packed, r_t *c, nk_size_t m,     \
                                             nk_size_t n, nk_size_t k, nk_size_t a_stride,                      \
                                             nk_size_t c_stride) {                                              \
        nk_dispatch_table.euclideans_packed_##T(a, b_packed, c, m, n, k, a_stride, c_stride);                   \
    }                                                                                                           \
    NK_DYNAMIC void nk_angulars_symmetric_##T(in_t const *vectors, nk_size_t n, nk_size_t k, nk_size_t stride,  \
                                              r_t *result, nk_size_t result_stride, nk_size_t row_start,   \
                                              nk_size_t row_count) {                                            \
        nk_dispatch_table.angulars_symmetric_##T(vectors, n, k, stride, result, result_stride, row_start,       \
                                                 row_count);                                                    \
    }                                                                                                           \
    NK_DYNAMIC void nk_euclideans_symmetric_##T(in_t const *vectors, nk_size_t n, nk_size_t k, nk_size_t stride, \
                                                r_t *result, nk_size_t result_stride, nk_size_t row_start, \
                                                nk_size_t row_count) {                                          \
        nk_dispatch_table.euclideans_symmetric_##T(vectors, n, k, stride, result, result_stride, row_start,     \
                                                   row_count);                                                  \
    }

NK_AMD_DISPATCH_DOTS_(i8, nk_i8_t, nk_i32_t)
NK_AMD_DISPATCH_DISTANCES_(i8, nk_i8_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(u8, nk_u8_t, nk_u32_t)
NK_AMD_DISPATCH_DISTANCES_(u8, nk_u8_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DISPATCH_DISTANCES_(bf16, nk_bf16_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DISPATCH_DISTANCES_(f16, nk_f16_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DISPATCH_DISTANCES_(e4m3, nk_e4m3_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DISPATCH_DISTANCES_(e5m2, nk_e5m2_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DISPATCH_DISTANCES_(e2m3, nk_e2m3_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DISPATCH_DISTANCES_(e3m2, nk_e3m2_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(i4, nk_i4x2_t, nk_i32_t)
NK_AMD_DISPATCH_DISTANCES_(i4, nk_i4x2_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(u4, nk_u4x2_t, nk_u32_t)
NK_AMD_DISPATCH_DISTANCES_(u4, nk_u4x2_t, nk_f32_t)
NK_AMD_DISPATCH_DOTS_(u1, nk_u1x8_t, nk_u32_t)
NK_AMD_DISPATCH_DOTS_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DISPATCH_DISTANCES_(f32, nk_f32_t, nk_f64_t)
NK_AMD_DISPATCH_DOTS_(f64, nk_f64_t, nk_f64_t)
NK_AMD_DISPATCH_DISTANCES_(f64, nk_f64_t, nk_f64_t)

NK_DYNAMIC int nk_uses_dynamic_dispatch(void) { return 1; }

/** The reference needs this once per thread for AMX tile permission (include/README.md:531-532). Here it creates
 *  the calling thread's streams ahead of its first product, when a GPU is there; calling it is optional. */
NK_DYNAMIC int nk_configure_thread(nk_capability_t capabilities) {
    if ((capabilities & nk_cap_gfx950_k) && (nk_capabilities() & nk_cap_gfx950_k)) {
        (void)nk_hip_thread_stream(0);
        (void)nk_hip_thread_stream(1);
    }
    return 1;
}

NK_DYNAMIC nk_capability_t nk_capabilities_compiled(void) { return nk_cap_serial_k | nk_cap_gfx950_k; }

/** Probes for a GPU on first use, not when the library is loaded, so that loading never starts HIP. */
NK_DYNAMIC nk_capability_t nk_capabilities(void) {
    static _Atomic nk_capability_t cached = nk_cap_any_k; /* (threads that ask at the same time store the same answer) */
    nk_capability_t known = atomic_load_explicit(&cached, memory_order_relaxed);
    if (known != nk_cap_any_k) return known;
    known = nk_cap_serial_k | (nk_hip_device_count() > 0 ? nk_cap_gfx950_k : 0);
    atomic_store_explicit(&cached, known, memory_order_relaxed);
    return known;
}

NK_DYNAMIC nk_capability_t nk_capabilities_available(void) { return nk_capabilities() & nk_capabilities_compiled(); }

NK_DYNAMIC void nk_dispatch_table_update(nk_capability_t caps) {
    nk_dispatch_i8_init_(caps);
    nk_dispatch_u8_init_(caps);
    nk_dispatch_bf16_init_(caps);
    nk_dispatch_f16_init_(caps);
    nk_dispatch_e4m3_init_(caps);
    nk_dispatch_e5m2_init_(caps);
    nk_dispatch_e2m3_init_(caps);
    nk_dispatch_e3m2_init_(caps);
    nk_dispatch_i4_init_(caps);
    nk_dispatch_u4_init_(caps);
    nk_dispatch_u1_init_(caps);
    nk_dispatch_f32_init_(caps);
    nk_dispatch_f64_init_(caps);
}

NK_DYNAMIC void nk_find_kernel_punned(nk_kernel_kind_t kind, nk_dtype_t dtype, nk_capability_t viable,
                                      nk_kernel_punned_t *kernel_output, nk_capability_t *capability_output) {
    nk_kernel_punned_t *m = kernel_output;
    nk_capability_t *c = capability_output;
    switch (dtype) {
    case nk_i8_k: nk_dispatch_i8_find_(viable, kind, m, c); return;
    case nk_u8_k: nk_dispatch_u8_find_(viable, kind, m, c); return;
    case nk_bf16_k: nk_dispatch_bf16_find_(viable, kind, m, c); return;
    case nk_f16_k: nk_dispatch_f16_find_(viable, kind, m, c); return;
    case nk_e4m3_k: nk_dispatch_e4m3_find_(viable, kind, m, c); return;
    case nk_e5m2_k: nk_dispatch_e5m2_find_(viable, kind, m, c); return;
    case nk_e2m3_k: nk_dispatch_e2m3_find_(viable, kind, m, c); return;
    case nk_e3m2_k: nk_dispatch_e3m2_find_(viable, kind, m, c); return;
    case nk_i4_k: nk_dispatch_i4_find_(viable, kind, m, c); return;
    case nk_u4_k: nk_dispatch_u4_find_(viable, kind, m, c); return;
    case nk_u1_k: nk_dispatch_u1_find_(viable, kind, m, c); return;
    case nk_f32_k: nk_dispatch_f32_find_(viable, kind, m, c); return;
    case nk_f64_k: nk_dispatch_f64_find_(viable, kind, m, c); return;
    default: break;
    }
    *m = (nk_kernel_punned_t)0;
    *c = (nk_capability_t)0;
}

NK_DYNAMIC nk_dtype_t nk_kernel_output_dtype(nk_kernel_kind_t kind, nk_dtype_t input) {
    if (kind == nk_kernel_angulars_packed_k || kind == nk_kernel_euclideans_packed_k ||
        kind == nk_kernel_angulars_symmetric_k || kind == nk_kernel_euclideans_symmetric_k) {
        switch (input) { /* reference: include/numkong/numkong.h:46-51 */
        case nk_i8_k:
        case nk_u8_k:
        case nk_bf16_k:
        case nk_f16_k:
        case nk_e4m3_k:
        case nk_e5m2_k:
        case nk_e2m3_k:
        case nk_e3m2_k:
        case nk_i4_k:
        case nk_u4_k: return nk_f32_k;
        case nk_f32_k:
        case nk_f64_k: return nk_f64_k;
        default: return nk_dtype_unknown_k; /* (u1 has the dot-product kinds only) */
        }
    }
    if (kind != nk_kernel_dots_packed_k && kind != nk_kernel_dots_symmetric_k) return nk_dtype_unknown_k;
    switch (input) {
    case nk_i8_k:
    case nk_i4_k: return nk_i32_k;
    case nk_u8_k:
    case nk_u4_k:
    case nk_u1_k: return nk_u32_k;
    case nk_bf16_k:
    case nk_f16_k:
    case nk_e4m3_k:
    case nk_e5m2_k:
    case nk_e2m3_k:
    case nk_e3m2_k: return nk_f32_k;
    case nk_f32_k:
    case nk_f64_k: return nk_f64_k;
    default: return nk_dtype_unknown_k;
    }
}

/** The table is bound to the compiled backend when the library is loaded; whether a GPU is present is
 *  found out by the kernels at call time (they follow the error convention if not). */
__attribute__((constructor)) static void nk_auto_init(void) { nk_dispatch_table_update(nk_capabilities_compiled()); }
