/**
 *  @brief Shared declarations of the dispatch layer: table, error stubs, per-dtype find/init.
 *  @file numkong_amd/csrc/dispatch.h
 *
 *  Mirrors the role of the reference's c/dispatch.h:37-506, reduced to the packed-dots, packed-distance and symmetric slots
 *  (reference slots: c/dispatch.h:279-336, 353-380) for i8, u8, bf16, f16, e4m3, e5m2, e2m3, e3m2, i4, u4, u1, f32, f64.
 */
#ifndef NUMKONG_AMD_DISPATCH_H
#define NUMKONG_AMD_DISPATCH_H

#include "numkong_amd/dots.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    nk_dots_packed_size_punned_t dots_packed_size_i8, dots_packed_size_u8, dots_packed_size_bf16,
        dots_packed_size_f16, dots_packed_size_e4m3, dots_packed_size_e5m2, dots_packed_size_e2m3, dots_packed_size_e3m2,
        dots_packed_size_i4, dots_packed_size_u4, dots_packed_size_u1, dots_packed_size_f32, dots_packed_size_f64;
    nk_dots_pack_punned_t dots_pack_i8, dots_pack_u8, dots_pack_bf16, dots_pack_f16, dots_pack_e4m3, dots_pack_e5m2, dots_pack_e2m3, dots_pack_e3m2,
        dots_pack_i4, dots_pack_u4, dots_pack_u1, dots_pack_f32, dots_pack_f64;
    nk_dots_packed_punned_t dots_packed_i8, dots_packed_u8, dots_packed_bf16, dots_packed_f16, dots_packed_e4m3,
        dots_packed_e5m2, dots_packed_e2m3, dots_packed_e3m2,
        dots_packed_i4, dots_packed_u4, dots_packed_u1, dots_packed_f32, dots_packed_f64;
    nk_dots_packed_punned_t angulars_packed_i8, angulars_packed_u8, angulars_packed_bf16, angulars_packed_f16,
        angulars_packed_e4m3, angulars_packed_e5m2, angulars_packed_e2m3, angulars_packed_e3m2, angulars_packed_i4,
        angulars_packed_u4, angulars_packed_f32, angulars_packed_f64;
    nk_dots_packed_punned_t euclideans_packed_i8, euclideans_packed_u8, euclideans_packed_bf16, euclideans_packed_f16,
        euclideans_packed_e4m3, euclideans_packed_e5m2, euclideans_packed_e2m3, euclideans_packed_e3m2,
        euclideans_packed_i4, euclideans_packed_u4, euclideans_packed_f32, euclideans_packed_f64;
    nk_dots_symmetric_punned_t dots_symmetric_i8, dots_symmetric_u8, dots_symmetric_bf16, dots_symmetric_f16,
        dots_symmetric_e4m3, dots_symmetric_e5m2, dots_symmetric_e2m3, dots_symmetric_e3m2,
        dots_symmetric_i4, dots_symmetric_u4, dots_symmetric_u1, dots_symmetric_f32, dots_symmetric_f64;
    nk_dots_symmetric_punned_t angulars_symmetric_i8, angulars_symmetric_u8, angulars_symmetric_bf16,
        angulars_symmetric_f16, angulars_symmetric_e4m3, angulars_symmetric_e5m2, angulars_symmetric_e2m3,
        angulars_symmetric_e3m2, angulars_symmetric_i4, angulars_symmetric_u4, angulars_symmetric_f32,
        angulars_symmetric_f64;
    nk_dots_symmetric_punned_t euclideans_symmetric_i8, euclideans_symmetric_u8, euclideans_symmetric_bf16,
        euclideans_symmetric_f16, euclideans_symmetric_e4m3, euclideans_symmetric_e5m2, euclideans_symmetric_e2m3,
        euclideans_symmetric_e3m2, euclideans_symmetric_i4, euclideans_symmetric_u4, euclideans_symmetric_f32,
        euclideans_symmetric_f64;
} nk_implementations_t;

extern nk_implementations_t nk_dispatch_table;

/* Error stubs (reference: c/numkong.c:78-81, 195-216). */
void nk_error_dense_(void const *a, void const *b, nk_size_t n, void *d);
nk_size_t nk_error_packed_size_(nk_size_t n, nk_size_t k);
void nk_error_pack_(void const *b, nk_size_t n, nk_size_t k, nk_size_t b_stride, void *b_packed);
void nk_error_dots_(void const *a, void const *b_packed, void *c, nk_size_t m, nk_size_t n, nk_size_t k,
                    nk_size_t a_stride, nk_size_t c_stride);
void nk_error_dots_symmetric_(void const *vectors, nk_size_t n_vectors, nk_size_t depth, nk_size_t stride, void *result,
                              nk_size_t result_stride, nk_size_t row_start, nk_size_t row_count);
/* the same two for the types with 8-byte outputs (f32, f64) */
void nk_error_dots_wide_(void const *a, void const *b_packed, void *c, nk_size_t m, nk_size_t n, nk_size_t k,
                         nk_size_t a_stride, nk_size_t c_stride);
void nk_error_dots_symmetric_wide_(void const *vectors, nk_size_t n_vectors, nk_size_t depth, nk_size_t stride,
                                   void *result, nk_size_t result_stride, nk_size_t row_start, nk_size_t row_count);

/* Per-dtype lookup and table initialisation (reference: c/dispatch.h:483-506). */
#define NK_AMD_DECLARE_DISPATCH_(T)                                                                              \
    void nk_dispatch_##T##_find_(nk_capability_t viable, nk_kernel_kind_t kind, nk_kernel_punned_t *kernel,      \
                                 nk_capability_t *used);                                                         \
    void nk_dispatch_##T##_init_(nk_capability_t caps);
NK_AMD_DECLARE_DISPATCH_(i8)
NK_AMD_DECLARE_DISPATCH_(u8)
NK_AMD_DECLARE_DISPATCH_(bf16)
NK_AMD_DECLARE_DISPATCH_(f16)
NK_AMD_DECLARE_DISPATCH_(e4m3)
NK_AMD_DECLARE_DISPATCH_(e5m2)
NK_AMD_DECLARE_DISPATCH_(e2m3)
NK_AMD_DECLARE_DISPATCH_(e3m2)
NK_AMD_DECLARE_DISPATCH_(i4)
NK_AMD_DECLARE_DISPATCH_(u4)
NK_AMD_DECLARE_DISPATCH_(u1)
NK_AMD_DECLARE_DISPATCH_(f32)
NK_AMD_DECLARE_DISPATCH_(f64)
#undef NK_AMD_DECLARE_DISPATCH_

/**
 *  Body shared by the dispatch_<T>.c files of the twelve types with every kind. The reference walks a ladder of CPU ISAs per dtype
 *  (c/dispatch_i8.c:9-323); here there is one backend, so the ladder has one rung, and a kind this
 *  library does not implement falls through to the reference's error fallback (c/dispatch_i8.c:321-322).
 */
#define NK_AMD_DEFINE_DISPATCH_WITH_(T, dots_stub, symmetric_stub)                                                                                  \
    void nk_dispatch_##T##_find_(nk_capability_t v, nk_kernel_kind_t k, nk_kernel_punned_t *m, nk_capability_t *c) { \
        typedef nk_kernel_punned_t m_t;                                                                               \
        if (v & nk_cap_gfx950_k) switch (k) {                                                                         \
            case nk_kernel_dots_packed_size_k:                                                                        \
                *m = (m_t)&nk_dots_packed_size_##T##_gfx950, *c = nk_cap_gfx950_k;                                    \
                return;                                                                                               \
            case nk_kernel_dots_pack_k: *m = (m_t)&nk_dots_pack_##T##_gfx950, *c = nk_cap_gfx950_k; return;          \
            case nk_kernel_dots_packed_k: *m = (m_t)&nk_dots_packed_##T##_gfx950, *c = nk_cap_gfx950_k; return;      \
            case nk_kernel_angulars_packed_k: *m = (m_t)&nk_angulars_packed_##T##_gfx950, *c = nk_cap_gfx950_k; return; \
            case nk_kernel_euclideans_packed_k:                                                                       \
                *m = (m_t)&nk_euclideans_packed_##T##_gfx950, *c = nk_cap_gfx950_k;                                   \
                return;                                                                                               \
            case nk_kernel_dots_symmetric_k: *m = (m_t)&nk_dots_symmetric_##T##_gfx950, *c = nk_cap_gfx950_k; return; \
            case nk_kernel_angulars_symmetric_k:                                                                      \
                *m = (m_t)&nk_angulars_symmetric_##T##_gfx950, *c = nk_cap_gfx950_k;                                  \
                return;                                                                                               \
            case nk_kernel_euclideans_symmetric_k:                                                                    \
                *m = (m_t)&nk_euclideans_symmetric_##T##_gfx950, *c = nk_cap_gfx950_k;                                \
                return;                                                                                               \
            default: break;                                                                                           \
            }                                                                                                         \
        switch (k) {                                                                                                  \
        case nk_kernel_dots_packed_size_k: *m = (m_t)nk_error_packed_size_, *c = 0; return;                          \
        case nk_kernel_dots_pack_k: *m = (m_t)nk_error_pack_, *c = 0; return;                                        \
        case nk_kernel_dots_packed_k:                                                                                 \
        case nk_kernel_angulars_packed_k:                                                                             \
        case nk_kernel_euclideans_packed_k: *m = (m_t)dots_stub, *c = 0; return;                       \
        case nk_kernel_dots_symmetric_k:                                                                              \
        case nk_kernel_angulars_symmetric_k:                                                                          \
        case nk_kernel_euclideans_symmetric_k: *m = (m_t)symmetric_stub, *c = 0; return;       \
        default: *m = (m_t)nk_error_dense_, *c = 0; return;                                                          \
        }                                                                                                             \
    }                                                                                                                 \
    void nk_dispatch_##T##_init_(nk_capability_t caps) {                                                              \
        nk_implementations_t *t = &nk_dispatch_table;                                                                 \
        nk_capability_t used;                                                                                         \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_packed_size_k, (nk_kernel_punned_t *)&t->dots_packed_size_##T,  \
                                &used);                                                                               \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_pack_k, (nk_kernel_punned_t *)&t->dots_pack_##T, &used);         \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_packed_k, (nk_kernel_punned_t *)&t->dots_packed_##T, &used);     \
        nk_dispatch_##T##_find_(caps, nk_kernel_angulars_packed_k, (nk_kernel_punned_t *)&t->angulars_packed_##T,    \
                                &used);                                                                               \
        nk_dispatch_##T##_find_(caps, nk_kernel_euclideans_packed_k,                                                  \
                                (nk_kernel_punned_t *)&t->euclideans_packed_##T, &used);                              \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_symmetric_k, (nk_kernel_punned_t *)&t->dots_symmetric_##T,      \
                                &used);                                                                               \
        nk_dispatch_##T##_find_(caps, nk_kernel_angulars_symmetric_k,                                                 \
                                (nk_kernel_punned_t *)&t->angulars_symmetric_##T, &used);                             \
        nk_dispatch_##T##_find_(caps, nk_kernel_euclideans_symmetric_k,                                               \
                                (nk_kernel_punned_t *)&t->euclideans_symmetric_##T, &used);                           \
    }

#define NK_AMD_DEFINE_DISPATCH_(T) NK_AMD_DEFINE_DISPATCH_WITH_(T, nk_error_dots_, nk_error_dots_symmetric_)
/** ... and for the two types whose outputs are 8 bytes wide (f32, f64). */
#define NK_AMD_DEFINE_DISPATCH_WIDE_(T) NK_AMD_DEFINE_DISPATCH_WITH_(T, nk_error_dots_wide_, nk_error_dots_symmetric_wide_)

/** The same for the type that has the dot-product kinds only (u1). */
#define NK_AMD_DEFINE_DISPATCH_DOTS_WITH_(T, dots_stub, symmetric_stub)                                               \
    void nk_dispatch_##T##_find_(nk_capability_t v, nk_kernel_kind_t k, nk_kernel_punned_t *m, nk_capability_t *c) { \
        typedef nk_kernel_punned_t m_t;                                                                               \
        if (v & nk_cap_gfx950_k) switch (k) {                                                                         \
            case nk_kernel_dots_packed_size_k:                                                                        \
                *m = (m_t)&nk_dots_packed_size_##T##_gfx950, *c = nk_cap_gfx950_k;                                    \
                return;                                                                                               \
            case nk_kernel_dots_pack_k: *m = (m_t)&nk_dots_pack_##T##_gfx950, *c = nk_cap_gfx950_k; return;          \
            case nk_kernel_dots_packed_k: *m = (m_t)&nk_dots_packed_##T##_gfx950, *c = nk_cap_gfx950_k; return;      \
            case nk_kernel_dots_symmetric_k: *m = (m_t)&nk_dots_symmetric_##T##_gfx950, *c = nk_cap_gfx950_k; return; \
            default: break;                                                                                           \
            }                                                                                                         \
        switch (k) {                                                                                                  \
        case nk_kernel_dots_packed_size_k: *m = (m_t)nk_error_packed_size_, *c = 0; return;                          \
        case nk_kernel_dots_pack_k: *m = (m_t)nk_error_pack_, *c = 0; return;                                        \
        case nk_kernel_dots_packed_k:                                                                                 \
        case nk_kernel_angulars_packed_k:                                                                             \
        case nk_kernel_euclideans_packed_k: *m = (m_t)dots_stub, *c = 0; return;                                \
        case nk_kernel_dots_symmetric_k:                                                                              \
        case nk_kernel_angulars_symmetric_k:                                                                          \
        case nk_kernel_euclideans_symmetric_k: *m = (m_t)symmetric_stub, *c = 0; return;                   \
        default: *m = (m_t)nk_error_dense_, *c = 0; return;                                                          \
        }                                                                                                             \
    }                                                                                                                 \
    void nk_dispatch_##T##_init_(nk_capability_t caps) {                                                              \
        nk_implementations_t *t = &nk_dispatch_table;                                                                 \
        nk_capability_t used;                                                                                         \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_packed_size_k, (nk_kernel_punned_t *)&t->dots_packed_size_##T,  \
                                &used);                                                                               \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_pack_k, (nk_kernel_punned_t *)&t->dots_pack_##T, &used);         \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_packed_k, (nk_kernel_punned_t *)&t->dots_packed_##T, &used);     \
        nk_dispatch_##T##_find_(caps, nk_kernel_dots_symmetric_k, (nk_kernel_punned_t *)&t->dots_symmetric_##T,      \
                                &used);                                                                               \
    }

#define NK_AMD_DEFINE_DISPATCH_DOTS_(T) NK_AMD_DEFINE_DISPATCH_DOTS_WITH_(T, nk_error_dots_, nk_error_dots_symmetric_)

#ifdef __cplusplus
}
#endif

#endif // NUMKONG_AMD_DISPATCH_H
