/**
 *  @brief C++ containers over the C ABI of <numkong_amd/dots.h>: typed entry points and an owning packed matrix.
 *  @file include/numkong_amd/matrix.hpp
 *
 *  Counterpart of the reference's C++ layer for this path: the typed free functions `dots_packed_size`, `dots_pack`,
 *  `dots_packed` (include/numkong/dots.hpp:94-150) and the owning, move-only `packed_matrix<T>` with `try_pack`
 *  (include/numkong/matrix.hpp:170-253), plus the distance and symmetric forms. C++17, header only, nothing but the C
 *  ABI underneath, so it follows that ABI's rules: pointers may be host or device memory, strides are bytes, calls are
 *  synchronous.
 *
 *  What differs from the reference's container: the packed image lives in DEVICE memory by default (allocated with
 *  `nk_hip_malloc`), because that is where the product reads it without staging; `device_allocator` can be replaced
 *  by any allocator of bytes with `allocate(n)` / `deallocate(p, n)`, e.g. one that hands out host memory.
 *
 *      using namespace nk_amd;
 *      auto packed = packed_matrix<bf16_t>::try_pack(b, rows_of_b, depth, b_stride_bytes);
 *      if (!packed.empty()) dots_packed(a, packed, c, rows_of_a, a_stride_bytes, c_stride_bytes);
 */
#ifndef NUMKONG_AMD_MATRIX_HPP
#define NUMKONG_AMD_MATRIX_HPP

#include <cstddef>
#include <utility>

#include "numkong_amd/dots.h"
#include "numkong_amd/hip_abi.h"

namespace nk_amd {

/** One tag per element type: its storage type, the type of its dot products, its code, its entry points. */
#define NK_AMD_DEFINE_TYPE_(name, raw, result, dimensions)                                                        \
    struct name##_t {                                                                                             \
        using raw_t = raw;                                                                                        \
        using dot_result_t = result;                                                                              \
        static constexpr nk_dtype_t dtype = nk_##name##_k;                                                        \
        static constexpr std::size_t dimensions_per_value = dimensions;                                           \
        static nk_size_t packed_size(nk_size_t n, nk_size_t k) noexcept { return nk_dots_packed_size_##name(n, k); } \
        static void pack(raw const *b, nk_size_t n, nk_size_t k, nk_size_t stride, void *packed) noexcept {       \
            nk_dots_pack_##name(b, n, k, stride, packed);                                                         \
        }                                                                                                         \
        static void packed(raw const *a, void const *b, result *c, nk_size_t m, nk_size_t n, nk_size_t k,         \
                           nk_size_t a_stride, nk_size_t c_stride) noexcept {                                     \
            nk_dots_packed_##name(a, b, c, m, n, k, a_stride, c_stride);                                          \
        }                                                                                                         \
        static void symmetric(raw const *v, nk_size_t n, nk_size_t k, nk_size_t stride, result *out,              \
                              nk_size_t out_stride, nk_size_t row_start, nk_size_t row_count) noexcept {          \
            nk_dots_symmetric_##name(v, n, k, stride, out, out_stride, row_start, row_count);                     \
        }                                                                                                         \
    };
NK_AMD_DEFINE_TYPE_(i8, nk_i8_t, nk_i32_t, 1)
NK_AMD_DEFINE_TYPE_(u8, nk_u8_t, nk_u32_t, 1)
NK_AMD_DEFINE_TYPE_(bf16, nk_bf16_t, nk_f32_t, 1)
NK_AMD_DEFINE_TYPE_(f16, nk_f16_t, nk_f32_t, 1)
NK_AMD_DEFINE_TYPE_(e4m3, nk_e4m3_t, nk_f32_t, 1)
NK_AMD_DEFINE_TYPE_(e5m2, nk_e5m2_t, nk_f32_t, 1)
NK_AMD_DEFINE_TYPE_(e2m3, nk_e2m3_t, nk_f32_t, 1)
NK_AMD_DEFINE_TYPE_(e3m2, nk_e3m2_t, nk_f32_t, 1)
NK_AMD_DEFINE_TYPE_(f32, nk_f32_t, nk_f64_t, 1)
NK_AMD_DEFINE_TYPE_(f64, nk_f64_t, nk_f64_t, 1)
#undef NK_AMD_DEFINE_TYPE_
/* the sub-byte types are named after their storage in the C ABI: two 4-bit or eight 1-bit values to a byte */
struct i4x2_t {
    using raw_t = nk_i4x2_t;
    using dot_result_t = nk_i32_t;
    static constexpr nk_dtype_t dtype = nk_i4_k;
    static constexpr std::size_t dimensions_per_value = 2;
    static nk_size_t packed_size(nk_size_t n, nk_size_t k) noexcept { return nk_dots_packed_size_i4(n, k); }
    static void pack(raw_t const *b, nk_size_t n, nk_size_t k, nk_size_t stride, void *packed) noexcept {
        nk_dots_pack_i4(b, n, k, stride, packed);
    }
    static void packed(raw_t const *a, void const *b, dot_result_t *c, nk_size_t m, nk_size_t n, nk_size_t k,
                       nk_size_t a_stride, nk_size_t c_stride) noexcept {
        nk_dots_packed_i4(a, b, c, m, n, k, a_stride, c_stride);
    }
    static void symmetric(raw_t const *v, nk_size_t n, nk_size_t k, nk_size_t stride, dot_result_t *out,
                          nk_size_t out_stride, nk_size_t row_start, nk_size_t row_count) noexcept {
        nk_dots_symmetric_i4(v, n, k, stride, out, out_stride, row_start, row_count);
    }
};
struct u4x2_t {
    using raw_t = nk_u4x2_t;
    using dot_result_t = nk_u32_t;
    static constexpr nk_dtype_t dtype = nk_u4_k;
    static constexpr std::size_t dimensions_per_value = 2;
    static nk_size_t packed_size(nk_size_t n, nk_size_t k) noexcept { return nk_dots_packed_size_u4(n, k); }
    static void pack(raw_t const *b, nk_size_t n, nk_size_t k, nk_size_t stride, void *packed) noexcept {
        nk_dots_pack_u4(b, n, k, stride, packed);
    }
    static void packed(raw_t const *a, void const *b, dot_result_t *c, nk_size_t m, nk_size_t n, nk_size_t k,
                       nk_size_t a_stride, nk_size_t c_stride) noexcept {
        nk_dots_packed_u4(a, b, c, m, n, k, a_stride, c_stride);
    }
    static void symmetric(raw_t const *v, nk_size_t n, nk_size_t k, nk_size_t stride, dot_result_t *out,
                          nk_size_t out_stride, nk_size_t row_start, nk_size_t row_count) noexcept {
        nk_dots_symmetric_u4(v, n, k, stride, out, out_stride, row_start, row_count);
    }
};

struct u1x8_t {
    using raw_t = nk_u1x8_t;
    using dot_result_t = nk_u32_t;
    static constexpr nk_dtype_t dtype = nk_u1_k;
    static constexpr std::size_t dimensions_per_value = 8;
    static nk_size_t packed_size(nk_size_t n, nk_size_t k) noexcept { return nk_dots_packed_size_u1(n, k); }
    static void pack(raw_t const *b, nk_size_t n, nk_size_t k, nk_size_t stride, void *packed) noexcept {
        nk_dots_pack_u1(b, n, k, stride, packed);
    }
    static void packed(raw_t const *a, void const *b, dot_result_t *c, nk_size_t m, nk_size_t n, nk_size_t k,
                       nk_size_t a_stride, nk_size_t c_stride) noexcept {
        nk_dots_packed_u1(a, b, c, m, n, k, a_stride, c_stride);
    }
    static void symmetric(raw_t const *v, nk_size_t n, nk_size_t k, nk_size_t stride, dot_result_t *out,
                          nk_size_t out_stride, nk_size_t row_start, nk_size_t row_count) noexcept {
        nk_dots_symmetric_u1(v, n, k, stride, out, out_stride, row_start, row_count);
    }
};

/** The distance kinds exist for every type but u1; `distances<T>` names their entry points and their result type
 *  (f32; f64 for f32 and f64 inputs). */
template <typename value_type_>
struct distances;
#define NK_AMD_DEFINE_DISTANCES_(tag, name, result)                                                                           \
    template <>                                                                                                   \
    struct distances<tag> {                                                                               \
        using raw_t = tag::raw_t;                                                                         \
        using distance_t = result;                                                                         \
        static void angulars_packed(raw_t const *a, void const *b, distance_t *c, nk_size_t m, nk_size_t n,         \
                                    nk_size_t k, nk_size_t a_stride, nk_size_t c_stride) noexcept {               \
            nk_angulars_packed_##name(a, b, c, m, n, k, a_stride, c_stride);                                      \
        }                                                                                                         \
        static void euclideans_packed(raw_t const *a, void const *b, distance_t *c, nk_size_t m, nk_size_t n,       \
                                      nk_size_t k, nk_size_t a_stride, nk_size_t c_stride) noexcept {             \
            nk_euclideans_packed_##name(a, b, c, m, n, k, a_stride, c_stride);                                    \
        }                                                                                                         \
        static void angulars_symmetric(raw_t const *v, nk_size_t n, nk_size_t k, nk_size_t stride, distance_t *out, \
                                       nk_size_t out_stride, nk_size_t row_start, nk_size_t row_count) noexcept { \
            nk_angulars_symmetric_##name(v, n, k, stride, out, out_stride, row_start, row_count);                 \
        }                                                                                                         \
        static void euclideans_symmetric(raw_t const *v, nk_size_t n, nk_size_t k, nk_size_t stride,              \
                                         distance_t *out, nk_size_t out_stride, nk_size_t row_start,                \
                                         nk_size_t row_count) noexcept {                                          \
            nk_euclideans_symmetric_##name(v, n, k, stride, out, out_stride, row_start, row_count);               \
        }                                                                                                         \
    };
NK_AMD_DEFINE_DISTANCES_(i8_t, i8, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(u8_t, u8, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(bf16_t, bf16, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(f16_t, f16, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(e4m3_t, e4m3, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(e5m2_t, e5m2, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(e2m3_t, e2m3, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(e3m2_t, e3m2, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(i4x2_t, i4, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(u4x2_t, u4, nk_f32_t)
NK_AMD_DEFINE_DISTANCES_(f32_t, f32, nk_f64_t)
NK_AMD_DEFINE_DISTANCES_(f64_t, f64, nk_f64_t)
#undef NK_AMD_DEFINE_DISTANCES_

/** Bytes of device memory; what `packed_matrix` keeps its image in unless told otherwise. */
struct device_allocator {
    char *allocate(std::size_t bytes) noexcept {
        void *pointer = nullptr;
        return nk_hip_malloc(&pointer, bytes) == 0 ? static_cast<char *>(pointer) : nullptr;
    }
    void deallocate(char *pointer, std::size_t) noexcept { (void)nk_hip_free(pointer); }
};

/** Typed forms of the three packed-dots entry points (reference: include/numkong/dots.hpp:94-150). `depth` counts
 *  dimensions (4-bit values for the 4-bit types), strides count bytes. */
template <typename value_type_>
std::size_t dots_packed_size(std::size_t rows, std::size_t depth) noexcept {
    return value_type_::packed_size(rows, depth);
}
template <typename value_type_>
void dots_pack(typename value_type_::raw_t const *b, std::size_t rows, std::size_t depth, std::size_t b_stride_bytes,
               void *b_packed) noexcept {
    value_type_::pack(b, rows, depth, b_stride_bytes, b_packed);
}
template <typename value_type_>
void dots_packed(typename value_type_::raw_t const *a, void const *b_packed, typename value_type_::dot_result_t *c,
                 std::size_t row_count, std::size_t column_count, std::size_t depth, std::size_t a_stride_bytes,
                 std::size_t c_stride_bytes) noexcept {
    value_type_::packed(a, b_packed, c, row_count, column_count, depth, a_stride_bytes, c_stride_bytes);
}

/**
 *  Owning, move-only, pre-packed matrix B (reference: include/numkong/matrix.hpp:170-253; same members).
 *  `try_pack` returns an empty object on failure (no GPU, unsupported dimensions, out of memory), never throws.
 */
template <typename value_type_, typename allocator_type_ = device_allocator>
struct packed_matrix {
    using value_type = value_type_;
    using result_type = typename value_type_::dot_result_t;
    using allocator_type = allocator_type_;
    using size_type = std::size_t;

  private:
    char *data_ = nullptr;
    size_type size_bytes_ = 0;
    size_type rows_ = 0;
    size_type depth_ = 0;
    allocator_type_ alloc_;

  public:
    packed_matrix() noexcept = default;
    explicit packed_matrix(allocator_type_ const &alloc) noexcept : alloc_(alloc) {}
    ~packed_matrix() noexcept {
        if (data_) alloc_.deallocate(data_, size_bytes_);
    }
    packed_matrix(packed_matrix &&other) noexcept
        : data_(std::exchange(other.data_, nullptr)), size_bytes_(std::exchange(other.size_bytes_, 0)),
          rows_(std::exchange(other.rows_, 0)), depth_(std::exchange(other.depth_, 0)), alloc_(std::move(other.alloc_)) {}
    packed_matrix &operator=(packed_matrix &&other) noexcept {
        if (this != &other) {
            if (data_) alloc_.deallocate(data_, size_bytes_);
            alloc_ = std::move(other.alloc_);
            data_ = std::exchange(other.data_, nullptr);
            size_bytes_ = std::exchange(other.size_bytes_, 0);
            rows_ = std::exchange(other.rows_, 0);
            depth_ = std::exchange(other.depth_, 0);
        }
        return *this;
    }
    packed_matrix(packed_matrix const &) = delete;
    packed_matrix &operator=(packed_matrix const &) = delete;

    /** Pack `rows` rows of `depth` dimensions, `b_stride_bytes` apart, host or device memory. */
    [[nodiscard]] static packed_matrix try_pack(typename value_type_::raw_t const *b, size_type rows, size_type depth,
                                                size_type b_stride_bytes, allocator_type_ alloc = {}) noexcept {
        packed_matrix packed(alloc);
        size_type const bytes = value_type_::packed_size(rows, depth);
        if (bytes == 0) return packed;
        char *data = packed.alloc_.allocate(bytes);
        if (!data) return packed;
        value_type_::pack(b, rows, depth, b_stride_bytes, data);
        char const *error = nk_amd_last_error();
        if (error && error[0]) {
            packed.alloc_.deallocate(data, bytes);
            return packed;
        }
        packed.data_ = data, packed.size_bytes_ = bytes, packed.rows_ = rows, packed.depth_ = depth;
        return packed;
    }

    constexpr size_type rows() const noexcept { return rows_; }
    constexpr size_type depth() const noexcept { return depth_; }
    constexpr size_type size_bytes() const noexcept { return size_bytes_; }
    constexpr bool empty() const noexcept { return data_ == nullptr; }
    constexpr void const *data() const noexcept { return data_; }
};

/** C = A * B^T against a packed B; false if B is empty (reference: include/numkong/dots.hpp:557-567). */
template <typename value_type_, typename allocator_type_>
bool dots_packed(typename value_type_::raw_t const *a, packed_matrix<value_type_, allocator_type_> const &b,
                 typename value_type_::dot_result_t *c, std::size_t row_count, std::size_t a_stride_bytes,
                 std::size_t c_stride_bytes) noexcept {
    if (b.empty()) return false;
    value_type_::packed(a, b.data(), c, row_count, b.rows(), b.depth(), a_stride_bytes, c_stride_bytes);
    return true;
}
template <typename value_type_, typename allocator_type_>
bool angulars_packed(typename value_type_::raw_t const *a, packed_matrix<value_type_, allocator_type_> const &b,
                     typename distances<value_type_>::distance_t *c, std::size_t row_count, std::size_t a_stride_bytes, std::size_t c_stride_bytes) noexcept {
    if (b.empty()) return false;
    distances<value_type_>::angulars_packed(a, b.data(), c, row_count, b.rows(), b.depth(), a_stride_bytes, c_stride_bytes);
    return true;
}
template <typename value_type_, typename allocator_type_>
bool euclideans_packed(typename value_type_::raw_t const *a, packed_matrix<value_type_, allocator_type_> const &b,
                       typename distances<value_type_>::distance_t *c, std::size_t row_count, std::size_t a_stride_bytes, std::size_t c_stride_bytes) noexcept {
    if (b.empty()) return false;
    distances<value_type_>::euclideans_packed(a, b.data(), c, row_count, b.rows(), b.depth(), a_stride_bytes, c_stride_bytes);
    return true;
}

/** Upper triangle of all pairs of one set of vectors, rows [row_start, row_start + row_count) of the result. */
template <typename value_type_>
void dots_symmetric(typename value_type_::raw_t const *vectors, std::size_t count, std::size_t depth,
                    std::size_t stride_bytes, typename value_type_::dot_result_t *result, std::size_t result_stride_bytes,
                    std::size_t row_start, std::size_t row_count) noexcept {
    value_type_::symmetric(vectors, count, depth, stride_bytes, result, result_stride_bytes, row_start, row_count);
}
template <typename value_type_>
void angulars_symmetric(typename value_type_::raw_t const *vectors, std::size_t count, std::size_t depth,
                        std::size_t stride_bytes, typename distances<value_type_>::distance_t *result, std::size_t result_stride_bytes, std::size_t row_start,
                        std::size_t row_count) noexcept {
    distances<value_type_>::angulars_symmetric(vectors, count, depth, stride_bytes, result, result_stride_bytes, row_start,
                                               row_count);
}
template <typename value_type_>
void euclideans_symmetric(typename value_type_::raw_t const *vectors, std::size_t count, std::size_t depth,
                          std::size_t stride_bytes, typename distances<value_type_>::distance_t *result, std::size_t result_stride_bytes,
                          std::size_t row_start, std::size_t row_count) noexcept {
    distances<value_type_>::euclideans_symmetric(vectors, count, depth, stride_bytes, result, result_stride_bytes, row_start,
                                                 row_count);
}

} // namespace nk_amd

#endif // NUMKONG_AMD_MATRIX_HPP
