/**
 *  @brief Exercises include/numkong_amd/matrix.hpp against plain loops: typed entry points, packed_matrix, distances,
 *         symmetric kinds, move semantics, a host-memory allocator.
 *  @file tests/cpp/test_matrix.cpp
 *
 *  Built by numkong_amd/csrc/Makefile into numkong_amd/lib/test_matrix and run by tests/test_containers.py. Prints one
 *  line per check; exits 0 when all hold. Without a GPU it checks that the containers refuse cleanly and says so.
 */
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "numkong_amd/matrix.hpp"

namespace {

int failures = 0;
void expect(bool ok, char const *what) {
    std::printf("%s: %s\n", ok ? "ok" : "FAILED", what);
    if (!ok) ++failures;
}

struct host_allocator {
    char *allocate(std::size_t bytes) noexcept { return static_cast<char *>(std::aligned_alloc(64, (bytes + 63) / 64 * 64)); }
    void deallocate(char *pointer, std::size_t) noexcept { std::free(pointer); }
};

float bf16_to_float(std::uint16_t bits) {
    std::uint32_t wide = static_cast<std::uint32_t>(bits) << 16;
    float value;
    std::memcpy(&value, &wide, 4);
    return value;
}
std::uint16_t float_to_bf16(float value) {
    std::uint32_t bits;
    std::memcpy(&bits, &value, 4);
    return static_cast<std::uint16_t>((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

} // namespace

int main() {
    using namespace nk_amd;
    std::mt19937 generator(7);
    std::size_t const m = 70, n = 45, k = 200;

    if (nk_hip_device_count() <= 0) {
        std::vector<nk_i8_t> b(n * k, 1);
        auto packed = packed_matrix<i8_t>::try_pack(b.data(), n, k, k);
        expect(packed.empty() && packed.rows() == 0 && packed.size_bytes() == 0, "no GPU: try_pack returns an empty matrix");
        std::vector<nk_i32_t> c(m * n, 0);
        std::vector<nk_i8_t> a(m * k, 1);
        expect(!dots_packed(a.data(), packed, c.data(), m, k, n * 4), "no GPU: the product over an empty matrix is refused");
        expect(dots_packed_size<i8_t>(n, k) == 64 + 2 * 16 * 512 + 2 * 256, "packed size needs no GPU");
        std::printf("no HIP device: containers refuse cleanly\n");
        return failures ? 1 : 0;
    }

    { // i8: exact, strided operands, device-resident image
        std::uniform_int_distribution<int> byte(-128, 127);
        std::size_t const a_stride = k + 8, b_stride = k + 3, c_stride = (n + 5) * 4;
        std::vector<nk_i8_t> a(m * a_stride), b(n * b_stride);
        for (auto &x : a) x = static_cast<nk_i8_t>(byte(generator));
        for (auto &x : b) x = static_cast<nk_i8_t>(byte(generator));
        auto packed = packed_matrix<i8_t>::try_pack(b.data(), n, k, b_stride);
        expect(!packed.empty() && packed.rows() == n && packed.depth() == k &&
                   packed.size_bytes() == dots_packed_size<i8_t>(n, k) && nk_hip_pointer_kind(packed.data()) == 1,
               "i8 try_pack: device-resident image of the announced size");
        std::vector<nk_i32_t> c(m * (n + 5), -7);
        bool const done = dots_packed(a.data(), packed, c.data(), m, a_stride, c_stride);
        bool exact = done;
        for (std::size_t i = 0; i < m && exact; ++i)
            for (std::size_t j = 0; j < n + 5; ++j) {
                long long sum = 0;
                for (std::size_t l = 0; l < k && j < n; ++l) sum += static_cast<long long>(a[i * a_stride + l]) * b[j * b_stride + l];
                if (c[i * (n + 5) + j] != (j < n ? static_cast<nk_i32_t>(sum) : -7)) exact = false;
            }
        expect(exact, "i8 dots_packed: exact, padding of C untouched");

        packed_matrix<i8_t> moved(std::move(packed));
        expect(packed.empty() && !moved.empty() && moved.rows() == n, "packed_matrix: move leaves the source empty");
        packed_matrix<i8_t> assigned;
        assigned = std::move(moved);
        std::vector<nk_i32_t> again(m * (n + 5), -7);
        expect(dots_packed(a.data(), assigned, again.data(), m, a_stride, c_stride) && again == c,
               "packed_matrix: a moved matrix computes the same product");

        // distances on the same image
        std::vector<nk_f32_t> angular(m * n), euclidean(m * n);
        bool ok = angulars_packed(a.data(), assigned, angular.data(), m, a_stride, n * 4) &&
                  euclideans_packed(a.data(), assigned, euclidean.data(), m, a_stride, n * 4);
        for (std::size_t i = 0; i < m && ok; ++i)
            for (std::size_t j = 0; j < n; ++j) {
                double dot = 0, aa = 0, bb = 0;
                for (std::size_t l = 0; l < k; ++l) {
                    double const x = a[i * a_stride + l], y = b[j * b_stride + l];
                    dot += x * y, aa += x * x, bb += y * y;
                }
                if (std::fabs(angular[i * n + j] - (1.0 - dot / std::sqrt(aa * bb))) > 1e-5) ok = false;
                if (std::fabs(euclidean[i * n + j] - std::sqrt(aa + bb - 2 * dot)) > 1e-3) ok = false;
            }
        expect(ok, "i8 angulars_packed / euclideans_packed: within 1e-5 / 1e-3 of the f64 formulas");

        // image in host memory: the product stages it
        auto on_host = packed_matrix<i8_t, host_allocator>::try_pack(b.data(), n, k, b_stride);
        std::vector<nk_i32_t> from_host(m * (n + 5), -7);
        expect(!on_host.empty() && nk_hip_pointer_kind(on_host.data()) == 0 &&
                   dots_packed(a.data(), on_host, from_host.data(), m, a_stride, c_stride) && from_host == c,
               "packed_matrix with a host allocator: same product");
    }

    { // bf16: against f64 sums
        std::normal_distribution<float> normal;
        std::vector<nk_bf16_t> a(m * k), b(n * k);
        for (auto &x : a) x = float_to_bf16(normal(generator));
        for (auto &x : b) x = float_to_bf16(normal(generator));
        auto packed = packed_matrix<bf16_t>::try_pack(b.data(), n, k, k * 2);
        std::vector<nk_f32_t> c(m * n);
        bool ok = dots_packed(a.data(), packed, c.data(), m, k * 2, n * 4);
        for (std::size_t i = 0; i < m && ok; ++i)
            for (std::size_t j = 0; j < n; ++j) {
                double sum = 0, magnitude = 0;
                for (std::size_t l = 0; l < k; ++l) {
                    double const product = static_cast<double>(bf16_to_float(a[i * k + l])) * bf16_to_float(b[j * k + l]);
                    sum += product, magnitude += std::fabs(product);
                }
                if (std::fabs(c[i * n + j] - sum) > 4e-7 * magnitude) ok = false;
            }
        expect(ok, "bf16 dots_packed: within 4e-7 of sum |a b| of the f64 sums");
    }

    { // i4: two nibbles per byte, depth counted in nibbles
        std::uniform_int_distribution<int> any(0, 255);
        std::size_t const bytes = k / 2;
        std::vector<nk_i4x2_t> a(m * bytes), b(n * bytes);
        for (auto &x : a) x = static_cast<nk_i4x2_t>(any(generator));
        for (auto &x : b) x = static_cast<nk_i4x2_t>(any(generator));
        auto packed = packed_matrix<i4x2_t>::try_pack(b.data(), n, k, bytes);
        std::vector<nk_i32_t> c(m * n);
        bool ok = dots_packed(a.data(), packed, c.data(), m, bytes, n * 4);
        auto nibble = [](nk_i4x2_t byte, int high) { return ((((byte >> (4 * high)) & 0xF) ^ 8) - 8); };
        for (std::size_t i = 0; i < m && ok; ++i)
            for (std::size_t j = 0; j < n; ++j) {
                int sum = 0;
                for (std::size_t l = 0; l < bytes; ++l)
                    sum += nibble(a[i * bytes + l], 0) * nibble(b[j * bytes + l], 0) + nibble(a[i * bytes + l], 1) * nibble(b[j * bytes + l], 1);
                if (c[i * n + j] != sum) ok = false;
            }
        expect(ok, "i4 dots_packed: exact against sign-extended nibbles");
        // distances of the 4-bit type: f32, from the same image
        std::vector<nk_f32_t> angular(m * n);
        ok = angulars_packed(a.data(), packed, angular.data(), m, bytes, n * 4);
        for (std::size_t i = 0; i < m && ok; ++i)
            for (std::size_t j = 0; j < n; ++j) {
                double dot = 0, aa = 0, bb = 0;
                for (std::size_t l = 0; l < bytes; ++l)
                    for (int high = 0; high < 2; ++high) {
                        double const x = nibble(a[i * bytes + l], high), y = nibble(b[j * bytes + l], high);
                        dot += x * y, aa += x * x, bb += y * y;
                    }
                double const expected = aa * bb > 0 ? std::fmax(1.0 - dot / std::sqrt(aa * bb), 0.0) : (dot == 0 ? 0.0 : 1.0);
                if (std::fabs(angular[i * n + j] - expected) > 1e-5) ok = false;
            }
        expect(ok, "i4 angulars_packed: within 1e-5 of the f64 formula");
    }

    { // f32: f64 results for the products and for the distances
        std::normal_distribution<float> normal;
        std::vector<nk_f32_t> a(m * k), b(n * k);
        for (auto &x : a) x = normal(generator);
        for (auto &x : b) x = normal(generator);
        auto packed = packed_matrix<f32_t>::try_pack(b.data(), n, k, k * 4);
        std::vector<nk_f64_t> c(m * n), euclidean(m * n);
        bool ok = dots_packed(a.data(), packed, c.data(), m, k * 4, n * 8) &&
                  euclideans_packed(a.data(), packed, euclidean.data(), m, k * 4, n * 8);
        for (std::size_t i = 0; i < m && ok; ++i)
            for (std::size_t j = 0; j < n; ++j) {
                double lanes[4] = {0, 0, 0, 0}, squared = 0; // the reference's four sums by k mod 4
                for (std::size_t l = 0; l < k; ++l) {
                    lanes[l & 3] += static_cast<double>(a[i * k + l]) * b[j * k + l];
                    double const d = static_cast<double>(a[i * k + l]) - b[j * k + l];
                    squared += d * d;
                }
                if (c[i * n + j] != ((lanes[0] + lanes[1]) + lanes[2]) + lanes[3]) ok = false;
                if (std::fabs(euclidean[i * n + j] - std::sqrt(squared)) > 1e-12 * std::sqrt(squared)) ok = false;
            }
        expect(ok, "f32 dots_packed: bit-exact against four f64 sums by k mod 4; euclideans_packed: f64, within 1e-12");
    }

    { // symmetric: upper triangle of a row window, the rest left alone
        std::uniform_int_distribution<int> byte(0, 255);
        std::size_t const count = 90, first = 11, rows = 50;
        std::vector<nk_u8_t> v(count * k);
        for (auto &x : v) x = static_cast<nk_u8_t>(byte(generator));
        std::vector<nk_u32_t> result(count * count, 0xABCDEF01u);
        dots_symmetric<u8_t>(v.data(), count, k, k, result.data(), count * 4, first, rows);
        bool ok = true;
        for (std::size_t i = 0; i < count && ok; ++i)
            for (std::size_t j = 0; j < count; ++j) {
                bool const owned = i >= first && i < first + rows && j >= i;
                unsigned long long sum = 0;
                for (std::size_t l = 0; l < k && owned; ++l) sum += static_cast<unsigned long long>(v[i * k + l]) * v[j * k + l];
                if (result[i * count + j] != (owned ? static_cast<nk_u32_t>(sum) : 0xABCDEF01u)) ok = false;
            }
        expect(ok, "u8 dots_symmetric: owned elements exact, everything else untouched");
        std::vector<nk_f32_t> distance(count * count, -3.0f);
        euclideans_symmetric<u8_t>(v.data(), count, k, k, distance.data(), count * 4, 0, count);
        ok = true;
        for (std::size_t i = 0; i < count && ok; ++i) {
            if (distance[i * count + i] != 0.0f) ok = false;
            for (std::size_t j = i + 1; j < count; ++j) {
                double squared = 0;
                for (std::size_t l = 0; l < k; ++l) {
                    double const d = static_cast<double>(v[i * k + l]) - v[j * k + l];
                    squared += d * d;
                }
                if (std::fabs(distance[i * count + j] - std::sqrt(squared)) > 1e-3 * std::sqrt(squared)) ok = false;
                if (distance[j * count + i] != -3.0f) ok = false;
            }
        }
        expect(ok, "u8 euclideans_symmetric: zero diagonal, upper triangle right, lower triangle untouched");
    }

    std::printf("%s\n", failures ? "some checks FAILED" : "all container checks passed");
    return failures ? 1 : 0;
}
