/**
 *  @brief The f32 and f64 members of the packed-dots family on gfx950: f64 results.
 *  @file numkong_amd/csrc/dots_gfx950_wide.hip
 *
 *  Replaces `nk_dots_{packed_size,pack,packed,symmetric}_{f32,f64}_<isa>` (reference instantiations:
 *  include/numkong/dots/serial.h:2458-2491; arithmetic: include/numkong/dot/serial.h:262-335,
 *  include/numkong/scalar/serial.h:128-136, include/numkong/reduce/serial.h:33-48). Both produce f64:
 *
 *    f32  every product is exact in f64; four running f64 sums take the products by k mod 4 and are combined as
 *         ((s0 + s1) + s2) + s3. Runs on the f64 matrix cores (`dots_f32_matrix_kernel`): one MFMA is a chain of
 *         fused multiply-adds along its depth, which is exactly how the reference advances one of its four sums.
 *    f64  compensated ("dot2"): two lanes by k mod 2, each a running sum plus the accumulated rounding errors of its
 *         products (by FMA) and of its additions (TwoSum); the four numbers are folded by one more chain of TwoSums.
 *         No matrix form exists for that, so it is a register-tiled kernel on the vector units, which on MI355X run
 *         f64 at the rate of the f64 matrix instructions (78.6 TFLOP/s either way): 256 threads compute a 64 x 64
 *         tile of C, 4 x 4 outputs each, A through LDS transposed (k-major).
 *
 *  Either way every output keeps the reference's own accumulators and takes its terms in the reference's own order
 *  along k, so the results are those of its serial kernels bit for bit. B comes from an image that is already k-major
 *  f64: [64-byte header][k padded to 32][n padded to 64] doubles, zeros in the padding, then a sum of squares per
 *  padded column for the distance kinds (`nk_{angulars,euclideans}_{packed,symmetric}_{f32,f64}`, reference
 *  include/numkong/spatials/serial.h:41-72), which finalise the same dot products in the epilogue.
 */
#include <type_traits>
#include "dots_gfx950.hpp"

// Every floating-point operation in this file rounds on its own (the compensated sums depend on it; the fused
// multiply-adds that are meant are written as such).
#pragma clang fp contract(off)

namespace {

constexpr int kWideTile = 64;  // rows and columns of C per workgroup
constexpr int kWideDepth = 8;  // k per step through LDS

struct WideArgs {
    uint8_t const *a;
    double const *b; // the image's doubles, right behind its header: element (k, column) at b[k * n_padded + column]
    int dtype;
    uint8_t *c;
    uint64_t a_stride, c_stride;
    uint32_t m, n, k, n_padded, k_padded;
    uint32_t tri_shift, tri_mask; // symmetric form: store only col >= row + tri_shift (mask all ones), see GemmArgs
    int metric;                   // 0: dot products, 1: angular, 2: euclidean distances (f64, like the products)
};

/** A running sum in two numbers: the rounded sum and what the additions so far have lost (each addition's error is
 *  recovered exactly by TwoSum). `value()` is then within a rounding of the exact sum of the terms. */
struct CompensatedSum {
    double sum = 0, lost = 0;
    __device__ __forceinline__ void add(double term) {
#pragma clang fp contract(off)
        double const tentative = sum + term;
        double const recovered = tentative - sum;
        lost += (sum - (tentative - recovered)) + (term - recovered);
        sum = tentative;
    }
    __device__ __forceinline__ void add(CompensatedSum const &other) { add(other.sum), lost += other.lost; }
    __device__ __forceinline__ double value() const { return sum + lost; }
};

/** The reference's f64 reciprocal square root (scalar/serial.h:35-45): bit-trick estimate, four Newton steps; and its
 *  finalisers for f32 and f64 inputs (spatial/serial.h:281-302). Contraction off: every operation rounds on its own. */
__device__ __forceinline__ double wide_rsqrt(double number) {
#pragma clang fp contract(off)
    double y = __builtin_bit_cast(double, 0x5FE6EB50C7B537A9ull - (__builtin_bit_cast(uint64_t, number) >> 1));
#pragma unroll
    for (int step = 0; step < 4; ++step) y = y * (1.5 - 0.5 * number * y * y);
    return y;
}
__device__ __forceinline__ double wide_distance(int metric, double dot, double query, double target) {
#pragma clang fp contract(off)
    if (metric == 1) {
        double const product = query * target;
        if (product > 0) {
            double const result = 1.0 - dot * wide_rsqrt(product);
            return result > 0 ? result : 0;
        }
        return dot == 0 ? 0.0 : 1.0;
    }
    double const squared = query + target - 2.0 * dot;
    return squared > 0 ? squared * wide_rsqrt(squared) : 0.0;
}

/** Sum of squares of every row of B (f32 or f64, row-major) in f64, behind the image's matrix: one wavefront per
 *  row, a compensated sum per lane over every 64th element, the lanes folded the same way. The reference sums the
 *  rounded squares one after the other with a compensation (reduce/serial.h:50-92); this is the same quantity to
 *  within a rounding, in another order. */
template <bool F64>
__global__ __launch_bounds__(256) void wide_norms_kernel(uint8_t const *__restrict__ b, uint64_t b_stride, uint32_t n,
                                                         uint32_t k, uint32_t n_padded, double *__restrict__ norms) {
    uint32_t const lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_padded) return;
    CompensatedSum total;
    if (row < n) {
        uint8_t const *source = b + (uint64_t)row * b_stride;
        for (uint32_t at = lane; at < k; at += 64) {
#pragma clang fp contract(off)
            double const value = F64 ? ((double const *)source)[at] : (double)((float const *)source)[at];
            total.add(value * value);
        }
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        CompensatedSum other;
        other.sum = __shfl_xor(total.sum, offset), other.lost = __shfl_xor(total.lost, offset);
        total.add(other);
    }
    if (lane == 0) norms[row] = total.value(); // (padding columns: 0)
}


/** B (n rows of k elements, row-major, f32 or f64) -> k-major f64 with zero padding; 32 x 32 blocks through LDS so
 *  that both sides are touched in runs. */
template <bool F64>
__global__ __launch_bounds__(256) void pack_wide_kernel(uint8_t const *__restrict__ b, uint64_t b_stride, uint32_t n,
                                                        uint32_t k, uint32_t n_padded, double *__restrict__ out,
                                                        PackedHeader header, uint32_t k_first) {
    __shared__ double block[32][33];
    if (blockIdx.x == 0 && blockIdx.y == 0 && k_first == 0 && threadIdx.x == 0) *(PackedHeader *)((uint8_t *)out - sizeof(PackedHeader)) = header;
    uint32_t const row0 = blockIdx.x * 32, k0 = k_first + blockIdx.y * 32; // (k_first: a grid covers 65535 blocks of depth at most)
    uint32_t const tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t const row = row0 + ty + 8 * i, at = k0 + tx;
        double value = 0;
        if (row < n && at < k) {
            uint8_t const *source = b + (uint64_t)row * b_stride;
            value = F64 ? ((double const *)source)[at] : (double)((float const *)source)[at];
        }
        block[ty + 8 * i][tx] = value;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t const at = k0 + ty + 8 * i, row = row0 + tx; // (padding rows and depths are written too, as zeros)
        out[(uint64_t)at * n_padded + row] = block[tx][ty + 8 * i];
    }
}

/** One step of the reference's compensated dot product (scalar/serial.h:128-136), contraction off: every operation
 *  below rounds on its own, which is what makes the recovered errors exact. */
__device__ __forceinline__ void dot2_step(double &sum, double &compensation, double a, double b) {
#pragma clang fp contract(off)
    double const product = a * b;
    double const product_error = __builtin_fma(a, b, -product);
    double const running = sum + product;
    double const recovered = running - sum;
    double const sum_error = (sum - (running - recovered)) + (product - recovered);
    sum = running;
    compensation += sum_error + product_error;
}

/** reduce/serial.h:33-48 over (s0, c0, s1, c1). */
__device__ __forceinline__ double fold_compensated(double const (&lane)[4]) {
#pragma clang fp contract(off)
    double running = 0, error = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) { // order: sum of lane 0, its compensation, sum of lane 1, its compensation
        double const value = lane[i];
        double const tentative = running + value;
        double const recovered = tentative - running;
        error += (running - (tentative - recovered)) + (value - recovered);
        running = tentative;
    }
    return running + error;
}

template <bool NORMS>
__global__ __launch_bounds__(256) void dots_f64_compensated_kernel(WideArgs g) {
    __shared__ double a_lds[2][kWideDepth][kWideTile + 1];
    __shared__ double b_lds[2][kWideDepth][kWideTile];
    __shared__ double row_parts[NORMS ? kWideTile : 1][4][2]; // distances: four partial sums of squares per row of A
    __shared__ double row_norms[NORMS ? kWideTile : 1];
    uint32_t const tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    uint32_t const row0 = blockIdx.y * kWideTile, col0 = blockIdx.x * kWideTile;
    // symmetric form: a tile wholly left of the diagonal has nothing to store
    if (((row0 + g.tri_shift) & g.tri_mask) > col0 + (kWideTile - 1)) return;
    typedef __attribute__((address_space(1))) double global_f64_t;
    typedef __attribute__((address_space(1))) uint64_t global_u64_t;
    // Trust, but verify: an image packed for another type or other dimensions poisons the outputs (all bits set),
    // the reference's error convention, instead of being read with this call's geometry.
    PackedHeader const *header = (PackedHeader const *)((uint8_t const *)g.b - sizeof(PackedHeader));
    if (!(header->magic == kMagic && header->version == kVersion && header->dtype == (uint32_t)g.dtype && header->n == g.n &&
          header->k == g.k)) {
        for (uint32_t at = tid; at < kWideTile * kWideTile; at += 256) {
            uint32_t const row = row0 + at / kWideTile, col = col0 + at % kWideTile;
            if (row < g.m && col < g.n && ((row + g.tri_shift) & g.tri_mask) <= col)
                *(global_u64_t *)(g.c + (uint64_t)row * g.c_stride + (uint64_t)col * 8) = ~0ull;
        }
        return;
    }

    // accumulators: per output, four numbers: (s0, c0, s1, c1)
    double acc[4][4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][j][v] = 0;

    // staging: A: thread t brings 2 consecutive k of row t / 4 ... (64 rows x 8 k = 512 values, 2 per thread);
    //          B: thread t brings 2 consecutive columns of depth t / 32 (8 x 64 = 512 values, 2 per thread)
    uint32_t const a_row = tid >> 2, a_k = (tid & 3) * 2;
    uint32_t const b_k = tid >> 5, b_col = (tid & 31) * 2;
    uint8_t const *a_source = g.a + (uint64_t)(row0 + a_row < g.m ? row0 + a_row : 0) * g.a_stride;
    bool const a_exists = row0 + a_row < g.m;
    double a_next[2], b_next[2];
    CompensatedSum squares; // distances: of this thread's share of its row of A
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            uint32_t const at = k0 + a_k + e;
            double value = 0;
            if (a_exists && at < g.k) value = ((double const *)a_source)[at];
            a_next[e] = value;
            if (NORMS) squares.add(value * value);
        }
        double const *b_source = g.b + (uint64_t)(k0 + b_k) * g.n_padded + col0 + b_col; // (inside the padded image)
        b_next[0] = b_source[0], b_next[1] = b_source[1];
    };
    auto stash = [&](int buffer) {
        a_lds[buffer][a_k][a_row] = a_next[0], a_lds[buffer][a_k + 1][a_row] = a_next[1];
        b_lds[buffer][b_k][b_col] = b_next[0], b_lds[buffer][b_k][b_col + 1] = b_next[1];
    };

    // The reference pads a row with zeros to its step of 2 values and runs them through the sums like any other;
    // so does this, and no further.
    uint32_t const depth = (g.k + 1) & ~1u;
    fetch(0);
    stash(0);
    __syncthreads();
    int buffer = 0;
    for (uint32_t k0 = 0; k0 < depth; k0 += kWideDepth) {
        bool const more = k0 + kWideDepth < depth;
        if (more) fetch(k0 + kWideDepth);
#pragma unroll
        for (int kk = 0; kk < kWideDepth; ++kk) {
            if (k0 + kk >= depth) break; // (uniform; only the last step can be short)
            double a_value[4], b_value[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a_value[i] = a_lds[buffer][kk][ty + 16 * i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b_value[j] = b_lds[buffer][kk][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    dot2_step(acc[i][j][2 * (kk & 1)], acc[i][j][2 * (kk & 1) + 1], a_value[i], b_value[j]);
                }
        }
        if (more) stash(buffer ^ 1);
        __syncthreads();
        buffer ^= 1;
    }

    double column_norm[4];
    if (NORMS) {
        row_parts[a_row][tid & 3][0] = squares.sum, row_parts[a_row][tid & 3][1] = squares.lost;
        __syncthreads();
        if (tid < kWideTile) {
            CompensatedSum total;
#pragma unroll
            for (int part = 0; part < 4; ++part) {
                CompensatedSum one;
                one.sum = row_parts[tid][part][0], one.lost = row_parts[tid][part][1];
                total.add(one);
            }
            row_norms[tid] = total.value();
        }
        __syncthreads();
        double const *norms = g.b + (uint64_t)g.k_padded * g.n_padded; // behind the matrix, one per padded column
#pragma unroll
        for (int j = 0; j < 4; ++j) column_norm[j] = norms[col0 + tx + 16 * j];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        uint32_t const row = row0 + ty + 16 * i;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t const col = col0 + tx + 16 * j;
            double result = fold_compensated(acc[i][j]);
            if (NORMS) {
                result = wide_distance(g.metric, result, row_norms[ty + 16 * i], column_norm[j]);
                if (g.tri_mask && row + g.tri_shift == col) result = 0; // a vector and itself: exactly 0
            }
            if (row < g.m && col < g.n && ((row + g.tri_shift) & g.tri_mask) <= col)
                __builtin_nontemporal_store(result, (global_f64_t *)(g.c + (uint64_t)row * g.c_stride + (uint64_t)col * 8));
        }
    }
}

constexpr int kMatrixRows = 128, kMatrixCols = 64; // rows and columns of C per workgroup of the f32 matrix kernel
constexpr int kMatrixDepth = 32;                     // k per step: two groups of four MFMA depths for each of the four sums
// A row of staged A is 128 bytes of f32, eight 16-byte units; unit u of row r sits at position u ^ (r % 8), so that the
// eight lanes of an LDS cycle, which read the same unit of eight consecutive rows, or write the eight units of one row,
// spread over all banks without padding. Two stages of A and of B (f64, [k][column]) fill the 64 KiB exactly.

/**
 *  f32 inputs on the f64 matrix cores. `v_mfma_f64_16x16x4_f64` is, per output, a chain of four fused multiply-adds in
 *  ascending order of its depth index, each rounded to f64 (checked on the part against a host chain, bit for bit,
 *  51,200 outputs with full-range f64 operands and accumulators). The reference keeps four f64 sums per output, sum r
 *  taking the products of k = r, r + 4, r + 8, ... in that order (dot/serial.h:262-296), and a product of two f32 values
 *  is exact in f64, so a fused multiply-add is the reference's multiply-then-add. Feeding one instruction the depths
 *  k0 + r, k0 + r + 4, k0 + r + 8, k0 + r + 12 therefore advances sum r of a 16 x 16 block of outputs exactly as the
 *  reference does, and four instructions (r = 0..3) consume 16 depths. Zero padding past the last depth adds products
 *  of +0, which leave a sum that started at +0 unchanged (such a sum is never -0).
 *
 *  512 threads, 8 wavefronts as 4 x 2, each 32 x 32 outputs = 2 x 2 blocks x 4 sums = 128 accumulator registers, two
 *  wavefronts per SIMD. A is staged as f32, [row][k] so that one 16-byte read gives a lane the four operands
 *  (r = 0..3) of its row and depth group, and widened where it is multiplied; B comes from the k-major f64 image into
 *  [k][column]. A step is 32 depths = 32 MFMAs per wavefront; loads from memory are asked for a whole step before the
 *  stash that takes them, and the stash, the barrier and the reads of LDS sit between groups of MFMAs.
 */
template <bool NORMS>
__global__ __launch_bounds__(512) void dots_f32_matrix_kernel(WideArgs g) {
    typedef double __attribute__((ext_vector_type(4))) f64x4_t;
    typedef double __attribute__((ext_vector_type(2))) f64x2_t;
    typedef float __attribute__((ext_vector_type(4))) f32x4_t;
    typedef __attribute__((address_space(1))) double global_f64_t;
    typedef __attribute__((address_space(1))) uint64_t global_u64_t;
    __shared__ __attribute__((aligned(16))) float a_lds[2][kMatrixRows][kMatrixDepth];
    __shared__ __attribute__((aligned(16))) double b_lds[2][kMatrixDepth][kMatrixCols];
    // distances: four partial sums of squares per row of A and their total, in the B stages once the loop is over
    double(*row_parts)[4][2] = (double(*)[4][2]) & b_lds[0][0][0];
    double *row_norms = &b_lds[1][0][0];
    static_assert(sizeof(double) * kMatrixRows * 8 <= sizeof(b_lds) / 2, "the partial sums fit one stage of B");
    uint32_t const tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t const row0 = blockIdx.y * kMatrixRows, col0 = blockIdx.x * kMatrixCols;
    // symmetric form: a tile wholly left of the diagonal has nothing to store
    if (((row0 + g.tri_shift) & g.tri_mask) > col0 + (kMatrixCols - 1)) return;
    PackedHeader const *header = (PackedHeader const *)((uint8_t const *)g.b - sizeof(PackedHeader));
    if (!(header->magic == kMagic && header->version == kVersion && header->dtype == (uint32_t)g.dtype && header->n == g.n &&
          header->k == g.k)) { // (an image of another type or shape: poison, as the f64 kernel does)
        for (uint32_t at = tid; at < kMatrixRows * kMatrixCols; at += 512) {
            uint32_t const row = row0 + at / kMatrixCols, col = col0 + at % kMatrixCols;
            if (row < g.m && col < g.n && ((row + g.tri_shift) & g.tri_mask) <= col)
                *(global_u64_t *)(g.c + (uint64_t)row * g.c_stride + (uint64_t)col * 8) = ~0ull;
        }
        return;
    }

    uint32_t const wave_row = (wave >> 1) * 32, wave_col = (wave & 1) * 32;
    uint32_t const in_block = lane & 15, depth_group = lane >> 4;
    f64x4_t acc[2][2][4]; // [row block][column block][sum r]; element v: row 4 v + lane / 16, column lane % 16
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = f64x4_t {0, 0, 0, 0};

    // staging: A: thread t brings 8 consecutive k of row t / 4; B: 2 consecutive columns of depths t / 32 and 16 + t / 32
    uint32_t const a_row = tid >> 2, a_k = (tid & 3) * 8;
    uint32_t const b_k = tid >> 5, b_col = (tid & 31) * 2;
    uint32_t const a_from = row0 + a_row < g.m ? row0 + a_row : g.m - 1; // (rows past the end repeat the last; never stored)
    uint8_t const *a_source = g.a + (uint64_t)a_from * g.a_stride;
    bool const aligned = ((((uint64_t)g.a) | g.a_stride) & 15) == 0;
    f32x4_t a_next[2];
    f64x2_t b_next[2];
    CompensatedSum squares; // distances: of this thread's share of its row of A
    // `whole`: the step lies inside the rows of A and they can be read 16 bytes at a time. It is a compile-time choice, one
    // loop for each: where both ways to load sit in one loop, waits for the loads come between them, in front of the MFMAs
    // that are there to cover them.
    auto fetch = [&](uint32_t k0, auto whole) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t const at = k0 + a_k + 4 * h;
            if (whole) a_next[h] = *(f32x4_t const *)(a_source + (uint64_t)at * 4);
            else {
#pragma unroll
                for (int e = 0; e < 4; ++e) a_next[h][e] = at + e < g.k ? ((float const *)a_source)[at + e] : 0.f;
            }
            b_next[h] = *(f64x2_t const *)(g.b + (uint64_t)(k0 + b_k + 16 * h) * g.n_padded + col0 + b_col); // (inside the padded image)
        }
    };
    auto stash = [&](int buffer) { // (the first use of what fetch() asked for: the wait for it sits here, behind a group of MFMAs)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            *(f32x4_t *)&a_lds[buffer][a_row][4 * ((a_k / 4 + h) ^ (a_row & 7))] = a_next[h];
            *(f64x2_t *)&b_lds[buffer][b_k + 16 * h][b_col] = b_next[h];
            if (NORMS) { // four exact squares summed with three roundings of their own small sum, then one compensated addition
                double const x0 = a_next[h][0], x1 = a_next[h][1], x2 = a_next[h][2], x3 = a_next[h][3];
                squares.add(__builtin_fma(x0, x0, __builtin_fma(x1, x1, __builtin_fma(x2, x2, x3 * x3))));
            }
        }
    };
    struct Operands {
        f32x4_t a[2];   // [row block]: as staged, widened where it is multiplied: nothing between two groups of MFMAs waits on LDS
        double b[2][4]; // [column block][sum r]
    };
    auto read_operands = [&](int buffer, int group, Operands &operands) { // 16 depths: 16 group + r + 4 (lane / 16)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t const row = wave_row + 16 * i + in_block;
            operands.a[i] = *(f32x4_t const *)&a_lds[buffer][row][4 * ((4 * group + depth_group) ^ (row & 7))];
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                operands.b[j][r] = b_lds[buffer][16 * group + r + 4 * depth_group][wave_col + 16 * j + in_block];
    };
    auto multiply = [&](Operands const &operands, int from, int to) { // sums `from` up to `to`, 4 MFMAs each
#pragma unroll
        for (int r = from; r < to; ++r)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j][r] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)operands.a[i][r], operands.b[j][r], acc[i][j][r], 0, 0, 0);
    };

    uint32_t const depth = (g.k + kMatrixDepth - 1) & ~(uint32_t)(kMatrixDepth - 1); // (the image is padded to 32)
    // One barrier per step, in the middle of its MFMAs: the first group's operands were read behind the previous barrier,
    // the second group's before this one, so every read of a stage precedes the barrier that lets the next writes into it,
    // and no wave waits on LDS with the matrix pipe idle.
    static_assert(kMatrixDepth == 32, "two groups of 16 depths per step");
    Operands first, second;
    std::false_type const piecewise;
    std::true_type const whole;
    fetch(0, piecewise);
    stash(0);
    if (kMatrixDepth < depth) fetch(kMatrixDepth, piecewise);
    __syncthreads();
    read_operands(0, 0, first);
    int buffer = 0;
    // One step: 32 MFMAs, and between them, where none of it holds the matrix pipe up: the stash of the step after this one
    // (its stage was last read before the previous barrier), the request for the step after that, the barrier, and the
    // reads of LDS, each asked for at least 8 MFMAs before its use. The scheduler is held to this order.
    auto step = [&](uint32_t k0, auto whole) { // (a whole step: neither the last nor the one before it)
        bool const more = whole || k0 + kMatrixDepth < depth;
        read_operands(buffer, 1, second);
        __builtin_amdgcn_sched_barrier(0);
        multiply(first, 0, 4);
        __builtin_amdgcn_sched_barrier(0);
        if (more) stash(buffer ^ 1);
        if (whole || k0 + 2 * kMatrixDepth < depth) fetch(k0 + 2 * kMatrixDepth, whole); // a whole step ahead of its stash()
        __builtin_amdgcn_sched_barrier(0);
        multiply(second, 0, 2);
        __builtin_amdgcn_sched_barrier(0);
        // a barrier that orders LDS only: __syncthreads() would also wait for the loads just asked for
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        if (more) read_operands(buffer ^ 1, 0, first);
        __builtin_amdgcn_sched_barrier(0);
        multiply(second, 2, 4);
        __builtin_amdgcn_sched_barrier(0);
        buffer ^= 1;
    };
    uint32_t k0 = 0;
    if (aligned)
        for (; k0 + 3 * kMatrixDepth <= g.k; k0 += kMatrixDepth) step(k0, whole);
    for (; k0 < depth; k0 += kMatrixDepth) step(k0, piecewise);

    double column_norm[2];
    if (NORMS) {
        row_parts[a_row][tid & 3][0] = squares.sum, row_parts[a_row][tid & 3][1] = squares.lost; // (no read of a stage follows the loop's last barrier)
        __syncthreads();
        if (tid < kMatrixRows) {
            CompensatedSum total;
#pragma unroll
            for (int part = 0; part < 4; ++part) {
                CompensatedSum one;
                one.sum = row_parts[tid][part][0], one.lost = row_parts[tid][part][1];
                total.add(one);
            }
            row_norms[tid] = total.value();
        }
        __syncthreads();
        double const *norms = g.b + (uint64_t)g.k_padded * g.n_padded; // behind the matrix, one per padded column
#pragma unroll
        for (int j = 0; j < 2; ++j) column_norm[j] = norms[col0 + wave_col + 16 * j + in_block];
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            uint32_t const in_tile = wave_row + 16 * i + 4 * v + depth_group, row = row0 + in_tile;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                uint32_t const col = col0 + wave_col + 16 * j + in_block;
                double result = ((acc[i][j][0][v] + acc[i][j][1][v]) + acc[i][j][2][v]) + acc[i][j][3][v];
                if (NORMS) {
                    result = wide_distance(g.metric, result, row_norms[in_tile], column_norm[j]);
                    if (g.tri_mask && row + g.tri_shift == col) result = 0; // a vector and itself: exactly 0
                }
                if (row < g.m && col < g.n && ((row + g.tri_shift) & g.tri_mask) <= col)
                    __builtin_nontemporal_store(result, (global_f64_t *)(g.c + (uint64_t)row * g.c_stride + (uint64_t)col * 8));
            }
        }
}

__global__ __launch_bounds__(256) void fill_wide_kernel(uint8_t *c, uint32_t m, uint32_t n, uint64_t c_stride, uint64_t bits,
                                                        uint32_t tri_shift, uint32_t tri_mask) {
    uint64_t const i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    uint64_t const row = i / n, col = i % n;
    if (row < m && (((uint32_t)row + tri_shift) & tri_mask) <= (uint32_t)col) *(uint64_t *)(c + row * c_stride + col * 8) = bits;
}

} // namespace

namespace nk_gfx950 {

bool wide_geometry(int dtype, size_t n, size_t k, WideGeometry &g) {
    if (dtype != kF32 && dtype != kF64) return false;
    if (n > 0x7FFFFFFFull || k > 0x3FFFFFFFull) return false;
    g.elem_bytes = dtype == kF64 ? 8 : 4;
    g.n = (uint32_t)n, g.k = (uint32_t)k;
    g.n_padded = (uint32_t)((n + kWideTile - 1) / kWideTile * kWideTile);
    g.k_padded = (uint32_t)((k + 31) / 32 * 32); // the pack kernel writes whole 32 x 32 blocks
    g.total_bytes = sizeof(PackedHeader) + (uint64_t)g.n_padded * g.k_padded * 8 + (uint64_t)g.n_padded * 8; // matrix, then sums of squares
    return true;
}

hipError_t wide_pack(int dtype, void const *b, size_t n, size_t k, size_t b_stride, void *b_packed, hipStream_t stream) {
    WideGeometry g;
    if (!wide_geometry(dtype, n, k, g)) return hipErrorInvalidValue;
    if (((uintptr_t)b | b_stride) & (g.elem_bytes - 1)) return hipErrorInvalidValue; // elements must be aligned
    PackedHeader h;
    memset(&h, 0, sizeof(h));
    h.magic = kMagic, h.version = kVersion, h.dtype = (uint32_t)dtype, h.elem_bytes = 8;
    h.n = g.n, h.k = g.k, h.n_tiles = g.n_padded / kWideTile, h.k_chunks = g.k_padded;
    h.nonce = next_image_nonce(), h.sums_offset = h.norms_offset = h.total_bytes = g.total_bytes;
    double *out = (double *)((uint8_t *)b_packed + sizeof(PackedHeader));
    if (!g.n_padded || !g.k_padded) {
        hipLaunchKernelGGL(write_header_kernel, dim3(1), dim3(64), 0, stream, (PackedHeader *)b_packed, h);
        return hipGetLastError();
    }
    // (the second grid dimension holds 65535 workgroups: deeper rows take several launches)
    for (uint32_t k_first = 0; k_first < g.k_padded; k_first += 65535u * 32) {
        uint32_t const depth_blocks = (g.k_padded - k_first) / 32 < 65535u ? (g.k_padded - k_first) / 32 : 65535u;
        dim3 const grid(g.n_padded / 32, depth_blocks);
        if (dtype == kF64) hipLaunchKernelGGL(pack_wide_kernel<true>, grid, dim3(256), 0, stream, (uint8_t const *)b, (uint64_t)b_stride, g.n, g.k, g.n_padded, out, h, k_first);
        else hipLaunchKernelGGL(pack_wide_kernel<false>, grid, dim3(256), 0, stream, (uint8_t const *)b, (uint64_t)b_stride, g.n, g.k, g.n_padded, out, h, k_first);
        hipError_t const status = hipGetLastError();
        if (status != hipSuccess) return status;
    }
    double *norms = out + (uint64_t)g.n_padded * g.k_padded;
    dim3 const norms_grid((g.n_padded + 3) / 4);
    if (dtype == kF64) hipLaunchKernelGGL(wide_norms_kernel<true>, norms_grid, dim3(256), 0, stream, (uint8_t const *)b, (uint64_t)b_stride, g.n, g.k, g.n_padded, norms);
    else hipLaunchKernelGGL(wide_norms_kernel<false>, norms_grid, dim3(256), 0, stream, (uint8_t const *)b, (uint64_t)b_stride, g.n, g.k, g.n_padded, norms);
    return hipGetLastError();
}

hipError_t wide_product(int dtype, void const *a, void const *b_packed, void *c, size_t m, size_t n, size_t k,
                        size_t a_stride, size_t c_stride, hipStream_t stream, bool triangle, uint32_t shift, int metric) {
    WideGeometry geo;
    if (metric < 0 || metric > 2) return hipErrorInvalidValue;
    if (!wide_geometry(dtype, n, k, geo)) return hipErrorInvalidValue;
    if (m > 0x7FFFFFFFull) return hipErrorInvalidValue;
    if (((uintptr_t)c | c_stride) & 7) return hipErrorInvalidValue;
    if ((uintptr_t)b_packed & 15) return hipErrorInvalidValue; // (the kernels read the image 16 bytes at a time)
    uint32_t const tri_mask = triangle ? 0xFFFFFFFFu : 0u;
    if (k == 0) {
        uint64_t const blocks = ((uint64_t)m * n + 255) / 256;
        if (blocks > 0x7FFFFFFFull) return hipErrorInvalidValue;
        hipLaunchKernelGGL(fill_wide_kernel, dim3((uint32_t)blocks), dim3(256), 0, stream, (uint8_t *)c, (uint32_t)m, (uint32_t)n,
                           (uint64_t)c_stride, 0ull, shift, tri_mask);
        return hipGetLastError();
    }
    if (((uintptr_t)a | a_stride) & (geo.elem_bytes - 1)) return hipErrorInvalidValue;
    WideArgs g;
    memset(&g, 0, sizeof(g));
    g.dtype = dtype;
    g.a = (uint8_t const *)a, g.b = (double const *)((uint8_t const *)b_packed + sizeof(PackedHeader)), g.c = (uint8_t *)c;
    g.a_stride = a_stride, g.c_stride = c_stride;
    g.m = (uint32_t)m, g.n = geo.n, g.k = geo.k, g.n_padded = geo.n_padded, g.k_padded = geo.k_padded;
    g.tri_mask = tri_mask, g.metric = metric;
    // The second grid dimension holds 65535 workgroups: taller products go band by band (a whole number of tiles of
    // both kernels each; a band's rows start `first` below the diagonal's origin).
    uint64_t const band = 32767ull * kMatrixRows;
    static_assert((32767ull * kMatrixRows) % kWideTile == 0 && 32767ull * kMatrixRows / kWideTile <= 65535, "a band is whole tiles of both kernels");
    for (uint64_t first = 0; first < m; first += band) {
        uint64_t const rows = m - first < band ? m - first : band;
        g.a = (uint8_t const *)a + first * a_stride, g.c = (uint8_t *)c + first * c_stride;
        g.m = (uint32_t)rows, g.tri_shift = shift + (uint32_t)first;
        dim3 const grid(geo.n_padded / kWideTile, (uint32_t)((rows + kWideTile - 1) / kWideTile));
        dim3 const matrix_grid(geo.n_padded / kMatrixCols, (uint32_t)((rows + kMatrixRows - 1) / kMatrixRows));
        if (dtype == kF64 && metric) hipLaunchKernelGGL(dots_f64_compensated_kernel<true>, grid, dim3(256), 0, stream, g);
        else if (dtype == kF64) hipLaunchKernelGGL(dots_f64_compensated_kernel<false>, grid, dim3(256), 0, stream, g);
        else if (metric) hipLaunchKernelGGL(dots_f32_matrix_kernel<true>, matrix_grid, dim3(512), 0, stream, g);
        else hipLaunchKernelGGL(dots_f32_matrix_kernel<false>, matrix_grid, dim3(512), 0, stream, g);
        hipError_t const status = hipGetLastError();
        if (status != hipSuccess) return status;
    }
    return hipSuccess;
}

} // namespace nk_gfx950
