/**
 *  @brief What the matrix cores of this GPU do, measured: the rate an MFMA-only loop sustains, and how the fp8, f16
 *         and bf16 forms round. The product kernels are designed around these facts; this program states them.
 *  @file tests/probes/mfma_probes.hip
 *
 *  Measurement code, not part of the library: nothing under numkong_amd/ builds, links or loads it.
 *
 *      mfma_probes ceiling [--json]     every MFMA form the kernels could use, fed from registers only, in the 8 x 2
 *                                       block arrangement of the 256 x 256 product tile, on random and on zero data:
 *                                       T(FL)OP/s over 20 back-to-back launches after 20 warm-up ones, shader clock
 *                                       (cycles by s_memtime over the 100 MHz s_memrealtime) and cycles per MFMA.
 *                                       That rate is what a kernel with free loads would reach on this part.
 *      mfma_probes numerics [--check]   how far apart two addends of one instruction may be before the smaller one is
 *                                       dropped, for the fp8 / bf8 forms (legacy and f8f6f4) and for f16 / bf16; the
 *                                       error of a depth-8192 e4m3 dot product on the fp8 MFMA next to f32
 *                                       accumulation of exact products (what the reference's kernels do,
 *                                       dot/serial.h:522-600) and to the same data widened to f16 on the f16 MFMA.
 *                                       --check exits non-zero unless the facts the kernels rely on hold.
 *      mfma_probes budget               what the rest of a product kernel costs the i8 32 x 32 x 32 loop on a part that
 *                                       runs at its power limit: idle cycles (s_sleep behind every 16 MFMAs), the
 *                                       product kernel's LDS fragment reads (8 ds_read_b128 per 16 MFMAs), its global
 *                                       loads (4 dwordx4 per 16 MFMAs, L2 hits, three iterations ahead), and all of
 *                                       them; rate, shader clock and the share of cycles the MFMA pipe is busy.
 *      mfma_probes stream               what the memory takes for the traffic of the retrieval shape (1024 x 1,048,576
 *                                       x 768, i8 -> i32: 0.75 GiB read, 4 GiB written) with no arithmetic at all:
 *                                       only written, only read, and both at once by separate workgroups.
 *
 *  Built by the Makefile next to it (tests/probes/mfma_probes); bench.py runs the first mode and reports it under
 *  `others.mfma_ceiling`, tests/test_mfma_numerics_gpu.py runs the second, and the last two are the commands behind the
 *  summaries profiles/mfma_budget.txt and profiles/memory_stream.txt.
 */
#include <hip/hip_runtime.h>

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <type_traits>
#include <vector>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

#define CHECK(call)                                                                               \
    do {                                                                                          \
        hipError_t status_ = (call);                                                              \
        if (status_ != hipSuccess) {                                                              \
            fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(status_));                       \
            exit(2);                                                                              \
        }                                                                                         \
    } while (0)

#pragma region Ceiling

enum Form { kI8Large, kI8Small, kBF16Large, kBF16Small, kF16Large, kFP8Legacy, kFP8Scaled, kF16OfE4M3, kBF16OfE4M3, kForms };
static char const *const kFormNames[kForms] = {"i8 32x32x32", "i8 16x16x64", "bf16 32x32x16", "bf16 16x16x32",
                                               "f16 32x32x16", "fp8 32x32x16 (legacy)", "fp8 32x32x64 (f8f6f4)",
                                               "f16 32x32x16 on e4m3 values", "bf16 32x32x16 on e4m3 values"};
static double const kFormOps[kForms] = {2.0 * 32 * 32 * 32, 2.0 * 16 * 16 * 64, 2.0 * 32 * 32 * 16, 2.0 * 16 * 16 * 32,
                                        2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 64, 2.0 * 32 * 32 * 16, 2.0 * 32 * 32 * 16};
static double const kFormPeak[kForms] = {5000, 5000, 2500, 2500, 2500, 5000, 5000, 2500, 2500}; // published dense peaks, T(FL)OP/s

/**
 *  One workgroup of four wavefronts per compute unit, every wavefront 256 accumulator registers: ROWS x COLS blocks,
 *  block (i, j) fed operand registers a[i] and b[j], which never change: the product kernel's inner loop with the loads,
 *  the LDS traffic and the barriers taken out. `clocks`: shader cycles and 100 MHz ticks the loop took, per workgroup.
 */
template <int FORM>
__global__ __launch_bounds__(256) void mfma_only_kernel(v8i const *operands, int iterations, float *sink, unsigned long long *clocks) {
    constexpr bool kLarge = FORM != kI8Small && FORM != kBF16Small;
    constexpr int ROWS = 8, COLS = kLarge ? 2 : 8;
    v8i a[ROWS], b[COLS];
    for (int i = 0; i < ROWS; ++i) a[i] = operands[(i * 64 + (threadIdx.x & 63)) % 1024];
    for (int j = 0; j < COLS; ++j) b[j] = operands[((ROWS + j) * 64 + (threadIdx.x & 63)) % 1024];
    typedef typename std::conditional<FORM == kI8Large, v16i, typename std::conditional<FORM == kI8Small, v4i, typename std::conditional<kLarge, v16f, v4f>::type>::type>::type acc_t;
    acc_t acc[ROWS][COLS];
    for (int i = 0; i < ROWS; ++i)
        for (int j = 0; j < COLS; ++j)
            for (int v = 0; v < (int)(sizeof(acc_t) / 4); ++v) acc[i][j][v] = 0;
    unsigned long long const cycles0 = clock64(), ticks0 = wall_clock64();
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int j = 0; j < COLS; ++j)
#pragma unroll
            for (int i = 0; i < ROWS; ++i) {
                v4i const a4 = {a[i][0], a[i][1], a[i][2], a[i][3]}, b4 = {b[j][0], b[j][1], b[j][2], b[j][3]};
                long const a2 = ((long)a[i][1] << 32) | (unsigned)a[i][0], b2 = ((long)b[j][1] << 32) | (unsigned)b[j][0];
                if constexpr (FORM == kI8Large) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a4, b4, acc[i][j], 0, 0, 0);
                if constexpr (FORM == kI8Small) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a4, b4, acc[i][j], 0, 0, 0);
                if constexpr (FORM == kBF16Large || FORM == kBF16OfE4M3) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a4), __builtin_bit_cast(v8bf, b4), acc[i][j], 0, 0, 0);
                if constexpr (FORM == kBF16Small) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a4), __builtin_bit_cast(v8bf, b4), acc[i][j], 0, 0, 0);
                if constexpr (FORM == kF16Large || FORM == kF16OfE4M3) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a4), __builtin_bit_cast(v8h, b4), acc[i][j], 0, 0, 0);
                if constexpr (FORM == kFP8Legacy) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(a2, b2, acc[i][j], 0, 0, 0);
                if constexpr (FORM == kFP8Scaled) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 0, 0, 0);
            }
    }
    unsigned long long const cycles1 = clock64(), ticks1 = wall_clock64();
    float total = 0;
    for (int i = 0; i < ROWS; ++i)
        for (int j = 0; j < COLS; ++j) total += (float)acc[i][j][0];
    sink[blockIdx.x * 256 + threadIdx.x] = total;
    if (threadIdx.x == 0) clocks[2 * blockIdx.x] = cycles1 - cycles0, clocks[2 * blockIdx.x + 1] = ticks1 - ticks0;
}

static uint64_t g_random_state = 0x9E3779B97F4A7C15ull;
static uint64_t next_random() { // (xorshift64*)
    g_random_state ^= g_random_state >> 12, g_random_state ^= g_random_state << 25, g_random_state ^= g_random_state >> 27;
    return g_random_state * 0x2545F4914F6CDD1Dull;
}
static double next_normal() {
    double const u = ((next_random() >> 11) + 1) * (1.0 / 9007199254740993.0), v = (next_random() >> 11) * (1.0 / 9007199254740992.0);
    return sqrt(-2.0 * log(u)) * cos(6.283185307179586 * v);
}
static uint16_t bf16_of(float f) {
    uint32_t bits;
    memcpy(&bits, &f, 4);
    return (uint16_t)((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16);
}
static uint16_t f16_of(float f) {
    _Float16 const h = (_Float16)f;
    uint16_t bits;
    memcpy(&bits, &h, 2);
    return bits;
}
static float e4m3_value(uint8_t c) {
    int const s = c >> 7, e = (c >> 3) & 15, m = c & 7;
    float const v = e == 15 && m == 7 ? NAN : (e == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10));
    return s ? -v : v;
}
static float e5m2_value(uint8_t c) {
    int const s = c >> 7, e = (c >> 2) & 31, m = c & 3;
    float const v = e == 31 ? (m ? NAN : INFINITY) : (e == 0 ? ldexpf((float)m, -16) : ldexpf((float)(4 + m), e - 17));
    return s ? -v : v;
}
/** Round to nearest e4m3 (ties to even), saturating at 448: the reference's rule for finite inputs (cast/serial.h:866-947). */
static uint8_t e4m3_of(float f) {
    uint8_t best = 0;
    float best_distance = INFINITY;
    for (int c = 0; c < 127; ++c) {
        float const distance = fabsf(fabsf(f) - e4m3_value((uint8_t)c));
        if (distance < best_distance || (distance == best_distance && !(c & 1))) best = (uint8_t)c, best_distance = distance;
    }
    return (uint8_t)(best | (f < 0 ? 0x80 : 0));
}

/** 16 KiB of operand data in the element type of `form`: full-range integers, N(0, 1) floats (for the last two forms
 *  rounded to e4m3 first: what the fp8 product kernels feed the f16 instruction, few mantissa bits set), or zeros. */
static std::vector<uint8_t> operand_data(int form, bool zeros) {
    std::vector<uint8_t> data(1024 * 32, 0);
    if (zeros) return data;
    for (size_t at = 0; at < data.size(); at += 2) {
        if (form == kI8Large || form == kI8Small) data[at] = (uint8_t)next_random(), data[at + 1] = (uint8_t)next_random();
        else if (form == kFP8Legacy || form == kFP8Scaled) data[at] = e4m3_of((float)next_normal()), data[at + 1] = e4m3_of((float)next_normal());
        else {
            float const value = form == kF16OfE4M3 || form == kBF16OfE4M3 ? e4m3_value(e4m3_of((float)next_normal())) : (float)next_normal();
            uint16_t const bits = form == kF16Large || form == kF16OfE4M3 ? f16_of(value) : bf16_of(value);
            memcpy(&data[at], &bits, 2);
        }
    }
    return data;
}

struct CeilingResult {
    double ms, tops, mhz, cycles_per_mfma;
};

template <int FORM>
static CeilingResult run_ceiling(bool zeros, int units, v8i *operands, float *sink, unsigned long long *clocks) {
    std::vector<uint8_t> const data = operand_data(FORM, zeros);
    CHECK(hipMemcpy(operands, data.data(), data.size(), hipMemcpyHostToDevice));
    constexpr bool kLarge = FORM != kI8Small && FORM != kBF16Small;
    int const per_iteration = 8 * (kLarge ? 2 : 8);
    int const iterations = kLarge ? 1500 : 1500; // about half a millisecond per launch
    hipEvent_t begin, end;
    CHECK(hipEventCreate(&begin));
    CHECK(hipEventCreate(&end));
    // (from idle the part ramps its clocks for some tens of milliseconds: 100 ms of the same loop first)
    for (auto const start = std::chrono::steady_clock::now(); std::chrono::steady_clock::now() - start < std::chrono::milliseconds(100);) {
        for (int warm = 0; warm < 20; ++warm) hipLaunchKernelGGL(mfma_only_kernel<FORM>, dim3(units), dim3(256), 0, 0, operands, iterations, sink, clocks);
        CHECK(hipDeviceSynchronize());
    }
    CHECK(hipEventRecord(begin, 0));
    constexpr int kLaunches = 20;
    for (int launch = 0; launch < kLaunches; ++launch) hipLaunchKernelGGL(mfma_only_kernel<FORM>, dim3(units), dim3(256), 0, 0, operands, iterations, sink, clocks);
    CHECK(hipEventRecord(end, 0));
    CHECK(hipEventSynchronize(end));
    CHECK(hipGetLastError());
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, begin, end));
    std::vector<unsigned long long> host_clocks(2 * units);
    CHECK(hipMemcpy(host_clocks.data(), clocks, host_clocks.size() * 8, hipMemcpyDeviceToHost));
    double cycles = 0, ticks = 0;
    for (int unit = 0; unit < units; ++unit) cycles += (double)host_clocks[2 * unit], ticks += (double)host_clocks[2 * unit + 1];
    CeilingResult result;
    result.ms = ms / kLaunches;
    result.tops = kFormOps[FORM] * per_iteration * iterations * 4.0 * units / (result.ms * 1e-3) / 1e12;
    result.mhz = cycles / ticks * 100.0;
    result.cycles_per_mfma = cycles / units / ((double)per_iteration * iterations);
    CHECK(hipEventDestroy(begin));
    CHECK(hipEventDestroy(end));
    return result;
}

static int ceiling_mode(bool json) {
    hipDeviceProp_t properties;
    CHECK(hipGetDeviceProperties(&properties, 0));
    int const units = properties.multiProcessorCount;
    v8i *operands;
    float *sink;
    unsigned long long *clocks;
    CHECK(hipMalloc(&operands, 1024 * 32));
    CHECK(hipMalloc(&sink, (size_t)units * 256 * 4));
    CHECK(hipMalloc(&clocks, (size_t)units * 16));
    CeilingResult results[kForms][2];
    for (int zeros = 0; zeros < 2; ++zeros) {
        results[kI8Large][zeros] = run_ceiling<kI8Large>(zeros, units, operands, sink, clocks);
        results[kI8Small][zeros] = run_ceiling<kI8Small>(zeros, units, operands, sink, clocks);
        results[kBF16Large][zeros] = run_ceiling<kBF16Large>(zeros, units, operands, sink, clocks);
        results[kBF16Small][zeros] = run_ceiling<kBF16Small>(zeros, units, operands, sink, clocks);
        results[kF16Large][zeros] = run_ceiling<kF16Large>(zeros, units, operands, sink, clocks);
        results[kFP8Legacy][zeros] = run_ceiling<kFP8Legacy>(zeros, units, operands, sink, clocks);
        results[kFP8Scaled][zeros] = run_ceiling<kFP8Scaled>(zeros, units, operands, sink, clocks);
        results[kF16OfE4M3][zeros] = run_ceiling<kF16OfE4M3>(zeros, units, operands, sink, clocks);
        results[kBF16OfE4M3][zeros] = run_ceiling<kBF16OfE4M3>(zeros, units, operands, sink, clocks);
    }
    if (json) printf("{\"compute_units\": %d, \"device\": \"%s\", \"forms\": {", units, properties.gcnArchName);
    else printf("MFMA-only loop, %d compute units (%s), 4 wavefronts each, 20 launches after 100 ms of the same loop\n%-30s %-7s %9s %10s %8s %8s %12s\n", units,
                properties.gcnArchName, "instruction", "data", "ms", "T(FL)OP/s", "of peak", "MHz", "cycles/MFMA");
    for (int form = 0; form < kForms; ++form)
        for (int zeros = 0; zeros < 2; ++zeros) {
            CeilingResult const &r = results[form][zeros];
            if (json)
                printf("%s\"%s, %s\": {\"tops\": %.1f, \"frac_of_peak\": %.4f, \"mhz\": %.0f, \"cycles_per_mfma\": %.2f}", form + zeros ? ", " : "",
                       kFormNames[form], zeros ? "zeros" : "random", r.tops, r.tops / kFormPeak[form], r.mhz, r.cycles_per_mfma);
            else
                printf("%-30s %-7s %9.4f %10.1f %8.3f %8.0f %12.2f\n", kFormNames[form], zeros ? "zeros" : "random", r.ms, r.tops, r.tops / kFormPeak[form], r.mhz,
                       r.cycles_per_mfma);
        }
    if (json) printf("}}\n");
    return 0;
}

#pragma endregion Ceiling

#pragma region Budget

/**
 *  The MFMA loop of the 256 x 256 i8 tile (8 x 2 blocks per wavefront) with parts of the product kernel's other work:
 *  LOADS global dwordx4 loads per 16 MFMAs, issued three iterations ahead into a ring of registers, the first two
 *  feeding B (all wander over 2 MiB: L2 hits); READS ds_read_b128 per 16 MFMAs, issued one iteration ahead, feeding A;
 *  SLEEP x 64 idle cycles behind every 16 MFMAs.
 */
template <int LOADS, int READS, int SLEEP>
__global__ __launch_bounds__(256) void budget_kernel(v4i const *operands, int iterations, float *sink, unsigned long long *clocks, v4i const *stream, unsigned stream_mask) {
    __shared__ v4i lds[4096];
    for (int i = threadIdx.x; i < 4096; i += 256) lds[i] = operands[i % 1024];
    __syncthreads();
    constexpr int RING = 4, L = LOADS > 0 ? LOADS : 1;
    v4i a[2][8], g[RING][L], b[2];
    unsigned const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = 0; i < 8; ++i) a[0][i] = a[1][i] = operands[(i * 64 + lane) % 1024];
    for (int j = 0; j < 2; ++j) b[j] = operands[((8 + j) * 64 + lane) % 1024];
    for (int r = 0; r < RING; ++r)
        for (int l = 0; l < L; ++l) g[r][l] = b[l & 1];
    v16i acc[8][2];
    for (int i = 0; i < 8; ++i)
        for (int j = 0; j < 2; ++j)
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    unsigned long long const cycles0 = clock64(), ticks0 = wall_clock64();
    unsigned at = (blockIdx.x * 4 + wave) * 64 * LOADS + lane;
    for (int it = 0; it < iterations; it += RING) {
#pragma unroll
        for (int r = 0; r < RING; ++r) {
            v4i operand_b[2] = {b[0], b[1]};
            if constexpr (LOADS >= 2) operand_b[0] = g[r][0], operand_b[1] = g[r][1];
            if constexpr (LOADS > 0) {
#pragma unroll
                for (int l = 0; l < LOADS; ++l) g[r][l] = stream[(at + l * 64) & stream_mask];
                at += 256 * 4 * 64 * LOADS;
            }
            if constexpr (READS > 0) {
#pragma unroll
                for (int i = 0; i < READS; ++i) a[(r + 1) & 1][i] = lds[(((it + r) & 7) * 512 + i * 64 + lane) & 4095];
            }
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[r & 1][i], operand_b[j], acc[i][j], 0, 0, 0);
            if constexpr (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
        }
    }
    unsigned long long const cycles1 = clock64(), ticks1 = wall_clock64();
    float total = 0;
    for (int i = 0; i < 8; ++i)
        for (int j = 0; j < 2; ++j) total += (float)acc[i][j][0];
    sink[blockIdx.x * 256 + threadIdx.x] = total;
    if (threadIdx.x == 0) clocks[2 * blockIdx.x] = cycles1 - cycles0, clocks[2 * blockIdx.x + 1] = ticks1 - ticks0;
}

/**
 *  The same tile with the 16 x 16 x 64 instruction: 16 x 4 blocks per wavefront, one trip a 64-deep step (64 MFMAs, the
 *  work of two trips of the loop above), with twice the loads and reads per trip so that the traffic per operation is
 *  the same: 2 x LOADS global loads two trips ahead, 2 x READS ds_read_b128 one trip ahead.
 */
template <int LOADS, int READS>
__global__ __launch_bounds__(256) void budget_small_kernel(v4i const *operands, int iterations, float *sink, unsigned long long *clocks, v4i const *stream, unsigned stream_mask) {
    __shared__ v4i lds[4096];
    for (int i = threadIdx.x; i < 4096; i += 256) lds[i] = operands[i % 1024];
    __syncthreads();
    constexpr int RING = 2, L = LOADS > 0 ? 2 * LOADS : 1;
    v4i a[2][16], g[RING][L], b[4];
    unsigned const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = 0; i < 16; ++i) a[0][i] = a[1][i] = operands[(i * 64 + lane) % 1024];
    for (int j = 0; j < 4; ++j) b[j] = operands[((8 + j) * 64 + lane) % 1024];
    for (int r = 0; r < RING; ++r)
        for (int l = 0; l < L; ++l) g[r][l] = b[l & 3];
    v4i acc[16][4];
    for (int i = 0; i < 16; ++i)
        for (int j = 0; j < 4; ++j) acc[i][j] = v4i {0, 0, 0, 0};
    unsigned long long const cycles0 = clock64(), ticks0 = wall_clock64();
    unsigned at = (blockIdx.x * 4 + wave) * 64 * L + lane;
    for (int it = 0; it < iterations; it += 2 * RING) { // (`iterations` counts 32-deep steps, as for the loop above)
#pragma unroll
        for (int r = 0; r < RING; ++r) {
            v4i operand_b[4] = {b[0], b[1], b[2], b[3]};
            if constexpr (LOADS >= 2) operand_b[0] = g[r][0], operand_b[1] = g[r][1], operand_b[2] = g[r][2], operand_b[3] = g[r][3];
            if constexpr (LOADS > 0) {
#pragma unroll
                for (int l = 0; l < L; ++l) g[r][l] = stream[(at + l * 64) & stream_mask];
                at += 256 * 4 * 64 * L;
            }
            if constexpr (READS > 0) {
#pragma unroll
                for (int i = 0; i < 2 * READS; ++i) a[(r + 1) & 1][i] = lds[(((it / 2 + r) & 3) * 1024 + i * 64 + lane) & 4095];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[r & 1][i], operand_b[j], acc[i][j], 0, 0, 0);
        }
    }
    unsigned long long const cycles1 = clock64(), ticks1 = wall_clock64();
    float total = 0;
    for (int i = 0; i < 16; ++i)
        for (int j = 0; j < 4; ++j) total += (float)acc[i][j][0];
    sink[blockIdx.x * 256 + threadIdx.x] = total;
    if (threadIdx.x == 0) clocks[2 * blockIdx.x] = cycles1 - cycles0, clocks[2 * blockIdx.x + 1] = ticks1 - ticks0;
}

template <class Kernel>
static void run_budget(char const *name, Kernel kernel, int units, v4i *operands, float *sink, unsigned long long *clocks, v4i *stream, unsigned mask) {
    int const iterations = 1500;
    hipEvent_t begin, end;
    CHECK(hipEventCreate(&begin));
    CHECK(hipEventCreate(&end));
    // (from idle the part ramps its clocks for some tens of milliseconds: 100 ms of the same loop first)
    for (auto const start = std::chrono::steady_clock::now(); std::chrono::steady_clock::now() - start < std::chrono::milliseconds(100);) {
        for (int warm = 0; warm < 20; ++warm) hipLaunchKernelGGL(kernel, dim3(units), dim3(256), 0, 0, operands, iterations, sink, clocks, stream, mask);
        CHECK(hipDeviceSynchronize());
    }
    CHECK(hipEventRecord(begin, 0));
    for (int launch = 0; launch < 20; ++launch) hipLaunchKernelGGL(kernel, dim3(units), dim3(256), 0, 0, operands, iterations, sink, clocks, stream, mask);
    CHECK(hipEventRecord(end, 0));
    CHECK(hipEventSynchronize(end));
    CHECK(hipGetLastError());
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, begin, end));
    ms /= 20;
    std::vector<unsigned long long> host_clocks(2 * units);
    CHECK(hipMemcpy(host_clocks.data(), clocks, host_clocks.size() * 8, hipMemcpyDeviceToHost));
    double cycles = 0, ticks = 0;
    for (int unit = 0; unit < units; ++unit) cycles += (double)host_clocks[2 * unit], ticks += (double)host_clocks[2 * unit + 1];
    double const tops = 65536.0 * 16 * iterations * 4 * units / (ms * 1e-3) / 1e12;
    printf("%-58s %8.4f %9.1f %8.3f %8.0f %9.0f %%\n", name, ms, tops, tops / 5000, cycles / ticks * 100.0, 3200.0 * 16 * iterations * units / cycles);
    CHECK(hipEventDestroy(begin));
    CHECK(hipEventDestroy(end));
}

static int budget_mode() {
    hipDeviceProp_t properties;
    CHECK(hipGetDeviceProperties(&properties, 0));
    int const units = properties.multiProcessorCount;
    v4i *operands, *stream;
    float *sink;
    unsigned long long *clocks;
    size_t const stream_bytes = 2u << 20;
    CHECK(hipMalloc(&operands, 16384));
    CHECK(hipMalloc(&stream, stream_bytes));
    CHECK(hipMalloc(&sink, (size_t)units * 256 * 4));
    CHECK(hipMalloc(&clocks, (size_t)units * 16));
    std::vector<uint8_t> data(stream_bytes);
    for (size_t at = 0; at < data.size(); ++at) data[at] = (uint8_t)next_random();
    CHECK(hipMemcpy(operands, data.data(), 16384, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(stream, data.data(), stream_bytes, hipMemcpyHostToDevice));
    unsigned const mask = (unsigned)(stream_bytes / 16 - 1);
    printf("i8 32x32x32 MFMA loop on random data with parts of a product kernel's other work, %d compute units (%s), 4 wavefronts each\n", units, properties.gcnArchName);
    printf("%-58s %8s %9s %8s %8s %10s\n", "per 16 MFMAs of a wavefront", "ms", "TOP/s", "of peak", "MHz", "MFMA busy");
    run_budget("nothing else", budget_kernel<0, 0, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("64 idle cycles", budget_kernel<0, 0, 1>, units, operands, sink, clocks, stream, mask);
    run_budget("128 idle cycles", budget_kernel<0, 0, 2>, units, operands, sink, clocks, stream, mask);
    run_budget("256 idle cycles", budget_kernel<0, 0, 4>, units, operands, sink, clocks, stream, mask);
    run_budget("512 idle cycles", budget_kernel<0, 0, 8>, units, operands, sink, clocks, stream, mask);
    run_budget("4 ds_read_b128", budget_kernel<0, 4, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("8 ds_read_b128 (the product kernel's)", budget_kernel<0, 8, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("2 global dwordx4 loads", budget_kernel<2, 0, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("4 global dwordx4 loads (the product kernel's)", budget_kernel<4, 0, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("8 ds_read_b128 and 4 global loads", budget_kernel<4, 8, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("8 ds_read_b128, 4 global loads, 128 idle cycles", budget_kernel<4, 8, 2>, units, operands, sink, clocks, stream, mask);
    run_budget("nothing else (again)", budget_kernel<0, 0, 0>, units, operands, sink, clocks, stream, mask);
    printf("the same tile with the 16x16x64 instruction (64 MFMAs per 64-deep step; figures per 16 MFMAs of the 32x32x32 loop; MFMA busy at 16 cycles an MFMA)\n");
    run_budget("16x16x64: nothing else", budget_small_kernel<0, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("16x16x64: 8 ds_read_b128", budget_small_kernel<0, 8>, units, operands, sink, clocks, stream, mask);
    run_budget("16x16x64: 4 global dwordx4 loads", budget_small_kernel<4, 0>, units, operands, sink, clocks, stream, mask);
    run_budget("16x16x64: 8 ds_read_b128 and 4 global loads", budget_small_kernel<4, 8>, units, operands, sink, clocks, stream, mask);
    return 0;
}

#pragma endregion Budget

#pragma region Stream

/** `readers_of_8` of every 8 workgroups read `source` once between them, the others write `target` once between them. */
__global__ __launch_bounds__(256) void stream_kernel(v4i const *source, size_t source_vectors, v4i *target, size_t target_vectors, int readers_of_8, int *sink, int past_caches) {
    bool const reader = (int)(blockIdx.x % 8) < readers_of_8;
    uint32_t const share = reader ? readers_of_8 : 8 - readers_of_8;
    uint32_t const index = blockIdx.x / 8 * share + (reader ? blockIdx.x % 8 : blockIdx.x % 8 - readers_of_8);
    size_t const count = (size_t)(gridDim.x / 8) * share;
    if (reader) {
        v4i mix = {0, 0, 0, 0};
        for (size_t at = (size_t)index * 256 + threadIdx.x; at < source_vectors; at += count * 256 * 4) {
            v4i loaded[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) loaded[u] = at + u * count * 256 < source_vectors ? __builtin_nontemporal_load(source + at + u * count * 256) : mix;
#pragma unroll
            for (int u = 0; u < 4; ++u) mix ^= loaded[u];
        }
        if (mix[0] == 0x12345678) sink[threadIdx.x] = mix[1];
    }
    else {
        v4i const value = {(int)blockIdx.x, 1, 2, 3};
        for (size_t at = (size_t)index * 256 + threadIdx.x; at < target_vectors; at += count * 256) {
            if (past_caches) __builtin_nontemporal_store(value, target + at);
            else target[at] = value;
        }
    }
}

static int stream_mode() {
    size_t const read_bytes = (size_t)768 << 20, written_bytes = (size_t)4 << 30; // B and C of 1024 x 1,048,576 x 768, i8 -> i32
    v4i *source, *target;
    int *sink;
    CHECK(hipMalloc(&source, read_bytes));
    CHECK(hipMalloc(&target, written_bytes));
    CHECK(hipMalloc(&sink, 4096));
    CHECK(hipMemset(source, 1, read_bytes));
    hipEvent_t begin, end;
    CHECK(hipEventCreate(&begin));
    CHECK(hipEventCreate(&end));
    printf("0.75 GiB read and 4 GiB written by 8192 workgroups of linear 16-byte accesses, 5 launches after 2\n%-58s %8s %8s %12s\n", "", "ms", "GB/s", "of 8 TB/s");
    for (int past_caches = 1; past_caches >= 0; --past_caches)
        for (int readers : {0, 8, 2}) {
            if (readers == 8 && !past_caches) continue;
            for (int launch = 0; launch < 7; ++launch) {
                if (launch == 2) CHECK(hipEventRecord(begin, 0));
                hipLaunchKernelGGL(stream_kernel, dim3(8192), dim3(256), 0, 0, source, read_bytes / 16, target, written_bytes / 16, readers, sink, past_caches);
            }
            CHECK(hipEventRecord(end, 0));
            CHECK(hipEventSynchronize(end));
            CHECK(hipGetLastError());
            float ms = 0;
            CHECK(hipEventElapsedTime(&ms, begin, end));
            ms /= 5;
            double const bytes = (readers ? (double)read_bytes : 0) + (readers < 8 ? (double)written_bytes : 0);
            char name[96];
            snprintf(name, sizeof name, "%s%s", readers == 0 ? "written only" : (readers == 8 ? "read only" : "both (2 of 8 workgroups read)"),
                     readers == 8 ? "" : (past_caches ? ", stores past the caches" : ", plain stores"));
            printf("%-58s %8.3f %8.0f %12.3f\n", name, ms, bytes / ms / 1e6, bytes / ms / 1e6 / 8000);
        }
    return 0;
}

#pragma endregion Stream

#pragma region Numerics

enum Mode { kLegacyFP8, kLegacyBF8, kScaledFP8, kScaledBF8, kHalf, kBrain, kModes };
static char const *const kModeNames[kModes] = {"v_mfma_f32_32x32x16_fp8_fp8", "v_mfma_f32_32x32x16_bf8_bf8", "v_mfma_scale_f32_32x32x64_f8f6f4 (fp8)",
                                               "v_mfma_scale_f32_32x32x64_f8f6f4 (bf8)", "v_mfma_f32_32x32x16_f16", "v_mfma_f32_32x32x16_bf16"};
static int bytes_per_lane(int mode) { return mode <= kLegacyBF8 ? 8 : (mode <= kScaledBF8 ? 32 : 16); }
static int depth_of(int mode) { return mode <= kLegacyBF8 ? 16 : (mode <= kScaledBF8 ? 64 : 16); }

/** `steps` instructions in a row on one wavefront: operands of step s at a + s * 64 * bytes_per_lane, accumulator from `c`.
 *  One kernel per instruction (the instruction is a compile-time choice: nothing but loads and the one MFMA in the loop).
 *  `UNIT_SCALES`: the block-scaled form with explicit scales of 2^0 (E8M0 code 127) instead of the plain f8f6f4 form. */
template <int MODE, bool UNIT_SCALES>
__global__ __launch_bounds__(64) void mfma_steps_kernel(uint8_t const *a, uint8_t const *b, float const *c, float *out, int steps) {
    int const lane = threadIdx.x;
    v16f acc;
    for (int v = 0; v < 16; ++v) acc[v] = c[lane * 16 + v];
    for (int s = 0; s < steps; ++s) {
        if constexpr (MODE <= kLegacyBF8) {
            long const x = *(long const *)(a + ((size_t)s * 64 + lane) * 8), y = *(long const *)(b + ((size_t)s * 64 + lane) * 8);
            acc = MODE == kLegacyFP8 ? __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(x, y, acc, 0, 0, 0) : __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(x, y, acc, 0, 0, 0);
        }
        else if constexpr (MODE <= kScaledBF8) {
            v8i const x = *(v8i const *)(a + ((size_t)s * 64 + lane) * 32), y = *(v8i const *)(b + ((size_t)s * 64 + lane) * 32);
            // (format selectors 0 = fp8, 1 = bf8; constant scales of zero make the compiler select the instruction without scales)
            constexpr int kFormat = MODE == kScaledFP8 ? 0 : 1;
            if constexpr (UNIT_SCALES) acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, acc, kFormat, kFormat, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
            else acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, acc, kFormat, kFormat, 0, 0, 0, 0);
        }
        else if constexpr (MODE == kHalf) {
            v8h const x = *(v8h const *)(a + ((size_t)s * 64 + lane) * 16), y = *(v8h const *)(b + ((size_t)s * 64 + lane) * 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(x, y, acc, 0, 0, 0);
        }
        else {
            v8bf const x = *(v8bf const *)(a + ((size_t)s * 64 + lane) * 16), y = *(v8bf const *)(b + ((size_t)s * 64 + lane) * 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc, 0, 0, 0);
        }
    }
    for (int v = 0; v < 16; ++v) out[lane * 16 + v] = acc[v];
}

/** Operands of `steps` instructions as the host sees them: element k of row r of step s. Lane l of a step holds row
 *  l % 32 and the depths [(l / 32) * depth / 2, (l / 32 + 1) * depth / 2). */
struct Operands {
    int mode, steps;
    std::vector<uint8_t> bytes;
    Operands(int mode_, int steps_) : mode(mode_), steps(steps_), bytes((size_t)steps_ * 64 * bytes_per_lane(mode_), 0) {}
    void set(int step, int row, int k, uint32_t code) {
        int const half = depth_of(mode) / 2, lane = row + 32 * (k / half), e = k % half;
        size_t const base = ((size_t)step * 64 + lane) * bytes_per_lane(mode);
        if (mode <= kScaledBF8) bytes[base + e] = (uint8_t)code;
        else bytes[base + 2 * e] = (uint8_t)code, bytes[base + 2 * e + 1] = (uint8_t)(code >> 8);
    }
};
/** Output (i, j) of a 32 x 32 block: lane j + 32 * ((i / 4) % 2), register (i % 4) + 4 * (i / 8). */
static float output_at(std::vector<float> const &out, int i, int j) { return out[(size_t)(j + 32 * ((i / 4) % 2)) * 16 + (i % 4) + 4 * (i / 8)]; }

static uint8_t *g_a, *g_b;
static float *g_c, *g_out;
static std::vector<float> run_steps(Operands const &a, Operands const &b, std::vector<float> const &c, bool unit_scales = false) {
    CHECK(hipMemcpy(g_a, a.bytes.data(), a.bytes.size(), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(g_b, b.bytes.data(), b.bytes.size(), hipMemcpyHostToDevice));
    CHECK(hipMemcpy(g_c, c.data(), 4096, hipMemcpyHostToDevice));
    CHECK(hipMemset(g_out, 0xFF, 4096));
    void (*kernel)(uint8_t const *, uint8_t const *, float const *, float *, int) = mfma_steps_kernel<kLegacyFP8, false>;
    switch (a.mode) {
    case kLegacyBF8: kernel = mfma_steps_kernel<kLegacyBF8, false>; break;
    case kScaledFP8: kernel = unit_scales ? mfma_steps_kernel<kScaledFP8, true> : mfma_steps_kernel<kScaledFP8, false>; break;
    case kScaledBF8: kernel = unit_scales ? mfma_steps_kernel<kScaledBF8, true> : mfma_steps_kernel<kScaledBF8, false>; break;
    case kHalf: kernel = mfma_steps_kernel<kHalf, false>; break;
    case kBrain: kernel = mfma_steps_kernel<kBrain, false>; break;
    default: break;
    }
    hipLaunchKernelGGL(kernel, dim3(1), dim3(64), 0, 0, g_a, g_b, g_c, g_out, a.steps);
    CHECK(hipGetLastError());
    std::vector<float> out(1024);
    CHECK(hipMemcpy(out.data(), g_out, 4096, hipMemcpyDeviceToHost));
    return out;
}

static uint32_t code_of(int mode, float value) {
    if (mode == kHalf) return f16_of(value);
    if (mode == kBrain) return bf16_of(value);
    bool const e4 = mode == kLegacyFP8 || mode == kScaledFP8;
    for (int c = 0; c < 256; ++c)
        if ((e4 ? e4m3_value((uint8_t)c) : e5m2_value((uint8_t)c)) == value && !signbit(e4 ? e4m3_value((uint8_t)c) : e5m2_value((uint8_t)c)) == !signbit(value)) return (uint32_t)c;
    return 0xFFFFFFFFu;
}

/** Largest g for which 1 * 1 + 2^-a * 2^-(g - a) comes back as 1 + 2^-g, the second product at depth `k_second`
 *  of the same instruction (or, `through_accumulator`, the 1 in the accumulator instead of a product). */
static int widest_gap_kept(int mode, int k_second, bool through_accumulator) {
    int kept = 0;
    for (int g = 1; g <= 23; ++g) {
        int found = 0;
        for (int first = 0; first <= g && !found; ++first) { // any split of the exponent the format can represent
            uint32_t const small_a = code_of(mode, ldexpf(1, -first)), small_b = code_of(mode, ldexpf(1, -(g - first)));
            if (small_a == 0xFFFFFFFFu || small_b == 0xFFFFFFFFu) continue;
            Operands a(mode, 1), b(mode, 1);
            std::vector<float> c(1024, 0.0f);
            if (through_accumulator) c[0] = 1.0f, a.set(0, 0, 0, small_a), b.set(0, 0, 0, small_b);
            else {
                a.set(0, 0, 0, code_of(mode, 1.0f)), b.set(0, 0, 0, code_of(mode, 1.0f));
                a.set(0, 0, k_second, small_a), b.set(0, 0, k_second, small_b);
            }
            found = output_at(run_steps(a, b, c), 0, 0) == 1.0f + ldexpf(1, -g);
        }
        if (!found) break;
        kept = g;
    }
    return kept;
}

struct ErrorStats {
    double mean, max;
};

/** 32 x 32 e4m3 dot products of depth `depth`, N(0, 1) scaled to half the largest finite value with 1 % zeros (the
 *  benchmark's fp8 family): normwise error |c - truth| / sum|a b| of the given matrix-core route against the f64 truth. */
static ErrorStats depth_error(int mode, int depth, std::vector<uint8_t> const &a_codes, std::vector<uint8_t> const &b_codes, std::vector<double> const &truth,
                              std::vector<double> const &magnitude, bool unit_scales = false) {
    int const per = depth_of(mode), steps = depth / per;
    Operands a(mode, steps), b(mode, steps);
    for (int row = 0; row < 32; ++row)
        for (int k = 0; k < depth; ++k) {
            uint8_t const x = a_codes[(size_t)row * depth + k], y = b_codes[(size_t)row * depth + k];
            a.set(k / per, row, k % per, mode == kHalf ? f16_of(e4m3_value(x)) : x);
            b.set(k / per, row, k % per, mode == kHalf ? f16_of(e4m3_value(y)) : y);
        }
    std::vector<float> const out = run_steps(a, b, std::vector<float>(1024, 0.0f), unit_scales);
    ErrorStats stats = {0, 0};
    for (int i = 0; i < 32; ++i)
        for (int j = 0; j < 32; ++j) {
            double const e = fabs((double)output_at(out, i, j) - truth[i * 32 + j]) / magnitude[i * 32 + j];
            stats.mean += e / 1024, stats.max = e > stats.max ? e : stats.max;
        }
    return stats;
}

static int numerics_mode(bool check) {
    size_t const most = (size_t)(8192 / 16) * 64 * 16 + 4096;
    CHECK(hipMalloc(&g_a, most));
    CHECK(hipMalloc(&g_b, most));
    CHECK(hipMalloc(&g_c, 4096));
    CHECK(hipMalloc(&g_out, 4096));
    int failures = 0;
    printf("Largest g with 1 + 2^-g exact (f32 keeps g <= 23), the two addends being:\n%-44s %16s %16s %16s\n", "instruction", "products, one lane", "products, two lanes",
           "accumulator + product");
    int kept[kModes][3];
    for (int mode = 0; mode < kModes; ++mode) {
        kept[mode][0] = widest_gap_kept(mode, 1, false), kept[mode][1] = widest_gap_kept(mode, depth_of(mode) / 2, false);
        kept[mode][2] = widest_gap_kept(mode, 0, true);
        printf("%-44s %16d %16d %16d\n", kModeNames[mode], kept[mode][0], kept[mode][1], kept[mode][2]);
    }
    // what the kernels rely on: f16 and bf16 products are summed without loss; the fp8 forms lose the low bits
    for (int mode = kHalf; mode <= kBrain; ++mode)
        for (int column = 0; column < 3; ++column)
            if (kept[mode][column] < 23) ++failures, printf("UNEXPECTED: %s keeps only %d bits\n", kModeNames[mode], kept[mode][column]);

    int const depth = 8192;
    std::vector<uint8_t> a_codes((size_t)32 * depth), b_codes((size_t)32 * depth);
    for (size_t at = 0; at < a_codes.size(); ++at) {
        a_codes[at] = next_random() % 100 == 0 ? 0 : e4m3_of((float)(next_normal() * 224.0));
        b_codes[at] = next_random() % 100 == 0 ? 0 : e4m3_of((float)(next_normal() * 224.0));
    }
    std::vector<double> truth(1024), magnitude(1024), serial_error(1024);
    ErrorStats serial = {0, 0};
    for (int i = 0; i < 32; ++i)
        for (int j = 0; j < 32; ++j) {
            double sum = 0, absolute = 0;
            float lanes[4] = {0, 0, 0, 0}; // the reference's scalar kernel: exact products into four f32 sums by k mod 4
            for (int k = 0; k < depth; ++k) {
                float const x = e4m3_value(a_codes[(size_t)i * depth + k]), y = e4m3_value(b_codes[(size_t)j * depth + k]);
                sum += (double)x * y, absolute += fabs((double)x * y), lanes[k % 4] += x * y;
            }
            truth[i * 32 + j] = sum, magnitude[i * 32 + j] = absolute;
            double const e = fabs((double)(((lanes[0] + lanes[1]) + lanes[2]) + lanes[3]) - sum) / absolute;
            serial.mean += e / 1024, serial.max = e > serial.max ? e : serial.max;
        }
    printf("\ne4m3 dot products of depth %d, 32 x 32 outputs, normwise error against the f64 truth (mean, max):\n", depth);
    printf("%-56s %.3e %.3e\n", "f32 sums of exact products (reference, dot/serial.h:522-600)", serial.mean, serial.max);
    constexpr int kRoutes = 4;
    ErrorStats const routes[kRoutes] = {depth_error(kLegacyFP8, depth, a_codes, b_codes, truth, magnitude), depth_error(kScaledFP8, depth, a_codes, b_codes, truth, magnitude),
                                        depth_error(kScaledFP8, depth, a_codes, b_codes, truth, magnitude, true), depth_error(kHalf, depth, a_codes, b_codes, truth, magnitude)};
    char const *const route_names[kRoutes] = {"v_mfma_f32_32x32x16_fp8_fp8, one accumulator", "v_mfma_f32_32x32x64_f8f6f4, one accumulator",
                                              "v_mfma_scale_f32_32x32x64_f8f6f4, scales 2^0, one acc.", "widened to f16, v_mfma_f32_32x32x16_f16, one accumulator"};
    for (int route = 0; route < kRoutes; ++route)
        printf("%-56s %.3e %.3e   = %.1f x, %.1f x the reference's (gate: 2 x)\n", route_names[route], routes[route].mean, routes[route].max,
               routes[route].mean / serial.mean, routes[route].max / serial.max);
    if (check) {
        if (!(routes[3].mean < routes[0].mean && routes[3].mean < routes[1].mean && routes[3].mean < routes[2].mean)) ++failures, printf("UNEXPECTED: the f16 route is not the more accurate one\n");
        if (!(kept[kLegacyFP8][0] < 23 && kept[kScaledFP8][0] < 23)) printf("NOTE: the fp8 forms keep full f32 precision on this part: the f16 detour is no longer needed\n");
        printf(failures ? "FAILED\n" : "ok\n");
    }
    return failures ? 1 : 0;
}

#pragma endregion Numerics

int main(int argc, char **argv) {
    bool json = false, check = false;
    for (int i = 2; i < argc; ++i) json |= !strcmp(argv[i], "--json"), check |= !strcmp(argv[i], "--check");
    if (argc >= 2 && !strcmp(argv[1], "ceiling")) return ceiling_mode(json);
    if (argc >= 2 && !strcmp(argv[1], "numerics")) return numerics_mode(check);
    if (argc >= 2 && !strcmp(argv[1], "budget")) return budget_mode();
    if (argc >= 2 && !strcmp(argv[1], "stream")) return stream_mode();
    fprintf(stderr, "usage: %s ceiling [--json] | numerics [--check] | budget | stream\n", argv[0]);
    return 2;
}
