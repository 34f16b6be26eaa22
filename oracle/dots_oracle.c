/**
 *  @brief CPU restatement of NumKong's packed batched dots, serial semantics. TEST INFRASTRUCTURE ONLY.
 *  @file oracle/dots_oracle.c
 *
 *  This file is the checker, not the product: only tests/, __graft_entry__.smoke() and the cpu_baseline
 *  leg of bench.py may load it. Nothing under numkong_amd/ links, imports or calls it, and the product
 *  has no CPU fallback.
 *
 *  What is restated, and from where (paths relative to the reference checkout):
 *    - element decode/encode for f16, bf16, e4m3 (OCP E4M3FN), e5m2 (OCP)
 *          include/numkong/cast/serial.h:586-623, 669-741, 750-784, 810-839, 866-947, 1042-1082, 1109-1180
 *    - packed size and layout of the serial backend: 64-byte header {columns, depth, padded depth},
 *      rows padded with zeros, per-column norms behind them
 *          include/numkong/dots/serial.h:103-108, 245-271, 286-333, instantiated :2493-2599
 *    - the serial product: integers accumulate exactly in 64 bits and are truncated to 32,
 *      floats accumulate exact products into 4 f32 lane sums (lane = k mod 4, increasing k) that are
 *      combined as ((s0 + s1) + s2) + s3; C is overwritten
 *          include/numkong/dots/serial.h:520-1072, include/numkong/dot/serial.h:376-600
 *    - the f64 ground truth of the reference's own tests: sum = sum + (f64)a * (f64)b in depth order
 *          include/numkong/dots.hpp:42-61, test/test_cross.hpp:26-71
 *
 *  The conversions are written from the formats' definitions (value = (-1)^s * 2^(e-bias) * 1.m,
 *  round-to-nearest-even onto the target grid, the overflow/NaN policies listed in the comment tables of
 *  cast/serial.h), not from the reference's control flow. Every function here is pinned by
 *  tests/test_oracle.py: against the reference library built from its own sources (oracle/_ref) where
 *  that exists, against committed vectors produced from it (tests/golden), against torch's float8/
 *  float16/bfloat16 decoders, and against closed forms (exact integer products, powers of two).
 *
 *    - the packed distances on top of the packed product: per-row and per-column sums of squares
 *      (integers exact, truncated to 32 bits; floats as the serial Neumaier-compensated f32 sum of
 *      include/numkong/reduce/serial.h:223-300), the scalar reciprocal square root (bit trick + three Newton
 *      steps, include/numkong/scalar/serial.h:22-33) and the finalisers angular = max(1 - dot * rsqrt(qn * tn), 0)
 *      / euclidean = sqrt(max(qn + tn - 2 * dot, 0)) with their corner cases
 *          include/numkong/spatial/serial.h:257-344, include/numkong/dots/serial.h:2756-2800
 *      Pinned bit for bit against nk_angulars_packed_{i8,u8}_serial / nk_euclideans_packed_{i8,u8}_serial (where
 *      every input of the finaliser is an exact integer), and for the float types, whose norms the reference
 *      takes from whatever nk_reduce_moments_* kernel its dispatch picks on the host, to within 4 f32 ulp of
 *      the serial kernels' results.
 *
 *    - the symmetric kinds (all pairs of one set of vectors, upper triangle of a row window): the same per-pair
 *      arithmetic as the packed kinds, the diagonal of the distances exactly 0
 *          include/numkong/dots/serial.h:2039-2435, 2802-2878
 *      Pinned against nk_dots_symmetric_<T>_serial (bit for bit, all six types) and
 *      nk_{angulars,euclideans}_symmetric_<T>_serial (bit for bit for i8/u8, float types as above), over windows that
 *      start and end off the reference's 32- and 128-row blocks, and against the packed restatement with B = A.
 *
 *    - the remaining narrow types of the dots family, products only (packed and symmetric): e2m3 and e3m2 (decoded by
 *      the formats' definition, 4 f32 lane sums like the other float types), i4 and u4 (two nibbles per byte, the even
 *      dimension in the low one, whole bytes even for an odd depth; exact) and u1 (eight bits per byte, popcount of
 *      the AND over whole bytes)
 *          include/numkong/cast/serial.h:533-538, 1280-1330, 1418-1470, include/numkong/dot/serial.h:602-800
 *      Pinned bit for bit against nk_cast_serial (all 256 byte values decode; encoder on finite probes incl. every
 *      tie) and nk_dots_packed_<T>_serial / nk_dots_symmetric_<T>_serial.
 *      Distance kinds of e2m3, e3m2, i4, u4 (u1 has none): the finalisers above over these products and the sums of
 *      squares of include/numkong/reduce/serial.h:323-404 (the 4-bit types count both halves of every byte they
 *      touch). Sums of squares pinned bit for bit against nk_reduce_moments_<T>_serial; distances against
 *      nk_{angulars,euclideans}_{packed,symmetric}_<T>_serial: bit for bit for u4, for i4 on non-negative values (the
 *      reference's distance kernels take their norms from the host-dispatched moments, and its AVX2 i4 moments square
 *      negative values as unsigned, include/numkong/reduce/haswell.h:3629-3633) and on signed values against the f64
 *      formulas; the 6-bit floats to the tolerance of the other float types.
 *
 *    - the two wide types (packed and symmetric), f64 results: f32 by four f64 lane sums, f64 by the
 *      compensated two-lane sum with its compensated fold
 *          include/numkong/dot/serial.h:262-335, include/numkong/scalar/serial.h:128-136, include/numkong/reduce/serial.h:33-48
 *      Pinned bit for bit against nk_dots_packed_{f32,f64}_serial / nk_dots_symmetric_{f32,f64}_serial, and by what
 *      the arithmetic fixes: integer-valued inputs (exact), and for f64 a sum that cancels catastrophically in plain
 *      f64 and comes out right only if the compensation works.
 *      Their distance kinds: Neumaier-compensated f64 sums of squares (include/numkong/reduce/serial.h:50-92), the f64
 *      reciprocal square root (bit trick + four Newton steps, include/numkong/scalar/serial.h:35-47) and the finalisers
 *      of include/numkong/spatial/serial.h:281-302. Sums of squares pinned bit for bit against
 *      nk_reduce_moments_{f32,f64}_serial; distances against nk_{angulars,euclideans}_{packed,symmetric}_{f32,f64}_serial
 *      to 16 units of 2^-53 (their norms come from the host-dispatched moments), and against closed forms.
 *
 *  The per-column norms behind the rows of the serial packed image (dots/serial.h:326-332) are the sums of squares
 *  above: the reference takes them from whatever nk_reduce_moments_<T> its dispatch table holds, so the image is
 *  pinned byte for byte, norms included, against nk_dots_pack_<T>_serial with that table set to the serial kernels
 *  (nk_dispatch_table_update), and header + rows against it under any table. Nothing here is "parity unpinned".
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

enum {
    NKO_I8 = 1 << 2,
    NKO_U8 = 1 << 6,
    NKO_F16 = 1 << 12,
    NKO_BF16 = 1 << 13,
    NKO_E4M3 = 1 << 14,
    NKO_E5M2 = 1 << 15,
    NKO_I4 = 1 << 16,   /* two 4-bit integers per byte, the even dimension in the low nibble */
    NKO_U4 = 1 << 17,
    NKO_E2M3 = 1 << 18, /* 6-bit floats, one per byte, bits 6 and 7 ignored */
    NKO_E3M2 = 1 << 19,
    NKO_U1 = 1 << 1, /* eight 1-bit values per byte; their dot product is the popcount of the AND */
    NKO_F64 = 1 << 10, /* the two wide types: 8-byte (f64) results */
    NKO_F32 = 1 << 11,
};

#define NKO_API __attribute__((visibility("default")))

static float bits_to_f32(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint32_t f32_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

/* Small IEEE-like formats: sign, `ebits` exponent bits with bias, `mbits` mantissa bits. */
typedef struct {
    int ebits, mbits, bias;
    int has_inf;       /* all-ones exponent encodes Inf (m = 0) and NaN (m != 0), as f16 and e5m2 do      */
    int nan_is_all_ones; /* only exponent and mantissa all ones is NaN, no Inf (E4M3FN)                   */
    int saturate;      /* overflow (and Inf input) clamps to the largest finite value instead of Inf      */
    uint32_t nan_code; /* magnitude bits written for a NaN input                                          */
} small_format_t;

static small_format_t const k_f16 = {5, 10, 15, 1, 0, 0, 0x7E00};
static small_format_t const k_e4m3 = {4, 3, 7, 0, 1, 1, 0x7F};
static small_format_t const k_e5m2 = {5, 2, 15, 1, 0, 0, 0x7D};
/* FP6: no Inf, no NaN, overflow saturates (cast/serial.h:1280-1330, 1333-1339, 1418-1470); a NaN input has no
 * defined image here and is not used. */
static small_format_t const k_e2m3 = {2, 3, 1, 0, 0, 1, 0x1F};
static small_format_t const k_e3m2 = {3, 2, 3, 0, 0, 1, 0x1F};

static float small_decode(small_format_t const *fmt, uint32_t code) {
    int const total = 1 + fmt->ebits + fmt->mbits;
    uint32_t const sign = (code >> (total - 1)) & 1;
    uint32_t const e = (code >> fmt->mbits) & ((1u << fmt->ebits) - 1);
    uint32_t const m = code & ((1u << fmt->mbits) - 1);
    uint32_t const e_max = (1u << fmt->ebits) - 1;
    float magnitude;
    if (fmt->has_inf && e == e_max) {
        if (m == 0) magnitude = INFINITY;
        else {
            /* quiet NaN; f16 keeps its payload in the top mantissa bits like the reference does */
            uint32_t payload = fmt->mbits == 10 ? (m << 13) : 0x00400000u;
            return bits_to_f32((sign << 31) | 0x7F800000u | payload);
        }
    }
    else if (fmt->nan_is_all_ones && e == e_max && m == (1u << fmt->mbits) - 1) {
        return bits_to_f32((sign << 31) | 0x7FC00000u);
    }
    else if (e == 0) { magnitude = ldexpf((float)m, 1 - fmt->bias - fmt->mbits); }
    else { magnitude = ldexpf((float)((1u << fmt->mbits) | m), (int)e - fmt->bias - fmt->mbits); }
    return sign ? -magnitude : magnitude;
}

/* Round-to-nearest-even of a finite f32 onto the format's grid, done on the integer significand. */
static uint32_t small_encode(small_format_t const *fmt, float x) {
    int const total = 1 + fmt->ebits + fmt->mbits;
    uint32_t const bits = f32_to_bits(x);
    uint32_t const sign = (bits >> 31) << (total - 1);
    uint32_t const magnitude_bits = bits & 0x7FFFFFFFu;
    uint32_t const e_max = (1u << fmt->ebits) - 1;
    uint32_t const max_finite = fmt->has_inf ? ((e_max << fmt->mbits) - 1)        /* largest below Inf   */
                                : fmt->nan_is_all_ones ? ((e_max << fmt->mbits) | ((1u << fmt->mbits) - 2)) /* E4M3FN: 0x7E */
                                                       : ((e_max << fmt->mbits) | ((1u << fmt->mbits) - 1)); /* FP6: every code is a number */
    uint32_t const inf_code = e_max << fmt->mbits;
    if (magnitude_bits > 0x7F800000u) {
        if (fmt->mbits == 10) { /* f16 keeps the truncated payload, never letting it become zero */
            uint32_t payload = (magnitude_bits & 0x007FFFFFu) >> 13;
            if (!payload) payload = 1;
            return sign | inf_code | payload;
        }
        return sign | fmt->nan_code;
    }
    if (magnitude_bits == 0x7F800000u) return sign | (fmt->saturate ? max_finite : inf_code);
    if (magnitude_bits == 0) return sign;

    int exponent2;
    float const fraction = frexpf(fabsf(x), &exponent2); /* |x| = fraction * 2^exponent2, fraction in [0.5, 1) */
    int unbiased = exponent2 - 1;                       /* |x| = 1.f * 2^unbiased */
    int const min_normal = 1 - fmt->bias;
    /* quantum = spacing of the grid at this magnitude */
    int const quantum_exp = (unbiased < min_normal ? min_normal : unbiased) - fmt->mbits;
    /* |x| / 2^quantum_exp is exactly representable in double; round it to nearest even */
    double const scaled = ldexp((double)fraction, exponent2 - quantum_exp);
    double rounded = nearbyint(scaled); /* default rounding mode: to nearest, ties to even */
    uint64_t q = (uint64_t)rounded;
    if (q == 0) return sign;
    /* q is either a subnormal mantissa (< 2^mbits) or a significand in [2^mbits, 2^(mbits+1)] */
    int overflow = 0;
    uint32_t code = 0;
    if (unbiased < min_normal) { code = (uint32_t)q; /* a carry into 2^mbits lands on the first normal by itself */ }
    else {
        int e = unbiased + fmt->bias;
        if (q == (2ull << fmt->mbits)) q >>= 1, e += 1;
        if ((uint32_t)e > e_max) overflow = 1;
        else code = ((uint32_t)e << fmt->mbits) | ((uint32_t)q & ((1u << fmt->mbits) - 1));
    }
    if (fmt->has_inf) {
        if (overflow || code >= inf_code) return sign | (fmt->saturate ? max_finite : inf_code);
    }
    else if (overflow || code > max_finite) { return sign | max_finite; }
    return sign | code;
}

NKO_API float nko_f16_to_f32(uint16_t x) { return small_decode(&k_f16, x); }
NKO_API uint16_t nko_f32_to_f16(float x) { return (uint16_t)small_encode(&k_f16, x); }
NKO_API float nko_e4m3_to_f32(uint8_t x) { return small_decode(&k_e4m3, x); }
NKO_API uint8_t nko_f32_to_e4m3(float x) { return (uint8_t)small_encode(&k_e4m3, x); }
NKO_API float nko_e5m2_to_f32(uint8_t x) { return small_decode(&k_e5m2, x); }
NKO_API uint8_t nko_f32_to_e5m2(float x) { return (uint8_t)small_encode(&k_e5m2, x); }
NKO_API float nko_e2m3_to_f32(uint8_t x) { return small_decode(&k_e2m3, x & 0x3Fu); }
NKO_API uint8_t nko_f32_to_e2m3(float x) { return (uint8_t)small_encode(&k_e2m3, x); }
NKO_API float nko_e3m2_to_f32(uint8_t x) { return small_decode(&k_e3m2, x & 0x3Fu); }
NKO_API uint8_t nko_f32_to_e3m2(float x) { return (uint8_t)small_encode(&k_e3m2, x); }

/* bf16 is the top half of an f32; the reference rounds by adding 0x7FFF plus the kept LSB and does not
 * special-case NaN or overflow (cast/serial.h:768-784), which is restated literally because it defines
 * the result for every bit pattern. */
NKO_API float nko_bf16_to_f32(uint16_t x) { return bits_to_f32((uint32_t)x << 16); }
NKO_API uint16_t nko_f32_to_bf16(float x) {
    uint32_t u = f32_to_bits(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static int element_bytes(int dtype) {
    switch (dtype) {
    case NKO_I8:
    case NKO_U8:
    case NKO_E4M3:
    case NKO_E5M2: return 1;
    case NKO_F16:
    case NKO_BF16: return 2;
    default: return 0;
    }
}

/* Sub-byte types: a row of `depth` dimensions is read as whole bytes, all of the last one included when the depth
 * does not fill it, exactly as the reference's loads do (cast/serial.h:519-538, dot/serial.h:705-718, 777-790, 824-832). */
static size_t effective_depth(int dtype, size_t depth) {
    if (dtype == NKO_U1) return (depth + 7) / 8 * 8; /* cast/serial.h:519-524 */
    return dtype == NKO_I4 || dtype == NKO_U4 ? (depth + 1) / 2 * 2 : depth;
}

/* Value of element `i` of a row as f32 (integers are exact in f32 too: |x| <= 255). */
static float element_f32(int dtype, void const *row, size_t i) {
    switch (dtype) {
    case NKO_U1: return (float)((((uint8_t const *)row)[i / 8] >> (i & 7)) & 1);
    case NKO_U4: return (float)((((uint8_t const *)row)[i / 2] >> (4 * (i & 1))) & 0xF);
    case NKO_I4: {
        int const nibble = (((uint8_t const *)row)[i / 2] >> (4 * (i & 1))) & 0xF;
        return (float)((nibble ^ 8) - 8); /* dot/serial.h:781-785 */
    }
    case NKO_E2M3: return nko_e2m3_to_f32(((uint8_t const *)row)[i]);
    case NKO_E3M2: return nko_e3m2_to_f32(((uint8_t const *)row)[i]);
    case NKO_I8: return (float)((int8_t const *)row)[i];
    case NKO_U8: return (float)((uint8_t const *)row)[i];
    case NKO_F16: return nko_f16_to_f32(((uint16_t const *)row)[i]);
    case NKO_BF16: return nko_bf16_to_f32(((uint16_t const *)row)[i]);
    case NKO_E4M3: return nko_e4m3_to_f32(((uint8_t const *)row)[i]);
    case NKO_E5M2: return nko_e5m2_to_f32(((uint8_t const *)row)[i]);
    default: return NAN;
    }
}

/* The same as f64, which also covers the two wide types. */
static double element_f64(int dtype, void const *row, size_t i) {
    if (dtype == NKO_F32) return (double)((float const *)row)[i];
    if (dtype == NKO_F64) return ((double const *)row)[i];
    return (double)element_f32(dtype, row, i);
}

NKO_API void nko_decode(int dtype, void const *src, size_t count, float *dst) {
    for (size_t i = 0; i < count; ++i) dst[i] = element_f32(dtype, src, i);
}

NKO_API void nko_encode(int dtype, float const *src, size_t count, void *dst) {
    for (size_t i = 0; i < count; ++i) switch (dtype) {
        case NKO_F16: ((uint16_t *)dst)[i] = nko_f32_to_f16(src[i]); break;
        case NKO_BF16: ((uint16_t *)dst)[i] = nko_f32_to_bf16(src[i]); break;
        case NKO_E4M3: ((uint8_t *)dst)[i] = nko_f32_to_e4m3(src[i]); break;
        case NKO_E5M2: ((uint8_t *)dst)[i] = nko_f32_to_e5m2(src[i]); break;
        case NKO_E2M3: ((uint8_t *)dst)[i] = nko_f32_to_e2m3(src[i]); break;
        case NKO_E3M2: ((uint8_t *)dst)[i] = nko_f32_to_e3m2(src[i]); break;
        default: break;
        }
}

#pragma region Serial packed layout

/* Per backend instantiation: values per 128-bit step, and the element width stored in the image
 * (dots/serial.h:2493-2599; f16 is stored already widened to f32). */
static size_t serial_step(int dtype) {
    switch (dtype) {
    case NKO_F16: return 4;
    case NKO_BF16: return 8;
    default: return 16;
    }
}
static size_t serial_packed_element_bytes(int dtype) { return dtype == NKO_F16 ? 4 : (size_t)element_bytes(dtype); }

static size_t serial_padded_depth(int dtype, size_t depth) {
    size_t const step = serial_step(dtype);
    size_t padded = (depth + step - 1) / step * step;
    size_t const stride_bytes = padded * serial_packed_element_bytes(dtype);
    /* a power-of-two row stride is broken up by one extra step (dots/serial.h:260-265) */
    if (stride_bytes && !(stride_bytes & (stride_bytes - 1))) padded += step;
    return padded;
}

NKO_API size_t nko_serial_packed_size(int dtype, size_t columns, size_t depth) {
    if (!element_bytes(dtype)) return 0;
    return 64 + columns * serial_padded_depth(dtype, depth) * serial_packed_element_bytes(dtype) + columns * 4;
}

static uint32_t row_sumsq_bits(int dtype, void const *row, size_t depth);

NKO_API void nko_serial_pack(int dtype, void const *b, size_t columns, size_t depth, size_t b_stride, void *packed) {
    size_t const padded = serial_padded_depth(dtype, depth);
    size_t const width = serial_packed_element_bytes(dtype);
    uint32_t header[16] = {0};
    header[0] = (uint32_t)columns, header[1] = (uint32_t)depth, header[2] = (uint32_t)padded;
    memcpy(packed, header, 64);
    unsigned char *rows = (unsigned char *)packed + 64;
    for (size_t j = 0; j < columns; ++j) {
        unsigned char const *source = (unsigned char const *)b + j * b_stride;
        unsigned char *target = rows + j * padded * width;
        memset(target, 0, padded * width);
        if (dtype == NKO_F16)
            for (size_t l = 0; l < depth; ++l) ((float *)target)[l] = nko_f16_to_f32(((uint16_t const *)source)[l]);
        else memcpy(target, source, depth * width);
    }
    /* the norms behind the rows: u32 for the integers, f32 for the floats (dots/serial.h:124-164, 326-332) */
    uint32_t *norms = (uint32_t *)(rows + columns * padded * width);
    for (size_t j = 0; j < columns; ++j) norms[j] = row_sumsq_bits(dtype, (unsigned char const *)b + j * b_stride, depth);
}

#pragma endregion Serial packed layout

#pragma region Products

/** C = A * B^T exactly as the serial backend rounds it, reading an image made by nko_serial_pack. */
NKO_API void nko_serial_packed(int dtype, void const *a, void const *packed, void *c, size_t rows, size_t columns,
                               size_t depth, size_t a_stride, size_t c_stride) {
    uint32_t header[16];
    memcpy(header, packed, 64);
    size_t const padded = header[2];
    size_t const width = serial_packed_element_bytes(dtype);
    unsigned char const *b_rows = (unsigned char const *)packed + 64;
    int const image_dtype = dtype == NKO_F16 ? 0 : dtype;
    for (size_t i = 0; i < rows; ++i) {
        unsigned char const *a_row = (unsigned char const *)a + i * a_stride;
        unsigned char *c_row = (unsigned char *)c + i * c_stride;
        for (size_t j = 0; j < columns; ++j) {
            unsigned char const *b_row = b_rows + j * padded * width;
            if (dtype == NKO_I8) {
                int64_t sum = 0;
                for (size_t l = 0; l < depth; ++l) sum += (int64_t)((int8_t const *)a_row)[l] * ((int8_t const *)b_row)[l];
                ((int32_t *)c_row)[j] = (int32_t)sum;
            }
            else if (dtype == NKO_U8) {
                uint64_t sum = 0;
                for (size_t l = 0; l < depth; ++l) sum += (uint64_t)a_row[l] * b_row[l];
                ((uint32_t *)c_row)[j] = (uint32_t)sum;
            }
            else {
                float lanes[4] = {0, 0, 0, 0};
                for (size_t l = 0; l < depth; ++l) {
                    float const x = element_f32(dtype, a_row, l);
                    float const y = image_dtype ? element_f32(image_dtype, b_row, l) : ((float const *)b_row)[l];
                    /* the product of two values with <= 11 significant bits is exact in f32; `volatile`
                     * keeps the compiler from contracting the multiply-add into one rounding */
                    volatile float product = x * y;
                    lanes[l & 3] += product;
                }
                ((float *)c_row)[j] = ((lanes[0] + lanes[1]) + lanes[2]) + lanes[3];
            }
        }
    }
}

/** f64 ground truth from the unpacked B: sum = sum + a * b in depth order (dots.hpp:42-61). Also returns,
 *  when `magnitude` is not NULL, sum |a * b| per element, the scale of the normwise error. */
NKO_API void nko_dots_f64(int dtype, void const *a, void const *b, double *c, double *magnitude, size_t rows,
                          size_t columns, size_t depth, size_t a_stride, size_t b_stride) {
    depth = effective_depth(dtype, depth);
    for (size_t i = 0; i < rows; ++i) {
        unsigned char const *a_row = (unsigned char const *)a + i * a_stride;
        for (size_t j = 0; j < columns; ++j) {
            unsigned char const *b_row = (unsigned char const *)b + j * b_stride;
            double sum = 0, absolute = 0;
            for (size_t l = 0; l < depth; ++l) {
                double const product = (double)element_f32(dtype, a_row, l) * (double)element_f32(dtype, b_row, l);
                sum = sum + product;
                absolute += fabs(product);
            }
            c[i * columns + j] = sum;
            if (magnitude) magnitude[i * columns + j] = absolute;
        }
    }
}

#pragma endregion Products

#pragma region Packed distances

/** Sum of squares of one row. Floats: Neumaier-compensated f32 running sum, as nk_reduce_moments_<T>_serial
 *  (reduce/serial.h:223-300); integers: exact in 64 bits, truncated to 32 (dots/serial.h:154-164). Returned as
 *  the bits of the f32 or of the u32. */
static uint32_t row_sumsq_bits(int dtype, void const *row, size_t depth) {
    depth = effective_depth(dtype, depth); /* (the 4-bit types count both halves of the last byte: reduce/serial.h:373-404) */
    if (dtype == NKO_I8 || dtype == NKO_U8 || dtype == NKO_I4 || dtype == NKO_U4) {
        uint64_t sum = 0;
        for (size_t l = 0; l < depth; ++l) {
            int64_t const v = (int64_t)element_f32(dtype, row, l); /* small integers: exact */
            sum += (uint64_t)(v * v);
        }
        return (uint32_t)sum;
    }
    volatile float running = 0, compensation = 0; /* volatile: every operation rounds to f32, in this order */
    for (size_t l = 0; l < depth; ++l) {
        float const value = element_f32(dtype, row, l);
        volatile float squared = value * value;
        volatile float tentative = running + squared;
        if (running >= squared) {
            volatile float lost = (running - tentative);
            lost = lost + squared;
            compensation = compensation + lost;
        }
        else {
            volatile float lost = (squared - tentative);
            lost = lost + running;
            compensation = compensation + lost;
        }
        running = tentative;
    }
    return f32_to_bits(running + compensation);
}

NKO_API void nko_row_sumsq(int dtype, void const *x, size_t rows, size_t depth, size_t stride, uint32_t *out_bits) {
    for (size_t i = 0; i < rows; ++i) out_bits[i] = row_sumsq_bits(dtype, (unsigned char const *)x + i * stride, depth);
}

/** scalar/serial.h:22-31: the bit-trick estimate refined by three Newton steps, all in f32. */
static float serial_rsqrt(float number) {
    volatile float y = bits_to_f32(0x5F375A86u - (f32_to_bits(number) >> 1));
    for (int step = 0; step < 3; ++step) {
        volatile float t = 0.5f * number;
        t = t * y;
        t = t * y;
        t = 1.5f - t;
        y = y * t;
    }
    return y;
}

/** spatial/serial.h:257-344. `dot`, `query` and `target` arrive as 32-bit patterns: f32 for the float types,
 *  i32 for i8 and i4 (their finalisers read both norms as signed), u32 for u8 and u4. */
static float serial_from_dot(int dtype, int metric, uint32_t dot_bits, uint32_t query_bits, uint32_t target_bits) {
    float dot, query, target;
    if (dtype == NKO_I8 || dtype == NKO_I4)
        dot = (float)(int32_t)dot_bits, query = (float)(int32_t)query_bits, target = (float)(int32_t)target_bits;
    else if (dtype == NKO_U8 || dtype == NKO_U4) dot = (float)dot_bits, query = (float)query_bits, target = (float)target_bits;
    else dot = bits_to_f32(dot_bits), query = bits_to_f32(query_bits), target = bits_to_f32(target_bits);
    if (metric == 1) {
        volatile float product = query * target;
        if (product > 0) {
            volatile float normalized = dot * serial_rsqrt(product);
            volatile float result = 1.0f - normalized;
            return result > 0 ? result : 0.0f;
        }
        return dot == 0 ? 0.0f : 1.0f;
    }
    volatile float squared = query + target;
    volatile float twice = 2.0f * dot;
    squared = squared - twice;
    if (!(squared > 0)) return 0.0f;
    volatile float root = squared * serial_rsqrt(squared); /* scalar/serial.h:33 */
    return root;
}

/** Sum of squares of one f32 or f64 row in f64: Neumaier-compensated running sum of the squares, one element after
 *  the other, as nk_reduce_moments_{f32,f64}_serial (reduce/serial.h:50-92). */
static double row_sumsq_wide(int dtype, void const *row, size_t depth) {
    double running = 0, compensation = 0;
    for (size_t l = 0; l < depth; ++l) {
        double const value = element_f64(dtype, row, l);
        double const squared = value * value;
        double const tentative = running + squared;
        if (running >= squared) compensation += (running - tentative) + squared;
        else compensation += (squared - tentative) + running;
        running = tentative;
    }
    return running + compensation;
}

NKO_API void nko_row_sumsq_wide(int dtype, void const *x, size_t rows, size_t depth, size_t stride, double *out) {
    for (size_t i = 0; i < rows; ++i) out[i] = row_sumsq_wide(dtype, (unsigned char const *)x + i * stride, depth);
}

/** scalar/serial.h:35-47: the bit-trick estimate refined by four Newton steps, all in f64. */
static double serial_rsqrt_wide(double number) {
    uint64_t bits;
    memcpy(&bits, &number, 8);
    bits = 0x5FE6EB50C7B537A9ull - (bits >> 1);
    double y;
    memcpy(&y, &bits, 8);
    for (int step = 0; step < 4; ++step) y = y * (1.5 - 0.5 * number * y * y);
    return y;
}

/** spatial/serial.h:281-302: the f64 finalisers of the f32 and f64 inputs. */
static double serial_from_dot_wide(int metric, double dot, double query, double target) {
    if (metric == 1) {
        double const product = query * target;
        if (product > 0) {
            double const result = 1.0 - dot * serial_rsqrt_wide(product);
            return result > 0 ? result : 0;
        }
        return dot == 0 ? 0.0 : 1.0;
    }
    double const squared = query + target - 2.0 * dot;
    return squared > 0 ? squared * serial_rsqrt_wide(squared) : 0.0;
}

NKO_API void nko_serial_dots(int dtype, void const *a, void const *b, void *c, size_t rows, size_t columns, size_t depth,
                             size_t a_stride, size_t b_stride, size_t c_stride);

/** nk_angulars_packed_<T>_serial (metric 1) / nk_euclideans_packed_<T>_serial (metric 2) from unpacked B:
 *  the serial product, then the finaliser per element with the row's and the column's sum of squares. */
NKO_API void nko_serial_spatials(int dtype, int metric, void const *a, void const *b, void *c, size_t rows,
                                 size_t columns, size_t depth, size_t a_stride, size_t b_stride, size_t c_stride) {
    nko_serial_dots(dtype, a, b, c, rows, columns, depth, a_stride, b_stride, c_stride); /* (= pack + packed, per pair) */
    if (dtype == NKO_F32 || dtype == NKO_F64) { /* f64 dots, f64 sums of squares, f64 results */
        double *target_norms = (double *)__builtin_malloc(columns * sizeof(double) + 8);
        nko_row_sumsq_wide(dtype, b, columns, depth, b_stride, target_norms);
        for (size_t i = 0; i < rows; ++i) {
            double const query_norm = row_sumsq_wide(dtype, (unsigned char const *)a + i * a_stride, depth);
            double *row = (double *)((unsigned char *)c + i * c_stride);
            for (size_t j = 0; j < columns; ++j) row[j] = serial_from_dot_wide(metric, row[j], query_norm, target_norms[j]);
        }
        __builtin_free(target_norms);
        return;
    }
    uint32_t *target_norms = (uint32_t *)__builtin_malloc(columns * sizeof(uint32_t) + 4);
    nko_row_sumsq(dtype, b, columns, depth, b_stride, target_norms);
    for (size_t i = 0; i < rows; ++i) {
        uint32_t const query_norm = row_sumsq_bits(dtype, (unsigned char const *)a + i * a_stride, depth);
        uint32_t *row = (uint32_t *)((unsigned char *)c + i * c_stride);
        for (size_t j = 0; j < columns; ++j)
            row[j] = f32_to_bits(serial_from_dot(dtype, metric, row[j], query_norm, target_norms[j]));
    }
    __builtin_free(target_norms);
}

/** f64 ground truth of the distances from the unpacked operands (test/test_cross.hpp:290-427 computes its
 *  references the same way: f64 dot and norms, then the formula). */
NKO_API void nko_spatials_f64(int dtype, int metric, void const *a, void const *b, double *c, size_t rows, size_t columns,
                              size_t depth, size_t a_stride, size_t b_stride) {
    depth = effective_depth(dtype, depth);
    for (size_t i = 0; i < rows; ++i) {
        unsigned char const *a_row = (unsigned char const *)a + i * a_stride;
        double query = 0;
        for (size_t l = 0; l < depth; ++l) query += element_f64(dtype, a_row, l) * element_f64(dtype, a_row, l);
        for (size_t j = 0; j < columns; ++j) {
            unsigned char const *b_row = (unsigned char const *)b + j * b_stride;
            double dot = 0, target = 0;
            for (size_t l = 0; l < depth; ++l) {
                double const x = element_f64(dtype, a_row, l), y = element_f64(dtype, b_row, l);
                dot += x * y, target += y * y;
            }
            double result;
            if (metric == 1) {
                double const product = query * target;
                result = product > 0 ? 1.0 - dot / sqrt(product) : (dot == 0 ? 0.0 : 1.0);
                if (result < 0) result = 0;
            }
            else {
                double const squared = query + target - 2.0 * dot;
                result = squared > 0 ? sqrt(squared) : 0.0;
            }
            c[i * columns + j] = result;
        }
    }
}

#pragma endregion Packed distances

#pragma region Symmetric kinds

/** One serial dot product of two unpacked rows, as 32 result bits: the arithmetic of nko_serial_packed. The
 *  symmetric kernels run the same per-pair state machines as the packed ones (dots/serial.h:2499-2603 name the
 *  same init/update/finalize functions for both; f16 goes through nk_dot_f16x8_*_serial, dot/serial.h:345-374,
 *  which keeps the same four lane sums, lane = k mod 4, as the f32x4 path of its packed kernel). */
static uint32_t serial_dot_bits(int dtype, void const *a_row, void const *b_row, size_t depth) {
    depth = effective_depth(dtype, depth);
    if (dtype == NKO_I8 || dtype == NKO_U8 || dtype == NKO_I4 || dtype == NKO_U4 || dtype == NKO_U1) {
        /* exact in 64 bits, truncated to 32: i64 for the signed types, u64 for the unsigned, the same bits either way */
        int64_t sum = 0;
        for (size_t l = 0; l < depth; ++l) sum += (int64_t)element_f32(dtype, a_row, l) * (int64_t)element_f32(dtype, b_row, l);
        return (uint32_t)(uint64_t)sum;
    }
    float lanes[4] = {0, 0, 0, 0};
    for (size_t l = 0; l < depth; ++l) {
        volatile float product = element_f32(dtype, a_row, l) * element_f32(dtype, b_row, l); /* exact, see above */
        lanes[l & 3] += product;
    }
    return f32_to_bits(((lanes[0] + lanes[1]) + lanes[2]) + lanes[3]);
}

/** The wide types. f32 (dot/serial.h:305-335): products, exact in f64, go to four f64 sums by k mod 4 (rows are padded
 *  with zeros to a multiple of 4, and the zeros are added like any other term), combined ((s0 + s1) + s2) + s3.
 *  f64 (dot/serial.h:262-303, scalar/serial.h:128-136, reduce/serial.h:33-48): two lanes by k mod 2 (padded to a multiple
 *  of 2), each a running sum and a compensation fed by the exact error of every product (by fma) and of every addition
 *  (TwoSum); the four numbers are folded in the order s0, c0, s1, c1 by one more compensated chain. This file is compiled
 *  with contraction off, so every operation written here rounds on its own. */
static double serial_dot_wide(int dtype, void const *a_row, void const *b_row, size_t depth) {
    if (dtype == NKO_F32) {
        float const *a = (float const *)a_row, *b = (float const *)b_row;
        double lanes[4] = {0, 0, 0, 0};
        size_t const padded = (depth + 3) / 4 * 4;
        for (size_t l = 0; l < padded; ++l) {
            double const x = l < depth ? (double)a[l] : 0.0, y = l < depth ? (double)b[l] : 0.0;
            lanes[l & 3] += x * y;
        }
        return ((lanes[0] + lanes[1]) + lanes[2]) + lanes[3];
    }
    double const *a = (double const *)a_row, *b = (double const *)b_row;
    double sums[2] = {0, 0}, compensations[2] = {0, 0};
    size_t const padded = (depth + 1) / 2 * 2;
    for (size_t l = 0; l < padded; ++l) {
        double const x = l < depth ? a[l] : 0.0, y = l < depth ? b[l] : 0.0;
        double const product = x * y;
        double const product_error = fma(x, y, -product);
        double const running = sums[l & 1] + product;
        double const recovered = running - sums[l & 1];
        double const sum_error = (sums[l & 1] - (running - recovered)) + (product - recovered);
        sums[l & 1] = running;
        compensations[l & 1] += sum_error + product_error;
    }
    double const values[4] = {sums[0], compensations[0], sums[1], compensations[1]};
    double running = 0, error = 0;
    for (int i = 0; i < 4; ++i) {
        double const tentative = running + values[i];
        double const recovered = tentative - running;
        error += (running - (tentative - recovered)) + (values[i] - recovered);
        running = tentative;
    }
    return running + error;
}

/** C = A * B^T with the serial backend's rounding from UNPACKED operands: what nk_dots_packed_<T>_serial returns for
 *  any of the ten types (for the six older ones it equals nko_serial_pack + nko_serial_packed, which also restate
 *  the serial image; for e2m3, e3m2, i4, u4, u1 only the arithmetic is restated: dot/serial.h:602-832). */
NKO_API void nko_serial_dots(int dtype, void const *a, void const *b, void *c, size_t rows, size_t columns, size_t depth,
                             size_t a_stride, size_t b_stride, size_t c_stride) {
    for (size_t i = 0; i < rows; ++i) {
        uint32_t *out = (uint32_t *)((unsigned char *)c + i * c_stride);
        for (size_t j = 0; j < columns; ++j) {
            void const *a_row = (unsigned char const *)a + i * a_stride, *b_row = (unsigned char const *)b + j * b_stride;
            if (dtype == NKO_F32 || dtype == NKO_F64) ((double *)out)[j] = serial_dot_wide(dtype, a_row, b_row, depth);
            else out[j] = serial_dot_bits(dtype, a_row, b_row, depth);
        }
    }
}

/** nk_dots_symmetric_<T>_serial (metric 0), nk_angulars_symmetric_<T>_serial (1), nk_euclideans_symmetric_<T>_serial
 *  (2): for the rows i of [row_start, row_start + row_count) and the columns j >= i only, result[i][j] = the dot
 *  product of vectors i and j (dots/serial.h:2361-2435: upper triangle, the rest of the result is not this call's),
 *  or its finaliser with the two vectors' sums of squares for j > i and exactly 0 on the diagonal
 *  (dots/serial.h:2802-2878). Everything else in `result` is left alone. */
NKO_API void nko_serial_symmetric(int dtype, int metric, void const *vectors, size_t count, size_t depth, size_t stride,
                                  void *result, size_t result_stride, size_t row_start, size_t row_count) {
    size_t const row_end = row_start + row_count < count ? row_start + row_count : count;
    int const wide = dtype == NKO_F32 || dtype == NKO_F64; /* (8-byte outputs, f64 sums of squares) */
    uint32_t *norms = NULL;
    double *wide_norms = NULL;
    if (metric && !wide) {
        norms = (uint32_t *)__builtin_malloc(count * sizeof(uint32_t) + 4);
        nko_row_sumsq(dtype, vectors, count, depth, stride, norms);
    }
    if (metric && wide) {
        wide_norms = (double *)__builtin_malloc(count * sizeof(double) + 8);
        nko_row_sumsq_wide(dtype, vectors, count, depth, stride, wide_norms);
    }
    for (size_t i = row_start; i < row_end; ++i) {
        unsigned char const *a_row = (unsigned char const *)vectors + i * stride;
        uint32_t *out = (uint32_t *)((unsigned char *)result + i * result_stride);
        for (size_t j = i; j < count; ++j) {
            if (wide) {
                double const dot = serial_dot_wide(dtype, a_row, (unsigned char const *)vectors + j * stride, depth);
                if (!metric) ((double *)out)[j] = dot;
                else ((double *)out)[j] = i == j ? 0.0 : serial_from_dot_wide(metric, dot, wide_norms[i], wide_norms[j]);
                continue;
            }
            uint32_t const dot = serial_dot_bits(dtype, a_row, (unsigned char const *)vectors + j * stride, depth);
            if (!metric) out[j] = dot;
            else out[j] = i == j ? 0u : f32_to_bits(serial_from_dot(dtype, metric, dot, norms[i], norms[j]));
        }
    }
    if (norms) __builtin_free(norms);
    if (wide_norms) __builtin_free(wide_norms);
}

#pragma endregion Symmetric kinds
