/**
 *  @brief gfx950 (MI355X, CDNA4) kernels for packed batched dot products: C = A * B^T.
 *  @file numkong_amd/csrc/dots_gfx950.hpp
 *
 *  Everything the HIP translation units share: the packed image, the packing kernels, the element types and the
 *  product kernel with its launch logic. dots_gfx950.hip holds the plain-C entry points of <numkong_amd/hip_abi.h>;
 *  dots_gfx950_<T>.hip instantiate the product kernels of one element type each, so that they compile side by side.
 *
 *  Replaces the per-ISA kernels the reference instantiates from
 *  include/numkong/dots/serial.h:245-333 (pack size, pack) and :520-1072 (packed product) for
 *  i8, u8, bf16, f16, e4m3, e5m2.
 *
 *  Packed image of B (n rows of k elements), all little-endian:
 *
 *      [ 64-byte header ][ tiles ][ per-column compensation terms, u32 x 32 x n_tiles ]
 *
 *  A "chunk" is 16 consecutive bytes of one B row (16 i8/fp8 values, 8 bf16/f16 values). Rows are grouped
 *  into tiles of 32; K is padded with zeros to a multiple of 8 chunks (128 bytes) and N with zero rows to
 *  a multiple of 32. Chunk `c` of row `r` of tile `t` lives at
 *
 *      data + ((t * k_chunks + c) * 32 + r) * 16
 *
 *  so the 64 lanes of a wavefront that execute one 32x32 MFMA step `q` (lane l supplies row l % 32 and
 *  chunk 2q + l / 32) read 1024 contiguous bytes at `data + (t * k_chunks + 2q) * 512 + l * 16`: the image
 *  is the MFMA operand-fragment order, and B goes from HBM to registers with one coalesced 128-bit load
 *  per lane per step, never through LDS. Which k sits in which operand slot of the instruction does not
 *  matter as long as A and B agree, and they do: A fragments are read from LDS with the same rule.
 *  e4m3, e5m2 and e3m2 are stored widened to f16 (see packed_bytes_of), so their chunks hold 8 values.
 *
 *  u8 has no unsigned MFMA. B is stored as b' = b ^ 0x80 (signed b - 128), A is turned into
 *  a' = a ^ 0x80 on its way into LDS, and  sum(a*b) = sum(a'*b') + 128*sum(a) + 128*sum(b')  (mod 2^32)
 *  with zero padding contributing nothing. 128*sum(b') per column is stored behind the tiles at pack
 *  time; sum(a) per row is accumulated with v_sad_u8 while A is staged.
 */#ifndef NUMKONG_AMD_DOTS_GFX950_HPP
#define NUMKONG_AMD_DOTS_GFX950_HPP

#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include "numkong_amd/hip_abi.h"

/** What crosses translation units: the product's arguments, its scratch memory, one launcher per element type. */
namespace nk_gfx950 {

// Tile rows per band of the walk over the tile grid. An XCD works on 32 tiles at a time, a band's height times as many
// columns: 8 x 4 is the shape with the smallest perimeter for the 256 x 256 and the 128 x 256 tile alike, and the
// perimeter is what the XCD's L2 fetches per sweep of the depth (measured at 8192^3, bytes read per launch: bf16 2.18 GB
// with 8, 2.75 GB with 4 or 16, 5.28 GB with 2; i8 0.82 GB with 8 or 4, 1.22 GB with 2 or 16). NK_TILE_BAND overrides it
// for such measurements (make EXTRA=-DNK_TILE_BAND=4).
#ifndef NK_TILE_BAND
#define NK_TILE_BAND 8
#endif
constexpr uint32_t kTileBand = NK_TILE_BAND;
#ifndef NK_DIRECT_STAGING
#define NK_DIRECT_STAGING 1
#endif
constexpr bool kDirectStaging = NK_DIRECT_STAGING != 0; // A straight into LDS where that applies (see dots_packed_kernel)

struct GemmArgs {
    uint8_t const *a;
    uint8_t const *bp; // packed image (header first)
    uint8_t *c;
    uint64_t a_stride, c_stride, k_src_bytes;
    uint32_t m, n, k;
    uint32_t n_tiles, k_chunks;
    uint32_t tiles_m, tiles_n;
    int avec; // widest load the A pointer and stride allow (1, 2, 4, 8 or 16 bytes)
    int metric; // 0: dot products, 1: angular distances, 2: euclidean distances (kernels built with NORMS)
    uint32_t chunk_stages; // chunked types: stages between folds of the accumulator (even, 2..16)
    // Symmetric products (C = A x A^T, upper triangle): only elements with col >= row + tri_shift are stored
    // (`tri_mask` all ones; 0 switches the test off), and the tiles to compute come as a list.
    uint32_t tri_shift, tri_mask;
    // Store-bound shapes: workgroup b starts b * stagger_ticks / gridDim.x ticks of the 100 MHz clock late, so that the
    // compute phases of some compute units fall into the store phases of others (0: all start together).
    uint32_t stagger_ticks;
    uint32_t store_policy; // 0: by the alignment of C's rows; 1: past the caches; 2: through them (test hook)
    uint32_t tile_count;       // tiles_m * tiles_n, or the length of the list
    uint32_t const *tile_list; // (tile row, tile column) pairs in walking order, or NULL for the full grid
};

/** Scratch memory of a triangular grid: the first tile of every band, then the list itself. */
struct TriangleScratch {
    uint32_t *words;
    size_t bytes;
};

/** The product (or its triangular form) for one element type: picks the tile shape and launches. Defined in
 *  dots_gfx950_<T>.hip. */
hipError_t launch_i8(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_u8(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_bf16(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_f16(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_e4m3(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_e5m2(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_e2m3(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_e3m2(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_i4(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_u4(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);
hipError_t launch_u1(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle);

/** The wide types (f32, f64; f64 results), dots_gfx950_wide.hip: image = header + k-major f64 with zero padding. */
struct WideGeometry {
    uint32_t elem_bytes, n, k, n_padded, k_padded;
    uint64_t total_bytes;
};
bool wide_geometry(int dtype, size_t n, size_t k, WideGeometry &g);
hipError_t wide_pack(int dtype, void const *b, size_t n, size_t k, size_t b_stride, void *b_packed, hipStream_t stream);
/** `triangle`: only the outputs with col >= row + shift (the symmetric kinds). `metric`: 0 dot products, 1 angular,
 *  2 euclidean distances. */
hipError_t wide_product(int dtype, void const *a, void const *b_packed, void *c, size_t m, size_t n, size_t k,
                        size_t a_stride, size_t c_stride, hipStream_t stream, bool triangle, uint32_t shift, int metric);

/** A fresh non-zero number for the header of a newly packed image. */
uint64_t next_image_nonce();
/** Tile shape forced by nk_hip_set_tile_config for the calling thread (0: the heuristic picks). */
int forced_tile_config();
/** Compute units of the current device, asked once per process. */
int compute_unit_count();

} // namespace nk_gfx950

namespace {

using namespace nk_gfx950;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef long v2l __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// nk_dtype_t codes (reference: include/numkong/types.h:923-952)
enum : int {
    kI8 = 1 << 2,
    kU8 = 1 << 6,
    kF16 = 1 << 12,
    kBF16 = 1 << 13,
    kE4M3 = 1 << 14,
    kE5M2 = 1 << 15,
    kI4 = 1 << 16, // two 4-bit integers per byte, the even dimension in the low nibble
    kU4 = 1 << 17,
    kE2M3 = 1 << 18, // 6-bit floats, one per byte (bits 6 and 7 ignored)
    kE3M2 = 1 << 19,
    kU1 = 1 << 1, // eight 1-bit values per byte
    kF64 = 1 << 10, // the two wide types: f64 results, a vector kernel of their own (dots_gfx950_wide.hip)
    kF32 = 1 << 11,
};

constexpr uint32_t kMagic = 0x35394B4Eu; // "NK95"
constexpr uint32_t kVersion = 4;
constexpr int kChunkBytes = 16;   // bytes of K per lane per operand load
constexpr int kTileRows = 32;     // B rows per tile = MFMA N
constexpr int kStageChunks = 8;   // chunks of K per pipeline stage (128 bytes per row)
constexpr int kStageBytes = kStageChunks * kChunkBytes;
constexpr int kTileChunkBytes = kTileRows * kChunkBytes; // 512: one chunk of all 32 rows of a tile

struct PackedHeader {
    uint32_t magic;
    uint32_t version;
    uint32_t dtype;
    uint32_t elem_bytes; // bytes per element as stored in the image (2 for fp8, which is widened to f16)
    uint32_t n;        // logical rows of B = columns of C
    uint32_t k;        // logical depth in elements
    uint32_t n_tiles;  // ceil(n / 32)
    uint32_t k_chunks; // padded depth in 16-byte chunks, multiple of 8
    uint64_t nonce; // a number no other pack call of this process (and, in practice, of any) has used; 0: none
    uint64_t sums_offset; // u32 x (32 * n_tiles): 128 * sum(b') per column for u8, zeros otherwise
    uint64_t total_bytes;
    uint64_t norms_offset; // u32 or f32 x (32 * n_tiles): sum(b^2) per column (exact mod 2^32 for the integer types)
};
static_assert(sizeof(PackedHeader) == 64, "header must stay 64 bytes");

struct Geometry {
    uint32_t elem_bytes;   // bytes per element in the caller's A and B (1 for the 4-bit types, two to a byte)
    uint32_t packed_bytes; // bytes per element in the image and in LDS (fp8 is widened to f16; 0 for bits)
    uint32_t n, k, n_tiles, k_chunks;
    uint64_t k_src_bytes;  // bytes of one source row
    uint64_t data_bytes, sums_bytes, norms_bytes, total_bytes;
};

/** Bits per element in the caller's A and B (0: not a type of this backend). */
inline int elem_bits_of(int dtype) {
    switch (dtype) {
    case kU1: return 1;
    case kI4:
    case kU4: return 4;
    case kI8:
    case kU8:
    case kE4M3:
    case kE5M2:
    case kE2M3:
    case kE3M2: return 8;
    case kF16:
    case kBF16: return 16;
    default: return 0;
    }
}

/** The fp8 MFMA forms of gfx950 align the products inside one lane's k-group to the largest of them and
 *  keep only about 14 bits (1 + 2^-14 comes back as 1), far from the f32 accumulation of the reference's
 *  kernels (dot/serial.h:522-600). e4m3 and e5m2 are therefore widened, exactly, to f16 and run on the f16
 *  MFMA, whose products and sums are kept to full f32 precision: B at pack time, A on its way into LDS.
 *  e3m2 goes the same way (every e3m2 value is an f16 value). e2m3 values are multiples of 1/8 below 8 in magnitude:
 *  eight times each is an i8 value, and the i8 MFMA sums their products exactly at twice the f16 rate, as long as the
 *  i32 sums of 64 x the products cannot overflow (60 * 60 * k < 2^31); deeper rows take the f16 route like e3m2. The
 *  4-bit integers are widened to i8 as well. Single bits stay bits in the image (sixteen to a chunk) and become i8
 *  zeros and ones in registers, on both sides, right in front of the MFMA (their dot product is the popcount of the AND). */
constexpr uint64_t kE2M3IntegerDepth = 0x7FFFFFFFull / 3600; // deepest e2m3 row whose i32 sums are safe
inline bool e2m3_as_integers(size_t k) { return k <= kE2M3IntegerDepth; }

/** Bytes per element in the image and in LDS (0: sub-byte, the 1-bit type). */
inline int packed_bytes_of(int dtype, size_t k) {
    switch (dtype) {
    case kE4M3:
    case kE5M2:
    case kE3M2: return 2;
    case kE2M3: return e2m3_as_integers(k) ? 1 : 2; // (as i8 values, eight times the e2m3 value; or as f16)
    case kI4:
    case kU4: return 1;
    case kU1: return 0;
    default: return elem_bits_of(dtype) / 8;
    }
}
/** Source bytes of a row behind one chunk of the image (a chunk is what one lane feeds one MFMA: 16 bytes of operand). */
inline int source_chunk_of(int dtype, size_t k) {
    switch (dtype) {
    case kE4M3:
    case kE5M2:
    case kE3M2:
    case kI4:
    case kU4: return 8;
    case kE2M3: return e2m3_as_integers(k) ? 16 : 8;
    case kU1: return 2;
    default: return 16;
    }
}
/** Bytes a chunk takes in the image: the 16 operand bytes, except for the 1-bit type, which keeps its 16 bits. */
inline int image_chunk_of(int dtype) { return dtype == kU1 ? 2 : kChunkBytes; }

inline bool make_geometry(int dtype, size_t n, size_t k, Geometry &g) {
    int const bits = elem_bits_of(dtype);
    if (!bits) return false;
    if (n > 0x7FFFFFFFull || k > 0x3FFFFFFFull) return false;
    g.elem_bytes = (uint32_t)(bits + 7) / 8, g.packed_bytes = (uint32_t)packed_bytes_of(dtype, k), g.n = (uint32_t)n, g.k = (uint32_t)k;
    g.k_src_bytes = ((uint64_t)k * bits + 7) / 8; // (sub-byte types: whole bytes, as the reference loads them, cast/serial.h:519-538)
    uint64_t const source_chunk = (uint64_t)source_chunk_of(dtype, k);
    uint64_t const chunks = (g.k_src_bytes + source_chunk - 1) / source_chunk;
    g.k_chunks = (uint32_t)((chunks + 2 * kStageChunks - 1) / (2 * kStageChunks) * (2 * kStageChunks)); // an even number of stages
    g.n_tiles = (uint32_t)((n + kTileRows - 1) / kTileRows);
    g.data_bytes = (uint64_t)g.n_tiles * g.k_chunks * kTileRows * image_chunk_of(dtype);
    g.sums_bytes = (uint64_t)g.n_tiles * kTileRows * sizeof(uint32_t);
    g.norms_bytes = g.sums_bytes;
    g.total_bytes = sizeof(PackedHeader) + g.data_bytes + g.sums_bytes + g.norms_bytes;
    return true;
}


/**
 *  Load one 16-byte chunk of which only the first `valid` bytes exist (valid may be <= 0 or >= 16),
 *  with loads no wider than the pointer's known alignment `avec`. Missing bytes read as zero; `xr`
 *  (0 or 0x80808080) is applied to existing bytes only, so zero padding stays zero for u8.
 */
__device__ __forceinline__ v4i load_chunk_guarded(uint8_t const *p, int valid, int avec, uint32_t xr) {
    v4i out;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        int const rem = valid - 4 * w;
        uint32_t x = 0;
        if (rem >= 4 && avec >= 4) { x = *(uint32_t const *)(p + 4 * w) ^ xr; }
        else if (rem > 0) {
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (b < rem) x |= (uint32_t)(uint8_t)(p[4 * w + b] ^ (uint8_t)xr) << (8 * b);
        }
        out[w] = (int)x;
    }
    return out;
}

__device__ __forceinline__ uint32_t sum_bytes_u8(v4i v) {
    uint32_t s = __builtin_amdgcn_sad_u8((uint32_t)v[0], 0u, 0u);
    s = __builtin_amdgcn_sad_u8((uint32_t)v[1], 0u, s);
    s = __builtin_amdgcn_sad_u8((uint32_t)v[2], 0u, s);
    s = __builtin_amdgcn_sad_u8((uint32_t)v[3], 0u, s);
    return s;
}

#ifndef NK_E4M3_VIA_BF16
#define NK_E4M3_VIA_BF16 0
#endif
/** e4m3 widened to bf16 and run on the bf16 MFMA instead of f16 (every e4m3 value is a bf16 value as well). Off: on
 *  e4m3 values the two instructions sustain the same rate (MFMA-only loop 1859 against 1848 TFLOP/s) and the product
 *  at 8192^3 takes 0.900 against 0.911 ms, within what two runs differ by, so the image keeps the f16 form. */
constexpr bool kE4M3ViaBF16 = NK_E4M3_VIA_BF16 != 0;

/** Eight OCP fp8 values (two dwords) -> eight f16 values (e4m3 optionally bf16 values), exact for every code incl.
 *  subnormals, Inf, NaN. */
template <bool E5M2>
__device__ __forceinline__ v4i widen_fp8x8(uint32_t lo, uint32_t hi) {
    typedef _Float16 v2h __attribute__((ext_vector_type(2)));
    if constexpr (!E5M2 && kE4M3ViaBF16) {
        typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
        v2bf const q0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false), q1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
        v2bf const q2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false), q3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
        v4i wide;
        wide[0] = __builtin_bit_cast(int, q0), wide[1] = __builtin_bit_cast(int, q1);
        wide[2] = __builtin_bit_cast(int, q2), wide[3] = __builtin_bit_cast(int, q3);
        return wide;
    }
    v2h p0, p1, p2, p3;
    if (E5M2) {
        p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(lo, 1.0f, false);
        p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(lo, 1.0f, true);
        p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(hi, 1.0f, false);
        p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_bf8(hi, 1.0f, true);
    }
    else {
        p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false);
        p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true);
        p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false);
        p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true);
    }
    v4i out;
    out[0] = __builtin_bit_cast(int, p0), out[1] = __builtin_bit_cast(int, p1);
    out[2] = __builtin_bit_cast(int, p2), out[3] = __builtin_bit_cast(int, p3);
    return out;
}

/**
 *  Eight 6-bit floats, one per byte (two dwords) -> eight f16 values, exact. Both formats are IEEE-like with
 *  subnormals and no Inf/NaN (e2m3: 2 exponent bits, bias 1; e3m2: 3 exponent bits, bias 3; reference decoders:
 *  cast/serial.h:1318-1330, 1455-1470), so the exponent and mantissa bits, moved under an f16's sign bit, read as the
 *  value scaled by a power of two, subnormals included: one packed multiply by 2^14 (e2m3) or 2^12 (e3m2) finishes
 *  two values at a time. Bits 6 and 7 of a byte are ignored, as the reference does. In use for e3m2; e2m3 has the
 *  cheaper integer route of widen_e2m3x4.
 */
template <bool E3M2>
__device__ __forceinline__ v4i widen_fp6x8(uint32_t lo, uint32_t hi) {
    typedef _Float16 v2h __attribute__((ext_vector_type(2)));
    constexpr int kShift = E3M2 ? 8 : 7; // exponent field up to bit 10 of the f16
    v2h const scale = E3M2 ? v2h {(_Float16)4096.0f, (_Float16)4096.0f} : v2h {(_Float16)16384.0f, (_Float16)16384.0f};
    v4i out;
#pragma unroll
    for (int pair = 0; pair < 4; ++pair) {
        uint32_t const word = pair < 2 ? lo : hi;
        // bytes 2 * (pair % 2) and 2 * (pair % 2) + 1 of the word, each in a 16-bit lane of its own
        uint32_t const codes = __builtin_amdgcn_perm(0u, word, pair % 2 ? 0x0C030C02u : 0x0C010C00u);
        uint32_t const bits = ((codes << 10) & 0x80008000u) | ((codes & 0x001F001Fu) << kShift);
        v2h const value = __builtin_bit_cast(v2h, bits) * scale;
        out[pair] = __builtin_bit_cast(int, value);
    }
    return out;
}

/**
 *  Four e2m3 values, one per byte -> four i8 values, each EIGHT TIMES the e2m3 value: with 2 exponent bits (bias 1) and
 *  3 mantissa bits every e2m3 value is a multiple of 1/8 of magnitude at most 7.5, so 8 x is an integer in [-60, 60]
 *  (reference decoder: cast/serial.h:1318-1330). Products of two such integers summed in i32 are exact, 64 times the
 *  dot product, and the i8 MFMA runs at twice the rate of the f16 one. All four bytes at once: with x = the low five
 *  bits (e, m), the magnitude is x for e <= 1 (m, or 8 + m), x + (x & 15) for e = 2 (16 + 2 m) and
 *  x + (x & 15) + 2 (x & 7) for e = 3 (32 + 4 m); no byte ever carries into its neighbour. The three per-byte masks
 *  (the two above and 0xFF for a set sign bit) come from 8-entry byte tables indexed by bits 3..5 of each byte, one
 *  v_perm_b32 each. Negative values by 0x80 - magnitude, flipped back. Bits 6 and 7 of a byte are ignored, as the
 *  reference does.
 */
__device__ __forceinline__ uint32_t widen_e2m3x4(uint32_t codes) {
    uint32_t const index = (codes >> 3) & 0x07070707u; // e + 4 * sign, per byte
    uint32_t const negate = __builtin_amdgcn_perm(0xFFFFFFFFu, 0x00000000u, index);  // 0xFF where the sign bit is set
    uint32_t const from_two = __builtin_amdgcn_perm(0x0F0F0000u, 0x0F0F0000u, index); // 0x0F where e >= 2
    uint32_t const at_three = __builtin_amdgcn_perm(0x07000000u, 0x07000000u, index); // 0x07 where e == 3
    uint32_t const low = codes & 0x1F1F1F1Fu;
    uint32_t const magnitude = low + (low & from_two) + ((low & at_three) << 1);
    uint32_t const negative = (0x80808080u - magnitude) ^ 0x80808080u;
    return (negative & negate) | (magnitude & ~negate);
}

/** Sixteen 4-bit integers (two dwords; the even dimension in the low nibble) -> sixteen i8 values: the low nibbles
 *  of a dword's four bytes, then its high nibbles (any order serves as long as A and B use the same one).
 *  Signed: a nibble n with bit 3 set becomes n | 0xF0, the byte-wise (n ^ 8) - 8 of dot/serial.h:781-785. */
template <bool SIGNED>
__device__ __forceinline__ v4i widen_i4x16(uint32_t lo, uint32_t hi) {
    auto extend = [](uint32_t nibbles) {
        if (!SIGNED) return nibbles;
        uint32_t const top = nibbles & 0x08080808u;
        return nibbles | ((top << 5) - (top << 1)); // 0xF0 where bit 3 is set (the last byte's carry leaves the word)
    };
    v4i out;
    out[0] = (int)extend(lo & 0x0F0F0F0Fu), out[1] = (int)extend((lo >> 4) & 0x0F0F0F0Fu);
    out[2] = (int)extend(hi & 0x0F0F0F0Fu), out[3] = (int)extend((hi >> 4) & 0x0F0F0F0Fu);
    return out;
}

/** Sixteen bits (the low half of `bits`, the first dimension in bit 0) -> sixteen i8 values 0 or 1. Four bits times
 *  0x00204081 land in bit 0 of four different bytes. */
__device__ __forceinline__ v4i widen_u1x16(uint32_t bits) {
    v4i out;
#pragma unroll
    for (int w = 0; w < 4; ++w) out[w] = (int)((((bits >> (4 * w)) & 0xFu) * 0x00204081u) & 0x01010101u);
    return out;
}

/** Widening of the source bytes behind one 16-byte chunk, by kind: 1 e4m3, 2 e5m2, 4 e3m2, 8 e2m3 of deep rows (8
 *  bytes to f16); 5 i4, 6 u4 (8 bytes to i8); 7 u1 (2 bytes to i8). Kind 3, e2m3 of rows that are not too deep, turns 16
 *  bytes into 16 i8 values in place (widen_e2m3x4) and does not come through here. */
template <int WIDEN>
__device__ __forceinline__ v4i widen_chunk(uint32_t lo, uint32_t hi) {
    if constexpr (WIDEN == 1) return widen_fp8x8<false>(lo, hi);
    else if constexpr (WIDEN == 2) return widen_fp8x8<true>(lo, hi);
    else if constexpr (WIDEN == 4) return widen_fp6x8<true>(lo, hi);
    else if constexpr (WIDEN == 8) return widen_fp6x8<false>(lo, hi);
    else if constexpr (WIDEN == 5) return widen_i4x16<true>(lo, hi);
    else if constexpr (WIDEN == 6) return widen_i4x16<false>(lo, hi);
    else return widen_u1x16(lo);
}
inline int widen_kind_of(int dtype, size_t k) {
    switch (dtype) {
    case kE4M3: return 1;
    case kE5M2: return 2;
    case kE2M3: return e2m3_as_integers(k) ? 3 : 8;
    case kE3M2: return 4;
    case kI4: return 5;
    case kU4: return 6;
    case kU1: return 7;
    default: return 0;
    }
}

#pragma region Packing

/** Sum of the squares of the 8 values of a 16-byte chunk of bf16 (f32 = bits << 16) or f16, in f64. */
template <bool BF16_VALUES>
__device__ __forceinline__ double chunk_sumsq_f64(v4i v) {
    double sum = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        float lo, hi;
        if (BF16_VALUES) {
            lo = __builtin_bit_cast(float, (uint32_t)v[w] << 16), hi = __builtin_bit_cast(float, (uint32_t)v[w] & 0xFFFF0000u);
        }
        else {
            typedef _Float16 v2h __attribute__((ext_vector_type(2)));
            int const word = v[w]; // a named copy: bit-casting the vector element expression itself reads element 0
            v2h const pair = __builtin_bit_cast(v2h, word);
            lo = (float)pair[0], hi = (float)pair[1];
        }
        sum = __builtin_fma((double)lo, (double)lo, sum);
        sum = __builtin_fma((double)hi, (double)hi, sum);
    }
    return sum;
}

/**
 *  Packing, one pass: a workgroup of 1024 threads takes one 32-row tile through the whole depth, 32 chunks of every
 *  row per step (thread t: row (t / 8) % 32, chunk 8 * (t / 256) + t % 8 of the step, so 8 neighbouring threads read
 *  128 (64, 16) contiguous source bytes of a row and 8 neighbouring rows write a 128-byte run of the image), and keeps
 *  the per-column terms of what it writes in registers on the way: the u8 compensation term (128 * the sum of the
 *  signed packed bytes of the row, mod 2^32; zero for the other types) and the column's sum of squares, which the
 *  angular and euclidean kinds need (reference: the norms behind the packed rows, dots/serial.h:326-332): exact mod
 *  2^32 for the integer types, accumulated in f64 and rounded once to f32 for the float types. A thread always works
 *  on the same row and on the chunks of one residue mod 32; the 32 partial sums of a row are added in ascending
 *  order of that residue, so the terms do not depend on anything but the row.
 *  WIDEN: 0 copies the elements, 3 rewrites e2m3 bytes as i8 values in place, 7 copies the 16 bits of a chunk of the
 *  1-bit type as they are, otherwise the kind of widen_chunk (8 source bytes per chunk).
 *  KIND, by what the image holds: 0 signed bytes (i8, the widened 4-bit types, e2m3 as 8 x its values), 1 u8 stored
 *  with its offset, 2 bf16, 3 f16 (and what is widened to it), 4 bits (no terms: zeros).
 *  `terms` == 0: the tiles only (callers that will never read the terms).
 */
constexpr int kPackThreads = 1024;
constexpr int kPackChunks = kPackThreads / kTileRows; // chunks of every row per step of a workgroup
template <int WIDEN, int KIND>
__global__ __launch_bounds__(kPackThreads) void pack_kernel(uint8_t const *__restrict__ b, uint64_t b_stride, uint32_t n,
                                                            uint64_t k_src_bytes, uint32_t k_chunks, uint32_t k,
                                                            uint8_t *__restrict__ data, uint32_t *__restrict__ sums,
                                                            uint32_t *__restrict__ norms, int avec, uint32_t xr, int terms,
                                                            PackedHeader header) {
    constexpr int kSrcChunk = WIDEN == 0 || WIDEN == 3 ? 16 : (WIDEN == 7 ? 2 : 8);
    constexpr int kImageChunk = WIDEN == 7 ? 2 : kChunkBytes;
    __shared__ int part_sum[kPackChunks][kTileRows];
    __shared__ uint32_t part_squares[kPackChunks][kTileRows];
    __shared__ double part_f64[kPackChunks][kTileRows];
    if (blockIdx.x == 0 && threadIdx.x == 0) *(PackedHeader *)(data - sizeof(PackedHeader)) = header; // (64 bytes in front of the tiles)
    uint32_t const tile = blockIdx.x;
    uint32_t const r = (threadIdx.x >> 3) & 31;
    uint32_t const part = ((threadIdx.x >> 8) << 3) | (threadIdx.x & 7); // chunk of the step = residue of the chunk mod 32
    uint64_t const row = (uint64_t)tile * kTileRows + r;
    uint8_t const *source = b + row * b_stride;
    uint8_t *target = data + ((uint64_t)tile * k_chunks * kTileRows + r) * kImageChunk;
    int sum = 0;
    uint32_t squares = 0;
    double squares_f64 = 0;
    auto take = [&](uint32_t c) {
        int64_t const left = (int64_t)k_src_bytes - (int64_t)c * kSrcChunk;
        int const valid = row < n ? (int)(left > kSrcChunk ? kSrcChunk : (left < 0 ? 0 : left)) : 0;
        v4i v = {0, 0, 0, 0};
        if (valid > 0) {
            uint8_t const *src = source + (uint64_t)c * kSrcChunk;
            if ((WIDEN == 0 || WIDEN == 3) && valid == 16 && avec >= 16) {
                v = __builtin_nontemporal_load((v4i const *)src); // (read once)
                v[0] ^= (int)xr, v[1] ^= (int)xr, v[2] ^= (int)xr, v[3] ^= (int)xr;
            }
            else { v = load_chunk_guarded(src, valid, avec, xr); }
            if constexpr (WIDEN == 3) {
#pragma unroll
                for (int w = 0; w < 4; ++w) v[w] = (int)widen_e2m3x4((uint32_t)v[w]);
            }
            else if constexpr (WIDEN != 0 && WIDEN != 7) v = widen_chunk<WIDEN>((uint32_t)v[0], (uint32_t)v[1]);
        }
        uint8_t *at = target + (uint64_t)c * (kTileRows * kImageChunk);
        if constexpr (WIDEN == 7) *(uint16_t *)at = (uint16_t)v[0];
        else *(v4i *)at = v;
        if (KIND == 0) {
#pragma unroll
            for (int w = 0; w < 4; ++w) squares = (uint32_t)__builtin_amdgcn_sdot4(v[w], v[w], (int)squares, false);
        }
        else if (KIND == 1) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                sum = __builtin_amdgcn_sdot4(v[w], 0x01010101, sum, false);
                squares = (uint32_t)__builtin_amdgcn_sdot4(v[w], v[w], (int)squares, false);
            }
        }
        else if (KIND == 2 || KIND == 3) { squares_f64 += chunk_sumsq_f64<KIND == 2>(v); }
    };
#pragma unroll 4
    for (uint32_t c = part; c < k_chunks; c += kPackChunks) take(c);
    if (!terms) return;
    part_sum[part][r] = sum, part_squares[part][r] = squares, part_f64[part][r] = squares_f64;
    __syncthreads();
    if (threadIdx.x < kTileRows) {
        uint32_t const mine = threadIdx.x;
        sum = 0, squares = 0, squares_f64 = 0;
#pragma unroll
        for (int p = 0; p < kPackChunks; ++p) sum += part_sum[p][mine], squares += part_squares[p][mine], squares_f64 += part_f64[p][mine];
        // u8 is stored as b - 128 (and its padding as 0): sum(b^2) = sum((b - 128)^2) + 256 * sum(b - 128) + 128^2 * k
        if (KIND == 1) squares += 256u * (uint32_t)sum + 16384u * k;
        sums[(uint64_t)tile * kTileRows + mine] = (uint32_t)sum * 128u;
        norms[(uint64_t)tile * kTileRows + mine] = KIND < 2 ? squares : (KIND == 4 ? 0u : __builtin_bit_cast(uint32_t, (float)squares_f64));
    }
}

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t *p, uint64_t count, uint32_t value) {
    uint64_t const i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) p[i] = value;
}

__global__ __launch_bounds__(64) void write_header_kernel(PackedHeader *dst, PackedHeader h) {
    if (threadIdx.x == 0) *dst = h;
}

/** `tri_mask` all ones: only the elements with col >= row + tri_shift (on or right of a diagonal); 0: all of them. */
__global__ __launch_bounds__(256) void fill_rows_kernel(uint8_t *c, uint32_t m, uint32_t n, uint64_t c_stride,
                                                        uint32_t value, uint32_t tri_shift, uint32_t tri_mask) {
    uint64_t const i = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    uint64_t const row = i / n, col = i % n;
    if (row < m && (((uint32_t)row + tri_shift) & tri_mask) <= (uint32_t)col) *(uint32_t *)(c + row * c_stride + col * 4) = value;
}

#pragma endregion Packing

#pragma region Element types

/**
 *  Float accumulation. One MFMA accumulator rounds once per 8 products at the magnitude of the whole running
 *  sum; over a depth of thousands that is 1.4x the error of the reference's scalar kernel for bf16 (4 lanes,
 *  dot/serial.h:406-439), 3x that of its 16-lane AVX-512 kernels (dot/genoa.h:237-256), and 4x the scalar
 *  kernel's for fp8, whose products and short sums are exact in f32 (dot/serial.h:522-600). The float types
 *  therefore fold the accumulator into a second one every `chunk_stages` stages (about an eighth of the depth,
 *  at most 16 stages = 1024 values): the running sums stay short, and the error drops to that of the reference's
 *  best kernels (measured ratios next to the tests). Two accumulator sets do not fit the 256 x 256 tile, so
 *  these types stop at 128 x 256. NK_HALF_SINGLE_ACCUMULATOR builds bf16/f16 without the second set (faster,
 *  less accurate; for comparison only).
 */
#ifdef NK_HALF_SINGLE_ACCUMULATOR
constexpr bool kHalfChunked = false;
#else
constexpr bool kHalfChunked = true;
#endif

struct I8 {
    static constexpr bool kChunked = false; // fold the accumulator into a second one every few stages
    static constexpr int kSrcChunk = 16; // source bytes of A behind one 16-byte LDS chunk
    static constexpr int kImageChunk = kChunkBytes; // bytes of one row's chunk in the image
    static constexpr bool kEightfold = false; // the MFMA sees eight times the values (e2m3 as integers)
    /** What a lane loaded from the image -> its MFMA operand. */
    static __device__ __forceinline__ v4i operand_b(v4i loaded) { return loaded; }
    static __device__ __forceinline__ v4i widen(v4i v) { return v; }
    typedef v16i acc_t;
    typedef uint32_t norm_t; // what a row's sum of squares accumulates in
    static constexpr int kDtype = kI8;
    static constexpr bool kUnsigned = false;
    static constexpr bool kDistances = true; // the distance kinds are built for this type (NORMS kernels)
    static constexpr bool kPrewiden = false; // widen A in place, ahead of its LDS write, spread over two k-steps
    /** Sum of the squares of the source values behind one staged chunk (`raw`: as loaded, `wide`: as it goes to LDS). */
    static __device__ __forceinline__ norm_t sumsq(v4i raw, v4i) {
        int sum = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum = __builtin_amdgcn_sdot4(raw[w], raw[w], sum, false);
        return (uint32_t)sum;
    }
    static __device__ __forceinline__ void mma(acc_t &acc, v4i a, v4i b) {
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
    }
    /** The same with nothing to add to: the first product of a sum (the zero is an operand of the instruction). */
    static __device__ __forceinline__ void mma_fresh(acc_t &acc, v4i a, v4i b) {
        acc_t const zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, zero, 0, 0, 0);
    }
};
struct U8 : I8 {
    static constexpr int kDtype = kU8;
    static constexpr bool kUnsigned = true;
    static __device__ __forceinline__ norm_t sumsq(v4i raw, v4i) {
        uint32_t sum = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) sum = __builtin_amdgcn_udot4((uint32_t)raw[w], (uint32_t)raw[w], sum, false);
        return sum;
    }
};
struct BF16 {
    static constexpr bool kChunked = kHalfChunked;
    static constexpr int kSrcChunk = 16; // source bytes of A behind one 16-byte LDS chunk
    static constexpr int kImageChunk = kChunkBytes;
    static constexpr bool kEightfold = false;
    static __device__ __forceinline__ v4i operand_b(v4i loaded) { return loaded; }
    static __device__ __forceinline__ v4i widen(v4i v) { return v; }
    typedef v16f acc_t;
    typedef double norm_t;
    static constexpr int kDtype = kBF16;
    static constexpr bool kUnsigned = false;
    static constexpr bool kDistances = true;
    static constexpr bool kPrewiden = false;
    /** The 8 products are exact in f32; their short sum is rounded a few times, the long sum runs in f64. The short
     *  sum is four `v_dot2_f32_bf16` (two products and the addend each; measured on the part for squares and a
     *  positive addend: within one unit in the last place of the exact sum in 99.3 % of a million cases, 1.43 at
     *  worst), a quarter of the instructions of unpacking to f32 and eight fused multiply-adds. */
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) {
        typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
        float sum = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            int const word = wide[w]; // a named copy: bit-casting the vector element expression itself reads element 0
            v2bf const pair = __builtin_bit_cast(v2bf, word);
            sum = __builtin_amdgcn_fdot2_f32_bf16(pair, pair, sum, false);
        }
        return (double)sum;
    }
    static __device__ __forceinline__ void mma(acc_t &acc, v4i a, v4i b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), acc, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ void mma_fresh(acc_t &acc, v4i a, v4i b) {
        acc_t const zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), zero, 0,
                                                      0, 0);
    }
};
struct F16 {
    static constexpr bool kChunked = kHalfChunked;
    static constexpr int kSrcChunk = 16; // source bytes of A behind one 16-byte LDS chunk
    static constexpr int kImageChunk = kChunkBytes;
    static constexpr bool kEightfold = false;
    static __device__ __forceinline__ v4i operand_b(v4i loaded) { return loaded; }
    static __device__ __forceinline__ v4i widen(v4i v) { return v; }
    typedef v16f acc_t;
    typedef double norm_t;
    static constexpr int kDtype = kF16;
    static constexpr bool kUnsigned = false;
    static constexpr bool kDistances = true;
    static constexpr bool kPrewiden = false;
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { // also e4m3 / e5m2, which are f16 by then
        typedef _Float16 v2h __attribute__((ext_vector_type(2)));
        float sum = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) { // (mixed-precision fused multiply-adds: `v_dot2_f32_f16` is up to 511 units off for f16 denormals, which e5m2's are)
            int const word = wide[w]; // a named copy: bit-casting the vector element expression itself reads element 0
            v2h const pair = __builtin_bit_cast(v2h, word);
            float const lo = (float)pair[0], hi = (float)pair[1];
            sum = __builtin_fmaf(lo, lo, sum), sum = __builtin_fmaf(hi, hi, sum);
        }
        return (double)sum;
    }
    /** The same short sum with four `v_dot2_f32_f16`, for types whose values are never f16 denormals (measured on
     *  the part for squares of normal numbers and a positive addend: as the bf16 form, 1.44 units at worst). */
    static __device__ __forceinline__ norm_t sumsq_of_normals(v4i wide) {
        typedef _Float16 v2h __attribute__((ext_vector_type(2)));
        float sum = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            int const word = wide[w]; // a named copy: bit-casting the vector element expression itself reads element 0
            v2h const pair = __builtin_bit_cast(v2h, word);
            sum = __builtin_amdgcn_fdot2(pair, pair, sum, false);
        }
        return (double)sum;
    }
    static __device__ __forceinline__ void mma(acc_t &acc, v4i a, v4i b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), acc, 0, 0,
                                                     0);
    }
    static __device__ __forceinline__ void mma_fresh(acc_t &acc, v4i a, v4i b) {
        acc_t const zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), zero, 0, 0,
                                                     0);
    }
};
/** fp8 runs widened to f16 (exact), on the f16 MFMA; see widen_fp8x8. */
struct E4M3 : std::conditional<kE4M3ViaBF16, BF16, F16>::type {
    typedef std::conditional<kE4M3ViaBF16, BF16, F16>::type base_t;
    static constexpr bool kChunked = true;
    static constexpr int kDtype = kE4M3;
    static constexpr int kSrcChunk = 8;
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_fp8x8<false>((uint32_t)v[0], (uint32_t)v[1]); }
    static __device__ __forceinline__ base_t::norm_t sumsq(v4i raw, v4i wide) {
        if constexpr (kE4M3ViaBF16) return BF16::sumsq(raw, wide);
        else return F16::sumsq_of_normals(wide); // smallest value 2^-9: no f16 denormals
    }
};
struct E5M2 : F16 {
    static constexpr bool kChunked = true;
    static constexpr int kDtype = kE5M2;
    static constexpr int kSrcChunk = 8;
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_fp8x8<true>((uint32_t)v[0], (uint32_t)v[1]); }
};
/** e2m3 runs as i8 values eight times as large on the i8 MFMA (see widen_e2m3x4): sums are exact integers, 64 times
 *  the dot product, converted to f32 once in the epilogue (one rounding for sums beyond 2^24, none below). */
struct E2M3 : I8 {
    static constexpr int kDtype = kE2M3;
    static constexpr bool kEightfold = true;
    static constexpr bool kPrewiden = true; // 13 operations per dword: too many to sit in front of the LDS writes
    static __device__ __forceinline__ v4i widen(v4i v) {
        v4i out;
#pragma unroll
        for (int w = 0; w < 4; ++w) out[w] = (int)widen_e2m3x4((uint32_t)v[w]);
        return out;
    }
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { return I8::sumsq(wide, wide); } // 64 x the sum of squares
};
/** e2m3 rows too deep for exact i32 sums (see kE2M3IntegerDepth) run widened to f16 like e3m2: every e2m3 value is an
 *  f16 value, the smallest non-zero one 1/8. */
struct E2M3Deep : F16 {
    static constexpr bool kChunked = true;
    static constexpr int kDtype = kE2M3;
    static constexpr int kSrcChunk = 8;
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_fp6x8<false>((uint32_t)v[0], (uint32_t)v[1]); }
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { return sumsq_of_normals(wide); }
};
/** e3m2 runs widened to f16 (its values times 16 do not fit i8); see widen_fp6x8. */
struct E3M2 : F16 {
    static constexpr bool kChunked = true;
    static constexpr int kDtype = kE3M2;
    static constexpr int kSrcChunk = 8;
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_fp6x8<true>((uint32_t)v[0], (uint32_t)v[1]); }
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { return sumsq_of_normals(wide); } // smallest value 2^-4
};
/** The 4-bit integers run widened to i8 on the i8 MFMA; see widen_i4x16. Unsigned nibbles are non-negative i8 values
 *  as they are: none of u8's offset arithmetic. */
struct I4 : I8 {
    static constexpr int kDtype = kI4;
    static constexpr int kSrcChunk = 8;
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_i4x16<true>((uint32_t)v[0], (uint32_t)v[1]); }
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { return I8::sumsq(wide, wide); }
};
/** Single bits run as i8 values 0 and 1: sixteen of them behind two source bytes, of A on its way into LDS and of B,
 *  whose image keeps the bits, in registers between the load and the MFMA. */
struct U1 : I8 {
    static constexpr int kDtype = kU1;
    static constexpr bool kDistances = false; // dot products only
    static constexpr int kSrcChunk = 2;
    static constexpr int kImageChunk = 2;
    static __device__ __forceinline__ v4i operand_b(v4i loaded) { return widen_u1x16((uint32_t)loaded[0]); }
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_u1x16((uint32_t)v[0]); }
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { return I8::sumsq(wide, wide); }
};
struct U4 : I8 {
    static constexpr int kDtype = kU4;
    static constexpr int kSrcChunk = 8;
    static __device__ __forceinline__ v4i widen(v4i v) { return widen_i4x16<false>((uint32_t)v[0], (uint32_t)v[1]); }
    static __device__ __forceinline__ norm_t sumsq(v4i, v4i wide) { return I8::sumsq(wide, wide); }
};

/**
 *  Distances from a dot product and two sums of squares, as the reference's scalar finalisers compute them
 *  (spatial/serial.h:257-344): integer inputs are converted to f32 first (the i8 kernels read both norms as
 *  signed 32-bit integers, the u8 kernels as unsigned); angular = max(1 - dot * rsqrt(qn * tn), 0), and 0 or
 *  1 when the product of the norms is not positive; euclidean = sqrt(max(qn + tn - 2 * dot, 0)).
 */
template <class T>
__device__ __forceinline__ float norm_as_f32(uint32_t bits) {
    if (T::kDtype == kI8 || T::kDtype == kI4) return (float)(int)bits;
    if (T::kDtype == kU8 || T::kDtype == kU4) return (float)bits;
    if (T::kEightfold) return (float)bits * 0.015625f; // integer sums of squares of 8 x the values
    return __builtin_bit_cast(float, bits);
}

/** What the accumulators hold -> what the caller gets, as 32-bit patterns: as they are, except that e2m3 sums are
 *  integers, 64 times the f32 result. */
template <class T>
__device__ __forceinline__ uint32_t finished_dot(uint32_t bits) {
    if (T::kEightfold) return __builtin_bit_cast(uint32_t, (float)(int)bits * 0.015625f);
    return bits;
}

/** METRIC: 1 angular, 2 euclidean. `query` and `target` are the row's and the column's sums of squares as f32
 *  (converted once per row and once per column of a tile). The reciprocal square root is the hardware's estimate
 *  (1 ulp) refined by one Newton step with fused residuals: identical rows must cancel to within a rounding or
 *  two, as the reference's three Newton steps do (splitting it into a factor per row and a factor per column
 *  would save half of the operations and lose exactly that). */
template <class T, int METRIC>
__device__ __forceinline__ uint32_t distance_from_dot(uint32_t dot_bits, float query, float target) {
    float const dot = T::kDtype == kI8 || T::kDtype == kI4
                          ? (float)(int)dot_bits
                          : (T::kDtype == kU8 || T::kDtype == kU4 ? (float)dot_bits : __builtin_bit_cast(float, dot_bits));
    float result;
    if (METRIC == 1) {
        float const product = query * target;
        float root = __builtin_amdgcn_rsqf(product);
        float const residual = __builtin_fmaf(-(product * root), root, 1.0f);
        root = __builtin_fmaf(root * 0.5f, residual, root);
        float unclipped = __builtin_fmaxf(__builtin_fmaf(-dot, root, 1.0f), 0.0f);
        // Where the dot product squared is the product of the norms exactly (one non-zero term, values of a few bits),
        // a division by a correctly rounded square root gives a cosine of exactly 1 or -1, and so does this.
        if (__builtin_fmaf(dot, dot, -product) == 0.0f) unclipped = dot > 0 ? 0.0f : 2.0f;
        result = product > 0 ? unclipped : (dot == 0 ? 0.0f : 1.0f);
    }
    else {
        // The hardware's reciprocal square root is good to about one unit in the last place; one Newton step on
        // the root itself (residual by a fused multiply-add) leaves it correctly rounded but for rare ties, as
        // the square roots of the reference's vector kernels are.
        float const squared = __builtin_fmaf(-2.0f, dot, query + target);
        float const inverse = __builtin_amdgcn_rsqf(squared);
        float root = squared * inverse;
        root = __builtin_fmaf(__builtin_fmaf(-root, root, squared), 0.5f * inverse, root);
        result = squared > 0 ? root : 0.0f;
    }
    return __builtin_bit_cast(uint32_t, result);
}

/** The hardware's reciprocal square root (good to about a unit in the last place) refined by one Newton step with a
 *  fused residual. Zero gives NaN (infinity times zero), which is what angular_from_factors wants of it. */
__device__ __forceinline__ float refined_rsqrt(float x) {
    float const root = __builtin_amdgcn_rsqf(x);
    float const residual = __builtin_fmaf(-(x * root), root, 1.0f);
    return __builtin_fmaf(root * 0.5f, residual, root);
}

/**
 *  The angular distance where it is cheap: 1 - dot * (rq * rt), with rq and rt the refined reciprocal square roots of
 *  the row's and the column's sums of squares, taken once per row and once per column of a tile instead of once per
 *  output. Three roundings of relative size 2^-24 enter the cosine instead of the one and a half of the full
 *  finaliser, so the form is only used where the cosine is at most a quarter in magnitude (`*cheap`): its error is
 *  then under a unit of 2^-24, below the rounding of the result itself (1 - cos lies in [0.75, 1.25] there). Zero or
 *  overflowed sums of squares make the factors NaN or infinite and fail the test. Everything else, identical rows
 *  above all, takes distance_from_dot.
 */
template <class T>
__device__ __forceinline__ float angular_from_factors(uint32_t dot_bits, float row_factor, float column_factor, bool *cheap) {
    float const dot = T::kDtype == kI8 || T::kDtype == kI4
                          ? (float)(int)dot_bits
                          : (T::kDtype == kU8 || T::kDtype == kU4 ? (float)dot_bits : __builtin_bit_cast(float, dot_bits));
    float const scale = row_factor * column_factor;
    *cheap = __builtin_fabsf(dot * scale) <= 0.25f; // (false for NaN)
    return __builtin_fmaf(-dot, scale, 1.0f);
}

#pragma endregion Element types

#pragma region Packed product

template <int V>
struct slot_c {
    static constexpr int value = V;
};

/** Second-level accumulators: real for the chunked types, empty (no registers) for the others. */
template <class acc_t, int TM, int TN, bool kChunked>
struct Totals {
    acc_t value[TM][TN];
    __device__ __forceinline__ void clear() {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) value[i][j][v] = 0;
    }
    __device__ __forceinline__ void fold(acc_t (&acc)[TM][TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                value[i][j] += acc[i][j];
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
            }
    }
    __device__ __forceinline__ void clear_block(int i, int j) {
#pragma unroll
        for (int v = 0; v < 16; ++v) value[i][j][v] = 0;
    }
    __device__ __forceinline__ auto finish(acc_t const (&acc)[TM][TN], int i, int j, int v) const {
        return acc[i][j][v] + value[i][j][v];
    }
};
template <class acc_t, int TM, int TN>
struct Totals<acc_t, TM, TN, false> {
    __device__ __forceinline__ void clear() {}
    __device__ __forceinline__ void fold(acc_t (&)[TM][TN]) {}
    __device__ __forceinline__ void clear_block(int, int) {}
    __device__ __forceinline__ auto finish(acc_t const (&acc)[TM][TN], int i, int j, int v) const { return acc[i][j][v]; }
};


/**
 *  Workgroup index -> output tile. Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each
 *  with a private L2, so ids are first regrouped into 8 contiguous ranges (one per XCD) and each range
 *  walks the tile grid in column-major bands of 8 tile rows: tiles resident on one XCD at the same time
 *  share A row blocks and B column tiles in that XCD's L2.
 */
__device__ __forceinline__ void tile_of_block(uint32_t pid, GemmArgs const &g, uint32_t &tm, uint32_t &tn) {
    uint32_t const tiles_m = g.tiles_m, tiles_n = g.tiles_n;
    uint32_t const total = g.tile_count;
    uint32_t const per_xcd = total / 8;
    uint32_t lid = pid;
    if (pid < per_xcd * 8) lid = (pid % 8) * per_xcd + pid / 8;
    if (g.tile_list) { // a triangular grid: the same walk with the tiles left of the diagonal left out, listed
        typedef __attribute__((address_space(4))) uint32_t const constant_u32_t;
        constant_u32_t *entry = (constant_u32_t *)g.tile_list + 2 * (uint64_t)lid;
        tm = entry[0], tn = entry[1];
        return;
    }
    constexpr uint32_t kBand = kTileBand;
    uint32_t const width = kBand * tiles_n;
    uint32_t const band = lid / width;
    uint32_t const first = band * kBand;
    uint32_t const rows = tiles_m - first < kBand ? tiles_m - first : kBand;
    uint32_t const in_band = lid % width;
    tm = first + in_band % rows;
    tn = in_band / rows;
}

/** First tile column of tile row `t` that holds an element on or right of the diagonal col = row + shift; tiles
 *  are 2^bm_log2 rows by 2^bn_log2 columns. */
__host__ __device__ inline uint32_t first_live_tile(uint32_t t, uint32_t bm_log2, uint32_t bn_log2, uint32_t shift) {
    return ((t << bm_log2) + shift) >> bn_log2;
}

/**
 *  The tile list of a triangular grid, in the order of `tile_of_block`: bands of kTileBand tile rows, column
 *  by column within a band, top to bottom within a column, and only tiles with something on or right of the
 *  diagonal. One workgroup per list: the bands' sizes are scanned 256 at a time, then every band is filled by all
 *  threads, a column each. A band's first columns form a staircase (row t joins at column first_live_tile(t)); the cells
 *  left of column c number the sum over its rows of max(0, c - first_live_tile(t)).
 */
struct TriangleGrid {
    uint32_t tiles_m, tiles_n, bm_log2, bn_log2, shift;
    uint32_t *band_start, *list;
};
struct TriangleGrids {
    TriangleGrid grid[2];
};
__global__ __launch_bounds__(256) void triangle_tiles_kernel(TriangleGrids grids) {
    TriangleGrid const &mine = grids.grid[blockIdx.x]; // one workgroup per list
    uint32_t const tiles_m = mine.tiles_m, tiles_n = mine.tiles_n, bm_log2 = mine.bm_log2, bn_log2 = mine.bn_log2,
                   shift = mine.shift;
    uint32_t *band_start = mine.band_start, *list = mine.list;
    __shared__ uint32_t scan[256];
    __shared__ uint32_t base;
    uint32_t const tid = threadIdx.x;
    uint32_t const bands = (tiles_m + kTileBand - 1) / kTileBand;
    if (tid == 0) base = 0, band_start[0] = 0;
    __syncthreads();
    for (uint32_t chunk = 0; chunk < bands; chunk += 256) {
        uint32_t const band = chunk + tid;
        uint32_t count = 0;
        if (band < bands) {
            uint32_t const first = band * kTileBand, last = first + kTileBand < tiles_m ? first + kTileBand : tiles_m;
            for (uint32_t t = first; t < last; ++t) {
                uint32_t const from = first_live_tile(t, bm_log2, bn_log2, shift);
                count += from < tiles_n ? tiles_n - from : 0;
            }
        }
        scan[tid] = count;
        __syncthreads();
        for (uint32_t step = 1; step < 256; step *= 2) {
            uint32_t const below = tid >= step ? scan[tid - step] : 0;
            __syncthreads();
            scan[tid] += below;
            __syncthreads();
        }
        if (band < bands) band_start[band + 1] = base + scan[tid];
        __syncthreads();
        if (tid == 255) base += scan[255];
        __syncthreads();
    }
    for (uint32_t band = 0; band < bands; ++band) {
        uint32_t const first = band * kTileBand, last = first + kTileBand < tiles_m ? first + kTileBand : tiles_m;
        uint32_t joins[kTileBand]; // where each row of the band joins (past the grid for rows that do not exist)
#pragma unroll
        for (uint32_t i = 0; i < kTileBand; ++i) joins[i] = first + i < last ? first_live_tile(first + i, bm_log2, bn_log2, shift) : 0xFFFFFFFFu;
        uint32_t const start = band_start[band];
        for (uint32_t column = joins[0] + tid; column < tiles_n; column += 256) {
            uint32_t at = start;
#pragma unroll
            for (uint32_t i = 0; i < kTileBand; ++i) at += column > joins[i] ? column - joins[i] : 0;
#pragma unroll
            for (uint32_t i = 0; i < kTileBand; ++i)
                if (joins[i] <= column) list[2 * (uint64_t)at] = first + i, list[2 * (uint64_t)at + 1] = column, ++at;
        }
    }
}

/**
 *  A persistent workgroup of 4 wavefronts (one per SIMD) walks over (32*TM) x (128*TN) tiles of C. Every
 *  wavefront owns all 32*TM rows of the tile and its own 32*TN columns: B fragments are loaded by exactly
 *  one wavefront, straight from the packed image into registers; the shared A block goes through LDS.
 *  Being persistent lets the stores of one tile drain while the next tile is already being computed.
 *
 *  A stage is 128 bytes of (packed-width) K per row = four MFMA k-steps. LDS holds two stages of A, rows
 *  128 bytes apart, the 16-byte chunk `c` of row `r` stored at chunk position c ^ ((r >> 1) & 7): the 16
 *  rows that one pass of a ds_read_b128 touches then fall into 16 different 16-byte bank groups (measured:
 *  SQ_LDS_BANK_CONFLICT = 0).
 *
 *  The steady-state loop handles two stages per trip so that every register slot and LDS buffer has a
 *  compile-time index, and its body is one basic block (no branches: prefetch indices are clamped instead),
 *  which keeps the compiler's s_waitcnt counting exact. Everything is fetched two stages ahead:
 *      k-step q MFMAs of (s, q) under the LDS reads of the A fragments of (s, q+1); then the B registers
 *               just consumed are refilled with B(s+2, q)
 *      k-step 2 also moves A(s+1), loaded two stages ago, from registers into the other LDS buffer and
 *               refills those registers with A(s+3)
 *      before the last k-step: one barrier; the first fragments of stage s+1 are read under its MFMAs
 *  The packed image pads K with zeros to an even number of stages; on the A side, the bytes a stage reads
 *  past the end of a row (the next row's, or nothing past the end of the matrix) are masked to zero on their
 *  way into LDS, so ragged depths run through the same loop. Only A that is not even dword-aligned takes a
 *  plain guarded loop instead.
 *
 *  A is the MFMA's first operand, so a lane ends up with one column and 16 rows of each 32x32 block and the
 *  epilogue stores dwords that are contiguous across lanes: 128 bytes per row per instruction, any C
 *  alignment. (The other orientation, one row and runs of 4 columns per lane stored as 128-bit vectors,
 *  needs a quarter of the store instructions but writes 32-byte pieces of 32 different rows; it measured
 *  12 % slower on the square shapes and 9 % slower on the retrieval shape.)
 */
/** Does a row of A stop short inside a stage's reads, or does the kernel read one stage more than the rows hold (the
 *  image's depth is padded to an even number of stages)? The types whose arithmetic cares (tail_matters_for) clear such
 *  bytes on their way into LDS; kernels compiled with WHOLE are for depths that fill an even number of stages exactly
 *  and leave those masks out of the loop. */
template <class T, bool NORMS>
constexpr bool tail_matters_for() {
    // floats (the image's zero padding times a NaN is a NaN), u8's row sums, the sums of squares of the distances;
    // the integer products need no care: whatever is read there meets zeros of the image
    return NORMS || T::kUnsigned || !__is_same(typename T::acc_t, v16i);
}

/** 16 bytes per lane from a buffer straight into LDS at `dst` + 16 x lane (`dst` the same in all lanes). A function of
 *  its own: the host pass does not know the instruction, and from inside a lambda of a kernel it would take the kernel's
 *  host side with it. */
typedef __attribute__((address_space(3))) void lds_void_t;
__device__ __forceinline__ void fetch_to_lds(__amdgpu_buffer_rsrc_t rsrc, lds_void_t *dst, uint32_t lane_offset, uint32_t offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, dst, 16, lane_offset, offset, 0, 0);
}

/**
 *  DIRECT: A goes from memory straight into LDS (`buffer_load_dwordx4 ... lds`: 64 lanes x 16 bytes land in 1 KiB of LDS
 *  in lane order, so a lane fetches the chunk that belongs at its position of the swizzled row), not through registers
 *  and `ds_write`. LDS is then a ring of four stages, each an array of its own (the compiler tracks what such a load
 *  writes per array, and only so do the waits for one stage's loads not wait for the next stages' as well); a stage's
 *  loads are issued three stages ahead, and one trip of the loop is four stages. For types that reach LDS as they are
 *  in memory, depths of a whole number of trips, the pipelined kernel across tiles, dot products only (the host
 *  checks).
 */
template <class T, int TM, int TN, bool ACROSS, bool NORMS = false, bool WHOLE = false, bool DIRECT = false>
__global__ __launch_bounds__(256, (TM * TN <= 2 ? 3 : (TM * TN <= 4 && !T::kChunked ? 2 : 1))) void dots_packed_kernel(GemmArgs g) {
    typedef typename T::acc_t acc_t;
    constexpr int BM = TM * 32;
    constexpr int NT = 256;
    constexpr int kStageLds = BM * kStageBytes;
    constexpr int kLoads = BM * kStageChunks / NT; // 16-byte LDS chunks per thread per stage = TM
    constexpr int kSrcStage = kStageChunks * T::kSrcChunk; // source bytes of A per row per stage
    static_assert(!DIRECT || (ACROSS && !NORMS && !T::kUnsigned && !T::kPrewiden && T::kSrcChunk == 16 && T::kImageChunk == 16),
                  "straight into LDS: only what needs nothing done to it on the way");
    __shared__ __attribute__((aligned(1024))) uint8_t lds[DIRECT ? 16 : 2 * kStageLds];
    __shared__ __attribute__((aligned(1024))) uint8_t ring0[DIRECT ? kStageLds : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t ring1[DIRECT ? kStageLds : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t ring2[DIRECT ? kStageLds : 16];
    __shared__ __attribute__((aligned(1024))) uint8_t ring3[DIRECT ? kStageLds : 16];
    __shared__ __attribute__((aligned(16))) uint32_t row_terms[T::kUnsigned ? BM : 4]; // u8 only: 128 * (sum of the bytes of each A row of the tile)
    __shared__ uint32_t row_part[T::kUnsigned ? 2 * BM * kStageChunks : 1]; // u8 only: the partial sums behind them
    typedef typename T::norm_t norm_t;
    __shared__ __attribute__((aligned(16))) uint32_t row_norms[NORMS ? BM : 4]; // distances only: sum of squares of each A row
    __shared__ __attribute__((aligned(16))) float row_factors[NORMS ? BM : 4];  // ... and its refined reciprocal square root
    __shared__ norm_t norm_part[NORMS ? 2 * BM * kStageChunks : 1];              // ... and the partial sums behind them

    uint32_t const tid = threadIdx.x, lane = tid & 63;
    // The wavefront index is the same in all lanes; telling the compiler keeps B addressing in scalar registers.
    uint32_t const wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // Trust, but verify: the image must have been packed for this dtype and these dimensions.
    PackedHeader const *header = (PackedHeader const *)g.bp;
    bool const image_ok = header->magic == kMagic && header->version == kVersion &&
                          header->dtype == (uint32_t)T::kDtype && header->n == g.n && header->k == g.k &&
                          header->k_chunks == g.k_chunks && header->n_tiles == g.n_tiles;
    uint8_t const *data = g.bp + sizeof(PackedHeader);
    constexpr int kImageTileChunk = kTileRows * T::kImageChunk; // one chunk of all 32 rows of a tile, as the image holds it
    uint32_t const *col_terms = (uint32_t const *)(data + (uint64_t)g.n_tiles * g.k_chunks * kImageTileChunk);
    uint32_t const *col_norms = col_terms + (uint64_t)g.n_tiles * kTileRows;

    uint32_t const stages = g.k_chunks / kStageChunks;
    // Stages the pipelined loop takes: all of them when A is at least dword-aligned, which is all that
    // multi-dword global loads need. (readfirstlane: the value is uniform, and it must stay in a scalar register
    // because the stage offsets of the buffer loads derive from it.)
    uint32_t const fast = __builtin_amdgcn_readfirstlane(g.avec >= (T::kSrcChunk < 4 ? T::kSrcChunk : 4) ? stages : 0);
    uint32_t const xr = T::kUnsigned ? 0x80808080u : 0u;
    uint32_t const a_pos = tid & 7;
    // A fragment reads: lane l takes row l % 32 of each 32-row block and chunk 2q + l / 32.
    uint32_t a_frag[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        uint32_t const r = lane & 31, c = 2 * q + (lane >> 5);
        a_frag[q] = r * kStageBytes + ((c ^ ((r >> 1) & 7)) << 4);
    }

    // A staging: thread t fetches chunk t % 8 of rows i*32 + t/8 of a tile and stores it at its swizzled
    // position. The offsets are the same for every tile: rows past the end of A are cut off by the size of
    // the tile's buffer descriptor (such loads return zeros, and their outputs are never stored).
    uint32_t a_off[kLoads]; // byte offset of the thread's source chunk from the tile's first row
    uint32_t a_lds[kLoads]; // where it goes in an LDS stage
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        uint32_t const r = i * 32 + (tid >> 3);
        a_off[i] = r * (uint32_t)g.a_stride + a_pos * T::kSrcChunk;
        a_lds[i] = r * kStageBytes + ((a_pos ^ ((r >> 1) & 7)) << 4);
    }
    uint32_t const b_lane = lane * T::kImageChunk;

    // Loads go through buffer descriptors: one scalar descriptor plus a 32-bit per-lane offset is the cheapest
    // address form to issue (a single address register per lane, no 64-bit vector adds), and a descriptor is
    // all that has to change from one tile to the next. B fragment streams of this wavefront: one descriptor
    // per 32-column tile (tile index clamped to the last one), every lane at offset lane * 16.
    struct TileView {
        uint32_t row0, col0;
        uint8_t const *a; // first row of the tile
        uint32_t a_bytes; // up to the end of its last row that exists
        uint8_t const *b; // first 32-column tile of this wavefront
        uint32_t b_bytes; // up to the end of the packed tiles (or as far as 32 bits reach)
        uint32_t b_tile[TN]; // offsets of the wavefront's tiles from `b`
    };
    auto view_of = [&](uint32_t tile) {
        TileView view;
        uint32_t tile_m, tile_n;
        tile_of_block(tile, g, tile_m, tile_n);
        view.row0 = tile_m * BM;
        view.col0 = tile_n * (128 * TN) + wave * (32 * TN);
        uint32_t const rows_here = g.m - view.row0 < (uint32_t)BM ? g.m - view.row0 : (uint32_t)BM;
        view.a = g.a + (uint64_t)view.row0 * g.a_stride;
        // (whole aligned loads: an aligned A never ends in the middle of one that could fault)
        constexpr uint32_t kLoadAlign = T::kSrcChunk < 4 ? T::kSrcChunk : 4; // (2-byte loads for the 1-bit type)
        view.a_bytes = (rows_here - 1) * (uint32_t)g.a_stride + (((uint32_t)g.k_src_bytes + kLoadAlign - 1) & ~(kLoadAlign - 1));
        uint32_t const tile_bytes = g.k_chunks * kImageTileChunk;
        uint32_t const first = view.col0 / 32 < g.n_tiles ? view.col0 / 32 : g.n_tiles - 1;
        view.b = data + (uint64_t)first * tile_bytes;
        uint64_t const left = (uint64_t)(g.n_tiles - first) * tile_bytes;
        view.b_bytes = left < 0xFFFFFFFFull ? (uint32_t)left : 0xFFFFFFFFu;
#pragma unroll
        for (int j = 0; j < TN; ++j) view.b_tile[j] = (first + j < g.n_tiles ? j : g.n_tiles - 1 - first) * tile_bytes;
        return view;
    };
    auto a_rsrc_of = [](TileView const &view) {
        return __builtin_amdgcn_make_buffer_rsrc((void *)view.a, 0, (int)view.a_bytes, 0x00020000);
    };
    auto b_rsrc_of = [](TileView const &view) {
        return __builtin_amdgcn_make_buffer_rsrc((void *)view.b, 0, (int)view.b_bytes, 0x00020000);
    };

    // When every stage of a tile goes through the pipelined loop, the prefetches of a tile's last stages
    // fetch the first stages of the workgroup's next tile instead of running dry: the pipeline is primed once
    // and then runs across tile boundaries, and the stores of one tile drain under the next tile's MFMAs.
    constexpr bool across = ACROSS; // the host checks that it holds: fast == stages and stages >= 4
    uint32_t const tile_count = g.tile_count;
    // u8 only: every thread sums the unsigned bytes it stages, per staged row, in LDS slots of its own (slot
    // i * 256 + tid: fire-and-forget LDS adds instead of 2 x kLoads registers held through the loop). Two sets:
    // what is staged ahead for the next tile goes to the other one, and the sets swap roles with every tile.
    uint32_t sums_here = 0; // offset of the set of the tile being computed
    if (T::kUnsigned) {
#pragma unroll
        for (int i = 0; i < 2 * kLoads; ++i) row_part[i * NT + tid] = 0;
    }
    auto add_row_sum = [&](int i, uint32_t value, uint32_t set) {
        __hip_atomic_fetch_add(&row_part[set + i * NT + tid], value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    // Distances: the same bookkeeping for the sums of squares of the rows (u32, or f64 for the float types).
    if (NORMS) {
#pragma unroll
        for (int i = 0; i < 2 * kLoads; ++i) norm_part[i * NT + tid] = 0;
    }
    auto add_row_norm = [&](int i, norm_t value, uint32_t set) {
        __hip_atomic_fetch_add(&norm_part[set + i * NT + tid], value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    };
    v4i a_reg[2][kLoads];
    v4i b_reg[2][TN][4];
    v4i af[2][TM];

    typedef __attribute__((address_space(1))) uint8_t global_u8_t;
    typedef __attribute__((address_space(1))) uint32_t global_u32_t;
    if (!image_ok) { // the image was not packed for this call: the reference's error convention, all bits set
        for (uint32_t tile = blockIdx.x; tile < g.tile_count; tile += gridDim.x) {
            uint32_t tile_m, tile_n;
            tile_of_block(tile, g, tile_m, tile_n);
            for (uint32_t at = tid; at < (uint32_t)BM * 128 * TN; at += NT) {
                uint32_t const row = tile_m * BM + at / (128 * TN), col = tile_n * (128 * TN) + at % (128 * TN);
                if (row < g.m && col < g.n && ((row + g.tri_shift) & g.tri_mask) <= col) *(global_u32_t *)((global_u8_t *)g.c + (uint64_t)row * g.c_stride + (uint64_t)col * 4) = 0xFFFFFFFFu;
            }
        }
        return;
    }
    // Persistent workgroups that all start at once stay in step: every compute unit multiplies while none stores,
    // then all of them store at once and share the memory bandwidth, and the two phases add up. Started at evenly
    // spread times instead, some compute while others store, and a shallow product runs at the rate of its stores.
    if (g.stagger_ticks) {
        unsigned long long const until = wall_clock64() + (unsigned long long)blockIdx.x * g.stagger_ticks / gridDim.x;
        while (wall_clock64() < until) __builtin_amdgcn_s_sleep(4);
    }
    TileView cur, nxt;
    acc_t acc[TM][TN];
    constexpr bool kChunked = T::kChunked;
    Totals<acc_t, TM, TN, kChunked> total; // second-level accumulators of the chunked types (see E4M3)

    // A(s) -> registers, in four parts so that the loads can be spread over four k-steps.
    auto load_a = [&](TileView const &view, uint32_t s, auto slot_tag, auto part_tag) {
        constexpr int slot = decltype(slot_tag)::value, part = decltype(part_tag)::value;
        __amdgpu_buffer_rsrc_t const rsrc = a_rsrc_of(view);
        uint32_t const stage_offset = __builtin_amdgcn_readfirstlane(s * kSrcStage); // (the same in all lanes: see load_b)
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            if (i * 4 / kLoads != part) continue;
            v4i v = {0, 0, 0, 0};
            if (T::kSrcChunk == 16) {
                v = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, a_off[i], stage_offset, 0));
            }
            else if (T::kSrcChunk == 2) { v[0] = (int)(uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, a_off[i], stage_offset, 0); }
            else {
                typedef unsigned v2u __attribute__((ext_vector_type(2)));
                v2u const narrow = __builtin_amdgcn_raw_buffer_load_b64(rsrc, a_off[i], stage_offset, 0);
                v[0] = (int)narrow[0], v[1] = (int)narrow[1];
            }
            a_reg[slot][i] = v;
        }
    };
    auto load_a_all = [&](TileView const &view, uint32_t s, auto slot_tag) {
        load_a(view, s, slot_tag, slot_c<0>()), load_a(view, s, slot_tag, slot_c<1>());
        load_a(view, s, slot_tag, slot_c<2>()), load_a(view, s, slot_tag, slot_c<3>());
    };
    // Element-wise work on the staged chunks happens here, after the loads have had time to land.
    // `mine` is 1 for a stage of this tile and 0 for one staged ahead for the next tile.
    // `s` is the stage the registers hold: the bytes of its chunk that lie past the end of the row are cleared
    // (for whole stages the masks come out as all ones; no branch either way).
    int const a_tail = (int)(uint32_t)g.k_src_bytes - (int)(a_pos * T::kSrcChunk); // bytes of the row from this thread's chunk on, stage 0
    constexpr bool kMaskTail = !WHOLE && tail_matters_for<T, NORMS>();
    auto masks_of = [&](uint32_t s, uint32_t (&keep)[(T::kSrcChunk + 3) / 4]) {
        int const left = a_tail - (int)(s * kSrcStage);
#pragma unroll
        for (int w = 0; w < (T::kSrcChunk + 3) / 4; ++w) {
            int const over = left - 4 * w, bytes = over < 0 ? 0 : (over > 4 ? 4 : over);
            keep[w] = bytes == 4 ? 0xFFFFFFFFu : ((1u << (8 * bytes)) - 1u);
        }
    };
    // Half of the staged chunks of stage `s`, masked and widened where they are (types with kPrewiden): what
    // store_a would do right in front of its LDS writes, done a k-step or two earlier among that k-step's MFMAs.
    auto prewiden = [&](auto slot_tag, uint32_t s, auto half_tag) {
        constexpr int slot = decltype(slot_tag)::value, half_of = decltype(half_tag)::value;
        constexpr int kSrcWords = (T::kSrcChunk + 3) / 4;
        uint32_t keep[kSrcWords];
        if (kMaskTail) masks_of(s, keep);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            if (i * 2 / kLoads != half_of) continue;
            v4i v = a_reg[slot][i];
            if (kMaskTail) {
#pragma unroll
                for (int w = 0; w < kSrcWords; ++w) v[w] &= (int)keep[w];
            }
            a_reg[slot][i] = T::widen(v);
        }
    };
    auto store_a = [&](auto buffer_tag, auto slot_tag, uint32_t s, uint32_t mine, auto widened_tag) {
        constexpr int buffer = decltype(buffer_tag)::value, slot = decltype(slot_tag)::value;
        constexpr bool widened = decltype(widened_tag)::value != 0; // prewiden has been over these registers
        uint8_t *dst = lds + buffer * kStageLds;
        constexpr int kSrcWords = (T::kSrcChunk + 3) / 4;
        uint32_t keep[kSrcWords];
        if (!widened && kMaskTail) masks_of(s, keep);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            v4i v = a_reg[slot][i];
            if (!widened && kMaskTail) {
#pragma unroll
                for (int w = 0; w < kSrcWords; ++w) v[w] &= (int)keep[w];
            }
            // (without a next tile to stage for, what is staged past the end is dropped)
            uint32_t const set = across && !mine ? sums_here ^ (uint32_t)(kLoads * NT) : sums_here;
            v4i const raw = v;
            if (T::kUnsigned) {
                uint32_t const sum = sum_bytes_u8(v);
                add_row_sum(i, across ? sum : sum * mine, set);
                v[0] ^= (int)xr, v[1] ^= (int)xr, v[2] ^= (int)xr, v[3] ^= (int)xr;
            }
            v4i const wide = widened ? v : T::widen(v);
            if (NORMS) {
                norm_t const squares = T::sumsq(raw, wide);
                add_row_norm(i, across || mine ? squares : (norm_t)0, set);
            }
            *(v4i *)(dst + a_lds[i]) = wide;
        }
    };
    auto load_b = [&](TileView const &view, uint32_t s, auto slot_tag, auto q_tag) {
        constexpr int slot = decltype(slot_tag)::value, q = decltype(q_tag)::value;
        __amdgpu_buffer_rsrc_t const rsrc = b_rsrc_of(view);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            // (the same in all lanes; saying so keeps the offset a scalar operand where the compiler has lost track of it,
            // instead of a loop over the lanes' values)
            uint32_t const tile_offset = __builtin_amdgcn_readfirstlane(view.b_tile[j] + s * (kStageChunks * kImageTileChunk));
            if constexpr (T::kImageChunk == 2) // (sixteen bits per lane: the rest of the register is never looked at)
                b_reg[slot][j][q][0] = (int)(uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, b_lane + q * 2 * kImageTileChunk, tile_offset, 0);
            else
                b_reg[slot][j][q] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc, b_lane + q * 2 * kImageTileChunk, tile_offset, 0));
        }
    };
    auto ring_of = [&](auto index_tag) -> uint8_t * {
        constexpr int index = decltype(index_tag)::value & 3;
        return index == 0 ? ring0 : (index == 1 ? ring1 : (index == 2 ? ring2 : ring3));
    };
    auto read_frags = [&](auto buffer_tag, auto q_tag, auto parity_tag) {
        constexpr int buffer = decltype(buffer_tag)::value, q = decltype(q_tag)::value,
                      parity = decltype(parity_tag)::value;
        uint8_t const *src = (DIRECT ? ring_of(buffer_tag) : lds + buffer * kStageLds) + a_frag[q];
#pragma unroll
        for (int i = 0; i < TM; ++i) af[parity][i] = *(v4i const *)(src + i * 32 * kStageBytes);
    };
    auto multiply = [&](auto slot_tag, auto q_tag) {
        constexpr int slot = decltype(slot_tag)::value, q = decltype(q_tag)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            v4i const b = T::operand_b(b_reg[slot][j][q]);
#pragma unroll
            for (int i = 0; i < TM; ++i) T::mma(acc[i][j], af[q & 1][i], b);
        }
    };
    // The same for the first k-step of a tile: its MFMAs start the sums from a zero operand, so that no accumulator is
    // ever cleared (the totals of the chunked types are, a block's in front of its MFMA).
    auto multiply_fresh = [&](auto slot_tag, auto q_tag) {
        constexpr int slot = decltype(slot_tag)::value, q = decltype(q_tag)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            v4i const b = T::operand_b(b_reg[slot][j][q]);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                total.clear_block(i, j);
                T::mma_fresh(acc[i][j], af[q & 1][i], b);
            }
        }
    };
    // What staging one chunk of A costs besides its LDS write: vector operations (u8: four exclusive-ors and the byte
    // sums; the distance kinds: the squares) and LDS adds (one per sum kept). The k-step that stages asks for them
    // behind its MFMAs, a chunk's worth each; left alone they all land between the last MFMA and the barrier.
    constexpr bool kIntegerSums = __is_same(typename T::acc_t, v16i);
    constexpr int kStageVector = (T::kUnsigned ? 8 : 0) + (NORMS ? (kIntegerSums ? 5 : 28) : 0);
    constexpr int kStageDs = 1 + (T::kUnsigned ? 1 : 0) + (NORMS ? 1 : 0);
    // Scheduling hints for one k-step. Masks: 0x008 MFMA, 0x020 VMEM read, 0x100 DS read, 0x200 DS write.
    // Fragment reads go one-to-one with the first TM MFMAs; the global loads of the k-step (TN of B
    // and a quarter of A) are spread over the remaining MFMAs; k-step 2 also carries the LDS writes.
    auto schedule_k_step = [&](auto writes_tag, auto vector_tag) {
        constexpr bool writes = decltype(writes_tag)::value != 0;
        constexpr int vector = decltype(vector_tag)::value; // vector operations to put behind every MFMA (0x002)
        constexpr int loads = TN + (kLoads >= 4 ? kLoads / 4 : 1);
        constexpr int rest = TM * (TN - 1);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (vector > 0) __builtin_amdgcn_sched_group_barrier(0x002, vector, 0);
        }
        if constexpr (rest == 0) {
            if (writes) __builtin_amdgcn_sched_group_barrier(0x200, kLoads, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, loads, 0);
        }
        else if constexpr (writes && kStageDs > 1) {
            // The LDS adds are atomics, and the compiler keeps atomics in program order with every other memory
            // operation, this k-step's loads included (which cannot go early anyway: the second half of the MFMAs
            // still reads the registers that B's loads refill). So the stage's k-step 2 stages first in program order,
            // a chunk in front of each MFMA of the second half, and all its loads go behind the last MFMA.
#pragma unroll
            for (int i = 0; i < rest; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (vector > 0) __builtin_amdgcn_sched_group_barrier(0x002, vector, 0);
                if (i < kLoads) __builtin_amdgcn_sched_group_barrier(0x080, kStageDs, 0); // (0x080: any LDS operation)
            }
            if (kLoads > rest) __builtin_amdgcn_sched_group_barrier(0x080, kStageDs * (kLoads - rest), 0);
            __builtin_amdgcn_sched_group_barrier(0x020, loads, 0);
        }
        else {
#pragma unroll
            for (int i = 0; i < rest; ++i) {
                if (writes && i < kLoads) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                if (i * loads / rest != (i + 1) * loads / rest || (loads > rest && i == 0))
                    __builtin_amdgcn_sched_group_barrier(0x020, loads > rest ? loads : 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (vector > 0) __builtin_amdgcn_sched_group_barrier(0x002, vector, 0);
            }
            if (writes && kLoads > rest) __builtin_amdgcn_sched_group_barrier(0x200, kLoads - rest, 0);
        }
    };
    // The first k-step of a tile of the chunked types: in front of every MFMA the 16 zeros of its block's total;
    // fragment reads and loads as in any k-step without LDS writes.
    auto schedule_fresh_k_step = [&]() {
        constexpr int loads = TN + (kLoads >= 4 ? kLoads / 4 : 1);
#pragma unroll
        for (int i = 0; i < TM * TN; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);
            if (i < TM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (i >= TM && i - TM < loads) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        if (TM * TN - TM < loads) __builtin_amdgcn_sched_group_barrier(0x020, loads - (TM * TN - TM), 0);
    };
    // One stage of the steady state; `P` = stage parity = LDS buffer = register slot. Stages s+2 and
    // s+3 are fetched here; past the tile's end they are the first stages of `nxt` (the next tile, or
    // this one again when nothing follows: loads of valid memory that nobody uses).
    // `inside`: how many of the stages s + 2, s + 3 are known to be this tile's (a tile's first two stages, whose numbers
    // are constants and which the host guarantees two or three more: see stage_direct).
    auto stage = [&](auto parity_tag, uint32_t s, auto entry_tag, auto inside_tag) __attribute__((always_inline)) {
        constexpr int P = decltype(parity_tag)::value;
        constexpr int entry = decltype(entry_tag)::value; // 0: in the middle of a sum; 2: the first stage of a tile
        constexpr int inside = ACROSS ? decltype(inside_tag)::value : 0; // (without ACROSS a tile may have two stages only)
        // vector operations behind each MFMA of the k-steps that widen in place: their share of half the chunks
        constexpr int kSpread = T::kPrewiden ? (kLoads * 28 + TM * TN - 1) / (TM * TN) : 0;
        bool const wrap2 = inside < 1 && s + 2 >= fast, wrap3 = inside < 2 && s + 3 >= fast;
        uint32_t const s2 = wrap2 ? s + 2 - fast : s + 2, s3 = wrap3 ? s + 3 - fast : s + 3;
        TileView const &a2 = wrap2 ? nxt : cur, &a3 = wrap3 ? nxt : cur, &b2 = a2;
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<P>(), slot_c<1>(), slot_c<1>());
        if constexpr (entry == 2) multiply_fresh(slot_c<P>(), slot_c<0>());
        else multiply(slot_c<P>(), slot_c<0>());
        load_b(b2, s2, slot_c<P>(), slot_c<0>()), load_a(a2, s2, slot_c<P>(), slot_c<2>());
        if constexpr (T::kPrewiden) prewiden(slot_c<P ^ 1>(), s + 1 < fast ? s + 1 : 0u, slot_c<0>());
        if constexpr (entry == 2 && kChunked) schedule_fresh_k_step();
        else schedule_k_step(slot_c<0>(), slot_c<kSpread>());
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<P>(), slot_c<2>(), slot_c<0>());
        multiply(slot_c<P>(), slot_c<1>());
        load_b(b2, s2, slot_c<P>(), slot_c<1>()), load_a(a2, s2, slot_c<P>(), slot_c<3>());
        if constexpr (T::kPrewiden) prewiden(slot_c<P ^ 1>(), s + 1 < fast ? s + 1 : 0u, slot_c<1>());
        schedule_k_step(slot_c<0>(), slot_c<kSpread>());
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<P>(), slot_c<3>(), slot_c<1>());
        multiply(slot_c<P>(), slot_c<2>());
        if constexpr (kStageDs == 1) load_b(b2, s2, slot_c<P>(), slot_c<2>());
        // A(s+1), loaded over the last two stages, goes to the other buffer (every wavefront left it
        // at the previous barrier); then its registers start being refilled with A(s+3).
        bool const mine = s + 1 < fast;
        store_a(slot_c<P ^ 1>(), slot_c<P ^ 1>(), mine ? s + 1 : 0u, mine ? 1u : 0u, slot_c<T::kPrewiden ? 1 : 0>());
        if constexpr (kStageDs > 1) load_b(b2, s2, slot_c<P>(), slot_c<2>()); // (see schedule_k_step)
        load_a(a3, s3, slot_c<P ^ 1>(), slot_c<0>());
        schedule_k_step(slot_c<1>(), slot_c<kStageVector>());
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<P ^ 1>(), slot_c<0>(), slot_c<0>());
        multiply(slot_c<P>(), slot_c<3>());
        load_b(b2, s2, slot_c<P>(), slot_c<3>()), load_a(a3, s3, slot_c<P ^ 1>(), slot_c<1>());
        schedule_k_step(slot_c<0>(), slot_c<0>());
    };

    // ---- A straight into LDS (DIRECT) ----
    // Fetch t of a wavefront brings the 8 rows from 8 * (4 t + wave) on: lane l lands at row l / 8, position l % 8 of
    // the 1 KiB that starts there, so it fetches the chunk that the swizzle puts at that position.
    uint32_t a_direct[DIRECT ? kLoads : 1];
    if constexpr (DIRECT) {
#pragma unroll
        for (int t = 0; t < kLoads; ++t) {
            uint32_t const r = 8 * (4 * t + wave) + (lane >> 3);
            a_direct[t] = r * (uint32_t)g.a_stride + (((lane & 7) ^ ((r >> 1) & 7)) << 4);
        }
    }
    auto fetch_a = [&](TileView const &view, uint32_t s, auto ring_tag, auto part_tag) __attribute__((always_inline)) {
        constexpr int part = decltype(part_tag)::value;
        __amdgpu_buffer_rsrc_t const rsrc = a_rsrc_of(view);
        uint32_t const stage_offset = __builtin_amdgcn_readfirstlane(s * kSrcStage);
        uint8_t *stage_base = ring_of(ring_tag);
#pragma unroll
        for (int t = 0; t < kLoads; ++t) {
            if (t * 4 / kLoads != part) continue;
            fetch_to_lds(rsrc, (lds_void_t *)(stage_base + (4 * t + wave) * 1024), a_direct[DIRECT ? t : 0], stage_offset);
        }
    };
    auto fetch_a_all = [&](TileView const &view, uint32_t s, auto ring_tag) __attribute__((always_inline)) {
        fetch_a(view, s, ring_tag, slot_c<0>()), fetch_a(view, s, ring_tag, slot_c<1>());
        fetch_a(view, s, ring_tag, slot_c<2>()), fetch_a(view, s, ring_tag, slot_c<3>());
    };
    // Every wavefront waits for its own fetches into a stage (the compiler puts that wait in front of any read of the
    // stage's array: one word is read for the purpose), then all meet: after that the stage is whole for everybody.
    // No fence: a fence would wait for the fetches of the later stages as well. The waits for the fragment reads
    // that are still in flight come with the word read (LDS answers in order).
    auto stage_arrived = [&](auto ring_tag) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        typedef __attribute__((address_space(3))) uint32_t const lds_u32_t;
        uint32_t const word = *(lds_u32_t *)(ring_of(ring_tag) + lane * 4);
        asm volatile("" ::"v"(word) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    // One stage: `R` = its place in the ring, `P` = the register slot of its B (stage parity). A(s+3) is fetched into
    // the ring stage that the barrier of the stage before has freed; B(s+2) into the registers just used.
    auto schedule_direct_k_step = [&]() {
        constexpr int loads = TN + (kLoads >= 4 ? kLoads / 4 : 1);
        constexpr int rest = TM * (TN - 1);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        }
        if constexpr (rest == 0) __builtin_amdgcn_sched_group_barrier(0x020, loads, 0);
        else {
#pragma unroll
            for (int i = 0; i < rest; ++i) {
                if (i * loads / (rest ? rest : 1) != (i + 1) * loads / (rest ? rest : 1) || (loads > rest && i == 0))
                    __builtin_amdgcn_sched_group_barrier(0x020, loads > rest ? loads : 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
        }
    };
    // (`inside`: stages s + 2 and s + 3 are known to be this tile's, as in a tile's first trip, whose stage numbers are
    // constants: left to choose, the compiler computes the choices once, in vector registers that it then spills, and
    // the reload of a spill is a load whose wait is a wait for everything prefetched)
    auto stage_direct = [&](auto ring_tag, uint32_t s, auto entry_tag, auto inside_tag) __attribute__((always_inline)) {
        constexpr int R = decltype(ring_tag)::value & 3, P = R & 1;
        constexpr int entry = decltype(entry_tag)::value;
        constexpr bool inside = decltype(inside_tag)::value != 0;
        bool const wrap2 = !inside && s + 2 >= fast, wrap3 = !inside && s + 3 >= fast;
        uint32_t const s2 = wrap2 ? s + 2 - fast : s + 2, s3 = wrap3 ? s + 3 - fast : s + 3;
        TileView const &b2 = wrap2 ? nxt : cur, &a3 = wrap3 ? nxt : cur;
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<R>(), slot_c<1>(), slot_c<1>());
        if constexpr (entry == 2) multiply_fresh(slot_c<P>(), slot_c<0>());
        else multiply(slot_c<P>(), slot_c<0>());
        load_b(b2, s2, slot_c<P>(), slot_c<0>()), fetch_a(a3, s3, slot_c<R + 3>(), slot_c<0>());
        if constexpr (entry == 2 && kChunked) schedule_fresh_k_step();
        else schedule_direct_k_step();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<R>(), slot_c<2>(), slot_c<0>());
        multiply(slot_c<P>(), slot_c<1>());
        load_b(b2, s2, slot_c<P>(), slot_c<1>()), fetch_a(a3, s3, slot_c<R + 3>(), slot_c<1>());
        schedule_direct_k_step();
        __builtin_amdgcn_sched_barrier(0);
        read_frags(slot_c<R>(), slot_c<3>(), slot_c<1>());
        multiply(slot_c<P>(), slot_c<2>());
        load_b(b2, s2, slot_c<P>(), slot_c<2>()), fetch_a(a3, s3, slot_c<R + 3>(), slot_c<2>());
        schedule_direct_k_step();
        stage_arrived(slot_c<R + 1>());
        read_frags(slot_c<R + 1>(), slot_c<0>(), slot_c<0>());
        multiply(slot_c<P>(), slot_c<3>());
        load_b(b2, s2, slot_c<P>(), slot_c<3>()), fetch_a(a3, s3, slot_c<R + 3>(), slot_c<3>());
        schedule_direct_k_step();
    };
    auto prime_direct = [&]() {
        __syncthreads();
        fetch_a_all(cur, 0, slot_c<0>());
        load_b(cur, 0, slot_c<0>(), slot_c<0>()), load_b(cur, 0, slot_c<0>(), slot_c<1>());
        load_b(cur, 0, slot_c<0>(), slot_c<2>()), load_b(cur, 0, slot_c<0>(), slot_c<3>());
        fetch_a_all(cur, 1, slot_c<1>());
        load_b(cur, 1, slot_c<1>(), slot_c<0>()), load_b(cur, 1, slot_c<1>(), slot_c<1>());
        load_b(cur, 1, slot_c<1>(), slot_c<2>()), load_b(cur, 1, slot_c<1>(), slot_c<3>());
        fetch_a_all(cur, 2, slot_c<2>());
        stage_arrived(slot_c<0>());
        read_frags(slot_c<0>(), slot_c<0>(), slot_c<0>());
    };

    // Fills the pipeline for a tile: stages 0 and 1 on their way, A(0) in LDS, its first fragments read.
    auto prime = [&]() {
        __syncthreads(); // the previous tile's last fragment reads are done
        load_a_all(cur, 0, slot_c<0>());
        load_b(cur, 0, slot_c<0>(), slot_c<0>()), load_b(cur, 0, slot_c<0>(), slot_c<1>());
        load_b(cur, 0, slot_c<0>(), slot_c<2>()), load_b(cur, 0, slot_c<0>(), slot_c<3>());
        load_a_all(cur, 1, slot_c<1>());
        load_b(cur, 1, slot_c<1>(), slot_c<0>()), load_b(cur, 1, slot_c<1>(), slot_c<1>());
        load_b(cur, 1, slot_c<1>(), slot_c<2>()), load_b(cur, 1, slot_c<1>(), slot_c<3>());
        store_a(slot_c<0>(), slot_c<0>(), 0u, 1u, slot_c<0>());
        // the first half of A(2), as k-steps 2 and 3 of a stage "-1" would have issued it
        // (with two stages in all it is A(0) again, which nobody uses)
        uint32_t const third = fast > 2 ? 2 : 0;
        load_a(cur, third, slot_c<0>(), slot_c<0>()), load_a(cur, third, slot_c<0>(), slot_c<1>());
        __syncthreads();
        read_frags(slot_c<0>(), slot_c<0>(), slot_c<0>());
    };
    if constexpr (across) {
        cur = view_of(blockIdx.x);
        if constexpr (DIRECT) prime_direct();
        else prime();
    }

    for (uint32_t tile = blockIdx.x; tile < tile_count; tile += gridDim.x) {
        cur = view_of(tile);
        bool const has_next = across && tile + gridDim.x < tile_count;
        nxt = view_of(has_next ? tile + gridDim.x : tile);
        uint32_t const row0 = cur.row0, col0 = cur.col0;

        // u8: the column terms of this tile are fetched now and used in the epilogue, so that nothing has to
        // wait for them (a wait for a load is a wait for every store issued before it).
        uint32_t col_term[TN], col_norm[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            col_term[j] = 0, col_norm[j] = 0;
            uint32_t const t = col0 / 32 + j < g.n_tiles ? col0 / 32 + j : g.n_tiles - 1;
            if constexpr (T::kUnsigned) col_term[j] = col_terms[(uint64_t)t * kTileRows + (lane & 31)];
            if constexpr (NORMS) col_norm[j] = col_norms[(uint64_t)t * kTileRows + (lane & 31)];
        }

        {
            if (across || fast > 0) { // (always, when the pipeline runs across tiles: the host checked)
                if constexpr (!across) prime();
                // Nothing is cleared at the start of a tile: in its first k-step the first MFMA of every block takes a
                // zero operand (and the totals of the chunked types are zeroed next to it). Chunked types: every
                // `chunk_stages` stages the running sums go into the totals.
                uint32_t until_fold = g.chunk_stages;
                auto fold_when_due = [&]() __attribute__((always_inline)) {
                    if constexpr (kChunked) {
                        until_fold -= 2;
                        if (until_fold == 0) {
                            __builtin_amdgcn_sched_barrier(0);
                            total.fold(acc);
                            until_fold = g.chunk_stages;
                        }
                    }
                };
                if constexpr (DIRECT) { // (four stages a trip: the host checked that the depth, and a chunk, are whole trips)
                    auto fold_after_trip = [&]() __attribute__((always_inline)) {
                        if constexpr (kChunked) {
                            until_fold -= 4;
                            if (until_fold == 0) {
                                __builtin_amdgcn_sched_barrier(0);
                                total.fold(acc);
                                until_fold = g.chunk_stages;
                            }
                        }
                    };
                    stage_direct(slot_c<0>(), 0u, slot_c<2>(), slot_c<1>()); // (at least eight stages: the host checked)
                    stage_direct(slot_c<1>(), 1u, slot_c<0>(), slot_c<1>());
                    stage_direct(slot_c<2>(), 2u, slot_c<0>(), slot_c<1>());
                    stage_direct(slot_c<3>(), 3u, slot_c<0>(), slot_c<1>());
                    fold_after_trip();
                    for (uint32_t s = 4; s < fast; s += 4) {
                        stage_direct(slot_c<0>(), s, slot_c<0>(), slot_c<0>());
                        stage_direct(slot_c<1>(), s + 1, slot_c<0>(), slot_c<0>());
                        stage_direct(slot_c<2>(), s + 2, slot_c<0>(), slot_c<0>());
                        stage_direct(slot_c<3>(), s + 3, slot_c<0>(), slot_c<0>());
                        fold_after_trip();
                    }
                }
                else {
                    stage(slot_c<0>(), 0u, slot_c<2>(), slot_c<2>()); // (with ACROSS at least four stages: the host checked)
                    stage(slot_c<1>(), 1u, slot_c<0>(), slot_c<1>());
                    fold_when_due();
                    for (uint32_t s = 2; s < fast; s += 2) {
                        stage(slot_c<0>(), s, slot_c<0>(), slot_c<0>());
                        stage(slot_c<1>(), s + 1, slot_c<0>(), slot_c<0>());
                        fold_when_due();
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }

            // Remaining stages: the ragged end of K, or everything when A cannot be read with vector loads.
            if (!across && fast < stages) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
                total.clear();
                uint8_t const *a_tile = g.a + (uint64_t)row0 * g.a_stride;
                uint32_t a_slow[kLoads]; // rows clamped to the last one: plain loads have no descriptor to stop them
#pragma unroll
                for (int i = 0; i < kLoads; ++i) {
                    uint32_t const r = i * 32 + (tid >> 3);
                    uint32_t const row = row0 + r < g.m ? r : g.m - 1 - row0;
                    a_slow[i] = row * (uint32_t)g.a_stride + a_pos * T::kSrcChunk;
                }
                uint32_t until_fold = g.chunk_stages;
                for (uint32_t s = fast; s < stages; ++s) {
                    __syncthreads();
                    int64_t const left = (int64_t)g.k_src_bytes - (int64_t)s * kSrcStage - (int64_t)a_pos * T::kSrcChunk;
                    int const valid = (int)(left > T::kSrcChunk ? T::kSrcChunk : (left < 0 ? 0 : left));
#pragma unroll
                    for (int i = 0; i < kLoads; ++i) {
                        v4i v = load_chunk_guarded(a_tile + (uint64_t)s * kSrcStage + a_slow[i], valid, g.avec, 0u);
                        v4i const raw = v;
                        if (T::kUnsigned) {
                            add_row_sum(i, sum_bytes_u8(v), sums_here);
#pragma unroll
                            for (int w = 0; w < 4; ++w) { // flip only bytes that exist: the zero padding stays zero
                                int const rem = valid - 4 * w;
                                uint32_t const mask = rem >= 4 ? 0x80808080u : (rem <= 0 ? 0u : (0x80808080u >> (8 * (4 - rem))));
                                v[w] ^= (int)mask;
                            }
                        }
                        v4i const wide = T::widen(v);
                        if (NORMS) add_row_norm(i, T::sumsq(raw, wide), sums_here);
                        *(v4i *)(lds + a_lds[i]) = wide;
                    }
                    load_b(cur, s, slot_c<0>(), slot_c<0>()), load_b(cur, s, slot_c<0>(), slot_c<1>());
                    load_b(cur, s, slot_c<0>(), slot_c<2>()), load_b(cur, s, slot_c<0>(), slot_c<3>());
                    __syncthreads();
                    read_frags(slot_c<0>(), slot_c<0>(), slot_c<0>());
                    read_frags(slot_c<0>(), slot_c<1>(), slot_c<1>());
                    multiply(slot_c<0>(), slot_c<0>());
                    read_frags(slot_c<0>(), slot_c<2>(), slot_c<0>());
                    multiply(slot_c<0>(), slot_c<1>());
                    read_frags(slot_c<0>(), slot_c<3>(), slot_c<1>());
                    multiply(slot_c<0>(), slot_c<2>());
                    multiply(slot_c<0>(), slot_c<3>());
                    if constexpr (kChunked) { // the same two-level accumulation as the pipelined loop
                        if (--until_fold == 0) {
                            total.fold(acc);
                            until_fold = g.chunk_stages;
                        }
                    }
                }
            }
        }

        // Epilogue. Accumulator register v of lane l holds C[8*(v/4) + 4*(l/32) + v%4][l%32] of its 32x32 tile.
        uint32_t const half = lane >> 5, col_in_tile = lane & 31;
        if (T::kUnsigned || NORMS) {
            __syncthreads();
            // The 8 threads that staged a row left its partial sums in 8 adjacent slots.
            if (tid < BM) {
                if (T::kUnsigned) {
                    uint32_t const *parts = &row_part[sums_here + tid * 8];
                    uint32_t sum = 0;
#pragma unroll
                    for (int part = 0; part < 8; ++part) sum += parts[part];
                    row_terms[tid] = sum * 128u;
                }
                if (NORMS) {
                    norm_t const *parts = &norm_part[sums_here + tid * 8];
                    norm_t sum = 0;
#pragma unroll
                    for (int part = 0; part < 8; ++part) sum += parts[part];
                    uint32_t bits;
                    if constexpr (sizeof(norm_t) == 8) bits = __builtin_bit_cast(uint32_t, (float)sum); // f64 -> f32, once
                    else bits = (uint32_t)sum;
                    row_norms[tid] = __builtin_bit_cast(uint32_t, norm_as_f32<T>(bits));
                    row_factors[tid] = refined_rsqrt(norm_as_f32<T>(bits));
                }
            }
            __syncthreads();
#pragma unroll
            for (int i = 0; i < kLoads; ++i) { // own slots: ready for the tile after next
                if (T::kUnsigned) row_part[sums_here + i * NT + tid] = 0;
                if (NORMS) norm_part[sums_here + i * NT + tid] = 0;
            }
            sums_here ^= (uint32_t)(kLoads * NT);
        }
        // Stores: a scalar base plus one 32-bit per-lane offset, through an explicitly global pointer. (A store
        // through a generic pointer counts as an LDS operation as well, and with such stores in flight the loads
        // prefetched for the next tile could only be waited for all at once.) Tiles that touch the matrix edge take
        // the masked copy of the loop.
        // Of a triangular grid, a wavefront's part of a tile is stored whole (all of it right of the diagonal), not
        // at all (all of it left), or through the masked copy.
        // What only the stores need is read from the kernel's arguments again, here, rather than held in a dozen
        // scalar registers through the loop (the empty asm hides from the compiler that it is the same memory).
        typedef __attribute__((address_space(4))) GemmArgs const late_args_t;
        late_args_t *late = (late_args_t *)__builtin_amdgcn_kernarg_segment_ptr();
        asm volatile("" : "+s"(late));
        // Stores go past the caches (`nt`): the output is written once and not read here, and the caches are left to the
        // operands (measured on one box, same run: bf16 8192^3 1.047 -> 0.972 ms, e4m3 1.027 -> 0.933 ms, i8 0.526 ->
        // 0.518 ms, i8 1024 x 1,048,576 x 768 1.455 -> 1.395 ms). Except where the rows of C do not start on 128-byte
        // lines and the product is not deep: a 128-byte run of a row then straddles two lines and would reach the
        // memory as two partial writes; through the L2 the parts of a line written by neighbouring wavefronts meet
        // first (measured, i8, nt -> plain: 8192 x 8191 x 1000
        // 0.199 -> 0.146 ms, 4096 x 4095 x 4096 0.099 -> 0.077, 1024 x 1,000,001 x 768 3.99 -> 1.92 ms; bf16 4096 x 4095 x
        // 4096 0.155 -> 0.143, but 8192 x 8191 x 8192 0.97 -> 1.04: a deep product wants its L2 for the operands).
        // The distance kinds keep `nt` (i8 angular 1024 x 1,000,001 x 768: 2.57 against 2.70 ms).
        bool const lines = (((uint64_t)late->c | late->c_stride) & 127) == 0;
        bool const streamed = NORMS || (late->store_policy ? late->store_policy == 1 : lines || stages > 64);
        // (the distance kinds force the diagonal to zero in the masked copy only: a part of a tile that holds a
        // diagonal element, even its corner alone, is not interior for them)
        bool const interior = row0 + BM <= late->m && col0 + 32 * TN <= late->n &&
                              (((row0 + (BM - 1) + (NORMS ? 1u : 0u) + late->tri_shift) & late->tri_mask) <= col0);
        bool const nothing = ((row0 + late->tri_shift) & late->tri_mask) > col0 + (32 * TN - 1);
        global_u8_t *c_tile = (global_u8_t *)late->c + (uint64_t)row0 * late->c_stride + (uint64_t)col0 * 4;
        auto store_all = [&](auto masked_tag, auto metric_tag, auto streamed_tag) {
            constexpr bool masked = decltype(masked_tag)::value != 0;
            constexpr int metric = decltype(metric_tag)::value;
            constexpr bool past_caches = decltype(streamed_tag)::value != 0;
            uint64_t const row_step = late->c_stride;
            // Lane l holds column l % 32; register v holds row 8 * (v / 4) + 4 * (l / 32) + v % 4.
            uint32_t const lane_offset = 4 * half * (uint32_t)late->c_stride + col_in_tile * 4;
            // Masked tiles: rows of the matrix from this lane's first one on, and how far right of the diagonal
            // col = row + tri_shift its first element lies (element (r, 32 j) from there is stored when
            // r - 32 j <= that distance; without a triangle everything is).
            int const rows_left = (int)(late->m - row0 - 4 * half);
            int const diagonal = late->tri_mask ? (int)(col0 + col_in_tile) - (int)(row0 + 4 * half + late->tri_shift) : 0x7FFFFFFF;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                bool const col_ok = col0 + j * 32 + col_in_tile < late->n;
                // Rows come in runs of 4 that start 8 apart: the base advances by one row or by five. The
                // empty asm keeps it a running scalar (otherwise every row's base is precomputed and the
                // scalar registers overflow).
                global_u8_t *row_base = c_tile + j * 128;
                v4i row_term4 = {0, 0, 0, 0}, row_norm4 = {0, 0, 0, 0};
                typedef float v4f __attribute__((ext_vector_type(4)));
                v4f row_factor4 = {0, 0, 0, 0};
                float const col_value = metric != 0 ? norm_as_f32<T>(col_norm[j]) : 0.0f;
                float const col_factor = metric == 1 ? refined_rsqrt(col_value) : 0.0f;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        int const r_fixed = i * 32 + 8 * (v / 4) + (v % 4); // row of lanes 0..31; lanes 32..63 are 4 rows below
                        // a named copy: bit-casting the vector element expression itself reads lane 0
                        auto const element = total.finish(acc, i, j, v);
                        uint32_t bits = finished_dot<T>(__builtin_bit_cast(uint32_t, element));
                        if (T::kUnsigned) {
                            // the terms of 4 consecutive rows in one LDS read
                            if (v % 4 == 0) row_term4 = *(v4i const *)&row_terms[i * 32 + 8 * (v / 4) + 4 * half];
                            bits += (uint32_t)row_term4[v % 4] + col_term[j];
                        }
                        if (metric == 1) {
                            // the cheap form where it is good enough (almost everywhere on vectors that are not near
                            // copies of each other), the full finaliser for the lanes where it is not
                            if (v % 4 == 0) row_factor4 = *(v4f const *)&row_factors[i * 32 + 8 * (v / 4) + 4 * half];
                            bool cheap;
                            float const quick = angular_from_factors<T>(bits, row_factor4[v % 4], col_factor, &cheap);
                            uint32_t result = __builtin_bit_cast(uint32_t, quick);
                            if (__builtin_amdgcn_ballot_w64(!cheap) != 0) { // (uniform: the wavefront branches as one)
                                int const row_bits = *(int const *)&row_norms[i * 32 + 8 * (v / 4) + 4 * half + v % 4];
                                uint32_t const full = distance_from_dot<T, 1>(bits, __builtin_bit_cast(float, row_bits), col_value);
                                result = cheap ? result : full;
                            }
                            bits = result;
                        }
                        else if (metric != 0) {
                            if (v % 4 == 0) row_norm4 = *(v4i const *)&row_norms[i * 32 + 8 * (v / 4) + 4 * half];
                            int const row_bits = row_norm4[v % 4];
                            bits = distance_from_dot<T, 2>(bits, __builtin_bit_cast(float, row_bits), col_value);
                        }
                        bool keep = true;
                        if (masked) {
                            keep = col_ok && r_fixed < rows_left && r_fixed - j * 32 <= diagonal;
                            // a vector's distance from itself is exactly 0 (dots/serial.h:2871-2876)
                            if (metric != 0 && r_fixed - j * 32 == diagonal) bits = 0;
                        }
                        if (keep) {
                            if (past_caches) __builtin_nontemporal_store(bits, (global_u32_t *)(row_base + lane_offset));
                            else *(global_u32_t *)(row_base + lane_offset) = bits;
                        }
                        row_base += (v % 4 == 3 ? 5 : 1) * row_step;
                        asm volatile("" : "+s"(row_base));
                    }
                    // u8 reads a row term per element: keep those reads from being hoisted by the hundred
                    // (registers are what the prefetched tile is short of here).
                    if (T::kUnsigned || metric != 0) __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        auto store_as = [&](auto metric_tag) {
            if (interior) {
                if (NORMS || streamed) store_all(slot_c<0>(), metric_tag, slot_c<1>());
                else if constexpr (!NORMS) store_all(slot_c<0>(), metric_tag, slot_c<0>());
            }
            else {
                if (NORMS || streamed) store_all(slot_c<1>(), metric_tag, slot_c<1>());
                else if constexpr (!NORMS) store_all(slot_c<1>(), metric_tag, slot_c<0>());
            }
        };
        if (nothing) {}
        else if constexpr (NORMS) { // which distance is a run-time choice: one kernel serves both
            if (late->metric == 2) store_as(slot_c<2>());
            else store_as(slot_c<1>());
        }
        else store_as(slot_c<0>());
    }
}

struct TileConfig {
    int tm, tn;
};
// Index 0 is "choose for me"; 1.. are explicit (5: e2m3 only).
constexpr TileConfig kConfigs[] = {{0, 0}, {8, 2}, {4, 2}, {4, 1}, {2, 1}, {4, 4}};
constexpr int kConfigCount = sizeof(kConfigs) / sizeof(kConfigs[0]);


/** Tiles of a bm x bn grid over m x n outputs with something on or right of the diagonal col = row + shift. */
inline uint32_t log2_of(uint32_t power_of_two) { return (uint32_t)__builtin_ctz(power_of_two); }
inline uint64_t live_tiles(uint64_t m, uint64_t n, uint32_t bm, uint32_t bn, uint32_t shift) {
    uint32_t const tiles_m = (uint32_t)((m + bm - 1) / bm), tiles_n = (uint32_t)((n + bn - 1) / bn);
    uint64_t count = 0;
    for (uint32_t t = 0; t < tiles_m; ++t) {
        uint32_t const from = first_live_tile(t, log2_of(bm), log2_of(bn), shift);
        count += from < tiles_n ? tiles_n - from : 0;
    }
    return count;
}
inline size_t triangle_scratch_bytes(uint64_t m, uint64_t n, uint32_t bm, uint32_t bn, uint32_t shift) {
    uint64_t const bands = ((m + bm - 1) / bm + kTileBand - 1) / kTileBand;
    return (size_t)(((bands + 1 + 1) & ~1ull) * 4 + live_tiles(m, n, bm, bn, shift) * 8);
}

/** `slots_only`: do not launch, only report how many workgroups of the kernel this call would use are resident on
 *  the device at once. */
template <class T, int TM, int TN>
hipError_t launch_one(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle, int *slots_only = nullptr) {
    constexpr int BM = TM * 32, BN = TN * 128;
    g.tiles_m = (g.m + BM - 1) / BM;
    g.tiles_n = (g.n + BN - 1) / BN;
    uint64_t tiles = (uint64_t)g.tiles_m * g.tiles_n;
    if (tiles > 0x7FFFFFFFull) return hipErrorInvalidValue;
    g.tile_list = nullptr;
    if (triangle) {
        tiles = live_tiles(g.m, g.n, BM, BN, g.tri_shift);
        if (!tiles) return hipSuccess;
        if (triangle_scratch_bytes(g.m, g.n, BM, BN, g.tri_shift) > triangle->bytes) return hipErrorInvalidValue;
        uint32_t const bands = (g.tiles_m + kTileBand - 1) / kTileBand;
        g.tile_list = triangle->words + ((bands + 1 + 1) & ~1u); // (written by the caller's triangle_tiles_kernel)
    }
    g.tile_count = (uint32_t)tiles;
    // The tile's A offsets are 32-bit: (rows of a tile) * stride must stay below 4 GiB.
    if ((uint64_t)BM * g.a_stride > 0xFFFFFFFFull) return hipErrorInvalidValue;
    // So are the per-lane C offsets: 4 rows plus the tile's width.
    if (4 * (uint64_t)g.c_stride + BN * 4 > 0xFFFFFFFFull) return hipErrorInvalidValue;
    // The offsets into a wavefront's B tiles are 32-bit as well.
    if ((uint64_t)(TN + 1) * g.k_chunks * kTileRows * T::kImageChunk > 0xFFFFFFFFull) return hipErrorInvalidValue;
    // The pipeline runs across tile boundaries when the pipelined loop takes the stages of a tile (A readable
    // with dword loads) and there are enough of them to prefetch three ahead.
    uint32_t const stages = g.k_chunks / kStageChunks;
    bool const across = g.avec >= (T::kSrcChunk < 4 ? T::kSrcChunk : 4) && stages >= 4;
    bool const norms = g.metric != 0;
    // depths that fill an even number of stages exactly: the pipelined kernel without the tail masks
    bool const whole = across && g.k_src_bytes % (2 * kStageChunks * T::kSrcChunk) == 0;
    void (*kernel)(GemmArgs) = across ? dots_packed_kernel<T, TM, TN, true, false> : dots_packed_kernel<T, TM, TN, false, false>;
    if constexpr (tail_matters_for<T, false>()) {
        if (whole) kernel = dots_packed_kernel<T, TM, TN, true, false, true>;
    }
    // A straight into LDS (see the kernel): the largest tile of the types that reach LDS as they are, depths of whole
    // trips of four stages, and for the two-accumulator types folds that fall between trips (measured at 8192^3,
    // alternating in one session: i8 0.438 -> 0.419 ms, bf16 0.930 -> 0.902, f16 0.997 -> 0.968; with a fold after every
    // second stage of the trip instead, the compiler ran out of registers in the folds and bf16 took 1.10 ms)
    bool direct = false;
    if constexpr (kDirectStaging && !T::kUnsigned && !T::kPrewiden && T::kSrcChunk == 16 && T::kImageChunk == 16 &&
                  ((TM == 8 && TN == 2) || (TM == 4 && TN == 2 && T::kChunked))) {
        direct = across && !norms && stages % 4 == 0 && stages >= 8 && (whole || !tail_matters_for<T, false>()) &&
                 (!T::kChunked || g.chunk_stages % 4 == 0) &&
                 (g.avec >= 16) && !(forced_tile_config() & 0x40000000);
        if (direct) kernel = dots_packed_kernel<T, TM, TN, true, false, tail_matters_for<T, false>(), true>;
    }
    if constexpr (T::kDistances) {
        if (norms) kernel = across ? dots_packed_kernel<T, TM, TN, true, true> : dots_packed_kernel<T, TM, TN, false, true>;
        if (norms && whole) kernel = dots_packed_kernel<T, TM, TN, true, true, true>;
    }
    else if (norms) return hipErrorInvalidValue;
    // Persistent grid: as many workgroups as fit on the device at once (queried once per kernel; threads that
    // ask at the same time store the same number).
    static std::atomic<int> resident_of[9];
    std::atomic<int> &slot = resident_of[direct ? 8 : (across ? 1 : 0) + (norms ? 2 : 0) + (whole ? 4 : 0)];
    int resident = slot.load(std::memory_order_relaxed);
    if (!resident) {
        int per_cu = 0;
        hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (void const *)kernel, 256, 0);
        if (e != hipSuccess) return e;
        int const units = compute_unit_count();
        resident = (per_cu > 0 ? per_cu : 1) * (units > 0 ? units : 256);
        slot.store(resident, std::memory_order_relaxed);
    }
    if (slots_only) {
        *slots_only = resident;
        return hipSuccess;
    }
    uint32_t const blocks = (uint32_t)(tiles < (uint64_t)resident ? tiles : (uint64_t)resident);
    // Shallow products with several tiles per workgroup are bound by their stores: spread the starts over about the
    // time one round of tiles takes to store (the chip writes some 5.5 TB/s in this pattern; ticks of 10 ns).
    g.stagger_ticks = 0;
    if (stages <= 16 && tiles >= 4 * (uint64_t)blocks) {
        double const round_bytes = (double)BM * BN * 4 * blocks;
        g.stagger_ticks = (uint32_t)(round_bytes / 5.5e12 * 1e8);
    }
    int const forced = forced_tile_config();
    if ((forced >> 8) & 0xFFFFF) g.stagger_ticks = (uint32_t)((forced >> 8) & 0xFFFFF) - 1; // (test hook: bits 8..27 = ticks + 1)
    g.store_policy = (uint32_t)(forced >> 28) & 3;                                          // (test hook: bits 28..29)
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, stream, g);
    return hipGetLastError();
}

template <class T>
hipError_t launch_config(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle, int config,
                         int *slots_only = nullptr) {
    switch (config) {
    case 1:
        if constexpr (T::kChunked) return hipErrorInvalidValue;
        else return launch_one<T, 8, 2>(g, stream, triangle, slots_only);
    case 2: return launch_one<T, 4, 2>(g, stream, triangle, slots_only);
    case 3: return launch_one<T, 4, 1>(g, stream, triangle, slots_only);
    case 5:
        if constexpr (T::kDtype != kE2M3) return hipErrorInvalidValue;
        else return launch_one<T, 4, 4>(g, stream, triangle, slots_only);
    default: return launch_one<T, 2, 1>(g, stream, triangle, slots_only);
    }
}

template <class T>
hipError_t launch_typed(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle) {
    int const forced = forced_tile_config();
    int config = forced & 0x7F;
    bool const chosen_here = config <= 0 || config >= kConfigCount;
    auto tiles_of = [&](GemmArgs const &args, int c) {
        uint64_t const bm = kConfigs[c].tm * 32, bn = (uint64_t)kConfigs[c].tn * 128;
        if (triangle) return live_tiles(args.m, args.n, (uint32_t)bm, (uint32_t)bn, args.tri_shift);
        return ((args.m + bm - 1) / bm) * ((args.n + bn - 1) / bn);
    };
    // Largest tile that still gives every one of the 256 CUs at least one workgroup.
    auto choose = [&](GemmArgs const &args, int first) {
        int best = 4;
        for (int c = first; c <= 4; ++c)
            if (tiles_of(args, c) >= 256) {
                best = c;
                break;
            }
        // Distances over a shallow depth are bound by the epilogue (a finaliser and a store per output): two
        // workgroups per CU of 128 x 128 tiles overlap it with the other's loop better than one large tile does
        // (measured on 1024 x 1,048,576 x 768: 2.17 against 2.33 ms angular, 1.98 against 2.07 ms euclidean).
        // Since then the angular finaliser has become cheap where the cosine is small, and what is left of an epilogue's
        // cost is its length: the code of TM x TN x 16 finalisers and stores does not fit the instruction cache for the
        // large tiles. Measured, shallow depths (best shape against the others, ms): i8 angular 1024 x 1,048,576 x 768
        // 128 x 256 1.73, 256 x 256 1.78, 128 x 128 1.90, 64 x 128 2.09, but 8192 x 131,072 x 768 and 8192 x 8192 x
        // 1024 128 x 128 (1.42 against 1.55; 0.114 against 0.120); u8 128 x 128 (2.29 against 2.54 and 2.91); bf16
        // angular 1024 x 524,288 x 768 64 x 128 1.58 against 1.72 (128 x 128) and 2.18 (128 x 256), 8192 x 8192 x 1024
        // 0.198 against 0.267 and 0.319, and still 3.39 against 3.77 at depth 2048; f16 and e4m3 likewise.
        uint32_t const depth_stages = args.k_chunks / kStageChunks;
        if (args.metric != 0 && T::kChunked) {
            if (depth_stages <= 32 && tiles_of(args, 4) >= 256) best = 4;
        }
        else if (args.metric != 0 && depth_stages <= 8) {
            if (!T::kUnsigned && args.m <= 2048 && best < 2 && tiles_of(args, 2) >= 256) best = 2;
            else if (best < 3 && tiles_of(args, 3) >= 256) best = 3;
        }
        if (T::kChunked && best == 1) best = 2; // two accumulator sets do not fit the 256 x 256 tile
        // Shallow products into rows of C that do not start on 128-byte lines: the stores go through the L2 (see the
        // epilogue) and take long enough to matter, and three small workgroups per compute unit overlap one's stores
        // with the others' loops, which one large tile cannot (measured, 64 x 128 against the tile chosen above: i8
        // 8192 x 8191 x 1000 0.129 against 0.142 ms, x 512 0.085 against 0.101; f16 8192 x 8191 x 1000 0.239 against
        // 0.280; i8 4096 x 4095 x 1000 0.036 against 0.039; deeper products and aligned rows lose by it).
        bool const lines = (((uintptr_t)args.c | args.c_stride) & 127) == 0;
        if (!lines && !triangle && args.metric == 0 && best < 4 && args.k_chunks / kStageChunks <= (T::kChunked ? 16u : 8u) &&
            tiles_of(args, 4) >= 256)
            best = 4;
        // e2m3 pays 13 vector operations for every dword of A it stages: a 128 x 512 tile (every wavefront 128 x 128)
        // stages half as much A per MFMA as 256 x 256 (8192^3: 0.51 against 0.59 ms; for i8 itself the two are equal)
        // (not the f16 route of very deep rows: its two accumulator sets do not fit that tile)
        if (T::kDtype == kE2M3 && !T::kChunked && !triangle && args.metric == 0 && first == 1 && tiles_of(args, 5) >= 256) best = 5;
        return best;
    };
    if (chosen_here) config = choose(g, 1);
    if (T::kChunked && config == 1) config = 2;
    // Where the tile list of a launch goes (the same arithmetic as launch_one's) and what it holds.
    auto grid_of = [](GemmArgs const &args, int c, TriangleScratch const &scratch) {
        uint32_t const bm = kConfigs[c].tm * 32, bn = kConfigs[c].tn * 128;
        TriangleGrid grid;
        grid.tiles_m = (args.m + bm - 1) / bm, grid.tiles_n = (args.n + bn - 1) / bn;
        grid.bm_log2 = log2_of(bm), grid.bn_log2 = log2_of(bn), grid.shift = args.tri_shift;
        uint32_t const bands = (grid.tiles_m + kTileBand - 1) / kTileBand;
        grid.band_start = scratch.words, grid.list = scratch.words + ((bands + 1 + 1) & ~1u);
        return grid;
    };

    // A triangular grid rarely fills a whole number of rounds of the persistent workgroups, and a last round that
    // is mostly empty costs as much as a full one. When that last round would be less than half full, the tile rows
    // from the top that fill whole rounds go to this tile shape and the rows below them, the narrow end of the
    // triangle, to a second launch with small tiles that spreads them over the whole device.
    if (triangle && (chosen_here || (forced & 0x80)) && config < 4) {
        int slots = 0;
        GemmArgs probe = g;
        hipError_t e = launch_config<T>(probe, stream, triangle, config, &slots);
        if (e != hipSuccess) return e;
        uint64_t const live = tiles_of(g, config);
        uint64_t const rounds = slots > 0 ? live / (uint64_t)slots : 0, rest = slots > 0 ? live % (uint64_t)slots : 0;
        if (rounds >= 1 && rest > 0 && rest * 2 <= (uint64_t)slots) {
            uint32_t const bm = kConfigs[config].tm * 32, bn = kConfigs[config].tn * 128;
            uint32_t const tiles_m = (g.m + bm - 1) / bm, tiles_n = (g.n + bn - 1) / bn;
            uint64_t count = 0;
            uint32_t keep = 0; // tile rows that stay with the large tiles
            for (; keep < tiles_m; ++keep) {
                uint32_t const from = first_live_tile(keep, log2_of(bm), log2_of(bn), g.tri_shift);
                uint64_t const here = from < tiles_n ? tiles_n - from : 0;
                if (count + here > rounds * (uint64_t)slots) break;
                count += here;
            }
            if (keep > 0 && keep < tiles_m) {
                GemmArgs top = g, bottom = g;
                top.m = keep * bm;
                bottom.m = g.m - top.m;
                bottom.a += (uint64_t)top.m * g.a_stride, bottom.c += (uint64_t)top.m * g.c_stride;
                bottom.tri_shift = g.tri_shift + top.m;
                // each launch builds its tile list in its own half of the scratch memory
                size_t const half = triangle->bytes / 2 / 8 * 8;
                TriangleScratch const first_half = {triangle->words, half}, second_half = {triangle->words + half / 4, half};
                int const small = choose(bottom, config + 1);
                TriangleGrids grids;
                grids.grid[0] = grid_of(top, config, first_half), grids.grid[1] = grid_of(bottom, small, second_half);
                hipLaunchKernelGGL(triangle_tiles_kernel, dim3(2), dim3(256), 0, stream, grids);
                if ((e = hipGetLastError()) != hipSuccess) return e;
                if ((e = launch_config<T>(top, stream, &first_half, config)) != hipSuccess) return e;
                return launch_config<T>(bottom, stream, &second_half, small);
            }
        }
    }
    if (triangle && tiles_of(g, config) > 0) {
        TriangleGrids grids;
        grids.grid[0] = grids.grid[1] = grid_of(g, config, *triangle);
        hipLaunchKernelGGL(triangle_tiles_kernel, dim3(1), dim3(256), 0, stream, grids);
        hipError_t const e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return launch_config<T>(g, stream, triangle, config);
}

inline int widest_load(void const *p, size_t stride) {
    uintptr_t const bits = (uintptr_t)p | (uintptr_t)stride;
    if (!(bits & 15)) return 16;
    if (!(bits & 7)) return 8;
    if (!(bits & 3)) return 4;
    if (!(bits & 1)) return 2;
    return 1;
}

#pragma endregion Packed product

} // namespace

#endif // NUMKONG_AMD_DOTS_GFX950_HPP
