"""Shared helpers for the tests: ctypes views of the oracle and of the reference library, input makers.

The oracle (oracle/liboracle.so) and the reference build (oracle/_ref/libnumkong.so) are loaded here and
only here; the product under test is numkong_amd/lib/libnumkong_amd.so.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_PATH = os.path.join(ROOT, "oracle", "liboracle.so")
REFERENCE_PATH = os.path.join(ROOT, "oracle", "_ref", "libnumkong.so")
GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")

# nk_dtype_t codes (reference: include/numkong/types.h:923-952)
CODES = {"i8": 1 << 2, "u8": 1 << 6, "f32": 1 << 11, "f16": 1 << 12, "bf16": 1 << 13, "e4m3": 1 << 14, "e5m2": 1 << 15,
         "i4": 1 << 16, "u4": 1 << 17, "e2m3": 1 << 18, "e3m2": 1 << 19, "u1": 1 << 1, "f64": 1 << 10}
STORAGE = {"i8": np.int8, "u8": np.uint8, "f16": np.uint16, "bf16": np.uint16, "e4m3": np.uint8, "e5m2": np.uint8,
           "i4": np.uint8, "u4": np.uint8, "e2m3": np.uint8, "e3m2": np.uint8, "u1": np.uint8,
           "f32": np.float32, "f64": np.float64}
OUTPUT = {"i8": np.int32, "u8": np.uint32, "f16": np.float32, "bf16": np.float32, "e4m3": np.float32, "e5m2": np.float32,
          "i4": np.int32, "u4": np.uint32, "e2m3": np.float32, "e3m2": np.float32, "u1": np.uint32,
          "f32": np.float64, "f64": np.float64}
FLOAT_DTYPES = ("bf16", "f16", "e4m3", "e5m2")
ALL_DTYPES = ("i8", "u8") + FLOAT_DTYPES  # the six types of the headline path
# the narrow types: 6-bit floats (one per byte), 4-bit integers (two per byte), bits (eight; dot-product kinds only)
NARROW_FLOAT_DTYPES = ("e2m3", "e3m2")
NARROW_INT_DTYPES = ("i4", "u4", "u1")
NARROW_DTYPES = NARROW_FLOAT_DTYPES + NARROW_INT_DTYPES
DIMENSIONS_PER_VALUE = {"i4": 2, "u4": 2, "u1": 8}
WIDE_DTYPES = ("f32", "f64")  # f64 results, for the dot products and for the distances
DISTANCE_DTYPES = ALL_DTYPES + ("e2m3", "e3m2", "i4", "u4")  # the types with the distance kinds (f32 results), packed and symmetric
# ... and f32 and f64, whose distances are f64
DISTANCE_OUTPUT = {**{t: np.float32 for t in DISTANCE_DTYPES}, "f32": np.float64, "f64": np.float64}
INTEGER_DTYPES = ("i8", "u8", "i4", "u4", "u1")  # bit-exact everywhere
# The reference's distance kernels take their sums of squares from the host-dispatched nk_reduce_moments_<T>, and the
# AVX2 one of i4 squares negative values as if they were unsigned (reduce/haswell.h:3629-3633), so for i4 only the
# serial kernels (restated by the oracle, nk_reduce_moments_i4_serial) can stand next to the f64 truth.
DISPATCHED_DISTANCES_UNUSABLE = ("i4",)


def depth_of(dtype: str, matrix: np.ndarray) -> int:
    """Dimensions of a row: the stored values times the dimensions each holds (two for the 4-bit types)."""
    return matrix.shape[1] * DIMENSIONS_PER_VALUE.get(dtype, 1)
KIND_SIZE, KIND_PACK, KIND_PACKED = ord("P"), ord("Q"), ord("G")
KIND_ANGULARS, KIND_EUCLIDEANS = ord("N"), ord("E")  # packed distances: same prototype as the packed product
# symmetric kinds (vectors, count, depth, stride, result, result_stride, row_start, row_count), by metric
SYMMETRIC_KINDS = {"dots": ord("y"), "angular": ord("n"), "euclidean": ord("D")}
SYMMETRIC_METRICS = {"dots": 0, "angular": 1, "euclidean": 2}
METRICS = {"angular": 1, "euclidean": 2}
METRIC_KINDS = {"angular": KIND_ANGULARS, "euclidean": KIND_EUCLIDEANS}
CAP_SERIAL = 1

_sz, _vp, _i32 = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int


def _ptr(array: np.ndarray) -> int:
    return array.ctypes.data


class Oracle:
    """This repository's CPU restatement (oracle/dots_oracle.c)."""

    def __init__(self, lib: ctypes.CDLL):
        self.lib = lib
        lib.nko_decode.argtypes = [_i32, _vp, _sz, _vp]
        lib.nko_encode.argtypes = [_i32, _vp, _sz, _vp]
        lib.nko_serial_packed_size.restype = _sz
        lib.nko_serial_packed_size.argtypes = [_i32, _sz, _sz]
        lib.nko_serial_pack.argtypes = [_i32, _vp, _sz, _sz, _sz, _vp]
        lib.nko_serial_packed.argtypes = [_i32, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz]
        lib.nko_dots_f64.argtypes = [_i32, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz]
        lib.nko_row_sumsq.argtypes = [_i32, _vp, _sz, _sz, _sz, _vp]
        lib.nko_row_sumsq_wide.argtypes = [_i32, _vp, _sz, _sz, _sz, _vp]
        lib.nko_serial_spatials.argtypes = [_i32, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz]
        lib.nko_spatials_f64.argtypes = [_i32, _i32, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz]
        lib.nko_serial_symmetric.argtypes = [_i32, _i32, _vp, _sz, _sz, _sz, _vp, _sz, _sz, _sz]
        lib.nko_serial_dots.argtypes = [_i32, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz]

    def decode(self, dtype: str, codes: np.ndarray) -> np.ndarray:
        codes = np.ascontiguousarray(codes, dtype=STORAGE[dtype])
        per = DIMENSIONS_PER_VALUE.get(dtype, 1)
        out = np.empty(codes.shape[:-1] + (codes.shape[-1] * per,), dtype=np.float32)
        self.lib.nko_decode(CODES[dtype], _ptr(codes), out.size, _ptr(out))
        return out

    def encode(self, dtype: str, values: np.ndarray) -> np.ndarray:
        values = np.ascontiguousarray(values, dtype=np.float32)
        out = np.empty(values.shape, dtype=STORAGE[dtype])
        self.lib.nko_encode(CODES[dtype], _ptr(values), values.size, _ptr(out))
        return out

    def packed_size(self, dtype: str, n: int, k: int) -> int:
        return int(self.lib.nko_serial_packed_size(CODES[dtype], n, k))

    def pack(self, dtype: str, b: np.ndarray) -> np.ndarray:
        n, k = b.shape
        packed = np.zeros(self.packed_size(dtype, n, k), dtype=np.uint8)
        self.lib.nko_serial_pack(CODES[dtype], _ptr(b), n, k, b.strides[0], _ptr(packed))
        return packed

    def dots_packed(self, dtype: str, a: np.ndarray, b: np.ndarray) -> np.ndarray:
        """C = A @ B.T with the serial backend's rounding (pack + packed product; the narrow types, whose serial image
        is not restated, straight from the unpacked rows)."""
        m, k = a.shape[0], depth_of(dtype, a)
        n = b.shape[0]
        c = np.empty((m, n), dtype=OUTPUT[dtype])
        if dtype in NARROW_DTYPES or dtype in WIDE_DTYPES:
            self.lib.nko_serial_dots(CODES[dtype], _ptr(a), _ptr(b), _ptr(c), m, n, k, a.strides[0], b.strides[0], c.strides[0])
            return c
        packed = self.pack(dtype, b)
        self.lib.nko_serial_packed(CODES[dtype], _ptr(a), _ptr(packed), _ptr(c), m, n, k, a.strides[0], c.strides[0])
        return c

    def row_sumsq(self, dtype: str, x: np.ndarray) -> np.ndarray:
        """Per-row sum of squares as the serial backend computes it: u32 for the integer types, f64 for f32 and f64
        inputs, f32 otherwise."""
        if dtype in WIDE_DTYPES:
            wide = np.empty(x.shape[0], dtype=np.float64)
            self.lib.nko_row_sumsq_wide(CODES[dtype], _ptr(x), x.shape[0], x.shape[1], x.strides[0], _ptr(wide))
            return wide
        out = np.empty(x.shape[0], dtype=np.uint32)
        self.lib.nko_row_sumsq(CODES[dtype], _ptr(x), x.shape[0], depth_of(dtype, x), x.strides[0], _ptr(out))
        return out if dtype in INTEGER_DTYPES else out.view(np.float32)

    def spatials_packed(self, metric: str, dtype: str, a: np.ndarray, b: np.ndarray) -> np.ndarray:
        """`nk_angulars_packed_<dtype>_serial` ("angular") / `nk_euclideans_packed_<dtype>_serial` ("euclidean")."""
        m, k = a.shape[0], depth_of(dtype, a)
        n = b.shape[0]
        c = np.empty((m, n), dtype=DISTANCE_OUTPUT[dtype])
        self.lib.nko_serial_spatials(CODES[dtype], METRICS[metric], _ptr(a), _ptr(b), _ptr(c), m, n, k, a.strides[0],
                                     b.strides[0], c.strides[0])
        return c

    def spatials_truth(self, metric: str, dtype: str, a: np.ndarray, b: np.ndarray) -> np.ndarray:
        """The distances from f64 dots and f64 norms."""
        m, k = a.shape[0], depth_of(dtype, a)
        n = b.shape[0]
        c = np.empty((m, n), dtype=np.float64)
        self.lib.nko_spatials_f64(CODES[dtype], METRICS[metric], _ptr(a), _ptr(b), _ptr(c), m, n, k, a.strides[0],
                                  b.strides[0])
        return c

    def symmetric(self, metric: str, dtype: str, vectors: np.ndarray, row_start: int = 0, row_count=None,
                  out: np.ndarray = None) -> np.ndarray:
        """`nk_{dots,angulars,euclideans}_symmetric_<dtype>_serial` into `out` (count x count; fresh and zeroed when
        not given): only result[i][j], i in the row window, j >= i, is written."""
        count, depth = vectors.shape[0], depth_of(dtype, vectors)
        if out is None:
            out = np.zeros((count, count), dtype=OUTPUT[dtype] if metric == "dots" else DISTANCE_OUTPUT[dtype])
        rows = count - row_start if row_count is None else row_count
        self.lib.nko_serial_symmetric(CODES[dtype], SYMMETRIC_METRICS[metric], _ptr(vectors), count, depth,
                                      vectors.strides[0], _ptr(out), out.strides[0], row_start, rows)
        return out

    def truth(self, dtype: str, a: np.ndarray, b: np.ndarray):
        """(f64 ground truth, sum |a*b|) as the reference's own tests compute it."""
        m, k = a.shape[0], depth_of(dtype, a)
        n = b.shape[0]
        c = np.empty((m, n), dtype=np.float64)
        mag = np.empty((m, n), dtype=np.float64)
        self.lib.nko_dots_f64(CODES[dtype], _ptr(a), _ptr(b), _ptr(c), _ptr(mag), m, n, k, a.strides[0], b.strides[0])
        return c, mag


class Reference:
    """The reference library built from its own sources; kernels are looked up like its bindings do."""

    def __init__(self, lib: ctypes.CDLL):
        self.lib = lib
        lib.nk_find_kernel_punned.argtypes = [_i32, _i32, ctypes.c_uint64, ctypes.POINTER(_vp), ctypes.POINTER(ctypes.c_uint64)]
        lib.nk_capabilities.restype = ctypes.c_uint64
        lib.nk_cast.argtypes = [_vp, _i32, _sz, _vp, _i32]
        lib.nk_configure_thread.argtypes = [ctypes.c_uint64]
        self.capabilities = int(lib.nk_capabilities())
        lib.nk_configure_thread(self.capabilities)

    def kernel(self, kind: int, dtype: str, viable: int):
        fn, cap = _vp(), ctypes.c_uint64()
        self.lib.nk_find_kernel_punned(kind, CODES[dtype], viable, ctypes.byref(fn), ctypes.byref(cap))
        if not fn.value or not cap.value:
            raise RuntimeError(f"reference has no kernel kind={chr(kind)} dtype={dtype} viable={viable:#x}")
        proto = {
            KIND_SIZE: ctypes.CFUNCTYPE(_sz, _sz, _sz),
            KIND_PACK: ctypes.CFUNCTYPE(None, _vp, _sz, _sz, _sz, _vp),
            KIND_PACKED: ctypes.CFUNCTYPE(None, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz),
            KIND_ANGULARS: ctypes.CFUNCTYPE(None, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz),
            KIND_EUCLIDEANS: ctypes.CFUNCTYPE(None, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz),
            SYMMETRIC_KINDS["dots"]: ctypes.CFUNCTYPE(None, _vp, _sz, _sz, _sz, _vp, _sz, _sz, _sz),
            SYMMETRIC_KINDS["angular"]: ctypes.CFUNCTYPE(None, _vp, _sz, _sz, _sz, _vp, _sz, _sz, _sz),
            SYMMETRIC_KINDS["euclidean"]: ctypes.CFUNCTYPE(None, _vp, _sz, _sz, _sz, _vp, _sz, _sz, _sz),
        }[kind]
        return proto(fn.value), int(cap.value)

    def cast(self, values: np.ndarray, from_dtype: str, to_dtype: str, viable: int = CAP_SERIAL) -> np.ndarray:
        """`nk_cast_serial` by default: the SIMD casts differ from it on NaN payloads and e5m2 overflow."""
        src_np = np.float32 if from_dtype == "f32" else STORAGE[from_dtype]
        dst_np = np.float32 if to_dtype == "f32" else STORAGE[to_dtype]
        values = np.ascontiguousarray(values, dtype=src_np)
        out = np.empty(values.shape, dtype=dst_np)
        fn, cap = _vp(), ctypes.c_uint64()
        self.lib.nk_find_kernel_punned(ord("-"), 0, viable, ctypes.byref(fn), ctypes.byref(cap))
        if not fn.value or not cap.value:
            raise RuntimeError("reference has no cast kernel for these capabilities")
        cast = ctypes.CFUNCTYPE(None, _vp, _i32, _sz, _vp, _i32)(fn.value)
        cast(_ptr(values), CODES[from_dtype], values.size, _ptr(out), CODES[to_dtype])
        return out

    def packed_size(self, dtype: str, n: int, k: int, viable: int = CAP_SERIAL) -> int:
        return int(self.kernel(KIND_SIZE, dtype, viable)[0](n, k))

    def pack(self, dtype: str, b: np.ndarray, viable: int = CAP_SERIAL) -> np.ndarray:
        n, k = b.shape[0], depth_of(dtype, b)
        packed = np.zeros(self.packed_size(dtype, n, k, viable) + 64, dtype=np.uint8)
        self.kernel(KIND_PACK, dtype, viable)[0](_ptr(b), n, k, b.strides[0], _ptr(packed))
        return packed

    def dots_packed(self, dtype: str, a: np.ndarray, b: np.ndarray, viable: int = CAP_SERIAL) -> np.ndarray:
        m, k = a.shape[0], depth_of(dtype, a)
        n = b.shape[0]
        packed = self.pack(dtype, b, viable)
        c = np.empty((m, n), dtype=OUTPUT[dtype])
        self.kernel(KIND_PACKED, dtype, viable)[0](_ptr(a), _ptr(packed), _ptr(c), m, n, k, a.strides[0], c.strides[0])
        return c

    def spatials_packed(self, kind: int, dtype: str, a: np.ndarray, b: np.ndarray, viable: int = CAP_SERIAL) -> np.ndarray:
        """`nk_angulars_packed_<dtype>` / `nk_euclideans_packed_<dtype>` of the chosen backend, f32 results."""
        m, k = a.shape[0], depth_of(dtype, a)
        n = b.shape[0]
        packed = self.pack(dtype, b, viable)
        c = np.empty((m, n), dtype=DISTANCE_OUTPUT[dtype])
        self.kernel(kind, dtype, viable)[0](_ptr(a), _ptr(packed), _ptr(c), m, n, k, a.strides[0], c.strides[0])
        return c

    def symmetric(self, metric: str, dtype: str, vectors: np.ndarray, row_start: int = 0, row_count=None,
                  out: np.ndarray = None, viable: int = CAP_SERIAL) -> np.ndarray:
        """The chosen backend's symmetric kernel into `out` (count x count; fresh and zeroed when not given)."""
        count, depth = vectors.shape[0], depth_of(dtype, vectors)
        if out is None:
            out = np.zeros((count, count), dtype=OUTPUT[dtype] if metric == "dots" else DISTANCE_OUTPUT[dtype])
        rows = count - row_start if row_count is None else row_count
        self.kernel(SYMMETRIC_KINDS[metric], dtype, viable)[0](_ptr(vectors), count, depth, vectors.strides[0], _ptr(out),
                                                               out.strides[0], row_start, rows)
        return out


def wide_distances_agree(metric, mine, ref, norms, ulps=16):
    """f64 distances from the same f64 dot products: what differs between two evaluations is the summation order of the
    sums of squares (a rounding or two of f64) and the last bits of the square root. Angular is 1 - x with |x| <= 1, so
    the difference is absolute; euclidean is a root of a difference that can cancel to a residue of the norms' size."""
    u = 2.0 ** -53
    if metric == "angular":
        return bool((np.abs(mine - ref) <= ulps * u).all())
    return bool(((np.abs(mine - ref) <= ulps * u * np.abs(ref)) | (np.abs(mine * mine - ref * ref) <= ulps * u * norms)).all())


def ulp_distance_f32(actual: np.ndarray, expected: np.ndarray) -> np.ndarray:
    """Units in the last place between two f32 arrays, the way the reference's tests count them (test/test.hpp:400-441):
    the distance between the bit patterns on the number line, the two zeros one step apart from nothing."""
    def ordered(x):
        bits = np.ascontiguousarray(x, dtype=np.float32).view(np.int32).astype(np.int64)
        return np.where(bits < 0, -(bits & 0x7FFFFFFF), bits)
    return np.abs(ordered(actual) - ordered(expected))


ULP_TABLE_HEADER = (f"{'kernel':<40s} {'max abs err':>12s} {'max rel err':>12s} {'mean rel err':>12s} {'mean ulp':>10s} {'max ulp':>12s} "
                    f"{'exact':>10s}")


def ulp_table_row(name: str, actual: np.ndarray, truth: np.ndarray) -> str:
    """One row of the reference's accuracy table for a mixed-precision reduction (test/test.hpp:491-514): largest
    absolute and relative error against the f64 truth rounded to f32, mean and largest distance in units in the last
    place, outputs that match exactly. Pairs with a NaN or an infinity on either side are skipped, as there."""
    expected = truth.astype(np.float32)
    use = np.isfinite(actual) & np.isfinite(expected)
    got, want = actual[use].astype(np.float32), expected[use]
    if not got.size:
        return f"{name:<40s} (no finite outputs)"
    absolute = np.abs(got.astype(np.float64) - want.astype(np.float64))
    relative = np.where(want != 0, absolute / np.maximum(np.abs(want.astype(np.float64)), 1e-300), absolute)
    ulps = ulp_distance_f32(got, want)
    return (f"{name:<40s} {absolute.max():12.2e} {relative.max():12.2e} {relative.mean():12.2e} {ulps.mean():10.1f} "
            f"{int(ulps.max()):12d} {int((ulps == 0).sum()):10d}")


def load_oracle() -> Oracle:
    if not os.path.exists(ORACLE_PATH):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), os.path.join(ROOT, "oracle", "liboracle.so")])
    return Oracle(ctypes.CDLL(ORACLE_PATH))


def load_reference():
    if not os.path.exists(REFERENCE_PATH):
        return None
    return Reference(ctypes.CDLL(REFERENCE_PATH))


def random_matrix(oracle: Oracle, dtype: str, rows: int, cols: int, rng: np.random.Generator, kind: str = "default",
                  pad: int = 0) -> np.ndarray:
    """Seeded inputs in the storage type of `dtype`; `pad` extra elements per row make strides non-trivial.

    kinds: "default"  ints uniform over the full range, floats N(0,1)
           "lognormal" floats +-exp(N(0,1))   (reference tests' family, test/test.hpp:204)
           "fp8"       N(0,1) scaled to half of the largest finite value, 1 % exact zeros
    """
    shape = (rows, cols + pad)
    if dtype in DIMENSIONS_PER_VALUE:  # `cols` dimensions, two or eight to a byte: every byte value, all of it random
        per = DIMENSIONS_PER_VALUE[dtype]
        packed = rng.integers(0, 256, size=(rows, (cols + per - 1) // per + pad), dtype=np.uint8)
        return packed[:, : (cols + per - 1) // per] if pad else packed
    if dtype in NARROW_FLOAT_DTYPES and kind == "default":  # every 6-bit code is a finite number; the top two bits are ignored
        full = rng.integers(0, 256, size=shape, dtype=np.uint8)
        return full[:, :cols] if pad else full
    if dtype in WIDE_DTYPES:  # N(0,1), or the reference tests' lognormal family with random signs
        z = rng.standard_normal(shape)
        if kind == "lognormal":
            z = np.exp(z) * rng.choice(np.array([-1.0, 1.0]), size=shape)
        full = z.astype(STORAGE[dtype])
        return full[:, :cols] if pad else full
    if dtype == "i8":
        full = rng.integers(-128, 128, size=shape, dtype=np.int8)
    elif dtype == "u8":
        full = rng.integers(0, 256, size=shape, dtype=np.uint8)
    else:
        z = rng.standard_normal(shape).astype(np.float32)
        if kind == "lognormal":
            z = (np.exp(z) * rng.choice(np.array([-1.0, 1.0], dtype=np.float32), size=shape)).astype(np.float32)
        elif kind == "fp8":
            z = z * np.float32(0.5 * (448.0 if dtype == "e4m3" else 57344.0))
        full = oracle.encode(dtype, z)
        if kind == "fp8":
            full[rng.random(shape) < 0.01] = 0
    return full[:, :cols] if pad else full
