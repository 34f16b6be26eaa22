"""Writes tests/golden/*.npz from the reference library (oracle/_ref/libnumkong.so).

Run in the development container, where the reference checkout exists:  python tests/golden/make_golden.py
The fixtures are data only: seeded inputs and what the reference's `_serial` kernels (and `nk_cast_serial`)
returned for them, so that the oracle stays pinned on machines without the reference.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tests import support  # noqa: E402


def main():
    oracle, reference = support.load_oracle(), support.load_reference()
    if reference is None:
        raise SystemExit("build oracle/_ref first: make -C oracle")
    out = support.GOLDEN_DIR
    rng = np.random.default_rng(2024)
    only = sys.argv[1] if len(sys.argv) > 1 else ""  # e.g. "spatials", "symmetric", "narrow" or "wide": rewrite only that family's files
    for dtype in support.FLOAT_DTYPES if only in ("", "cast", "dots") else []:
        codes = np.arange(256 if support.STORAGE[dtype] == np.uint8 else 65536).astype(support.STORAGE[dtype])
        if len(codes) > 256:
            codes = np.concatenate([codes[::61], np.array([0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0xFC00, 0x7E00, 0x8000,
                                                           0x7F7F, 0x7F80, 0xFF80, 0x7FC0], np.uint16)])
        values = np.concatenate([
            rng.standard_normal(1500).astype(np.float32) * np.float32(s) for s in (1e-6, 1e-3, 1, 300, 5e4)
        ] + [np.array([0, -0.0, np.inf, -np.inf, np.nan, 448, 449, 464, 465, 480, 57344, 61439.9, 61440, 65504, 65519.9,
                       65520, 2.0**-9, 2.0**-10, 1.5 * 2.0**-10, 2.0**-16, 2.0**-17, 1.5 * 2.0**-17, 2.0**-24, 2.0**-25,
                       1.0001 * 2.0**-25, 1e-40, 3e38], np.float32)])
        np.savez_compressed(os.path.join(out, f"cast_{dtype}.npz"), dtype=dtype, codes=codes,
                            decoded=reference.cast(codes, dtype, "f32"), values=values,
                            encoded=reference.cast(values, "f32", dtype))
    cases = [("ragged", 13, 21, 77, "default"), ("deep", 6, 10, 2049, "default")]
    for dtype in support.ALL_DTYPES if only in ("", "cast", "dots") else []:
        for tag, m, n, k, kind in cases + ([("fp8", 8, 12, 300, "fp8")] if dtype[0] == "e" else []) + (
                [("lognormal", 8, 12, 300, "lognormal")] if dtype in ("f16", "bf16") else []):
            a = support.random_matrix(oracle, dtype, m, k, rng, kind, pad=3)
            b = support.random_matrix(oracle, dtype, n, k, rng, kind, pad=1)
            if dtype in support.FLOAT_DTYPES and tag == "ragged":  # hand-placed special values
                specials = {"e4m3": [0x7F, 0x7E, 0xFE, 0x01, 0x80], "e5m2": [0x7C, 0xFC, 0x7D, 0x7B, 0x01],
                            "f16": [0x7C00, 0xFC00, 0x7E00, 0x0001, 0x7BFF], "bf16": [0x7F80, 0xFF80, 0x7FC0, 0x0001, 0x7F7F]}[dtype]
                a = a.copy(); b = b.copy()
                for i, code in enumerate(specials):
                    a[i, 5 * i + 1] = code
                    b[2 * i + 1, 3 * i + 2] = code
            a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
            np.savez_compressed(os.path.join(out, f"dots_{dtype}_{tag}.npz"), dtype=dtype, a=a, b=b,
                                c_serial=reference.dots_packed(dtype, a, b),
                                serial_packed_size=reference.packed_size(dtype, n, k))
    # Packed distances: finite inputs, one zero row and one pair of identical rows, serial kernels of the reference.
    rng = np.random.default_rng(2025)
    # (i4: non-negative values only. The reference's distance kernels take their norms from the host-dispatched
    # nk_reduce_moments_i4, whose AVX2 form squares negative values as unsigned ones, so what they return for signed
    # inputs depends on the machine that records the fixture.)
    for dtype in support.DISTANCE_DTYPES if only in ("", "spatials") else []:
        m, n, k = 12, 10, 203
        a = np.ascontiguousarray(support.random_matrix(oracle, dtype, m, k, rng))
        b = np.ascontiguousarray(support.random_matrix(oracle, dtype, n, k, rng))
        if dtype == "i4":
            a, b = a & 0x77, b & 0x77
        if dtype == "e5m2":  # the encoder overflows to Inf; keep the distances finite
            a = np.where((a & 0x7F) > 0x7B, (a & 0x80) | 0x7B, a).astype(a.dtype)
            b = np.where((b & 0x7F) > 0x7B, (b & 0x80) | 0x7B, b).astype(b.dtype)
        a[1] = 0
        b[2] = a[3]
        np.savez_compressed(os.path.join(out, f"spatials_{dtype}.npz"), dtype=dtype, a=a, b=b,
                            angulars_serial=reference.spatials_packed(support.KIND_ANGULARS, dtype, a, b),
                            euclideans_serial=reference.spatials_packed(support.KIND_EUCLIDEANS, dtype, a, b))
    # Symmetric kinds: 45 vectors, the window of rows [5, 39) (off the reference's 4- and 32-row blocks); only the
    # elements the call owns are kept (row in the window, column >= row), the rest of the arrays is zero.
    rng = np.random.default_rng(2026)
    for dtype in support.DISTANCE_DTYPES if only in ("", "symmetric") else []:
        count, depth, row_start, row_count = 45, 203, 5, 34
        vectors = np.ascontiguousarray(support.random_matrix(oracle, dtype, count, depth, rng))
        if dtype == "i4":
            vectors = vectors & 0x77
        if dtype == "e5m2":
            vectors = np.where((vectors & 0x7F) > 0x7B, (vectors & 0x80) | 0x7B, vectors).astype(vectors.dtype)
        vectors[7] = 0
        vectors[30] = vectors[11]
        i, j = np.arange(count)[:, None], np.arange(count)[None, :]
        own = (i >= row_start) & (i < row_start + row_count) & (j >= i)
        results = {metric: np.where(own, reference.symmetric(metric, dtype, vectors, row_start, row_count), 0)
                   for metric in ("dots", "angular", "euclidean")}
        np.savez_compressed(os.path.join(out, f"symmetric_{dtype}.npz"), dtype=dtype, vectors=vectors, row_start=row_start,
                            row_count=row_count, dots_serial=results["dots"].astype(support.OUTPUT[dtype]),
                            angulars_serial=results["angular"].astype(np.float32),
                            euclideans_serial=results["euclidean"].astype(np.float32))
    # The narrow types (dot-product kinds only): a ragged packed product with an odd depth, all 256 decodings of the
    # 6-bit floats, and a symmetric window; owned elements only, zeros elsewhere.
    rng = np.random.default_rng(2027)
    for dtype in support.NARROW_DTYPES if only in ("", "narrow") else []:
        a = np.ascontiguousarray(support.random_matrix(oracle, dtype, 13, 77, rng, pad=3))
        b = np.ascontiguousarray(support.random_matrix(oracle, dtype, 21, 77, rng, pad=1))
        count, depth, row_start, row_count = 45, 202, 5, 34
        vectors = np.ascontiguousarray(support.random_matrix(oracle, dtype, count, depth, rng))
        i, j = np.arange(count)[:, None], np.arange(count)[None, :]
        own = (i >= row_start) & (i < row_start + row_count) & (j >= i)
        extra = {"decoded": reference.cast(np.arange(256, dtype=np.uint8), dtype, "f32")} if dtype in support.NARROW_FLOAT_DTYPES else {}
        np.savez_compressed(os.path.join(out, f"narrow_{dtype}.npz"), dtype=dtype, a=a, b=b,
                            c_serial=reference.dots_packed(dtype, a, b), vectors=vectors, row_start=row_start,
                            row_count=row_count,
                            symmetric_serial=np.where(own, reference.symmetric("dots", dtype, vectors, row_start, row_count), 0)
                            .astype(support.OUTPUT[dtype]), **extra)
    # The wide types (f64 results): a ragged packed product with an odd depth and a symmetric window, lognormal inputs.
    rng = np.random.default_rng(2028)
    for dtype in support.WIDE_DTYPES if only in ("", "wide") else []:
        a = np.ascontiguousarray(support.random_matrix(oracle, dtype, 13, 77, rng, "lognormal", pad=3))
        b = np.ascontiguousarray(support.random_matrix(oracle, dtype, 21, 77, rng, "lognormal", pad=1))
        count, depth, row_start, row_count = 45, 203, 5, 34
        vectors = np.ascontiguousarray(support.random_matrix(oracle, dtype, count, depth, rng, "lognormal"))
        i, j = np.arange(count)[:, None], np.arange(count)[None, :]
        own = (i >= row_start) & (i < row_start + row_count) & (j >= i)
        np.savez_compressed(os.path.join(out, f"wide_{dtype}.npz"), dtype=dtype, a=a, b=b,
                            c_serial=reference.dots_packed(dtype, a, b), vectors=vectors, row_start=row_start,
                            row_count=row_count,
                            symmetric_serial=np.where(own, reference.symmetric("dots", dtype, vectors, row_start, row_count), 0.0),
                            angulars_serial=reference.spatials_packed(support.KIND_ANGULARS, dtype, a, b),
                            euclideans_serial=reference.spatials_packed(support.KIND_EUCLIDEANS, dtype, a, b),
                            angulars_symmetric_serial=np.where(own, reference.symmetric("angular", dtype, vectors, row_start, row_count), 0.0),
                            euclideans_symmetric_serial=np.where(own, reference.symmetric("euclidean", dtype, vectors, row_start, row_count), 0.0))
    print("wrote", len(os.listdir(out)) - 1, "fixtures to", out)


if __name__ == "__main__":
    main()
