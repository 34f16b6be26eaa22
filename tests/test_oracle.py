"""Pins the CPU oracle (oracle/dots_oracle.c) before anything is compared with it.

Checks, in the order of strength:
  * against the reference library compiled from its own sources (oracle/_ref), when it was built:
    `nk_cast_serial` for all conversions, `nk_dots_*_serial` for sizes, packed bytes and products, bit for bit;
  * against vectors committed under tests/golden (made from that library by tests/golden/make_golden.py),
    so the same facts hold where the reference is absent;
  * against independent library routines: torch's float8_e4m3fn / float8_e5m2 / float16 / bfloat16 decoders;
  * against what arithmetic fixes: the 428-byte packed-size example (64 + 7*48 + 7*4), exact integer
    products from numpy int64, powers of two, f64 matmul of decoded inputs.
NaN payloads are never compared: the reference's own cast backends disagree on them.
"""
import ctypes
import os

import numpy as np
import pytest

from tests import support
from tests.support import ALL_DTYPES, DISTANCE_DTYPES, FLOAT_DTYPES, INTEGER_DTYPES, NARROW_DTYPES, NARROW_FLOAT_DTYPES, STORAGE, WIDE_DTYPES


def same_floats(x, y):
    x, y = np.asarray(x), np.asarray(y)
    nan = np.isnan(x)
    return np.array_equal(nan, np.isnan(y)) and np.array_equal(x[~nan].view(np.uint32), y[~nan].view(np.uint32))


def all_codes(dtype):
    return np.arange(256 if STORAGE[dtype] == np.uint8 else 65536).astype(STORAGE[dtype])


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_decode_matches_torch(oracle, dtype):
    import torch

    torch_dtype = {"bf16": torch.bfloat16, "f16": torch.float16, "e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}[dtype]
    codes = all_codes(dtype)
    view = torch.from_numpy(codes.view(np.int16) if codes.itemsize == 2 else codes).view(torch_dtype)
    assert same_floats(oracle.decode(dtype, codes), view.to(torch.float32).numpy())


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_decode_closed_form(oracle, dtype):
    """value = (-1)^s * 2^(e-bias) * (1 + m / 2^mbits), subnormals m * 2^(1-bias-mbits), in Python floats."""
    ebits, mbits, bias = {"bf16": (8, 7, 127), "f16": (5, 10, 15), "e4m3": (4, 3, 7), "e5m2": (5, 2, 15)}[dtype]
    codes = all_codes(dtype)
    got = oracle.decode(dtype, codes)
    for code in codes[:: max(1, len(codes) // 4096)].tolist() + [0, 1, len(codes) // 2 - 1, len(codes) - 1]:
        s, e, m = code >> (ebits + mbits), (code >> mbits) & ((1 << ebits) - 1), code & ((1 << mbits) - 1)
        if e == (1 << ebits) - 1 and dtype != "e4m3":
            expected = float("nan") if m else float("inf")
        elif dtype == "e4m3" and e == 15 and m == 7:
            expected = float("nan")
        elif e == 0:
            expected = m * 2.0 ** (1 - bias - mbits)
        else:
            expected = (1 + m / 2.0**mbits) * 2.0 ** (e - bias)
        expected = -expected if s else expected
        assert (np.isnan(got[code]) and np.isnan(expected)) or float(got[code]) == expected, hex(code)


def _encode_probe_values(oracle, dtype):
    rng = np.random.default_rng(1)
    scales = [1e-8, 1e-6, 1e-3, 1, 100, 1e4, 1e6]
    values = [rng.standard_normal(20000).astype(np.float32) * np.float32(s) for s in scales]
    values.append(np.array([0, -0.0, np.inf, -np.inf, np.nan, 448, 449, 464, 465, 480, 57344, 61439.9, 61440, 65504,
                            65519.9, 65520, 2.0**-9, 2.0**-10, 1.5 * 2.0**-10, 2.0**-16, 2.0**-17, 1.5 * 2.0**-17,
                            2.0**-24, 2.0**-25, 1.0001 * 2.0**-25, 1e-40, 3e38], dtype=np.float32))
    grid = np.sort(oracle.decode(dtype, all_codes(dtype)[: len(all_codes(dtype)) // 2]))
    grid = grid[np.isfinite(grid)]
    if len(grid) > 4096:
        grid = grid[:: len(grid) // 4096]
    mids = ((grid[:-1].astype(np.float64) + grid[1:]) / 2).astype(np.float32)
    edge = np.concatenate([grid, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf))])
    values += [edge, -edge]
    return np.concatenate(values)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_conversions_match_reference_serial(oracle, reference, dtype):
    codes = all_codes(dtype)
    assert same_floats(oracle.decode(dtype, codes), reference.cast(codes, dtype, "f32"))
    values = _encode_probe_values(oracle, dtype)
    assert np.array_equal(oracle.encode(dtype, values), reference.cast(values, "f32", dtype))


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_encode_round_trip_and_ties(oracle, dtype):
    """Every finite code encodes back to itself; exact midpoints go to the even neighbour; policies on overflow."""
    codes = all_codes(dtype)
    values = oracle.decode(dtype, codes)
    finite = np.isfinite(values)
    assert np.array_equal(oracle.encode(dtype, values[finite]), codes[finite])
    half = codes[: len(codes) // 2]
    grid = oracle.decode(dtype, half)
    keep = np.isfinite(grid)
    grid, half = grid[keep], half[keep]
    mids = (grid[:-1].astype(np.float64) + grid[1:].astype(np.float64)) / 2
    exact = mids.astype(np.float32).astype(np.float64) == mids
    encoded = oracle.encode(dtype, mids[exact].astype(np.float32))
    lower, upper = half[:-1][exact], half[1:][exact]
    assert np.array_equal(encoded, np.where(lower % 2 == 0, lower, upper))
    big = np.array([1e30, -1e30, np.inf, -np.inf], dtype=np.float32)
    expected = {"e4m3": [0x7E, 0xFE, 0x7E, 0xFE], "e5m2": [0x7C, 0xFC, 0x7C, 0xFC], "f16": [0x7C00, 0xFC00, 0x7C00, 0xFC00],
                "bf16": [0x7149, 0xF149, 0x7F80, 0xFF80]}[dtype]  # bf16: 1e30 is finite in bf16
    got = oracle.encode(dtype, big).tolist()
    if dtype == "bf16":
        assert got[2:] == expected[2:] and abs(float(oracle.decode(dtype, np.array(got[:1], np.uint16))[0]) / 1e30 - 1) < 1e-2
    else:
        assert got == expected
    assert np.isnan(oracle.decode(dtype, oracle.encode(dtype, np.array([np.nan], np.float32)))).all()


def test_packed_size_known_answers(oracle):
    # reference layout: 64 + n * padded_depth * width + n * 4; depth padded to 16 (i8), 8 (bf16), 4 (f16 as f32)
    assert oracle.packed_size("i8", 7, 37) == 64 + 7 * 48 + 7 * 4 == 428
    assert oracle.packed_size("i8", 2048, 2048) == 64 + 2048 * (2048 + 16) + 2048 * 4  # power-of-two stride is broken up
    assert oracle.packed_size("bf16", 4096, 4096) == 64 + 4096 * (4096 + 8) * 2 + 4096 * 4
    assert oracle.packed_size("f16", 3, 5) == 64 + 3 * (8 + 4) * 4 + 3 * 4  # 5 -> 8 f32 values = 32 B, a power of two -> +4 values
    assert oracle.packed_size("e4m3", 10, 1000) == 64 + 10 * 1008 + 40


SHAPES = [(5, 7, 37, 0, 0), (33, 29, 1000, 13, 7), (64, 64, 64, 0, 0), (1, 1, 1, 0, 0), (16, 130, 63, 3, 0),
          (37, 48, 2049, 0, 5), (8, 8, 4096, 0, 0)]


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_serial_layout_and_product_match_reference(oracle, reference, dtype):
    rng = np.random.default_rng(7)
    for n, k in [(1, 1), (7, 37), (128, 1536), (5, 64), (3, 128), (9, 4096), (4, 2048), (2, 1000), (17, 8192)]:
        assert oracle.packed_size(dtype, n, k) == reference.packed_size(dtype, n, k)
    kinds = ["default"] if dtype in ("i8", "u8") else ["default", "lognormal"] + (["fp8"] if dtype[0] == "e" else [])
    for m, n, k, pad_a, pad_b in SHAPES:
        for kind in kinds:
            a = support.random_matrix(oracle, dtype, m, k, rng, kind, pad_a)
            b = support.random_matrix(oracle, dtype, n, k, rng, kind, pad_b)
            mine, theirs = oracle.pack(dtype, b), reference.pack(dtype, b)
            padded = int(mine[8:12].view(np.uint32)[0])
            body = 64 + n * padded * (4 if dtype == "f16" else a.itemsize)
            assert np.array_equal(mine[:body], theirs[:body])
            if dtype in ("i8", "u8"):
                assert np.array_equal(mine, theirs[: len(mine)])  # integer norms too: every backend's are exact
            else:
                # The float norms behind the rows come from the reduce kernel in the reference's dispatch table
                # (dots/serial.h:124-143): with the table set to the serial kernels the whole image is pinned.
                reference.lib.nk_dispatch_table_update(ctypes.c_uint64(support.CAP_SERIAL))
                try:
                    assert np.array_equal(mine, reference.pack(dtype, b)[: len(mine)])
                finally:
                    reference.lib.nk_dispatch_table_update(ctypes.c_uint64(reference.capabilities))
            assert same_floats(oracle.dots_packed(dtype, a, b).view(np.float32), reference.dots_packed(dtype, a, b).view(np.float32))


def finite_inputs(oracle, dtype, rows, cols, rng):
    """Seeded rows without Inf/NaN codes (the e5m2 encoder overflows to Inf; distances are gated on finite inputs)."""
    x = support.random_matrix(oracle, dtype, rows, cols, rng)
    if dtype == "e5m2":
        x = np.where((x & 0x7F) > 0x7B, (x & 0x80) | 0x7B, x).astype(x.dtype)
    return x


def reference_distance_inputs(oracle, dtype, rows, cols, rng):
    """Inputs on which the reference's distance kernels can serve as the pin. They take their sums of squares from the
    host-dispatched nk_reduce_moments_<T> (dots/serial.h:165-170), and the AVX2 one of i4 squares a nibble as if it
    were unsigned (reduce/haswell.h:3629-3633: a table of 0..15 squared behind signed values, so -5 counts as 121),
    unlike nk_reduce_moments_i4_serial, which the oracle follows and test_row_sums_of_squares pins bit for bit with
    negative values. So i4 is compared on non-negative values here, where every backend agrees, and on signed values
    against the f64 truth in test_four_bit_distances_follow_the_serial_moments."""
    x = finite_inputs(oracle, dtype, rows, cols, rng)
    return x & 0x77 if dtype == "i4" else x


@pytest.mark.parametrize("dtype", DISTANCE_DTYPES)
def test_row_sums_of_squares_match_reference_serial(oracle, reference, dtype):
    """nk_reduce_moments_<T>_serial: exact integers (the 4-bit types count both halves of every byte they touch),
    Neumaier-compensated f32 for the float types, bit for bit."""
    if reference is None:
        pytest.skip("reference build not present")
    rng = np.random.default_rng(21)
    moments, _ = reference_moments(reference, dtype)
    for rows, cols in [(3, 1), (5, 37), (4, 1000), (2, 8192)]:
        x = finite_inputs(oracle, dtype, rows, cols, rng)
        mine = oracle.row_sumsq(dtype, x)
        for i in range(rows):
            assert mine[i:i + 1].view(np.uint32)[0] == moments(x[i]), (dtype, rows, cols, i)


def reference_moments(reference, dtype):
    import ctypes

    fn, cap = ctypes.c_void_p(), ctypes.c_uint64()
    reference.lib.nk_find_kernel_punned(ord("R"), support.CODES[dtype], support.CAP_SERIAL, ctypes.byref(fn), ctypes.byref(cap))
    assert fn.value and cap.value
    call = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p)(fn.value)

    def sumsq_bits(row):
        row = np.ascontiguousarray(row)
        total, squares = np.zeros(1, np.uint64), np.zeros(1, np.uint64)
        call(row.ctypes.data, row.size * support.DIMENSIONS_PER_VALUE.get(dtype, 1), row.itemsize, total.ctypes.data,
             squares.ctypes.data)
        # integers: u64 sum of squares, truncated like dots/serial.h:154-164; floats: the f32 in the low half
        return int(squares[0]) & 0xFFFFFFFF

    return sumsq_bits, int(cap.value)


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", DISTANCE_DTYPES)
def test_packed_distances_match_reference_serial(oracle, reference, dtype, metric):
    """Integer types: every input of the finaliser is an exact integer, so the restated reciprocal square root
    and formulas must reproduce nk_{angulars,euclideans}_packed_<T>_serial bit for bit. Float types: the reference
    takes its norms from the host-dispatched nk_reduce_moments_*, one rounding away from the serial sum at most,
    which the finaliser turns into a few roundings: within 8 * 2^-24 absolute for angular, and of the sum of the two
    norms under the root for euclidean (where identical rows cancel to a residue of that size)."""
    if reference is None:
        pytest.skip("reference build not present")
    rng = np.random.default_rng(22)
    for m, n, k in [(1, 1, 1), (5, 7, 37), (33, 21, 300), (16, 16, 1024), (9, 4, 4099)]:
        a, b = reference_distance_inputs(oracle, dtype, m, k, rng), reference_distance_inputs(oracle, dtype, n, k, rng)
        if m > 4:
            a[1] = 0  # a zero row: the "product of norms is not positive" branch
            b[2] = a[3][:k] if n > 2 else b[0]  # identical rows: distance 0 up to rounding
        mine = oracle.spatials_packed(metric, dtype, a, b)
        ref = reference.spatials_packed(support.METRIC_KINDS[metric], dtype, a, b)
        if dtype in INTEGER_DTYPES:
            assert np.array_equal(mine.view(np.uint32), ref.view(np.uint32)), (dtype, metric, m, n, k)
        else:
            u = 2.0 ** -24
            if metric == "angular":  # 1 - x with |x| <= 1: absolute roundings
                assert np.abs(mine.astype(np.float64) - ref).max() <= 8 * u, (dtype, metric, m, n, k)
            else:  # sqrt(qn + tn - 2 dot): roundings of the size of the norms, under the root
                norms = oracle.row_sumsq(dtype, a).astype(np.float64)[:, None] + oracle.row_sumsq(dtype, b).astype(np.float64)[None, :]
                gap = np.abs(mine.astype(np.float64) ** 2 - ref.astype(np.float64) ** 2)
                close = np.abs(mine.astype(np.float64) - ref) <= 8 * u * np.abs(ref)  # a few ulp of the distance itself,
                assert (close | (gap <= 8 * u * np.maximum(norms, 1e-30))).all(), (dtype, metric, m, n, k)  # or a cancelled residue


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", DISTANCE_DTYPES)
def test_packed_distances_closed_forms(oracle, dtype, metric):
    """Known answers that need no reference: orthogonal rows are at angular 1 / euclidean sqrt(|a|^2 + |b|^2),
    a row against itself at 0, against its double (same direction) at angular 0 / euclidean |a|, zero rows at 0."""
    # (the 4-bit types: the value in the low half of a byte, 0 in the high half)
    one = {"i8": 1, "u8": 1, "bf16": 0x3F80, "f16": 0x3C00, "e4m3": 0x38, "e5m2": 0x3C, "e2m3": 0x08, "e3m2": 0x0C, "i4": 1, "u4": 1}[dtype]
    two = {"i8": 2, "u8": 2, "bf16": 0x4000, "f16": 0x4000, "e4m3": 0x40, "e5m2": 0x40, "e2m3": 0x10, "e3m2": 0x10, "i4": 2, "u4": 2}[dtype]
    k = 64
    rows = np.zeros((4, k), dtype=support.STORAGE[dtype])
    rows[0, :16] = one   # |.|^2 = 16
    rows[1, 16:32] = one  # orthogonal to row 0
    rows[2, :16] = two   # row 0 doubled
    got = oracle.spatials_packed(metric, dtype, rows, rows)
    truth = oracle.spatials_truth(metric, dtype, rows, rows)
    if metric == "angular":
        expected = np.array([[0, 1, 0, 1], [1, 0, 1, 1], [0, 1, 0, 1], [1, 1, 1, 0]], dtype=np.float64)
        expected[0, 3] = expected[3, 0] = expected[1, 3] = expected[3, 1] = expected[2, 3] = expected[3, 2] = 0  # zero norm and zero dot
    else:
        expected = np.array([[0, np.sqrt(32), 4, 4], [np.sqrt(32), 0, np.sqrt(80), 4], [4, np.sqrt(80), 0, 8], [4, 4, 8, 0]])
    assert np.allclose(truth, expected, atol=1e-12)
    assert np.allclose(got, expected, atol=2e-6)


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", ["i4", "u4"])
def test_four_bit_distances_follow_the_serial_moments(oracle, dtype, metric):
    """Signed and unsigned 4-bit values over their full range, odd depths included (both halves of the last byte count,
    reduce/serial.h:373-404): the restated kernels against the distances from f64 dots and norms. All inputs of the
    finaliser are exact integers, so what is left is its own few f32 roundings."""
    rng = np.random.default_rng(23)
    for m, n, k in [(3, 5, 1), (9, 7, 19), (12, 33, 257)]:
        a, b = support.random_matrix(oracle, dtype, m, k, rng), support.random_matrix(oracle, dtype, n, k, rng)
        got, truth = oracle.spatials_packed(metric, dtype, a, b).astype(np.float64), oracle.spatials_truth(metric, dtype, a, b)
        scale = 1.0 if metric == "angular" else np.maximum(truth, 1.0)
        assert (np.abs(got - truth) <= 4e-7 * scale).all(), (dtype, metric, m, n, k)


def upper_window(count, row_start, row_count):
    """Mask of what a symmetric call owns: rows of the window, columns on or right of the diagonal."""
    i, j = np.arange(count)[:, None], np.arange(count)[None, :]
    return (i >= row_start) & (i < row_start + row_count) & (j >= i)


# (count, depth, row_start, row_count): windows that start and end off the reference's 4-, 32- and 128-row blocks
SYMMETRIC_CASES = [(1, 1, 0, 1), (7, 37, 0, 7), (45, 300, 0, 45), (45, 300, 5, 17), (150, 70, 0, 150), (150, 70, 33, 100),
                   (150, 70, 128, 500), (70, 1030, 64, 6)]


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_symmetric_dots_match_reference_serial(oracle, reference, dtype):
    """nk_dots_symmetric_<T>_serial, bit for bit, on the elements the call owns (the reference may also write a few
    below the diagonal when a window ends inside one of its 32-row blocks; those are not part of the contract)."""
    if reference is None:
        pytest.skip("reference build not present")
    rng = np.random.default_rng(61)
    for count, depth, row_start, row_count in SYMMETRIC_CASES:
        vectors = finite_inputs(oracle, dtype, count, depth, rng)
        mine = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
        ref = reference.symmetric("dots", dtype, vectors, row_start, row_count)
        own = upper_window(count, row_start, row_count)
        assert np.array_equal(mine.view(np.uint32)[own], ref.view(np.uint32)[own]), (dtype, count, depth, row_start)
        assert not mine[~own].any()  # the restatement writes nothing else


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", DISTANCE_DTYPES)
def test_symmetric_distances_match_reference_serial(oracle, reference, dtype, metric):
    """nk_{angulars,euclideans}_symmetric_<T>_serial: integers bit for bit, floats to the tolerance of the packed
    distances above (the same host-dispatched norms enter); the diagonal is exactly 0 in both."""
    if reference is None:
        pytest.skip("reference build not present")
    rng = np.random.default_rng(62)
    for count, depth, row_start, row_count in SYMMETRIC_CASES:
        # (the reference's distance kinds do not clamp a window that runs past the last vector, unlike its dots
        # kind, dots/serial.h:2380 against :2815-2821: such a call is outside its contract and is not made here)
        row_count = min(row_count, count - row_start)
        vectors = reference_distance_inputs(oracle, dtype, count, depth, rng)
        if count > 40:
            vectors[2] = 0
            vectors[9] = vectors[40]  # identical vectors off the diagonal
        mine = oracle.symmetric(metric, dtype, vectors, row_start, row_count)
        ref = reference.symmetric(metric, dtype, vectors, row_start, row_count)
        own = upper_window(count, row_start, row_count)
        assert not mine[~own].any()
        assert not np.diag(mine).any() and not np.diag(ref)[row_start:row_start + row_count].any()
        if dtype in INTEGER_DTYPES:
            assert np.array_equal(mine.view(np.uint32)[own], ref.view(np.uint32)[own]), (dtype, metric, count, row_start)
            continue
        u = 2.0 ** -24
        x, y = mine.astype(np.float64)[own], ref.astype(np.float64)[own]
        if metric == "angular":
            assert np.abs(x - y).max() <= 8 * u
        else:
            squares = oracle.row_sumsq(dtype, vectors).astype(np.float64)
            norms = (squares[:, None] + squares[None, :])[own]
            assert ((np.abs(x - y) <= 8 * u * np.abs(y)) | (np.abs(x * x - y * y) <= 8 * u * np.maximum(norms, 1e-30))).all()


@pytest.mark.parametrize("dtype", DISTANCE_DTYPES)
def test_symmetric_equals_packed_with_both_sides_the_same(oracle, dtype):
    """Needs no reference: the upper triangle of the symmetric kinds is the packed kinds with B = A (same per-pair
    arithmetic), the diagonal of the distances is 0, and the row windows tile the full call."""
    rng = np.random.default_rng(63)
    vectors = finite_inputs(oracle, dtype, 53, 129, rng)
    upper = np.triu(np.ones((53, 53), dtype=bool))
    full = oracle.symmetric("dots", dtype, vectors)
    assert np.array_equal(full[upper].view(np.uint32), oracle.dots_packed(dtype, vectors, vectors)[upper].view(np.uint32))
    pieces = np.zeros_like(full)
    for start, rows in ((0, 10), (10, 1), (11, 31), (42, 100)):
        oracle.symmetric("dots", dtype, vectors, start, rows, out=pieces)
    assert np.array_equal(pieces.view(np.uint32), full.view(np.uint32))
    for metric in ("angular", "euclidean"):
        got = oracle.symmetric(metric, dtype, vectors)
        packed = oracle.spatials_packed(metric, dtype, vectors, vectors)
        strict = np.triu(np.ones((53, 53), dtype=bool), 1)
        assert np.array_equal(got[strict].view(np.uint32), packed[strict].view(np.uint32))
        assert not np.diag(got).any()


@pytest.mark.parametrize("dtype", NARROW_FLOAT_DTYPES)
def test_six_bit_floats_match_reference_and_definition(oracle, reference, dtype):
    """All 256 byte values decode as the format defines them (sign, `e` exponent bits with bias, `m` mantissa bits,
    subnormals, no Inf or NaN, bits 6 and 7 ignored), and as nk_cast_serial decodes them; the encoder agrees with it on
    finite probes including every tie between neighbours of the grid."""
    ebits, mbits, bias = {"e2m3": (2, 3, 1), "e3m2": (3, 2, 3)}[dtype]
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.decode(dtype, codes[None, :])[0]
    for code in range(256):
        sign, e, m = (code >> 5) & 1, (code >> mbits) & ((1 << ebits) - 1), code & ((1 << mbits) - 1)
        expected = m * 2.0 ** (1 - bias - mbits) if e == 0 else (1 + m / 2.0 ** mbits) * 2.0 ** (e - bias)
        assert float(got[code]) == (-expected if sign else expected), hex(code)
    assert float(got.max()) == {"e2m3": 7.5, "e3m2": 28.0}[dtype]
    if reference is None:
        pytest.skip("reference build not present")
    assert same_floats(got, reference.cast(codes, dtype, "f32"))
    rng = np.random.default_rng(3)
    grid = np.unique(np.abs(got))
    mids = ((grid[:-1].astype(np.float64) + grid[1:]) / 2).astype(np.float32)
    probes = np.concatenate([grid, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                             np.array([30, 100, 1e6, 1e-3, 1e-8], np.float32)]
                            + [rng.standard_normal(20000).astype(np.float32) * np.float32(scale) for scale in (0.01, 0.3, 2, 10, 100)])
    probes = np.concatenate([probes, -probes])
    assert np.array_equal(oracle.encode(dtype, probes), reference.cast(probes, "f32", dtype))


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
def test_narrow_products_match_reference_serial(oracle, reference, dtype):
    """nk_dots_packed_<T>_serial and nk_dots_symmetric_<T>_serial for e2m3, e3m2, i4, u4, u1, bit for bit, depths that
    do not fill the last byte of a sub-byte type (whole bytes are read) included."""
    if reference is None:
        pytest.skip("reference build not present")
    rng = np.random.default_rng(64)
    for m, n, k in [(1, 1, 1), (3, 5, 16), (7, 9, 100), (4, 4, 33), (13, 21, 77), (5, 6, 2050)]:
        a, b = support.random_matrix(oracle, dtype, m, k, rng), support.random_matrix(oracle, dtype, n, k, rng)
        assert np.array_equal(oracle.dots_packed(dtype, a, b).view(np.uint32), reference.dots_packed(dtype, a, b).view(np.uint32)), (dtype, m, n, k)
    for count, depth, row_start, row_count in SYMMETRIC_CASES[:6]:
        vectors = support.random_matrix(oracle, dtype, count, depth, rng)
        own = upper_window(count, row_start, row_count)
        mine = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
        ref = reference.symmetric("dots", dtype, vectors, row_start, row_count)
        assert np.array_equal(mine.view(np.uint32)[own], ref.view(np.uint32)[own]), (dtype, count, depth, row_start)


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
def test_narrow_products_closed_forms(oracle, dtype):
    """Needs no reference. 4-bit integers and bits: the exact product of the unpacked values (low bits first, i4
    sign-extended) in numpy int64. 6-bit floats: every value is a multiple of 1/8 (e2m3) or 1/16 (e3m2) below 2^5, so short dots are
    exact in f32 and must equal the f64 product of the decoded values."""
    rng = np.random.default_rng(65)
    a, b = support.random_matrix(oracle, dtype, 9, 64, rng), support.random_matrix(oracle, dtype, 11, 64, rng)
    got = oracle.dots_packed(dtype, a, b)
    if dtype in ("i4", "u4", "u1"):
        def unpack(x):
            if dtype == "u1":
                return np.unpackbits(x, axis=1, bitorder="little").astype(np.int64)
            nibbles = np.stack([x & 0xF, x >> 4], axis=-1).reshape(x.shape[0], -1).astype(np.int64)
            return np.where(nibbles >= 8, nibbles - 16, nibbles) if dtype == "i4" else nibbles
        exact = unpack(a) @ unpack(b).T
        assert np.array_equal(got.astype(np.int64) & 0xFFFFFFFF, exact & 0xFFFFFFFF)
        assert np.array_equal(oracle.decode(dtype, a).astype(np.int64), unpack(a))
    else:
        decoded_a, decoded_b = oracle.decode(dtype, a).astype(np.float64), oracle.decode(dtype, b).astype(np.float64)
        assert np.array_equal(got.astype(np.float64), decoded_a @ decoded_b.T)
        truth, _ = oracle.truth(dtype, a, b)
        assert np.array_equal(truth, decoded_a @ decoded_b.T)


@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_wide_products_match_reference_serial(oracle, reference, dtype):
    """nk_dots_packed_{f32,f64}_serial and nk_dots_symmetric_{f32,f64}_serial (f64 results), bit for bit: N(0,1) and
    lognormal inputs with random signs, depths off the 4- and 2-value steps."""
    if reference is None:
        pytest.skip("reference build not present")
    rng = np.random.default_rng(66)
    for kind in ("default", "lognormal"):
        for m, n, k in [(1, 1, 1), (3, 5, 16), (7, 9, 101), (4, 4, 33), (13, 21, 77), (5, 6, 2050)]:
            a, b = support.random_matrix(oracle, dtype, m, k, rng, kind), support.random_matrix(oracle, dtype, n, k, rng, kind)
            assert np.array_equal(oracle.dots_packed(dtype, a, b).view(np.uint64), reference.dots_packed(dtype, a, b).view(np.uint64)), (dtype, kind, m, n, k)
    for count, depth, row_start, row_count in SYMMETRIC_CASES[:6]:
        vectors = support.random_matrix(oracle, dtype, count, depth, rng)
        own = upper_window(count, row_start, row_count)
        mine = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
        ref = reference.symmetric("dots", dtype, vectors, row_start, row_count)
        assert np.array_equal(mine.view(np.uint64)[own], ref.view(np.uint64)[own]), (dtype, count, depth, row_start)
        assert not mine[~own].any()


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_wide_distances_match_reference_serial(oracle, reference, dtype, metric):
    """nk_{angulars,euclideans}_{packed,symmetric}_{f32,f64}_serial (f64 results): the sums of squares bit for bit
    against nk_reduce_moments_{f32,f64}_serial, the distances to 16 units of 2^-53 (the reference takes its sums of
    squares from the host-dispatched moments, whose order differs; dots and finaliser are restated exactly)."""
    if reference is None:
        pytest.skip("reference build not present")
    import ctypes

    rng = np.random.default_rng(68)
    fn, cap = ctypes.c_void_p(), ctypes.c_uint64()
    reference.lib.nk_find_kernel_punned(ord("R"), support.CODES[dtype], support.CAP_SERIAL, ctypes.byref(fn), ctypes.byref(cap))
    moments = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p)(fn.value)
    for kind in ("default", "lognormal"):
        for m, n, k in [(1, 1, 1), (5, 7, 37), (33, 21, 300), (9, 4, 4099)]:
            a, b = support.random_matrix(oracle, dtype, m, k, rng, kind), support.random_matrix(oracle, dtype, n, k, rng, kind)
            if m > 4:
                a[1] = 0
                b[2] = a[3]
            squares = oracle.row_sumsq(dtype, a)
            for i in range(m):
                total, sumsq = np.zeros(1), np.zeros(1)
                moments(a[i].ctypes.data, k, a.itemsize, total.ctypes.data, sumsq.ctypes.data)
                assert squares[i:i + 1].view(np.uint64)[0] == sumsq.view(np.uint64)[0], (dtype, kind, m, k, i)
            norms = squares[:, None] + oracle.row_sumsq(dtype, b)[None, :]
            mine = oracle.spatials_packed(metric, dtype, a, b)
            ref = reference.spatials_packed(support.METRIC_KINDS[metric], dtype, a, b)
            assert mine.dtype == ref.dtype == np.float64
            assert support.wide_distances_agree(metric, mine, ref, norms), (dtype, metric, kind, m, n, k)
            truth = oracle.spatials_truth(metric, dtype, a, b)  # plain f64 sums: a loose band against a common mistake
            assert support.wide_distances_agree(metric, mine, truth, norms, ulps=64 * k)
    for count, depth, row_start, row_count in SYMMETRIC_CASES[:6]:
        row_count = min(row_count, count - row_start)
        vectors = support.random_matrix(oracle, dtype, count, depth, rng)
        if count > 40:
            vectors[2] = 0
            vectors[9] = vectors[40]
        own = upper_window(count, row_start, row_count)
        mine = oracle.symmetric(metric, dtype, vectors, row_start, row_count)
        ref = reference.symmetric(metric, dtype, vectors, row_start, row_count)
        assert not mine[~own].any() and not np.diag(mine).any() and not np.diag(ref)[row_start:row_start + row_count].any()
        squares = oracle.row_sumsq(dtype, vectors)
        assert support.wide_distances_agree(metric, mine[own], ref[own], (squares[:, None] + squares[None, :])[own]), (dtype, metric, count)
        strict = np.triu(np.ones((count, count), dtype=bool), 1) & own
        packed = oracle.spatials_packed(metric, dtype, vectors, vectors)
        assert np.array_equal(mine[strict].view(np.uint64), packed[strict].view(np.uint64))


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_wide_distances_closed_forms(oracle, dtype, metric):
    """Needs no reference: orthogonal rows, a row against itself and its double, a zero row (the layout of
    test_packed_distances_closed_forms), to a few units of 2^-53."""
    k = 64
    rows = np.zeros((4, k), dtype=support.STORAGE[dtype])
    rows[0, :16] = 1
    rows[1, 16:32] = 1
    rows[2, :16] = 2
    got = oracle.spatials_packed(metric, dtype, rows, rows)
    if metric == "angular":
        expected = np.array([[0, 1, 0, 0], [1, 0, 1, 0], [0, 1, 0, 0], [0, 0, 0, 0]], dtype=np.float64)
    else:
        expected = np.array([[0, np.sqrt(32), 4, 4], [np.sqrt(32), 0, np.sqrt(80), 4], [4, np.sqrt(80), 0, 8], [4, 4, 8, 0]])
    assert np.abs(got - expected).max() <= 8 * 2.0 ** -53 * 8


def test_wide_products_closed_forms(oracle):
    """Needs no reference. Small integers: every sum is exact in f64, so both kinds equal the int64 product. f64 only:
    sums that plain f64 gets wrong and a sum in twice the working precision gets right: 1e100 + 1 - 1e100 = 1, and a
    long alternating series whose large terms cancel, checked against exact rational arithmetic."""
    from fractions import Fraction

    rng = np.random.default_rng(67)
    ints_a, ints_b = rng.integers(-1000, 1000, (9, 130)), rng.integers(-1000, 1000, (11, 130))
    for dtype in WIDE_DTYPES:
        got = oracle.dots_packed(dtype, ints_a.astype(support.STORAGE[dtype]), ints_b.astype(support.STORAGE[dtype]))
        assert np.array_equal(got, (ints_a @ ints_b.T).astype(np.float64))
    a = np.array([[1e100, 1.0, -1e100, 3.0]])
    b = np.array([[1.0, 1.0, 1.0, 0.5]])
    assert oracle.dots_packed("f64", a, b)[0, 0] == 2.5 and float(a[0] @ b[0]) != 2.5  # (numpy's plain sum loses the 1)
    x = (rng.standard_normal((4, 257)) * 10.0 ** rng.integers(-8, 9, (4, 257)))
    y = (rng.standard_normal((3, 257)) * 10.0 ** rng.integers(-8, 9, (3, 257)))
    got = oracle.dots_packed("f64", x, y)
    for i in range(4):
        for j in range(3):
            exact = sum(Fraction(float(p)) * Fraction(float(q)) for p, q in zip(x[i], y[j]))
            scale = sum(abs(Fraction(float(p)) * Fraction(float(q))) for p, q in zip(x[i], y[j]))
            # within one rounding of the exact value plus the second-order term of a doubled precision
            assert abs(Fraction(float(got[i, j])) - exact) <= abs(exact) * Fraction(1, 2 ** 52) + scale * Fraction(257 ** 2, 2 ** 104)


@pytest.mark.parametrize("dtype", ["i8", "u8"])
def test_integer_product_closed_form(oracle, dtype):
    rng = np.random.default_rng(11)
    for m, n, k, pad_a, pad_b in SHAPES + [(3, 5, 70000, 0, 0)]:
        a = support.random_matrix(oracle, dtype, m, k, rng, pad=pad_a)
        b = support.random_matrix(oracle, dtype, n, k, rng, pad=pad_b)
        exact = a.astype(np.int64) @ b.astype(np.int64).T
        assert np.array_equal(oracle.dots_packed(dtype, a, b).astype(np.int64) & 0xFFFFFFFF, exact & 0xFFFFFFFF)
    # extremes: every product is (-128)^2 or 255^2
    k = 4096
    a = np.full((2, k), -128 if dtype == "i8" else 255, dtype=STORAGE[dtype])
    assert int(oracle.dots_packed(dtype, a, a)[0, 0]) == k * (16384 if dtype == "i8" else 65025)


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_float_product_properties(oracle, dtype):
    rng = np.random.default_rng(13)
    a = support.random_matrix(oracle, dtype, 9, 333, rng)
    b = support.random_matrix(oracle, dtype, 11, 333, rng)
    truth, magnitude = oracle.truth(dtype, a, b)
    decoded = lambda x: oracle.decode(dtype, np.ascontiguousarray(x)).astype(np.float64)
    assert np.allclose(truth, decoded(a) @ decoded(b).T, rtol=0, atol=1e-12 * magnitude.max())
    assert np.allclose(magnitude, np.abs(decoded(a)) @ np.abs(decoded(b)).T, rtol=1e-12)
    serial = oracle.dots_packed(dtype, a, b)
    assert np.all(np.abs(serial - truth) <= 333 * 2.0**-24 * magnitude)  # f32 accumulation stays within k ulps
    # powers of two sum exactly: a = b = 2^-3 everywhere -> k / 64
    one_eighth = oracle.encode(dtype, np.full((2, 256), 0.125, np.float32))
    assert np.all(oracle.dots_packed(dtype, one_eighth, one_eighth) == 4.0)
    # a dropped k-tail or a transposed operand would break this asymmetric case
    a2 = oracle.encode(dtype, np.arange(1, 7, dtype=np.float32).reshape(2, 3))
    b2 = oracle.encode(dtype, np.array([[1, 0, 0], [0, 1, 0], [0, 0, 1], [1, 1, 1]], np.float32))
    assert np.array_equal(oracle.dots_packed(dtype, a2, b2), np.array([[1, 2, 3, 6], [4, 5, 6, 15]], np.float32))


def test_special_values_follow_ieee(oracle):
    enc = lambda dtype, *v: oracle.encode(dtype, np.array([v], np.float32))
    for dtype in ("f16", "bf16", "e5m2"):
        inf_one, zero_one, one_one = enc(dtype, np.inf, 1), enc(dtype, 0, 1), enc(dtype, 1, 1)
        assert oracle.dots_packed(dtype, inf_one, one_one)[0, 0] == np.inf
        assert np.isnan(oracle.dots_packed(dtype, inf_one, zero_one)[0, 0])  # inf * 0
        assert np.isnan(oracle.dots_packed(dtype, enc(dtype, np.inf, -np.inf), one_one)[0, 0])  # inf - inf
    assert np.isnan(oracle.dots_packed("e4m3", enc("e4m3", np.nan, 1), enc("e4m3", 1, 1))[0, 0])
    assert oracle.dots_packed("e4m3", enc("e4m3", np.inf, 0), enc("e4m3", 1, 1))[0, 0] == 448.0  # saturating encoder


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(support.GOLDEN_DIR) if f.endswith(".npz")) if os.path.isdir(support.GOLDEN_DIR) else [])
def test_golden_vectors(oracle, name):
    """Vectors written from the reference's serial kernels; hold with or without the reference checkout."""
    data = np.load(os.path.join(support.GOLDEN_DIR, name))
    if name.startswith("cast_"):
        dtype = str(data["dtype"])
        assert same_floats(oracle.decode(dtype, data["codes"]), data["decoded"])
        assert np.array_equal(oracle.encode(dtype, data["values"]), data["encoded"])
    elif name.startswith("wide_"):
        dtype, a, b, vectors = str(data["dtype"]), data["a"], data["b"], data["vectors"]
        assert np.array_equal(oracle.dots_packed(dtype, a, b).view(np.uint64), data["c_serial"].view(np.uint64))
        mine = oracle.symmetric("dots", dtype, vectors, int(data["row_start"]), int(data["row_count"]))
        assert np.array_equal(mine.view(np.uint64), data["symmetric_serial"].view(np.uint64))
        norms = oracle.row_sumsq(dtype, a)[:, None] + oracle.row_sumsq(dtype, b)[None, :]
        squares = oracle.row_sumsq(dtype, vectors)
        for metric, key in (("angular", "angulars"), ("euclidean", "euclideans")):  # f64 distances: 16 units of 2^-53
            assert support.wide_distances_agree(metric, oracle.spatials_packed(metric, dtype, a, b), data[key + "_serial"], norms)
            mine = oracle.symmetric(metric, dtype, vectors, int(data["row_start"]), int(data["row_count"]))
            assert support.wide_distances_agree(metric, mine, data[key + "_symmetric_serial"], squares[:, None] + squares[None, :])
    elif name.startswith("narrow_"):
        dtype, a, b, vectors = str(data["dtype"]), data["a"], data["b"], data["vectors"]
        assert same_floats(oracle.dots_packed(dtype, a, b).view(np.float32), data["c_serial"].view(np.float32))
        if dtype in NARROW_FLOAT_DTYPES:
            assert same_floats(oracle.decode(dtype, np.arange(256, dtype=np.uint8)[None, :])[0], data["decoded"])
        mine = oracle.symmetric("dots", dtype, vectors, int(data["row_start"]), int(data["row_count"]))
        assert same_floats(mine.view(np.float32), data["symmetric_serial"].view(np.float32))
    elif name.startswith("symmetric_"):
        dtype, vectors = str(data["dtype"]), data["vectors"]
        row_start, row_count = int(data["row_start"]), int(data["row_count"])
        u = 2.0 ** -24
        squares = oracle.row_sumsq(dtype, vectors).astype(np.float64)
        norms = squares[:, None] + squares[None, :]
        mine = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
        assert same_floats(mine.view(np.float32), data["dots_serial"].view(np.float32))
        for metric, key in (("angular", "angulars_serial"), ("euclidean", "euclideans_serial")):
            mine, ref = oracle.symmetric(metric, dtype, vectors, row_start, row_count).astype(np.float64), data[key].astype(np.float64)
            if dtype in INTEGER_DTYPES:
                assert np.array_equal(mine, ref), (dtype, metric)
            elif metric == "angular":
                assert np.abs(mine - ref).max() <= 8 * u
            else:
                assert ((np.abs(mine - ref) <= 8 * u * np.abs(ref)) | (np.abs(mine ** 2 - ref ** 2) <= 8 * u * norms)).all()
    elif name.startswith("spatials_"):
        dtype = str(data["dtype"])
        a, b = data["a"], data["b"]
        u = 2.0 ** -24
        norms = oracle.row_sumsq(dtype, a).astype(np.float64)[:, None] + oracle.row_sumsq(dtype, b).astype(np.float64)[None, :]
        for metric, key in (("angular", "angulars_serial"), ("euclidean", "euclideans_serial")):
            mine, ref = oracle.spatials_packed(metric, dtype, a, b).astype(np.float64), data[key].astype(np.float64)
            if dtype in INTEGER_DTYPES:
                assert np.array_equal(mine, ref), (dtype, metric)
            elif metric == "angular":
                assert np.abs(mine - ref).max() <= 8 * u
            else:
                assert ((np.abs(mine - ref) <= 8 * u * np.abs(ref)) | (np.abs(mine ** 2 - ref ** 2) <= 8 * u * norms)).all()
    else:
        dtype = str(data["dtype"])
        a, b = data["a"], data["b"]
        assert oracle.packed_size(dtype, b.shape[0], b.shape[1]) == int(data["serial_packed_size"])
        got = oracle.dots_packed(dtype, a, b)
        assert same_floats(got.view(np.float32), data["c_serial"].view(np.float32))
