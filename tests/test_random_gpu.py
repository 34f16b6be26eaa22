"""Seeded random shapes, strides and offsets for every element type of the dots family, through the C ABI, on a real
MI355X: the packed product (`nk_dots_packed_<T>`, reference include/numkong/dots.h:248-287) of operands that sit in
larger arrays (row pitches that are not multiples of 16 or 4 bytes, first element off an aligned address), against the
oracle's restatement of the serial kernels. Integers and the two wide types bit for bit; the other floats through the
gate of tests/test_dots_gpu.py (mean error against the f64 truth at most twice the serial kernel's, NaN / Inf masks
identical). The shapes straddle every tile edge and every path through the kernels: the pipelined loop with and
without tail masks, the guarded loop for rows that are not dword-aligned, depths from 1 to a few stages.
`NK_RANDOM_CASES` (default 10 per type) and `NK_RANDOM_SEED` (default 7000) widen or move the sample.
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from numkong_amd import api  # noqa: E402
from tests import support  # noqa: E402
from tests.support import ALL_DTYPES, INTEGER_DTYPES, NARROW_DTYPES, WIDE_DTYPES  # noqa: E402
from tests.test_dots_gpu import assert_float_gate, best_dispatch, to_gpu  # noqa: E402

pytestmark = pytest.mark.gpu


def embedded(oracle, dtype, rows, cols, rng, pad, offset):
    """A (rows x cols) matrix of stored values inside a wider array, starting `offset` values into it; returns the
    host view (contiguous copy for the oracle) and the device view (same pitch and offset as on the host)."""
    if dtype in support.DIMENSIONS_PER_VALUE:  # stored bytes, each holding two or eight dimensions: every byte value
        whole = rng.integers(0, 256, size=(rows, cols + pad + offset), dtype=np.uint8)
    else:
        whole = support.random_matrix(oracle, dtype, rows, cols + pad + offset, rng)
    host = np.ascontiguousarray(whole[:, offset:offset + cols])
    device = to_gpu(whole)[:, offset:offset + cols]
    return host, device


@pytest.mark.parametrize("dtype", ALL_DTYPES + NARROW_DTYPES + WIDE_DTYPES)
def test_random_shapes_strides_and_offsets(oracle, dtype):
    rng = np.random.default_rng(int(os.environ.get("NK_RANDOM_SEED", "7000")) + sorted(api.DTYPES).index(dtype))
    for case in range(int(os.environ.get("NK_RANDOM_CASES", "10"))):
        m, n = int(rng.integers(1, 300)), int(rng.integers(1, 700))
        cols = int(rng.choice([int(rng.integers(1, 40)), int(rng.integers(40, 1100)), 64 * int(rng.integers(1, 17))]))
        pad_a, pad_b = int(rng.integers(0, 9)), int(rng.integers(0, 9))
        off_a, off_b = int(rng.integers(0, 5)), int(rng.integers(0, 5))
        a, ga = embedded(oracle, dtype, m, cols, rng, pad_a, off_a)
        b, gb = embedded(oracle, dtype, n, cols, rng, pad_b, off_b)
        where = f"{dtype} case {case}: {m}x{n}x{cols} pads {pad_a},{pad_b} offsets {off_a},{off_b}"
        got = nk.dots_packed(ga, nk.dots_pack(gb, dtype)).cpu().numpy()
        serial = oracle.dots_packed(dtype, a, b)
        if dtype in INTEGER_DTYPES:
            assert np.array_equal(got.view(np.uint32), serial.view(np.uint32)), where
        elif dtype in WIDE_DTYPES:
            assert np.array_equal(got.view(np.uint64), serial.view(np.uint64)), where
        else:
            truth, magnitude = oracle.truth(dtype, a, b)
            assert_float_gate(dtype, got, serial, truth, magnitude, where, best_dispatch(dtype, a, b))


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", ALL_DTYPES + WIDE_DTYPES)
def test_random_distances_strides_and_offsets(oracle, dtype, metric):
    """The packed distances (`nk_angulars_packed_<T>`, `nk_euclideans_packed_<T>`, reference
    include/numkong/spatials.h:139-266) over the same kind of embedded operands: the six 8- and 16-bit types through
    the gate of tests/test_spatials_gpu.py, f32 and f64 within 16 units of 2^-53 of the serial restatement."""
    from tests.test_spatials_gpu import GPU_CALL, assert_distance_gate

    rng = np.random.default_rng(int(os.environ.get("NK_RANDOM_SEED", "7000")) + 100 + sorted(api.DTYPES).index(dtype))
    for case in range(max(1, int(os.environ.get("NK_RANDOM_CASES", "10")) // 2)):
        m, n = int(rng.integers(1, 300)), int(rng.integers(1, 400))
        cols = int(rng.choice([int(rng.integers(1, 40)), int(rng.integers(40, 1100)), 64 * int(rng.integers(1, 17))]))
        pad_a, pad_b = int(rng.integers(0, 9)), int(rng.integers(0, 9))
        off_a, off_b = int(rng.integers(0, 5)), int(rng.integers(0, 5))
        a, ga = embedded(oracle, dtype, m, cols, rng, pad_a, off_a)
        b, gb = embedded(oracle, dtype, n, cols, rng, pad_b, off_b)
        if dtype == "e5m2":  # the reference-rule encoder overflows to Inf: keep the distances finite
            keep = lambda x: np.where((x & 0x7F) > 0x7B, (x & 0x80) | 0x7B, x).astype(x.dtype)
            a, b = keep(a), keep(b)
            ga, gb = to_gpu(np.pad(a, ((0, 0), (off_a, pad_a))))[:, off_a:off_a + cols], to_gpu(np.pad(b, ((0, 0), (off_b, pad_b))))[:, off_b:off_b + cols]
        where = f"{dtype} {metric} case {case}: {m}x{n}x{cols} pads {pad_a},{pad_b} offsets {off_a},{off_b}"
        got = GPU_CALL[metric](ga, nk.dots_pack(gb, dtype)).cpu().numpy()
        if dtype in WIDE_DTYPES:
            serial = oracle.spatials_packed(metric, dtype, a, b)
            norms = oracle.row_sumsq(dtype, a)[:, None] + oracle.row_sumsq(dtype, b)[None, :]
            assert got.dtype == np.float64 and support.wide_distances_agree(metric, got, serial, norms), where
        else:
            assert_distance_gate(oracle, metric, dtype, a, b, got, where)
