"""Parity of the wide types of the dots family (f32 and f64 inputs, f64 results) with the reference, through the C ABI,
on a real MI355X.

`nk_dots_packed_size_<T>`, `nk_dots_pack_<T>`, `nk_dots_packed_<T>`, `nk_dots_symmetric_<T>` for f32 and f64: reference
include/numkong/dots/serial.h:2458-2491, arithmetic include/numkong/dot/serial.h:262-335 (f32: exact products into four
f64 lane sums; f64: the compensated two-lane sum of scalar/serial.h:128-136 folded by reduce/serial.h:33-48). The GPU
kernels (f32: the f64 MFMA, whose chain of fused multiply-adds along its depth advances one lane sum; f64: vector units)
keep the reference's own accumulators per output in the reference's own order along k, so the bar here is the
integer one: BIT-EXACT against the oracle's restatement of the serial kernels (which tests/test_oracle.py pins bit for
bit against the reference library), not a tolerance.

The distance kinds (`nk_{angulars,euclideans}_{packed,symmetric}_{f32,f64}`, f64 results; reference
include/numkong/spatials/serial.h:41-72, finalisers include/numkong/spatial/serial.h:281-302) finalise those same dot
products with the reference's own f64 arithmetic (bit-trick reciprocal square root, four Newton steps), so what can differ
from the serial kernel is the order in which the sums of squares are added up: a rounding or two of f64. Tolerance: 16
units of 2^-53, absolute for angular (a value in [0, 2]), relative for euclidean or, where two nearly equal vectors
cancel, of the sum of the two norms under the root (tests/support.py: wide_distances_agree); the oracle is pinned against
the reference's serial kernels to the same tolerance in tests/test_oracle.py.
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from numkong_amd import api  # noqa: E402
from tests import support  # noqa: E402
from tests.support import WIDE_DTYPES  # noqa: E402
from tests.test_dots_gpu import DEV, gpu_dots, to_gpu  # noqa: E402
from tests.test_symmetric_gpu import owned  # noqa: E402

pytestmark = pytest.mark.gpu
POISON = 0x7FF8123456789ABC  # a quiet NaN as f64


def same_bits(x, y):
    return np.array_equal(np.ascontiguousarray(x).view(np.uint64), np.ascontiguousarray(y).view(np.uint64))


SHAPES = [(1, 1, 1), (3, 5, 7), (33, 70, 200), (64, 64, 64), (100, 37, 333), (65, 129, 1001), (31, 300, 130), (130, 33, 4100)]


@pytest.mark.parametrize("kind", ["default", "lognormal"])
@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_shapes_bit_exact(oracle, dtype, kind):
    rng = np.random.default_rng(900)
    for m, n, k in SHAPES:
        a, b = support.random_matrix(oracle, dtype, m, k, rng, kind), support.random_matrix(oracle, dtype, n, k, rng, kind)
        got = gpu_dots(dtype, a, b)
        assert got.dtype == np.float64 and same_bits(got, oracle.dots_packed(dtype, a, b)), f"{dtype} {kind} {m}x{n}x{k}"


@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_past_one_grid_of_workgroups(oracle, dtype):
    """Rows deeper than 65535 x 32 values and products taller than 65535 tiles take several launches inside one call (the
    reference has no such bound: dots/serial.h:2458-2491): a depth of 2,100,001 on 2 x 3 outputs, bit for bit against the
    serial restatement; 4,200,000 rows of depth 3 against one column, bit for bit against a plain f64 product of small
    integers. (The symmetric kinds cannot reach a second band: a window of more than 4,194,176 rows of a result that
    wide does not fit any memory, so the per-band shift of their diagonal is exercised by no test.)"""
    rng = np.random.default_rng(905)
    a, b = support.random_matrix(oracle, dtype, 2, 2_100_001, rng), support.random_matrix(oracle, dtype, 3, 2_100_001, rng)
    assert same_bits(gpu_dots(dtype, a, b), oracle.dots_packed(dtype, a, b))
    tall = rng.integers(-50, 50, (4_200_000, 3)).astype(support.STORAGE[dtype])
    one = rng.integers(-50, 50, (1, 3)).astype(support.STORAGE[dtype])
    got = gpu_dots(dtype, tall, one)
    assert np.array_equal(got, tall.astype(np.float64) @ one.astype(np.float64).T)


def test_closed_forms():
    """Small integers: exact in both kinds. f64: 1e100 + 1 - 1e100 + 1.5 = 2.5, which a plain f64 sum gets wrong."""
    rng = np.random.default_rng(901)
    ints_a, ints_b = rng.integers(-1000, 1000, (70, 130)), rng.integers(-1000, 1000, (90, 130))
    for dtype in WIDE_DTYPES:
        got = gpu_dots(dtype, ints_a.astype(support.STORAGE[dtype]), ints_b.astype(support.STORAGE[dtype]))
        assert np.array_equal(got, (ints_a @ ints_b.T).astype(np.float64))
    a = np.array([[1e100, 1.0, -1e100, 3.0]])
    b = np.array([[1.0, 1.0, 1.0, 0.5]])
    assert gpu_dots("f64", a, b)[0, 0] == 2.5


@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_c_abi_strides_host_pointers_and_mismatch(oracle, dtype):
    rng = np.random.default_rng(902)
    lib = nk.library()
    m, n, k, pad = 37, 61, 515, 3
    a_wide, b_wide = support.random_matrix(oracle, dtype, m, k + pad, rng), support.random_matrix(oracle, dtype, n, k + pad, rng)
    a, b = np.ascontiguousarray(a_wide[:, :k]), np.ascontiguousarray(b_wide[:, :k])
    size = getattr(lib, f"nk_dots_packed_size_{dtype}")(n, k)
    assert size == 64 + 8 * 64 * (-(-k // 32) * 32) + 8 * 64  # header + f64 x (n padded to 64) x (k padded to 32) + sums of squares
    packed = np.zeros(size, np.uint8)
    getattr(lib, f"nk_dots_pack_{dtype}")(b_wide.ctypes.data, n, k, b_wide.strides[0], packed.ctypes.data)
    c = np.full((m, n + 2), np.float64(-7.0))
    getattr(lib, f"nk_dots_packed_{dtype}")(a_wide.ctypes.data, packed.ctypes.data, c.ctypes.data, m, n, k, a_wide.strides[0],
                                            c.strides[0])
    assert not lib.nk_amd_last_error()
    assert (c[:, n:] == -7.0).all() and same_bits(c[:, :n], oracle.dots_packed(dtype, a, b))
    # an image packed for another depth poisons the outputs (all bits set), as the other types do
    ga = to_gpu(a)
    other = nk.dots_pack(to_gpu(np.ascontiguousarray(b_wide[:, : k - 1])), dtype)
    out = torch.zeros((m, n), dtype=torch.float64, device=DEV)
    status = lib.nk_amd_dots_packed_async(api.DTYPES[dtype][0], ga.data_ptr(), other.buffer.data_ptr(), out.data_ptr(), m, n, k,
                                          a.strides[0], n * 8, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert status == 0 and (out.cpu().numpy().view(np.uint64) == 0xFFFFFFFFFFFFFFFF).all()


@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_symmetric_windows(oracle, dtype):
    rng = np.random.default_rng(903)
    for count, depth, row_start, row_count in [(5, 8, 0, 5), (300, 64, 100, 77), (700, 131, 333, 1000), (130, 515, 0, 130)]:
        vectors = support.random_matrix(oracle, dtype, count, depth, rng, "lognormal")
        out = torch.full((count, count), POISON, dtype=torch.int64, device=DEV).view(torch.float64)
        nk.dots_symmetric(to_gpu(vectors), dtype, out=out, start_row=row_start, end_row=min(count, row_start + row_count))
        bits = out.view(torch.int64).cpu().numpy().view(np.uint64)
        own = owned(count, row_start, row_count)
        assert (bits[~own] == POISON).all()
        serial = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
        assert np.array_equal(bits[own], serial.view(np.uint64)[own]), (dtype, count, depth, row_start)


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(support.GOLDEN_DIR) if f.startswith("wide_")))
def test_golden_vectors(oracle, name):
    """Inputs and serial-kernel outputs recorded from the reference library: reproduced bit for bit."""
    data = np.load(os.path.join(support.GOLDEN_DIR, name))
    dtype, a, b, vectors = str(data["dtype"]), data["a"], data["b"], data["vectors"]
    row_start, row_count = int(data["row_start"]), int(data["row_count"])
    assert same_bits(gpu_dots(dtype, a, b), data["c_serial"])
    count = vectors.shape[0]
    out = torch.zeros((count, count), dtype=torch.float64, device=DEV)
    nk.dots_symmetric(to_gpu(vectors), dtype, out=out, start_row=row_start, end_row=row_start + row_count)
    assert same_bits(out.cpu().numpy(), data["symmetric_serial"])
    norms = oracle.row_sumsq(dtype, a)[:, None] + oracle.row_sumsq(dtype, b)[None, :]
    squares = oracle.row_sumsq(dtype, vectors)
    for metric, key, call in (("angular", "angulars", nk.angulars_symmetric), ("euclidean", "euclideans", nk.euclideans_symmetric)):
        assert support.wide_distances_agree(metric, gpu_wide_distances(metric, dtype, a, b), data[key + "_serial"], norms)
        out = torch.zeros((count, count), dtype=torch.float64, device=DEV)
        call(to_gpu(vectors), dtype, out=out, start_row=row_start, end_row=row_start + row_count)
        assert support.wide_distances_agree(metric, out.cpu().numpy(), data[key + "_symmetric_serial"], squares[:, None] + squares[None, :])


@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_full_size_properties(oracle, dtype):
    """2048 x 2048 x 2048: sampled rows bit-exact against the oracle; the symmetric kind equals the packed kind with
    both sides the same on the upper triangle and leaves the rest of a fresh result zero."""
    count, depth = 2048, 2048
    rng = np.random.default_rng(904)
    vectors = support.random_matrix(oracle, dtype, count, depth, rng)
    gv = to_gpu(vectors)
    rectangle = nk.dots_packed(gv, nk.dots_pack(gv, dtype))
    whole = nk.dots_symmetric(gv, dtype)
    upper = torch.triu(torch.ones((count, count), dtype=torch.bool, device=DEV))
    assert torch.equal(whole.view(torch.int64)[upper], rectangle.view(torch.int64)[upper])
    assert not whole.view(torch.int64)[~upper].any()
    rows = np.array([0, 1001, 2047])
    sample = rectangle[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    assert same_bits(sample, oracle.dots_packed(dtype, vectors[rows], vectors))


def gpu_wide_distances(metric, dtype, a, b):
    call = {"angular": nk.angulars_packed, "euclidean": nk.euclideans_packed}[metric]
    return call(to_gpu(a), nk.dots_pack(to_gpu(b), dtype)).cpu().numpy()


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_packed_distances(oracle, dtype, metric):
    rng = np.random.default_rng(905)
    for kind in ("default", "lognormal"):
        for m, n, k in SHAPES:
            a, b = support.random_matrix(oracle, dtype, m, k, rng, kind), support.random_matrix(oracle, dtype, n, k, rng, kind)
            if m > 4 and n > 4:
                a[1] = 0         # zero row
                b[2] = a[3]      # identical rows
                b[4] = 0
            got = gpu_wide_distances(metric, dtype, a, b)
            assert got.dtype == np.float64 and np.isfinite(got).all()
            serial = oracle.spatials_packed(metric, dtype, a, b)
            norms = oracle.row_sumsq(dtype, a)[:, None] + oracle.row_sumsq(dtype, b)[None, :]
            assert support.wide_distances_agree(metric, got, serial, norms), f"{dtype} {metric} {kind} {m}x{n}x{k}"
            if m > 4 and n > 4:
                assert got[1, 4] == 0
                if metric == "angular":
                    assert (got[1] == 0).all()


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_symmetric_distances(oracle, dtype, metric):
    rng = np.random.default_rng(906)
    call = {"angular": nk.angulars_symmetric, "euclidean": nk.euclideans_symmetric}[metric]
    for count, depth, row_start, row_count in [(5, 8, 0, 5), (300, 64, 100, 77), (700, 131, 333, 1000), (130, 515, 0, 130)]:
        vectors = support.random_matrix(oracle, dtype, count, depth, rng, "lognormal")
        if count > 40:
            vectors[2] = 0
            vectors[9] = vectors[40]
        row_count = min(row_count, count - row_start)
        out = torch.full((count, count), POISON, dtype=torch.int64, device=DEV).view(torch.float64)
        call(to_gpu(vectors), dtype, out=out, start_row=row_start, end_row=row_start + row_count)
        bits = out.view(torch.int64).cpu().numpy().view(np.uint64)
        own = owned(count, row_start, row_count)
        assert (bits[~own] == POISON).all()
        window = np.arange(row_start, row_start + row_count)
        assert (bits[window, window] == 0).all()  # a vector and itself: exactly 0
        got, serial = bits.view(np.float64), oracle.symmetric(metric, dtype, vectors, row_start, row_count)
        squares = oracle.row_sumsq(dtype, vectors)
        assert support.wide_distances_agree(metric, got[own], serial[own], (squares[:, None] + squares[None, :])[own]), (dtype, metric, count)


@pytest.mark.parametrize("dtype", WIDE_DTYPES)
def test_distances_through_the_c_abi_with_host_pointers(oracle, dtype):
    rng = np.random.default_rng(907)
    lib = nk.library()
    m, n, k = 19, 45, 203
    a, b = support.random_matrix(oracle, dtype, m, k, rng), support.random_matrix(oracle, dtype, n, k, rng)
    packed = np.zeros(getattr(lib, f"nk_dots_packed_size_{dtype}")(n, k), np.uint8)
    getattr(lib, f"nk_dots_pack_{dtype}")(b.ctypes.data, n, k, b.strides[0], packed.ctypes.data)
    norms = oracle.row_sumsq(dtype, a)[:, None] + oracle.row_sumsq(dtype, b)[None, :]
    for metric, stem in (("angular", "nk_angulars_packed_"), ("euclidean", "nk_euclideans_packed_")):
        c = np.full((m, n + 1), -7.0)
        getattr(lib, stem + dtype)(a.ctypes.data, packed.ctypes.data, c.ctypes.data, m, n, k, a.strides[0], c.strides[0])
        assert not lib.nk_amd_last_error() and (c[:, n] == -7.0).all()
        assert support.wide_distances_agree(metric, c[:, :n], oracle.spatials_packed(metric, dtype, a, b), norms)
