"""Parity of the wide types of the dots family (f32 and f64 inputs, f64 results) with the reference, through the C ABI,
on a real MI355X.

`nk_dots_packed_size_<T>`, `nk_dots_pack_<T>`, `nk_dots_packed_<T>`, `nk_dots_symmetric_<T>` for f32 and f64: reference
include/numkong/dots/serial.h:2458-2491, arithmetic include/numkong/dot/serial.h:262-335 (f32: exact products into four
f64 lane sums; f64: the compensated two-lane sum of scalar/serial.h:128-136 folded by reduce/serial.h:33-48). The GPU
kernels (f32: the f64 MFMA, whose chain of fused multiply-adds along its depth advances one lane sum; f64: vector units)
keep the reference's own accumulators per output in the reference's own order along k, so the bar here is the
integer one: BIT-EXACT against the oracle's restatement of the serial kernels (which tests/test_oracle.py pins bit for
bit against the reference library), not a tolerance.
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
    assert size == 64 + 8 * 64 * (-(-k // 32) * 32)  # header + f64 x (n padded to 64) x (k padded to 32)
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
    with pytest.raises(TypeError):
        nk.angulars_packed(ga, other)  # dot-product kinds only


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
