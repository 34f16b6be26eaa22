"""Parity of the symmetric kinds with the reference, through the C ABI, on a real MI355X.

`nk_dots_symmetric_<T>`, `nk_angulars_symmetric_<T>`, `nk_euclideans_symmetric_<T>` (reference:
include/numkong/dots.h:298-359, include/numkong/spatials.h:76-120, semantics in include/numkong/dots/serial.h:2361-2435
and :2802-2878) take one set of vectors and a window of rows and own result[i][j] for the rows i of the window and
the columns j >= i; the reference's own test (test/test_cross.hpp:77-112) compares exactly those elements. Checked here:

  * owned elements: integers bit for bit against the oracle's restatement of the serial kernel; floats through the gates
    of tests/test_dots_gpu.py (products) and tests/test_spatials_gpu.py (distances), against the serial restatement and,
    when oracle/_ref is present, the kernel the reference dispatches to on this host;
  * the diagonal of the distances is exactly 0;
  * nothing else is written: the result starts as a poison pattern and every element the call does not own keeps it
    (stricter than the reference, which may spill below the diagonal inside its 32-row blocks);
  * the upper triangle equals the packed kinds with both sides the same, bit for bit, at full size, and row windows
    tile the full call.
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from numkong_amd import api  # noqa: E402
from tests import support  # noqa: E402
from tests.support import ALL_DTYPES, FLOAT_DTYPES, OUTPUT  # noqa: E402
from tests.test_dots_gpu import DEV, assert_float_gate, to_gpu  # noqa: E402
from tests.test_spatials_gpu import errors as distance_errors, finite_inputs  # noqa: E402

pytestmark = pytest.mark.gpu
U = 2.0 ** -24
POISON = 0x7FC12345  # a quiet NaN as f32, a large positive number as i32 / u32
GPU_CALL = {"dots": nk.dots_symmetric, "angular": nk.angulars_symmetric, "euclidean": nk.euclideans_symmetric}
_REFERENCE = []


def reference_library():
    if not _REFERENCE:
        _REFERENCE.append(support.load_reference())
    return _REFERENCE[0]


def owned(count, row_start, row_count):
    i, j = np.arange(count)[:, None], np.arange(count)[None, :]
    return (i >= row_start) & (i < row_start + row_count) & (j >= i)


def gpu_symmetric(metric, dtype, vectors, row_start=0, row_count=None, config=0):
    """The call on a poisoned result; returns the raw 32-bit patterns."""
    count = vectors.shape[0]
    out_dtype = torch.float32 if metric != "dots" or OUTPUT[dtype] == np.float32 else torch.int32
    out = torch.full((count, count), POISON, dtype=torch.int32, device=DEV).view(out_dtype)
    end = count if row_count is None else min(count, row_start + row_count)
    nk.library().nk_hip_set_tile_config(config)
    try:
        GPU_CALL[metric](to_gpu(vectors), dtype, out=out, start_row=row_start, end_row=end)
    finally:
        nk.library().nk_hip_set_tile_config(0)
    return out.view(torch.int32).cpu().numpy().view(np.uint32)


def check_dots(oracle, dtype, vectors, row_start, row_count, config, where):
    count = vectors.shape[0]
    own = owned(count, row_start, row_count)
    bits = gpu_symmetric("dots", dtype, vectors, row_start, row_count, config)
    assert (bits[~own] == POISON).all(), f"wrote outside its window {where}"
    serial = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
    if dtype in support.INTEGER_DTYPES:
        if dtype in ("i8", "u8"):
            exact = (vectors.astype(np.int64) @ vectors.astype(np.int64).T) & 0xFFFFFFFF
            assert np.array_equal(bits[own].astype(np.int64), exact[own]), where
        assert np.array_equal(bits[own], serial.view(np.uint32)[own]), where
        return
    truth, magnitude = oracle.truth(dtype, vectors, vectors)
    dispatched = None
    if reference_library() is not None:
        reference = reference_library()
        dispatched = reference.symmetric("dots", dtype, vectors, row_start, row_count, viable=reference.capabilities)[own]
    assert_float_gate(dtype, bits.view(np.float32)[own], serial[own], truth[own], magnitude[own], where, dispatched)


def check_distances(oracle, metric, dtype, vectors, row_start, row_count, config, where):
    count = vectors.shape[0]
    row_count = min(row_count, count - row_start)  # (the reference's distance kinds do not clamp the window themselves)
    own = owned(count, row_start, row_count)
    bits = gpu_symmetric(metric, dtype, vectors, row_start, row_count, config)
    assert (bits[~own] == POISON).all(), f"wrote outside its window {where}"
    got = bits.view(np.float32)
    window = np.arange(row_start, row_start + row_count)
    assert (bits[window, window] == 0).all(), f"diagonal is not exactly zero {where}"
    strict = own & ~np.eye(count, dtype=bool)
    if not strict.any():
        return
    assert np.isfinite(got[strict]).all(), where
    truth = oracle.spatials_truth(metric, dtype, vectors, vectors)[strict]
    decoded = vectors.astype(np.float64) if dtype in ("i8", "u8") else oracle.decode(dtype, vectors).astype(np.float64)
    squares = (decoded ** 2).sum(axis=1)
    norms = (squares[:, None] + squares[None, :])[strict]
    e_gpu = distance_errors(metric, got[strict], truth, norms)
    references = [("serial", oracle.symmetric(metric, dtype, vectors, row_start, row_count)[strict])]
    if reference_library() is not None and dtype not in support.DISPATCHED_DISTANCES_UNUSABLE:
        reference = reference_library()
        references.append(("dispatched", reference.symmetric(metric, dtype, vectors, row_start, row_count,
                                                              viable=reference.capabilities)[strict]))
    for name, ref in references:  # the gate of the packed distances
        e_ref = distance_errors(metric, ref, truth, norms)
        slack = U / np.sqrt(e_gpu.size)
        assert e_gpu.mean() <= 2 * e_ref.mean() + slack, f"mean error {e_gpu.mean():.3e} vs {name} {e_ref.mean():.3e} {where}"
        assert e_gpu.max() <= 2 * max(e_ref.max(), 2 * U), f"max error {e_gpu.max():.3e} vs {name} {e_ref.max():.3e} {where}"


# (count, depth, row_start, row_count): full calls and windows off every tile boundary, one ending past the last vector
SMALL_CASES = [(1, 1, 0, 1), (5, 7, 0, 5), (70, 200, 0, 70), (300, 64, 0, 300), (300, 64, 100, 77)]
LARGE_CASES = [(700, 130, 0, 700), (700, 130, 333, 1000), (1000, 515, 37, 411), (1000, 515, 992, 8), (2100, 96, 1055, 500)]


def cases_for(dtype, config, distances):
    """Every tile shape sees the small grids; the large ones (a CPU second or more each for the serial restatement of
    the float types) run under the heuristic and, one of them, under the two tile shapes it picks from most."""
    if dtype not in FLOAT_DTYPES and not distances:
        return SMALL_CASES + LARGE_CASES
    if config == 0:
        return SMALL_CASES + (LARGE_CASES[:4] if dtype not in FLOAT_DTYPES else LARGE_CASES[1:3])
    return SMALL_CASES + (LARGE_CASES[1:2] if config in (2, 3) else [])


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("config", [0, 1, 2, 3, 4])
def test_dots_windows_every_tile_config(oracle, dtype, config):
    rng = np.random.default_rng(500 + config)
    for count, depth, row_start, row_count in cases_for(dtype, config, False):
        vectors = support.random_matrix(oracle, dtype, count, depth, rng)
        check_dots(oracle, dtype, vectors, row_start, row_count, config,
                   f"{dtype} dots {count}x{depth} rows {row_start}+{row_count} config {config}")


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("config", [0, 1, 2, 3, 4])
def test_distance_windows_every_tile_config(oracle, dtype, metric, config):
    rng = np.random.default_rng(600 + config)
    for count, depth, row_start, row_count in cases_for(dtype, config, True):
        vectors = finite_inputs(oracle, dtype, count, depth, rng)
        if count > 60:
            vectors[row_start + 2] = 0                     # a zero vector in the window
            vectors[count - 1] = vectors[row_start + 3]    # two identical vectors off the diagonal
        check_distances(oracle, metric, dtype, vectors, row_start, row_count, config,
                        f"{dtype} {metric} {count}x{depth} rows {row_start}+{row_count} config {config}")


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", ALL_DTYPES + ("e3m2", "i4"))
@pytest.mark.parametrize("config", [0, 1, 2, 3, 4])
def test_diagonal_in_the_corner_of_a_tile(oracle, dtype, metric, config):
    """Windows that start one row past a 32-row boundary: the diagonal then runs through the bottom-left corner of
    32-row blocks, the only element of such a block on it. The self-distance must still be exactly 0
    (dots/serial.h:2866-2871), for every tile shape."""
    rng = np.random.default_rng(650 + config)
    for row_start in (1, 33, 65, 129):
        count, depth, row_count = 330, 64 if dtype != "i4" else 96, 200
        vectors = finite_inputs(oracle, dtype, count, depth, rng)
        check_distances(oracle, metric, dtype, vectors, row_start, row_count, config,
                        f"{dtype} {metric} {count}x{depth} rows {row_start}+{row_count} config {config}")


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(support.GOLDEN_DIR) if f.startswith("symmetric_")))
def test_golden_vectors(oracle, name):
    """Inputs and serial-kernel outputs recorded from the reference library (owned elements, zeros elsewhere)."""
    data = np.load(os.path.join(support.GOLDEN_DIR, name))
    dtype, vectors = str(data["dtype"]), data["vectors"]
    row_start, row_count = int(data["row_start"]), int(data["row_count"])
    count = vectors.shape[0]
    own = owned(count, row_start, row_count)
    check_dots(oracle, dtype, vectors, row_start, row_count, 0, name)
    bits = gpu_symmetric("dots", dtype, vectors, row_start, row_count)
    if dtype in support.INTEGER_DTYPES:
        assert np.array_equal(bits[own], data["dots_serial"].view(np.uint32)[own])
    for metric, key in (("angular", "angulars_serial"), ("euclidean", "euclideans_serial")):
        check_distances(oracle, metric, dtype, vectors, row_start, row_count, 0, name)
        got = gpu_symmetric(metric, dtype, vectors, row_start, row_count).view(np.float32)[own]
        recorded = data[key][own].astype(np.float64)
        if metric == "angular":
            assert np.abs(got - recorded).max() <= 16 * U
        else:
            assert np.abs(got - recorded).max() <= 16 * U * max(1.0, float(np.abs(recorded).max())) + 0.02  # cancelled rows


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_c_abi_host_pointers_strides_and_stream(oracle, dtype):
    """Host operands with padded strides (what lies left of the diagonal in the caller's result survives the round
    trip), then device operands on the caller's stream with a caller-owned workspace."""
    rng = np.random.default_rng(71)
    lib = nk.library()
    count, depth, pad, row_start, row_count = 77, 131, 5, 13, 40
    full = finite_inputs(oracle, dtype, count, depth + pad, rng)
    vectors = np.ascontiguousarray(full[:, :depth])
    own = owned(count, row_start, row_count)
    expected = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
    result = np.full((count, count + 3), POISON, np.uint32)
    getattr(lib, f"nk_dots_symmetric_{dtype}")(full.ctypes.data, count, depth, full.strides[0], result.ctypes.data,
                                                result.strides[0], row_start, row_count)
    assert not lib.nk_amd_last_error()
    assert (result[:, count:] == POISON).all() and (result[:, :count][~own] == POISON).all()
    if dtype in ("i8", "u8"):
        assert np.array_equal(result[:, :count][own], expected.view(np.uint32)[own])
    else:
        truth, magnitude = oracle.truth(dtype, vectors, vectors)
        assert_float_gate(dtype, result[:, :count].view(np.float32)[own], expected[own], truth[own], magnitude[own], f"{dtype} host")
    # device pointers, the three kinds, on the caller's stream
    code = api.DTYPES[dtype][0]
    width = vectors.itemsize
    gv = to_gpu(vectors)
    size = lib.nk_amd_symmetric_workspace_size(code, count, depth, row_start, row_count)
    workspace = torch.empty(size + 256, dtype=torch.uint8, device=DEV)
    aligned = (workspace.data_ptr() + 255) // 256 * 256
    stream = torch.cuda.current_stream().cuda_stream
    for metric in ("dots", "angular", "euclidean"):
        out = torch.full((count, count), POISON, dtype=torch.int32, device=DEV)
        args = (support.SYMMETRIC_KINDS[metric], code, gv.data_ptr(), count, depth, depth * width, out.data_ptr(), count * 4,
                row_start, row_count, aligned)
        assert lib.nk_amd_symmetric_async(*args, size - 1, stream) != 0 and b"workspace too small" in lib.nk_hip_last_error()
        assert lib.nk_amd_symmetric_async(*args, size, stream) == 0, lib.nk_hip_last_error()
        torch.cuda.synchronize()
        bits = out.cpu().numpy().view(np.uint32)
        assert (bits[~own] == POISON).all()
        assert np.array_equal(bits, gpu_symmetric(metric, dtype, vectors, row_start, row_count)), metric  # same kernels, same bits


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_full_size_equals_packed_kinds_and_windows_tile(oracle, dtype):
    """4096 vectors of depth 1024: the upper triangle is, bit for bit, the packed kind with both sides the same (one
    accumulation order per output, whatever the tile grid); four uneven row windows reproduce the single call; a
    sample of rows agrees with the oracle."""
    count, depth = 4096, 1024
    rng = np.random.default_rng(73)
    vectors = finite_inputs(oracle, dtype, count, depth, rng)
    gv = to_gpu(vectors)
    packed = nk.dots_pack(gv, dtype)
    upper = torch.triu(torch.ones((count, count), dtype=torch.bool, device=DEV))
    strict = torch.triu(torch.ones((count, count), dtype=torch.bool, device=DEV), 1)
    for metric, packed_call in (("dots", nk.dots_packed), ("angular", nk.angulars_packed), ("euclidean", nk.euclideans_packed)):
        whole = GPU_CALL[metric](gv, dtype)
        rectangle = packed_call(gv, packed)
        mask = upper if metric == "dots" else strict
        assert torch.equal(whole.view(torch.int32)[mask], rectangle.view(torch.int32)[mask]), metric
        assert not whole.view(torch.int32)[~upper].any()  # a fresh result is zero-filled by the Python mirror
        if metric != "dots":
            assert not torch.diagonal(whole.view(torch.int32)).any()
        pieces = torch.zeros_like(whole)
        for start, end in ((0, 100), (100, 1500), (1500, 1501), (1501, count)):
            GPU_CALL[metric](gv, dtype, out=pieces, start_row=start, end_row=end)
        assert torch.equal(pieces.view(torch.int32), whole.view(torch.int32)), metric
    rows = np.array([0, 1, 777, 2048, 4095])
    sample = nk.dots_symmetric(gv, dtype)[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    for at, row in enumerate(rows):
        reference_row = oracle.dots_packed(dtype, vectors[row:row + 1], vectors[row:])[0]
        if dtype in ("i8", "u8"):
            assert np.array_equal(sample[at, row:].view(np.uint32), reference_row.view(np.uint32))
        else:
            truth, magnitude = oracle.truth(dtype, vectors[row:row + 1], vectors[row:])
            assert_float_gate(dtype, sample[at, row:], reference_row, truth[0], magnitude[0], f"{dtype} row {row}")


def test_degenerate_calls(oracle):
    """Depth 0 gives zero dots and zero distances on the owned elements; empty windows and windows past the end write
    nothing; the Python mirror refuses an inverted window."""
    vectors = torch.zeros((40, 0), dtype=torch.int8, device=DEV)
    own = owned(40, 3, 20)
    for metric in GPU_CALL:
        out = torch.full((40, 40), POISON, dtype=torch.int32, device=DEV)
        GPU_CALL[metric](vectors, "i8", out=out.view(torch.float32) if metric != "dots" else out, start_row=3, end_row=23)
        bits = out.cpu().numpy().view(np.uint32)
        assert (bits[own] == 0).all() and (bits[~own] == POISON).all()
    rng = np.random.default_rng(79)
    gv = to_gpu(support.random_matrix(oracle, "bf16", 50, 64, rng))
    out = torch.full((50, 50), POISON, dtype=torch.int32, device=DEV).view(torch.float32)
    nk.dots_symmetric(gv, "bf16", out=out, start_row=20, end_row=20)
    lib = nk.library()
    lib.nk_dots_symmetric_bf16(gv.data_ptr(), 50, 64, 128, out.data_ptr(), 200, 50, 10)  # starts past the last vector
    assert not lib.nk_amd_last_error()
    assert (out.view(torch.int32).cpu().numpy().view(np.uint32) == POISON).all()
    with pytest.raises(ValueError):
        nk.dots_symmetric(gv, "bf16", start_row=30, end_row=20)
