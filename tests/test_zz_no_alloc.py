"""The entry point that allocates nothing, `nk_amd_symmetric_static_async`, against `nk_amd_symmetric_async`.

Both run the same kernels; the first takes its workspace from a fixed array in device memory instead of an argument.
Two calls in a row, the second with a smaller input, so that whatever the first left in the shared array would show;
every kind and several element types; bit for bit. Sizes past the array's capacity must be refused with a message."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from numkong_amd import api  # noqa: E402
from tests import support  # noqa: E402
from tests.test_dots_gpu import DEV, to_gpu  # noqa: E402
from tests.test_spatials_gpu import finite_inputs  # noqa: E402

pytestmark = pytest.mark.gpu
POISON = 0x7FC12345


def both_ways(lib, metric, dtype, vectors, row_start, row_count):
    count, depth = vectors.shape[0], support.depth_of(dtype, vectors)
    code, kind = api.DTYPES[dtype][0], support.SYMMETRIC_KINDS[metric]
    gv = to_gpu(vectors)
    stride = gv.shape[1] * gv.element_size()
    stream = torch.cuda.current_stream().cuda_stream
    size = lib.nk_amd_symmetric_workspace_size(code, count, depth, row_start, row_count)
    workspace = torch.empty(size, dtype=torch.uint8, device=DEV)
    expected = torch.full((count, count), POISON, dtype=torch.int32, device=DEV)
    assert lib.nk_amd_symmetric_async(kind, code, gv.data_ptr(), count, depth, stride, expected.data_ptr(), count * 4, row_start,
                                      row_count, workspace.data_ptr(), size, stream) == 0, lib.nk_hip_last_error()
    got = torch.full((count, count), POISON, dtype=torch.int32, device=DEV)
    assert lib.nk_amd_symmetric_static_async(kind, code, gv.data_ptr(), count, depth, stride, got.data_ptr(), count * 4, row_start,
                                             row_count, stream) == 0, lib.nk_hip_last_error()
    torch.cuda.synchronize()
    return got.cpu().numpy().view(np.uint32), expected.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("dtype", ["i8", "u8", "bf16", "e4m3"])
def test_static_workspace_matches_callers_workspace(oracle, dtype):
    lib = nk.library()
    rng = np.random.default_rng(2024)
    # the second call is smaller than the first in count and depth, and starts off a tile boundary
    for count, depth, row_start, row_count in [(700, 515, 0, 700), (300, 130, 37, 200)]:
        vectors = finite_inputs(oracle, dtype, count, depth, rng)
        for metric in ("dots", "angular", "euclidean"):
            got, expected = both_ways(lib, metric, dtype, vectors, row_start, row_count)
            assert np.array_equal(got, expected), f"{dtype} {metric} {count}x{depth} rows {row_start}+{row_count}"
            own = (np.arange(count)[:, None] >= row_start) & (np.arange(count)[:, None] < row_start + row_count) & \
                  (np.arange(count)[None, :] >= np.arange(count)[:, None])
            assert (got[~own] == POISON).all() and (got[own] != POISON).any()
    if dtype == "i8":  # and against the closed form, so that both being wrong the same way would show
        vectors = finite_inputs(oracle, dtype, 300, 130, rng)
        got, _ = both_ways(lib, "dots", dtype, vectors, 0, 300)
        exact = (vectors.astype(np.int64) @ vectors.astype(np.int64).T) & 0xFFFFFFFF
        upper = np.triu(np.ones((300, 300), dtype=bool))
        assert np.array_equal(got[upper].astype(np.int64), exact[upper])


def test_sizes_past_the_capacity_are_refused():
    lib = nk.library()
    capacity = lib.nk_amd_symmetric_static_capacity()
    assert capacity == 32 << 20
    count, depth = 8192, 8192  # a 64 MiB image
    code = api.DTYPES["i8"][0]
    assert lib.nk_amd_symmetric_workspace_size(code, count, depth, 0, count) > capacity
    vectors = torch.zeros((count, depth), dtype=torch.int8, device=DEV)
    result = torch.full((count, count), POISON, dtype=torch.int32, device=DEV)
    status = lib.nk_amd_symmetric_static_async(support.SYMMETRIC_KINDS["dots"], code, vectors.data_ptr(), count, depth, depth,
                                               result.data_ptr(), count * 4, 0, count, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert status != 0 and b"needs" in lib.nk_hip_last_error() and b"holds" in lib.nk_hip_last_error()
    assert (result.cpu().numpy().view(np.uint32) == POISON).all()  # nothing was launched
