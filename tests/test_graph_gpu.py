"""The asynchronous entry points under HIP graph capture, on a real MI355X.

`nk_amd_dots_packed_async`, `nk_amd_spatials_packed_async` and `nk_amd_symmetric_async` only launch kernels on the
caller's stream (no allocation, no synchronisation, no memset), so a caller may record them into a graph once and
replay it: the serving-loop form of `nk_dots_packed_<T>` (reference include/numkong/dots.h:248-287, which has no
stream notion of its own). Every replay is checked against the eager result bit for bit, with eager work and
synchronisations of the program's own between the replays, and with the inputs changed between two of them.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from tests import support  # noqa: E402
from tests.test_dots_gpu import DEV, to_gpu  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["i8", "bf16", "e2m3", "f32"])
def test_packed_product_and_distances_replay(oracle, dtype):
    rng = np.random.default_rng(8000)
    m, n, k = 300, 700, 1024
    a = to_gpu(support.random_matrix(oracle, dtype, m, k, rng))
    other = to_gpu(support.random_matrix(oracle, dtype, m, k, rng))
    packed = nk.dots_pack(to_gpu(support.random_matrix(oracle, dtype, n, k, rng)), dtype)
    lib, code = nk.library(), nk.api.DTYPES[dtype][0]
    eager = nk.dots_packed(a, packed).clone()  # (also the warm-up call: kernels loaded, occupancy queried)
    eager_angular = nk.angulars_packed(a, packed).clone()
    out, out_angular = torch.zeros_like(eager), torch.zeros_like(eager_angular)
    row_bytes, out_bytes = a.stride(0) * a.element_size(), out.stride(0) * out.element_size()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):  # (the synchronous entry points of the Python mirror wait for the device: not for capture)
        stream = torch.cuda.current_stream().cuda_stream
        assert lib.nk_amd_dots_packed_async(code, a.data_ptr(), packed.buffer.data_ptr(), out.data_ptr(), m, n, packed.depth,
                                            row_bytes, out_bytes, stream) == 0
        assert lib.nk_amd_spatials_packed_async(support.KIND_ANGULARS, code, a.data_ptr(), packed.buffer.data_ptr(),
                                                out_angular.data_ptr(), m, n, packed.depth, row_bytes, out_bytes, stream) == 0
    for replay in range(4):
        out.fill_(0), out_angular.fill_(0)  # eager work between the replays
        if replay == 2:  # new queries in the same buffer: the graph reads the buffer, not a snapshot
            a.copy_(other)
            eager, eager_angular = nk.dots_packed(a, packed).clone(), nk.angulars_packed(a, packed).clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.uint8), eager.view(torch.uint8)), f"{dtype} product, replay {replay}"
        assert torch.equal(out_angular.view(torch.uint8), eager_angular.view(torch.uint8)), f"{dtype} angular, replay {replay}"


def test_symmetric_call_replays_with_the_callers_workspace(oracle):
    rng = np.random.default_rng(8001)
    count, depth = 520, 256
    lib = nk.library()
    code = nk.api.DTYPES["i8"][0]
    vectors = to_gpu(support.random_matrix(oracle, "i8", count, depth, rng))
    eager = nk.dots_symmetric(vectors, "i8").clone()
    workspace = torch.empty(lib.nk_amd_symmetric_workspace_size(code, count, depth, 0, count) + 256, dtype=torch.uint8, device=DEV)
    base = (workspace.data_ptr() + 255) // 256 * 256
    out = torch.zeros((count, count), dtype=torch.int32, device=DEV)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = lib.nk_amd_symmetric_async(support.SYMMETRIC_KINDS["dots"], code, vectors.data_ptr(), count, depth, depth,
                                            out.data_ptr(), count * 4, 0, count, base, workspace.numel() - 256,
                                            torch.cuda.current_stream().cuda_stream)
        assert status == 0
    for replay in range(3):
        out.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay}"
