"""The containers over the C ABI: include/numkong_amd/matrix.hpp (C++: typed entry points, owning packed_matrix) through
the program tests/cpp/test_matrix.cpp, and the Python PackedMatrix (`a @ packed`, DLPack operands).

Reference counterparts: include/numkong/matrix.hpp:170-253, include/numkong/dots.hpp:94-150, python/matrix.c:151-227,
324-490, python/dlpack_interop.c."""
import os
import subprocess

import numpy as np
import pytest

import numkong_amd as nk
from tests import support

PROGRAM = os.path.join(support.ROOT, "numkong_amd", "lib", "test_matrix")


def run_program():
    if not os.path.exists(PROGRAM):
        pytest.fail(f"{PROGRAM} is missing: build it with `make -C numkong_amd/csrc`")
    done = subprocess.run([PROGRAM], capture_output=True, text=True, timeout=300)
    return done.returncode, done.stdout + done.stderr


def test_cpp_containers_without_a_gpu_refuse_cleanly():
    if nk.library().nk_hip_device_count() > 0:
        pytest.skip("a GPU is present: covered by the GPU test")
    code, text = run_program()
    assert code == 0 and "FAILED" not in text and "containers refuse cleanly" in text, text


@pytest.mark.gpu
def test_cpp_containers_on_the_gpu():
    code, text = run_program()
    assert code == 0 and "FAILED" not in text and "all container checks passed" in text, text
    assert text.count("ok:") >= 9


@pytest.mark.gpu
def test_python_packed_matrix_operator_and_dlpack(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(91)
    a, b = support.random_matrix(oracle, "i8", 33, 100, rng), support.random_matrix(oracle, "i8", 21, 100, rng)
    ga, gb = torch.from_numpy(a).to("cuda:0"), torch.from_numpy(b).to("cuda:0")
    packed = nk.dots_pack(gb, "i8")
    assert packed.shape == (21, 100) and packed.nbytes == nk.dots_packed_size("i8", 21, 100)
    assert type(packed).packed_size(21, 100, dtype="i8") == packed.nbytes and (packed.width, packed.depth, packed.dtype) == (21, 100, "i8")
    expected = a.astype(np.int64) @ b.astype(np.int64).T
    assert np.array_equal((ga @ packed).cpu().numpy(), expected)

    class Exporter:  # any object that exports DLPack, not a torch.Tensor
        def __init__(self, tensor):
            self.tensor = tensor

        def __dlpack__(self, **kwargs):
            return self.tensor.__dlpack__(**kwargs)

        def __dlpack_device__(self):
            return self.tensor.__dlpack_device__()

    again = nk.dots_packed(Exporter(ga), nk.dots_pack(Exporter(gb), "i8"))
    assert np.array_equal(again.cpu().numpy(), expected)
    # a window of rows, as the reference's start_row / end_row: the other rows of out stay as they were
    window = torch.full((33, 21), -7, dtype=torch.int32, device="cuda:0")
    assert nk.dots_packed(ga, packed, out=window, start_row=5, end_row=20) is window
    kept = np.full((33, 21), -7, np.int64)
    kept[5:20] = expected[5:20]
    assert np.array_equal(window.cpu().numpy(), kept)
    with pytest.raises(ValueError):
        nk.dots_packed(ga, packed, start_row=20, end_row=5)


@pytest.mark.gpu
def test_python_dtype_is_inferred_from_the_tensor(oracle):
    """``dots_pack(b)`` and the symmetric calls without a dtype take it from the tensor's element type, as the
    reference's ``dtype=None`` does (python/matrix.c:632-647); the types that have no tensor type must be named."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(92)
    a, b = support.random_matrix(oracle, "bf16", 20, 96, rng), support.random_matrix(oracle, "bf16", 30, 96, rng)
    ga, gb = torch.from_numpy(a).to("cuda:0").view(torch.bfloat16), torch.from_numpy(b).to("cuda:0").view(torch.bfloat16)
    packed = nk.dots_pack(gb)
    assert packed.dtype == "bf16"
    named = nk.dots_packed(torch.from_numpy(a).to("cuda:0"), nk.dots_pack(torch.from_numpy(b).to("cuda:0"), "bf16"))
    assert torch.equal(nk.dots_packed(ga, packed), named)
    bytes_ = torch.from_numpy(rng.integers(0, 256, (12, 64), dtype=np.uint8)).to("cuda:0")
    assert nk.dots_pack(bytes_).dtype == "u8"
    signed = torch.from_numpy(rng.integers(-128, 128, (12, 64), dtype=np.int8)).to("cuda:0")
    assert torch.equal(nk.dots_symmetric(signed), nk.dots_symmetric(signed, "i8"))
    assert torch.equal(nk.angulars_symmetric(ga), nk.angulars_symmetric(torch.from_numpy(a).to("cuda:0"), "bf16"))
    with pytest.raises(TypeError):
        nk.dots_pack(torch.zeros((4, 8), dtype=torch.int32, device="cuda:0"))


@pytest.mark.gpu
def test_python_host_operands(oracle):
    """What a caller of the reference has: numpy arrays (and torch CPU tensors) in host memory. The library stages them,
    the packed image stays in host memory and is uploaded once, results come back as host arrays of the caller's kind."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(93)
    a = rng.integers(-128, 128, (45, 200), dtype=np.int8)
    b = rng.integers(-128, 128, (70, 200), dtype=np.int8)
    expected = a.astype(np.int64) @ b.astype(np.int64).T
    packed = nk.dots_pack(b)  # dtype from the array
    assert packed.dtype == "i8" and not packed.buffer.is_cuda and packed.nbytes == nk.dots_packed_size("i8", 70, 200)
    c = nk.dots_packed(a, packed, threads=8)  # (the reference's callers pass it; the GPU has its own parallelism)
    assert isinstance(c, np.ndarray) and c.dtype == np.int32 and np.array_equal(c, expected)
    assert np.array_equal(a @ packed, expected)  # numpy hands the operator to PackedMatrix.__rmatmul__
    out = np.full((45, 70), -3, np.int32)
    assert nk.dots_packed(a, packed, out=out, start_row=10, end_row=30) is out
    assert np.array_equal(out[10:30], expected[10:30]) and (out[:10] == -3).all() and (out[30:] == -3).all()
    # torch CPU tensors give torch CPU tensors; a host A against an image in GPU memory works as well
    on_gpu = nk.dots_pack(torch.from_numpy(b).to("cuda:0"))
    c_cpu = nk.dots_packed(torch.from_numpy(a), on_gpu)
    assert isinstance(c_cpu, torch.Tensor) and not c_cpu.is_cuda and np.array_equal(c_cpu.numpy(), expected)
    # raw bf16 bits in a uint16 array: the dtype has to be named; results equal the GPU-resident call bit for bit
    a16, b16 = support.random_matrix(oracle, "bf16", 33, 128, rng), support.random_matrix(oracle, "bf16", 40, 128, rng)
    host = nk.dots_packed(a16.view(np.uint16), nk.dots_pack(b16.view(np.uint16), "bf16"))
    resident = nk.dots_packed(torch.from_numpy(a16).to("cuda:0"), nk.dots_pack(torch.from_numpy(b16).to("cuda:0"), "bf16"))
    assert host.dtype == np.float32 and np.array_equal(host.view(np.uint32), resident.cpu().numpy().view(np.uint32))
    gram = nk.dots_symmetric(a)
    assert isinstance(gram, np.ndarray) and np.array_equal(np.triu(gram), np.triu(a.astype(np.int64) @ a.astype(np.int64).T))
    distances = nk.angulars_packed(a16.view(np.uint16), nk.dots_pack(b16.view(np.uint16), "bf16"))
    on_device = nk.angulars_packed(torch.from_numpy(a16).to("cuda:0"), nk.dots_pack(torch.from_numpy(b16).to("cuda:0"), "bf16"))
    assert np.array_equal(distances.view(np.uint32), on_device.cpu().numpy().view(np.uint32))
    nk.library().nk_hip_image_cache_clear()
