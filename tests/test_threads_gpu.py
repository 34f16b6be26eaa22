"""Concurrent callers against one shared packed B, on a real MI355X, through the C ABI.

The reference's callers split A into 64-row tiles and hand them to their own threads, every thread calling
`nk_dots_packed_<T>` on its tiles against the one read-only packed B (include/README.md:549-560,
python/matrix.c:466-483), after `nk_configure_thread` once per thread. The calls must be safe side by side and the
assembled C must equal, bit for bit, what one call over all of A gives. Checked with the packed B in device memory and
with everything in host memory (where the calls also share the device copy of the image that the library keeps)."""
import ctypes
import queue
import threading

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from tests import support  # noqa: E402
from tests.test_dots_gpu import DEV, to_gpu  # noqa: E402

pytestmark = pytest.mark.gpu
THREADS, TILE = 8, 64


def run_tiles(call, rows):
    """`call(first, count)` for every 64-row tile of `rows` rows, handed out to THREADS host threads."""
    lib = nk.library()
    tiles: "queue.SimpleQueue[int]" = queue.SimpleQueue()
    for first in range(0, rows, TILE):
        tiles.put(first)
    failures = []

    def worker():
        lib.nk_configure_thread(ctypes.c_uint64(lib.nk_capabilities()))
        while True:
            try:
                first = tiles.get_nowait()
            except queue.Empty:
                return
            call(first, min(TILE, rows - first))
            message = lib.nk_amd_last_error()
            if message:
                failures.append(message.decode())

    threads = [threading.Thread(target=worker) for _ in range(THREADS)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[:3]


@pytest.mark.parametrize("dtype", ["i8", "bf16"])
def test_row_tiles_from_eight_threads_device_operands(oracle, dtype):
    m, n, k = 1500, 1111, 1000
    rng = np.random.default_rng(910)
    a_host = support.random_matrix(oracle, dtype, m, k, rng)
    b_host = support.random_matrix(oracle, dtype, n, k, rng)
    a, packed = to_gpu(a_host), nk.dots_pack(to_gpu(b_host), dtype)
    whole = nk.dots_packed(a, packed)
    out_dtype = torch.int32 if dtype == "i8" else torch.float32
    lib = nk.library()
    entry = getattr(lib, f"nk_dots_packed_{dtype}")
    row_bytes, out_stride = a.shape[1] * a.element_size(), n * 4
    for attempt in range(3):
        pieces = torch.full((m, n), -1, dtype=torch.int32, device=DEV).view(out_dtype)
        torch.cuda.synchronize()

        def call(first, count):
            entry(a.data_ptr() + first * row_bytes, packed.buffer.data_ptr(), pieces.data_ptr() + first * out_stride,
                  count, n, k, row_bytes, out_stride)

        run_tiles(call, m)
        assert torch.equal(pieces.view(torch.int32), whole.view(torch.int32)), f"{dtype} attempt {attempt}"
    if dtype == "i8":
        exact = a_host.astype(np.int64) @ b_host.astype(np.int64).T
        assert np.array_equal(whole.cpu().numpy().astype(np.int64), exact)


@pytest.mark.parametrize("dtype", ["i8", "bf16"])
def test_row_tiles_from_eight_threads_host_operands(oracle, dtype):
    """Everything in plain host memory, as a caller of the reference's library has it."""
    m, n, k = 700, 515, 520
    rng = np.random.default_rng(911)
    a = support.random_matrix(oracle, dtype, m, k, rng)
    b = support.random_matrix(oracle, dtype, n, k, rng)
    lib = nk.library()
    size = nk.dots_packed_size(dtype, n, k)
    image = np.zeros(size, np.uint8)
    getattr(lib, f"nk_dots_pack_{dtype}")(b.ctypes.data, n, k, b.strides[0], image.ctypes.data)
    assert not lib.nk_amd_last_error()
    entry = getattr(lib, f"nk_dots_packed_{dtype}")
    whole = np.empty((m, n), support.OUTPUT[dtype])
    entry(a.ctypes.data, image.ctypes.data, whole.ctypes.data, m, n, k, a.strides[0], whole.strides[0])
    assert not lib.nk_amd_last_error()
    pieces = np.full((m, n), -1, np.int32).view(support.OUTPUT[dtype])

    def call(first, count):
        entry(a.ctypes.data + first * a.strides[0], image.ctypes.data, pieces.ctypes.data + first * pieces.strides[0],
              count, n, k, a.strides[0], pieces.strides[0])

    run_tiles(call, m)
    assert np.array_equal(pieces.view(np.uint32), whole.view(np.uint32))
    if dtype == "i8":
        assert np.array_equal(whole.astype(np.int64), a.astype(np.int64) @ b.astype(np.int64).T)
    else:
        assert np.array_equal(whole.view(np.uint32), nk.dots_packed(to_gpu(a), nk.dots_pack(to_gpu(b), dtype)).cpu().numpy().view(np.uint32))


@pytest.mark.parametrize("dtype", ["i8", "bf16"])
def test_eight_threads_miss_the_image_cache_at_once(oracle, dtype):
    """A host image that no earlier call has uploaded (packed on the device, then copied to the host): the first calls
    from eight threads all miss the cache of device copies together. One of them uploads the image, the others wait for
    that copy, and nobody may multiply with a copy whose transfers are still in flight. The image is large enough to go
    up in several pieces."""
    m, n, k = 512, 4100, 4096 if dtype == "i8" else 2048
    rng = np.random.default_rng(913)
    a = support.random_matrix(oracle, dtype, m, k, rng)
    b = support.random_matrix(oracle, dtype, n, k, rng)
    lib = nk.library()
    entry = getattr(lib, f"nk_dots_packed_{dtype}")
    expected = nk.dots_packed(to_gpu(a), nk.dots_pack(to_gpu(b), dtype)).cpu().numpy()
    for attempt in range(3):
        lib.nk_hip_image_cache_clear()
        image = nk.dots_pack(to_gpu(b), dtype).buffer.cpu().numpy()  # a fresh number in its header every time
        assert image.nbytes > 16 << 20
        pieces = np.full((m, n), -1, np.int32).view(support.OUTPUT[dtype])
        start = threading.Barrier(THREADS)

        def call(first, count):
            entry(a.ctypes.data + first * a.strides[0], image.ctypes.data, pieces.ctypes.data + first * pieces.strides[0],
                  count, n, k, a.strides[0], pieces.strides[0])

        failures = []

        def worker(index):
            lib.nk_configure_thread(ctypes.c_uint64(lib.nk_capabilities()))
            start.wait()
            call(index * TILE, TILE)
            message = lib.nk_amd_last_error()
            if message:
                failures.append(message.decode())

        threads = [threading.Thread(target=worker, args=(index,)) for index in range(THREADS)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not failures, failures[:3]
        assert np.array_equal(pieces.view(np.uint32), expected.view(np.uint32)), f"{dtype} attempt {attempt}"
    lib.nk_hip_image_cache_clear()


def test_tile_config_hook_is_per_thread():
    """The test hook that forces a tile shape reaches the calling thread's launches only."""
    lib = nk.library()
    rng = np.random.default_rng(912)
    a = torch.from_numpy(rng.integers(-128, 128, (300, 256), dtype=np.int8)).to(DEV)
    packed = nk.dots_pack(torch.from_numpy(rng.integers(-128, 128, (200, 256), dtype=np.int8)).to(DEV), "i8")
    expected = nk.dots_packed(a, packed)
    results = {}

    def other():
        lib.nk_hip_set_tile_config(4)
        results["other"] = nk.dots_packed(a, packed)

    lib.nk_hip_set_tile_config(2)
    try:
        t = threading.Thread(target=other)
        t.start()
        t.join()
        results["mine"] = nk.dots_packed(a, packed)
    finally:
        lib.nk_hip_set_tile_config(0)
    assert torch.equal(results["mine"], expected) and torch.equal(results["other"], expected)


def test_staging_buffers_are_kept_and_trimmed():
    """A thread's staging buffers stay between calls; `nk_hip_thread_trim` gives back the slots larger than its first
    argument, then everything if more than its second is still held; a host-pointer product afterwards works as
    before (gfx950.c keeps 256 MiB per slot and 2 GiB per thread this way)."""
    lib = nk.library()
    lib.nk_hip_thread_buffer.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
    lib.nk_hip_thread_buffer.restype = ctypes.c_int
    lib.nk_hip_thread_cached_bytes.restype = ctypes.c_size_t
    lib.nk_hip_thread_trim.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
    lib.nk_hip_thread_trim.restype = None
    lib.nk_hip_thread_release.restype = None
    lib.nk_hip_thread_release()
    assert lib.nk_hip_thread_cached_bytes() == 0
    small, large, again = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.nk_hip_thread_buffer(0, 0, 1 << 20, ctypes.byref(small)) == 0 and small.value
    assert lib.nk_hip_thread_buffer(1, 1, 3 << 20, ctypes.byref(large)) == 0 and large.value
    held = lib.nk_hip_thread_cached_bytes()
    assert held >= (1 << 20) + (3 << 20)
    assert lib.nk_hip_thread_buffer(0, 0, 1 << 19, ctypes.byref(again)) == 0 and again.value == small.value  # kept, not regrown
    assert lib.nk_hip_thread_cached_bytes() == held
    lib.nk_hip_thread_trim(2 << 20, 1 << 30)  # the 3 MiB slot goes, the 1 MiB slot stays
    assert (1 << 20) <= lib.nk_hip_thread_cached_bytes() < (3 << 20)
    lib.nk_hip_thread_trim(1 << 30, 1 << 19)  # more than the total cap is still held: everything goes
    assert lib.nk_hip_thread_cached_bytes() == 0
    rng = np.random.default_rng(914)
    a = rng.integers(-128, 128, (70, 200), dtype=np.int8)
    b = rng.integers(-128, 128, (90, 200), dtype=np.int8)
    packed = nk.dots_pack(to_gpu(b), "i8").buffer.cpu().numpy()
    c = np.full((70, 90), -1, np.int32)
    lib.nk_dots_packed_i8(a.ctypes.data, packed.ctypes.data, c.ctypes.data, 70, 90, 200, a.strides[0], c.strides[0])
    assert not lib.nk_amd_last_error()
    assert np.array_equal(c.astype(np.int64), a.astype(np.int64) @ b.astype(np.int64).T)
    assert lib.nk_hip_thread_cached_bytes() > 0
    lib.nk_hip_thread_release()
    lib.nk_hip_image_cache_clear()


def test_image_cache_claim_abandon_publish():
    """The life of a cache entry as the host layer drives it: the first claim of an unknown image reserves it (2), an
    abandoned reservation leaves no trace, a published copy is found by later claims (1) until the cache is cleared."""
    lib = nk.library()
    for name in ("nk_hip_image_cache_claim", "nk_hip_image_cache_find"):
        getattr(lib, name).argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
        getattr(lib, name).restype = ctypes.c_int
    lib.nk_hip_image_cache_publish.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.nk_hip_image_cache_publish.restype = ctypes.c_int
    lib.nk_hip_image_cache_abandon.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    lib.nk_hip_image_cache_abandon.restype = None
    lib.nk_hip_image_cache_release.argtypes = [ctypes.c_void_p]
    lib.nk_hip_image_cache_release.restype = None
    lib.nk_hip_image_cache_clear()
    rng = np.random.default_rng(915)
    b = rng.integers(-128, 128, (64, 128), dtype=np.int8)
    packed = nk.dots_pack(to_gpu(b), "i8")
    image = packed.buffer.cpu().numpy()
    where = ctypes.c_void_p()
    assert lib.nk_hip_image_cache_find(image.ctypes.data, image.nbytes, ctypes.byref(where)) == 0
    assert lib.nk_hip_image_cache_claim(image.ctypes.data, image.nbytes, ctypes.byref(where)) == 2 and not where.value
    lib.nk_hip_image_cache_abandon(image.ctypes.data, image.nbytes)
    assert lib.nk_hip_image_cache_find(image.ctypes.data, image.nbytes, ctypes.byref(where)) == 0
    assert lib.nk_hip_image_cache_claim(image.ctypes.data, image.nbytes, ctypes.byref(where)) == 2
    # the cache owns what is published to it and frees it when the entry goes: give it memory of the library's own
    lib.nk_hip_malloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    copy = ctypes.c_void_p()
    assert lib.nk_hip_malloc(ctypes.byref(copy), image.nbytes) == 0
    lib.nk_hip_memcpy_h2d.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    assert lib.nk_hip_memcpy_h2d(copy, image.ctypes.data, image.nbytes, None) == 0
    torch.cuda.synchronize()
    assert lib.nk_hip_image_cache_publish(image.ctypes.data, image.nbytes, copy) == 1
    lib.nk_hip_image_cache_release(copy)  # the uploader's own use of it
    assert lib.nk_hip_image_cache_claim(image.ctypes.data, image.nbytes, ctypes.byref(where)) == 1 and where.value == copy.value
    lib.nk_hip_image_cache_release(where)
    # a product with the host image now runs against that copy
    a = rng.integers(-128, 128, (40, 128), dtype=np.int8)
    c = np.full((40, 64), -1, np.int32)
    lib.nk_dots_packed_i8(a.ctypes.data, image.ctypes.data, c.ctypes.data, 40, 64, 128, a.strides[0], c.strides[0])
    assert not lib.nk_amd_last_error()
    assert np.array_equal(c.astype(np.int64), a.astype(np.int64) @ b.astype(np.int64).T)
    lib.nk_hip_image_cache_clear()
    assert lib.nk_hip_image_cache_find(image.ctypes.data, image.nbytes, ctypes.byref(where)) == 0
