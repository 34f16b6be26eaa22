"""Parity of the narrow types of the dots family (e2m3, e3m2, i4, u4, u1) with the reference, through the C ABI, on a real MI355X.

`nk_dots_packed_size_<T>`, `nk_dots_pack_<T>`, `nk_dots_packed_<T>`, `nk_dots_symmetric_<T>` for the 6-bit floats (one
per byte), the 4-bit integers (two per byte, depth counted in 4-bit values) and single bits (eight per byte, depth in
bits, the product is the popcount of the AND): reference include/numkong/dots/serial.h:2601-2695, arithmetic in
include/numkong/dot/serial.h:602-832. On the GPU the 6-bit floats are widened, exactly, to f16 and the 4-bit integers
and the bits to i8, B at pack time and A on its way into LDS.

  * i4 / u4 / u1: bit-exact against the oracle's restatement of the serial kernels and against numpy int64 products of the
    unpacked nibbles;
  * e2m3 / e3m2: the float gate of tests/test_dots_gpu.py against the serial restatement and the host-dispatched kernel;
    where every partial sum is exact in f32 (short depths: all values are multiples of 1/16 below 32) bit-exact as well;
  * the widening itself: all 256 byte values, on the A side and on the B side, one at a time against a unit vector;
  * the distance kinds of e2m3, e3m2, i4, u4 (`nk_{angulars,euclideans}_{packed,symmetric}_<T>`, reference
    include/numkong/spatials/serial.h:143-240): the gates of tests/test_spatials_gpu.py and tests/test_symmetric_gpu.py
    (f32 outputs: error against the f64 truth next to the serial kernel's; for i4 the serial kernel only, see
    tests/support.py). u1 has no distance kinds and is refused.
"""
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from tests import support  # noqa: E402
from tests.support import NARROW_DTYPES, NARROW_FLOAT_DTYPES, NARROW_INT_DTYPES  # noqa: E402
from tests.test_dots_gpu import DEV, assert_float_gate, best_dispatch, gpu_dots, to_gpu  # noqa: E402
from tests.test_spatials_gpu import assert_distance_gate, gpu_distances  # noqa: E402
from tests.test_symmetric_gpu import POISON, check_distances, gpu_symmetric, owned, reference_library  # noqa: E402

pytestmark = pytest.mark.gpu


def unpack_nibbles(dtype, x):
    """The integer values behind the bytes of a sub-byte type, low bits first."""
    if dtype == "u1":
        return np.unpackbits(x, axis=1, bitorder="little").astype(np.int64)
    nibbles = np.stack([x & 0xF, x >> 4], axis=-1).reshape(x.shape[0], -1).astype(np.int64)
    return np.where(nibbles >= 8, nibbles - 16, nibbles) if dtype == "i4" else nibbles


def check(oracle, dtype, a, b, config=0, where=""):
    got = gpu_dots(dtype, a, b, config)
    serial = oracle.dots_packed(dtype, a, b)
    if dtype in NARROW_INT_DTYPES:
        exact = (unpack_nibbles(dtype, a) @ unpack_nibbles(dtype, b).T) & 0xFFFFFFFF
        assert np.array_equal(got.view(np.uint32).astype(np.int64), exact), where
        assert np.array_equal(got.view(np.uint32), serial.view(np.uint32)), where
    else:
        truth, magnitude = oracle.truth(dtype, a, b)
        assert_float_gate(dtype, got, serial, truth, magnitude, where, best_dispatch(dtype, a, b))


# (m, n, depth in dimensions): odd depths leave half a byte over for the 4-bit types
SHAPES = [(1, 1, 1), (3, 5, 7), (33, 70, 200), (64, 64, 64), (100, 37, 333), (257, 129, 1000), (31, 300, 130), (130, 33, 4100)]


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
@pytest.mark.parametrize("config", [0, 1, 2, 3, 4])
def test_small_shapes_every_tile_config(oracle, dtype, config):
    rng = np.random.default_rng(700 + config)
    for m, n, k in SHAPES:
        a = support.random_matrix(oracle, dtype, m, k, rng)
        b = support.random_matrix(oracle, dtype, n, k, rng)
        check(oracle, dtype, a, b, config, f"{dtype} {m}x{n}x{k} config {config}")


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
def test_every_byte_value_widens_exactly(oracle, dtype):
    """Row r of one operand holds the byte r first and zeros after it, the other operand a one in one position: the
    products are the decoded values themselves, for all 256 bytes, with the bytes on the A side and on the B side."""
    depth = 32  # dimensions
    stored = depth // support.DIMENSIONS_PER_VALUE.get(dtype, 1)
    every = np.zeros((256, stored), np.uint8)
    every[:, 0] = np.arange(256)
    one = {"e2m3": 0x08, "e3m2": 0x0C, "i4": 0x01, "u4": 0x01, "u1": 0x01}[dtype]
    units = np.zeros((2, stored), np.uint8)
    units[0, 0] = one                                      # picks dimension 0
    units[1, 0] = {"i4": 0x10, "u4": 0x10, "u1": 0x02}.get(dtype, 0)  # picks dimension 1 (the high nibble, the second bit)
    decoded = oracle.decode(dtype, every)
    expected = decoded[:, :2] if dtype in NARROW_INT_DTYPES else np.stack([decoded[:, 0], np.zeros(256, np.float32)], axis=1)
    as_a = gpu_dots(dtype, every, units)
    as_b = gpu_dots(dtype, units, every)
    assert np.array_equal(as_a.astype(np.float64), expected.astype(np.float64))
    assert np.array_equal(as_b.astype(np.float64).T, expected.astype(np.float64))


@pytest.mark.parametrize("dtype", NARROW_FLOAT_DTYPES)
def test_short_dots_are_exact(oracle, dtype):
    """Depth 64: every product is a multiple of 2^-8 below 2^10 and every partial sum stays far below 2^24 of them, so
    whatever the order, f32 accumulation is exact: the GPU, the serial kernel and the f64 truth agree bit for bit."""
    rng = np.random.default_rng(81)
    a, b = support.random_matrix(oracle, dtype, 200, 64, rng), support.random_matrix(oracle, dtype, 300, 64, rng)
    got = gpu_dots(dtype, a, b)
    truth, _ = oracle.truth(dtype, a, b)
    assert np.array_equal(got.astype(np.float64), truth)
    assert np.array_equal(got.view(np.uint32), oracle.dots_packed(dtype, a, b).view(np.uint32))


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
def test_deep_and_strided(oracle, dtype):
    """Depth 8192 (64 to 128 pipeline stages), then rows with padding between them on both sides and a C with a
    padded stride through the plain C entry points with host pointers."""
    rng = np.random.default_rng(83)
    a, b = support.random_matrix(oracle, dtype, 48, 8192, rng), support.random_matrix(oracle, dtype, 80, 8192, rng)
    check(oracle, dtype, a, b, 0, f"{dtype} deep")
    lib = nk.library()
    m, n, k, pad = 37, 61, 514, 3
    a_full, b_full = support.random_matrix(oracle, dtype, m, k, rng, pad=pad), support.random_matrix(oracle, dtype, n, k, rng, pad=pad)
    a_full, b_full = np.ascontiguousarray(a_full), np.ascontiguousarray(b_full)  # (views of the padded arrays above)
    a_wide = np.full((m, a_full.shape[1] + pad), 0xEE, np.uint8)
    b_wide = np.full((n, b_full.shape[1] + pad), 0xEE, np.uint8)
    a_wide[:, : a_full.shape[1]], b_wide[:, : b_full.shape[1]] = a_full, b_full
    packed = np.zeros(getattr(lib, f"nk_dots_packed_size_{dtype}")(n, k), np.uint8)
    getattr(lib, f"nk_dots_pack_{dtype}")(b_wide.ctypes.data, n, k, b_wide.strides[0], packed.ctypes.data)
    c = np.full((m, n + 2), 0x5A5A5A5A, np.uint32)
    getattr(lib, f"nk_dots_packed_{dtype}")(a_wide.ctypes.data, packed.ctypes.data, c.ctypes.data, m, n, k, a_wide.strides[0],
                                            c.strides[0])
    assert not lib.nk_amd_last_error()
    assert (c[:, n:] == 0x5A5A5A5A).all()
    serial = oracle.dots_packed(dtype, a_full, b_full)
    got = np.ascontiguousarray(c[:, :n])
    if dtype in NARROW_INT_DTYPES:
        assert np.array_equal(got, serial.view(np.uint32))
    else:
        truth, magnitude = oracle.truth(dtype, a_full, b_full)
        assert_float_gate(dtype, got.view(np.float32), serial, truth, magnitude, f"{dtype} strided", best_dispatch(dtype, a_full, b_full))


def test_e2m3_rows_too_deep_for_integer_sums(oracle):
    """e2m3 runs as integers eight times as large on the i8 MFMA while 60 * 60 * depth stays below 2^31 (depth <=
    596,523); deeper rows, which the reference takes like any others (dots/serial.h:2601-2678), run widened to f16.
    Both sides of the switch, products and distances, against the serial restatement, the f64 truth and the kernel the
    reference dispatches to; with all values at the format's largest magnitude the integer route's sums are the
    largest they can be, and must still be exact."""
    rng = np.random.default_rng(91)
    for depth in (596_523, 596_524, 700_001):
        a, b = support.random_matrix(oracle, "e2m3", 5, depth, rng), support.random_matrix(oracle, "e2m3", 37, depth, rng)
        assert nk.dots_packed_size("e2m3", 37, depth) > 0
        check(oracle, "e2m3", a, b, 0, f"e2m3 depth {depth}")
        for metric in ("angular", "euclidean"):
            assert_distance_gate(oracle, metric, "e2m3", a, b, gpu_distances(metric, "e2m3", a, b), f"e2m3 {metric} depth {depth}")
    extreme = np.full((3, 596_523), 0x1F, np.uint8)  # +7.5 everywhere: 64 x the dot product is 3600 x depth, just below 2^31
    extreme[1] = 0x3F                                # -7.5
    got = gpu_dots("e2m3", extreme, extreme)
    exact = np.float32(56.25 * 596_523) * np.array([[1, -1, 1], [-1, 1, -1], [1, -1, 1]], np.float32)
    assert np.array_equal(got, exact)


def test_u1_image_keeps_bits(oracle):
    """The image of the 1-bit type holds the bits themselves, sixteen to a chunk (dots/serial.h:2680-2689 packs bytes
    of bits as well): header + n / 8 * depth bytes rounded up to whole tiles and stages + the (unused) column terms;
    chunk c of row r of tile t at ((t * chunks + c) * 32 + r) * 2."""
    rng = np.random.default_rng(92)
    for n, depth in [(70, 1000), (33, 4099), (1, 1)]:
        b = support.random_matrix(oracle, "u1", n, depth, rng)
        tiles, chunks = -(-n // 32), -(-(-(-depth // 16)) // 16) * 16
        size = nk.dots_packed_size("u1", n, depth)
        assert size == 64 + tiles * chunks * 64 + tiles * 256
        image = nk.dots_pack(to_gpu(b), "u1").buffer.cpu().numpy()
        assert image.size == size
        masked = b.copy()  # (bits past the depth in the last byte are the caller's: whole bytes are taken, as the reference does)
        padded = np.zeros((tiles * 32, chunks * 2), np.uint8)
        padded[:n, : masked.shape[1]] = masked
        expected = padded.reshape(tiles, 32, chunks, 2).transpose(0, 2, 1, 3).reshape(-1)
        assert np.array_equal(image[64 : 64 + expected.size], expected)
        assert not image[64 + expected.size :].any()
    assert nk.dots_packed_size("u1", 8192, 8192) == 64 + 256 * 512 * 64 + 256 * 256  # 8 MiB of bits, not 64 MiB of bytes


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(support.GOLDEN_DIR) if f.startswith("narrow_")))
def test_golden_vectors(oracle, name):
    """Inputs and serial-kernel outputs recorded from the reference library."""
    data = np.load(os.path.join(support.GOLDEN_DIR, name))
    dtype, a, b, vectors = str(data["dtype"]), data["a"], data["b"], data["vectors"]
    row_start, row_count = int(data["row_start"]), int(data["row_count"])
    check(oracle, dtype, a, b, 0, name)
    got = gpu_dots(dtype, a, b)
    bits = gpu_symmetric("dots", dtype, vectors, row_start, row_count)
    own = owned(vectors.shape[0], row_start, row_count)
    assert (bits[~own] == POISON).all()
    if dtype in NARROW_INT_DTYPES:
        assert np.array_equal(got.view(np.uint32), data["c_serial"].view(np.uint32))
        assert np.array_equal(bits[own], data["symmetric_serial"].view(np.uint32)[own])
    else:
        assert np.abs(got - data["c_serial"]).max() <= 2.0 ** -20 * np.abs(data["c_serial"]).max()
        assert np.abs(bits.view(np.float32)[own] - data["symmetric_serial"][own]).max() <= 2.0 ** -20 * np.abs(data["symmetric_serial"]).max()


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
def test_symmetric_windows(oracle, dtype):
    """The symmetric kind over windows off the tile boundaries; owned elements only are written."""
    rng = np.random.default_rng(87)
    for count, depth, row_start, row_count in [(5, 8, 0, 5), (300, 64, 100, 77), (700, 130, 333, 1000), (1000, 514, 37, 411)]:
        vectors = support.random_matrix(oracle, dtype, count, depth, rng)
        own = owned(count, row_start, row_count)
        bits = gpu_symmetric("dots", dtype, vectors, row_start, row_count)
        assert (bits[~own] == POISON).all()
        serial = oracle.symmetric("dots", dtype, vectors, row_start, row_count)
        if dtype in NARROW_INT_DTYPES:
            assert np.array_equal(bits[own], serial.view(np.uint32)[own])
        else:
            truth, magnitude = oracle.truth(dtype, vectors, vectors)
            dispatched = None
            if reference_library() is not None:
                reference = reference_library()
                dispatched = reference.symmetric("dots", dtype, vectors, row_start, row_count, viable=reference.capabilities)[own]
            assert_float_gate(dtype, bits.view(np.float32)[own], serial[own], truth[own], magnitude[own], f"{dtype} {count}", dispatched)


@pytest.mark.parametrize("dtype", NARROW_DTYPES)
def test_full_size_properties(oracle, dtype):
    """4096 x 4096 x 4096: the symmetric kind equals the packed kind with both sides the same on the upper triangle, bit
    for bit; sampled rows agree with the oracle; the distance kinds equal their packed forms above the diagonal (u1: are
    refused)."""
    count, depth = 4096, 4096
    rng = np.random.default_rng(89)
    vectors = support.random_matrix(oracle, dtype, count, depth, rng)
    gv = to_gpu(vectors)
    packed = nk.dots_pack(gv, dtype)
    assert packed.depth == depth
    rectangle = nk.dots_packed(gv, packed)
    whole = nk.dots_symmetric(gv, dtype)
    upper = torch.triu(torch.ones((count, count), dtype=torch.bool, device=DEV))
    assert torch.equal(whole.view(torch.int32)[upper], rectangle.view(torch.int32)[upper])
    rows = np.array([0, 1001, 4095])
    sample = rectangle[torch.from_numpy(rows).to(DEV)].cpu().numpy()
    serial = oracle.dots_packed(dtype, vectors[rows], vectors)
    if dtype in NARROW_INT_DTYPES:
        assert np.array_equal(sample.view(np.uint32), serial.view(np.uint32))
    else:
        truth, magnitude = oracle.truth(dtype, vectors[rows], vectors)
        assert_float_gate(dtype, sample, serial, truth, magnitude, f"{dtype} full size")
    if dtype != "u1":
        for packed_kind, symmetric_kind in ((nk.angulars_packed, nk.angulars_symmetric), (nk.euclideans_packed, nk.euclideans_symmetric)):
            both = packed_kind(gv, packed)
            triangle = symmetric_kind(gv, dtype)
            strict = torch.triu(torch.ones((count, count), dtype=torch.bool, device=DEV), 1)
            assert torch.equal(triangle.view(torch.int32)[strict], both.view(torch.int32)[strict])
            assert not torch.diagonal(triangle).any()
        return
    with pytest.raises(TypeError):
        nk.angulars_packed(gv, packed)
    status = nk.library().nk_amd_spatials_packed_async(support.KIND_ANGULARS, support.CODES[dtype], gv.data_ptr(),
                                                       packed.buffer.data_ptr(), rectangle.data_ptr(), 8, 8, depth,
                                                       vectors.strides[0], count * 4, None)
    assert status != 0  # no distance kernels behind these types


DISTANCE_NARROW = ("e2m3", "e3m2", "i4", "u4")


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", DISTANCE_NARROW)
@pytest.mark.parametrize("config", [0, 2, 4])
def test_packed_distances(oracle, dtype, metric, config):
    """Storage columns x dimensions per value = depth: odd depths of the 4-bit types are the odd storage widths here."""
    rng = np.random.default_rng(500 + config)
    for m, n, k in [(1, 1, 1), (3, 5, 7), (33, 70, 200), (100, 37, 333), (257, 129, 1000), (40, 33, 4100)]:
        a, b = support.random_matrix(oracle, dtype, m, k, rng), support.random_matrix(oracle, dtype, n, k, rng)
        if m > 4 and n > 4:
            a[1] = 0         # zero row
            b[2] = a[3]      # identical rows: both distances cancel to ~0
            b[4] = 0
        got = gpu_distances(metric, dtype, a, b, config)
        assert_distance_gate(oracle, metric, dtype, a, b, got, f"{dtype} {metric} {m}x{n}x{k} config {config}")
        if m > 4 and n > 4:
            assert got[1, 4] == 0
            if metric == "angular":
                assert (got[1] == 0).all()


@pytest.mark.parametrize("metric", ["angular", "euclidean"])
@pytest.mark.parametrize("dtype", DISTANCE_NARROW)
def test_symmetric_distances(oracle, dtype, metric):
    rng = np.random.default_rng(510)
    for count, depth, row_start, row_count in [(5, 7, 0, 5), (300, 64, 100, 77), (700, 130, 333, 1000), (1000, 515, 37, 411)]:
        vectors = support.random_matrix(oracle, dtype, count, depth, rng)
        if count > 40:
            vectors[2] = 0
            vectors[9] = vectors[40]
        check_distances(oracle, metric, dtype, vectors, row_start, row_count, 0, f"{dtype} {metric} {count}x{depth} rows {row_start}+{row_count}")


def test_e2m3_wide_tile(oracle):
    """The 128 x 512 tile that large e2m3 products take (tile configuration 5): exact on shapes off its edges (every
    e2m3 sum below 2^24 / 64 is exact in f32) and equal to the default shape bit for bit."""
    rng = np.random.default_rng(520)
    for m, n, k in [(1, 1, 1), (130, 33, 200), (257, 1100, 515), (100, 513, 4100)]:
        a, b = support.random_matrix(oracle, "e2m3", m, k, rng), support.random_matrix(oracle, "e2m3", n, k, rng)
        got = gpu_dots("e2m3", a, b, config=5)
        exact = oracle.decode("e2m3", a).astype(np.float64) @ oracle.decode("e2m3", b).astype(np.float64).T
        assert np.array_equal(got.astype(np.float64), exact), (m, n, k)
        assert np.array_equal(got.view(np.uint32), gpu_dots("e2m3", a, b).view(np.uint32))
