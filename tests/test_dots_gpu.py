"""Parity of the gfx950 kernels with the reference semantics, through the C ABI, on a real MI355X.

Integers must be bit-exact (the reference's integer backends all equal the exact product mod 2^32).
Floats are compared with the f64 ground truth next to TWO reference CPU kernels on the same inputs: the serial
kernel as restated by the oracle (which tests/test_oracle.py pins bit-for-bit against the reference library),
and, when the reference build oracle/_ref is present, the kernel the reference dispatches to on this host
(16-lane AVX-512 on the GPU boxes). The gate is the tighter of the two:

  normwise error  e = |c - truth| / sum|a*b|   per element, over elements with a finite truth
  gate:  mean(e_gpu) <= 2 * mean(e_ref) + 2^-24 / sqrt(count)   (the slack only matters for a handful of outputs)
         max(e_gpu)  <= 2 * max(max(e_ref), floor)         floor = 2^-24 against the serial kernel (one f32 rounding unit
                                                            of the magnitude sum), 2.5 * 2^-24 against the dispatched one
         every element: |c_gpu - truth| <= 2 * max(|c_ref - truth|, 2.5 * 2^-24 * sum|a*b|)
         NaN, +Inf and -Inf masks identical to the serial kernel's (the reference's AVX-512 e5m2 kernels do
         not propagate Inf/NaN, so masks are not compared with them and their non-finite outputs are skipped).

The floor keeps the max statistic meaningful where all kernels sit at a few roundings of the result: on small
samples, and at shallow depths against the 16-lane AVX-512 kernels, whose lanes each add only depth / 16 products
and round to nearest where the MFMA's 16-product sums truncate. Measured over 490,000 outputs at depth 130, in
units of 2^-24 (mean, 99.99th percentile, max): bf16 GPU 0.095, 1.95, 3.71; serial 0.088, 1.49, 2.50; dispatched
0.080, 1.28, 1.98. The means agree; only the largest few outputs in a million differ. Measured on 192 x 256 outputs at depth 4096-8192 (GPU / serial, GPU / dispatched, mean
of the normwise error): bf16 0.52-0.56, 1.13; f16 0.27, 0.52; e4m3 0.96, 1.16; e5m2 0.99, 1.13.
"""
import ctypes
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from numkong_amd import api  # noqa: E402
from tests import support  # noqa: E402
from tests.support import ALL_DTYPES, FLOAT_DTYPES, OUTPUT  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
U = 2.0**-24


def to_gpu(array):
    a = np.ascontiguousarray(array)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def gpu_dots(dtype, a, b, config=0):
    nk.library().nk_hip_set_tile_config(config)
    try:
        packed = nk.dots_pack(to_gpu(b), dtype)
        c = nk.dots_packed(to_gpu(a), packed)
    finally:
        nk.library().nk_hip_set_tile_config(0)
    out = c.cpu().numpy()
    return out.view(np.uint32) if dtype == "u8" else out


_REFERENCE = []


def best_dispatch(dtype, a, b):
    """The same product by the kernel the reference library dispatches to on this host, or None without the build."""
    if not _REFERENCE:
        _REFERENCE.append(support.load_reference())
    reference = _REFERENCE[0]
    return None if reference is None else reference.dots_packed(dtype, a, b, viable=reference.capabilities)


PER_ELEMENT_FLOOR = 2.5  # `c` of the per-element bound below, in units of 2^-24 of sum|a*b|


def assert_float_gate(dtype, got, serial, truth, magnitude, where="", dispatched=None):
    assert np.array_equal(np.isnan(got), np.isnan(serial)), f"NaN mask differs {where}"
    assert np.array_equal(np.isposinf(got), np.isposinf(serial)), f"+Inf mask differs {where}"
    assert np.array_equal(np.isneginf(got), np.isneginf(serial)), f"-Inf mask differs {where}"
    for name, ref in (("serial", serial), ("dispatched", dispatched)):
        if ref is None:
            continue
        finite = np.isfinite(truth) & (magnitude > 0) & np.isfinite(ref)
        if not finite.any():
            continue
        e_gpu = np.abs(got[finite].astype(np.float64) - truth[finite]) / magnitude[finite]
        e_ref = np.abs(ref[finite].astype(np.float64) - truth[finite]) / magnitude[finite]
        slack = U / np.sqrt(e_gpu.size)  # the standard error of a mean of single-rounding errors: decides tiny samples only
        assert e_gpu.mean() <= 2 * e_ref.mean() + slack, f"mean error {e_gpu.mean():.3e} vs {name} {e_ref.mean():.3e} {where}"
        floor = U if name == "serial" else 2.5 * U
        assert e_gpu.max() <= 2 * max(e_ref.max(), floor), f"max error {e_gpu.max():.3e} vs {name} {e_ref.max():.3e} {where}"
        # Every element on its own: |c - truth| <= 2 * max(|c_ref - truth|, c * 2^-24 * sum|a*b|). The floor guards the
        # elements where the reference kernel happens to land on the truth; c = 2.5 is five roundings of f32 at the
        # magnitude of the whole sum, what a short chain of MFMA partial sums (each rounded once) can add up to.
        bound = 2 * np.maximum(e_ref, PER_ELEMENT_FLOOR * U)
        worst = int(np.argmax(e_gpu - bound))
        assert (e_gpu <= bound).all(), (f"{int((e_gpu > bound).sum())} of {e_gpu.size} elements past the per-element bound vs {name}; "
                                        f"worst {e_gpu[worst]:.3e} against its reference's {e_ref[worst]:.3e} {where}")


def assert_relative_gate(got, references, truth, magnitude, where=""):
    """The same comparison with each error taken relative to the result itself, e = |c - truth| / |truth|: the mean
    within twice the reference kernel's, and the maximum within twice the reference kernel's or, where that kernel
    happens to land on the truth, twice the per-element floor of assert_float_gate at the sample's worst-conditioned
    element. An element's relative error is its normwise error times kappa = sum|a*b| / |truth|, the same factor for
    every kernel, and kappa has a heavy tail (a sum of thousands of products that nearly cancels): both statistics are
    carried by the few outputs nearest to zero, so this gate is for samples of thousands of outputs and says little that
    the per-element bound has not said already."""
    for name, ref in references:
        if ref is None:
            continue
        use = np.isfinite(truth) & (truth != 0) & np.isfinite(ref) & np.isfinite(got)
        if not use.any():
            continue
        size = np.abs(truth[use])
        e_gpu = np.abs(got[use].astype(np.float64) - truth[use]) / size
        e_ref = np.abs(ref[use].astype(np.float64) - truth[use]) / size
        kappa = magnitude[use] / size
        floor = PER_ELEMENT_FLOOR * U * kappa.max()
        assert e_gpu.mean() <= 2 * e_ref.mean() + U * kappa.mean() / np.sqrt(e_gpu.size), (
            f"mean relative error {e_gpu.mean():.3e} vs {name} {e_ref.mean():.3e} {where}")
        assert e_gpu.max() <= 2 * max(e_ref.max(), floor), f"max relative error {e_gpu.max():.3e} vs {name} {e_ref.max():.3e} {where}"


def check(oracle, dtype, a, b, config=0, where=""):
    got = gpu_dots(dtype, a, b, config)
    if dtype in ("i8", "u8"):
        exact = (a.astype(np.int64) @ b.astype(np.int64).T) & 0xFFFFFFFF
        assert np.array_equal(got.astype(np.int64) & 0xFFFFFFFF, exact), where
        assert np.array_equal(got.view(np.uint32), oracle.dots_packed(dtype, a, b).view(np.uint32)), where
    else:
        truth, magnitude = oracle.truth(dtype, a, b)
        assert_float_gate(dtype, got, oracle.dots_packed(dtype, a, b), truth, magnitude, where, best_dispatch(dtype, a, b))


SHAPES = [(1, 1, 1), (3, 5, 7), (33, 70, 200), (64, 64, 64), (100, 37, 333), (257, 129, 1000), (31, 300, 129), (130, 33, 4100)]


@pytest.mark.parametrize("dtype", ALL_DTYPES)
@pytest.mark.parametrize("config", [0, 1, 2, 3, 4])
def test_small_shapes_every_tile_config(oracle, dtype, config):
    rng = np.random.default_rng(100 + config)
    for m, n, k in SHAPES:
        a = support.random_matrix(oracle, dtype, m, k, rng)
        b = support.random_matrix(oracle, dtype, n, k, rng)
        check(oracle, dtype, a, b, config, f"{dtype} {m}x{n}x{k} config {config}")


@pytest.mark.parametrize("dtype", ["i8", "u8", "bf16", "e4m3"])
@pytest.mark.parametrize("store", [1, 2])
def test_both_kinds_of_store(oracle, dtype, store):
    """Outputs stored past the caches (what rows of C on 128-byte lines get) and through them (what other rows get),
    each forced (bits 28..29 of the test hook) over whole tiles and edge tiles of aligned and unaligned rows."""
    rng = np.random.default_rng(300 + store)
    for config, (m, n, k) in ((4, (200, 300, 260)), (4, (192, 256, 128)), (3, (260, 257, 130)), (2, (300, 544, 200)), (0, (130, 96, 70))):
        if config == 1 and dtype not in ("i8", "u8"):
            continue
        a = support.random_matrix(oracle, dtype, m, k, rng)
        b = support.random_matrix(oracle, dtype, n, k, rng)
        check(oracle, dtype, a, b, config | (store << 28), f"{dtype} {m}x{n}x{k} config {config} store {store}")


def test_staging_straight_into_lds():
    """i8 at the 256 x 256 tile (bf16 and f16 at 128 x 256) takes A from memory straight into LDS (a ring of four stages, four stages a trip of the
    loop) when the depth is a whole number of trips; bit 30 of the test hook keeps the staging through registers. Both
    must equal the exact product: tiles off the edges of A and B, a padded A, one tile and several tiles per workgroup
    (the pipeline runs on across them), and depths of two to sixteen trips."""
    rng = np.random.default_rng(77)
    for m, n, k, pad in ((300, 515, 1024, 0), (257, 1000, 1536, 16), (1024, 256, 4096, 0), (2100, 33000, 2048, 0), (70000, 300, 1024, 32)):
        a_wide = rng.integers(-128, 128, (m, k + pad), dtype=np.int8)
        b = rng.integers(-128, 128, (n, k), dtype=np.int8)
        ga, packed = to_gpu(a_wide)[:, :k], nk.dots_pack(to_gpu(b), "i8")
        results = []
        for hook in (1, 1 | (1 << 30)):
            nk.library().nk_hip_set_tile_config(hook)
            try:
                results.append(nk.dots_packed(ga, packed))
            finally:
                nk.library().nk_hip_set_tile_config(0)
        assert torch.equal(results[0], results[1]), f"{m}x{n}x{k}"
        rows = torch.from_numpy(rng.choice(m, min(m, 300), replace=False)).to(DEV)
        exact = ga[rows].double() @ to_gpu(b).double().T
        assert torch.equal(results[0][rows].double(), exact), f"{m}x{n}x{k}"
    # bf16 and f16 at their largest tile (128 x 256) do the same when their folds fall between trips: same bits either way
    oracle = support.load_oracle()
    for dtype, (m, n, k) in (("bf16", (300, 515, 2048)), ("f16", (1100, 9000, 4096)), ("bf16", (2100, 16500, 2048))):
        a, b = support.random_matrix(oracle, dtype, m, k, rng), support.random_matrix(oracle, dtype, n, k, rng)
        ga, packed = to_gpu(a), nk.dots_pack(to_gpu(b), dtype)
        results = []
        for hook in (2, 2 | (1 << 30)):
            nk.library().nk_hip_set_tile_config(hook)
            try:
                results.append(nk.dots_packed(ga, packed))
            finally:
                nk.library().nk_hip_set_tile_config(0)
        assert torch.equal(results[0].view(torch.int32), results[1].view(torch.int32)), f"{dtype} {m}x{n}x{k}"
        sample = np.sort(rng.choice(m, 40, replace=False))
        truth, magnitude = oracle.truth(dtype, a[sample], b[:500])
        assert_float_gate(dtype, results[0][torch.from_numpy(sample).to(DEV)][:, :500].cpu().numpy(), oracle.dots_packed(dtype, a[sample], b[:500]),
                          truth, magnitude, f"{dtype} {m}x{n}x{k} straight into LDS")


@pytest.mark.parametrize("dtype", FLOAT_DTYPES)
def test_float_input_families(oracle, dtype):
    rng = np.random.default_rng(5)
    kinds = ["lognormal"] + (["fp8"] if dtype[0] == "e" else [])
    for kind in kinds:
        for m, n, k in [(48, 80, 1536), (64, 96, 8192)]:
            a = support.random_matrix(oracle, dtype, m, k, rng, kind)
            b = support.random_matrix(oracle, dtype, n, k, rng, kind)
            check(oracle, dtype, a, b, 0, f"{dtype} {kind} {m}x{n}x{k}")


@pytest.mark.parametrize("name", sorted(f for f in os.listdir(support.GOLDEN_DIR) if f.startswith("dots_")))
def test_golden_vectors(oracle, name):
    """Inputs and serial-kernel outputs recorded from the reference library, special values included."""
    data = np.load(os.path.join(support.GOLDEN_DIR, name))
    dtype, a, b, c_serial = str(data["dtype"]), data["a"], data["b"], data["c_serial"]
    got = gpu_dots(dtype, a, b)
    if dtype in ("i8", "u8"):
        assert np.array_equal(got.view(np.uint32), c_serial.view(np.uint32))
    else:
        truth, magnitude = oracle.truth(dtype, a, b)
        assert_float_gate(dtype, got, c_serial, truth, magnitude, name, best_dispatch(dtype, a, b))


@pytest.mark.parametrize("dtype", ["e4m3", "e5m2"])
def test_every_fp8_code_decodes_exactly(oracle, dtype):
    """code * 1.0 through both operand paths (A is widened on its way into LDS, B when it is packed)."""
    codes = np.arange(256, dtype=np.uint8)
    expected = oracle.decode(dtype, codes)
    one = oracle.encode(dtype, np.array([1.0], np.float32))[0]
    for k in (1, 16, 100):
        a = np.zeros((256, k), np.uint8)
        a[:, k - 1] = codes
        b = np.zeros((3, k), np.uint8)
        b[:, k - 1] = one
        for got in (gpu_dots(dtype, a, b)[:, 1], gpu_dots(dtype, b, a)[1, :]):
            nan = np.isnan(expected)
            assert np.array_equal(np.isnan(got), nan) and np.array_equal(got[~nan], expected[~nan])


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_subnormals_are_not_flushed(oracle, dtype):
    tiny = np.array([[1, 2, 3, 0x8001]], np.uint16)  # smallest subnormals
    big = oracle.encode(dtype, np.array([[1.0, 1.0, 1.0, 2.0]], np.float32))
    expected = oracle.dots_packed(dtype, tiny, big)
    assert expected[0, 0] != 0
    assert np.array_equal(gpu_dots(dtype, tiny, big), expected)
    assert np.array_equal(gpu_dots(dtype, big, tiny), expected)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_strides_alignment_and_untouched_padding(oracle, dtype):
    """Row strides larger than the row, A not 16-byte aligned, C rows wider than n: only m x n is written."""
    rng = np.random.default_rng(9)
    lib = nk.library()
    cases = [(37, 29, 1000, 13, 7, 3, 1), (64, 130, 63, 3, 0, 5, 0), (5, 130, 2049, 1, 1, 0, 3),
             # dword-aligned rows whose depth ends inside a dword: the pipelined loop masks what it reads past a row
             (37, 29, 1001, 3, 0, 1, 0), (130, 70, 1003, 1, 2, 0, 4), (300, 33, 77, 3, 0, 0, 0)]
    for m, n, k, pad_a, pad_b, pad_c, skew in cases:
        a_full = support.random_matrix(oracle, dtype, m, k + pad_a + skew, rng)
        b_full = support.random_matrix(oracle, dtype, n, k + pad_b, rng)
        a, b = a_full[:, skew:skew + k].copy(), b_full[:, :k]
        poison = 0x7FFF if a_full.itemsize == 2 else 0x7F  # NaN in every float type here: padding must never reach a product
        a_full[:, :skew] = poison
        a_full[:, skew + k:] = poison
        ga, gb = to_gpu(a_full), to_gpu(b_full)
        packed = torch.empty(nk.dots_packed_size(dtype, n, k), dtype=torch.uint8, device=DEV)
        c = torch.full((m, n + pad_c), 0x5A5A5A5A, dtype=torch.int32, device=DEV)
        width = a_full.itemsize
        getattr(lib, f"nk_dots_pack_{dtype}")(gb.data_ptr(), n, k, b_full.shape[1] * width, packed.data_ptr())
        assert not lib.nk_amd_last_error()
        getattr(lib, f"nk_dots_packed_{dtype}")(ga.data_ptr() + skew * width, packed.data_ptr(), c.data_ptr(), m, n, k,
                                               a_full.shape[1] * width, (n + pad_c) * 4)
        assert not lib.nk_amd_last_error()
        out = c.cpu().numpy()
        assert (out[:, n:] == 0x5A5A5A5A).all()
        got = np.ascontiguousarray(out[:, :n]).view(OUTPUT[dtype])
        if dtype in ("i8", "u8"):
            assert np.array_equal(got.view(np.uint32), oracle.dots_packed(dtype, a, b).view(np.uint32))
        else:
            truth, magnitude = oracle.truth(dtype, a, b)
            assert_float_gate(dtype, got, oracle.dots_packed(dtype, a, b), truth, magnitude)


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_host_pointers_are_staged(oracle, dtype):
    """The reference API takes plain host pointers; so does this one (staged through device buffers)."""
    rng = np.random.default_rng(21)
    lib = nk.library()
    m, n, k = 19, 45, 300
    a = support.random_matrix(oracle, dtype, m, k, rng, pad=2)
    b = support.random_matrix(oracle, dtype, n, k, rng, pad=4)
    packed = np.zeros(nk.dots_packed_size(dtype, n, k), np.uint8)
    c = np.full((m, n + 2), 7, OUTPUT[dtype])
    getattr(lib, f"nk_dots_pack_{dtype}")(a.ctypes.data * 0 + b.ctypes.data, n, k, b.strides[0], packed.ctypes.data)
    assert not lib.nk_amd_last_error()
    getattr(lib, f"nk_dots_packed_{dtype}")(a.ctypes.data, packed.ctypes.data, c.ctypes.data, m, n, k, a.strides[0], c.strides[0])
    assert not lib.nk_amd_last_error()
    assert (c[:, n:] == 7).all()
    device = gpu_dots(dtype, a, b)
    assert np.array_equal(np.ascontiguousarray(c[:, :n]).view(np.uint32), device.view(np.uint32))  # same kernel, same bits
    # a packed image is relocatable bytes: device image == host image, but for the number that tells pack calls apart
    # (header bytes 32..39), by which the library finds the device copy of a host image again
    image = nk.dots_pack(to_gpu(b), dtype).buffer.cpu().numpy()
    nonce, other = packed[32:40].copy().view(np.uint64)[0], image[32:40].copy().view(np.uint64)[0]
    assert nonce != 0 and other != 0 and nonce != other
    image[32:40] = packed[32:40]
    assert np.array_equal(image, packed)
    # the bytes stay valid wherever they are copied: a copy of the host image, and the device image brought to the host
    for relocated in (packed.copy(), nk.dots_pack(to_gpu(b), dtype).buffer.cpu().numpy()):
        again = np.full((m, n + 2), 7, OUTPUT[dtype])
        getattr(lib, f"nk_dots_packed_{dtype}")(a.ctypes.data, relocated.ctypes.data, again.ctypes.data, m, n, k, a.strides[0], again.strides[0])
        assert not lib.nk_amd_last_error()
        assert np.array_equal(again.view(np.uint32), c.view(np.uint32))
    # packing other rows into the same host buffer gives a new image, not the cached one's results
    shuffled = np.ascontiguousarray(b[::-1])
    getattr(lib, f"nk_dots_pack_{dtype}")(shuffled.ctypes.data, n, k, shuffled.strides[0], packed.ctypes.data)
    again = np.full((m, n + 2), 7, OUTPUT[dtype])
    getattr(lib, f"nk_dots_packed_{dtype}")(a.ctypes.data, packed.ctypes.data, again.ctypes.data, m, n, k, a.strides[0], again.strides[0])
    assert np.array_equal(again[:, :n].view(np.uint32), c[:, :n][:, ::-1].view(np.uint32))


@pytest.mark.parametrize("dtype", ALL_DTYPES)
def test_packed_image_layout(oracle, dtype):
    """header | tiles[(t * k_chunks + c) * 32 + r] of 16 bytes | 128 * sum(b ^ 0x80 as i8) per column (u8) | sum(b^2)
    per column."""
    rng = np.random.default_rng(33)
    n, k = 70, 203
    b = support.random_matrix(oracle, dtype, n, k, rng)
    image = nk.dots_pack(to_gpu(b), dtype).buffer.cpu().numpy()
    header = image[:64].view(np.uint32)
    if dtype in ("e4m3", "e5m2"):  # stored widened to f16, exactly
        rows = oracle.encode("f16", oracle.decode(dtype, b)).view(np.uint8).reshape(n, -1)
    elif dtype == "u8":
        rows = b ^ 0x80
    else:
        rows = np.ascontiguousarray(b).view(np.uint8).reshape(n, -1)
    row_bytes = rows.shape[1]
    chunks = -(-(-(-row_bytes // 16)) // 16) * 16  # an even number of 8-chunk stages
    tiles = -(-n // 32)
    assert header[0] == 0x35394B4E and header[2] == api.DTYPES[dtype][0] and header[3] == row_bytes // k
    assert (header[4], header[5], header[6], header[7]) == (n, k, tiles, chunks)
    padded = np.zeros((tiles * 32, chunks * 16), np.uint8)
    padded[:n, :row_bytes] = rows
    expected = padded.reshape(tiles, 32, chunks, 16).transpose(0, 2, 1, 3).reshape(-1)
    data = image[64:64 + expected.size]
    assert np.array_equal(data, expected)
    tail = image[64 + expected.size:].view(np.uint32)
    assert tail.size == 2 * tiles * 32
    terms, norms = tail[:tiles * 32], tail[tiles * 32:]
    if dtype == "u8":
        sums = (b.astype(np.int64) - 128).sum(axis=1) * 128
        assert np.array_equal(terms[:n].astype(np.int64), sums & 0xFFFFFFFF) and (terms[n:] == 0).all()
    else:
        assert (terms == 0).all()
    # per-column sums of squares: exact (mod 2^32) for the integer types, f64-accumulated and rounded once otherwise
    if dtype in ("i8", "u8"):
        assert np.array_equal(norms[:n].astype(np.int64), (b.astype(np.int64) ** 2).sum(axis=1) & 0xFFFFFFFF)
    else:
        exact = (oracle.decode(dtype, b).astype(np.float64) ** 2).sum(axis=1)
        assert np.array_equal(norms[:n].view(np.float32), exact.astype(np.float32))


def test_mismatched_image_poisons_output_and_zero_sizes(oracle):
    lib = nk.library()
    b = to_gpu(np.ones((40, 64), np.int8))
    packed = nk.dots_pack(b, "i8")
    a = to_gpu(np.ones((8, 64), np.int8))
    c = torch.zeros((8, 40), dtype=torch.int32, device=DEV)
    # wrong dtype for this image, and wrong depth: every output becomes 0xFFFFFFFF, nothing else is touched
    lib.nk_dots_packed_u8(a.data_ptr(), packed.buffer.data_ptr(), c.data_ptr(), 8, 40, 64, 64, 160)
    assert (c.cpu().numpy() == -1).all()
    c.zero_()
    lib.nk_dots_packed_i8(a.data_ptr(), packed.buffer.data_ptr(), c.data_ptr(), 8, 40, 48, 64, 160)
    assert (c.cpu().numpy() == -1).all()
    # m = 0 or n = 0: nothing happens; k = 0: C is zeroed (the reference zeroes C and adds nothing)
    c.fill_(5)
    lib.nk_dots_packed_i8(a.data_ptr(), packed.buffer.data_ptr(), c.data_ptr(), 0, 40, 64, 64, 160)
    assert (c.cpu().numpy() == 5).all()
    empty = torch.zeros(nk.dots_packed_size("i8", 40, 0), dtype=torch.uint8, device=DEV)
    lib.nk_dots_pack_i8(b.data_ptr(), 40, 0, 64, empty.data_ptr())
    lib.nk_dots_packed_i8(a.data_ptr(), empty.data_ptr(), c.data_ptr(), 8, 40, 0, 64, 160)
    assert not lib.nk_amd_last_error() and (c.cpu().numpy() == 0).all()


def test_python_mirror_out_argument(oracle):
    rng = np.random.default_rng(2)
    a = to_gpu(support.random_matrix(oracle, "bf16", 70, 128, rng))
    packed = nk.dots_pack(to_gpu(support.random_matrix(oracle, "bf16", 50, 128, rng)), "bf16")
    fresh = nk.dots_packed(a, packed)
    out = torch.zeros_like(fresh)
    assert nk.dots_packed(a, packed, out=out) is out and torch.equal(out, fresh)
    with pytest.raises(ValueError):
        nk.dots_packed(a[:, :64], packed)
    with pytest.raises(ValueError):
        nk.dots_packed(a, packed, out=torch.zeros(70, 51, device=DEV))
    with pytest.raises(TypeError):
        nk.dots_packed(a, packed, out=torch.zeros(70, 50, dtype=torch.int32, device=DEV))
