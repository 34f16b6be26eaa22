"""The five BASELINE configurations at their full sizes, on a real MI355X, through the C ABI.

At these sizes the CPU oracle is only run on sampled rows; the whole result is covered by properties that
do not depend on size: exact integer products against an f64 GEMM of the same operands (integers below
2^53 are exact in f64, so this is a closed form, computed by an independent library routine), invariance
under the caller's 64-row tiling (python/matrix.c:473-482 splits A this way), and NaN/Inf masks predicted
from IEEE rules by the f64 GEMM.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

import numkong_amd as nk  # noqa: E402
from tests import support  # noqa: E402
from tests.test_dots_gpu import DEV, assert_float_gate, assert_relative_gate, best_dispatch, to_gpu  # noqa: E402

pytestmark = pytest.mark.gpu

TORCH_VIEW = {"bf16": torch.bfloat16, "f16": torch.float16, "e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}


def gpu_random(oracle, dtype, rows, cols, seed, kind="default"):
    """Same families as support.random_matrix, generated in row blocks to bound host memory."""
    rng = np.random.default_rng(seed)
    blocks = [to_gpu(support.random_matrix(oracle, dtype, min(4096, rows - r), cols, rng, kind)) for r in range(0, rows, 4096)]
    return torch.cat(blocks)


def as_f64(dtype, t):
    if dtype in ("i8", "u8"):
        return t.double()
    return t.view(TORCH_VIEW[dtype]).double()


def exact_rows(dtype, a, b, rows):
    """f64 GEMM of a few rows of A against all of B, in column blocks."""
    sub = as_f64(dtype, a[rows])
    return torch.cat([sub @ as_f64(dtype, b[j:j + 65536]).T for j in range(0, b.shape[0], 65536)], dim=1)


ULP_ROWS = []  # the reference-style accuracy table of this run, printed once at the end of the module


@pytest.fixture(scope="module", autouse=True)
def ulp_table(request):
    yield
    if ULP_ROWS:
        capture = request.config.pluginmanager.getplugin("capturemanager")
        with capture.global_and_fixture_disabled():
            print("\n" + support.ULP_TABLE_HEADER)
            print("\n".join(ULP_ROWS), flush=True)


def sampled_oracle_gate(oracle, dtype, a, b, c, rows, cols, label=None):
    """The float gate on a sample of rows and columns of the full result, next to both reference kernels, and the
    sample's rows of the reference-style accuracy table (test/test.hpp:491-514)."""
    a_host = a[rows].cpu().numpy()
    b_host = b[cols].cpu().numpy()
    if a_host.dtype == np.int16:
        a_host, b_host = a_host.view(np.uint16), b_host.view(np.uint16)
    got = c[rows][:, cols].cpu().numpy()
    truth, magnitude = oracle.truth(dtype, a_host, b_host)
    serial, dispatched = oracle.dots_packed(dtype, a_host, b_host), best_dispatch(dtype, a_host, b_host)
    shape = label or f"{a.shape[0]}x{b.shape[0]}x{a.shape[1]}"
    ULP_ROWS.append(support.ulp_table_row(f"dots_packed_{dtype}_gfx950 {shape}", got, truth))
    ULP_ROWS.append(support.ulp_table_row(f"dots_packed_{dtype}_serial {shape}", serial, truth))
    if dispatched is not None:
        ULP_ROWS.append(support.ulp_table_row(f"dots_packed_{dtype} (host dispatch) {shape}", dispatched, truth))
    assert_float_gate(dtype, got, serial, truth, magnitude, f"{dtype} sample", dispatched)
    assert_relative_gate(got, (("serial", serial), ("dispatched", dispatched)), truth, magnitude, f"{dtype} sample {shape}")


def tiling_invariance(dtype, a, packed, c):
    """Calling the kernel on 64-row tiles of A gives the same bits as one call."""
    for start in (0, 64 * 7, a.shape[0] - 64):
        tile = nk.dots_packed(a[start:start + 64], packed)
        assert torch.equal(tile.view(torch.int32), c[start:start + 64].view(torch.int32))  # bits, so NaN == NaN


def test_config1_i8_2048_cubed_bit_exact(oracle):
    a = gpu_random(oracle, "i8", 2048, 2048, 42)
    b = gpu_random(oracle, "i8", 2048, 2048, 43)
    packed = nk.dots_pack(b, "i8")
    c = nk.dots_packed(a, packed)
    assert torch.equal(c.double(), a.double() @ b.double().T)
    rows = np.arange(0, 2048, 97)
    assert np.array_equal(c[rows].cpu().numpy(), oracle.dots_packed("i8", a[rows].cpu().numpy(), b.cpu().numpy()))
    tiling_invariance("i8", a, packed, c)


def test_config2_bf16_4096_cubed(oracle):
    a = gpu_random(oracle, "bf16", 4096, 4096, 44)
    b = gpu_random(oracle, "bf16", 4096, 4096, 45)
    packed = nk.dots_pack(b, "bf16")
    c = nk.dots_packed(a, packed)
    rows, cols = np.arange(5, 4096, 173), np.arange(3, 4096, 29)
    sampled_oracle_gate(oracle, "bf16", a, b, c, rows, cols)
    truth = exact_rows("bf16", a, b, torch.arange(0, 4096, 64, device=DEV))
    scale = exact_rows("bf16", a.view(torch.bfloat16).abs().view(torch.int16), b.view(torch.bfloat16).abs().view(torch.int16),
                       torch.arange(0, 4096, 64, device=DEV))
    assert ((c[::64].double() - truth).abs() / scale).max().item() < 4096 / 8 * 2.0**-24
    tiling_invariance("bf16", a, packed, c)


@pytest.mark.parametrize("dtype", ["e4m3", "e5m2"])
def test_config3_fp8_8192_cubed(oracle, dtype):
    """N(0,1) scaled to half of the largest finite value, reference-rule cast, 1 % zeros. The e5m2 encoder
    overflows to Inf (cast/serial.h:1160-1163), so its literal inputs make almost every output NaN: masks are
    gated on them, accuracy on a second run whose inputs are clamped to the finite range before the cast."""
    a = gpu_random(oracle, dtype, 8192, 8192, 46, "fp8")
    b = gpu_random(oracle, dtype, 8192, 8192, 47, "fp8")
    packed = nk.dots_pack(b, dtype)
    c = nk.dots_packed(a, packed)
    probe = torch.arange(0, 8192, 128, device=DEV)
    truth = exact_rows(dtype, a, b, probe)
    got = c[probe]
    assert torch.equal(torch.isnan(got), torch.isnan(truth))
    assert torch.equal(torch.isposinf(got), torch.isposinf(truth)) and torch.equal(torch.isneginf(got), torch.isneginf(truth))
    rows, cols = np.arange(7, 8192, 521), np.arange(1, 8192, 37)
    sampled_oracle_gate(oracle, dtype, a, b, c, rows, cols)
    tiling_invariance(dtype, a, packed, c)
    if dtype == "e5m2":
        assert torch.isnan(got).float().mean().item() > 0.9  # the literal configuration is almost all NaN
        limit = 0x7B  # largest finite magnitude code
        clamp = lambda t: torch.where((t & 0x7F) > limit, (t & 0x80) | limit, t)
        a2, b2 = clamp(a), clamp(b)
        c2 = nk.dots_packed(a2, nk.dots_pack(b2, dtype))
        assert torch.isfinite(c2[probe]).all()
        sampled_oracle_gate(oracle, dtype, a2, b2, c2, rows, cols, "8192x8192x8192 clamped")


@pytest.mark.parametrize("dtype", ["i8", "u8"])
def test_config4_tall_skinny_retrieval(oracle, dtype):
    """1024 queries x 1,048,576 database vectors of dimension 768: C is 4 GiB, offsets need 64 bits."""
    m, n, k = 1024, 1 << 20, 768
    queries = gpu_random(oracle, dtype, m, k, 48)
    database = gpu_random(oracle, dtype, n, k, 49)
    packed = nk.dots_pack(database, dtype)
    c = nk.dots_packed(queries, packed)
    as_unsigned = (lambda t: t.double() + (t < 0).double() * 2.0**32) if dtype == "u8" else (lambda t: t.double())
    rows = torch.tensor([0, 1, 63, 64, 511, 777, 1022, 1023], device=DEV)
    assert torch.equal(as_unsigned(c[rows]), exact_rows(dtype, queries, database, rows))
    cols = torch.cat([torch.arange(0, 4096, device=DEV), torch.arange(n - 4096, n, device=DEV),
                      torch.arange(12345, n, 262139, device=DEV)])
    assert torch.equal(as_unsigned(c[:, cols]), queries.double() @ database[cols].double().T)
    sample = database[cols[:64]].cpu().numpy()
    assert np.array_equal(c[:8][:, cols[:64]].cpu().numpy().view(np.uint32),
                          oracle.dots_packed(dtype, queries[:8].cpu().numpy(), sample).view(np.uint32))
    del c
    torch.cuda.empty_cache()


def test_config5_f16_and_i8_8192_cubed_and_ragged(oracle):
    for m, n, k in [(8192, 8192, 8192), (8192, 8191, 1000)]:
        a = gpu_random(oracle, "i8", m, k, 50)
        b = gpu_random(oracle, "i8", n, k, 51)
        packed = nk.dots_pack(b, "i8")
        c = nk.dots_packed(a, packed)
        assert c.stride(0) * 4 == n * 4  # contiguous: rows of the ragged case are only 4-byte aligned
        for start in range(0, m, 2048):
            assert torch.equal(c[start:start + 2048].double(), a[start:start + 2048].double() @ b.double().T)
        tiling_invariance("i8", a, packed, c)
        del a, b, c, packed
        a = gpu_random(oracle, "f16", m, k, 52, "lognormal")
        b = gpu_random(oracle, "f16", n, k, 53, "lognormal")
        packed = nk.dots_pack(b, "f16")
        c = nk.dots_packed(a, packed)
        rows, cols = np.arange(11, m, 601), np.concatenate([np.arange(2, n, 41), [n - 1]])
        sampled_oracle_gate(oracle, "f16", a, b, c, rows, cols)
        tiling_invariance("f16", a, packed, c)
        del a, b, c, packed
        torch.cuda.empty_cache()
