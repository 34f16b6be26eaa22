"""The C-ABI boundary without a GPU: the library loads, exports what include/*.h declares, and its host
logic (sizes, dispatch, lookup, the error convention) behaves like the reference's c/numkong.c."""
import ctypes
import os
import re

import numpy as np
import pytest

import numkong_amd as nk
from numkong_amd import api
from tests import support

INCLUDE = os.path.join(support.ROOT, "include", "numkong_amd")
CAP_GFX950 = 1 << 62
TYPES = ("i8", "u8", "bf16", "f16", "e4m3", "e5m2")


def declared_symbols():
    names = set()
    for header in os.listdir(INCLUDE):
        text = open(os.path.join(INCLUDE, header)).read()
        names |= set(re.findall(r"\b(nk_(?:hip|amd)_[a-z0-9_]+)\s*\(", text))
        names |= set(re.findall(r"NK_DYNAMIC[^;(]*?\b(nk_[a-z0-9_]+)\s*\(", text))
        for t in TYPES:  # the backend-suffixed kernels come from a macro
            names |= {f"nk_dots_packed_size_{t}_gfx950", f"nk_dots_pack_{t}_gfx950", f"nk_dots_packed_{t}_gfx950"}
            names |= {f"nk_angulars_packed_{t}_gfx950", f"nk_euclideans_packed_{t}_gfx950"}
            names |= {f"nk_angulars_packed_{t}", f"nk_euclideans_packed_{t}"}  # also declared through a macro
            for family in ("dots", "angulars", "euclideans"):
                names |= {f"nk_{family}_symmetric_{t}", f"nk_{family}_symmetric_{t}_gfx950"}
    return {n for n in names if "##" not in n}


def test_library_exports_every_declared_symbol():
    lib = nk.library()
    names = declared_symbols()
    assert len(names) >= 30 * 2 + 36 + 8 + 19
    missing = [n for n in sorted(names) if not hasattr(lib, n)]
    assert not missing, missing
    for t in TYPES:
        for stem in ("nk_dots_packed_size_", "nk_dots_pack_", "nk_dots_packed_", "nk_angulars_packed_", "nk_euclideans_packed_",
                     "nk_dots_symmetric_", "nk_angulars_symmetric_", "nk_euclideans_symmetric_"):
            assert hasattr(lib, stem + t)


def test_packed_size_formula():
    """header + ceil(n/32) tiles * chunks (padded to an even number of 8-chunk stages) * 512 B + 128 B of column
    terms and 128 B of column sums of squares per tile; fp8 stored as f16."""
    for t, width in (("i8", 1), ("u8", 1), ("bf16", 2), ("f16", 2), ("e4m3", 2), ("e5m2", 2)):
        for n, k in [(1, 1), (32, 128), (33, 129), (2048, 2048), (8191, 1000), (1048576, 768)]:
            tiles = -(-n // 32)
            chunks = -(-(-(-k * width // 16)) // 16) * 16
            assert nk.dots_packed_size(t, n, k) == 64 + tiles * chunks * 512 + tiles * 256, (t, n, k)
        assert nk.dots_packed_size(t, 0, 0) == 64
        assert nk.dots_packed_size(t, 1 << 40, 8) == 0  # dimensions beyond 32 bits are refused, as the error stub does
    # e2m3 is stored as i8 values (eight times as large) while the i32 sums of 64 x its products cannot overflow,
    # 60 * 60 * k < 2^31, and widened to f16 like e3m2 beyond that depth: twice the bytes per element
    assert nk.dots_packed_size("e2m3", 8, 596523) == 64 + -(-596523 // 256) * 16 * 512 + 256
    assert nk.dots_packed_size("e2m3", 8, 596524) == 64 + -(-596524 // 128) * 16 * 512 + 256
    # single bits stay bits: sixteen to a 2-byte chunk, 32 rows and 16 chunks to a unit
    assert nk.dots_packed_size("u1", 100, 1000) == 64 + 4 * 64 * 64 + 4 * 256
    # the two wide types keep f64 values k-major: header + 8 bytes x (n padded to 64) x (k padded to 32), and a sum of
    # squares per padded column behind them
    assert nk.dots_packed_size("f32", 100, 70) == nk.dots_packed_size("f64", 100, 70) == 64 + 8 * 128 * 96 + 8 * 128
    with pytest.raises(TypeError):
        nk.dots_packed_size("f16c", 4, 4)


def find(lib, kind, dtype_code, viable):
    fn, cap = ctypes.c_void_p(), ctypes.c_uint64(123)
    lib.nk_find_kernel_punned(kind, dtype_code, viable, ctypes.byref(fn), ctypes.byref(cap))
    return fn.value, cap.value


def test_lookup_and_capabilities():
    lib = nk.library()
    assert lib.nk_uses_dynamic_dispatch() == 1
    assert lib.nk_configure_thread(ctypes.c_uint64(lib.nk_capabilities())) == 1
    assert lib.nk_capabilities_compiled() == (1 | CAP_GFX950)
    assert lib.nk_capabilities() & 1
    assert lib.nk_capabilities_available() == lib.nk_capabilities() & lib.nk_capabilities_compiled()
    for t in TYPES:
        code = api.DTYPES[t][0]
        for kind, stem in ((ord("P"), "nk_dots_packed_size_"), (ord("Q"), "nk_dots_pack_"), (ord("G"), "nk_dots_packed_")):
            fn, cap = find(lib, kind, code, CAP_GFX950 | 1)
            backend = ctypes.cast(getattr(lib, f"{stem}{t}_gfx950"), ctypes.c_void_p).value
            assert fn == backend and cap == CAP_GFX950
            fn, cap = find(lib, kind, code, 1)  # serial only: no kernel behind it here -> error stub, capability 0
            assert fn and fn != backend and cap == 0
        for kind, stem in ((ord("y"), "nk_dots_symmetric_"), (ord("n"), "nk_angulars_symmetric_"),
                           (ord("D"), "nk_euclideans_symmetric_")):
            fn, cap = find(lib, kind, code, CAP_GFX950)
            assert fn == ctypes.cast(getattr(lib, f"{stem}{t}_gfx950"), ctypes.c_void_p).value and cap == CAP_GFX950
            fn, cap = find(lib, kind, code, 1)
            assert fn and cap == 0
        fn, cap = find(lib, ord("Y"), code, CAP_GFX950)  # symmetric hamming distances: not on this path
        assert fn and cap == 0
    assert find(lib, ord("G"), 1 << 20, CAP_GFX950) == (None, 0)  # f64c: unknown dtype -> null kernel
    for name in ("e2m3", "e3m2", "i4", "u4", "f32", "f64"):  # every kind as well; dot products in their own widened types
        code = api.DTYPES[name][0]
        for kind, stem in ((ord("P"), "nk_dots_packed_size_"), (ord("Q"), "nk_dots_pack_"), (ord("G"), "nk_dots_packed_"),
                           (ord("y"), "nk_dots_symmetric_"), (ord("N"), "nk_angulars_packed_"), (ord("E"), "nk_euclideans_packed_"),
                           (ord("n"), "nk_angulars_symmetric_"), (ord("D"), "nk_euclideans_symmetric_")):
            fn, cap = find(lib, kind, code, CAP_GFX950 | 1)
            assert fn == ctypes.cast(getattr(lib, f"{stem}{name}_gfx950"), ctypes.c_void_p).value and cap == CAP_GFX950
            assert ctypes.cast(getattr(lib, f"{stem}{name}"), ctypes.c_void_p).value  # the dispatched entry point
        expected = {"i4": 1 << 4, "u4": 1 << 8, "f32": 1 << 10, "f64": 1 << 10}.get(name, 1 << 11)
        assert lib.nk_kernel_output_dtype(ord("G"), code) == lib.nk_kernel_output_dtype(ord("y"), code) == expected
        for kind in (ord("N"), ord("E"), ord("n"), ord("D")):  # f32 distances, f64 for the two wide types
            assert lib.nk_kernel_output_dtype(kind, code) == (1 << 10 if name in ("f32", "f64") else 1 << 11)
    for name in ("u1",):  # the dot-product kinds only
        code = api.DTYPES[name][0]
        for kind, stem in ((ord("P"), "nk_dots_packed_size_"), (ord("Q"), "nk_dots_pack_"), (ord("G"), "nk_dots_packed_"),
                           (ord("y"), "nk_dots_symmetric_")):
            fn, cap = find(lib, kind, code, CAP_GFX950 | 1)
            assert fn == ctypes.cast(getattr(lib, f"{stem}{name}_gfx950"), ctypes.c_void_p).value and cap == CAP_GFX950
        for kind in (ord("N"), ord("E"), ord("n"), ord("D")):
            fn, cap = find(lib, kind, code, CAP_GFX950)
            assert fn and cap == 0
        expected = {"u1": 1 << 8}[name]
        assert lib.nk_kernel_output_dtype(ord("G"), code) == lib.nk_kernel_output_dtype(ord("y"), code) == expected
        assert lib.nk_kernel_output_dtype(ord("N"), code) == 0
    out = {"i8": 1 << 4, "u8": 1 << 8, "bf16": 1 << 11, "f16": 1 << 11, "e4m3": 1 << 11, "e5m2": 1 << 11}
    for t, expected in out.items():
        assert lib.nk_kernel_output_dtype(ord("G"), api.DTYPES[t][0]) == expected
        assert lib.nk_kernel_output_dtype(ord("y"), api.DTYPES[t][0]) == expected
        assert lib.nk_kernel_output_dtype(ord("n"), api.DTYPES[t][0]) == 1 << 11
        assert lib.nk_kernel_output_dtype(ord("D"), api.DTYPES[t][0]) == 1 << 11
    assert lib.nk_kernel_output_dtype(ord("i"), api.DTYPES["i8"][0]) == 0


def test_error_convention_without_backend():
    """With the table re-targeted to no capability, the entry points are the reference's error stubs:
    size 0, pack leaves the buffer alone, the product fills exactly n*4 bytes of each C row with 0xFF."""
    lib = nk.library()
    try:
        lib.nk_dispatch_table_update(0)
        assert lib.nk_dots_packed_size_i8(5, 7) == 0
        packed = np.full(256, 0x5A, np.uint8)
        b = np.ones((5, 7), np.int8)
        lib.nk_dots_pack_i8(b.ctypes.data, 5, 7, 7, packed.ctypes.data)
        assert (packed == 0x5A).all()
        c = np.zeros((3, 8), np.int32)
        a = np.ones((3, 7), np.int8)
        lib.nk_dots_packed_i8(a.ctypes.data, packed.ctypes.data, c.ctypes.data, 3, 5, 7, 7, 32)
        assert (c[:, :5] == -1).all() and (c[:, 5:] == 0).all()
        f = np.zeros((2, 4), np.float32)
        lib.nk_dots_packed_bf16(a.ctypes.data, packed.ctypes.data, f.ctypes.data, 2, 3, 2, 4, 16)
        assert np.isnan(f[:, :3]).all() and (f[:, 3] == 0).all()
        # the symmetric stub poisons the whole count x count result, whatever the window (c/numkong.c:218-227)
        g = np.zeros((5, 6), np.int32)
        lib.nk_dots_symmetric_i8(b.ctypes.data, 5, 7, 7, g.ctypes.data, 24, 1, 2)
        assert (g[:, :5] == -1).all() and (g[:, 5] == 0).all()
        # the wide types' stubs poison 8 bytes per output
        d = np.zeros((3, 6), np.float64)
        lib.nk_dots_packed_f64(d.ctypes.data, packed.ctypes.data, d.ctypes.data, 3, 5, 6, 48, 48)
        assert np.isnan(d[:, :5]).all() and (d[:, 5] == 0).all()
    finally:
        lib.nk_dispatch_table_update(lib.nk_capabilities_compiled())
    assert lib.nk_dots_packed_size_i8(5, 7) == 64 + 16 * 512 + 256


def test_no_gpu_means_loud_failure_not_fallback():
    lib = nk.library()
    if lib.nk_hip_device_count() > 0:
        pytest.skip("a GPU is present")
    a = np.ones((2, 16), np.int8)
    packed = np.zeros(nk.dots_packed_size("i8", 2, 16), np.uint8)
    lib.nk_dots_pack_i8(a.ctypes.data, 2, 16, 16, packed.ctypes.data)
    assert b"no HIP device" in lib.nk_amd_last_error()
    c = np.zeros((2, 2), np.int32)
    lib.nk_dots_packed_i8(a.ctypes.data, packed.ctypes.data, c.ctypes.data, 2, 2, 16, 16, 8)
    assert (c == -1).all() and b"no HIP device" in lib.nk_amd_last_error()
    c[:] = 0
    lib.nk_dots_symmetric_i8(a.ctypes.data, 2, 16, 16, c.ctypes.data, 8, 0, 2)
    assert (c == -1).all() and b"no HIP device" in lib.nk_amd_last_error()


def test_symmetric_workspace_size():
    """The packed image of the vectors from the window's 32-row boundary on, rounded up to 256 bytes, plus room for the
    tile lists of two launches: each at most 8 bytes per 64 x 128 tile of the window and a word per 8 tile rows."""
    lib = nk.library()
    for t in TYPES:
        code = api.DTYPES[t][0]
        for n, k, start, rows in [(100, 64, 0, 100), (1000, 300, 37, 411), (8192, 1024, 4096, 4096)]:
            size = lib.nk_amd_symmetric_workspace_size(code, n, k, start, rows)
            image = nk.dots_packed_size(t, n - start // 32 * 32, k)
            tiles = -(-min(rows, n - start) // 64) * -(-(n - start // 32 * 32) // 128)
            assert (image + 255) // 256 * 256 < size <= (image + 255) // 256 * 256 + 2 * (8 * tiles + 4 * (tiles // 8 + 4) + 8)
        assert lib.nk_amd_symmetric_workspace_size(code, 100, 64, 100, 5) == 0  # an empty window needs nothing
        assert lib.nk_amd_symmetric_workspace_size(code, 100, 64, 0, 0) == 0


def test_python_mirror_validates_arguments():
    import torch

    cpu = torch.zeros(4, 4, dtype=torch.int8)
    if not torch.cuda.is_available():  # host operands are staged by the library: without a GPU it says so, it never computes
        with pytest.raises(nk.NumKongAmdError, match="no HIP device"):
            nk.dots_pack(cpu, "i8")
        with pytest.raises(nk.NumKongAmdError, match="no HIP device"):
            nk.dots_symmetric(cpu, "i8")
    with pytest.raises(ValueError):
        nk.dots_pack(torch.zeros(4, 4, 2, dtype=torch.int8), "i8")  # two dimensions
    with pytest.raises(TypeError):
        nk.dots_pack(cpu, "f16c")
    with pytest.raises(TypeError):
        nk.dots_pack([[1, 2]], "i8")
    with pytest.raises(TypeError):
        nk.dots_packed(cpu, object())
    with pytest.raises(ValueError):
        nk.dots_symmetric(cpu[:, ::2], "i8")  # rows must be contiguous
    with pytest.raises(TypeError):
        nk.angulars_symmetric(cpu, "f16c")
    with pytest.raises(TypeError):
        nk.euclideans_symmetric(cpu, "u1")  # single bits have the dot-product kinds only
