"""ctypes binding of libnumkong_amd.so and the host-side mirror of the reference's Python API.

Reference behaviour mirrored here (python/matrix.c):
  * ``dots_pack(b, dtype)`` -> ``PackedMatrix``                     (:151-227)
  * ``dots_packed(a, packed, out=None)`` -> ``C = A @ B.T``          (:324-490)
  * ``dots_symmetric(vectors, dtype, out=None, start_row=None, end_row=None)`` and the two distance forms:
    upper triangle of all pairs of one set of vectors                (:492-622)
  * output dtype per input dtype: i8->i32, u8->u32, floats->f32     (include/numkong/numkong.h:41-45)
  * shape / dtype / stride validation raising ``ValueError``/``TypeError`` (:162-197, :378-421)

There is no CPU fallback: if the shared library is missing, loading raises; if a call fails on the
GPU side, ``NumKongAmdError`` is raised with the library's own message.

Operands may live in GPU memory (torch CUDA tensors, DLPack exporters) or in host memory (numpy arrays, torch CPU
tensors: what a caller of the reference has). Host operands are staged by the library (pinned buffers, two streams;
a packed image in host memory is uploaded once and found again by the number in its header); the result is then a
host array of the same kind as ``a``. The arithmetic always runs on the GPU.

Streams: the synchronous calls run on streams the library keeps per host thread. They are blocking streams, so they
are ordered behind work queued on the legacy default stream (torch's default) and return when the result is
complete. ONLY the legacy default stream is ordered with them: operands produced on any other stream of the
caller's, blocking or not (blocking streams are ordered against the default stream, not against each other), and
work this library's own ``*_async`` entry points were given on such a stream, must be synchronised before a
synchronous call reads them; or the ``*_async`` entry points are used with that stream throughout.
"""
from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))

# nk_dtype_t codes (reference: include/numkong/types.h:923-952)
NK_I8, NK_I32, NK_U8, NK_U32 = 1 << 2, 1 << 4, 1 << 6, 1 << 8
NK_F64, NK_F32, NK_F16, NK_BF16, NK_E4M3, NK_E5M2 = 1 << 10, 1 << 11, 1 << 12, 1 << 13, 1 << 14, 1 << 15
NK_I4, NK_U4, NK_E2M3, NK_E3M2, NK_U1 = 1 << 16, 1 << 17, 1 << 18, 1 << 19, 1 << 1

# name -> (nk code, bytes per stored value, output torch dtype name, dimensions per stored value)
DTYPES = {
    "i8": (NK_I8, 1, "int32", 1),
    "u8": (NK_U8, 1, "int32", 1),  # u32 results are returned as their int32 bit patterns
    "bf16": (NK_BF16, 2, "float32", 1),
    "f16": (NK_F16, 2, "float32", 1),
    "e4m3": (NK_E4M3, 1, "float32", 1),
    "e5m2": (NK_E5M2, 1, "float32", 1),
    "e2m3": (NK_E2M3, 1, "float32", 1),  # 6-bit floats, one per byte
    "e3m2": (NK_E3M2, 1, "float32", 1),
    "i4": (NK_I4, 1, "int32", 2),  # two 4-bit values per byte: a (rows, depth / 2) byte tensor, as the reference's
    "u4": (NK_U4, 1, "int32", 2),  # bindings take them (python/matrix.c:603: depth *= dimensions per value)
    "u1": (NK_U1, 1, "int32", 8),  # eight bits per byte; the dot product is popcount(a & b)
    "f32": (NK_F32, 4, "float64", 1),  # the two wide types give f64 results
    "f64": (NK_F64, 8, "float64", 1),
}


# the types that also have the distance kinds (the 6-bit floats and 4-bit integers have dot products only)
DISTANCE_DTYPES = ("i8", "u8", "bf16", "f16", "e4m3", "e5m2", "e2m3", "e3m2", "i4", "u4", "f32", "f64")


class NumKongAmdError(RuntimeError):
    """A call into libnumkong_amd.so failed (no GPU, bad packed image, launch error)."""


def library_path() -> str:
    """The in-tree build, unless NUMKONG_AMD_LIBRARY names another build of the same library."""
    return os.environ.get("NUMKONG_AMD_LIBRARY") or os.path.join(_HERE, "lib", "libnumkong_amd.so")


_LIB: Optional[ctypes.CDLL] = None


def library() -> ctypes.CDLL:
    """Load the in-tree shared library (built by ``make -C numkong_amd/csrc``). Never falls back."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = library_path()
    if not os.path.exists(path):
        raise NumKongAmdError(
            f"{path} is missing: build it with `make -C numkong_amd/csrc` (there is no CPU fallback)"
        )
    try:  # torch ships its own HIP runtime: load it first, so that the library binds to the same one
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(path)
    sz, vp, i32 = ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int
    for name in DTYPES:
        getattr(lib, f"nk_dots_packed_size_{name}").restype = sz
        getattr(lib, f"nk_dots_packed_size_{name}").argtypes = [sz, sz]
        getattr(lib, f"nk_dots_pack_{name}").restype = None
        getattr(lib, f"nk_dots_pack_{name}").argtypes = [vp, sz, sz, sz, vp]
        getattr(lib, f"nk_dots_packed_{name}").restype = None
        getattr(lib, f"nk_dots_packed_{name}").argtypes = [vp, vp, vp, sz, sz, sz, sz, sz]
        for stem in ("nk_angulars_packed_", "nk_euclideans_packed_") if name in DISTANCE_DTYPES else ():
            getattr(lib, stem + name).restype = None
            getattr(lib, stem + name).argtypes = [vp, vp, vp, sz, sz, sz, sz, sz]
        stems = ("nk_dots_symmetric_", "nk_angulars_symmetric_", "nk_euclideans_symmetric_")
        for stem in stems if name in DISTANCE_DTYPES else stems[:1]:
            getattr(lib, stem + name).restype = None
            getattr(lib, stem + name).argtypes = [vp, sz, sz, sz, vp, sz, sz, sz]
    lib.nk_amd_symmetric_workspace_size.restype = sz
    lib.nk_amd_symmetric_workspace_size.argtypes = [i32, sz, sz, sz, sz]
    lib.nk_amd_symmetric_async.restype = i32
    lib.nk_amd_symmetric_async.argtypes = [i32, i32, vp, sz, sz, sz, vp, sz, sz, sz, vp, sz, vp]
    lib.nk_amd_symmetric_static_capacity.restype = sz
    lib.nk_amd_symmetric_static_capacity.argtypes = []
    lib.nk_amd_symmetric_static_async.restype = i32
    lib.nk_amd_symmetric_static_async.argtypes = [i32, i32, vp, sz, sz, sz, vp, sz, sz, sz, vp]
    lib.nk_amd_last_error.restype = ctypes.c_char_p
    lib.nk_amd_dots_pack_async.restype = i32
    lib.nk_amd_dots_pack_async.argtypes = [i32, vp, sz, sz, sz, vp, vp]
    lib.nk_amd_dots_packed_async.restype = i32
    lib.nk_amd_dots_packed_async.argtypes = [i32, vp, vp, vp, sz, sz, sz, sz, sz, vp]
    lib.nk_amd_spatials_packed_async.restype = i32
    lib.nk_amd_spatials_packed_async.argtypes = [i32, i32, vp, vp, vp, sz, sz, sz, sz, sz, vp]
    lib.nk_hip_last_error.restype = ctypes.c_char_p
    lib.nk_hip_set_tile_config.argtypes = [i32]
    lib.nk_hip_set_tile_config.restype = None
    lib.nk_hip_device_count.restype = i32
    lib.nk_capabilities.restype = ctypes.c_uint64
    lib.nk_configure_thread.argtypes = [ctypes.c_uint64]
    lib.nk_configure_thread.restype = i32
    lib.nk_capabilities_compiled.restype = ctypes.c_uint64
    lib.nk_capabilities_available.restype = ctypes.c_uint64
    lib.nk_find_kernel_punned.restype = None
    lib.nk_find_kernel_punned.argtypes = [i32, i32, ctypes.c_uint64, ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_uint64)]
    lib.nk_dispatch_table_update.argtypes = [ctypes.c_uint64]
    lib.nk_dispatch_table_update.restype = None
    lib.nk_kernel_output_dtype.argtypes = [i32, i32]
    lib.nk_kernel_output_dtype.restype = i32
    _LIB = lib
    return lib


def _check(where: str) -> None:
    message = library().nk_amd_last_error()
    if message:
        raise NumKongAmdError(f"{where}: {message.decode()}")


def dots_packed_size(dtype: str, width: int, depth: int) -> int:
    if dtype not in DTYPES:
        raise TypeError(f"unsupported dtype {dtype!r}; expected one of {sorted(DTYPES)}")
    return int(getattr(library(), f"nk_dots_packed_size_{dtype}")(width, depth))


@dataclass
class PackedMatrix:
    """B packed for the GPU kernels; ``buffer`` is a uint8 tensor holding the relocatable image, in GPU memory when B was
    there and in host memory otherwise (the library then keeps a device copy, found again by the number in the header)."""

    __array_ufunc__ = None  # numpy: `array @ packed` is this class's to answer (__rmatmul__), not a ufunc over objects

    dtype: str
    width: int  # rows of B = columns of C
    depth: int
    buffer: "object"

    @property
    def nbytes(self) -> int:
        return int(self.buffer.numel())

    @property
    def shape(self):
        """(width, depth), as the reference's PackedMatrix reports it."""
        return (self.width, self.depth)

    @classmethod
    def packed_size(cls, width: int, depth: int, dtype: str = None) -> int:
        """Bytes of the packed image for a shape and dtype: the reference's ``PackedMatrix.packed_size(width, depth, /,
        dtype)`` (python/matrix.c:75-129), which asks for the dtype as well."""
        if dtype is None:
            raise TypeError("packed_size() requires 'dtype' argument")
        return dots_packed_size(dtype, int(width), int(depth))

    def __rmatmul__(self, a):
        """``a @ packed`` is ``dots_packed(a, packed)``: the reference's ``Tensor @ PackedMatrix`` (python/matrix.c:324-490)."""
        return dots_packed(a, self)


def _inferred_dtype(t) -> str:
    """The packing dtype of a tensor whose element type says it (the reference's ``dtype=None``, python/matrix.c:632-647);
    the sub-byte and 6-bit types have no tensor type of their own and must be named."""
    import torch

    names = {torch.int8: "i8", torch.uint8: "u8", torch.bfloat16: "bf16", torch.float16: "f16", torch.float32: "f32",
             torch.float64: "f64"}
    for attribute, name in (("float8_e4m3fn", "e4m3"), ("float8_e5m2", "e5m2")):
        if hasattr(torch, attribute):
            names[getattr(torch, attribute)] = name
    t = _as_tensor(t)
    if not isinstance(t, torch.Tensor) or t.dtype not in names:
        raise TypeError("dtype cannot be inferred from this input; name one of " + str(sorted(DTYPES)))
    return names[t.dtype]


def _is_numpy(t) -> bool:
    return type(t).__module__ == "numpy" and type(t).__name__ == "ndarray"


def _as_tensor(t):
    """A torch view of the operand, without a copy: numpy arrays (host memory), DLPack exporters, tensors as they are."""
    import torch

    if isinstance(t, torch.Tensor):
        return t
    if _is_numpy(t):
        import numpy

        if t.dtype == numpy.uint16:  # raw bf16 / f16 bits: torch has no arithmetic on uint16 and needs none here
            t = t.view(numpy.int16)
        elif t.dtype == numpy.uint32:
            t = t.view(numpy.int32)
        return torch.from_numpy(t)
    if hasattr(t, "__dlpack__"):
        return torch.from_dlpack(t)  # any DLPack exporter (reference: python/dlpack_interop.c)
    return t


def _as_matrix(t, dtype: str, what: str):
    import torch

    if dtype not in DTYPES:
        raise TypeError(f"unsupported dtype {dtype!r}; expected one of {sorted(DTYPES)}")
    t = _as_tensor(t)
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what} must be a torch.Tensor, a numpy array or export DLPack")
    if t.dim() != 2:
        raise ValueError(f"{what} must be 2-dimensional, got {t.dim()} dimensions")
    if t.element_size() != DTYPES[dtype][1]:
        raise TypeError(f"{what} has {t.element_size()}-byte elements, dtype {dtype!r} needs {DTYPES[dtype][1]}")
    if t.shape[1] > 1 and t.stride(1) != 1:
        raise ValueError(f"{what} rows must be contiguous (stride of the last dimension must be 1)")
    return t


def dots_pack(b, dtype: str = None) -> PackedMatrix:
    """Pack row-major ``b`` (width x depth, raw element bits in a same-width torch dtype); ``dtype`` defaults to the
    tensor's own element type."""
    import torch

    if dtype is None:
        dtype = _inferred_dtype(b)
    b = _as_matrix(b, dtype, "b")
    width, depth = int(b.shape[0]), int(b.shape[1]) * DTYPES[dtype][3]
    size = dots_packed_size(dtype, width, depth)
    if size == 0:
        raise NumKongAmdError("nk_dots_packed_size returned 0 (unsupported dtype or dimensions)")
    buffer = torch.empty(size, dtype=torch.uint8, device=b.device)
    stride = int(b.stride(0)) * b.element_size() if width > 1 else int(b.shape[1]) * b.element_size()
    getattr(library(), f"nk_dots_pack_{dtype}")(b.data_ptr(), width, depth, stride, buffer.data_ptr())
    _check("nk_dots_pack_" + dtype)
    return PackedMatrix(dtype, width, depth, buffer)


def _result_matrix(out, shape, out_dtype_name: str, like, as_numpy: bool, zeroed: bool):
    """The tensor the library writes into and what the caller gets back: ``out`` itself when given (a tensor or a
    numpy array, validated), else a new matrix where ``like`` lives, handed back as a numpy array for numpy operands."""
    import torch

    out_dtype = getattr(torch, out_dtype_name)
    if out is None:
        tensor = (torch.zeros if zeroed else torch.empty)(shape, dtype=out_dtype, device=like.device)
        return tensor, (tensor.numpy() if as_numpy else tensor)
    tensor = _as_tensor(out)
    if not isinstance(tensor, torch.Tensor) or tensor.dim() != 2:
        raise ValueError("out must be a 2-dimensional tensor or array")
    if tuple(tensor.shape) != tuple(shape):
        raise ValueError(f"out has shape {tuple(tensor.shape)}, expected {tuple(shape)}")
    if tensor.dtype != out_dtype:
        raise TypeError(f"out must have dtype {out_dtype}")
    if shape[1] > 1 and tensor.stride(1) != 1:
        raise ValueError("out rows must be contiguous")
    return tensor, out


def _packed_product(stem: str, out_dtype_name, a, packed: PackedMatrix, out, start_row=None, end_row=None):
    if not isinstance(packed, PackedMatrix):
        raise TypeError("packed must be a PackedMatrix from dots_pack()")
    as_numpy = _is_numpy(a)
    a = _as_matrix(a, packed.dtype, "a")
    height, depth = int(a.shape[0]), int(a.shape[1]) * DTYPES[packed.dtype][3]
    if depth != packed.depth:
        raise ValueError(f"depth mismatch: a has {depth} columns, packed matrix has depth {packed.depth}")
    out, result = _result_matrix(out, (height, packed.width), out_dtype_name, a, as_numpy, False)
    a_stride = int(a.stride(0)) * a.element_size() if height > 1 else int(a.shape[1]) * a.element_size()
    c_stride = int(out.stride(0)) * out.element_size() if height > 1 else packed.width * out.element_size()
    # rows [start_row, end_row) of a, into the same rows of out; the others are left as they were
    # (reference: python/matrix.c:453-464)
    first = 0 if start_row is None or int(start_row) < 0 else int(start_row)
    last = height if end_row is None or int(end_row) < 0 else int(end_row)
    if first > height or last > height or first > last:
        raise ValueError(f"Invalid row range [{first}, {last}) for matrix with {height} rows")
    if last > first:
        getattr(library(), stem + packed.dtype)(
            a.data_ptr() + first * a_stride, packed.buffer.data_ptr(), out.data_ptr() + first * c_stride, last - first,
            packed.width, depth, a_stride, c_stride
        )
    _check(stem + packed.dtype)
    return result


def dots_packed(a, packed: PackedMatrix, out=None, start_row=None, end_row=None, threads=None):
    """``C[height x width] = a @ B.T`` with widened accumulators; ``out`` (optional) is overwritten. With ``start_row``
    / ``end_row`` only those rows of ``a`` are multiplied, into the same rows of ``out`` (reference:
    ``dots_packed(a, b, /, *, out=None, start_row=None, end_row=None)``, python/matrix.c:780-796). ``threads``, which
    the reference's calls also take (python/matrix.c:354-358), is accepted and means nothing here: the rows are spread
    over the GPU's compute units by the one launch."""
    return _packed_product("nk_dots_packed_", DTYPES[packed.dtype][2] if isinstance(packed, PackedMatrix) else "float32",
                           a, packed, out, start_row, end_row)


def _needs_distances(dtype: str) -> None:
    if dtype not in DISTANCE_DTYPES:
        raise TypeError(f"dtype {dtype!r} has the dot-product kinds only; distances need one of {DISTANCE_DTYPES}")


def _distance_dtype(dtype) -> str:
    """float32 distances, float64 for f32 and f64 inputs (reference: include/numkong/spatials.h:72-137)."""
    return "float64" if dtype in ("f32", "f64") else "float32"


def angulars_packed(a, packed: PackedMatrix, out=None, start_row=None, end_row=None, threads=None):
    """Angular distances ``1 - cos(a_i, b_j)`` as float32, float64 for f32 and f64 inputs (reference:
    ``nk_angulars_packed_<dtype>``)."""
    if isinstance(packed, PackedMatrix):
        _needs_distances(packed.dtype)
    return _packed_product("nk_angulars_packed_", _distance_dtype(getattr(packed, "dtype", None)), a, packed, out,
                           start_row, end_row)


def euclideans_packed(a, packed: PackedMatrix, out=None, start_row=None, end_row=None, threads=None):
    """Euclidean distances ``|a_i - b_j|`` as float32, float64 for f32 and f64 inputs (reference:
    ``nk_euclideans_packed_<dtype>``)."""
    if isinstance(packed, PackedMatrix):
        _needs_distances(packed.dtype)
    return _packed_product("nk_euclideans_packed_", _distance_dtype(getattr(packed, "dtype", None)), a, packed, out,
                           start_row, end_row)


def _symmetric(stem: str, out_dtype_name: str, vectors, dtype: str, out, start_row, end_row):
    as_numpy = _is_numpy(vectors)
    vectors = _as_matrix(vectors, dtype, "vectors")
    count, depth = int(vectors.shape[0]), int(vectors.shape[1]) * DTYPES[dtype][3]
    # (the reference leaves what it does not write uninitialised; zeros are easier on the eye)
    out, result = _result_matrix(out, (count, count), out_dtype_name, vectors, as_numpy, True)
    first = 0 if start_row is None else int(start_row)
    last = count if end_row is None else int(end_row)
    if first < 0 or last < 0 or first > count or last > count or first > last:
        raise ValueError(f"Invalid row range [{first}, {last}) for {count} vectors")
    stride = int(vectors.stride(0)) * vectors.element_size() if count > 1 else int(vectors.shape[1]) * vectors.element_size()
    out_stride = int(out.stride(0)) * out.element_size() if count > 1 else count * out.element_size()
    getattr(library(), stem + dtype)(vectors.data_ptr(), count, depth, stride, out.data_ptr(), out_stride, first, last - first)
    _check(stem + dtype)
    return result


def dots_symmetric(vectors, dtype: str = None, out=None, start_row=None, end_row=None, threads=None):
    """Upper triangle (diagonal included) of ``vectors @ vectors.T`` for the rows ``[start_row, end_row)``, widened as
    in ``dots_packed``; the rest of ``out`` is left as it was (zeros when allocated here). ``dtype`` defaults to the
    tensor's own element type."""
    if dtype is None:
        dtype = _inferred_dtype(vectors)
    if dtype not in DTYPES:
        raise TypeError(f"unsupported dtype {dtype!r}; expected one of {sorted(DTYPES)}")
    return _symmetric("nk_dots_symmetric_", DTYPES[dtype][2], vectors, dtype, out, start_row, end_row)


def angulars_symmetric(vectors, dtype: str = None, out=None, start_row=None, end_row=None, threads=None):
    """Upper triangle of the pairwise angular distances as float32 (float64 for f32 and f64 inputs); the diagonal is
    exactly 0."""
    if dtype is None:
        dtype = _inferred_dtype(vectors)
    _needs_distances(dtype)
    return _symmetric("nk_angulars_symmetric_", _distance_dtype(dtype), vectors, dtype, out, start_row, end_row)


def euclideans_symmetric(vectors, dtype: str = None, out=None, start_row=None, end_row=None, threads=None):
    """Upper triangle of the pairwise euclidean distances as float32 (float64 for f32 and f64 inputs); the diagonal is
    exactly 0."""
    if dtype is None:
        dtype = _inferred_dtype(vectors)
    _needs_distances(dtype)
    return _symmetric("nk_euclideans_symmetric_", _distance_dtype(dtype), vectors, dtype, out, start_row, end_row)
