"""MI355X-native packed batched dot products behind NumKong's C ABI.

The product is ``numkong_amd/lib/libnumkong_amd.so`` (hand-written gfx950 HIP kernels plus a C
dispatch layer exporting the reference's ``nk_dots_packed_size_*``, ``nk_dots_pack_*``,
``nk_dots_packed_*`` symbols). This package is the thin Python host side over it: it mirrors the
reference's Python entry points ``dots_pack`` / ``dots_packed`` / ``dots_symmetric`` and the distance forms
(reference: python/matrix.c:151-227, 324-622) for tensors that already live on the GPU, using PyTorch only to own device memory.
"""
from .api import (  # noqa: F401
    DISTANCE_DTYPES,
    DTYPES,
    NumKongAmdError,
    PackedMatrix,
    angulars_packed,
    angulars_symmetric,
    dots_pack,
    dots_packed,
    dots_packed_size,
    dots_symmetric,
    euclideans_packed,
    euclideans_symmetric,
    library,
    library_path,
)
