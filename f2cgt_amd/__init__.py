"""f2cgt_amd — MI355X-native (gfx950) drop-in for the fused feature-decompression +
neighbour-aggregation operators of F2CGT.

    import f2cgt_amd
    capi = f2cgt_amd.load()          # the module the reference imports as `F2CGTLib`
    out = capi.vq_decompress_spmm_csr(codes, codebooks, indptr, indices, feat_dim)

`load()` imports the in-tree pybind extension (f2cgt_amd/lib/F2CGTLib.*.so, built by
`python -m f2cgt_amd.build`) and also registers it as the top-level module `F2CGTLib`, so
`import F2CGTLib as capi` in existing callers keeps working.  There is no CPU fallback:
a missing extension raises ImportError.
"""
from __future__ import annotations

import os
import sys

__all__ = ["load", "lib_dir", "capi_path"]

_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")


def lib_dir() -> str:
    return _LIB


def capi_path() -> str:
    """Path of the C-ABI shared library (see include/f2cgt.h); F2CGT_AMD_CAPI_LIB names another build of it
    (same ABI), e.g. to compare two builds in one session."""
    return os.environ.get("F2CGT_AMD_CAPI_LIB") or os.path.join(_LIB, "libf2cgt_hip.so")


def load():
    """Import and return the `F2CGTLib` extension module."""
    import torch  # noqa: F401  (libtorch and the HIP runtime must be loaded first)

    if "F2CGTLib" in sys.modules:
        return sys.modules["F2CGTLib"]
    if not os.path.exists(capi_path()):
        raise ImportError(
            "f2cgt_amd: %s is missing; build it with `python -m f2cgt_amd.build`" % capi_path())
    if _LIB not in sys.path:
        sys.path.insert(0, _LIB)
    try:
        import F2CGTLib  # type: ignore
    except ImportError as exc:  # no fallback on purpose
        raise ImportError(
            "f2cgt_amd: the F2CGTLib extension is not built or not loadable (%s); "
            "run `python -m f2cgt_amd.build`" % exc) from exc
    return F2CGTLib
