"""ctypes binding of libflexsae_amd.so, the C-ABI library of HIP kernels (include/flexsae_amd.h).

There is no fallback: if the library is missing or does not load, every fused op raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# FLEXSAE_AMD_LIBRARY names another build of the library to load instead of the in-tree one
LIB_PATH = os.environ.get("FLEXSAE_AMD_LIBRARY") or os.path.join(_HERE, "libflexsae_amd.so")

ABI_VERSION = 3

# flexsae_status
OK = 0
ERR_INVALID_ARGUMENT = -1
ERR_UNSUPPORTED = -2
ERR_WORKSPACE = -3
ERR_LAUNCH = -4
ERR_ALIGNMENT = -5
ERR_SCRATCH_LIMIT = -6

# flexsae_dtype
F32, BF16, F16 = 0, 1, 2

FLAG_INDEX_RANGE = 1
BWD_OUTPUTS_PREZEROED = 1
BWD_REUSE_PAIR_LIST = 2
BWD_SWEEP_ONLY = 4
BWD_REDUCE_ONLY = 8
BWD_SCALE_BY_GRAD_OUT = 16
BWD_NO_DW = 32
BWD_SKIP_EPILOGUE = 64
BWD_HOT_LATENTS = 128
BWD_HOT_NO_HEADROOM = 512
BWD_REUSE_HOT_TABLES = 1024
BWD_DENSE_LATENTS = 2048
TOPK_BWD_FP32_RESIDUAL = 256


class Shape(ctypes.Structure):
    """Mirror of ``flexsae_shape``."""

    _fields_ = [
        ("B", ctypes.c_int64), ("K", ctypes.c_int64), ("F", ctypes.c_int64), ("D", ctypes.c_int64),
        ("weight_dtype", ctypes.c_int32), ("vals_dtype", ctypes.c_int32),
        ("bias_dtype", ctypes.c_int32), ("target_dtype", ctypes.c_int32),
    ]


class FlexSAELibraryError(RuntimeError):
    pass


_p = ctypes.c_void_p
_sz = ctypes.c_size_t
_i64 = ctypes.c_int64
_int = ctypes.c_int
_shape_p = ctypes.POINTER(Shape)

# name -> (restype, argtypes); one entry per declaration in include/flexsae_amd.h
SIGNATURES = {
    "flexsae_abi_version": (_int, []),
    "flexsae_build_id": (ctypes.c_char_p, []),
    "flexsae_status_string": (ctypes.c_char_p, [_int]),
    "flexsae_fwd_workspace_bytes": (_sz, [_shape_p]),
    "flexsae_hier_fwd": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _p, _p]),
    "flexsae_hier_fwd_static": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "flexsae_topk_fwd": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _p, _p]),
    "flexsae_hier_bwd_workspace_bytes": (_sz, [_shape_p, _i64]),
    "flexsae_hier_bwd": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _int, _p, _p, _p, _sz, _int, _p, _p]),
    "flexsae_hier_fwd_bwd_supported": (_int, [_shape_p]),
    "flexsae_hier_fwd_bwd_workspace_bytes": (_sz, [_shape_p, _i64]),
    "flexsae_hier_fwd_bwd": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _int, _p, _p, _p, _sz, _int, _p, _p]),
    "flexsae_hier_sgd_step": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _sz, _int, _p, _p]),
    "flexsae_scale": (_int, [_p, _p, _int, _i64, _p, _p]),
    "flexsae_hier_bwd_atomic": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _p, _int, _p, _p]),
    "flexsae_csr_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "flexsae_csr_build": (_int, [_p, _i64, _i64, _i64, _p, _p, _p, _sz, _p, _p]),
    "flexsae_hier_pair_list_layout": (_int, [_shape_p, ctypes.POINTER(_sz), ctypes.POINTER(_sz)]),
    "flexsae_hier_import_pair_list": (_int, [_shape_p, _p, _p, _p, _sz, _p]),
    "flexsae_topk_bwd": (_int, [_shape_p, _p, _p, _p, _p, _p, _p, _p, _p, _int, _p, _p, _p, _sz, _int, _p]),
    "flexsae_topk_bwd_workspace_bytes": (_sz, [_shape_p, _i64]),
    "flexsae_cast_from_f32": (_int, [_p, _int, _p, _i64, _p]),
    "flexsae_scale_from_f32": (_int, [_p, _int, _p, _i64, _p, _p]),
    "flexsae_hier_hot_latents_supported": (_int, [_shape_p]),
    "flexsae_hier_hot_stats": (_int, [_shape_p, _p, _p, _p]),
    "flexsae_hier_pair_stats": (_int, [_shape_p, _p, _p, _p]),
    "flexsae_hier_fwd_bwd_workspace_bytes_flags": (_sz, [_shape_p, _i64, _int]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise FlexSAELibraryError when it is absent or stale."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FlexSAELibraryError(
            f"{LIB_PATH} not found: build it with `python -m flexsae_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no CPU or eager fallback for the fused ops.")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as exc:  # pragma: no cover - depends on the machine
        raise FlexSAELibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise FlexSAELibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.flexsae_abi_version() != ABI_VERSION:
        raise FlexSAELibraryError(
            f"{LIB_PATH} has ABI version {lib.flexsae_abi_version()}, expected {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def build_id() -> str:
    """Hash of the sources and flags the loaded library was built from (flexsae_amd/build.py)."""
    return load().flexsae_build_id().decode()


def status_string(code: int) -> str:
    return load().flexsae_status_string(int(code)).decode()


def check(code: int, what: str) -> None:
    if code != OK:
        raise FlexSAELibraryError(f"{what} failed: {status_string(code)} (status {code})")
