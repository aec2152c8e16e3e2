"""ctypes binding of libxma_rocm.so (the C ABI declared in include/xma_rocm.h).

The library is built offline by ``build.py`` next to this package.  There is no
fallback: if it is missing, or a call returns an error code, the caller gets an
exception.
"""

from __future__ import annotations

import ctypes
import os
import threading


LIBRARY_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libxma_rocm.so")
ABI_VERSION = 1

_lib = None
_lock = threading.Lock()


class RocmLibraryError(RuntimeError):
    pass


_p, _i64, _i32, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); one line per declaration of include/xma_rocm.h
SIGNATURES = {
    "xma_rocm_abi_version": (_int, []),
    "xma_rocm_last_error": (ctypes.c_char_p, []),
    "xma_rocm_continuous_count_workspace_bytes": (_sz, [_i64, _i32]),
    "xma_rocm_continuous_count": (_int, [_p, _int, _i64, _p, _i32, _p, _sz, _p]),
    "xma_rocm_continuous_count_set_workspace_bytes": (_sz, [_i64, _i32]),
    "xma_rocm_continuous_count_set": (_int, [_p, _int, _i64, _p, _i32, _p, _sz, _p]),
    "xma_rocm_route_workspace_bytes": (_sz, [_i64, _i32]),
    "xma_rocm_route_set_rank_method": (_int, [_int]),
    "xma_rocm_route": (_int, [_p, _int, _i64, _i32, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "xma_rocm_route_static_max_units_times_experts": (_sz, []),
    "xma_rocm_route_static": (_int, [_p, _int, _i64, _i32, _p, _p, _p, _p, _p, _p]),
    "xma_rocm_scatter2scatter_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32]),
    "xma_rocm_scatter2scatter": (
        _int,
        [_p, _i64, _p, _i64, _i64, _int, _p, _p, _p, _i64, _p, _i64, _p, _i64, _i32, _i32, _i32, _i32, _int, _int, _int, _int,
         _p, _sz, _p],
    ),
    "xma_rocm_scatter2scatter_bias": (
        _int,
        [_p, _i64, _p, _i64, _i64, _int, _p, _p, _p, _i64, _p, _i64, _p, _p, _i64, _i64, _i32, _i32, _i32, _i32, _int, _int,
         _int, _int, _p, _sz, _p],
    ),
    "xma_rocm_expert_column_sums": (_int, [_p, _i64, _p, _i32, _p, _p, _p, _i64, _i32, _i32, _int, _p]),
    "xma_rocm_down_projection_dx_swiglu": (
        _int,
        [_p, _i64, _p, _i64, _i64, _p, _p, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _i32, _i32, _i32, _i32, _int,
         _p, _sz, _p],
    ),
    "xma_rocm_group_bwd_W": (
        _int,
        [_p, _i64, _int, _i32, _p, _p, _i64, _int, _i32, _p, _p, _p, _i64, _i64, _i32, _i32, _i32, _int, _p],
    ),
    "xma_rocm_scatter2scatter_few_rows_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32, _int, _int]),
    "xma_rocm_scatter2scatter_few_rows": (
        _int,
        [_p, _i64, _p, _i64, _i64, _int, _p, _p, _p, _i64, _p, _i64, _p, _i64, _p, _p, _i64, _i64, _i32, _i32, _i32, _i32,
         _int, _int, _int, _int, _p, _sz, _p],
    ),
    "xma_rocm_group_bwd_W_few_rows": (
        _int,
        [_p, _i64, _int, _i32, _p, _p, _i64, _int, _i32, _p, _p, _p, _i64, _i64, _i32, _i32, _i32, _i64, _int, _p],
    ),
    "xma_rocm_group": (_int, [_p, _i64, _p, _p, _i64, _p, _i64, _i32, _i32, _int, _p]),
    "xma_rocm_combine": (_int, [_p, _i64, _p, _p, _i64, _i64, _i32, _i32, _int, _p]),
    "xma_rocm_combine_bwd": (_int, [_p, _i64, _p, _i64, _p, _i64, _i32, _i32, _int, _p]),
    "xma_rocm_swiglu_packed_forward": (_int, [_p, _i64, _p, _i64, _i64, _i32, _int, _p]),
    "xma_rocm_swiglu_packed_backward": (_int, [_p, _i64, _p, _i64, _p, _i64, _i64, _i32, _int, _p]),
    "xma_rocm_swiglu_forward": (_int, [_p, _i64, _p, _i64, _p, _i64, _i64, _i32, _int, _p]),
    "xma_rocm_swiglu_backward": (_int, [_p, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _i64, _i32, _int, _p]),
    "xma_rocm_router_topk": (_int, [_p, _i64, _i64, _i32, _i32, _int, _p, _p, _int, _p]),
    "xma_rocm_router_gate_topk_supported": (_int, [_i32, _i32, _i32, _int]),
    "xma_rocm_router_gate_topk": (_int, [_p, _i64, _p, _i64, _i64, _i32, _i32, _i32, _int, _p, _i64, _p, _p, _int, _p]),
    "xma_rocm_router_topk_bwd": (_int, [_p, _i64, _i64, _i32, _i32, _int, _p, _int, _p, _p, _i64, _p]),
    "xma_rocm_diag_mfma_stream": (_int, [_p, _i32, _p, _i32, _p]),
}


def is_library_built() -> bool:
    return os.path.isfile(LIBRARY_PATH)


def get_library() -> ctypes.CDLL:
    """Load the library once; raise RocmLibraryError when it is absent or of another ABI."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not is_library_built():
                raise RocmLibraryError(
                    f"{LIBRARY_PATH} is missing: build it with `python accelerated-model-architectures_amd/build.py` "
                    "(hipcc --offload-arch=gfx950); KernelBackend.rocm has no fallback"
                )
            lib = ctypes.CDLL(LIBRARY_PATH)
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            if lib.xma_rocm_abi_version() != ABI_VERSION:
                raise RocmLibraryError(f"ABI version {lib.xma_rocm_abi_version()} != {ABI_VERSION}")
            _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = get_library().xma_rocm_last_error().decode(errors="replace")
        raise RocmLibraryError(f"{what} failed with code {rc}: {msg}")
