"""ctypes binding of libmoonep_hip.so (the C ABI declared in include/moonep_hip.h).

The library is loaded on first use.  There is no fallback: if it has not been
built, every operator raises.
"""

from __future__ import annotations

import ctypes as C
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoonep_hip.so")

_lock = threading.Lock()
_lib = None

# combine modes / dispatch flags (include/moonep_hip.h)
COMBINE_PRIMARIES = 0
COMBINE_ALL = 1
COMBINE_TWO_LEVEL = 2
COMBINE_WEIGHTED = 3
DISPATCH_WRITE_DUPS = 1
DISPATCH_NO_ZERO_FILL = 2
REDUCE_NO_CLEAR = 1
REDUCE_CLEAR_ONLY = 2

_p = C.c_void_p
_i = C.c_int
_i64 = C.c_int64
_sz = C.c_size_t

_SIGNATURES = {
    "mep_version": (_i, []),
    "mep_init": (_i, []),
    "mep_strerror": (C.c_char_p, [_i]),
    "mep_stream_create_limited": (_i, [_i, C.POINTER(_p)]),
    "mep_stream_destroy": (_i, [_p]),
    "mep_stream_cu_census": (_i, [_p, _i, _p]),
    "mep_plan_scratch_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "mep_plan": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "mep_plan_warm": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _sz, _p, _sz, _p]),
    "mep_plan_ranks": (_i, [_p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "mep_dispatch": (_i, [_p, _p, _p, _p, _p, _i64, _p, _i64, _i, _i, _i, _i, _i, _i, _i, _i,
                          C.c_uint, _p]),
    "mep_dedup_scratch_bytes": (_sz, [_i, _i]),
    "mep_build_dedup": (_i, [_p, _i, _i, _i, _i, _i, _p, _p, _p, _p, _sz, _p]),
    "mep_build_dedup_static": (_i, [_p, _i, _i, _i, _i, _i, _p, _p, _p, _p]),
    "mep_dispatch_epilogue": (_i, [_p, _p, _p, _p, _i, _i, _i, _p]),
    "mep_combine_prologue": (_i, [_p, _p, _p, _p, _i, _i, _i, _p]),
    "mep_combine": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p]),
    "mep_prefetch": (_i, [_i, C.POINTER(_p), C.POINTER(_p), C.POINTER(_i64), C.POINTER(_i64),
                          _p, _i, _i, _i, _p]),
    "mep_prefetch_pull": (_i, [_i, C.POINTER(_p), C.POINTER(_i64), C.POINTER(_p), C.POINTER(_i64),
                               C.POINTER(_i64), _p, _i, _i, _i, _p]),
    "mep_grad_reduce": (_i, [_p, _p, _i64, _p, _i, _i, _i, _i64, C.c_uint, _p]),
    "mep_set_gemm_row_tile": (_i, [_i]),
    "mep_grouped_gemm_nt": (_i, [_p, _p, _p, _p, _i, _p, _p, _i, _i, _i, _i, _p]),
    "mep_grouped_swiglu_nt": (_i, [_p, _p, _p, _p, _i, _p, _p, _p, _i, _i, _i, _p]),
    "mep_grouped_gemm_dual_nt": (_i, [_p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _p]),
    "mep_grouped_gemm_nn": (_i, [_p, _p, _p, _i, _p, _p, _i, _i, _i, _p]),
    "mep_grouped_gemm_dual_nn": (_i, [_p, _p, _p, _p, _p, _i, _p, _i, _i, _i, _p]),
    "mep_grouped_gemm_wgrad": (_i, [_p, _p, _p, _i, _p, _i, _i, _i64, _i, _p]),
    "mep_grouped_gemm_wgrad_tn": (_i, [_p, _p, _p, _i, _p, _i, _i, _i64, _i, _p]),
    "mep_transpose_bf16": (_i, [_p, _p, _i, _i, _i, _p]),
    "mep_swiglu_bwd": (_i, [_p, _p, _p, _p, _p, _i, _p, _p, _p, _p, _i, _i, _p]),
}

EXPORTS = tuple(_SIGNATURES)
ABI_VERSION = 200     # mep_version() of the library these signatures were written against
# hipError_t values that say "no usable GPU in this process" (hipErrorNoDevice,
# hipErrorInvalidDevice, hipErrorInsufficientDriver): loading the library there is fine
_NO_GPU_CODES = (100, 101, 35)


def lib():
    """The loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} is missing: build it with `python -m moonep_amd.build` "
                        "(hipcc, gfx950). moonep_amd has no CPU or eager fallback."
                    )
                handle = C.CDLL(LIB_PATH)
                for name, (res, args) in _SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = res
                    fn.argtypes = args
                found = handle.mep_version()
                if found != ABI_VERSION:
                    raise RuntimeError(
                        f"{LIB_PATH} has ABI version {found}, this binding needs {ABI_VERSION}: "
                        "rebuild it with `python -m moonep_amd.build`")
                # LDS opt-ins of the current device, outside any stream capture
                rc = handle.mep_init()
                if rc != 0 and rc not in _NO_GPU_CODES:
                    raise RuntimeError(f"mep_init failed: {handle.mep_strerror(rc).decode()} (code {rc})")
                _lib = handle
    return _lib


def init_device() -> None:
    """``mep_init`` for the current device (a process may use several)."""
    check(lib().mep_init(), "mep_init")


def check(code: int, what: str) -> None:
    """Turn a non-zero return code of the C ABI into RuntimeError."""
    if code != 0:
        msg = lib().mep_strerror(code).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")


def ptr(t) -> int | None:
    """Device address of a tensor (None stays NULL)."""
    return None if t is None else t.data_ptr()


def current_stream() -> int:
    import torch

    return torch.cuda.current_stream().cuda_stream
