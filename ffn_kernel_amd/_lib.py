"""ctypes binding of libffnk.so — the C ABI declared in include/ffnk.h.

The library is the product path: if it is missing, loading fails loudly (there is no
PyTorch/CPU fallback behind these calls).
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_int, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libffnk.so"

OP_LINEAR_FWD, OP_FFN_FWD, OP_LINEAR_BWD, OP_FFN_UP, OP_FFN_DOWN, OP_BWD_DX, OP_BWD_DW, OP_FFN_BWD = range(8)
PATH_MFMA_TILED, PATH_STREAM, PATH_GENERIC = range(3)
STATIC_SCRATCH_BYTES = 32 << 20  # FFNK_STATIC_SCRATCH_BYTES

# Every symbol include/ffnk.h declares, with its ctypes signature.
_SIGNATURES = {
    "ffnk_version": (c_int, []),
    "ffnk_last_error": (c_char_p, []),
    "ffnk_debug_force_tile": (c_int, [c_int]),
    "ffnk_debug_force_splits": (c_int, [c_int]),
    "ffnk_debug_force_bwd_gather": (c_int, [c_int]),
    "ffnk_debug_force_group_m": (c_int, [c_int]),
    "ffnk_route": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "ffnk_workspace_bytes": (c_size_t, [c_int, c_int64, c_int64, c_int64]),
    "ffnk_workspace_bytes_ffn_bwd": (c_size_t, [c_int64] * 9),
    "ffnk_tile_config": (c_int, [c_int, c_int64, c_int64, c_int64, c_void_p]),
    "ffnk_masked_linear_fwd": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p,
                                       c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t,
                                       c_void_p]),
    "ffnk_masked_ffn_fwd": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                    c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                    c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "ffnk_masked_ffn_fwd_ev": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                       c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                       c_int64, c_int64, c_void_p, c_size_t, c_void_p, c_void_p]),
    "ffnk_masked_ffn_fwd_static": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                           c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
                                           c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "ffnk_masked_linear_bwd": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64,
                                       c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                       c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "ffnk_masked_ffn_bwd": (c_int, [c_void_p, c_int64, c_void_p, c_int64,            # g, x
                                    c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,  # W1 W3 U1 U3, strides
                                    c_void_p, c_void_p, c_int64, c_int64,            # W2 U2, strides
                                    c_void_p,                                        # mask
                                    c_void_p, c_int64,                               # dx
                                    c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,  # dW1 dW3 dU1 dU3
                                    c_void_p, c_void_p, c_int64, c_int64,            # dW2 dU2
                                    c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    # the *_routed variants: the plain signature (+ pre where optional) + const ffnk_routing_t*
    "ffnk_masked_linear_fwd_routed": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p,
                                              c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t,
                                              c_void_p, c_void_p]),
    "ffnk_masked_linear_bwd_routed": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                              c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                              c_int64, c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p,
                                              c_void_p]),
    "ffnk_masked_ffn_fwd_routed": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                           c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64,
                                           c_void_p, c_int64,                        # pre (NULL: not kept)
                                           c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p, c_void_p]),
    "ffnk_masked_ffn_bwd_routed": (c_int, [c_void_p, c_int64, c_void_p, c_int64,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                           c_void_p, c_void_p, c_int64, c_int64,
                                           c_void_p,
                                           c_void_p, c_int64,                        # pre (NULL: recompute)
                                           c_void_p, c_int64,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                           c_void_p, c_void_p, c_int64, c_int64,
                                           c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p, c_void_p]),
    "ffnk_masked_ffn_can_save": (c_int, [c_int64, c_int64, c_int64]),
    "ffnk_masked_ffn_fwd_save": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                         c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int64,
                                         c_void_p, c_int64,                          # pre
                                         c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "ffnk_masked_ffn_bwd_saved": (c_int, [c_void_p, c_int64, c_void_p, c_int64,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                          c_void_p, c_void_p, c_int64, c_int64,
                                          c_void_p,
                                          c_void_p, c_int64,                         # pre
                                          c_void_p, c_int64,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                          c_void_p, c_void_p, c_int64, c_int64,
                                          c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


class TileConfig(ctypes.Structure):
    """Mirror of ffnk_tile_config_t."""
    _fields_ = [(n, c_int32) for n in ("path", "block_m", "block_n", "block_k", "waves_m", "waves_n",
                                       "lds_stages", "group_m", "split_k", "direct_lds", "in_place")]

    def as_dict(self) -> dict:
        return {n: getattr(self, n) for n, _ in self._fields_}


class RoutingStruct(ctypes.Structure):
    """Mirror of ffnk_routing_t: device addresses of perm int32[M] and counts int32[2]."""
    _fields_ = [("perm", c_void_p), ("counts", c_void_p)]


class FfnkError(RuntimeError):
    """A positive (hipError_t) return from the library."""


_lib = None


def load() -> ctypes.CDLL:
    """Load libffnk.so once and attach signatures.  Raises if the library was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m ffn_kernel_amd.build` "
            "(hipcc, gfx950). There is no fallback path.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """Map a C-ABI return code to a Python exception (negative: bad argument, positive: HIP)."""
    if code == 0:
        return
    msg = load().ffnk_last_error().decode("utf-8", "replace")
    if code < 0:
        raise ValueError(f"{what}: {msg} (ffnk code {code})")
    raise FfnkError(f"{what}: {msg} (hipError_t {code})")


def workspace_bytes(op: int, M: int, K: int, N: int) -> int:
    n = load().ffnk_workspace_bytes(op, M, K, N)
    if n == ctypes.c_size_t(-1).value:
        raise ValueError(f"ffnk_workspace_bytes: invalid op/extents op={op} M={M} K={K} N={N}")
    return n


def tile_config(op: int, M: int, K: int, N: int) -> dict:
    cfg = TileConfig()
    check(load().ffnk_tile_config(op, M, K, N, ctypes.byref(cfg)), "ffnk_tile_config")
    return cfg.as_dict()
