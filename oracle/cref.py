"""ctypes wrapper of oracle/_build/libmasked_ref.so (the plain-C double-precision oracle)."""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_int64, c_void_p

import numpy as np
import torch

from .build import LIB, build_oracle

_lib = None


def _load():
    global _lib
    if _lib is None:
        if not LIB.exists():
            build_oracle(verbose=False)
        _lib = ctypes.CDLL(str(LIB))
        _lib.ref_masked_linear_fwd.argtypes = [c_void_p] * 5 + [c_int64] * 3
        _lib.ref_masked_ffn_fwd.argtypes = [c_void_p] * 9 + [c_int64] * 3 + [c_int]
        _lib.ref_masked_linear_bwd.argtypes = [c_void_p] * 8 + [c_int64] * 3
        _lib.ref_masked_ffn_bwd.argtypes = [c_void_p] * 16 + [c_int64] * 3 + [c_int]
        _lib.ref_route.argtypes = [c_void_p, c_int64, c_void_p, c_void_p]
        for f in (_lib.ref_masked_linear_fwd, _lib.ref_masked_ffn_fwd, _lib.ref_masked_linear_bwd,
                  _lib.ref_masked_ffn_bwd, _lib.ref_route):
            f.restype = None
    return _lib


def _bits(t: torch.Tensor) -> np.ndarray:
    """Raw bf16 bit patterns of a CPU bf16 tensor as a contiguous uint16 array."""
    assert t.dtype == torch.bfloat16 and t.device.type == "cpu"
    return np.ascontiguousarray(t.contiguous().view(torch.int16).numpy().view(np.uint16))


def _mask(mask: torch.Tensor) -> np.ndarray:
    return np.ascontiguousarray(mask.cpu().numpy().astype(np.uint8))


def _p(a: np.ndarray):
    return a.ctypes.data_as(c_void_p)


def linear_fwd(x, Wv, Wt, mask) -> torch.Tensor:
    M, K = x.shape
    N = Wv.shape[0]
    xb, vb, tb, mb = _bits(x), _bits(Wv), _bits(Wt), _mask(mask)
    y = np.zeros((M, N), dtype=np.float64)
    _load().ref_masked_linear_fwd(_p(xb), _p(vb), _p(tb), _p(mb), _p(y), M, K, N)
    return torch.from_numpy(y)


def ffn_fwd(x, W, mask, round_mid: bool = False) -> torch.Tensor:
    M, d = x.shape
    h = W["w1"].shape[0]
    arrs = [_bits(x)] + [_bits(W[k]) for k in ("w1", "w2", "w3", "u1", "u2", "u3")] + [_mask(mask)]
    out = np.zeros((M, d), dtype=np.float64)
    _load().ref_masked_ffn_fwd(*[_p(a) for a in arrs], _p(out), M, d, h, int(round_mid))
    return torch.from_numpy(out)


def linear_bwd(g, x, Wv, Wt, mask):
    M, K = x.shape
    N = Wv.shape[0]
    arrs = [_bits(g), _bits(x), _bits(Wv), _bits(Wt), _mask(mask)]
    dx = np.zeros((M, K)); dWv = np.zeros((N, K)); dWt = np.zeros((N, K))
    _load().ref_masked_linear_bwd(*[_p(a) for a in arrs], _p(dx), _p(dWv), _p(dWt), M, K, N)
    return torch.from_numpy(dx), torch.from_numpy(dWv), torch.from_numpy(dWt)


def ffn_bwd(g, x, W, mask, round_mid: bool = False):
    """(dx [M, d], dict of weight gradients in nn.Linear layout) from the C loops."""
    M, d = x.shape
    h = W["w1"].shape[0]
    arrs = [_bits(g), _bits(x)] + [_bits(W[k]) for k in ("w1", "w2", "w3", "u1", "u2", "u3")] + [_mask(mask)]
    dx = np.zeros((M, d))
    outs = {"w1": np.zeros((h, d)), "w2": np.zeros((d, h)), "w3": np.zeros((h, d)),
            "u1": np.zeros((h, d)), "u2": np.zeros((d, h)), "u3": np.zeros((h, d))}
    _load().ref_masked_ffn_bwd(*[_p(a) for a in arrs], _p(dx), *[_p(outs[k]) for k in ("w1", "w2", "w3", "u1", "u2", "u3")],
                               M, d, h, int(round_mid))
    return torch.from_numpy(dx), {k: torch.from_numpy(v) for k, v in outs.items()}


def route(mask):
    mb = _mask(mask)
    M = mb.shape[0]
    perm = np.zeros(M, dtype=np.int32)
    counts = np.zeros(2, dtype=np.int32)
    _load().ref_route(_p(mb), M, _p(perm), _p(counts))
    return perm, counts
