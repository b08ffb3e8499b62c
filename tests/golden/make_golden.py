"""Write the small golden fixtures under tests/golden/ (inputs + expected outputs, data only).

    python tests/golden/make_golden.py

Expected values come from the double-precision C oracle (oracle/masked_ref.c), which the CPU tests
pin against closed forms, library routines and brute force.  bf16 tensors are stored as their raw
uint16 bit patterns so that the fixtures do not depend on a torch version.
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

from ffn_kernel_amd import workloads as wl  # noqa: E402
from oracle import cref  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def main() -> None:
    gen = torch.Generator().manual_seed(20240)
    # MaskedLinear forward + backward
    M, K, N = 37, 48, 40
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_linear("golden_linear", M, K, N, mask, seed=11, with_grad=True, w_std=0.1)
    y = cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask)
    dx, dWv, dWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    perm, counts = cref.route(w.mask)
    np.savez_compressed(HERE / "linear_M37_K48_N40.npz", x=bits(w.x), Wv=bits(w.Wv), Wt=bits(w.Wt),
                        mask=w.mask.numpy(), grad=bits(w.grad), y=y.numpy(), dx=dx.numpy(), dWv=dWv.numpy(),
                        dWt=dWt.numpy(), perm=perm, counts=counts)
    # MaskedFFN forward (exact and with the intermediate rounded to bf16 once)
    M, d, h = 19, 32, 48
    mask = torch.rand(M, generator=gen) < 0.5
    f = wl.make_ffn("golden_ffn", M, d, h, mask, seed=12, w_std=0.1)
    out = cref.ffn_fwd(f.x, f.W, f.mask)
    out_r = cref.ffn_fwd(f.x, f.W, f.mask, round_mid=True)
    np.savez_compressed(HERE / "ffn_M19_d32_h48.npz", x=bits(f.x), mask=f.mask.numpy(), out=out.numpy(),
                        out_round_mid=out_r.numpy(), **{k: bits(v) for k, v in f.W.items()})
    # a decode-shaped case (d, h multiples of 128)
    M, d, h = 5, 128, 128
    mask = torch.tensor([True, False, False, True, False])
    f = wl.make_ffn("golden_decode", M, d, h, mask, seed=13, w_std=0.08)
    out_r = cref.ffn_fwd(f.x, f.W, f.mask, round_mid=True)
    np.savez_compressed(HERE / "ffn_decode_M5_d128_h128.npz", x=bits(f.x), mask=f.mask.numpy(),
                        out_round_mid=out_r.numpy(), **{k: bits(v) for k, v in f.W.items()})
    # MaskedFFN backward (exact chain rule; the op the reference leaves unimplemented)
    M, d, h = 21, 32, 48
    mask = torch.rand(M, generator=gen) < 0.5
    f = wl.make_ffn("golden_ffn_bwd", M, d, h, mask, seed=14, w_std=0.1)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    dx, dW = cref.ffn_bwd(g, f.x, f.W, f.mask)
    np.savez_compressed(HERE / "ffn_bwd_M21_d32_h48.npz", x=bits(f.x), g=bits(g), mask=f.mask.numpy(), dx=dx.numpy(),
                        **{k: bits(v) for k, v in f.W.items()}, **{"d" + k: v.numpy() for k, v in dW.items()})
    print("wrote", sorted(p.name for p in HERE.glob("*.npz")))


if __name__ == "__main__":
    main()
