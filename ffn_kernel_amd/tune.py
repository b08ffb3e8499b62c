"""Tile tuner for gfx950 — the counterpart of the reference's find_spec searches
(find_spec/find.py:6-64, find_spec/bf16_linear_fwd.py, bf16_ffn_fwd.py, bf16_linear_bwd.py).

The reference grid-searches Triton block sizes per sequence length and stores the winner in JSON
tables.  Here the candidate set is the tile shapes compiled into libffnk (include/ffnk.h,
ffnk_debug_force_tile); the tuner times every candidate on a list of shapes with HIP events,
reports min-of-k like the reference (find.py:35-63), and prints which candidate the built-in
table (csrc/tile_table.hpp) picks, so that the table can be checked against measurements.

    python -m ffn_kernel_amd.tune [--trials 5] [--json out.json] [--shapes cfg | M,K,N ...]
"""
from __future__ import annotations

import argparse
import json
import sys

import torch

from . import _lib
from .ops import masked_ffn_forward, masked_linear_backward, masked_linear_forward

TILES = {0: "256x256/8w", 1: "256x256/4w", 2: "128x128/4w", 3: "small/4w"}


def _time(fn, trials: int) -> float:
    fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(trials):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        best = min(best, a.elapsed_time(b))
    return best


def tune_shape(op: str, M: int, K: int, N: int, trials: int, dev) -> dict:
    """op = linear_fwd (K in, N out), ffn_fwd (K = d, N = h) or linear_bwd."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    mask = (torch.rand(M, generator=g) < 0.5).to(dev)
    mk = lambda r, c: (torch.randn(r, c, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    if op == "ffn_fwd":
        W = [mk(N, K), mk(K, N), mk(N, K), mk(N, K), mk(K, N), mk(N, K)]  # w1, w2, w3, u1, u2, u3 (nn.Linear layout)
        fn = lambda: masked_ffn_forward(x, *[w.T for w in W], mask)
        flops = 2 * M * K * N * 3
        table = {"up": _lib.tile_config(_lib.OP_FFN_UP, M, K, N), "down": _lib.tile_config(_lib.OP_FFN_DOWN, M, K, N)}
    elif op == "linear_fwd":
        Wv, Wt = mk(N, K), mk(N, K)
        fn = lambda: masked_linear_forward(x, Wv.T, Wt.T, mask)
        flops = 2 * M * K * N
        table = {"fwd": _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)}
    elif op == "linear_bwd":
        Wv, Wt = mk(N, K), mk(N, K)
        grad = torch.randn(M, N, generator=g).to(torch.bfloat16).to(dev)
        fn = lambda: masked_linear_backward(grad, x, Wv.T, Wt.T, mask)
        flops = 4 * M * K * N
        table = {"dx": _lib.tile_config(_lib.OP_BWD_DX, M, K, N), "dw": _lib.tile_config(_lib.OP_BWD_DW, M, K, N)}
    else:
        raise ValueError(op)
    lib = _lib.load()
    rec = {"op": op, "M": M, "K": K, "N": N, "candidates_ms": {}, "table": table}
    try:
        for tile, name in TILES.items():
            lib.ffnk_debug_force_tile(tile)
            rec["candidates_ms"][name] = _time(fn, trials)
        lib.ffnk_debug_force_tile(-1)
        rec["table_ms"] = _time(fn, trials)
    finally:
        lib.ffnk_debug_force_tile(-1)
    best = min(rec["candidates_ms"], key=rec["candidates_ms"].get)
    rec["best"] = best
    rec["best_ms"] = rec["candidates_ms"][best]
    rec["table_vs_best"] = rec["table_ms"] / rec["best_ms"]
    rec["routed_tflops_table"] = flops / rec["table_ms"] / 1e9
    return rec


DEFAULT_SHAPES = [
    ("linear_fwd", 2048, 1024, 1024),    # cfg1
    ("linear_fwd", 8192, 1024, 1024),
    ("linear_fwd", 32768, 4096, 4096),
    ("ffn_fwd", 2048, 1024, 2048),
    ("ffn_fwd", 8192, 1024, 2048),       # cfg2
    ("ffn_fwd", 128, 4096, 14336),       # just above the decode path
    ("ffn_fwd", 1024, 4096, 14336),
    ("ffn_fwd", 4096, 4096, 14336),
    ("ffn_fwd", 32768, 4096, 14336),     # cfg4
    ("linear_bwd", 8192, 1024, 1024),    # cfg3
]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m ffn_kernel_amd.tune")
    ap.add_argument("--trials", type=int, default=5)
    ap.add_argument("--json", default=None)
    ap.add_argument("--shapes", nargs="*", default=None, help="op:M,K,N ... (default: the benchmark configurations)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("ffn_kernel_amd.tune needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    shapes = DEFAULT_SHAPES
    if args.shapes:
        shapes = []
        for s in args.shapes:
            op, dims = s.split(":")
            shapes.append((op, *map(int, dims.split(","))))
    out = []
    for op, M, K, N in shapes:
        rec = tune_shape(op, M, K, N, args.trials, dev)
        out.append(rec)
        cand = "  ".join(f"{k}={v:.3f}" for k, v in rec["candidates_ms"].items())
        print(f"{op:11s} M={M:6d} K={K:5d} N={N:5d} | {cand} | table={rec['table_ms']:.3f} ms "
              f"({rec['routed_tflops_table']:.0f} TFLOP/s routed) best={rec['best']} table/best={rec['table_vs_best']:.3f}",
              flush=True)
    if args.json:
        with open(args.json, "w") as f:
            json.dump(out, f, indent=1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
