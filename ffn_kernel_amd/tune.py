"""Tile tuner for gfx950: searches the plan lattice on the GPU and PRODUCES the measured part of the tile
table, as the reference's find_spec searches produce its JSON tables (find_spec/find.py:18-64 lattice
search with min-of-3 timing; find_spec/bf16_linear_fwd.py, bf16_ffn_fwd.py, bf16_linear_bwd.py:86-99 emit
the tables that ffn_kernel/linear.py:8-12 reads at import).

The lattice is (tile id) x (split-K factor) per operation, layer shape and M bucket:
  * MaskedFFN forward: the SwiGLU GEMM's tile, and the down projection's (tile, split-K factor), timed
    per stage with the events of ffnk_masked_ffn_fwd_ev;
  * MaskedLinear forward: (tile, split-K factor) of the routed GEMM, whole call;
  * MaskedLinear backward: the weight-gradient GEMM's split-K factor, whole call.
Every candidate is forced through ffnk_debug_force_tile / ffnk_debug_force_splits and timed min-of-k;
the baseline is the library's rules and cost model alone (ffnk_debug_force_tile(-2)).  Wherever the best
candidate beats the baseline by more than --margin, an entry goes into csrc/tile_table_gen.hpp, which
pick_routed_plan / pick_routed_tile / pick_splitk_tile (csrc/tile_table.hpp) consult before the rules.

    python -m ffn_kernel_amd.tune                 # sweep, print the comparison
    python -m ffn_kernel_amd.tune --emit          # ... and rewrite csrc/tile_table_gen.hpp (then rebuild)
    python -m ffn_kernel_amd.tune --quick         # two buckets per layer (smoke test of the harness)
"""
from __future__ import annotations

import argparse
import ctypes
import json
import sys
from pathlib import Path

import torch

from . import _lib
from .ops import masked_linear_backward, masked_linear_forward

TILES = {0: "256x256/8w", 1: "256x256/4w", 2: "128x128/4w", 3: "small/4w"}
SPLITS = (1, 2, 3, 4, 6, 7, 8, 12, 14, 16)
TUNED_PLAIN, TUNED_DUAL, TUNED_SPLITK = 0, 1, 2
GEN_PATH = Path(__file__).resolve().parent / "csrc" / "tile_table_gen.hpp"

# M buckets [lo, hi]; each is measured at its upper end.  Below 65 rows the FFN runs the streaming kernels.
BUCKETS = [(65, 128), (129, 256), (257, 512), (513, 1024), (1025, 2048), (2049, 4096), (4097, 8192), (8193, 16384),
           (16385, 32768)]
FFN_LAYERS = [(1024, 2048), (4096, 14336)]      # (d, h): cfg2 and cfg4 / cfg5
LINEAR_LAYERS = [(1024, 1024), (4096, 4096)]    # (K, N): cfg1 / cfg3 and an LLM-size projection


class _Events:
    """Three hipEvent_t for the stage boundaries of ffnk_masked_ffn_fwd_ev."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.ev = (ctypes.c_void_p * 3)()
        for i in range(3):
            h = ctypes.c_void_p()
            if self.hip.hipEventCreate(ctypes.byref(h)) != 0:
                raise RuntimeError("hipEventCreate failed")
            self.ev[i] = h

    def ms(self, i, j):
        out = ctypes.c_float()
        if self.hip.hipEventElapsedTime(ctypes.byref(out), self.ev[i], self.ev[j]) != 0:
            raise RuntimeError("hipEventElapsedTime failed")
        return out.value


def _randn(shape, std, gen, dev):
    return (torch.randn(shape, generator=gen, device=dev) * std).to(torch.bfloat16)


class _Forced:
    """Force (tile, splits) for the duration of a block; always back to the table afterwards."""

    def __init__(self, tile, splits):
        self.tile, self.splits = tile, splits

    def __enter__(self):
        lib = _lib.load()
        lib.ffnk_debug_force_tile(self.tile)
        lib.ffnk_debug_force_splits(self.splits)

    def __exit__(self, *exc):
        lib = _lib.load()
        lib.ffnk_debug_force_tile(-1)
        lib.ffnk_debug_force_splits(-1)


def _ffn_stage_ms(x, W, mask, trials, ev):
    """min-of-k (up-projection ms, down-projection ms) of one MaskedFFN forward under the current override."""
    lib = _lib.load()
    M, d = x.shape
    h = W["w1"].shape[0]
    out = torch.empty((M, d), device=x.device, dtype=torch.bfloat16)
    ws = torch.empty(_lib.workspace_bytes(_lib.OP_FFN_FWD, M, d, h), dtype=torch.uint8, device=x.device)
    up, down = float("inf"), float("inf")
    for i in range(trials + 1):
        rc = lib.ffnk_masked_ffn_fwd_ev(x.data_ptr(), d, W["w1"].data_ptr(), W["w3"].data_ptr(), W["u1"].data_ptr(),
                                        W["u3"].data_ptr(), 1, d, W["w2"].data_ptr(), W["u2"].data_ptr(), 1, h,
                                        mask.data_ptr(), out.data_ptr(), d, M, d, h, ws.data_ptr(), ws.numel(),
                                        torch.cuda.current_stream().cuda_stream, ctypes.cast(ev.ev, ctypes.c_void_p))
        _lib.check(rc, "ffnk_masked_ffn_fwd_ev")
        torch.cuda.synchronize()
        if i > 0:  # the first call warms up
            up, down = min(up, ev.ms(0, 1)), min(down, ev.ms(1, 2))
    return up, down


def _call_ms(fn, trials):
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


def _cdiv(a, b):
    return -(-a // b)


def _valid_splits(contraction, M):
    """Split-K factors worth trying: ranges of whole 64-element slabs, at least 8 each, none empty; past
    8192 rows the tiles fill the chip on their own and the fp32 partials would run into gigabytes."""
    nk = contraction // 64
    out = [1]
    if contraction % 64 == 0 and M <= 8192:
        for s in SPLITS[1:]:
            if nk // s >= 8 and _cdiv(nk, _cdiv(nk, s)) == s:
                out.append(s)
    return out


def tune_ffn(d, h, bucket, trials, dev, ev):
    lo, M = bucket
    gen = torch.Generator(device=dev).manual_seed(M)
    x = _randn((M, d), 1.0, gen, dev)
    mask = torch.rand(M, generator=gen, device=dev) < 0.5
    W = {k: _randn((h, d), 0.02, gen, dev) for k in ("w1", "w3", "u1", "u3")}
    W.update({k: _randn((d, h), 0.02, gen, dev) for k in ("w2", "u2")})
    with _Forced(-2, -1):
        base_up, base_down = _ffn_stage_ms(x, W, mask, trials, ev)
        base_cfg = {"up": _lib.tile_config(_lib.OP_FFN_UP, M, d, h), "down": _lib.tile_config(_lib.OP_FFN_DOWN, M, d, h)}
    ups, downs = {}, {}
    for tile in TILES:
        for s in _valid_splits(h, M):
            if tile == 1 and s > 1:
                continue  # the four-wave 256x256 tile is not run split
            with _Forced(tile, s):
                got_s = _lib.tile_config(_lib.OP_FFN_DOWN, M, d, h)["split_k"]
                if got_s != s:
                    continue  # the shape does not take this factor
                u, dn = _ffn_stage_ms(x, W, mask, trials, ev)
            ups[tile] = min(ups.get(tile, float("inf")), u)
            downs[(tile, s)] = dn
    return {"op": "ffn_fwd", "d": d, "h": h, "m_lo": lo, "m_hi": M, "rules": base_cfg, "rules_up_ms": base_up,
            "rules_down_ms": base_down, "up_ms": ups, "down_ms": downs}


def tune_linear_fwd(K, N, bucket, trials, dev):
    lo, M = bucket
    gen = torch.Generator(device=dev).manual_seed(M + 1)
    x = _randn((M, K), 1.0, gen, dev)
    mask = torch.rand(M, generator=gen, device=dev) < 0.5
    Wv, Wt = _randn((N, K), 0.02, gen, dev), _randn((N, K), 0.02, gen, dev)
    fn = lambda: masked_linear_forward(x, Wv.T, Wt.T, mask)
    with _Forced(-2, -1):
        base = _call_ms(fn, trials)
        base_cfg = _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)
    cand = {}
    if base_cfg["path"] == _lib.PATH_MFMA_TILED:
        for tile in TILES:
            for s in _valid_splits(K, M):
                if tile == 1 and s > 1:
                    continue
                with _Forced(tile, s):
                    if _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)["split_k"] != s:
                        continue
                    cand[(tile, s)] = _call_ms(fn, trials)
    return {"op": "linear_fwd", "K": K, "N": N, "m_lo": lo, "m_hi": M, "rules": base_cfg, "rules_ms": base, "ms": cand}


def tune_linear_bwd(K, N, bucket, trials, dev):
    lo, M = bucket
    gen = torch.Generator(device=dev).manual_seed(M + 2)
    x = _randn((M, K), 1.0, gen, dev)
    g = _randn((M, N), 1.0, gen, dev)
    mask = torch.rand(M, generator=gen, device=dev) < 0.5
    Wv, Wt = _randn((N, K), 0.02, gen, dev), _randn((N, K), 0.02, gen, dev)
    fn = lambda: masked_linear_backward(g, x, Wv.T, Wt.T, mask)
    with _Forced(-2, -1):
        base = _call_ms(fn, trials)
        base_cfg = _lib.tile_config(_lib.OP_BWD_DW, M, K, N)
    cand = {}
    slabs = max(1, (M // 2) // 64)
    for s in SPLITS:
        if s > slabs:
            continue
        with _Forced(-2, s):
            cand[s] = _call_ms(fn, trials)
    return {"op": "linear_bwd", "K": K, "N": N, "m_lo": lo, "m_hi": M, "rules": base_cfg, "rules_ms": base, "ms": cand}


def plans_from(records, margin):
    """Table entries (op, m_lo, m_hi, k, n, tile, splits) for every record whose best candidate beats the
    rules by more than `margin`."""
    out = []
    for r in records:
        if r["op"] == "ffn_fwd":
            if r["up_ms"]:
                tile = min(r["up_ms"], key=r["up_ms"].get)
                if r["up_ms"][tile] < r["rules_up_ms"] * (1 - margin):
                    out.append((TUNED_DUAL, r["m_lo"], r["m_hi"], r["d"], r["h"], tile, 1))
            if r["down_ms"]:
                tile, s = min(r["down_ms"], key=r["down_ms"].get)
                if r["down_ms"][(tile, s)] < r["rules_down_ms"] * (1 - margin):
                    out.append((TUNED_PLAIN, r["m_lo"], r["m_hi"], r["h"], r["d"], tile, s))
        elif r["op"] == "linear_fwd" and r["ms"]:
            tile, s = min(r["ms"], key=r["ms"].get)
            if r["ms"][(tile, s)] < r["rules_ms"] * (1 - margin):
                out.append((TUNED_PLAIN, r["m_lo"], r["m_hi"], r["K"], r["N"], tile, s))
        elif r["op"] == "linear_bwd" and r["ms"]:
            s = min(r["ms"], key=r["ms"].get)
            if r["ms"][s] < r["rules_ms"] * (1 - margin):
                tile = {(256, 256): 0, (128, 128): 2}.get((r["rules"]["block_m"], r["rules"]["block_n"]), 2)
                out.append((TUNED_SPLITK, r["m_lo"], r["m_hi"], r["N"], r["K"], tile, s))  # R = N, Cc = K (dW stored [N, K])
    # one entry per key: a linear layer and an FFN's down projection can share (k, n); keep the first
    seen, uniq = set(), []
    for e in sorted(out):
        if e[:5] not in seen:
            seen.add(e[:5])
            uniq.append(e)
    return uniq


def render_header(plans) -> str:
    lines = ["// Measured plans of the gfx950 tile table.  GENERATED by `python -m ffn_kernel_amd.tune --emit`: do not edit.",
             "// {op, m_lo, m_hi, k, n, tile, splits}; see TunedPlan in tile_table.hpp.",
             "#pragma once", "namespace ffnk {", "constexpr TunedPlan kTunedPlans[] = {"]
    for e in plans:
        lines.append("    {%d, %d, %d, %d, %d, %d, %d}," % e)
    lines += ["    {-1, 0, 0, 0, 0, 0, 0},", "};", "}  // namespace ffnk", ""]
    return "\n".join(lines)


def _fmt(d):
    return "  ".join(f"{k}={v:.3f}" for k, v in d.items())


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m ffn_kernel_amd.tune")
    ap.add_argument("--trials", type=int, default=5, help="timed calls per candidate; the minimum counts")
    ap.add_argument("--margin", type=float, default=0.04, help="a candidate must beat the rules by this fraction")
    ap.add_argument("--emit", action="store_true", help=f"rewrite {GEN_PATH.name}")
    ap.add_argument("--out", type=Path, default=GEN_PATH, help="where --emit writes")
    ap.add_argument("--json", default=None, help="dump every measurement")
    ap.add_argument("--quick", action="store_true", help="two buckets per layer")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("ffn_kernel_amd.tune needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ev = _Events()
    buckets = [BUCKETS[1], BUCKETS[4]] if args.quick else BUCKETS
    records = []
    for d, h in FFN_LAYERS:
        for b in buckets:
            if b[1] * h * 2 > 4 << 30:
                continue
            r = tune_ffn(d, h, b, args.trials, dev, ev)
            records.append(r)
            print(f"ffn_fwd    d={d:5d} h={h:5d} M<={b[1]:6d} | rules up {r['rules_up_ms']:.3f} "
                  f"(tile {r['rules']['up']['block_m']}x{r['rules']['up']['block_n']}/{r['rules']['up']['waves_m'] * r['rules']['up']['waves_n']}w)"
                  f" down {r['rules_down_ms']:.3f} | up by tile: {_fmt({TILES[k]: v for k, v in r['up_ms'].items()})}"
                  f" | best down: {min(r['down_ms'], key=r['down_ms'].get)} {min(r['down_ms'].values()):.3f}", flush=True)
    for K, N in LINEAR_LAYERS:
        for b in buckets:
            r = tune_linear_fwd(K, N, b, args.trials, dev)
            records.append(r)
            best = min(r["ms"], key=r["ms"].get) if r["ms"] else None
            print(f"linear_fwd K={K:5d} N={N:5d} M<={b[1]:6d} | rules {r['rules_ms']:.3f} | best {best} "
                  f"{r['ms'][best] if best else float('nan'):.3f}", flush=True)
            r = tune_linear_bwd(K, N, b, args.trials, dev)
            records.append(r)
            best = min(r["ms"], key=r["ms"].get)
            print(f"linear_bwd K={K:5d} N={N:5d} M<={b[1]:6d} | rules {r['rules_ms']:.3f} (splits {r['rules']['split_k']}) | "
                  f"by splits: {_fmt({str(k): v for k, v in r['ms'].items()})}", flush=True)
    plans = plans_from(records, args.margin)
    print(f"{len(plans)} measured plans beat the rules by more than {args.margin:.0%}:")
    for e in plans:
        print("   op=%d M in [%d, %d] k=%d n=%d -> tile %d, splits %d" % e)
    if args.json:
        def keyed(d):
            return {str(k): v for k, v in d.items()} if isinstance(d, dict) else d
        with open(args.json, "w") as f:
            json.dump([{k: keyed(v) for k, v in r.items()} for r in records], f, indent=1)
    if args.emit:
        args.out.write_text(render_header(plans))
        print(f"wrote {args.out}; rebuild the library (python -m ffn_kernel_amd.build) to use it")
    return 0


if __name__ == "__main__":
    sys.exit(main())
