"""Tile tuner for gfx950: searches the plan lattice on the GPU and PRODUCES the measured part of the tile
table, as the reference's find_spec searches produce its JSON tables (find_spec/find.py:18-64 lattice
search with min-of-3 timing; find_spec/bf16_linear_fwd.py, bf16_ffn_fwd.py, bf16_linear_bwd.py:86-99 emit
the tables that ffn_kernel/linear.py:8-12 reads at import).

The lattice is (tile id) x (split-K factor) x (M-tiles per super-group of the tile order) per operation, layer shape
and M bucket - the reference's searches walk BLOCK_SIZE_M/N/K x GROUP_SIZE_M the same way (find_spec/bf16_linear_fwd.py:45-53):
  * MaskedFFN forward: the SwiGLU GEMM's tile, and the down projection's (tile, split-K factor), timed
    per stage with the events of ffnk_masked_ffn_fwd_ev;
  * MaskedLinear forward: (tile, split-K factor) of the routed GEMM, whole call;
  * MaskedLinear backward: the form of the weight-gradient GEMM (from routed transposes on the rules' tile, the same
    with both GEMMs of the fused launch behind the ring of four LDS stages, or from g and x read in place) and its
    split-K factor, whole call.
The super-group size is searched in a second stage, from 4096 rows up (below that a call has too few M-tiles for the
order to matter): the first stage's winner - or the rules' plan, pinned - with 2, 4, 8 and 16 M-tiles per super-group
(ffnk_debug_force_group_m) against that plan with the tile's own size.
Every candidate is forced through ffnk_debug_force_tile / ffnk_debug_force_splits (/ ffnk_debug_force_bwd_gather) and timed min-of-k;
the baseline is the library's rules and cost model alone (ffnk_debug_force_tile(-2)).  The host never
knows how many rows each group holds, and a tile's time jumps where a group's tile count crosses a
multiple of the CU count, so one mask says little about a bucket: every bucket is measured on several
scenarios (its upper end with an i.i.d. mask, its upper end with contiguous spans, a point inside it).
All candidates run the first scenario; the few that beat the baseline there run the others.  An entry
goes into csrc/tile_table_gen.hpp, which pick_routed_plan / pick_routed_tile / pick_splitk_tile
(csrc/tile_table.hpp) consult before the rules, only for a candidate that loses on no scenario and whose
geometric-mean time beats the baseline by more than --margin.

    python -m ffn_kernel_amd.tune                 # sweep, print the comparison
    python -m ffn_kernel_amd.tune --emit          # ... and rewrite csrc/tile_table_gen.hpp (then rebuild)
    python -m ffn_kernel_amd.tune --passes 2 --emit   # two sweeps; a plan must win in both (the committed table)
    python -m ffn_kernel_amd.tune --quick         # two buckets per layer (smoke test of the harness)
    python -m ffn_kernel_amd.tune --ffn 5120,13824 --linear 5120,5120 --emit   # ... with a model's own layers added
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

TILES = {0: "256x256/8w", 1: "256x256/4w", 2: "128x128/4w", 3: "small/4w", 4: "128x128/ring4"}
GROUP_MS = (2, 4, 8, 16)   # M-tiles per super-group tried in the second stage
GM_MIN_ROWS = 4096         # ... for buckets that reach this many rows
TILE_IN_PLACE = 5  # weight-gradient plans only (kTileGatherDw in csrc/capi.hip): g and x read where they lie
SPLITS = (1, 2, 3, 4, 6, 7, 8, 12, 14, 16)
TUNED_PLAIN, TUNED_DUAL, TUNED_SPLITK, TUNED_DOWN = 0, 1, 2, 3  # TunedOp in csrc/tile_table.hpp
GEN_PATH = Path(__file__).resolve().parent / "csrc" / "tile_table_gen.hpp"

# M buckets [lo, hi]; each is measured at its upper end.  Below 65 rows the FFN runs the streaming kernels.
BUCKETS = [(65, 128), (129, 256), (257, 512), (513, 1024), (1025, 2048), (2049, 4096), (4097, 8192), (8193, 16384),
           (16385, 32768), (32769, 65536), (65537, 131072)]  # up to the last key of the reference's tables (bf16_ffn_bwd.json)
FFN_LAYERS = [(1024, 2048), (2048, 8192), (4096, 14336), (5120, 13824), (8192, 28672)]  # (d, h): cfg2, a mid-size layer, cfg4 / cfg5, two larger LLM layers
LINEAR_LAYERS = [(1024, 1024), (2048, 2048), (4096, 4096), (8192, 8192)]  # (K, N): cfg1 / cfg3 and LLM-size projections


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
    """Force (tile, splits) for the duration of a block; always back to the table afterwards.  The weight-gradient
    form goes with the tile: TILE_IN_PLACE forces it on (over the rules' tile for the dx GEMM), any other candidate
    forces it off, and the baseline (-2, -1) leaves it to the rules."""

    def __init__(self, tile, splits, group_m=0):
        self.tile, self.splits, self.group_m = tile, splits, group_m

    def __enter__(self):
        lib = _lib.load()
        lib.ffnk_debug_force_tile(-2 if self.tile == TILE_IN_PLACE else self.tile)
        lib.ffnk_debug_force_splits(self.splits)
        lib.ffnk_debug_force_bwd_gather(-1 if (self.tile, self.splits) == (-2, -1) else int(self.tile == TILE_IN_PLACE))
        lib.ffnk_debug_force_group_m(self.group_m)

    def __exit__(self, *exc):
        lib = _lib.load()
        lib.ffnk_debug_force_tile(-1)
        lib.ffnk_debug_force_splits(-1)
        lib.ffnk_debug_force_bwd_gather(-1)
        lib.ffnk_debug_force_group_m(0)


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


def _span_mask(M, frac, n_seq, gen, dev):
    """n_seq sequences of M / n_seq rows, each with one contiguous span of about frac of its rows set."""
    mask = torch.zeros(M, dtype=torch.bool, device=dev)
    seq = max(1, M // n_seq)
    span = max(1, int(seq * frac))
    for b in range(n_seq):
        start = b * seq + int(torch.randint(0, max(1, seq - span), (1,), generator=gen, device=dev))
        mask[start:start + span] = True
    return mask


def _scenarios(bucket, gen, dev):
    """[(M, mask)]: the bucket's upper end with an i.i.d. mask, the same with spans, and a point inside."""
    lo, hi = bucket
    mid = lo + (hi - lo) * 2 // 5
    return [(hi, torch.rand(hi, generator=gen, device=dev) < 0.5),
            (hi, _span_mask(hi, 0.3, 4, gen, dev)),
            (mid, _span_mask(mid, 0.6, 2, gen, dev))]


def _shortlist(base0, cand0, margin, keep=3):
    """Keys of the candidates that beat the baseline on the first scenario, best first, at most `keep`."""
    good = sorted((t, k) for k, t in cand0.items() if t < base0 * (1 - margin))
    return [k for _, k in good[:keep]]


def _geomean(xs):
    p = 1.0
    for x in xs:
        p *= x
    return p ** (1.0 / len(xs))


def _tile_id(cfg, dual):
    """Tile id behind an answer of ffnk_tile_config for a routed GEMM."""
    if cfg["block_m"] == 256:
        return 0 if cfg["waves_m"] * cfg["waves_n"] == 8 else 1
    if cfg["lds_stages"] == 4:
        return 4
    return 2 if cfg["block_m"] == 128 and (dual or cfg["block_n"] == 128) else 3


def _gm_stage(measure, ref, own, margin):
    """Second stage: measure(g) -> [ms per scenario] (or None) of one pinned plan with g M-tiles per super-group.
    A size is selected if, against the same plan with the tile's own size, it loses on no scenario and wins by more
    than margin in the geometric mean - and loses on no scenario against `ref` either, the times of the plan the
    first stage chose (or of the rules, which may pick other tiles inside the bucket than the pinned plan).
    Returns ({g: [ms]} including the own size, selected g or None)."""
    base = measure(own)
    if base is None:
        return {}, None
    got = {own: base}
    for g in GROUP_MS:
        if g != own:
            ts = measure(g)
            if ts is not None:
                got[g] = ts
    cands = {g: ts for g, ts in got.items() if g != own and all(t <= r * 1.01 for t, r in zip(ts, ref))}
    best, _ = _select(base, cands, margin)
    return got, best


def _select(base, cand, margin):
    """(key, geometric-mean ratio) of the best candidate measured on every scenario that loses on none and
    beats the baseline's geometric mean by more than margin; (None, 1.0) when there is none."""
    best, best_r = None, 1.0 - margin
    for k, ts in cand.items():
        if len(ts) != len(base) or any(t > b * 1.01 for t, b in zip(ts, base)):
            continue
        r = _geomean([t / b for t, b in zip(ts, base)])
        if r < best_r:
            best, best_r = k, r
    return best, (best_r if best is not None else 1.0)


def tune_ffn(d, h, bucket, trials, dev, ev, margin):
    lo, hi = bucket
    gen = torch.Generator(device=dev).manual_seed(hi)
    W = {k: _randn((h, d), 0.02, gen, dev) for k in ("w1", "w3", "u1", "u3")}
    W.update({k: _randn((d, h), 0.02, gen, dev) for k in ("w2", "u2")})
    scen = [(_randn((M, d), 1.0, gen, dev), mask) for M, mask in _scenarios(bucket, gen, dev)]
    base_up, base_down = [], []
    with _Forced(-2, -1):
        for x, mask in scen:
            u, dn = _ffn_stage_ms(x, W, mask, trials, ev)
            base_up.append(u)
            base_down.append(dn)
        base_cfg = {"up": _lib.tile_config(_lib.OP_FFN_UP, hi, d, h), "down": _lib.tile_config(_lib.OP_FFN_DOWN, hi, d, h)}

    def run(tile, s, x, mask):
        """(up ms, down ms) under the override, or None when the shape does not take the factor."""
        with _Forced(tile, s):
            if _lib.tile_config(_lib.OP_FFN_DOWN, x.shape[0], d, h)["split_k"] != s:
                return None
            return _ffn_stage_ms(x, W, mask, trials, ev)

    ups0, downs0 = {}, {}
    for tile in TILES:
        for s in _valid_splits(h, hi):
            if tile == 1 and s > 1:
                continue  # the four-wave 256x256 tile is not run split
            got = run(tile, s, *scen[0])
            if got is None:
                continue
            if s == 1:
                ups0[tile] = got[0]
            downs0[(tile, s)] = got[1]
    ups = {t: [ups0[t]] for t in _shortlist(base_up[0], ups0, margin)}
    downs = {k: [downs0[k]] for k in _shortlist(base_down[0], downs0, margin)}
    for key in sorted(set((t, 1) for t in ups) | set(downs)):
        for x, mask in scen[1:]:
            got = run(key[0], key[1], x, mask)
            if got is None:
                break
            if key[1] == 1 and key[0] in ups:
                ups[key[0]].append(got[0])
            if key in downs:
                downs[key].append(got[1])
    # second stage: the super-group size, on the winner of each stage or on the rules' plan at the bucket's upper end
    gm = {}
    if hi >= GM_MIN_ROWS and base_cfg["up"]["path"] == _lib.PATH_MFMA_TILED:
        best_up, _ = _select(base_up, ups, margin)
        best_down, _ = _select(base_down, downs, margin)
        up_plan = (best_up if best_up is not None else _tile_id(base_cfg["up"], True), 1)
        down_plan = best_down if best_down is not None else (_tile_id(base_cfg["down"], False), base_cfg["down"]["split_k"])

        def stage(plan, which):
            def measure(g):
                ts = []
                for x, mask in scen:
                    with _Forced(plan[0], plan[1], g):
                        if which == 1 and _lib.tile_config(_lib.OP_FFN_DOWN, x.shape[0], d, h)["split_k"] != plan[1]:
                            return None
                        ts.append(_ffn_stage_ms(x, W, mask, trials, ev)[which])
                return ts
            return measure
        up_ref = ups[best_up] if best_up is not None else base_up
        down_ref = downs[best_down] if best_down is not None else base_down
        got_up, g_up = _gm_stage(stage(up_plan, 0), up_ref, base_cfg["up"]["group_m"], margin)
        got_down, g_down = _gm_stage(stage(down_plan, 1), down_ref, base_cfg["down"]["group_m"], margin)
        gm = {"up_plan": up_plan, "up_ms": got_up, "up_group_m": g_up, "down_plan": down_plan, "down_ms": got_down,
              "down_group_m": g_down}
    return {"op": "ffn_fwd", "d": d, "h": h, "m_lo": lo, "m_hi": hi, "rules": base_cfg, "rules_up_ms": base_up,
            "rules_down_ms": base_down, "up_first_ms": ups0, "down_first_ms": downs0, "up_ms": ups, "down_ms": downs,
            "group_m": gm}


def _tune_call(make_fn, scen_inputs, candidates, trials, margin):
    """Whole-call counterpart of tune_ffn's search: make_fn(inputs) -> callable; candidates yields
    (key, tile, splits, accept(M) -> bool).  Returns (baseline ms per scenario, {key: ms on the first
    scenario}, {key: [ms per scenario]} for the shortlist)."""
    fns = [make_fn(inp) for inp in scen_inputs]
    with _Forced(-2, -1):
        base = [_call_ms(fn, trials) for fn in fns]
    first = {}
    for key, tile, s, accept in candidates:
        with _Forced(tile, s):
            if accept(scen_inputs[0][0].shape[0]):
                first[key] = (_call_ms(fns[0], trials), tile, s, accept)
    first_ms = {k: v[0] for k, v in first.items()}
    full = {}
    for key in _shortlist(base[0], first_ms, margin):
        _, tile, s, accept = first[key]
        ts = [first_ms[key]]
        with _Forced(tile, s):
            for inp, fn in zip(scen_inputs[1:], fns[1:]):
                if not accept(inp[0].shape[0]):
                    break
                ts.append(_call_ms(fn, trials))
        full[key] = ts
    return base, first_ms, full


def tune_linear_fwd(K, N, bucket, trials, dev, margin):
    lo, hi = bucket
    gen = torch.Generator(device=dev).manual_seed(hi + 1)
    Wv, Wt = _randn((N, K), 0.02, gen, dev), _randn((N, K), 0.02, gen, dev)
    scen = [(_randn((M, K), 1.0, gen, dev), mask) for M, mask in _scenarios(bucket, gen, dev)]
    with _Forced(-2, -1):
        base_cfg = _lib.tile_config(_lib.OP_LINEAR_FWD, hi, K, N)
    cands = []
    if base_cfg["path"] == _lib.PATH_MFMA_TILED:
        for tile in TILES:
            for s in _valid_splits(K, hi):
                if tile == 1 and s > 1:
                    continue
                cands.append(((tile, s), tile, s,
                              lambda M, s=s: _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)["split_k"] == s))
    base, first, full = _tune_call(lambda inp: (lambda: masked_linear_forward(inp[0], Wv.T, Wt.T, inp[1])),
                                   scen, cands, trials, margin)
    gm = {}
    if hi >= GM_MIN_ROWS and base_cfg["path"] == _lib.PATH_MFMA_TILED:
        best, _ = _select(base, full, margin)
        plan = best if best is not None else (_tile_id(base_cfg, False), base_cfg["split_k"])

        def measure(g):
            ts = []
            for x, mask in scen:
                with _Forced(plan[0], plan[1], g):
                    if _lib.tile_config(_lib.OP_LINEAR_FWD, x.shape[0], K, N)["split_k"] != plan[1]:
                        return None
                    ts.append(_call_ms(lambda: masked_linear_forward(x, Wv.T, Wt.T, mask), trials))
            return ts
        got, g_sel = _gm_stage(measure, full[best] if best is not None else base, base_cfg["group_m"], margin)
        gm = {"plan": plan, "ms": got, "group_m": g_sel}
    return {"op": "linear_fwd", "K": K, "N": N, "m_lo": lo, "m_hi": hi, "rules": base_cfg, "rules_ms": base,
            "first_ms": first, "ms": full, "group_m": gm}


def tune_linear_bwd(K, N, bucket, trials, dev, margin):
    lo, hi = bucket
    gen = torch.Generator(device=dev).manual_seed(hi + 2)
    Wv, Wt = _randn((N, K), 0.02, gen, dev), _randn((N, K), 0.02, gen, dev)
    scen = [(_randn((M, K), 1.0, gen, dev), mask, _randn((M, N), 1.0, gen, dev)) for M, mask in _scenarios(bucket, gen, dev)]
    with _Forced(-2, -1):
        base_cfg = _lib.tile_config(_lib.OP_BWD_DW, hi, K, N)
    with _Forced(-2, 1):
        xpose_cfg = _lib.tile_config(_lib.OP_BWD_DW, hi, K, N)  # the rules' tile for the form that reads transposes
    slabs = max(1, (lo // 4) // 64)  # every factor must leave whole slabs in the smaller group of the smallest scenario
    # tile -2: the rules' tile, from transposes, with the factor forced; tile 4: both GEMMs of the fused launch behind
    # the ring of four stages; TILE_IN_PLACE: no transposes
    cands = [((tile, s), tile, s, lambda M: True) for tile in (-2, 4, TILE_IN_PLACE) for s in SPLITS if s <= slabs]
    base, first, full = _tune_call(lambda inp: (lambda: masked_linear_backward(inp[2], inp[0], Wv.T, Wt.T, inp[1])),
                                   scen, cands, trials, margin)
    return {"op": "linear_bwd", "K": K, "N": N, "m_lo": lo, "m_hi": hi, "rules": base_cfg, "rules_xpose": xpose_cfg, "rules_ms": base,
            "first_ms": first, "ms": full}


def plans_from(records, margin):
    """Table entries (op, m_lo, m_hi, k, n, tile, splits, group_m) for every record with a candidate that loses on
    no scenario and beats the rules' geometric-mean time by more than `margin`; a super-group size that won the second
    stage comes with the plan it was measured on (the first stage's winner, or the rules' plan pinned)."""
    out = []
    for r in records:
        gm = r.get("group_m") or {}
        if r["op"] == "ffn_fwd":
            tile, _ = _select(r["rules_up_ms"], r["up_ms"], margin)
            if tile is not None or gm.get("up_group_m"):
                plan = gm["up_plan"] if gm.get("up_group_m") else (tile, 1)
                out.append((TUNED_DUAL, r["m_lo"], r["m_hi"], r["d"], r["h"], plan[0], 1, gm.get("up_group_m") or 0))
            key, _ = _select(r["rules_down_ms"], r["down_ms"], margin)
            if key is not None or gm.get("down_group_m"):
                plan = gm["down_plan"] if gm.get("down_group_m") else key
                out.append((TUNED_DOWN, r["m_lo"], r["m_hi"], r["h"], r["d"], plan[0], plan[1], gm.get("down_group_m") or 0))
        elif r["op"] == "linear_fwd":
            key, _ = _select(r["rules_ms"], r["ms"], margin)
            if key is not None or gm.get("group_m"):
                plan = gm["plan"] if gm.get("group_m") else key
                out.append((TUNED_PLAIN, r["m_lo"], r["m_hi"], r["K"], r["N"], plan[0], plan[1], gm.get("group_m") or 0))
        elif r["op"] == "linear_bwd":
            key, _ = _select(r["rules_ms"], r["ms"], margin)
            if key is not None:
                tile, s = key
                if tile < 0:
                    tile = {(256, 256): 0, (128, 128): 2}.get((r["rules_xpose"]["block_m"], r["rules_xpose"]["block_n"]), 2)
                out.append((TUNED_SPLITK, r["m_lo"], r["m_hi"], r["N"], r["K"], tile, s, 0))  # R = N, Cc = K (dW stored [N, K])
    # one entry per key (the operation is part of it: a linear layer and an FFN's down projection of the
    # same extents are different kernels and keep their own plans)
    seen, uniq = set(), []
    for e in sorted(out):
        if e[:5] not in seen:
            seen.add(e[:5])
            uniq.append(e)
    return uniq


def render_header(plans) -> str:
    lines = ["// Measured plans of the gfx950 tile table.  GENERATED by `python -m ffn_kernel_amd.tune --emit`: do not edit.",
             "// {op, m_lo, m_hi, k, n, tile, splits, group_m}; see TunedPlan in tile_table.hpp.",
             "#pragma once", "namespace ffnk {", "constexpr TunedPlan kTunedPlans[] = {"]
    for e in plans:
        lines.append("    {%d, %d, %d, %d, %d, %d, %d, %d}," % e)
    lines += ["    {-1, 0, 0, 0, 0, 0, 0, 0},", "};", "}  // namespace ffnk", ""]
    return "\n".join(lines)


def read_header(path) -> list:
    """The entries of a generated header (the terminator excluded), as render_header wrote them."""
    import re
    out = []
    for m in re.finditer(r"^\s*\{(-?\d+(?:,\s*-?\d+){7})\},", Path(path).read_text(), re.M):
        e = tuple(int(v) for v in m.group(1).split(","))
        if e[0] >= 0:
            out.append(e)
    return out


OPS = ("ffn_fwd", "linear_fwd", "linear_bwd")
OP_KINDS = {"ffn_fwd": (TUNED_DUAL, TUNED_DOWN), "linear_fwd": (TUNED_PLAIN,), "linear_bwd": (TUNED_SPLITK,)}


def _fmt_list(ts):
    return "/".join(f"{t:.3f}" for t in ts)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m ffn_kernel_amd.tune")
    ap.add_argument("--trials", type=int, default=5, help="timed calls per candidate; the minimum counts")
    ap.add_argument("--margin", type=float, default=0.04, help="a candidate must beat the rules by this fraction")
    ap.add_argument("--emit", action="store_true", help=f"rewrite {GEN_PATH.name}")
    ap.add_argument("--out", type=Path, default=GEN_PATH, help="where --emit writes")
    ap.add_argument("--json", default=None, help="dump every measurement")
    ap.add_argument("--quick", action="store_true", help="two buckets per layer")
    ap.add_argument("--ffn", action="append", default=None, metavar="D,H",
                    help="MaskedFFN layer to measure besides the default ones (repeatable)")
    ap.add_argument("--linear", action="append", default=None, metavar="K,N",
                    help="MaskedLinear layer to measure besides the default ones (repeatable)")
    ap.add_argument("--passes", type=int, default=1,
                    help="independent sweeps; only a plan that every one of them selects enters the table (timing "
                         "noise makes plans near the margin come and go between sweeps)")
    ap.add_argument("--ops", default=",".join(OPS), help="operations to measure (comma separated); --emit keeps the "
                    f"plans that {GEN_PATH.name} holds for the others")
    args = ap.parse_args(argv)
    ops = [o for o in args.ops.split(",") if o]
    if not ops or any(o not in OPS for o in ops):
        ap.error(f"--ops takes a comma separated subset of {', '.join(OPS)}")

    def pairs(specs, default):
        out = list(default)
        for spec in specs or []:
            try:
                a, b = (int(v) for v in spec.split(","))
            except ValueError:
                ap.error(f"expected two integers separated by a comma, got {spec}")
            if a <= 0 or b <= 0 or a % 8 or b % 8:
                ap.error(f"layer extents must be positive multiples of 8, got {spec}")
            if (a, b) not in out:
                out.append((a, b))
        return out

    ffn_layers = pairs(args.ffn, FFN_LAYERS)
    linear_layers = pairs(args.linear, LINEAR_LAYERS)
    if not torch.cuda.is_available():
        print("ffn_kernel_amd.tune needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ev = _Events()
    buckets = [BUCKETS[1], BUCKETS[4]] if args.quick else BUCKETS

    def ratios(base, cand):
        return "  ".join(f"{k}:" + "/".join(f"{t / b_:.2f}" for t, b_ in zip(ts, base)) for k, ts in cand.items()) or "-"

    def gm_text(r):
        """Second stage of a record: per stage, the pinned plan (tile, splits), the tile's own super-group size, and
        group_m:time / the plan's time with its own size, per scenario."""
        gm = r.get("group_m") or {}
        parts = []
        for stage, plan, ms in (("up ", "up_plan", "up_ms"), ("down ", "down_plan", "down_ms"), ("", "plan", "ms")):
            if plan not in gm or not gm[ms]:
                continue
            own = r["rules"][stage.strip()]["group_m"] if stage else r["rules"]["group_m"]
            others = {g: ts for g, ts in gm[ms].items() if g != own}
            parts.append(f"{stage}group_m on {tuple(gm[plan])} (own {own}): {ratios(gm[ms][own], others)}")
        return (" | " + " ; ".join(parts)) if parts else ""

    per_pass = []
    for pass_no in range(max(1, args.passes)):
        if args.passes > 1:
            print(f"== sweep {pass_no + 1} of {args.passes} ==", flush=True)
        records = []
        for d, h in (ffn_layers if "ffn_fwd" in ops else []):
            for b in buckets:
                if b[1] * h * 2 > 4 << 30:
                    continue
                r = tune_ffn(d, h, b, args.trials, dev, ev, args.margin)
                records.append(r)
                up = r["rules"]["up"]
                print(f"ffn_fwd    d={d:5d} h={h:5d} M<={b[1]:6d} | rules up {_fmt_list(r['rules_up_ms'])} "
                      f"(tile {up['block_m']}x{up['block_n']}/{up['waves_m'] * up['waves_n']}w) down {_fmt_list(r['rules_down_ms'])}"
                      f" | up tile:ratio per scenario {ratios(r['rules_up_ms'], r['up_ms'])}"
                      f" | down (tile, splits):ratio {ratios(r['rules_down_ms'], r['down_ms'])}" + gm_text(r), flush=True)
        for K, N in linear_layers:
            for b in buckets:
                if "linear_fwd" in ops:
                    r = tune_linear_fwd(K, N, b, args.trials, dev, args.margin)
                    records.append(r)
                    print(f"linear_fwd K={K:5d} N={N:5d} M<={b[1]:6d} | rules {_fmt_list(r['rules_ms'])} | (tile, splits):ratio "
                          f"{ratios(r['rules_ms'], r['ms'])}" + gm_text(r), flush=True)
                if "linear_bwd" in ops:
                    r = tune_linear_bwd(K, N, b, args.trials, dev, args.margin)
                    records.append(r)
                    print(f"linear_bwd K={K:5d} N={N:5d} M<={b[1]:6d} | rules {_fmt_list(r['rules_ms'])} (splits {r['rules']['split_k']}"
                          f"{', in place' if r['rules']['in_place'] else ''}) | (tile, splits):ratio {ratios(r['rules_ms'], r['ms'])}",
                          flush=True)
        per_pass.append(plans_from(records, args.margin))
    plans = [e for e in per_pass[0] if all(e in other for other in per_pass[1:])]
    if args.passes > 1:
        print(f"plans per sweep: {[len(p_) for p_ in per_pass]}; selected by every sweep: {len(plans)}")
    if len(ops) < len(OPS):
        measured = {k for o in ops for k in OP_KINDS[o]}
        kept = [e for e in read_header(GEN_PATH) if e[0] not in measured]
        print(f"{len(kept)} plans of the operations not measured in this run are kept from {GEN_PATH.name}")
        plans = sorted(plans + kept)
    print(f"{len(plans)} measured plans lose on no scenario and beat the rules by more than {args.margin:.0%}:")
    for e in plans:
        print("   op=%d M in [%d, %d] k=%d n=%d -> tile %d, splits %d, group_m %d" % e)
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
