"""Headline benchmark: MaskedFFN forward, routed bf16 TFLOP/s at d=4096, h=14336, M=32768 on one
MI355X (BASELINE.json's metric, `configs[3]`).

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload cfg4|cfg2|cfg1|cfg3|decode1v|decode1t|decode8|decode32|decode64|decode64v|prefillN]
                    [--no-route-cache]
                    [--workload gemm_ref|gemm_ref_down|copy1g]   (reference points, not this library: the vendor
                     library's plain GEMM on the up / down projection's shape; the 1 GiB copy that calibrates counters)

A step is one pass of the hot path over the whole synthetic batch, inputs already resident in HBM:
  cfg4 / cfg2 / decodeN / prefillN : one MaskedFFN.apply (row partition + up-projection with SwiGLU +
                                     down-projection);
  cfg1                             : one MaskedLinear.apply (forward);
  cfg3                             : one MaskedLinear backward (dx, dW_v, dW_t from the upstream gradient).
Prints ONE JSON line.  The default run (cfg4) also times the decode shapes of BASELINE.json's
`configs[4]` and reports them as `roofline_decode` in the same line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM bytes per launch of each workload's roofline kernel(s), from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# runs of this file, scaled by what the same counters read for the 1 GiB copy of --workload copy1g.
# Counters cannot be read from inside the process: the figures are written by
# `python -m ffn_kernel_amd.profile_summary` next to the profile summaries and only read here.
TRAFFIC_FILE = ROOT / "profiles" / "traffic.json"


def measured_traffic(workload: str):
    try:
        entry = json.loads(TRAFFIC_FILE.read_text()).get(workload)
    except (OSError, ValueError):
        return None
    return None if entry is None else entry.get("bytes")


class HipEvents:
    """hipEvent_t handles created through the HIP runtime torch already loaded, so that stage
    boundaries inside one C-ABI call can be timed on the stream the kernels run on."""

    def __init__(self, n: int):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.ev = (ctypes.c_void_p * n)()
        for i in range(n):
            h = ctypes.c_void_p()
            rc = self.hip.hipEventCreate(ctypes.byref(h))
            if rc != 0:
                raise RuntimeError(f"hipEventCreate failed: {rc}")
            self.ev[i] = h

    def record(self, i: int, stream: int) -> None:
        rc = self.hip.hipEventRecord(self.ev[i], ctypes.c_void_p(stream))
        if rc != 0:
            raise RuntimeError(f"hipEventRecord failed: {rc}")

    def elapsed_ms(self, i: int, j: int) -> float:
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), self.ev[i], self.ev[j])
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return ms.value

    def close(self):
        for h in self.ev:
            self.hip.hipEventDestroy(h)


def _ffn_call_with_events(w, events, W=None):
    """One ffnk_masked_ffn_fwd_ev call (same path as MaskedFFN.apply) recording stage events."""
    import torch
    from ffn_kernel_amd import _lib
    lib = _lib.load()
    x = w.x
    M, d = x.shape
    h = w.h
    W = W or w.W
    out = torch.empty((M, d), device=x.device, dtype=torch.bfloat16)
    ws = torch.empty(_lib.workspace_bytes(_lib.OP_FFN_FWD, M, d, h), dtype=torch.uint8, device=x.device)
    rc = lib.ffnk_masked_ffn_fwd_ev(x.data_ptr(), x.stride(0), W["w1"].data_ptr(), W["w3"].data_ptr(),
                                    W["u1"].data_ptr(), W["u3"].data_ptr(), 1, d, W["w2"].data_ptr(),
                                    W["u2"].data_ptr(), 1, h, w.mask.data_ptr(), out.data_ptr(), d, M, d, h,
                                    ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream,
                                    ctypes.cast(events.ev, ctypes.c_void_p))
    _lib.check(rc, "ffnk_masked_ffn_fwd_ev")
    return out


def _time_cpu(fn, rows_cap):
    """Median of up to three runs of fn(rows), with rows sized to about 5 s per run."""
    probe = min(256, rows_cap)
    fn(probe)  # warm-up
    t0 = time.perf_counter()
    fn(probe)
    per_row = (time.perf_counter() - t0) / probe
    rows = max(probe, min(rows_cap, int(5.0 / max(per_row, 1e-9))))
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        fn(rows)
        times.append(time.perf_counter() - t0)
        if sum(times) > 25:
            break
    return rows, sorted(times)[len(times) // 2], len(times)


def _cpu_baseline_ffn(w, rows: int) -> dict:
    """The reference's PyTorch module maths (both branches, blended by mask, bf16) on the host CPU,
    on the first rows of the same workload."""
    import torch
    from oracle import modules as om
    torch.set_num_threads(os.cpu_count() or 1)
    W = {k: v.cpu() for k, v in w.W.items()}
    x, mask = w.x.cpu(), w.mask.cpu()
    with torch.no_grad():
        rows, t, n = _time_cpu(lambda r: om.ffn_blend(x[:r], W, mask[:r]), rows)
    routed = 2 * rows * w.d * w.h * 3
    return {"value": routed / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {rows} rows of the workload, blend-form bf16 torch CPU (executes 2x the routed "
                      f"FLOPs), median of {n} runs, {t * 1e3:.1f} ms"}


def _cpu_baseline_linear(w, rows: int, backward: bool) -> dict:
    """The reference's TorchLinear module maths (blend form, bf16; backward through autograd as its test
    takes it) on the host CPU, on the first rows of the same workload."""
    import torch
    from oracle import modules as om
    torch.set_num_threads(os.cpu_count() or 1)
    x, Wv, Wt, mask = w.x.cpu(), w.Wv.cpu(), w.Wt.cpu(), w.mask.cpu()
    g = None if w.grad is None else w.grad.cpu()
    if backward:
        fn = lambda r: om.linear_backward_autograd(g[:r], x[:r], Wv, Wt, mask[:r], dtype=torch.bfloat16)
    else:
        fn = lambda r: om.linear_blend(x[:r], Wv, Wt, mask[:r])
    with torch.set_grad_enabled(backward):
        rows, t, n = _time_cpu(fn, rows)
    K, N = x.shape[1], Wv.shape[0]
    routed = (4 if backward else 2) * rows * K * N
    what = "forward + autograd backward of the blend-form bf16 module" if backward else "blend-form bf16 module forward"
    return {"value": routed / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {rows} rows of the workload, {what} on torch CPU, median of {n} runs, {t * 1e3:.2f} ms"}


def _decode_rooflines(dev, weight_sets, steps: int) -> list:
    """BASELINE.json configs[4]: MaskedFFN at d=4096, h=14336 for M in {1, 8, 32, 64} (Bernoulli mask;
    M=1 visual-only and text-only), one call = algorithmic bytes over the call's duration, against
    8 TB/s.  Three weight sets larger than the Infinity Cache rotate, so the weights come from HBM."""
    import torch
    from ffn_kernel_amd import MaskedFFN
    from ffn_kernel_amd import workloads as wl
    out = []
    ns = len(weight_sets)
    for M, kind in ((1, "visual"), (1, "text"), (8, "bernoulli"), (32, "bernoulli"), (64, "bernoulli"), (64, "visual")):
        x, mask = wl.cfg5_inputs(M, kind)
        x, mask = x.to(dev), mask.to(dev)
        calls = [wl.FFNWorkload("d", x, W, mask).op_args() for W in weight_sets]
        for i in range(20):
            MaskedFFN.apply(*calls[i % ns])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            MaskedFFN.apply(*calls[i % ns])
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) * 1e6 / steps
        nbytes = wl.FFNWorkload("d", x, weight_sets[0], mask).algorithmic_bytes()
        gbs = nbytes / (us * 1e-6) / 1e9
        out.append({"M": M, "mask": kind, "algorithmic_bytes": nbytes, "us": us, "achieved_GBs": gbs,
                    "frac": gbs / PEAK_HBM_GBS})
    return out


def _bench_linear(args, dev) -> dict:
    """cfg1 (MaskedLinear forward) / cfg3 (MaskedLinear backward)."""
    import torch
    from ffn_kernel_amd import MaskedLinear, _lib
    from ffn_kernel_amd import workloads as wl
    from ffn_kernel_amd.ops import masked_linear_backward
    backward = args.workload == "cfg3"
    w_cpu = wl.cfg3_linear_bwd() if backward else wl.cfg1_linear_fwd()
    w = w_cpu.to(dev)
    M, K = w.x.shape
    N = w.Wv.shape[0]
    if backward:
        step = lambda: masked_linear_backward(w.grad, w.x, w.Wv.T, w.Wt.T, w.mask)
        flops = w_cpu.routed_flops_bwd
        metric = "MaskedLinear bwd routed bf16 TFLOP/s"
        kernels = "all launches of one backward call (row partition unless shared, fused dx | dW GEMM on g and x in place, reduce of the split partials)"
        tile = {"dx": _lib.tile_config(_lib.OP_BWD_DX, M, K, N), "dw": _lib.tile_config(_lib.OP_BWD_DW, M, K, N)}
    else:
        step = lambda: MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, w.mask)
        flops = w_cpu.routed_flops_fwd
        metric = "MaskedLinear fwd routed bf16 TFLOP/s"
        kernels = "all launches of one forward call (row partition, routed GEMM)"
        tile = _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    # Device time of one call: HIP events on the launch stream around single calls (the loop above is
    # bound by the host's launch rate at these sizes).
    ev = HipEvents(2)
    stream = torch.cuda.current_stream().cuda_stream
    dev_ms = []
    for _ in range(max(args.steps, 5)):
        ev.record(0, stream)
        step()
        ev.record(1, stream)
        torch.cuda.synchronize()
        dev_ms.append(ev.elapsed_ms(0, 1))
    ev.close()
    dev_avg = sum(dev_ms) / len(dev_ms)
    achieved = flops / (dev_avg * 1e-3) / 1e12
    value = flops / (ms_per_step * 1e-3) / 1e12
    result = {
        "metric": metric, "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic", "pct_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS,
        "config": {"workload": w_cpu.name, "M": M, "K": K, "N": N, "visual_rows": int(w_cpu.mask.sum()), "tile": tile,
                   "row_partition": "per call" if args.no_route_cache else "shared between calls with the same mask"},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": measured_traffic(args.workload),
                     "kernel": kernels, "kernel_ms": dev_avg, "kernel_ms_min": min(dev_ms), "algorithmic_flops": flops},
    }
    if args.cpu_rows > 0:
        result["cpu_baseline"] = _cpu_baseline_linear(w_cpu, min(args.cpu_rows, M), backward)
    return result


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default: 20 for cfg4, 200 for the microsecond-scale workloads, whose "
                         "first launches after a synchronisation would otherwise dominate)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps first (default: 5, or 20 with 200 steps)")
    ap.add_argument("--workload", default="cfg4")
    ap.add_argument("--cpu-rows", type=int, default=1 << 30,
                    help="upper bound on the rows of the workload timed on the CPU (0 = skip); the sample is "
                         "sized to about 5 s per run")
    ap.add_argument("--no-route-cache", action="store_true",
                    help="partition the rows anew in every call instead of sharing one partition between calls "
                         "that run with the same mask (ffn_kernel_amd.set_route_cache); a model's layers all "
                         "route by one mask, so the default measures a call as a layer sees it")
    ap.add_argument("--no-decode", action="store_true",
                    help="cfg4 only: skip the decode-shape measurements (roofline_decode), e.g. under a profiler")
    args = ap.parse_args()
    big = args.workload in ("cfg4", "gemm_ref", "gemm_ref_down", "copy1g")
    if args.steps is None:
        args.steps = 20 if big else 200
    if args.warmup is None:
        args.warmup = 5 if big else 20
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (rows are independent, so more GPUs "
              "would each run this same kernel on their slice of M)", file=sys.stderr)
        return 2

    import torch
    from ffn_kernel_amd import MaskedFFN, _lib
    from ffn_kernel_amd import workloads as wl

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.no_route_cache:
        from ffn_kernel_amd import set_route_cache
        set_route_cache(False)
    if args.workload == "copy1g":
        # Calibration for the FETCH_SIZE / WRITE_SIZE counters: a plain device copy of exactly 1 GiB
        # (reads 1 GiB, writes 1 GiB per launch).  Not a benchmark of this library.
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(args.warmup + args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"workload": "copy1g", "bytes_read": 1 << 30, "bytes_written": 1 << 30}))
        return 0
    if args.workload in ("gemm_ref", "gemm_ref_down"):
        # Reference points for the two GEMM launches of cfg4: the vendor library's plain bf16 GEMM
        # (torch's F.linear) on the shape the up-projection + SwiGLU launch computes,
        # [32768, 4096] x [28672, 4096]^T (gemm_ref), and on the down projection's,
        # [32768, 14336] x [4096, 14336]^T (gemm_ref_down).  Not a benchmark of this library; run under
        # rocprofv3 to read the vendor kernel's launch geometry and counters beside routed_gemm_kernel's.
        gm, gn, gk = (32768, 28672, 4096) if args.workload == "gemm_ref" else (32768, 4096, 14336)
        g = torch.Generator().manual_seed(0)
        a = torch.randn(gm, gk, generator=g).to(torch.bfloat16).to(dev)
        b = (torch.randn(gn, gk, generator=g) * 0.02).to(torch.bfloat16).to(dev)
        for _ in range(args.warmup):
            torch.nn.functional.linear(a, b)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            torch.nn.functional.linear(a, b)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        print(json.dumps({"workload": args.workload, "M": gm, "N": gn, "K": gk, "ms_per_step": ms,
                          "tflops": 2 * gm * gn * gk / (ms * 1e-3) / 1e12}))
        return 0
    if args.workload in ("cfg1", "cfg3"):
        print(json.dumps(_bench_linear(args, dev)), flush=True)
        return 0
    if args.workload == "cfg4":
        w_cpu = wl.cfg4_ffn_fwd()
    elif args.workload == "cfg2":
        w_cpu = wl.cfg2_ffn_fwd()
    elif args.workload.startswith("decode"):
        spec = args.workload[6:] or "64"
        kind = {"v": "visual", "t": "text"}.get(spec[-1], "bernoulli")
        w_cpu = wl.cfg5_ffn_decode(int(spec.rstrip("vt")), kind)
    elif args.workload.startswith("prefill"):
        # mid-size batches at the cfg4/cfg5 layer shape (Bernoulli mask): few output tiles, split-K down projection
        w_cpu = wl.cfg5_ffn_decode(int(args.workload[7:] or "1024"), "bernoulli")
    else:
        raise SystemExit(f"unknown workload {args.workload}")
    w = w_cpu.to(dev)
    M = w.x.shape[0]
    tile = _lib.tile_config(_lib.OP_FFN_UP, M, w.d, w.h)
    decode = tile["path"] == _lib.PATH_STREAM

    # Decode calls are bound by streaming the weights: rotate three distinct weight sets (each larger
    # than the 256 MB Infinity Cache) so that what is measured is HBM, not cache.
    def more_weight_sets(first):
        sets = [first]
        for r in (1, 2):
            g = torch.Generator(device=dev).manual_seed(9000 + r)
            sets.append({k: (torch.randn(v.shape, generator=g, device=dev) * 0.02).to(torch.bfloat16)
                         for k, v in first.items()})
        return sets

    weight_sets = more_weight_sets(w.W) if decode else [w.W]
    arg_sets = [wl.FFNWorkload(w.name, w.x, W, w.mask).op_args() for W in weight_sets]
    ns = len(arg_sets)

    for i in range(args.warmup):
        MaskedFFN.apply(*arg_sets[i % ns])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        MaskedFFN.apply(*arg_sets[i % ns])
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # Stage durations from HIP events recorded on the launch stream inside the same C-ABI call.
    ev = HipEvents(3)
    up_ms, down_ms = [], []
    for i in range(max(args.steps, 3)):
        _ffn_call_with_events(w, ev, weight_sets[i % ns])
        torch.cuda.synchronize()
        up_ms.append(ev.elapsed_ms(0, 1))
        down_ms.append(ev.elapsed_ms(1, 2))
    ev.close()
    up_avg = sum(up_ms) / len(up_ms)
    down_avg = sum(down_ms) / len(down_ms)

    traffic = measured_traffic(args.workload)
    if decode:
        # Weight-streaming regime: a call is two stream_kernel launches (up-projection + SwiGLU, then
        # the down-projection) of 25-100 us each, back to back.  At that size an event recorded between
        # them adds a gap of its own to both halves, so the roofline entry is the pair: the call's
        # algorithmic bytes over the call's duration in the timed loop.  The event split is reported
        # beside it for orientation only.
        call_bytes = w_cpu.algorithmic_bytes()
        achieved = call_bytes / (ms_per_step * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": achieved / PEAK_HBM_GBS, "traffic": traffic,
                    "kernel": "decode stream kernels of one call (up-projection + SwiGLU, down-projection)",
                    "kernel_ms": ms_per_step, "algorithmic_bytes": call_bytes,
                    "up_ms_with_event_gap": up_avg, "down_ms_with_event_gap": down_avg}
    else:
        up_flops = 2 * M * w.d * w.h * 2  # gate and up projections of the routed branch
        achieved = up_flops / (up_avg * 1e-3) / 1e12
        roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": achieved / PEAK_BF16_TFLOPS, "traffic": traffic,
                    "kernel": "routed_gemm_kernel (up-projection + SwiGLU: whole-round launch + remainder launch)",
                    "kernel_ms": up_avg,
                    "down_kernel_ms": down_avg,
                    "down_achieved": 2 * M * w.d * w.h / (down_avg * 1e-3) / 1e12}

    value = w_cpu.routed_flops / (ms_per_step * 1e-3) / 1e12
    result = {
        "metric": "MaskedFFN fwd routed bf16 TFLOP/s",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "pct_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS,
        "config": {"workload": w_cpu.name, "M": M, "d": w.d, "h": w.h,
                   "visual_rows": int(w_cpu.mask.sum()), "tile": tile,
                   "row_partition": "per call" if (args.no_route_cache or decode) else "shared between calls with the same mask"},
        "roofline": roofline,
    }
    if args.workload == "cfg4" and not args.no_decode:
        # The same layer at decode sizes (HBM-bound): the cfg4 weights plus two more sets rotate.
        result["roofline_decode"] = _decode_rooflines(dev, more_weight_sets(w.W), steps=max(args.steps, 200))
    if args.cpu_rows > 0:
        result["cpu_baseline"] = _cpu_baseline_ffn(w_cpu, min(args.cpu_rows, M))
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
