"""Headline benchmark: MaskedFFN forward, routed bf16 TFLOP/s at d=4096, h=14336, M=32768 on one
MI355X (BASELINE.json's metric, `configs[3]`).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4|cfg2|decode1v|decode1t|decode8|decode32|decode64|prefill1024]

A step is one MaskedFFN.apply over the whole synthetic batch (row partition + up-projection with
SwiGLU + down-projection), inputs already resident in HBM.  Prints ONE JSON line.
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

# HBM bytes per launch of the roofline kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# file (KiB per dispatch, scaled by what the same counters read for the 1 GiB copy of --workload copy1g:
# FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  The counter runs and the arithmetic are kept as text under
# profiles/ (routed_gemm_kernel_ffn_fwd_M32768_d4096_h14336.txt, stream_*_kernel_ffn_decode_*.txt).
# Recorded, not measured live: counters cannot be read from inside the process.
MEASURED_TRAFFIC_BYTES = {
    # up-projection: the whole-round launch plus the remainder launch (FETCH_SIZE * 2.0 + WRITE_SIZE each)
    "cfg4": (5.4863e6 * 2.0 + 9.1223e5 + 2.3258e5 * 2.0 + 5388.9) * 1024,
    # decode: all launches of one call (up-projection, down-projection, reduce where there is one)
    "decode1v": (1.1476e5 * 2.0 + 40 + 5.7481e4 * 2.0 + 8) * 1024,
    "decode8": (2.2979e5 * 2.0 + 320 + 1.1568e5 * 2.0 + 64) * 1024,
    "decode32": (2.3053e5 * 2.0 + 897 + 1.184e5 * 2.0 + 2048 + 1039 * 2.0 + 256) * 1024,
    "decode64": (2.3159e5 * 2.0 + 1792 + 1.2203e5 * 2.0 + 4096 + 2063 * 2.0 + 512) * 1024,
}


class HipEvents:
    """hipEvent_t handles created through the HIP runtime torch already loaded, so that stage
    boundaries inside one C-ABI call can be timed on the stream the kernels run on."""

    def __init__(self, n: int):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.ev = (ctypes.c_void_p * n)()
        for i in range(n):
            h = ctypes.c_void_p()
            rc = self.hip.hipEventCreate(ctypes.byref(h))
            if rc != 0:
                raise RuntimeError(f"hipEventCreate failed: {rc}")
            self.ev[i] = h

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


def _cpu_baseline(w, rows: int) -> dict:
    """The reference's PyTorch module maths (both branches, blended by mask, bf16) on the host CPU,
    on the first `rows` rows of the same workload."""
    import torch
    from oracle import modules as om
    torch.set_num_threads(os.cpu_count() or 1)
    W = {k: v.cpu() for k, v in w.W.items()}
    with torch.no_grad():
        probe = min(256, rows)
        om.ffn_blend(w.x[:probe].cpu(), W, w.mask[:probe].cpu())  # warm-up
        t0 = time.perf_counter()
        om.ffn_blend(w.x[:probe].cpu(), W, w.mask[:probe].cpu())
        per_row = (time.perf_counter() - t0) / probe
        # about 5 s per timed run, three runs
        rows = max(probe, min(rows, int(5.0 / max(per_row, 1e-9))))
        x = w.x[:rows].cpu()
        mask = w.mask[:rows].cpu()
        times = []
        for _ in range(3):
            t0 = time.perf_counter()
            om.ffn_blend(x, W, mask)
            times.append(time.perf_counter() - t0)
            if sum(times) > 25:
                break
    t = sorted(times)[len(times) // 2]
    routed = 2 * rows * w.d * w.h * 3
    return {"value": routed / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {rows} rows of the workload, blend-form bf16 torch CPU (executes 2x the routed "
                      f"FLOPs), median of {len(times)} runs, {t * 1e3:.1f} ms"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="cfg4")
    ap.add_argument("--cpu-rows", type=int, default=1 << 30,
                    help="upper bound on the rows of the workload timed on the CPU (0 = skip); the sample is "
                         "sized to about 5 s per run")
    args = ap.parse_args()
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
    weight_sets = [w.W]
    if decode:
        for r in (1, 2):
            g = torch.Generator().manual_seed(9000 + r)
            weight_sets.append({k: (torch.randn(v.shape, generator=g) * 0.02).to(torch.bfloat16).to(dev)
                                for k, v in w_cpu.W.items()})
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

    traffic = MEASURED_TRAFFIC_BYTES.get(args.workload)
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
                   "visual_rows": int(w_cpu.mask.sum()), "tile": tile},
        "roofline": roofline,
    }
    if args.cpu_rows > 0:
        result["cpu_baseline"] = _cpu_baseline(w_cpu, min(args.cpu_rows, M))
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
