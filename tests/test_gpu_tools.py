"""The user-facing tools on the GPU: the check CLI (the non-interactive counterpart of the reference's
test_linear.py / test_ffn.py --check flows) and the tuner that produces the measured tile table."""
import json
import re

import pytest
import torch

from ffn_kernel_amd import _lib, check, tune

from helpers import note

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("argv", [
    ["linear", "--check", "--max-mult", "2"],
    ["linear", "--check", "--bsz", "2", "--max-mult", "1", "--d", "512"],
    ["ffn", "--check", "--max-mult", "2"],
    ["ffn", "--check", "--bwd", "--max-mult", "1", "--d", "512", "--h", "1024"],
])
def test_check_cli_passes(dev, argv, capsys):
    note(f"check CLI {' '.join(argv)}")
    assert check.main(argv) == 0
    lines = [json.loads(l) for l in capsys.readouterr().out.splitlines() if l.startswith("{")]
    assert lines and all(l["ok"] for l in lines)
    assert all(k.startswith("rel_l2") and v <= 2e-2 for l in lines for k, v in l.items() if k.startswith("rel_l2"))


def test_check_cli_times_both_modules(dev, capsys):
    note("check CLI timing mode")
    assert check.main(["ffn", "--max-mult", "1"]) == 0
    rec = json.loads([l for l in capsys.readouterr().out.splitlines() if l.startswith("{")][-1])
    assert rec["pytorch_ms"] > 0 and rec["hip_ms"] > 0


def test_tuner_emits_a_table_the_library_can_compile(dev, tmp_path, capsys):
    """A short sweep (two M buckets per layer) through every candidate, forced via the C ABI; the
    emitted header has the generated file's format, and the overrides are back to the table after it."""
    note("tuner --quick --emit")
    out = tmp_path / "tile_table_gen.hpp"
    assert tune.main(["--quick", "--trials", "2", "--emit", "--out", str(out), "--json", str(tmp_path / "t.json")]) == 0
    text = out.read_text()
    entries = re.findall(r"^\s*\{(-?\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+)\},$", text, re.M)
    assert entries and entries[-1][0] == "-1"
    for op, lo, hi, k, n, tile, splits, group_m in entries[:-1]:
        assert int(group_m) in (0, 2, 4, 8, 16)
        # tile 5 is a form of the weight-gradient GEMM (operands read in place), not a tile of the routed GEMMs
        assert int(op) in (0, 1, 2, 3) and int(lo) <= int(hi) and 0 <= int(tile) <= (5 if int(op) == 2 else 4) and 1 <= int(splits) <= 16
    recs = json.loads((tmp_path / "t.json").read_text())
    assert {r["op"] for r in recs} == {"ffn_fwd", "linear_fwd", "linear_bwd"}
    lib = _lib.load()
    assert lib.ffnk_debug_force_tile(-1) == -1 and lib.ffnk_debug_force_splits(-1) == -1 and lib.ffnk_debug_force_bwd_gather(-1) == -1
    assert lib.ffnk_debug_force_group_m(0) == 0


def test_forced_splits_results_match(dev):
    """A forced split-K factor changes the summation order only: results stay within bf16 of the unsplit ones."""
    note("forced splits: linear fwd M=300 K=2048 N=512")
    from ffn_kernel_amd import MaskedLinear
    from ffn_kernel_amd import workloads as wl
    from oracle import cref
    from helpers import assert_close
    M, K, N = 300, 2048, 512
    mask = torch.rand(M, generator=torch.Generator().manual_seed(3)) < 0.5
    w = wl.make_linear("t", M, K, N, mask, seed=5, w_std=0.05)
    dw = w.to(dev)
    ref = cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask)
    lib = _lib.load()
    try:
        for s in (1, 2, 4):
            lib.ffnk_debug_force_splits(s)
            assert _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)["split_k"] == s
            assert_close(MaskedLinear.apply(dw.x, dw.Wv.T, dw.Wt.T, dw.mask), ref, f"splits {s}")
    finally:
        lib.ffnk_debug_force_splits(-1)


_BENCH = str(__import__("pathlib").Path(__file__).resolve().parents[1] / "bench.py")


@pytest.mark.parametrize("workload", ["cfg2", "cfg3", "decode8"])
def test_bench_prints_one_json_line_with_roofline_and_cpu_baseline(dev, workload):
    """bench.py's contract on a short run: one JSON object, the headline fields, a roofline for the
    dominant kernel and the CPU baseline of the same workload."""
    import subprocess
    import sys
    note(f"bench.py --workload {workload}")
    proc = subprocess.run([sys.executable, _BENCH, "--workload", workload, "--steps", "3", "--warmup", "1", "--cpu-rows", "64"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 3 and rec["warmup"] == 1 and rec["dtype"] == "bf16"
    assert rec["value"] > 0 and rec["ms_per_step"] > 0 and "workload" in rec["config"]
    roof = rec["roofline"]
    assert roof["bound"] in ("mfma", "hbm") and roof["unit"] in ("TFLOP/s", "GB/s")
    assert 0 < roof["frac"] < 1 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9
    assert roof["traffic"] is None or roof["traffic"] > 0
    cpu = rec["cpu_baseline"]
    assert cpu["value"] > 0 and cpu["cores"] >= 1 and cpu["kind"] == "port" and cpu["sample"]
