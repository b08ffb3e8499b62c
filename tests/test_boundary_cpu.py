"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the header
declares, size/introspection entry points answer, argument validation raises, and the workload
generators are deterministic."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

from ffn_kernel_amd import MaskedFFN, MaskedLinear, _lib
from ffn_kernel_amd import workloads as wl

ROOT = Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "ffnk.h").read_text()
    declared = set(re.findall(r"FFNK_API\s+[\w\s\*]+?\b(ffnk_\w+)\s*\(", header))
    assert declared == set(_lib.EXPORTED_SYMBOLS), declared ^ set(_lib.EXPORTED_SYMBOLS)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name)
    assert lib.ffnk_version() == int(re.search(r"#define FFNK_VERSION (\d+)", header).group(1))


def test_workspace_bytes():
    assert _lib.workspace_bytes(_lib.OP_LINEAR_FWD, 0, 8, 8) >= 0
    a = _lib.workspace_bytes(_lib.OP_LINEAR_FWD, 2048, 1024, 1024)
    assert a >= 2048 * 4 + 8
    f = _lib.workspace_bytes(_lib.OP_FFN_FWD, 32768, 4096, 14336)
    assert f >= 32768 * 14336 * 2  # the bf16 intermediate
    b = _lib.workspace_bytes(_lib.OP_LINEAR_BWD, 8192, 1024, 1024)
    assert b >= 2 * 8192 * 1024 * 2  # both transposed operands
    with pytest.raises(ValueError):
        _lib.workspace_bytes(99, 1, 1, 1)
    with pytest.raises(ValueError):
        _lib.workspace_bytes(_lib.OP_LINEAR_FWD, -1, 1, 1)


def test_tile_table_entries():
    big = _lib.tile_config(_lib.OP_FFN_UP, 32768, 4096, 14336)
    assert big["path"] == _lib.PATH_MFMA_TILED and big["block_m"] == 256 and big["direct_lds"] == 1
    assert big["block_k"] == 64 and big["lds_stages"] == 2  # two 64-element slabs, loaded global->LDS
    assert big["waves_m"] * big["waves_n"] == 4  # four waves of 128x128
    half = _lib.tile_config(_lib.OP_LINEAR_FWD, 2048, 96, 1024)
    assert half["direct_lds"] == 0  # the direct path moves whole 128-byte lines: K % 64 == 0
    # the four-wave 256x256 tile exists on the direct path only; a staged shape that would pick it runs eight waves
    long_k = _lib.tile_config(_lib.OP_LINEAR_FWD, 32768, 4096, 4096)
    assert long_k["direct_lds"] == 1 and long_k["block_m"] == 256 and long_k["waves_m"] * long_k["waves_n"] == 4
    # single-weight 256x256 tiles keep their token panel in a ring of three LDS stages (the weight panel in two)
    assert long_k["lds_stages"] == 3
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 32768, 4096, 14336)["lds_stages"] == 3
    staged = _lib.tile_config(_lib.OP_LINEAR_FWD, 32768, 4096 + 8, 4096)
    assert staged["direct_lds"] == 0 and staged["block_m"] == 256 and staged["waves_m"] * staged["waves_n"] == 8
    # M <= 8: dot-product streams, one wavefront per 1024-element K slice, no cross-workgroup split
    dec = _lib.tile_config(_lib.OP_FFN_FWD, 8, 4096, 14336)
    assert dec["path"] == _lib.PATH_STREAM and dec["lds_stages"] == 0 and dec["block_m"] == 8
    assert dec["block_k"] == 1024 and dec["split_k"] == 4
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 8, 4096, 14336)["split_k"] == 14
    # 9 <= M <= 64: LDS-transposed streams, 128-element chunks, three in flight, split-K down projection
    mid = _lib.tile_config(_lib.OP_FFN_UP, 64, 4096, 14336)
    assert mid["path"] == _lib.PATH_STREAM and mid["block_k"] == 128 and mid["lds_stages"] == 3
    assert mid["block_n"] == 32 and mid["split_k"] == 1 and mid["direct_lds"] == 1  # two wavefronts, direct slab loads
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 64, 4096, 14336)["split_k"] >= 4
    low = _lib.tile_config(_lib.OP_FFN_UP, 16, 4096, 14336)
    assert low["block_n"] == 32 and low["direct_lds"] == 0 and low["lds_stages"] == 4  # slab through registers
    # small M whose extents are not whole 512-element slices run on the LDS-transposed streams too ...
    odd = _lib.tile_config(_lib.OP_FFN_UP, 4, 1152, 1408)
    assert odd["path"] == _lib.PATH_STREAM and odd["lds_stages"] >= 3
    # ... and extents under 1024 on the fragment-layout streams
    tiny = _lib.tile_config(_lib.OP_FFN_UP, 4, 384, 640)
    assert tiny["path"] == _lib.PATH_STREAM and tiny["lds_stages"] == 0
    assert _lib.tile_config(_lib.OP_FFN_FWD, 65, 4096, 14336)["path"] == _lib.PATH_MFMA_TILED
    small = _lib.tile_config(_lib.OP_LINEAR_FWD, 2048, 1024, 1024)
    assert small["block_m"] * small["block_n"] < 256 * 256  # small problems get small tiles
    tail = _lib.tile_config(_lib.OP_LINEAR_FWD, 2048, 72, 1024)
    assert tail["direct_lds"] == 0 and tail["block_k"] == 64 and tail["lds_stages"] == 2
    # few output tiles over a long contraction: the down projection / the linear layer cut K ...
    for M in (65, 128, 512, 1024):
        dn = _lib.tile_config(_lib.OP_FFN_DOWN, M, 4096, 14336)
        assert dn["path"] == _lib.PATH_MFMA_TILED and dn["split_k"] > 1, (M, dn)
        assert (14336 // 64) // dn["split_k"] >= 8  # at least eight slabs per range
        # ... and the workspace holds perm/counts, the [M, h] intermediate and the fp32 partials
        need = M * 4 + 8 + M * 14336 * 2 + dn["split_k"] * M * 4096 * 4
        assert _lib.workspace_bytes(_lib.OP_FFN_FWD, M, 4096, 14336) >= need
    # just past one round of 256x256 tiles: unsplit, the last partial round runs as a split tail
    # whose 256 fp32 tiles the workspace holds
    one = _lib.tile_config(_lib.OP_FFN_DOWN, 4096, 4096, 14336)
    assert one["split_k"] == 1 and one["block_m"] == 256 and one["block_n"] == 256
    assert _lib.workspace_bytes(_lib.OP_FFN_FWD, 4096, 4096, 14336) >= 4096 * 4 + 8 + 4096 * 14336 * 2 + 256 * 256 * 256 * 4
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 32768, 4096, 14336)["split_k"] == 1
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 2048, 72, 264)["split_k"] == 1      # K % 64 != 0: no split
    lin = _lib.tile_config(_lib.OP_LINEAR_FWD, 200, 4096, 1024)
    assert lin["path"] == _lib.PATH_MFMA_TILED and lin["split_k"] > 1
    assert _lib.workspace_bytes(_lib.OP_LINEAR_FWD, 200, 4096, 1024) >= 200 * 4 + 8 + lin["split_k"] * 200 * 1024 * 4
    # decode-sized linear calls run on the streaming kernels
    assert _lib.tile_config(_lib.OP_LINEAR_FWD, 1, 4096, 4096)["path"] == _lib.PATH_STREAM
    assert _lib.tile_config(_lib.OP_LINEAR_FWD, 64, 4096, 4096)["path"] == _lib.PATH_STREAM
    assert _lib.tile_config(_lib.OP_LINEAR_FWD, 64, 4096, 4100)["path"] == _lib.PATH_MFMA_TILED  # ragged N
    # the factor reported is the one launched: by the rules alone, the fused dx / dW launch of the usual layout runs
    # cfg3's weight-gradient GEMM unsplit and on g and x where they lie, whatever the stand-alone GEMM's rule would
    # pick; a forced factor and a forced form are kept
    lib = _lib.load()
    try:
        lib.ffnk_debug_force_tile(-2)
        dw = _lib.tile_config(_lib.OP_BWD_DW, 8192, 1024, 1024)
        assert dw["split_k"] == 1 and dw["in_place"] == 1 and (dw["block_m"], dw["block_n"], dw["lds_stages"]) == (128, 128, 2)
        big = _lib.tile_config(_lib.OP_BWD_DW, 8192, 4096, 4096)      # compute-bound: routed transposes, 256x256 tiles
        assert big["in_place"] == 0 and big["block_m"] == 256
        assert _lib.tile_config(_lib.OP_BWD_DW, 512, 4096, 4096)["in_place"] == 1   # few rows: the transposes are a launch for nothing
        assert _lib.tile_config(_lib.OP_BWD_DW, 8192, 1028, 1024)["in_place"] == 0  # K % 8 != 0: rows are not 16-byte chunks
        lib.ffnk_debug_force_splits(4)
        assert _lib.tile_config(_lib.OP_BWD_DW, 8192, 1024, 1024)["split_k"] == 4
        lib.ffnk_debug_force_bwd_gather(0)
        assert _lib.tile_config(_lib.OP_BWD_DW, 8192, 1024, 1024)["in_place"] == 0
        lib.ffnk_debug_force_bwd_gather(1)
        assert _lib.tile_config(_lib.OP_BWD_DW, 8192, 4096, 4096)["in_place"] == 1
        # M-tiles per super-group of the tile order: the tile's own unless a plan or the hook says otherwise
        assert _lib.tile_config(_lib.OP_FFN_UP, 32768, 4096, 14336)["group_m"] == 8
        assert _lib.tile_config(_lib.OP_FFN_DOWN, 32768, 4096, 14336)["group_m"] == 4
        assert _lib.tile_config(_lib.OP_BWD_DX, 32768, 4096, 4096)["group_m"] == 8   # K-major weights
        assert lib.ffnk_debug_force_group_m(2) == 0
        assert _lib.tile_config(_lib.OP_FFN_UP, 32768, 4096, 14336)["group_m"] == 2
        assert _lib.tile_config(_lib.OP_LINEAR_FWD, 32768, 4096, 4096)["group_m"] == 2
        assert lib.ffnk_debug_force_group_m(1000) == 2 and lib.ffnk_debug_force_group_m(0) == 0   # out of range: back to the plans
    finally:
        lib.ffnk_debug_force_splits(-1)
        lib.ffnk_debug_force_tile(-1)
        lib.ffnk_debug_force_bwd_gather(-1)
        lib.ffnk_debug_force_group_m(0)
    with pytest.raises(ValueError):
        _lib.tile_config(77, 1, 1, 1)


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    lib = _lib.load()
    assert lib.ffnk_route(None, 10, None, None, None) == -1
    assert b"NULL" in lib.ffnk_last_error()
    assert lib.ffnk_masked_linear_fwd(None, 8, None, None, 1, 8, None, None, 8, -5, 8, 8, None, 0, None) == -2
    cfg = _lib.TileConfig()
    assert lib.ffnk_tile_config(0, 1, 1, 1, None) == -1
    # M == 0 is a valid no-op that touches no pointer
    assert lib.ffnk_masked_linear_fwd(None, 8, None, None, 1, 8, None, None, 8, 0, 8, 8, None, 0, None) == 0


def test_ffn_backward_entry_rejects_bad_arguments_without_a_gpu():
    lib = _lib.load()
    P = ctypes.c_void_p
    one = P(16)  # a non-NULL, 16-byte aligned stand-in; rejected calls touch no memory
    def call(d=64, h=64, up_sk=1, ws=None, ws_bytes=0, dx_stride=64, M=8, g=one):
        return lib.ffnk_masked_ffn_bwd(g, d, one, d, one, one, one, one, up_sk, d, one, one, 1, h, one, one, dx_stride,
                                       one, one, one, one, 1, d, one, one, 1, h, M, d, h, ws, ws_bytes, None)
    assert call(g=None) == -1                       # NULL g
    assert call(dx_stride=8) == -3                  # dx rows shorter than d
    assert call(d=60) == -3 and b"multiples of 8" in lib.ffnk_last_error()
    assert call(up_sk=64) == -3                     # up-projection weights not K-contiguous
    assert call() == -5                             # no workspace
    need = _lib.workspace_bytes(_lib.OP_FFN_BWD, 8192, 1024, 2048)
    assert need >= 8192 * 3 * 2048 * 2              # t1|t3 and dh in bf16, routed order
    assert need >= _lib.workspace_bytes(_lib.OP_FFN_FWD, 8192, 1024, 2048)


def test_ffn_save_entries_reject_bad_arguments_without_a_gpu():
    """The training forward that keeps the pre-activations and the backward that reads them."""
    lib = _lib.load()
    P = ctypes.c_void_p
    one = P(16)
    assert lib.ffnk_masked_ffn_can_save(4096, 4096, 14336) == 1
    assert lib.ffnk_masked_ffn_can_save(64, 4096, 14336) == 0   # decode sizes stream the weights
    assert lib.ffnk_masked_ffn_can_save(300, 36, 20) == 0       # any-stride kernels
    def fwd(M=128, d=64, h=64, pre=one, pre_stride=128, ws=None, ws_bytes=0):
        return lib.ffnk_masked_ffn_fwd_save(one, d, one, one, one, one, 1, d, one, one, 1, h, one, one, d, pre, pre_stride,
                                            M, d, h, ws, ws_bytes, None)
    assert fwd(pre=None) == -1
    assert fwd(M=8, d=1024, h=1024, pre_stride=2048) == -3 and b"LDS-tiled" in lib.ffnk_last_error()  # decode size
    assert fwd(pre_stride=64) == -3                                    # rows shorter than 2h
    assert fwd() == -5                                                 # passes validation, no workspace
    def bwd(pre=one, pre_stride=128):
        return lib.ffnk_masked_ffn_bwd_saved(one, 64, one, 64, one, one, one, one, 1, 64, one, one, 1, 64, one, pre,
                                             pre_stride, one, 64, one, one, one, one, 1, 64, one, one, 1, 64, 128, 64, 64,
                                             None, 0, None)
    assert bwd(pre=None) == -1
    assert bwd(pre_stride=100) == -3
    assert bwd() == -5


def test_ops_validate_inputs():
    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    w = torch.zeros(8, 8, dtype=torch.bfloat16)
    m = torch.zeros(4, dtype=torch.bool)
    with pytest.raises(ValueError, match="GPU"):
        MaskedLinear.apply(x, w.T, w.T, m)
    with pytest.raises(ValueError, match="bfloat16"):
        MaskedLinear.apply(x.float(), w.T, w.T, m)
    with pytest.raises(ValueError, match="2-D"):
        MaskedLinear.apply(x[None], w.T, w.T, m)
    with pytest.raises(ValueError):
        MaskedFFN.apply(x, w.T, w.T, w.T, w.T, w.T, w.T, m)


def test_workloads_are_seeded_and_shaped():
    a, b = wl.cfg1_linear_fwd(0), wl.cfg1_linear_fwd(0)
    assert torch.equal(a.x, b.x) and torch.equal(a.mask, b.mask) and torch.equal(a.Wv, b.Wv)
    assert a.x.shape == (2048, 1024) and a.mask.sum().item() == 2 * wl.IMAGE_TOKENS
    assert not torch.equal(a.x, wl.cfg1_linear_fwd(1).x)
    m4 = wl.cfg4_mask(0)
    per_seq = m4.sum(1).tolist()
    assert set(per_seq) == {0, 2 * 576, 5 * 576, 4096}
    c3 = wl.cfg3_linear_bwd()
    assert c3.grad.shape == (8192, 1024) and 0.45 < c3.mask.float().mean() < 0.55
    c5 = wl.cfg5_ffn_decode(1, "visual", d=64, h=128)
    assert c5.algorithmic_bytes() == 3 * 64 * 128 * 2 + 2 * 64 * 2 + 1
    c5b = wl.cfg5_ffn_decode(8, "bernoulli", d=64, h=128)
    nv = int(c5b.mask.sum())
    assert c5b.algorithmic_bytes() == 3 * 64 * 128 * 2 * (int(nv > 0) + int(nv < 8)) + 2 * 8 * 64 * 2 + 8
    assert wl.cfg2_ffn_fwd().routed_flops == 2 * 8192 * 1024 * 2048 * 3


def test_reference_import_name_resolves():
    """The reference's import line (ffn_kernel/__init__.py:1, README.md:46, 81) works unchanged."""
    from ffn_kernel import MaskedFFN as F2, MaskedLinear as L2
    assert L2 is MaskedLinear and F2 is MaskedFFN


def test_row_limit_is_what_one_route_launch_handles():
    assert _lib.workspace_bytes(_lib.OP_LINEAR_FWD, 1 << 24, 64, 64) > 0
    with pytest.raises(ValueError):
        _lib.workspace_bytes(_lib.OP_LINEAR_FWD, (1 << 24) + 1, 64, 64)


def test_measured_plans_are_consulted_before_the_rules():
    """Every entry of the generated table is what ffnk_tile_config reports for a shape inside its bucket,
    ffnk_debug_force_tile(-2) falls back to the rules, and the tuner's renderer reproduces the committed
    file byte for byte from its own entries."""
    from ffn_kernel_amd import tune
    text = tune.GEN_PATH.read_text()
    entries = [tuple(map(int, e)) for e in re.findall(r"^\s*\{(\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+), (\d+)\},$", text, re.M)]
    assert tune.render_header(entries) == text
    # what `--ops` keeps of a table it re-measures only in part is read back with the tuner's own parser
    assert tune.read_header(tune.GEN_PATH) == entries
    assert {k for kinds in tune.OP_KINDS.values() for k in kinds} == {tune.TUNED_PLAIN, tune.TUNED_DUAL, tune.TUNED_SPLITK, tune.TUNED_DOWN}
    geom = {0: (256, 256, 8), 1: (256, 256, 4), 2: (128, 128, 4), 4: (128, 128, 4)}
    lib = _lib.load()
    checked = 0
    for op, lo, hi, k, n, tile, splits, group_m in entries:
        assert group_m in (0, 2, 4, 8, 16) and (group_m == 0 or op != tune.TUNED_SPLITK)
        if op == tune.TUNED_DUAL:
            cfg = _lib.tile_config(_lib.OP_FFN_UP, hi, k, n)
            if tile in geom:
                assert (cfg["block_m"], cfg["waves_m"] * cfg["waves_n"]) == (geom[tile][0], geom[tile][2]), (op, hi, k, n, cfg)
            assert cfg["group_m"] == (group_m or 8), (op, hi, k, n, cfg)  # the plan's super-group size, else the SwiGLU tiles' own
            checked += 1
        elif op == tune.TUNED_PLAIN:
            cfg = _lib.tile_config(_lib.OP_LINEAR_FWD, hi, k, n)
            if cfg["path"] == _lib.PATH_MFMA_TILED:
                assert cfg["split_k"] == splits, (op, hi, k, n, cfg)
                if tile in geom and splits == 1:
                    assert (cfg["block_m"], cfg["block_n"]) == geom[tile][:2]
                checked += 1
            # a linear layer's plan is not an FFN down projection's, even at the same extents
            if not any(e[0] == tune.TUNED_DOWN and e[3:5] == (k, n) and e[1] <= hi <= e[2] for e in entries):
                try:
                    lib.ffnk_debug_force_tile(-2)
                    rules = _lib.tile_config(_lib.OP_FFN_DOWN, hi, n, k)
                finally:
                    lib.ffnk_debug_force_tile(-1)
                assert _lib.tile_config(_lib.OP_FFN_DOWN, hi, n, k) == rules, (hi, k, n)
        elif op == tune.TUNED_DOWN:
            cfg = _lib.tile_config(_lib.OP_FFN_DOWN, hi, n, k)  # FFN extents: K = d = output columns, N = h = contraction
            if cfg["path"] == _lib.PATH_MFMA_TILED:
                assert cfg["split_k"] == splits, (op, hi, k, n, cfg)
                if tile in geom:
                    assert (cfg["block_m"], cfg["block_n"]) == geom[tile][:2]
                checked += 1
        elif op == tune.TUNED_SPLITK:
            # k = R = N, n = Cc = K of the MaskedLinear backward; the measured factor is launched as it is,
            # also where the fused launch's own cost model would have chosen otherwise
            for M in (hi, (lo + hi) // 2):
                cfg = _lib.tile_config(_lib.OP_BWD_DW, M, n, k)
                assert cfg["split_k"] == splits, (op, M, k, n, cfg)
                # the plan names the form as well: tile 5 reads g and x in place, any other tile reads transposes
                assert cfg["in_place"] == int(tile == tune.TILE_IN_PLACE), (op, M, k, n, cfg)
                if tile in geom:
                    assert (cfg["block_m"], cfg["block_n"]) == geom[tile][:2]
                if tile == tune.TILE_IN_PLACE:
                    assert (cfg["block_m"], cfg["block_n"], cfg["lds_stages"]) == (128, 128, 2)
            checked += 1
    assert checked > 0 or not entries
    ops_seen = {e[0] for e in entries}
    assert ops_seen <= {tune.TUNED_PLAIN, tune.TUNED_DUAL, tune.TUNED_SPLITK, tune.TUNED_DOWN}
    if entries:
        op, lo, hi, k, n, tile, splits, _ = next((e for e in entries if e[0] == tune.TUNED_DOWN), entries[0])
        try:
            assert lib.ffnk_debug_force_tile(-2) == -1
            rules = _lib.tile_config(_lib.OP_FFN_DOWN, hi, n, k)
        finally:
            lib.ffnk_debug_force_tile(-1)
        assert isinstance(rules["split_k"], int)


def test_bench_refuses_more_than_one_gpu():
    """This build measures one GPU: bench.py --gpus N with N above 1 exits with a message, before it touches a device."""
    import subprocess
    import sys
    bench = Path(__file__).resolve().parents[1] / "bench.py"
    proc = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert "one GPU" in proc.stderr and not proc.stdout.strip()


def test_tuner_checks_its_layer_arguments_before_it_needs_a_gpu():
    """--ffn D,H / --linear K,N add layers to the sweep: extents that the MFMA paths cannot take are refused
    at the command line; without a GPU the tuner then says so and returns 2."""
    from ffn_kernel_amd import tune
    with pytest.raises(SystemExit):
        tune.main(["--ffn", "100,200"])
    with pytest.raises(SystemExit):
        tune.main(["--linear", "1024"])
    if not torch.cuda.is_available():
        assert tune.main(["--ffn", "2048,5632", "--linear", "2048,2048", "--quick"]) == 2


def test_lean_ffn_backward_workspace_never_exceeds_the_any_layout_one():
    lib = _lib.load()
    for M, d, h in ((0, 64, 64), (1, 64, 128), (300, 256, 512), (4096, 4096, 14336), (8192, 4096, 14336), (333, 72, 200)):
        worst = _lib.workspace_bytes(_lib.OP_FFN_BWD, M, d, h)
        for usn, dsk, dsn in ((d, 1, h), (d, d, 1), (d + 8, 1, h + 8), (d, 3, h)):
            for gk in (1, h):
                lean = lib.ffnk_workspace_bytes_ffn_bwd(M, d, h, d, usn, dsk, dsn, gk, gk)
                assert 0 < lean <= worst, (M, d, h, usn, dsk, dsn, gk, lean, worst)
    assert lib.ffnk_workspace_bytes_ffn_bwd(8192, 4096, 14336, 4096, 4096, 1, 14336, 1, 1) < 1 << 30
    assert lib.ffnk_workspace_bytes_ffn_bwd(-1, 64, 64, 64, 64, 1, 64, 1, 1) == ctypes.c_size_t(-1).value
