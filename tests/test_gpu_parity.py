"""GPU parity: the HIP path (through the C ABI) against the CPU oracle.

Tolerance (floating point): max-abs <= 2e-2 (or <= 1 bf16 ulp of the reference where bf16 cannot
resolve 2e-2) and rel-L2 <= 5e-3 against a double-precision reference.  Routing is bit-exact.
"""
import ctypes

import numpy as np
import pytest
import torch

from ffn_kernel_amd import MaskedFFN, MaskedLinear, _lib
from ffn_kernel_amd import workloads as wl
from ffn_kernel_amd.ops import masked_ffn_backward, masked_ffn_forward, masked_linear_backward
from oracle import cref
from oracle import modules as om
from helpers import assert_close, assert_close_bf16_pair, assert_close_pipeline, note

pytestmark = pytest.mark.gpu


# ------------------------------------------------------------------ routing (integer, bit-exact)
@pytest.mark.parametrize("M", [0, 1, 2, 15, 16, 17, 63, 64, 65, 255, 4095, 4096, 4097, 10000, 32768, 100003, 262144, 262145,
                               600001])  # past 262144 rows a block of the partition kernel places several 1024-row chunks
@pytest.mark.parametrize("p", [0.0, 0.5, 1.0])
def test_route_bit_exact(dev, M, p):
    note(f"route M={M} p={p}")
    gen = torch.Generator().manual_seed(M * 7 + int(p * 10))
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    perm_ref, counts_ref = om.stable_partition(mask.numpy())
    mask_d = mask.to(dev)
    perm = torch.full((max(M, 1),), -1, dtype=torch.int32, device=dev)
    counts = torch.full((2,), -1, dtype=torch.int32, device=dev)
    rc = _lib.load().ffnk_route(mask_d.data_ptr() if M else None, M, perm.data_ptr(), counts.data_ptr(),
                                torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "ffnk_route")
    torch.cuda.synchronize()
    assert counts.cpu().numpy().tolist() == counts_ref.tolist()
    assert np.array_equal(perm.cpu().numpy()[:M], perm_ref)


def test_route_unaligned_mask_view(dev):
    note("route on a mask view that starts at an odd byte")
    gen = torch.Generator().manual_seed(5)
    big = (torch.rand(9000, generator=gen) < 0.4).to(dev)
    for off in (1, 3, 7, 13):
        mask = big[off:off + 8191]
        perm_ref, counts_ref = om.stable_partition(mask.cpu().numpy())
        perm = torch.empty(8191, dtype=torch.int32, device=dev)
        counts = torch.empty(2, dtype=torch.int32, device=dev)
        _lib.check(_lib.load().ffnk_route(mask.data_ptr(), 8191, perm.data_ptr(), counts.data_ptr(),
                                          torch.cuda.current_stream().cuda_stream), "ffnk_route")
        assert counts.cpu().numpy().tolist() == counts_ref.tolist()
        assert np.array_equal(perm.cpu().numpy(), perm_ref)


# ------------------------------------------------------------------ MaskedLinear forward
def _run_linear(w, dev):
    d = w.to(dev)
    y = MaskedLinear.apply(d.x, d.Wv.T, d.Wt.T, d.mask)
    torch.cuda.synchronize()
    return y


LINEAR_SHAPES = [
    # (M, K, N, p_visual)            what it exercises
    (37, 48, 40, 0.5),               # tiny, ragged everything, K tail (register-staged loads)
    (1, 64, 64, 1.0),                # single visual row
    (1, 64, 64, 0.0),                # single text row
    (129, 64, 200, 0.3),             # direct loads, ragged N
    (300, 128, 136, 0.7),            # partial tiles in both groups
    (513, 1024, 1024, 0.5),          # Bernoulli mask
    (2048, 1024, 1024, -1),          # cfg1 (span mask)
    (4096, 512, 2048, 0.5),          # 256x256 tile family
    (1000, 72, 264, 0.5),            # K % 64 != 0, K % 8 == 0
    (100, 2048, 512, 0.5),           # few output tiles, long K: split-K + reduce pass
    # decode sizes (M <= 64): the weight-streaming kernels of the FFN down projection
    (1, 4096, 1024, 1.0),            # dot-product streams, one row
    (8, 512, 100, 0.5),              # dot-product streams, ragged N, one slice
    (5, 1024, 1000, 0.4),
    (24, 2048, 512, 0.5),            # LDS-transposed streams, split-K + reduce
    (40, 1024, 192, 0.5),            # eight chunks, no split
    (64, 2048, 256, 0.5),
    (33, 1152, 320, 0.0),            # nine chunks, one modality absent
    (200, 3136, 260, 0.4),           # split-K with 49 slabs (unequal ranges), ragged N
    (96, 1024, 250, 0.5),            # N % 4 != 0: no split
]


@pytest.mark.parametrize("M,K,N,p", LINEAR_SHAPES)
def test_linear_fwd_vs_oracle(dev, M, K, N, p):
    note(f"linear fwd M={M} K={K} N={N} p={p}")
    if p < 0:
        w = wl.cfg1_linear_fwd()
    else:
        gen = torch.Generator().manual_seed(M + K + N)
        mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
        w = wl.make_linear("t", M, K, N, mask, seed=M)
    y = _run_linear(w, dev)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    ref = cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask)
    assert_close(y, ref, f"linear fwd {M}x{K}x{N}")
    # and against the reference's own (blend-form, bf16) PyTorch module maths
    blend = om.linear_blend(w.x, w.Wv, w.Wt, w.mask)
    assert_close_bf16_pair(y, blend, "vs blend-form bf16 module")


def test_linear_row_selection_is_exact(dev):
    """W_v = I, W_t = 2 I: every output row equals x or 2 x bit for bit."""
    note("linear identity weights")
    M, K = 777, 256
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    mask = torch.rand(M, generator=gen) < 0.5
    eye = torch.eye(K).to(torch.bfloat16)
    y = MaskedLinear.apply(x.to(dev), eye.to(dev).T, (2 * eye).to(dev).T, mask.to(dev)).cpu()
    expect = torch.where(mask[:, None], x, 2 * x)
    assert torch.equal(y, expect)


@pytest.mark.parametrize("M", [3, 17, 64])
def test_linear_decode_rows_exact_and_absent_weight_untouched(dev, M):
    """Decode sizes run on the weight-streaming kernels: identity weights select bit for bit, and the
    weight of a modality with no rows is never read (NaN poison)."""
    note(f"linear decode identity/poison M={M}")
    K = 1024
    gen = torch.Generator().manual_seed(M)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    mask = torch.rand(M, generator=gen) < 0.5
    assert _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, K)["path"] == _lib.PATH_STREAM
    eye = torch.eye(K).to(torch.bfloat16)
    y = MaskedLinear.apply(x.to(dev), eye.to(dev).T, (2 * eye).to(dev).T, mask.to(dev)).cpu()
    assert torch.equal(y, torch.where(mask[:, None], x, 2 * x))
    poison = torch.full((K, K), float("nan"), dtype=torch.bfloat16)
    y = MaskedLinear.apply(x.to(dev), eye.to(dev).T, poison.to(dev).T, torch.ones(M, dtype=torch.bool, device=dev)).cpu()
    assert torch.equal(y, x)
    y = MaskedLinear.apply(x.to(dev), poison.to(dev).T, eye.to(dev).T, torch.zeros(M, dtype=torch.bool, device=dev)).cpu()
    assert torch.equal(y, x)


@pytest.mark.parametrize("p", [1.0, 0.0, 0.5])
def test_linear_decode_long_k_single_modality(dev, p):
    """Streamed linear with 16-chunk K ranges: one modality absent or both present."""
    M, K, N = 40, 8192, 4096
    note(f"linear decode long K p={p}")
    cfg = _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)
    assert cfg["path"] == _lib.PATH_STREAM and cfg["split_k"] == 4
    gen = torch.Generator().manual_seed(11)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_linear("t", M, K, N, mask, seed=5)
    y = _run_linear(w, dev)
    assert_close(y, om.linear_select(w.x, w.Wv, w.Wt, w.mask, torch.float64), f"linear decode long K p={p}")


def test_linear_unused_branch_never_touched(dev):
    """Poisoning the text weight with NaN must leave visual rows finite (the blend form would not)."""
    note("linear NaN poison")
    M, K, N = 300, 128, 128
    gen = torch.Generator().manual_seed(4)
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_linear("t", M, K, N, mask, seed=9)
    Wt = torch.full_like(w.Wt, float("nan"))
    y = MaskedLinear.apply(w.x.to(dev), w.Wv.to(dev).T, Wt.to(dev).T, mask.to(dev)).cpu()
    assert torch.isfinite(y[mask]).all()
    assert torch.isnan(y[~mask]).all()
    ref = cref.linear_fwd(w.x, w.Wv, w.Wt, torch.ones(M, dtype=torch.bool))
    assert_close(y[mask], ref[mask], "visual rows")


def test_linear_row_permutation_equivariance(dev):
    """Permuting rows of (x, mask) permutes the output rows bit for bit."""
    note("linear permutation equivariance")
    M, K, N = 1000, 256, 320
    gen = torch.Generator().manual_seed(8)
    mask = torch.rand(M, generator=gen) < 0.4
    w = wl.make_linear("t", M, K, N, mask, seed=2).to(dev)
    y = MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, w.mask)
    pi = torch.randperm(M, generator=gen).to(dev)
    y2 = MaskedLinear.apply(w.x[pi].contiguous(), w.Wv.T, w.Wt.T, w.mask[pi].contiguous())
    assert torch.equal(y[pi], y2)


def test_linear_generic_path_odd_shapes(dev):
    """K not a multiple of 8 and a [K, N]-contiguous weight go through other code paths."""
    note("linear generic path")
    for (M, K, N) in [(50, 30, 17), (9, 1, 5), (64, 100, 3)]:
        gen = torch.Generator().manual_seed(M)
        mask = torch.rand(M, generator=gen) < 0.5
        w = wl.make_linear("t", M, K, N, mask, seed=M)
        y = _run_linear(w, dev)
        assert_close(y, cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask), f"generic {M}x{K}x{N}")
    # weight given as a contiguous [K, N] tensor (stride (N, 1)): re-laid once by the op
    M, K, N = 256, 128, 192
    mask = torch.rand(M, generator=torch.Generator().manual_seed(1)) < 0.5
    w = wl.make_linear("t", M, K, N, mask, seed=5)
    d = w.to(dev)
    y = MaskedLinear.apply(d.x, d.Wv.T.contiguous(), d.Wt.T.contiguous(), d.mask)
    assert_close(y, cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask), "[K,N]-contiguous weights")


def test_linear_strided_x_and_empty(dev):
    note("linear strided x / empty")
    M, K, N = 200, 64, 128
    mask = torch.rand(M, generator=torch.Generator().manual_seed(1)) < 0.5
    w = wl.make_linear("t", M, K, N, mask, seed=6)
    wide = torch.zeros(M, 2 * K, dtype=torch.bfloat16, device=dev)
    wide[:, :K] = w.x.to(dev)
    y = MaskedLinear.apply(wide[:, :K], w.Wv.to(dev).T, w.Wt.to(dev).T, mask.to(dev))
    assert_close(y, cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask), "row-strided x")
    y0 = MaskedLinear.apply(torch.empty(0, K, dtype=torch.bfloat16, device=dev), w.Wv.to(dev).T, w.Wt.to(dev).T,
                            torch.empty(0, dtype=torch.bool, device=dev))
    assert y0.shape == (0, N)


# ------------------------------------------------------------------ MaskedFFN forward
FFN_SHAPES = [
    (19, 32, 48, 0.5),        # K tails in both stages
    (1, 64, 128, 1.0),
    (1, 64, 128, 0.0),
    (8, 256, 512, 0.5),
    (64, 512, 1024, 0.5),
    (333, 128, 320, 0.3),
    (2048, 1024, 2048, 0.5),
    (50, 36, 20, 0.5),        # generic path (d, h not multiples of 8)
    # few output tiles over a long contraction: split-K down projection + reduce pass
    (100, 256, 2048, 0.5),
    (65, 1024, 2240, 0.4),    # 35 slabs: ranges of unequal length
    (300, 512, 4096, 1.0),    # one modality only
    (700, 264, 3072, 0.6),    # ragged output tile
]


def test_ffn_fwd_split_k_table():
    """The shapes above that are meant to exercise the split-K down projection do."""
    for M, d, h in ((100, 256, 2048), (65, 1024, 2240), (300, 512, 4096), (700, 264, 3072)):
        cfg = _lib.tile_config(_lib.OP_FFN_DOWN, M, d, h)
        assert cfg["path"] == _lib.PATH_MFMA_TILED and cfg["split_k"] > 1, (M, d, h, cfg)
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 32768, 4096, 14336)["split_k"] == 1


@pytest.mark.parametrize("M,d,h,p", FFN_SHAPES)
def test_ffn_fwd_vs_oracle(dev, M, d, h, p):
    note(f"ffn fwd M={M} d={d} h={h} p={p}")
    gen = torch.Generator().manual_seed(M + d + h)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_ffn("t", M, d, h, mask, seed=M, w_std=0.05)
    out = MaskedFFN.apply(*w.to(dev).op_args())
    torch.cuda.synchronize()
    assert out.dtype == torch.bfloat16 and out.shape == (M, d)
    # The [M, h] intermediate is stored in bf16 (as the reference stores it, ffn.py:113), so the
    # exact reference rounds it once too; the unrounded maths is reported alongside.
    assert_close(out, cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True), f"ffn {M}x{d}x{h}")
    rep = om.error_report(out.float().cpu(), cref.ffn_fwd(w.x, w.W, w.mask))
    assert rep["rel_l2"] <= om.REL_L2_TOL and rep["max_excess"] <= 2.0, rep
    assert_close_bf16_pair(out, om.ffn_blend(w.x, w.W, w.mask), "vs blend-form bf16 module")


# decode shapes (M <= 64, d and h multiples of 256): the weight-streaming kernels
DECODE_SHAPES = [(1, "visual"), (1, "text"), (2, "bernoulli"), (8, "bernoulli"), (15, "bernoulli"), (16, "visual"),
                 (17, "bernoulli"), (32, "bernoulli"), (33, "text"), (47, "bernoulli"), (64, "bernoulli"),
                 (64, "visual")]


@pytest.mark.parametrize("M,kind", DECODE_SHAPES)
@pytest.mark.parametrize("d,h", [(256, 512), (512, 1792)])
def test_ffn_decode_path_vs_oracle(dev, M, kind, d, h):
    note(f"ffn decode M={M} kind={kind} d={d} h={h}")
    assert _lib.tile_config(_lib.OP_FFN_FWD, M, d, h)["path"] == _lib.PATH_STREAM
    w = wl.cfg5_ffn_decode(M, kind, seed=M, d=d, h=h)
    w = wl.FFNWorkload(w.name, w.x, {k: (v.float() * 2.5).to(torch.bfloat16) for k, v in w.W.items()}, w.mask)
    out = MaskedFFN.apply(*w.to(dev).op_args())
    torch.cuda.synchronize()
    assert_close(out, cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True), f"decode {M} {kind}")
    # an absent modality's weights are never read: poison them
    if kind in ("visual", "text"):
        W = dict(w.W)
        for k in (("u1", "u2", "u3") if kind == "visual" else ("w1", "w2", "w3")):
            W[k] = torch.full_like(W[k], float("nan"))
        out2 = MaskedFFN.apply(*wl.FFNWorkload("p", w.x, W, w.mask).to(dev).op_args())
        assert torch.equal(out2, out)


# M <= 8 with K extents in whole 512-element slices: the contiguous-row dot-product streams
DOT_SHAPES = [(1, "visual"), (1, "text"), (2, "bernoulli"), (3, "visual"), (4, "bernoulli"), (5, "text"),
              (7, "bernoulli"), (8, "bernoulli"), (8, "visual")]


@pytest.mark.parametrize("M,kind", DOT_SHAPES)
@pytest.mark.parametrize("d,h", [(512, 1024), (1024, 4096), (4096, 1536), (1536, 7168)])
def test_ffn_decode_dot_path_vs_oracle(dev, M, kind, d, h):
    note(f"ffn decode dot M={M} kind={kind} d={d} h={h}")
    cfg = _lib.tile_config(_lib.OP_FFN_UP, M, d, h)
    assert cfg["path"] == _lib.PATH_STREAM and cfg["block_m"] == M and cfg["block_k"] in (512, 1024)
    w = wl.cfg5_ffn_decode(M, kind, seed=40 + M, d=d, h=h)
    w = wl.FFNWorkload(w.name, w.x, {k: (v.float() * 2.5).to(torch.bfloat16) for k, v in w.W.items()}, w.mask)
    out = MaskedFFN.apply(*w.to(dev).op_args())
    torch.cuda.synchronize()
    assert_close(out, cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True), f"decode dot {M} {kind}")
    if kind in ("visual", "text"):
        W = dict(w.W)
        for k in (("u1", "u2", "u3") if kind == "visual" else ("w1", "w2", "w3")):
            W[k] = torch.full_like(W[k], float("nan"))
        out2 = MaskedFFN.apply(*wl.FFNWorkload("p", w.x, W, w.mask).to(dev).op_args())
        assert torch.equal(out2, out)


# 9 <= M <= 64 (and smaller M off the dot kernels' extents) with d, h >= 1024: LDS-transposed streams
TILE_STREAM_SHAPES = [(9, "bernoulli"), (16, "visual"), (17, "bernoulli"), (31, "text"), (33, "text"),
                      (48, "bernoulli"), (64, "bernoulli"), (64, "visual"), (5, "bernoulli")]


@pytest.mark.parametrize("M,kind", TILE_STREAM_SHAPES)
@pytest.mark.parametrize("d,h", [(1024, 2048), (2048, 1024), (1152, 1408)])
def test_ffn_decode_tile_stream_vs_oracle(dev, M, kind, d, h):
    note(f"ffn decode tile stream M={M} kind={kind} d={d} h={h}")
    cfg = _lib.tile_config(_lib.OP_FFN_UP, M, d, h)
    assert cfg["path"] == _lib.PATH_STREAM
    if M > 8 or d % 512:
        assert cfg["block_k"] == 128 and cfg["lds_stages"] >= 3
    w = wl.cfg5_ffn_decode(M, kind, seed=70 + M, d=d, h=h)
    w = wl.FFNWorkload(w.name, w.x, {k: (v.float() * 1.5).to(torch.bfloat16) for k, v in w.W.items()}, w.mask)
    out = MaskedFFN.apply(*w.to(dev).op_args())
    torch.cuda.synchronize()
    assert_close(out, cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True), f"decode tile stream {M} {kind}")
    if kind in ("visual", "text"):
        W = dict(w.W)
        for k in (("u1", "u2", "u3") if kind == "visual" else ("w1", "w2", "w3")):
            W[k] = torch.full_like(W[k], float("nan"))
        out2 = MaskedFFN.apply(*wl.FFNWorkload("p", w.x, W, w.mask).to(dev).op_args())
        assert torch.equal(out2, out)


@pytest.mark.parametrize("kind", ["visual", "text", "bernoulli"])
def test_ffn_decode_long_ranges(dev, kind):
    """Decode call whose down projection is split into K ranges of 16 chunks; one modality absent or
    both present, and the absent modality's weights are never read."""
    M, d, h = 48, 4096, 8192
    note(f"ffn decode long ranges M={M} kind={kind}")
    assert _lib.tile_config(_lib.OP_FFN_DOWN, M, d, h)["split_k"] == 4  # 16 chunks per range
    w = wl.cfg5_ffn_decode(M, kind, seed=7, d=d, h=h)
    out = MaskedFFN.apply(*w.to(dev).op_args())
    torch.cuda.synchronize()
    assert_close(out, om.ffn_select(w.x, w.W, w.mask, torch.float64, round_intermediate=True), f"long ranges {kind}")
    if kind != "bernoulli":
        W = dict(w.W)
        for k in (("u1", "u2", "u3") if kind == "visual" else ("w1", "w2", "w3")):
            W[k] = torch.full_like(W[k], float("nan"))
        out2 = MaskedFFN.apply(*wl.FFNWorkload("p", w.x, W, w.mask).to(dev).op_args())
        assert torch.equal(out2, out)


def test_ffn_decode_matches_tiled_path_rows(dev):
    """The same rows run as a decode call and inside a larger (tiled-path) call agree to bf16 accuracy."""
    note("ffn decode vs tiled")
    d, h = 512, 1024
    big = wl.make_ffn("t", 200, d, h, torch.rand(200, generator=torch.Generator().manual_seed(3)) < 0.5, seed=4,
                      w_std=0.05).to(dev)
    full = MaskedFFN.apply(*big.op_args())
    small = wl.FFNWorkload("s", big.x[:48].contiguous(), big.W, big.mask[:48].contiguous())
    part = MaskedFFN.apply(*small.op_args())
    assert_close_bf16_pair(part, full[:48].float().cpu(), "decode rows vs tiled rows")


def test_ffn_cfg2(dev):
    note("ffn cfg2")
    w = wl.cfg2_ffn_fwd()
    out = MaskedFFN.apply(*w.to(dev).op_args())
    # double-precision torch reference on the select form (the C loops would take minutes here)
    ref = om.ffn_select(w.x, w.W, w.mask, torch.float64, round_intermediate=True)
    rep = assert_close(out, ref, "cfg2")
    assert_close(out, om.ffn_select(w.x, w.W, w.mask, torch.float64), "cfg2 vs unrounded intermediate")
    print("cfg2 error:", rep)


def test_ffn_closed_forms(dev):
    """W3 = 0 or W1 = 0 gives exact zeros on visual rows; text rows unaffected."""
    note("ffn closed forms")
    M, d, h = 130, 64, 128
    mask = torch.rand(M, generator=torch.Generator().manual_seed(2)) < 0.5
    w = wl.make_ffn("t", M, d, h, mask, seed=3, w_std=0.05)
    ref = cref.ffn_fwd(w.x, w.W, w.mask)
    for zero in ("w3", "w1"):
        W = dict(w.W)
        W[zero] = torch.zeros_like(W[zero])
        w2 = wl.FFNWorkload("z", w.x, W, w.mask).to(dev)
        out = MaskedFFN.apply(*w2.op_args()).cpu()
        assert (out[mask] == 0).all()
        assert_close(out[~mask], ref[~mask], "text rows")


# ------------------------------------------------------------------ MaskedFFN backward
FFN_BWD_SHAPES = [
    (37, 64, 128, 0.5),
    (64, 64, 64, 1.0),      # no text rows: dU* must be exact zeros
    (64, 64, 64, 0.0),
    (300, 256, 512, 0.5),
    (1000, 512, 384, 0.3),
    (2048, 1024, 2048, 0.5),
    (150, 256, 1024, 0.5),  # dx GEMM: few output tiles over a 2048-long contraction, split over K
]


@pytest.mark.parametrize("M,d,h,p", FFN_BWD_SHAPES)
def test_ffn_bwd_vs_oracle(dev, M, d, h, p):
    """The reference raises NotImplementedError here (ops.py:34-38); the oracle is the chain rule of
    its PyTorch module (pinned on the CPU against autograd and finite differences)."""
    note(f"ffn bwd M={M} d={d} h={h} p={p}")
    gen = torch.Generator().manual_seed(M + d + h + 3)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_ffn("t", M, d, h, mask, seed=M + 2, w_std=0.05)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    dw = w.to(dev)
    x = dw.x.clone().requires_grad_(True)
    Wp = {k: v.clone().requires_grad_(True) for k, v in dw.W.items()}
    out = MaskedFFN.apply(x, Wp["w1"].T, Wp["w2"].T, Wp["w3"].T, Wp["u1"].T, Wp["u2"].T, Wp["u3"].T, dw.mask)
    out.backward(g.to(dev))
    torch.cuda.synchronize()
    # exact chain rule with the intermediates rounded to bf16 where the kernels store them in bf16
    dx, dW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64, round_intermediates=True)
    assert x.grad.shape == (M, d)
    assert_close_pipeline(x.grad, dx, "dx")
    for k in ("w1", "w2", "w3", "u1", "u2", "u3"):
        assert Wp[k].grad.shape == w.W[k].shape and Wp[k].grad.is_contiguous()
        assert_close_pipeline(Wp[k].grad, dW[k], f"d{k}")
    # and against the unrounded maths, at bf16-pipeline accuracy
    dx_e, dW_e = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64)
    rep = om.error_report(x.grad.float().cpu(), dx_e)
    assert rep["rel_l2"] <= 1.5e-2, rep
    for k in dW_e:
        rep = om.error_report(Wp[k].grad.float().cpu(), dW_e[k])
        assert rep["rel_l2"] <= 1.5e-2 or dW_e[k].abs().max() == 0, (k, rep)
    absent = ("u1", "u2", "u3") if p == 1.0 else ("w1", "w2", "w3") if p == 0.0 else ()
    for k in absent:
        assert (Wp[k].grad == 0).all()


@pytest.mark.parametrize("M,d,h,down_contig", [(300, 256, 512, True), (333, 72, 200, False), (500, 128, 96, False),
                                               (2100, 512, 1024, True)])
def test_ffn_bwd_weight_layouts(dev, M, d, h, down_contig):
    """The backward GEMMs read the weights in place when the layout allows it (the transposed views of
    [out, in] weights that the reference passes: K-major kernels; a contiguous [h, d] down weight: the
    forward's kernels) and copy them otherwise (d or h not a multiple of 64).  Same gradients either way."""
    note(f"ffn bwd layouts M={M} d={d} h={h} down_contig={down_contig}")
    gen = torch.Generator().manual_seed(M + d + h)
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_ffn("t", M, d, h, mask, seed=M + 5, w_std=0.05)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    dw = w.to(dev)
    x = dw.x.clone().requires_grad_(True)
    Wp = {k: v.clone().requires_grad_(True) for k, v in dw.W.items()}
    # down weights as contiguous [h, d] tensors (stride_n == 1) instead of views of [d, h] ones
    W2T = {k: Wp[k].T.contiguous().detach().requires_grad_(True) for k in ("w2", "u2")} if down_contig else None
    dn = (lambda k: W2T[k]) if down_contig else (lambda k: Wp[k].T)
    out = MaskedFFN.apply(x, Wp["w1"].T, dn("w2"), Wp["w3"].T, Wp["u1"].T, dn("u2"), Wp["u3"].T, dw.mask)
    out.backward(g.to(dev))
    torch.cuda.synchronize()
    dx, dW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64, round_intermediates=True)
    assert_close_pipeline(x.grad, dx, "dx")
    for k in ("w1", "w3", "u1", "u3"):
        assert_close_pipeline(Wp[k].grad, dW[k], f"d{k}")
    for k in ("w2", "u2"):
        got = W2T[k].grad.T if down_contig else Wp[k].grad
        assert_close_pipeline(got, dW[k], f"d{k}")


def test_ffn_bwd_weights_that_are_slices_of_larger_tensors(dev):
    """Weights whose rows are longer than the extent used (column slices of wider tensors: row stride >
    d or h, still 16-byte aligned) are read in place with their own row stride, forward and backward."""
    note("ffn bwd sliced weights")
    M, d, h = 700, 256, 384
    gen = torch.Generator().manual_seed(5)
    mask = torch.rand(M, generator=gen) < 0.45
    w = wl.make_ffn("t", M, d, h, mask, seed=9, w_std=0.05)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    dw = w.to(dev)
    x = dw.x.clone().requires_grad_(True)
    wide = {}
    for k, v in dw.W.items():  # [out, in] weights embedded in [out, in + 64] tensors
        big = torch.zeros(v.shape[0], v.shape[1] + 64, dtype=v.dtype, device=dev)
        big[:, 8:8 + v.shape[1]] = v
        wide[k] = big.requires_grad_(True)
    view = lambda k: wide[k][:, 8:8 + dw.W[k].shape[1]].T
    out = MaskedFFN.apply(x, view("w1"), view("w2"), view("w3"), view("u1"), view("u2"), view("u3"), dw.mask)
    out.backward(g.to(dev))
    torch.cuda.synchronize()
    ref = cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True)
    assert_close(out, ref, "out")
    dx, dW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64, round_intermediates=True)
    assert_close_pipeline(x.grad, dx, "dx")
    for k in dW:
        got = wide[k].grad[:, 8:8 + dw.W[k].shape[1]]
        assert_close_pipeline(got, dW[k], f"d{k}")
        assert (wide[k].grad[:, :8] == 0).all() and (wide[k].grad[:, 8 + dw.W[k].shape[1]:] == 0).all()


def test_ffn_bwd_non_finite_rows_stay_in_their_modality(dev):
    """The weight-gradient GEMMs load the rows of dt and of the intermediate in 64-row slabs that run past
    a modality's last row; what lies there (the other modality's rows) must not count - not even as
    0 * inf.  A non-finite upstream gradient on text rows leaves the visual weights' gradients, and the
    visual rows of dx, exactly as they are without it."""
    note("ffn bwd non-finite rows")
    M, d, h = 333, 128, 256
    gen = torch.Generator().manual_seed(11)
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_ffn("t", M, d, h, mask, seed=4, w_std=0.05).to(dev)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16).to(dev)
    g_bad = g.clone()
    g_bad[~w.mask] = float("inf")

    def grads(gg):
        x = w.x.clone().requires_grad_(True)
        Wp = {k: v.clone().requires_grad_(True) for k, v in w.W.items()}
        out = MaskedFFN.apply(x, Wp["w1"].T, Wp["w2"].T, Wp["w3"].T, Wp["u1"].T, Wp["u2"].T, Wp["u3"].T, w.mask)
        out.backward(gg)
        torch.cuda.synchronize()
        return x.grad, {k: v.grad for k, v in Wp.items()}

    dx0, dW0 = grads(g)
    dx1, dW1 = grads(g_bad)
    for k in ("w1", "w2", "w3"):
        assert torch.isfinite(dW1[k]).all() and torch.equal(dW1[k], dW0[k]), k
    assert torch.equal(dx1[w.mask], dx0[w.mask])
    assert not torch.isfinite(dW1["u2"]).all()


@pytest.mark.parametrize("M,d,h,p", [(300, 256, 512, 0.5), (1000, 512, 384, 0.3), (777, 128, 320, 1.0), (4500, 1024, 1024, 0.6)])
def test_ffn_saved_pre_activations(dev, M, d, h, p):
    """A forward that keeps the pre-activations returns the same output, pre-activations that match the
    oracle's t1 | t3 in routed order, and a backward from them that equals the recomputing backward
    bit for bit (both take the same GEMM sums through the same bf16 rounding)."""
    note(f"ffn saved pre-activations M={M} d={d} h={h} p={p}")
    from ffn_kernel_amd.ops import masked_ffn_backward, masked_ffn_forward
    gen = torch.Generator().manual_seed(M + 17)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_ffn("t", M, d, h, mask, seed=M + 1, w_std=0.05)
    dw = w.to(dev)
    args = (dw.x, dw.W["w1"].T, dw.W["w2"].T, dw.W["w3"].T, dw.W["u1"].T, dw.W["u2"].T, dw.W["u3"].T, dw.mask)
    out_plain = masked_ffn_forward(*args)
    out, pre = masked_ffn_forward(*args, save_pre=True)
    assert pre is not None and pre.shape == (M, 2 * h) and pre.dtype == torch.bfloat16
    assert torch.equal(out, out_plain)
    perm, _ = om.stable_partition(mask.numpy())
    xr = w.x.double()[torch.from_numpy(perm).long()]
    mr = mask[torch.from_numpy(perm).long()]
    t1 = torch.where(mr[:, None], xr @ w.W["w1"].double().T, xr @ w.W["u1"].double().T)
    t3 = torch.where(mr[:, None], xr @ w.W["w3"].double().T, xr @ w.W["u3"].double().T)
    assert_close(pre[:, :h], t1, "saved t1")
    assert_close(pre[:, h:], t3, "saved t3")
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16).to(dev)
    keep = pre.clone()
    a = masked_ffn_backward(g, *args)
    b = masked_ffn_backward(g, *args, pre=pre)
    assert torch.equal(pre, keep)  # read-only
    for u, v in zip(a, b):
        assert torch.equal(u, v)


def test_ffn_forward_keeps_nothing_at_decode_sizes(dev):
    note("ffn save_pre at decode sizes")
    from ffn_kernel_amd.ops import masked_ffn_forward
    w = wl.cfg5_ffn_decode(24, "bernoulli", seed=3, d=1024, h=2048).to(dev)
    out, pre = masked_ffn_forward(*w.op_args(), save_pre=True)
    assert pre is None and torch.equal(out, masked_ffn_forward(*w.op_args()))
    x = w.x.clone().requires_grad_(True)
    MaskedFFN.apply(x, *w.op_args()[1:]).sum().backward()  # recomputing backward
    assert x.grad is not None and torch.isfinite(x.grad).all()


def test_ffn_bwd_is_deterministic_and_validates(dev):
    note("ffn bwd determinism / validation")
    from ffn_kernel_amd.ops import masked_ffn_backward
    mask = torch.rand(500, generator=torch.Generator().manual_seed(5)) < 0.5
    w = wl.make_ffn("t", 500, 128, 256, mask, seed=9, w_std=0.05).to(dev)
    g = torch.randn(500, 128, generator=torch.Generator().manual_seed(6)).to(torch.bfloat16).to(dev)
    args = (g, w.x, w.W["w1"].T, w.W["w2"].T, w.W["w3"].T, w.W["u1"].T, w.W["u2"].T, w.W["u3"].T, w.mask)
    a = masked_ffn_backward(*args)
    b = masked_ffn_backward(*args)
    for ta, tb in zip(a, b):
        assert torch.equal(ta, tb)
    # weights given in the other layout ([d, h] memory) are re-laid, gradients keep the caller's strides
    Wc = {k: v.T.contiguous() for k, v in w.W.items()}
    c = masked_ffn_backward(g, w.x, Wc["w1"], Wc["w2"], Wc["w3"], Wc["u1"], Wc["u2"], Wc["u3"], w.mask)
    assert c[1].is_contiguous() and c[1].shape == (128, 256)
    for ta, tc in zip(a, c):
        assert_close_bf16_pair(tc, ta.float().cpu(), "layout variant")
    with pytest.raises(ValueError):
        masked_ffn_backward(g[:, :100], w.x, *args[2:])
    bad = wl.make_ffn("t", 8, 60, 64, torch.ones(8, dtype=torch.bool), seed=1).to(dev)
    with pytest.raises(ValueError):
        masked_ffn_backward(bad.x, bad.x, *[bad.W[k].T for k in ("w1", "w2", "w3", "u1", "u2", "u3")], bad.mask)


# ------------------------------------------------------------------ MaskedLinear backward
BWD_SHAPES = [
    (37, 48, 40, 0.5),
    (64, 64, 64, 1.0),        # no text rows: dW_t must be exact zeros
    (64, 64, 64, 0.0),
    (300, 128, 136, 0.5),
    (1000, 256, 320, 0.3),
    (2048, 1024, 1024, 0.5),
    (50, 30, 17, 0.5),        # generic path
]


@pytest.mark.parametrize("M,K,N,p", BWD_SHAPES)
def test_linear_bwd_vs_oracle(dev, M, K, N, p):
    note(f"linear bwd M={M} K={K} N={N} p={p}")
    gen = torch.Generator().manual_seed(M + K + N + 1)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_linear("t", M, K, N, mask, seed=M + 1, with_grad=True, w_std=0.05)
    d = w.to(dev)
    x = d.x.clone().requires_grad_(True)
    Wv = d.Wv.clone().requires_grad_(True)
    Wt = d.Wt.clone().requires_grad_(True)
    y = MaskedLinear.apply(x, Wv.T, Wt.T, d.mask)
    y.backward(d.grad)
    torch.cuda.synchronize()
    dx, dWv, dWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    assert x.grad.shape == (M, K) and Wv.grad.shape == (N, K) and Wv.grad.is_contiguous()
    assert_close(x.grad, dx, "dx")
    assert_close(Wv.grad, dWv, "dWv")
    assert_close(Wt.grad, dWt, "dWt")
    if p == 1.0:
        assert (Wt.grad == 0).all()
    if p == 0.0:
        assert (Wv.grad == 0).all()


def test_linear_bwd_is_deterministic(dev):
    note("linear bwd determinism")
    w = wl.make_linear("t", 1500, 256, 256, torch.rand(1500, generator=torch.Generator().manual_seed(0)) < 0.5,
                       seed=3, with_grad=True).to(dev)
    outs = []
    for _ in range(3):
        from ffn_kernel_amd import masked_linear_backward
        outs.append(masked_linear_backward(w.grad, w.x, w.Wv.T, w.Wt.T, w.mask))
    for o in outs[1:]:
        for a, b in zip(outs[0], o):
            assert torch.equal(a, b)


def test_linear_bwd_cfg3(dev):
    note("linear bwd cfg3")
    w = wl.cfg3_linear_bwd()
    d = w.to(dev)
    from ffn_kernel_amd import masked_linear_backward
    dx, dbv, dbt = masked_linear_backward(d.grad, d.x, d.Wv.T, d.Wt.T, d.mask)
    rdx, rdWv, rdWt = om.linear_backward_select(w.grad, w.x, w.Wv, w.Wt, w.mask, torch.float64)
    assert_close(dx, rdx, "dx")
    assert_close(dbv.T, rdWv, "dWv")
    assert_close(dbt.T, rdWt, "dWt")
    # invariant: dW_v + dW_t is the unmasked x^T g
    # (each term carries its own bf16 rounding, half an ulp = 2^-9 relative)
    tot = (w.grad.double().T @ w.x.double())
    gv, gt = dbv.T.double().cpu(), dbt.T.double().cpu()
    assert ((gv + gt - tot).abs() <= 2.0 ** -8 * (gv.abs() + gt.abs()) + 1e-6).all()


# ------------------------------------------------------------------ nn.Module wrappers (3-D inputs)
def test_modules_match_reference_modules(dev):
    """The wrappers load the reference PyTorch modules' state_dicts and reproduce them on [B, S, D]
    inputs, forward (both) and backward (linear), as test_linear.py:92-102 compares them."""
    note("module wrappers")
    from ffn_kernel_amd import MaskedFFNModule, MaskedLinearModule
    torch.manual_seed(0)
    B, S, D, Hh = 2, 150, 64, 128
    x = torch.randn(B, S, D).to(torch.bfloat16)
    mask = torch.rand(B, S) < 0.4
    ref_lin = om.TorchLinear(D, 96).bfloat16()
    mod = MaskedLinearModule(D, 96, device=dev)
    mod.load_state_dict(ref_lin.state_dict())
    xd = x.to(dev).requires_grad_(True)
    y = mod(xd, mask.to(dev))
    assert y.shape == (B, S, 96)
    y.sum().backward()
    xr = x.float().requires_grad_(True)
    ref = om.TorchLinear(D, 96)
    ref.load_state_dict({k: v.float() for k, v in ref_lin.state_dict().items()})
    yr = ref(xr, mask)
    yr.sum().backward()
    assert_close(y, yr.detach().double(), "module y")
    assert_close(xd.grad, xr.grad.double(), "module dx")
    assert_close(mod.linear_v.weight.grad, ref.linear_v.weight.grad.double(), "module dWv")
    assert_close(mod.linear_t.weight.grad, ref.linear_t.weight.grad.double(), "module dWt")
    ref_ffn = om.TorchFFN(D, Hh).bfloat16()
    ffn = MaskedFFNModule(D, Hh, device=dev)
    ffn.load_state_dict(ref_ffn.state_dict())
    out = ffn(x.to(dev), mask.to(dev))
    assert out.shape == (B, S, D)
    assert_close_bf16_pair(out, ref_ffn(x, mask).float(), "module ffn vs reference module")
    out2 = ffn(x.to(dev).flatten(0, 1), mask.to(dev).flatten())
    assert torch.equal(out2, out.flatten(0, 1))
    # the FFN module trains: gradients of its parameters against the exact chain rule
    g = torch.randn(B, S, D, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    xf = x.to(dev).requires_grad_(True)
    ffn.zero_grad(set_to_none=True)
    ffn(xf, mask.to(dev)).backward(g.to(dev))
    W = {k: getattr(ref_ffn, k).weight.detach() for k in ("w1", "w2", "w3", "u1", "u2", "u3")}
    dx, dW = om.ffn_backward_select(g.flatten(0, 1), x.flatten(0, 1), W, mask.flatten(), torch.float64,
                                    round_intermediates=True)
    assert_close_pipeline(xf.grad.flatten(0, 1), dx, "module ffn dx")
    for k in W:
        assert_close_pipeline(getattr(ffn, k).weight.grad, dW[k], f"module ffn d{k}")


# ------------------------------------------------------------------ HIP graph capture
@pytest.mark.parametrize("M,d,h", [(8, 1024, 2048), (40, 1024, 2048), (300, 256, 1024), (1500, 512, 512)])
def test_ffn_forward_is_graph_capturable(dev, M, d, h):
    """The entry points only enqueue kernels on the given stream (no allocation, memset, copy or sync),
    so a call can be captured into a HIP graph and replayed; every replay is checked against an eager
    call on the same inputs, with eager work in between."""
    note(f"ffn forward under graph capture M={M} d={d} h={h}")
    gen = torch.Generator().manual_seed(M)
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_ffn("t", M, d, h, mask, seed=M + 5, w_std=0.05).to(dev)
    x_static = w.x.clone()
    args = (x_static,) + w.op_args()[1:]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            MaskedFFN.apply(*args)  # warm-up outside capture (library load, allocator pools)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = MaskedFFN.apply(*args)
    for rep in range(3):
        x_new = (torch.randn(M, d, generator=gen) * (rep + 1)).to(torch.bfloat16).to(dev)
        x_static.copy_(x_new)
        graph.replay()
        torch.cuda.synchronize()
        eager = MaskedFFN.apply(x_new, *w.op_args()[1:])
        torch.cuda.synchronize()
        assert torch.equal(out_static, eager), rep


@pytest.mark.parametrize("M,K,N", [(4100, 1024, 384), (900, 256, 512)])
def test_linear_forward_and_backward_are_graph_capturable(dev, M, K, N):
    """MaskedLinear forward and backward (the in-place weight-gradient form with its reduce pass, the row partition
    made inside the captured region) captured into one HIP graph: every replay against eager calls on the same inputs,
    with eager work in between."""
    note(f"linear fwd + bwd under graph capture M={M} K={K} N={N}")
    from ffn_kernel_amd.ops import masked_linear_forward
    gen = torch.Generator().manual_seed(M + 3)
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_linear("t", M, K, N, mask, seed=M + 5, with_grad=True, w_std=0.05).to(dev)
    x_static, g_static = w.x.clone(), w.grad.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):  # warm-up outside capture (library load, allocator pools)
            masked_linear_forward(x_static, w.Wv.T, w.Wt.T, w.mask)
            masked_linear_backward(g_static, x_static, w.Wv.T, w.Wt.T, w.mask)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_static = masked_linear_forward(x_static, w.Wv.T, w.Wt.T, w.mask)
        grads_static = masked_linear_backward(g_static, x_static, w.Wv.T, w.Wt.T, w.mask)
    for rep in range(3):
        x_new = (torch.randn(M, K, generator=gen) * (rep + 1)).to(torch.bfloat16).to(dev)
        g_new = torch.randn(M, N, generator=gen).to(torch.bfloat16).to(dev)
        x_static.copy_(x_new)
        g_static.copy_(g_new)
        graph.replay()
        torch.cuda.synchronize()
        y = masked_linear_forward(x_new, w.Wv.T, w.Wt.T, w.mask)
        grads = masked_linear_backward(g_new, x_new, w.Wv.T, w.Wt.T, w.mask)
        torch.cuda.synchronize()
        assert torch.equal(y_static, y), rep
        for a, b in zip(grads_static, grads):
            assert torch.equal(a, b), rep


def test_ffn_forward_keeps_pre_activations_only_when_a_backward_can_follow(dev, monkeypatch):
    note("ffn save_pre decision")
    from ffn_kernel_amd import ops
    seen = []
    real = ops.masked_ffn_forward
    def spy(*args, save_pre=False, **kw):
        seen.append(save_pre)
        return real(*args, save_pre=save_pre, **kw)
    monkeypatch.setattr(ops, "masked_ffn_forward", spy)
    mask = torch.rand(200, generator=torch.Generator().manual_seed(1)) < 0.5
    w = wl.make_ffn("t", 200, 128, 256, mask, seed=2, w_std=0.05).to(dev)
    args = w.op_args()
    MaskedFFN.apply(*args)                                   # nothing requires grad
    x = args[0].clone().requires_grad_(True)
    with torch.no_grad():
        MaskedFFN.apply(x, *args[1:])                        # evaluation with trainable inputs
    out = MaskedFFN.apply(x, *args[1:])                      # training
    out.sum().backward()
    assert seen == [False, False, True] and x.grad is not None


# ------------------------------------------------------------------ every compiled tile, forced
@pytest.fixture
def force_tile():
    """ffnk_debug_force_tile for the duration of one test; always back to the tile table afterwards."""
    lib = _lib.load()
    try:
        yield lib.ffnk_debug_force_tile
    finally:
        lib.ffnk_debug_force_tile(-1)


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("M,K,N,p", [(700, 256, 512, 0.5), (333, 192, 320, 0.3), (1100, 1024, 264, 1.0), (500, 200, 264, 0.5)])
def test_forced_tile_linear_fwd_bwd(dev, force_tile, tile, M, K, N, p):
    """Each of the four tile shapes every GEMM family is compiled for (256x256 with 8 or 4 waves,
    128x128, 128x64, 128x128 behind a four-stage ring) runs the MaskedLinear forward and backward: the table alone never picks all of
    them at test sizes."""
    note(f"forced tile {tile}: linear fwd+bwd M={M} K={K} N={N} p={p}")
    gen = torch.Generator().manual_seed(M + tile)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_linear("t", M, K, N, mask, seed=M + K, with_grad=True, w_std=0.05)
    dw = w.to(dev)
    force_tile(tile)
    y = MaskedLinear.apply(dw.x, dw.Wv.T, dw.Wt.T, dw.mask)
    dx, dWv, dWt = masked_linear_backward(dw.grad, dw.x, dw.Wv.T, dw.Wt.T, dw.mask)
    torch.cuda.synchronize()
    force_tile(-1)
    assert_close(y, cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask), "y")
    rdx, rdWv, rdWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    assert_close(dx, rdx, "dx")
    assert_close(dWv.T, rdWv, "dWv")
    assert_close(dWt.T, rdWt, "dWt")
    if p == 1.0:
        assert torch.count_nonzero(dWt) == 0


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("M,d,h,p", [(700, 256, 512, 0.5), (300, 128, 320, 0.4),
                                     (70, 128, 192, 0.5),     # one ragged slab of contraction rows per modality
                                     (180, 192, 256, 0.45)])  # two, the second ragged
def test_forced_tile_ffn_fwd_bwd(dev, force_tile, tile, M, d, h, p):
    note(f"forced tile {tile}: ffn fwd+bwd M={M} d={d} h={h}")
    gen = torch.Generator().manual_seed(M + tile)
    mask = torch.rand(M, generator=gen) < p
    w = wl.make_ffn("t", M, d, h, mask, seed=M + 3, w_std=0.05)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    dw = w.to(dev)
    force_tile(tile)
    out, pre = masked_ffn_forward(*dw.op_args(), save_pre=True)
    grads_saved = masked_ffn_backward(g.to(dev), *dw.op_args(), pre=pre)
    grads = masked_ffn_backward(g.to(dev), *dw.op_args())
    torch.cuda.synchronize()
    force_tile(-1)
    assert_close(out, cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True), "ffn out")
    rdx, rdW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64, round_intermediates=True)
    for got in (grads, grads_saved):
        assert_close_pipeline(got[0], rdx, "dx")
        for i, k in enumerate(("w1", "w2", "w3", "u1", "u2", "u3")):
            assert_close_pipeline(got[1 + i].T, rdW[k], f"d{k}")


def test_ffn_fwd_bwd_on_unaligned_views(dev):
    """x and the upstream gradient as column slices of wider tensors whose row stride is not a multiple
    of 8 elements and whose first element is not 16-byte aligned: the ops copy such views (as the
    reference's .contiguous() calls do) instead of handing them to a kernel that cannot address them."""
    note("ffn fwd+bwd on unaligned column-sliced x and grad")
    M, d, h = 300, 256, 512
    gen = torch.Generator().manual_seed(77)
    mask = torch.rand(M, generator=gen) < 0.5
    w = wl.make_ffn("t", M, d, h, mask, seed=78, w_std=0.05)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    dw = w.to(dev)
    wide_x = torch.zeros(M, d + 100, dtype=torch.bfloat16, device=dev)
    wide_x[:, 4:4 + d] = dw.x
    wide_g = torch.zeros(M, d + 36, dtype=torch.bfloat16, device=dev)
    wide_g[:, 3:3 + d] = g.to(dev)
    x = wide_x[:, 4:4 + d].detach().requires_grad_(True)
    Wp = {k: v.clone().requires_grad_(True) for k, v in dw.W.items()}
    out = MaskedFFN.apply(x, Wp["w1"].T, Wp["w2"].T, Wp["w3"].T, Wp["u1"].T, Wp["u2"].T, Wp["u3"].T, dw.mask)
    out.backward(wide_g[:, 3:3 + d])
    torch.cuda.synchronize()
    assert_close(out, cref.ffn_fwd(w.x, w.W, w.mask, round_mid=True), "out")
    rdx, rdW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64, round_intermediates=True)
    assert_close_pipeline(x.grad, rdx, "dx")
    for k in rdW:
        assert_close_pipeline(Wp[k].grad, rdW[k], f"d{k}")
    # the same views through MaskedLinear: forward and backward stay on the MFMA path's results
    lw = wl.make_linear("t", M, d, 192, mask, seed=79, with_grad=True, w_std=0.05)
    dl = lw.to(dev)
    wide_x[:, 4:4 + d] = dl.x
    wide_gl = torch.zeros(M, 192 + 4, dtype=torch.bfloat16, device=dev)
    wide_gl[:, 1:193] = dl.grad
    y = MaskedLinear.apply(wide_x[:, 4:4 + d], dl.Wv.T, dl.Wt.T, dl.mask)
    dx, dWv, dWt = masked_linear_backward(wide_gl[:, 1:193], wide_x[:, 4:4 + d], dl.Wv.T, dl.Wt.T, dl.mask)
    assert_close(y, cref.linear_fwd(lw.x, lw.Wv, lw.Wt, lw.mask), "linear y")
    rdx, rdWv, rdWt = cref.linear_bwd(lw.grad, lw.x, lw.Wv, lw.Wt, lw.mask)
    assert_close(dx, rdx, "linear dx")
    assert_close(dWv.T, rdWv, "linear dWv")
    assert_close(dWt.T, rdWt, "linear dWt")


@pytest.mark.parametrize("M,K,N,p", [(4100, 1024, 384, 0.5), (4100, 1024, 384, 1.0), (4100, 1024, 384, 0.0), (8300, 1024, 1024, 0.3)])
def test_linear_bwd_fused_launch(dev, M, K, N, p):
    """Shapes whose dx and weight-gradient GEMMs both run on 128x128 tiles share one launch (dx tiles
    behind the weight-gradient tiles): gradients against the oracle, exact zeros for an absent modality,
    bit-identical on a second call."""
    note(f"linear bwd fused launch M={M} K={K} N={N} p={p}")
    assert _lib.tile_config(_lib.OP_BWD_DX, M, K, N)["block_m"] == 128 and _lib.tile_config(_lib.OP_BWD_DX, M, K, N)["block_n"] == 128
    assert _lib.tile_config(_lib.OP_BWD_DW, M, K, N)["block_m"] == 128
    gen = torch.Generator().manual_seed(M + N)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_linear("t", M, K, N, mask, seed=M, with_grad=True, w_std=0.05)
    d = w.to(dev)
    dx, dWv, dWt = masked_linear_backward(d.grad, d.x, d.Wv.T, d.Wt.T, d.mask)
    rdx, rdWv, rdWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    assert_close(dx, rdx, "dx")
    assert_close(dWv.T, rdWv, "dWv")
    assert_close(dWt.T, rdWt, "dWt")
    if p == 1.0:
        assert torch.count_nonzero(dWt) == 0
    if p == 0.0:
        assert torch.count_nonzero(dWv) == 0
    again = masked_linear_backward(d.grad, d.x, d.Wv.T, d.Wt.T, d.mask)
    for a, b in zip((dx, dWv, dWt), again):
        assert torch.equal(a, b)


@pytest.mark.parametrize("group_m", [1, 2, 16])
def test_forced_super_group_size(dev, group_m):
    """The tile order is a permutation of the same tiles for every super-group size (ffnk_debug_force_group_m), also
    where the launch is cut into whole rounds and a remainder: MaskedLinear and MaskedFFN forward against the oracle
    on shapes with more than 256 tiles of 256 rows, and the reduce pass of a split tail walks the same order."""
    note(f"forced group_m={group_m}")
    lib = _lib.load()
    M, K, N = 8300, 128, 2304
    mask = torch.rand(M, generator=torch.Generator().manual_seed(11)) < 0.45
    wlin = wl.make_linear("t", M, K, N, mask, seed=12, w_std=0.05)
    wffn = wl.make_ffn("t", M, 128, 1152, mask, seed=13, w_std=0.05)
    dl, df = wlin.to(dev), wffn.to(dev)
    try:
        lib.ffnk_debug_force_group_m(group_m)
        lib.ffnk_debug_force_tile(0)
        assert _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)["group_m"] == group_m
        y = MaskedLinear.apply(dl.x, dl.Wv.T, dl.Wt.T, dl.mask)
        out = MaskedFFN.apply(df.x, *[df.W[k].T for k in ("w1", "w2", "w3", "u1", "u2", "u3")], df.mask)
        torch.cuda.synchronize()
    finally:
        lib.ffnk_debug_force_group_m(0)
        lib.ffnk_debug_force_tile(-1)
    assert_close(y, cref.linear_fwd(wlin.x, wlin.Wv, wlin.Wt, wlin.mask), "linear fwd")
    assert_close(out, cref.ffn_fwd(wffn.x, wffn.W, wffn.mask, round_mid=True), "ffn fwd")


@pytest.fixture
def force_bwd_form():
    """ffnk_debug_force_bwd_gather / ffnk_debug_force_splits for one test; back to the plans afterwards."""
    lib = _lib.load()

    def force(in_place, splits):
        lib.ffnk_debug_force_bwd_gather(in_place)
        lib.ffnk_debug_force_splits(splits)
    try:
        yield force
    finally:
        lib.ffnk_debug_force_bwd_gather(-1)
        lib.ffnk_debug_force_splits(-1)


@pytest.mark.parametrize("splits", [-1, 1, 3])
@pytest.mark.parametrize("in_place", [0, 1])
@pytest.mark.parametrize("M,K,N,p,layout", [
    (37, 48, 40, 0.5, "views"),          # one ragged slab per modality, ragged tiles
    (300, 128, 136, 0.5, "views"),
    (1000, 256, 320, 0.3, "kn"),         # weights stored [K, N]: the gradients' memory is [K, N] as well
    (777, 136, 200, 0.0, "views"),       # no visual rows
    (515, 128, 128, 1.0, "kn"),          # no text rows
    (4100, 1024, 384, 0.5, "views"),     # one launch for both GEMMs
    (2500, 512, 1024, 0.6, "strided"),   # g and x are column slices of wider tensors
])
def test_linear_bwd_weight_gradients_in_place_and_from_transposes(dev, force_bwd_form, in_place, splits, M, K, N, p, layout):
    """The weight-gradient GEMM has two forms - g and x read where they lie (rows found through the partition), or
    routed transposes written first - and each runs split or unsplit: every combination against the oracle, exact
    zeros for an absent modality, bit-identical on a second call."""
    note(f"linear bwd forms in_place={in_place} splits={splits} M={M} K={K} N={N} p={p} {layout}")
    gen = torch.Generator().manual_seed(M + N + 7)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_linear("t", M, K, N, mask, seed=M + 2, with_grad=True, w_std=0.05)
    d = w.to(dev)
    g, x = d.grad, d.x
    if layout == "strided":
        gw_, xw_ = torch.full((M, N + 24), float("nan"), device=dev, dtype=torch.bfloat16), torch.full(
            (M, K + 40), float("nan"), device=dev, dtype=torch.bfloat16)
        gw_[:, 8:8 + N] = g
        xw_[:, 16:16 + K] = x
        g, x = gw_[:, 8:8 + N], xw_[:, 16:16 + K]
    if layout == "kn":
        b1, b2 = d.Wv.T.contiguous(), d.Wt.T.contiguous()
    else:
        b1, b2 = d.Wv.T, d.Wt.T
    force_bwd_form(in_place, splits)
    assert _lib.tile_config(_lib.OP_BWD_DW, M, K, N)["in_place"] == in_place
    dx, db1, db2 = masked_linear_backward(g, x, b1, b2, d.mask)
    again = masked_linear_backward(g, x, b1, b2, d.mask)
    force_bwd_form(-1, -1)
    torch.cuda.synchronize()
    assert db1.stride() == b1.stride()
    rdx, rdWv, rdWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    assert_close(dx, rdx, "dx")
    assert_close(db1.T, rdWv, "dWv")
    assert_close(db2.T, rdWt, "dWt")
    if p == 1.0:
        assert torch.count_nonzero(db2) == 0
    if p == 0.0:
        assert torch.count_nonzero(db1) == 0
    for a, b in zip((dx, db1, db2), again):
        assert torch.equal(a, b)


def test_linear_bwd_forms_on_random_shapes(dev, force_bwd_form):
    """Both forms of the weight-gradient GEMM on 24 seeded random shapes (single rows, groups shorter than a slab,
    K and N below a tile, padded row strides, masks from all-text to all-visual) against the row-select form in
    double precision computed with torch on the GPU."""
    gen = torch.Generator().manual_seed(2024)

    def rnd(lo, hi):
        return int(torch.randint(lo, hi + 1, (1,), generator=gen))
    for case in range(24):
        M = (1, 2, 63, 65)[case] if case < 4 else rnd(3, 3000)
        K, N = 8 * rnd(1, 65), 8 * rnd(1, 65)
        p = (0.0, 1.0, 0.5, 0.02, 0.98)[case % 5]
        pad_g, pad_x = 8 * rnd(0, 2), 8 * rnd(0, 2)
        note(f"linear bwd random case {case}: M={M} K={K} N={N} p={p} pads {pad_g} {pad_x}")
        mask = (torch.rand(M, generator=gen) < p).to(dev)
        gw_ = (torch.randn(M, N + pad_g, generator=gen)).to(torch.bfloat16).to(dev)
        xw_ = (torch.randn(M, K + pad_x, generator=gen)).to(torch.bfloat16).to(dev)
        g, x = gw_[:, :N], xw_[:, :K]
        Wv = (torch.randn(N, K, generator=gen) * 0.05).to(torch.bfloat16).to(dev)
        Wt = (torch.randn(N, K, generator=gen) * 0.05).to(torch.bfloat16).to(dev)
        gd, xd = g.double(), x.double()
        mv = mask.double()[:, None]
        ref_dx = torch.where(mask[:, None], gd @ Wv.double(), gd @ Wt.double()).cpu()
        ref_dwv = ((gd * mv).T @ xd).cpu()          # [N, K]
        ref_dwt = ((gd * (1 - mv)).T @ xd).cpu()
        for in_place in (0, 1):
            force_bwd_form(in_place, -1)
            dx, dbv, dbt = masked_linear_backward(g, x, Wv.T, Wt.T, mask)
            force_bwd_form(-1, -1)
            assert_close(dx, ref_dx, f"case {case} form {in_place} dx")
            assert_close(dbv.T, ref_dwv, f"case {case} form {in_place} dWv")
            assert_close(dbt.T, ref_dwt, f"case {case} form {in_place} dWt")
            if not bool(mask.any()):
                assert torch.count_nonzero(dbv) == 0
            if bool(mask.all()):
                assert torch.count_nonzero(dbt) == 0


@pytest.mark.parametrize("in_place", [0, 1])
def test_linear_bwd_non_finite_rows_stay_in_their_modality(dev, force_bwd_form, in_place):
    """Inf / NaN in the text rows of g and x reach dW_t only: the visual gradient is what it is without them, also
    where a slab of 64 contraction rows holds the end of one modality (rows past it are cleared, not multiplied by 0)."""
    note(f"linear bwd non-finite isolation in_place={in_place}")
    M, K, N = 1000, 256, 192
    mask = torch.rand(M, generator=torch.Generator().manual_seed(5)) < 0.4
    w = wl.make_linear("t", M, K, N, mask, seed=9, with_grad=True, w_std=0.05)
    d = w.to(dev)
    g, x = d.grad.clone(), d.x.clone()
    text = (~d.mask).nonzero().flatten()
    g[text[::3], ::5] = float("inf")
    x[text[1::3], ::7] = float("nan")
    x[text[2::3], 1::7] = float("-inf")
    force_bwd_form(in_place, -1)
    _, clean_v, _ = masked_linear_backward(d.grad, d.x, d.Wv.T, d.Wt.T, d.mask)
    dx, dWv, dWt = masked_linear_backward(g, x, d.Wv.T, d.Wt.T, d.mask)
    force_bwd_form(-1, -1)
    assert torch.equal(dWv, clean_v)
    assert torch.isfinite(dx[d.mask]).all()
    assert not torch.isfinite(dWt).all()


@pytest.mark.parametrize("M,d,h,layout", [(300, 256, 512, "views"), (2100, 512, 1024, "views"), (4100, 256, 1024, "views"),
                                          (300, 256, 512, "down_contig"), (333, 72, 200, "views"),
                                          (500, 128, 96, "views")])
def test_ffn_bwd_lean_workspace_is_enough_and_changes_nothing(dev, M, d, h, layout, monkeypatch):
    """The backward sizes its workspace for the layout at hand (ffnk_workspace_bytes_ffn_bwd): never more than the
    any-layout size, nothing written past its end (guard bytes behind it stay intact), and gradients bit-identical
    to a run on the any-layout workspace."""
    from ffn_kernel_amd import ops
    note(f"ffn bwd lean workspace M={M} d={d} h={h} {layout}")
    gen = torch.Generator().manual_seed(M + d)
    mask = (torch.rand(M, generator=gen) < 0.5).to(dev)
    w = wl.make_ffn("t", M, d, h, mask.cpu(), seed=M + 7, w_std=0.05).to(dev)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16).to(dev)
    Wt = {k: v.T for k, v in w.W.items()}
    if layout == "down_contig":
        Wt["w2"], Wt["u2"] = Wt["w2"].contiguous(), Wt["u2"].contiguous()
    args = (g, w.x, Wt["w1"], Wt["w2"], Wt["w3"], Wt["u1"], Wt["u2"], Wt["u3"], mask)
    sizes, guards = [], []
    real_workspace = ops._workspace

    def guarded(nbytes, device):
        t = torch.empty(max(nbytes, 16) + 4096, dtype=torch.uint8, device=device)
        t[max(nbytes, 16):] = 0xA5
        sizes.append(nbytes)
        guards.append(t)
        return t[:max(nbytes, 16)]

    monkeypatch.setattr(ops, "_workspace", guarded)
    lean = ops.masked_ffn_backward(*args)
    torch.cuda.synchronize()
    worst = _lib.workspace_bytes(_lib.OP_FFN_BWD, M, d, h)
    assert len(sizes) == 1 and sizes[0] <= worst
    assert bool((guards[0][max(sizes[0], 16):] == 0xA5).all()), "the backward wrote past its workspace"
    # the same call on the any-layout workspace
    monkeypatch.setattr(ops, "_workspace", real_workspace)
    lib = _lib.load()
    monkeypatch.setattr(lib, "ffnk_workspace_bytes_ffn_bwd", lambda *a: worst, raising=False)
    ref = ops.masked_ffn_backward(*args)
    torch.cuda.synchronize()
    for a, b, name in zip(lean, ref, ("da", "dw1", "dw2", "dw3", "du1", "du2", "du3")):
        assert torch.equal(a, b), name
    if d % 64 == 0 and h % 64 == 0:
        assert sizes[0] < worst  # weights and intermediates read in place: no room for copies or transposes


# ------------------------------------------------------------------ one row partition shared by several calls
def _count_route_launches(monkeypatch):
    """Count the partitions made from Python (ops.route) while the block runs."""
    from ffn_kernel_amd import ops
    calls = []
    real = ops.route
    monkeypatch.setattr(ops, "route", lambda mask: (calls.append(mask.shape[0]), real(mask))[1])
    return calls


def test_routing_is_shared_between_the_calls_of_a_layer_and_with_the_backward(dev, monkeypatch):
    """The operations of a layer run with one mask: the partition is made once (ops.shared_routing) and handed
    to every call through the *_routed entry points; a forward's partition serves its backward.  Results are
    those of calls that each partition the rows themselves, bit for bit."""
    note("shared routing: linear fwd + bwd + ffn fwd + bwd on one mask")
    from ffn_kernel_amd import ops
    M, K, N, d, h = 700, 256, 384, 256, 512
    gen = torch.Generator().manual_seed(41)
    mask = (torch.rand(M, generator=gen) < 0.4).to(dev)
    lw = wl.make_linear("l", M, K, N, mask.cpu(), seed=42, with_grad=True).to(dev)
    fw = wl.make_ffn("f", M, d, h, mask.cpu(), seed=43).to(dev)

    def layer():
        x = lw.x.clone().requires_grad_(True)
        y = MaskedLinear.apply(x, lw.Wv.T, lw.Wt.T, mask)
        y.backward(lw.grad)
        xf = fw.x.clone().requires_grad_(True)
        o = MaskedFFN.apply(xf, *fw.op_args()[1:7], mask)
        o.backward(torch.ones_like(o))
        return y.detach(), x.grad, o.detach(), xf.grad

    old = ops.set_route_cache(False)
    try:
        want = layer()
    finally:
        ops.set_route_cache(old)
    ops.set_route_cache(False)
    ops.set_route_cache(True)  # start from an empty cache
    calls = _count_route_launches(monkeypatch)
    got = layer()
    assert calls == [M], f"one partition for the whole layer, got {calls}"
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    # an explicit partition works the same and bypasses the cache
    r = ops.route(mask)
    assert torch.equal(ops.masked_linear_forward(lw.x, lw.Wv.T, lw.Wt.T, mask, routing=r), want[0])
    with pytest.raises(ValueError, match="rows"):
        ops.masked_linear_forward(lw.x[:600], lw.Wv.T, lw.Wt.T, mask[:600], routing=r)


def test_a_mask_changed_in_place_is_partitioned_again(dev, monkeypatch):
    """The shared partition is keyed on the mask's memory, view and version counter: a write into the mask,
    a different view of it, or another mask at the same extents each get their own partition, and the results
    follow the mask as it is at the time of the call."""
    note("shared routing: stale partitions cannot be hit")
    from ffn_kernel_amd import ops
    M, K, N = 900, 128, 256
    gen = torch.Generator().manual_seed(51)
    mask = (torch.rand(M, generator=gen) < 0.5).to(dev)
    w = wl.make_linear("l", M, K, N, mask.cpu(), seed=52).to(dev)

    def ref(m):
        return torch.where(m[:, None], w.x.float() @ w.Wv.float().T, w.x.float() @ w.Wt.float().T).double().cpu()

    ops.set_route_cache(False)
    ops.set_route_cache(True)
    calls = _count_route_launches(monkeypatch)
    assert_close(MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, mask), ref(mask), "first mask")
    MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, mask)
    assert len(calls) == 1
    mask[:300] = ~mask[:300]                      # in place: same memory, new version
    assert_close(MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, mask), ref(mask), "mask changed in place")
    assert len(calls) == 2
    other = ~mask                                  # another tensor
    assert_close(MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, other), ref(other), "another mask")
    assert len(calls) == 3
    both = torch.cat([mask, other])
    view = both[M:]                                # same storage as `both`, other offset
    assert_close(MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, both[:M]), ref(mask), "view at offset 0")
    assert_close(MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, view), ref(other), "view at offset M")
    assert len(calls) == 5
    # decode sizes never share a partition (the streaming kernels read the mask themselves)
    MaskedLinear.apply(w.x[:40], w.Wv.T, w.Wt.T, mask[:40])
    assert len(calls) == 5


def test_routed_entry_points_reject_half_a_partition(dev):
    note("ffnk_masked_linear_fwd_routed with perm but no counts")
    lib = _lib.load()
    M, K, N = 128, 64, 64
    x = torch.zeros(M, K, device=dev, dtype=torch.bfloat16)
    W = torch.zeros(N, K, device=dev, dtype=torch.bfloat16)
    y = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    mask = torch.zeros(M, dtype=torch.bool, device=dev)
    perm = torch.zeros(M, dtype=torch.int32, device=dev)
    ws = torch.empty(_lib.workspace_bytes(_lib.OP_LINEAR_FWD, M, K, N), dtype=torch.uint8, device=dev)
    half = _lib.RoutingStruct(perm.data_ptr(), None)
    rc = lib.ffnk_masked_linear_fwd_routed(x.data_ptr(), K, W.data_ptr(), W.data_ptr(), 1, K, mask.data_ptr(), y.data_ptr(),
                                           N, M, K, N, ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream,
                                           ctypes.byref(half))
    assert rc == -1  # FFNK_E_NULL
