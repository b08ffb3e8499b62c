"""Full-size GPU checks (the sizes the benchmarks run at), through properties that do not need a
full-size CPU reference: routing vs numpy, exact row spot checks against the C oracle, batch-
composition invariance, uniform-mask sequences against a plain fp32 library matmul, exact scaling,
and decode vs tiled-path agreement."""
import numpy as np
import pytest
import torch

from ffn_kernel_amd import MaskedFFN, MaskedLinear, _lib
from ffn_kernel_amd import workloads as wl
from oracle import cref
from oracle import modules as om
from helpers import assert_close, assert_close_bf16_pair, note

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cfg4(dev):
    note("building cfg4 workload (M=32768, d=4096, h=14336)")
    w = wl.cfg4_ffn_fwd()
    d = w.to(dev)
    out = MaskedFFN.apply(*d.op_args())
    torch.cuda.synchronize()
    return w, d, out


def test_cfg4_routing_bit_exact(dev, cfg4):
    w, d, _ = cfg4
    M = w.x.shape[0]
    perm = torch.empty(M, dtype=torch.int32, device=dev)
    counts = torch.empty(2, dtype=torch.int32, device=dev)
    _lib.check(_lib.load().ffnk_route(d.mask.data_ptr(), M, perm.data_ptr(), counts.data_ptr(),
                                      torch.cuda.current_stream().cuda_stream), "ffnk_route")
    perm_ref, counts_ref = om.stable_partition(w.mask.numpy())
    assert np.array_equal(perm.cpu().numpy(), perm_ref) and counts.cpu().tolist() == counts_ref.tolist()


def test_cfg4_rows_against_c_oracle(cfg4):
    """24 rows (visual and text, including tile edges of both groups) recomputed in double precision."""
    note("cfg4 row spot check")
    w, _, out = cfg4
    gen = torch.Generator().manual_seed(7)
    nv = int(w.mask.sum())
    vis = torch.nonzero(w.mask).flatten()
    txt = torch.nonzero(~w.mask).flatten()
    rows = torch.cat([vis[[0, 255, 256, nv - 1]], txt[[0, 255, 256, len(txt) - 1]],
                      torch.randint(0, w.x.shape[0], (16,), generator=gen)])
    sub = wl.FFNWorkload("rows", w.x[rows].contiguous(), w.W, w.mask[rows].contiguous())
    ref = cref.ffn_fwd(sub.x, sub.W, sub.mask, round_mid=True)
    rep = assert_close(out[rows.to(out.device)], ref, "cfg4 rows")
    print("cfg4 row error:", rep)


def test_cfg4_batch_composition_invariance(dev, cfg4):
    """A row's result does not depend on which other rows share the call: two sequences, or one, alone
    (another tile schedule) reproduce their rows of the full call - bit for bit wherever the K order is
    shared, i.e. everywhere except the few tiles of a call's last, partial round, which are summed in K
    ranges; those, and a quarter sequence (1024 rows, whose whole down projection is split over K),
    agree to bf16 accuracy."""
    note("cfg4 batch invariance")
    w, d, out = cfg4
    for rows in (8192, 4096):
        assert _lib.tile_config(_lib.OP_FFN_DOWN, rows, w.d, w.h)["split_k"] == 1
    for sl in (slice(0, 8192), slice(5 * 4096, 7 * 4096), slice(3 * 4096, 4 * 4096)):
        sub = wl.FFNWorkload("seq", d.x[sl].contiguous(), d.W, d.mask[sl].contiguous())
        part = MaskedFFN.apply(*sub.op_args())
        same_rows = (part == out[sl]).all(dim=1).float().mean().item()
        assert same_rows >= 0.85, same_rows
        assert_close_bf16_pair(part, out[sl].float().cpu(), "one or two sequences vs the full call")
    assert _lib.tile_config(_lib.OP_FFN_DOWN, 1024, w.d, w.h)["split_k"] > 1
    sl = slice(3 * 4096, 3 * 4096 + 1024)
    sub = wl.FFNWorkload("seq", d.x[sl].contiguous(), d.W, d.mask[sl].contiguous())
    part = MaskedFFN.apply(*sub.op_args())
    assert_close_bf16_pair(part, out[sl].float().cpu(), "1024 rows (split-K down projection) vs the full call")


def test_cfg4_uniform_sequences_against_library_matmul(dev, cfg4):
    """The all-visual and all-text sequences are plain FFNs: compare with fp32 torch matmuls on the GPU."""
    note("cfg4 uniform sequences")
    w, d, out = cfg4
    per_seq = w.mask.reshape(8, 4096).sum(1)
    checked = 0
    for seq in range(8):
        if per_seq[seq] not in (0, 4096):
            continue
        k1, k2, k3 = ("w1", "w2", "w3") if per_seq[seq] == 4096 else ("u1", "u2", "u3")
        xs = d.x[seq * 4096:(seq + 1) * 4096].float()
        t1 = xs @ d.W[k1].float().T
        t3 = xs @ d.W[k3].float().T
        hmid = (t1 * torch.sigmoid(t1) * t3).to(torch.bfloat16).float()
        ref = hmid @ d.W[k2].float().T
        assert_close(out[seq * 4096:(seq + 1) * 4096], ref.double().cpu(), f"uniform sequence {seq}")
        checked += 1
    assert checked >= 2


def test_cfg4_mixed_sequences_every_row(dev, cfg4):
    """The sequences that mix visual and text tokens (visual fraction 0.3 / 0.7) are the routed case:
    every one of their rows is checked against the select form in fp32 library matmuls on the GPU."""
    note("cfg4 mixed sequences, every row")
    w, d, out = cfg4
    per_seq = w.mask.reshape(8, 4096).sum(1)
    checked = 0
    for seq in range(8):
        if per_seq[seq] in (0, 4096):
            continue
        sl = slice(seq * 4096, (seq + 1) * 4096)
        x = d.x[sl].float()
        m = d.mask[sl]
        ref = torch.empty(4096, w.d, device=dev, dtype=torch.float32)
        for sel, (k1, k2, k3) in ((m, ("w1", "w2", "w3")), (~m, ("u1", "u2", "u3"))):
            t1 = x[sel] @ d.W[k1].float().T
            t3 = x[sel] @ d.W[k3].float().T
            hmid = (t1 * torch.sigmoid(t1) * t3).to(torch.bfloat16).float()
            ref[sel] = hmid @ d.W[k2].float().T
        assert_close(out[sl], ref.double().cpu(), f"mixed sequence {seq} ({int(per_seq[seq])} visual rows)")
        checked += 1
    assert checked >= 2


def test_ffn_split_tail_of_the_down_projection(dev):
    """8500 rows x 4096 output columns: 34 or 35 row tiles x 16 column tiles of 256x256, i.e. two whole
    rounds of 256 tiles and a remainder that runs cut into K ranges with a reduce pass.  Checked against
    fp32 library matmuls of the select form on the GPU (every row, so the remainder's rows are covered)."""
    note("ffn split tail M=8500 d=4096 h=1024")
    M, d, h = 8500, 4096, 1024
    cfg = _lib.tile_config(_lib.OP_FFN_DOWN, M, d, h)
    assert cfg["block_m"] == 256 and cfg["block_n"] == 256 and cfg["split_k"] == 1
    gen = torch.Generator().manual_seed(21)
    mask = torch.rand(M, generator=gen) < 0.45
    w = wl.make_ffn("t", M, d, h, mask, seed=22, w_std=0.03)
    dw = w.to(dev)
    out = MaskedFFN.apply(*dw.op_args())
    x = dw.x.float()
    ref = torch.empty(M, d, device=dev, dtype=torch.float32)
    for sel, (k1, k2, k3) in ((dw.mask, ("w1", "w2", "w3")), (~dw.mask, ("u1", "u2", "u3"))):
        t1 = x[sel] @ dw.W[k1].float().T
        t3 = x[sel] @ dw.W[k3].float().T
        hmid = (t1 * torch.sigmoid(t1) * t3).to(torch.bfloat16).float()
        ref[sel] = hmid @ dw.W[k2].float().T
    assert_close(out, ref.double().cpu(), "split tail")
    # twice the same call: the reduce order is fixed
    assert torch.equal(out, MaskedFFN.apply(*dw.op_args()))


def test_linear_split_tail(dev):
    """MaskedLinear forward on the 256x256 tile with a remainder round that is cut into K ranges."""
    note("linear split tail M=8500 K=1024 N=4096")
    M, K, N = 8500, 1024, 4096
    cfg = _lib.tile_config(_lib.OP_LINEAR_FWD, M, K, N)
    assert cfg["block_m"] == 256 and cfg["block_n"] == 256 and cfg["split_k"] == 1
    gen = torch.Generator().manual_seed(31)
    mask = torch.rand(M, generator=gen) < 0.55
    w = wl.make_linear("t", M, K, N, mask, seed=32).to(dev)
    y = MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, w.mask)
    ref = torch.where(w.mask[:, None], w.x.float() @ w.Wv.float().T, w.x.float() @ w.Wt.float().T)
    assert_close(y, ref.double().cpu(), "linear split tail")
    assert torch.equal(y, MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, w.mask))


def test_linear_fullsize_scaling_is_exact(dev):
    """y(2x) == 2 y(x) bit for bit (power-of-two scaling commutes with every rounding)."""
    note("cfg1/cfg3-size linear scaling")
    w = wl.cfg3_linear_bwd().to(dev)
    y1 = MaskedLinear.apply(w.x, w.Wv.T, w.Wt.T, w.mask)
    y2 = MaskedLinear.apply(w.x * 2, w.Wv.T, w.Wt.T, w.mask)
    assert torch.equal(y2, y1 * 2)


@pytest.mark.parametrize("M,kind", [(1, "visual"), (1, "text"), (8, "bernoulli"), (32, "bernoulli"), (64, "bernoulli"),
                                    (32, "visual"), (64, "text")])
def test_cfg5_decode_fullsize(dev, M, kind):
    """Decode path at d=4096, h=14336: agrees with the tiled path on the same rows (embedded in a
    65-row call, which the tile table sends to the GEMM kernels), and never reads an absent modality."""
    note(f"cfg5 M={M} {kind}")
    w = wl.cfg5_ffn_decode(M, kind).to(dev)
    assert _lib.tile_config(_lib.OP_FFN_FWD, M, 4096, 14336)["path"] == _lib.PATH_STREAM
    out = MaskedFFN.apply(*w.op_args())
    pad = 65 - M
    xb = torch.cat([w.x, w.x[:1].expand(pad, -1)]).contiguous()
    mb = torch.cat([w.mask, w.mask[:1].expand(pad)]).contiguous()
    big = MaskedFFN.apply(xb, *w.op_args()[1:7], mb)
    assert_close_bf16_pair(out, big[:M].float().cpu(), "decode vs tiled")
    if kind in ("visual", "text"):
        W = dict(w.W)
        for k in (("u1", "u2", "u3") if kind == "visual" else ("w1", "w2", "w3")):
            W[k] = torch.full_like(W[k], float("nan"))
        out2 = MaskedFFN.apply(*wl.FFNWorkload("p", w.x, W, w.mask).op_args())
        assert torch.equal(out2, out)
    # every row against the select form in fp32 library matmuls on the GPU, at the tolerance of the tiled path
    assert_close(out, _ffn_select_fp32(w.x, w.W, w.mask), f"decode M={M} {kind}, every row")
    # one row in double precision
    wc = wl.cfg5_ffn_decode(M, kind)
    sub = wl.FFNWorkload("r", wc.x[:1], wc.W, wc.mask[:1])
    assert_close(out[:1], cref.ffn_fwd(sub.x, sub.W, sub.mask, round_mid=True), "decode row 0")


def _ffn_select_fp32(x, W, mask):
    """The reference module's maths (test_ffn.py:43-47) in row-select form: fp32 library matmuls on the
    GPU, the intermediate rounded to bf16 once as the kernels store it.  Returns float64 on the host."""
    xf = x.float()
    ref = torch.zeros(x.shape[0], W["w2"].shape[0], device=x.device, dtype=torch.float32)
    for sel, (k1, k2, k3) in ((mask, ("w1", "w2", "w3")), (~mask, ("u1", "u2", "u3"))):
        if not bool(sel.any()):
            continue
        t1 = xf[sel] @ W[k1].float().T
        t3 = xf[sel] @ W[k3].float().T
        hmid = (t1 * torch.sigmoid(t1) * t3).to(torch.bfloat16).float()
        ref[sel] = hmid @ W[k2].float().T
    return ref.double().cpu()


def _span_mask(M, seq, spans, span, seed):
    """The reference's generate_mask idea (test_linear.py:15-21) per sequence: `spans` contiguous visual
    spans of `span` tokens at seeded, non-overlapping positions in every `seq`-token sequence."""
    gen = torch.Generator().manual_seed(seed)
    mask = torch.zeros(M, dtype=torch.bool)
    for s0 in range(0, M, seq):
        slots = torch.randperm(seq // span, generator=gen)[:spans]
        for k in slots.tolist():
            mask[s0 + k * span:s0 + (k + 1) * span] = True
    return mask


def test_linear_fwd_bwd_at_the_end_of_the_reference_sweep(dev):
    """MaskedLinear forward and backward at M = 63488, K = N = 1024: the last point of the reference's own
    --check sweep (test_linear.py:88, seq_len = 2048 * 31), past the 32768 rows of the largest benchmark
    shape.  Every row and every gradient against fp32 library matmuls of the select form on the GPU."""
    note("linear fwd+bwd M=63488 K=N=1024")
    M, K, N = 63488, 1024, 1024
    mask = _span_mask(M, 2048, 1, 1024, seed=3)   # one 1024-token image per 2048-token sequence, as test_linear.py:11-21
    w = wl.make_linear("sweep-end", M, K, N, mask, seed=4).to(dev)
    g = torch.Generator(device=dev).manual_seed(5)
    grad = torch.randn(M, N, device=dev, generator=g).to(torch.bfloat16)
    x = w.x.clone().requires_grad_(True)
    wv = w.Wv.clone().requires_grad_(True)
    wt = w.Wt.clone().requires_grad_(True)
    y = MaskedLinear.apply(x, wv.T, wt.T, w.mask)
    y.backward(grad)
    m2 = w.mask[:, None]
    xf, gf = w.x.float(), grad.float()
    assert_close(y, torch.where(m2, xf @ w.Wv.float().T, xf @ w.Wt.float().T).double().cpu(), "y")
    assert_close(x.grad, torch.where(m2, gf @ w.Wv.float(), gf @ w.Wt.float()).double().cpu(), "dx")
    # weight gradients sum 31744 rows each: compare at the scale of the sum (what a bf16 result can hold)
    for name, got, sel in (("dWv", wv.grad, w.mask), ("dWt", wt.grad, ~w.mask)):
        ref = (gf[sel].T @ xf[sel]).double().cpu()
        rep = om.error_report(got.float().cpu(), ref)
        assert rep["rel_l2"] <= om.REL_L2_TOL and rep["max_excess"] <= 1.0, (name, rep)


def test_ffn_fwd_at_the_last_key_of_the_reference_tables(dev):
    """MaskedFFN forward at M = 131072, d = 1024, h = 2048: the last key of the reference's largest tile
    table (ffn_kernel/bf16_ffn_bwd.json) at test_ffn.py:87-88's layer.  Every row against fp32 library
    matmuls of the select form on the GPU."""
    note("ffn fwd M=131072 d=1024 h=2048")
    M, d, h = 131072, 1024, 2048
    mask = _span_mask(M, 2048, 2, 576, seed=6)
    w = wl.make_ffn("tables-end", M, d, h, mask, seed=7).to(dev)
    out = MaskedFFN.apply(*w.op_args())
    for lo in range(0, M, 32768):   # the fp32 reference in four pieces
        sl = slice(lo, lo + 32768)
        assert_close(out[sl], _ffn_select_fp32(w.x[sl], w.W, w.mask[sl]), f"rows {lo}..{lo + 32768}")


def test_gather_offsets_past_32_bits_take_the_staged_path(dev):
    """Token rows whose byte offsets from the first row do not fit 32 bits (here: 40000 rows at a row stride
    of 65536 elements, a view into a wider buffer) cannot use the global->LDS loads, which address with
    32-bit offsets; the forward and the backward must notice and run their register-staged loops - at size,
    with the rows that need the upper offset bits among those checked."""
    note("linear fwd+bwd, row stride 65536 elements, M=40000")
    M, K, N, ld = 40000, 256, 512, 65536
    assert M * ld * 2 >= 1 << 32
    gen = torch.Generator().manual_seed(8)
    mask = (torch.rand(M, generator=gen) < 0.5).to(dev)
    g = torch.Generator(device=dev).manual_seed(9)
    wide = torch.empty(M, ld, device=dev, dtype=torch.bfloat16)
    wide[:, :K] = torch.randn(M, K, device=dev, generator=g).to(torch.bfloat16)
    x = wide[:, :K]
    assert x.stride(0) == ld
    Wv = (torch.randn(N, K, device=dev, generator=g) * 0.05).to(torch.bfloat16)
    Wt = (torch.randn(N, K, device=dev, generator=g) * 0.05).to(torch.bfloat16)
    y = MaskedLinear.apply(x, Wv.T, Wt.T, mask)
    xf = x.float()
    ref = torch.where(mask[:, None], xf @ Wv.float().T, xf @ Wt.float().T)
    assert_close(y, ref.double().cpu(), "strided x, forward")
    del wide, x, xf, ref
    torch.cuda.empty_cache()
    # the backward gathers grad rows the same way: a wide grad buffer
    gwide = torch.empty(M, ld, device=dev, dtype=torch.bfloat16)
    gwide[:, :N] = torch.randn(M, N, device=dev, generator=g).to(torch.bfloat16)
    grad = gwide[:, :N]
    xs = torch.randn(M, K, device=dev, generator=g).to(torch.bfloat16)
    from ffn_kernel_amd import masked_linear_backward
    dx, dwv, dwt = masked_linear_backward(grad, xs, Wv.T, Wt.T, mask)
    gf = grad.float()
    assert_close(dx, torch.where(mask[:, None], gf @ Wv.float(), gf @ Wt.float()).double().cpu(), "strided grad, dx")
    for name, got, sel in (("dWv", dwv, mask), ("dWt", dwt, ~mask)):
        ref = (xs.float()[sel].T @ gf[sel]).double().cpu()   # logical [K, N]
        rep = om.error_report(got.float().cpu(), ref)
        assert rep["rel_l2"] <= om.REL_L2_TOL and rep["max_excess"] <= 1.0, (name, rep)
