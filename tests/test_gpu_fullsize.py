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
    # one row in double precision
    wc = wl.cfg5_ffn_decode(M, kind)
    sub = wl.FFNWorkload("r", wc.x[:1], wc.W, wc.mask[:1])
    assert_close(out[:1], cref.ffn_fwd(sub.x, sub.W, sub.mask, round_mid=True), "decode row 0")
