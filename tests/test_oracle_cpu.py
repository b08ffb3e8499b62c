"""Pins of the CPU oracle (no GPU): every oracle function is checked against something it was not
written from — closed forms, library routines, brute force, invariants — so that a dropped term,
a swapped weight or a transposed operand fails here."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from ffn_kernel_amd import workloads as wl
from oracle import cref
from oracle import modules as om


def _mk_linear(M, K, N, p, seed, with_grad=False):
    gen = torch.Generator().manual_seed(seed)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    return wl.make_linear("t", M, K, N, mask, seed, with_grad=with_grad, w_std=0.1)


# ------------------------------------------------------------------ routing
def test_stable_partition_brute_force_all_masks():
    """All 2^M masks for M <= 10: perm equals a stable sort of rows by (not mask)."""
    for M in range(0, 11):
        for bits in itertools.product([False, True], repeat=M):
            mask = np.array(bits, dtype=bool)
            perm, counts = om.stable_partition(mask)
            expect = sorted(range(M), key=lambda i: (not mask[i], i))
            assert perm.tolist() == expect
            assert counts.tolist() == [int(mask.sum()), M - int(mask.sum())]
            cperm, ccounts = cref.route(torch.from_numpy(mask))
            assert cperm.tolist() == expect and ccounts.tolist() == counts.tolist()


def test_partition_is_a_permutation_and_groups_are_pure():
    gen = torch.Generator().manual_seed(0)
    mask = (torch.rand(5000, generator=gen) < 0.37).numpy()
    perm, counts = om.stable_partition(mask)
    assert sorted(perm.tolist()) == list(range(5000))
    assert mask[perm[:counts[0]]].all() and not mask[perm[counts[0]:]].any()
    assert (np.diff(perm[:counts[0]]) > 0).all() and (np.diff(perm[counts[0]:]) > 0).all()


# ------------------------------------------------------------------ linear forward
def test_linear_identity_weights_exact():
    M, K = 50, 32
    w = _mk_linear(M, K, K, 0.5, 1)
    eye = torch.eye(K).to(torch.bfloat16)
    for fn in (lambda: om.linear_select(w.x, eye, 2 * eye, w.mask, torch.float64),
               lambda: cref.linear_fwd(w.x, eye, 2 * eye, w.mask),
               lambda: om.linear_blend(w.x, eye, 2 * eye, w.mask).double()):
        y = fn()
        assert torch.equal(y, torch.where(w.mask[:, None], w.x.double(), 2 * w.x.double()))


def test_linear_equal_weights_is_plain_matmul():
    w = _mk_linear(33, 40, 24, 0.5, 2)
    ref = w.x.double() @ w.Wv.double().T
    assert torch.allclose(om.linear_select(w.x, w.Wv, w.Wv, w.mask, torch.float64), ref, rtol=0, atol=1e-12)
    assert torch.allclose(cref.linear_fwd(w.x, w.Wv, w.Wv, w.mask), ref, rtol=0, atol=1e-12)


@pytest.mark.parametrize("p", [0.0, 1.0])
def test_linear_uniform_masks_reduce_to_F_linear(p):
    w = _mk_linear(20, 16, 12, p, 3)
    W = w.Wv if p == 1.0 else w.Wt
    ref = F.linear(w.x.double(), W.double())
    assert torch.allclose(cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask), ref, atol=1e-12, rtol=0)
    assert torch.allclose(om.linear_select(w.x, w.Wv, w.Wt, w.mask, torch.float64), ref, atol=1e-12, rtol=0)
    assert torch.allclose(om.linear_blend(w.x.double(), w.Wv.double(), w.Wt.double(), w.mask), ref, atol=1e-12, rtol=0)


def test_linear_c_loops_vs_torch_where_ragged():
    for (M, K, N) in [(7, 5, 3), (8, 32, 32), (37, 48, 40), (1, 1, 1)]:
        w = _mk_linear(M, K, N, 0.5, M)
        xv = w.x.double() @ w.Wv.double().T
        xt = w.x.double() @ w.Wt.double().T
        ref = torch.where(w.mask[:, None], xv, xt)
        assert torch.allclose(cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask), ref, atol=1e-11, rtol=0)
        assert torch.allclose(om.linear_select(w.x, w.Wv, w.Wt, w.mask, torch.float64), ref, atol=1e-11, rtol=0)
        # the reference's bf16 module form agrees to bf16 accuracy
        rep = om.error_report(om.linear_blend(w.x, w.Wv, w.Wt, w.mask), ref)
        assert rep["rel_l2"] < 1e-2


def test_blend_and_select_differ_only_on_nonfinite_unused_branch():
    w = _mk_linear(16, 8, 8, 0.5, 4)
    Wt_nan = torch.full_like(w.Wt, float("nan"))
    sel = om.linear_select(w.x, w.Wv, Wt_nan, w.mask)
    assert torch.isfinite(sel[w.mask]).all()
    blend = om.linear_blend(w.x, w.Wv, Wt_nan, w.mask)
    assert torch.isnan(blend).all()  # NaN * 0 poisons the blend form


def test_module_form_matches_functional_form():
    """The nn.Module restatement (3-D inputs) equals the 2-D functional blend."""
    torch.manual_seed(0)
    mod = om.TorchLinear(16, 12).bfloat16()
    x = torch.randn(2, 9, 16).bfloat16()
    mask = torch.rand(2, 9) < 0.5
    y = mod(x, mask)
    y2 = om.linear_blend(x.reshape(18, 16), mod.linear_v.weight, mod.linear_t.weight, mask.reshape(18))
    assert torch.equal(y.reshape(18, 12), y2)
    ffn = om.TorchFFN(16, 24).bfloat16()
    W = {k: getattr(ffn, k).weight.detach() for k in ("w1", "w2", "w3", "u1", "u2", "u3")}
    o = ffn(x, mask)
    o2 = om.ffn_blend(x.reshape(18, 16), W, mask.reshape(18))
    assert torch.equal(o.reshape(18, 16), o2)


# ------------------------------------------------------------------ SwiGLU / FFN
def test_silu_closed_forms():
    t = torch.tensor([0.0, 50.0, -50.0, 1.0], dtype=torch.float64)
    s = t * torch.sigmoid(t)
    assert s[0] == 0 and abs(s[1] - 50.0) < 1e-12 and abs(s[2]) < 1e-12
    assert abs(s[3] - 1.0 / (1.0 + np.exp(-1.0))) < 1e-15
    # C oracle: d = h = 1, w1 = 1, w3 = 1, w2 = 1 -> out = silu(x) * x
    one = torch.ones(1, 1, dtype=torch.bfloat16)
    W = {k: one for k in ("w1", "w2", "w3", "u1", "u2", "u3")}
    for xv in (0.0, 1.0, -2.0, 8.0):
        x = torch.tensor([[xv]], dtype=torch.bfloat16)
        out = cref.ffn_fwd(x, W, torch.tensor([True]))
        assert abs(out.item() - xv * xv / (1 + np.exp(-xv))) < 1e-12


def test_ffn_zero_gate_or_up_gives_zero():
    gen = torch.Generator().manual_seed(5)
    mask = torch.rand(12, generator=gen) < 0.5
    w = wl.make_ffn("t", 12, 16, 24, mask, 5, w_std=0.1)
    for z in ("w1", "w3"):
        W = dict(w.W); W[z] = torch.zeros_like(W[z])
        for out in (cref.ffn_fwd(w.x, W, mask), om.ffn_select(w.x, W, mask, torch.float64)):
            assert (out[mask] == 0).all() and (out[~mask] != 0).any()


def test_ffn_c_loops_vs_torch_select_and_blend():
    for (M, d, h) in [(19, 32, 48), (5, 7, 3), (64, 64, 128)]:
        gen = torch.Generator().manual_seed(M)
        mask = torch.rand(M, generator=gen) < 0.5
        w = wl.make_ffn("t", M, d, h, mask, M, w_std=0.1)
        a = cref.ffn_fwd(w.x, w.W, mask)
        b = om.ffn_select(w.x, w.W, mask, torch.float64)
        assert torch.allclose(a, b, atol=1e-11, rtol=0)
        rep = om.error_report(om.ffn_blend(w.x, w.W, mask), a)
        assert rep["rel_l2"] < 2e-2
        # swapping visual and text weights together with the mask is the same function
        Wsw = {"w1": w.W["u1"], "w2": w.W["u2"], "w3": w.W["u3"], "u1": w.W["w1"], "u2": w.W["w2"], "u3": w.W["w3"]}
        assert torch.equal(cref.ffn_fwd(w.x, Wsw, ~mask), a)
        # rounding the intermediate to bf16 once moves the result by a bf16-sized amount only
        c = cref.ffn_fwd(w.x, w.W, mask, round_mid=True)
        d2 = om.ffn_select(w.x, w.W, mask, torch.float64, round_intermediate=True)
        assert torch.allclose(c, d2, atol=1e-9, rtol=0)
        assert om.error_report(c, a)["rel_l2"] < 5e-3


def test_ffn_h_identity_reduces_to_linear():
    """W3 rows = e_0 scaled so that x W3 == const 1 on a constant feature: out = W2 silu(x W1)."""
    M, d = 10, 8
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    x[:, 0] = 1.0
    h = 6
    W1 = (torch.randn(h, d, generator=gen) * 0.3).to(torch.bfloat16)
    W3 = torch.zeros(h, d, dtype=torch.bfloat16); W3[:, 0] = 1.0  # x W3^T == 1
    W2 = (torch.randn(d, h, generator=gen) * 0.3).to(torch.bfloat16)
    W = {"w1": W1, "w2": W2, "w3": W3, "u1": W1, "u2": W2, "u3": W3}
    out = cref.ffn_fwd(x, W, torch.ones(M, dtype=torch.bool))
    t1 = x.double() @ W1.double().T
    ref = (t1 * torch.sigmoid(t1)) @ W2.double().T
    assert torch.allclose(out, ref, atol=1e-12, rtol=0)


# ------------------------------------------------------------------ linear backward
def test_backward_matches_autograd_and_c_loops():
    for (M, K, N, p) in [(23, 16, 12, 0.5), (9, 5, 7, 0.3), (16, 8, 8, 1.0), (16, 8, 8, 0.0)]:
        w = _mk_linear(M, K, N, p, M, with_grad=True)
        a = om.linear_backward_autograd(w.grad, w.x, w.Wv, w.Wt, w.mask, torch.float64)
        b = om.linear_backward_select(w.grad, w.x, w.Wv, w.Wt, w.mask, torch.float64)
        c = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
        for ta, tb, tc in zip(a, b, c):
            assert torch.allclose(ta, tb, atol=1e-10, rtol=0)
            assert torch.allclose(ta, tc, atol=1e-10, rtol=0)
        if p == 1.0:
            assert (c[2] == 0).all()
        if p == 0.0:
            assert (c[1] == 0).all()


def test_backward_invariants():
    w = _mk_linear(40, 12, 10, 0.5, 11, with_grad=True)
    dx, dWv, dWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    assert torch.allclose(dWv + dWt, w.grad.double().T @ w.x.double(), atol=1e-10, rtol=0)
    dx2, _, _ = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wv, w.mask)
    assert torch.allclose(dx2, w.grad.double() @ w.Wv.double(), atol=1e-10, rtol=0)


def test_backward_finite_differences():
    w = _mk_linear(6, 4, 3, 0.5, 13, with_grad=True)
    x, Wv, Wt, g = w.x.double(), w.Wv.double(), w.Wt.double(), w.grad.double()
    f = lambda x_, Wv_, Wt_: (om.linear_select(x_, Wv_, Wt_, w.mask, torch.float64) * g).sum()
    dx, dWv, dWt = cref.linear_bwd(w.grad, w.x, w.Wv, w.Wt, w.mask)
    eps = 1e-6
    for (t, grad, idx) in ((x, dx, 0), (Wv, dWv, 1), (Wt, dWt, 2)):
        for i in range(t.shape[0]):
            for j in range(t.shape[1]):
                tp = t.clone(); tp[i, j] += eps
                tm = t.clone(); tm[i, j] -= eps
                args_p = [x, Wv, Wt]; args_p[idx] = tp
                args_m = [x, Wv, Wt]; args_m[idx] = tm
                fd = (f(*args_p) - f(*args_m)) / (2 * eps)
                assert abs(fd - grad[i, j]) < 1e-6


# ------------------------------------------------------------------ FFN backward
def _mk_ffn_bwd(M, d, h, p, seed):
    gen = torch.Generator().manual_seed(seed)
    mask = torch.rand(M, generator=gen) < p if 0 < p < 1 else torch.full((M,), bool(p))
    w = wl.make_ffn("t", M, d, h, mask, seed=seed, w_std=0.3)
    g = torch.randn(M, d, generator=gen).to(torch.bfloat16)
    return w, g


def test_ffn_backward_select_matches_autograd_and_c_loops():
    for (M, d, h, p) in [(23, 16, 24, 0.5), (9, 8, 8, 0.3), (16, 8, 16, 1.0), (16, 8, 16, 0.0)]:
        w, g = _mk_ffn_bwd(M, d, h, p, M)
        dx, dW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64)
        dx2, dW2 = om.ffn_backward_autograd(g, w.x, w.W, w.mask, torch.float64)
        dx3, dW3 = cref.ffn_bwd(g, w.x, w.W, w.mask)
        assert torch.allclose(dx, dx2, atol=1e-10, rtol=0)
        assert torch.allclose(dx, dx3, atol=1e-10, rtol=0)
        for k in dW:
            assert torch.allclose(dW[k], dW2[k], atol=1e-10, rtol=0), k
            assert torch.allclose(dW[k], dW3[k], atol=1e-10, rtol=0), k
        # the bf16-storage variant of the C loops rounds where the torch one does
        dx4, dW4 = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64, round_intermediates=True)
        dx5, dW5 = cref.ffn_bwd(g, w.x, w.W, w.mask, round_mid=True)
        assert torch.allclose(dx4, dx5, atol=1e-2, rtol=1e-2)  # a rounding boundary may fall either way
        assert (dx4 - dx5).abs().median() < 1e-9
        absent = ("u1", "u2", "u3") if p == 1.0 else ("w1", "w2", "w3") if p == 0.0 else ()
        for k in absent:
            assert (dW[k] == 0).all()


def test_ffn_backward_finite_differences():
    w, g = _mk_ffn_bwd(5, 4, 6, 0.5, 29)
    w.mask[0], w.mask[1] = True, False  # both groups present
    x = w.x.double()
    W = {k: v.double() for k, v in w.W.items()}
    gd = g.double()
    f = lambda x_, W_: (om.ffn_select(x_, W_, w.mask, torch.float64) * gd).sum()
    dx, dW = om.ffn_backward_select(g, w.x, w.W, w.mask, torch.float64)
    eps = 1e-6
    for i in range(x.shape[0]):
        for j in range(x.shape[1]):
            xp = x.clone(); xp[i, j] += eps
            xm = x.clone(); xm[i, j] -= eps
            assert abs((f(xp, W) - f(xm, W)) / (2 * eps) - dx[i, j]) < 1e-6
    for k in W:
        for (i, j) in [(0, 0), (1, 2), (W[k].shape[0] - 1, W[k].shape[1] - 1)]:
            Wp = dict(W); Wp[k] = W[k].clone(); Wp[k][i, j] += eps
            Wm = dict(W); Wm[k] = W[k].clone(); Wm[k][i, j] -= eps
            assert abs((f(x, Wp) - f(x, Wm)) / (2 * eps) - dW[k][i, j]) < 1e-6, k


def test_ffn_backward_reductions():
    # a constant, large gate makes silu the identity and silu' one: the FFN is then the product of
    # two linear maps through t3, whose gradients are plain matrix products
    M, d, h = 12, 8, 16
    w, g = _mk_ffn_bwd(M, d, h, 1.0, 3)
    x = w.x.double(); x[:, 0] = 1.0
    W = {k: v.double() for k, v in w.W.items()}
    W["w1"] = torch.zeros(h, d, dtype=torch.float64); W["w1"][:, 0] = 40.0  # t1 = 40 everywhere
    dx, dW = om.ffn_backward_select(g, x, W, w.mask, torch.float64)
    gd = g.double()
    dh = gd @ W["w2"]
    assert torch.allclose(dW["w3"], (dh * 40.0).T @ x, atol=1e-8, rtol=1e-12)
    assert torch.allclose(dW["w2"], gd.T @ (40.0 * (x @ W["w3"].T)), atol=1e-8, rtol=1e-12)
    # the bf16-rounded variant stays within bf16 accuracy of the exact one
    w2, g2 = _mk_ffn_bwd(64, 32, 48, 0.5, 5)
    a = om.ffn_backward_select(g2, w2.x, w2.W, w2.mask, torch.float64)
    b = om.ffn_backward_select(g2, w2.x, w2.W, w2.mask, torch.float64, round_intermediates=True)
    assert om.error_report(b[0], a[0])["rel_l2"] < 1e-2
    for k in a[1]:
        assert om.error_report(b[1][k], a[1][k])["rel_l2"] < 1e-2


# ------------------------------------------------------------------ tolerance helper
def test_error_report_flags_a_wrong_row():
    w = _mk_linear(64, 32, 32, 0.5, 17)
    ref = cref.linear_fwd(w.x, w.Wv, w.Wt, w.mask)
    good = ref.to(torch.bfloat16)
    assert om.within_tolerance(om.error_report(good, ref))
    bad = good.clone()
    wrong = cref.linear_fwd(w.x, w.Wt, w.Wv, w.mask).to(torch.bfloat16)  # weights swapped
    bad[3] = wrong[3]
    assert not om.within_tolerance(om.error_report(bad, ref))
