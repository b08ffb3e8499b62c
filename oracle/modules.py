"""Restatement of the reference's PyTorch path and of the maths it implements (CPU, torch).

Blend form  = what the reference's oracle modules compute: both branches for every row, then
              `v * m + t * ~m` (test_linear.py:47-49, test_ffn.py:43-47).
Select form = the same function written row-wise: row m uses the visual weights if mask[m]
              else the text weights.  Identical for finite values; differs only when the unused
              branch is non-finite (NaN * 0), which the routed kernels never compute.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------- routing
def stable_partition(mask: np.ndarray):
    """perm = indices of True rows ascending, then indices of False rows ascending; and counts.
    Same row -> weight assignment as the reference's per-row mask test (linear.py:120-149)."""
    mask = np.asarray(mask).astype(bool).reshape(-1)
    idx = np.arange(mask.shape[0], dtype=np.int32)
    perm = np.concatenate([idx[mask], idx[~mask]]).astype(np.int32)
    return perm, np.array([int(mask.sum()), int((~mask).sum())], dtype=np.int32)


# ----------------------------------------------------------------------------- blend form (reference oracle)
class TorchLinear(torch.nn.Module):
    """test_linear.py:41-49 / README.md:49-57."""

    def __init__(self, in_dim: int, out_dim: int):
        super().__init__()
        self.linear_v = torch.nn.Linear(in_dim, out_dim, bias=False)
        self.linear_t = torch.nn.Linear(in_dim, out_dim, bias=False)

    def forward(self, x, visual_mask):
        m = visual_mask[:, :, None]
        return self.linear_v(x) * m + self.linear_t(x) * (~m)


class TorchFFN(torch.nn.Module):
    """test_ffn.py:32-47 / README.md:83-98."""

    def __init__(self, hidden_size: int, intermediate_size: int):
        super().__init__()
        mk = lambda i, o: torch.nn.Linear(i, o, bias=False)
        self.w1, self.w2, self.w3 = mk(hidden_size, intermediate_size), mk(intermediate_size, hidden_size), mk(hidden_size, intermediate_size)
        self.u1, self.u2, self.u3 = mk(hidden_size, intermediate_size), mk(intermediate_size, hidden_size), mk(hidden_size, intermediate_size)

    @torch.no_grad()
    def forward(self, x, mask):
        m = mask[:, :, None]
        proj1 = F.silu(self.w1(x)) * self.w3(x)
        proj2 = F.silu(self.u1(x)) * self.u3(x)
        return self.w2(proj1) * m + self.u2(proj2) * ~m


def linear_blend(x, Wv, Wt, mask):
    """Blend form on 2-D inputs. x [M,K]; Wv, Wt nn.Linear-style [N,K]; mask [M] bool. Runs in x.dtype."""
    m = mask[:, None]
    return F.linear(x, Wv) * m + F.linear(x, Wt) * (~m)


def ffn_blend(x, W, mask):
    """Blend form of the FFN. W: dict w1,w3,u1,u3 [h,d]; w2,u2 [d,h]. Runs in x.dtype (bf16 rounds
    after every Linear, silu and product, as ATen does)."""
    m = mask[:, None]
    p1 = F.silu(F.linear(x, W["w1"])) * F.linear(x, W["w3"])
    p2 = F.silu(F.linear(x, W["u1"])) * F.linear(x, W["u3"])
    return F.linear(p1, W["w2"]) * m + F.linear(p2, W["u2"]) * ~m


# ----------------------------------------------------------------------------- select form, high precision
def linear_select(x, Wv, Wt, mask, dtype=torch.float32):
    """y[m] = x[m] @ (Wv if mask[m] else Wt)^T, computed in `dtype`, unused branch never touched."""
    x, Wv, Wt = x.to(dtype), Wv.to(dtype), Wt.to(dtype)
    y = torch.empty((x.shape[0], Wv.shape[0]), dtype=dtype)
    y[mask] = x[mask] @ Wv.T
    y[~mask] = x[~mask] @ Wt.T
    return y


def ffn_select(x, W, mask, dtype=torch.float32, round_intermediate=False):
    """FFN in `dtype`, row-selected.  round_intermediate=True rounds the [M,h] intermediate to bf16
    once (what a kernel that stores it in bf16 does, as the reference does at ffn.py:113)."""
    xd = x.to(dtype)
    out = torch.empty((x.shape[0], W["w2"].shape[0]), dtype=dtype)
    for sel, (k1, k2, k3) in ((mask, ("w1", "w2", "w3")), (~mask, ("u1", "u2", "u3"))):
        xs = xd[sel]
        t1 = xs @ W[k1].to(dtype).T
        t3 = xs @ W[k3].to(dtype).T
        hmid = t1 * torch.sigmoid(t1) * t3
        if round_intermediate:
            hmid = hmid.to(torch.bfloat16).to(dtype)
        out[sel] = hmid @ W[k2].to(dtype).T
    return out


def linear_backward_select(g, x, Wv, Wt, mask, dtype=torch.float32):
    """(dx [M,K], dWv [N,K], dWt [N,K]) of y = linear_select, for upstream gradient g [M,N]; weights
    and their gradients nn.Linear-style [N,K]."""
    g, x, Wv, Wt = g.to(dtype), x.to(dtype), Wv.to(dtype), Wt.to(dtype)
    dx = torch.empty_like(x)
    dx[mask] = g[mask] @ Wv
    dx[~mask] = g[~mask] @ Wt
    dWv = g[mask].T @ x[mask]
    dWt = g[~mask].T @ x[~mask]
    return dx, dWv, dWt


def linear_backward_autograd(g, x, Wv, Wt, mask, dtype=torch.float32):
    """Same gradients through autograd of the blend form (how the reference's --check takes them:
    test_linear.py:92-102)."""
    x = x.to(dtype).clone().requires_grad_(True)
    Wv = Wv.to(dtype).clone().requires_grad_(True)
    Wt = Wt.to(dtype).clone().requires_grad_(True)
    y = linear_blend(x, Wv, Wt, mask)
    y.backward(g.to(dtype))
    return x.grad, Wv.grad, Wt.grad


def ffn_backward_select(g, x, W, mask, dtype=torch.float64, round_intermediates=False):
    """Gradients of out = ffn_select(x, W, mask) for upstream gradient g [M, d], by the chain rule
    written out row-selected (the decomposition README.md:159-172 sketches; silu'(t) is the textbook
    s + t s (1 - s), not the README's term).  Returns (dx [M, d], dict of weight gradients in
    nn.Linear layout: w1, w3, u1, u3 [h, d]; w2, u2 [d, h]).  round_intermediates=True rounds
    t1, t3, dh, dt1, dt3 and the intermediate to bf16 where a kernel that stores them in bf16 does."""
    rnd = (lambda t: t.to(torch.bfloat16).to(dtype)) if round_intermediates else (lambda t: t)
    gd, xd = g.to(dtype), x.to(dtype)
    dx = torch.empty_like(xd)
    dW = {}
    for sel, (k1, k2, k3) in ((mask, ("w1", "w2", "w3")), (~mask, ("u1", "u2", "u3"))):
        xs, gs = xd[sel], gd[sel]
        A1, A2, A3 = W[k1].to(dtype), W[k2].to(dtype), W[k3].to(dtype)
        t1, t3 = rnd(xs @ A1.T), rnd(xs @ A3.T)
        dh = rnd(gs @ A2)
        s = torch.sigmoid(t1)
        silu = t1 * s
        dt1 = rnd(dh * t3 * (s + silu * (1 - s)))
        dt3 = rnd(dh * silu)
        hmid = rnd(silu * t3)
        dx[sel] = dt1 @ A1 + dt3 @ A3
        dW[k1] = dt1.T @ xs
        dW[k3] = dt3.T @ xs
        dW[k2] = gs.T @ hmid
    return dx, dW


def ffn_backward_autograd(g, x, W, mask, dtype=torch.float64):
    """The same gradients through autograd of the blend form (the reference's oracle module maths)."""
    xr = x.to(dtype).clone().requires_grad_(True)
    Wr = {k: v.to(dtype).clone().requires_grad_(True) for k, v in W.items()}
    out = ffn_blend(xr, Wr, mask)
    out.backward(g.to(dtype))
    return xr.grad, {k: v.grad for k, v in Wr.items()}


# ----------------------------------------------------------------------------- tolerances
MAX_ABS_TOL = 2e-2
REL_L2_TOL = 5e-3


def error_report(got: torch.Tensor, ref: torch.Tensor) -> dict:
    """Errors of `got` (any dtype) against `ref` (fp32/fp64):
      max_abs              largest |got - ref|
      rel_l2               ||got - ref|| / ||ref||
      max_abs_vs_bf16_ref  largest |got - bf16(ref)|  (0 = identical to the correctly rounded result)
      max_ulp_large        largest error in bf16 ulps of the reference element, over elements with
                           |ref| >= 4 (where half a bf16 ulp already reaches 1.6e-2 .. and 2e-2 is
                           not representable)
      max_excess           largest |got - ref| / max(2e-2, one bf16 ulp of the reference element);
                           <= 1 means every element is within 2e-2 or within one bf16 ulp
    bf16 output rounding alone is half an ulp = 2^(e-8) for |y| in [2^e, 2^(e+1)): 3.1e-2 at |y| >= 8."""
    got64, ref64 = got.double(), ref.double()
    if got64.numel() == 0:
        return {"max_abs": 0.0, "rel_l2": 0.0, "max_abs_vs_bf16_ref": 0.0, "max_ulp_large": 0.0,
                "max_excess": 0.0, "ref_abs_max": 0.0}
    diff = (got64 - ref64).abs()
    diff_bf = (got64 - ref.to(torch.bfloat16).double()).abs()
    mag = ref64.abs().clamp_min(2.0 ** -126)
    ulp = torch.exp2(torch.floor(torch.log2(mag)) - 7)  # one bf16 ulp at the reference's magnitude
    large = ref64.abs() >= 4
    denom = ref64.norm().item()
    return {
        "max_abs": diff.max().item(),
        "rel_l2": (diff.norm().item() / denom) if denom > 0 else diff.norm().item(),
        "max_abs_vs_bf16_ref": diff_bf.max().item(),
        "max_ulp_large": (diff / ulp)[large].max().item() if large.any() else 0.0,
        "max_excess": (diff / torch.clamp(ulp, min=MAX_ABS_TOL)).max().item(),
        "ref_abs_max": ref64.abs().max().item(),
    }


def within_tolerance(rep: dict) -> bool:
    """Every element within max-abs 2e-2 of the reference — or within one bf16 ulp of it where one
    ulp exceeds 2e-2, i.e. where bf16 cannot represent the result to 2e-2 — and rel-L2 <= 5e-3."""
    return rep["max_excess"] <= 1.0 and rep["rel_l2"] <= REL_L2_TOL
