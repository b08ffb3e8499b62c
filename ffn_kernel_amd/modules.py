"""nn.Module wrappers around MaskedLinear / MaskedFFN with the parameter names of the reference's
README modules (`TritonLinear`, README.md:60-74 / test_linear.py:52-65; `Triton` FFN, README.md:101-124 /
test_ffn.py:50-72), so that their state_dicts are interchangeable with the reference's PyTorch
`Torch` modules (`linear_v`, `linear_t`; `w1..w3`, `u1..u3`).

Inputs may be 2-D `[M, D]` with mask `[M]` or 3-D `[B, S, D]` with mask `[B, S]`; the modules
flatten and unflatten as the reference's wrappers do.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .ops import MaskedFFN, MaskedLinear


def _flatten(x: torch.Tensor, mask: torch.Tensor):
    if x.dim() == 3:
        if mask.shape != x.shape[:2]:
            raise ValueError(f"mask shape {tuple(mask.shape)} does not match x {tuple(x.shape)}")
        return x.flatten(0, 1), mask.flatten(0, 1), x.shape[0]
    if x.dim() == 2:
        return x, mask.reshape(-1), None
    raise ValueError(f"x must be [M, D] or [B, S, D], got {tuple(x.shape)}")


def _unflatten(y: torch.Tensor, batch):
    return y if batch is None else y.unflatten(0, (batch, -1))


class MaskedLinearModule(nn.Module):
    """Two bias-free Linear layers, one per modality; rows are routed by `visual_mask`.
    Differentiable (forward + backward), like the reference's `Triton` module of test_linear.py."""

    def __init__(self, in_dim: int, out_dim: int, device=None, dtype=torch.bfloat16):
        super().__init__()
        self.linear_v = nn.Linear(in_dim, out_dim, bias=False, device=device, dtype=dtype)
        self.linear_t = nn.Linear(in_dim, out_dim, bias=False, device=device, dtype=dtype)

    def forward(self, x: torch.Tensor, visual_mask: torch.Tensor) -> torch.Tensor:
        x2, m, batch = _flatten(x, visual_mask)
        y = MaskedLinear.apply(x2, self.linear_v.weight.T, self.linear_t.weight.T, m)
        return _unflatten(y, batch)


class MaskedFFNModule(nn.Module):
    """SwiGLU FFN with visual weights (w1, w2, w3) and text weights (u1, u2, u3).  The reference's
    `Triton` module of test_ffn.py / README.md:101-124 runs under no_grad on `.weight.data` because
    its op has no backward; this one passes the parameters themselves, so it trains as well (wrap the
    call in torch.no_grad() for inference, as with any module)."""

    def __init__(self, hidden_size: int, intermediate_size: int, device=None, dtype=torch.bfloat16):
        super().__init__()
        mk = lambda i, o: nn.Linear(i, o, bias=False, device=device, dtype=dtype)
        self.w1, self.w2, self.w3 = mk(hidden_size, intermediate_size), mk(intermediate_size, hidden_size), mk(hidden_size, intermediate_size)
        self.u1, self.u2, self.u3 = mk(hidden_size, intermediate_size), mk(intermediate_size, hidden_size), mk(hidden_size, intermediate_size)

    def forward(self, x: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        x2, m, batch = _flatten(x, mask)
        y = MaskedFFN.apply(x2, self.w1.weight.T, self.w2.weight.T, self.w3.weight.T,
                            self.u1.weight.T, self.u2.weight.T, self.u3.weight.T, m)
        return _unflatten(y, batch)
