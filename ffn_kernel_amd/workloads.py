"""Seeded synthetic workloads: the five benchmark configurations (shapes, weight scales and
mask patterns) this package is measured and tested on.

Everything is generated on the CPU with a torch.Generator so that the same seed gives the same
tensors on every machine, then moved to the requested device.  Mask patterns follow the
reference's generators (contiguous visual spans at seeded positions, test_linear.py:15-21,
test_ffn.py:12-18) extended to several spans, per-sequence visual fractions and i.i.d. masks.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

IMAGE_TOKENS = 576  # visual tokens per image span


def span_mask(batch: int, seq: int, spans_per_seq: List[int], gen: torch.Generator,
              span: int = IMAGE_TOKENS) -> torch.Tensor:
    """bool [batch, seq]: sequence b gets spans_per_seq[b] non-overlapping visual spans of `span`
    tokens at seeded positions (a sequence whose spans cover it entirely is all-visual)."""
    mask = torch.zeros((batch, seq), dtype=torch.bool)
    for b in range(batch):
        n = spans_per_seq[b]
        if n * span >= seq:
            mask[b] = True
            continue
        # choose n starts among the gaps: place spans in order with random slack between them
        slack = seq - n * span
        cuts = torch.sort(torch.randint(0, slack + 1, (n,), generator=gen)).values.tolist()
        for i, c in enumerate(cuts):
            start = c + i * span
            mask[b, start:start + span] = True
    return mask


def bernoulli_mask(M: int, p: float, gen: torch.Generator) -> torch.Tensor:
    return torch.rand(M, generator=gen) < p


def _randn_bf16(shape, std: float, gen: torch.Generator) -> torch.Tensor:
    return (torch.randn(shape, generator=gen, dtype=torch.float32) * std).to(torch.bfloat16)


@dataclass
class LinearWorkload:
    """MaskedLinear inputs. Wv/Wt are nn.Linear-style [N, K]; pass Wv.T / Wt.T to the op."""
    name: str
    x: torch.Tensor        # [M, K]
    Wv: torch.Tensor       # [N, K]
    Wt: torch.Tensor       # [N, K]
    mask: torch.Tensor     # [M] bool
    grad: Optional[torch.Tensor] = None  # [M, N] upstream gradient (backward workloads)

    @property
    def routed_flops_fwd(self) -> int:
        M, K = self.x.shape
        return 2 * M * K * self.Wv.shape[0]

    @property
    def routed_flops_bwd(self) -> int:
        return 2 * self.routed_flops_fwd  # dx + (dW_v and dW_t together)

    def to(self, device) -> "LinearWorkload":
        g = None if self.grad is None else self.grad.to(device)
        return LinearWorkload(self.name, self.x.to(device), self.Wv.to(device), self.Wt.to(device),
                              self.mask.to(device), g)


@dataclass
class FFNWorkload:
    """MaskedFFN inputs. Weights are nn.Linear-style: W1,W3,U1,U3 [h, d]; W2,U2 [d, h]."""
    name: str
    x: torch.Tensor
    W: Dict[str, torch.Tensor] = field(default_factory=dict)  # keys w1,w2,w3,u1,u2,u3
    mask: torch.Tensor = None

    @property
    def d(self) -> int:
        return self.x.shape[1]

    @property
    def h(self) -> int:
        return self.W["w1"].shape[0]

    @property
    def routed_flops(self) -> int:
        return 2 * self.x.shape[0] * self.d * self.h * 3

    def algorithmic_bytes(self) -> int:
        """Bytes that must move for this call: the weights of each modality present (three
        matrices each), x, out and the mask."""
        M = self.x.shape[0]
        nv = int(self.mask.sum())
        present = int(nv > 0) + int(nv < M)
        return 3 * self.d * self.h * 2 * present + 2 * M * self.d * 2 + M

    def to(self, device) -> "FFNWorkload":
        return FFNWorkload(self.name, self.x.to(device), {k: v.to(device) for k, v in self.W.items()},
                           self.mask.to(device))

    def op_args(self):
        """Positional arguments of MaskedFFN.apply (note the w1, w2, w3 order of the reference)."""
        W = self.W
        return (self.x, W["w1"].T, W["w2"].T, W["w3"].T, W["u1"].T, W["u2"].T, W["u3"].T, self.mask)


def make_linear(name: str, M: int, K: int, N: int, mask: torch.Tensor, seed: int, with_grad: bool = False,
                w_std: float = 0.02) -> LinearWorkload:
    gen = torch.Generator().manual_seed(seed)
    x = _randn_bf16((M, K), 1.0, gen)
    Wv = _randn_bf16((N, K), w_std, gen)
    Wt = _randn_bf16((N, K), w_std, gen)
    grad = _randn_bf16((M, N), 1.0, gen) if with_grad else None
    return LinearWorkload(name, x, Wv, Wt, mask.reshape(-1).clone(), grad)


def make_ffn(name: str, M: int, d: int, h: int, mask: torch.Tensor, seed: int, w_std: float = 0.02) -> FFNWorkload:
    gen = torch.Generator().manual_seed(seed)
    x = _randn_bf16((M, d), 1.0, gen)
    W = {}
    for k in ("w1", "w3", "u1", "u3"):
        W[k] = _randn_bf16((h, d), w_std, gen)
    for k in ("w2", "u2"):
        W[k] = _randn_bf16((d, h), w_std, gen)
    return FFNWorkload(name, x, W, mask.reshape(-1).clone())


# ---- the five configurations ----

def cfg1_linear_fwd(seed: int = 0) -> LinearWorkload:
    """MaskedLinear forward: M = 1 x 2048, K = N = 1024; two 576-token visual spans (56 % visual)."""
    gen = torch.Generator().manual_seed(1000 + seed)
    mask = span_mask(1, 2048, [2], gen)
    return make_linear("cfg1_linear_fwd_M2048_K1024_N1024", 2048, 1024, 1024, mask, seed)


def cfg2_ffn_fwd(seed: int = 0) -> FFNWorkload:
    """MaskedFFN forward: M = 4 x 2048, d = 1024, h = 2048; two visual spans per sequence."""
    gen = torch.Generator().manual_seed(2000 + seed)
    mask = span_mask(4, 2048, [2, 2, 2, 2], gen)
    return make_ffn("cfg2_ffn_fwd_M8192_d1024_h2048", 8192, 1024, 2048, mask, seed)


def cfg3_linear_bwd(seed: int = 0) -> LinearWorkload:
    """MaskedLinear backward: M = 8192, K = N = 1024, i.i.d. Bernoulli(0.5) mask."""
    gen = torch.Generator().manual_seed(3000 + seed)
    mask = bernoulli_mask(8192, 0.5, gen)
    return make_linear("cfg3_linear_bwd_M8192_K1024_N1024", 8192, 1024, 1024, mask, seed, with_grad=True)


def cfg4_mask(seed: int = 0, batch: int = 8, seq: int = 4096) -> torch.Tensor:
    """Per-sequence visual fraction from {0.0, 0.3, 0.7, 1.0} as 576-token blocks (0, 2, 5 blocks or
    the whole sequence); every fraction occurs at least once, order seeded."""
    gen = torch.Generator().manual_seed(4000 + seed)
    kinds = [0, 2, 5, -1]  # -1 = all visual
    picks = kinds + [kinds[i] for i in torch.randint(0, 4, (max(batch - 4, 0),), generator=gen).tolist()]
    picks = [picks[i] for i in torch.randperm(len(picks), generator=gen).tolist()][:batch]
    spans = [seq // IMAGE_TOKENS + 1 if k < 0 else k for k in picks]
    return span_mask(batch, seq, spans, gen)


def cfg4_ffn_fwd(seed: int = 0, batch: int = 8, seq: int = 4096, d: int = 4096, h: int = 14336) -> FFNWorkload:
    """MaskedFFN forward at LLM scale: M = 8 x 4096, d = 4096, h = 14336."""
    mask = cfg4_mask(seed, batch, seq)
    return make_ffn(f"cfg4_ffn_fwd_M{batch * seq}_d{d}_h{h}", batch * seq, d, h, mask, seed)


def cfg5_ffn_decode(M: int, kind: str = "bernoulli", seed: int = 0, d: int = 4096, h: int = 14336) -> FFNWorkload:
    """Decode-shaped MaskedFFN: M in {1, 8, 32, 64}; kind in {"bernoulli", "visual", "text"}."""
    gen = torch.Generator().manual_seed(5000 + seed + 17 * M)
    if kind == "bernoulli":
        mask = bernoulli_mask(M, 0.5, gen)
    elif kind == "visual":
        mask = torch.ones(M, dtype=torch.bool)
    elif kind == "text":
        mask = torch.zeros(M, dtype=torch.bool)
    else:
        raise ValueError(kind)
    return make_ffn(f"cfg5_ffn_decode_M{M}_{kind}_d{d}_h{h}", M, d, h, mask, seed)


def cfg5_inputs(M: int, kind: str = "bernoulli", seed: int = 0, d: int = 4096):
    """(x, mask) of cfg5_ffn_decode(M, kind, seed) without generating its weights (x is the first draw of
    that workload's generator), for callers that bring their own weight sets."""
    w_gen = torch.Generator().manual_seed(seed)
    x = _randn_bf16((M, d), 1.0, w_gen)
    gen = torch.Generator().manual_seed(5000 + seed + 17 * M)
    if kind == "bernoulli":
        mask = bernoulli_mask(M, 0.5, gen)
    elif kind in ("visual", "text"):
        mask = torch.full((M,), kind == "visual", dtype=torch.bool)
    else:
        raise ValueError(kind)
    return x, mask
