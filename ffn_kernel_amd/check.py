"""Non-interactive counterpart of the reference's test_linear.py / test_ffn.py scripts
(test_linear.py:68-132, test_ffn.py:75-117, README.md:126-149): sweep sequence lengths, time the
plain-PyTorch modules (both branches + blend, on the GPU) against the MaskedLinear / MaskedFFN
modules, and with --check report the L2 distance of outputs (and gradients with --bwd).

    python -m ffn_kernel_amd.check linear [--bsz 1] [--bwd] [--check] [--max-mult 4]
    python -m ffn_kernel_amd.check ffn    [--bsz 1] [--bwd] [--check] [--max-mult 4] [--d 1024] [--h 2048]

Prints one JSON object per sequence length.  Exit status 1 if --check finds a relative L2 distance
above --tol.
"""
from __future__ import annotations

import argparse
import json
import random
import sys

import torch
import torch.nn as nn
import torch.nn.functional as F

from .modules import MaskedFFNModule, MaskedLinearModule


class TorchLinear(nn.Module):
    """Baseline: both Linears on every row, blended by the mask (test_linear.py:41-49)."""

    def __init__(self, in_dim, out_dim):
        super().__init__()
        self.linear_v = nn.Linear(in_dim, out_dim, bias=False)
        self.linear_t = nn.Linear(in_dim, out_dim, bias=False)

    def forward(self, x, visual_mask):
        m = visual_mask[:, :, None]
        return self.linear_v(x) * m + self.linear_t(x) * (~m)


class TorchFFN(nn.Module):
    """Baseline: both SwiGLU FFNs on every row, blended by the mask (test_ffn.py:32-47)."""

    def __init__(self, hidden_size, intermediate_size):
        super().__init__()
        mk = lambda i, o: nn.Linear(i, o, bias=False)
        self.w1, self.w2, self.w3 = mk(hidden_size, intermediate_size), mk(intermediate_size, hidden_size), mk(hidden_size, intermediate_size)
        self.u1, self.u2, self.u3 = mk(hidden_size, intermediate_size), mk(intermediate_size, hidden_size), mk(hidden_size, intermediate_size)

    def blend(self, x, mask):
        m = mask[:, :, None]
        p1 = F.silu(self.w1(x)) * self.w3(x)
        p2 = F.silu(self.u1(x)) * self.u3(x)
        return self.w2(p1) * m + self.u2(p2) * ~m

    @torch.no_grad()
    def forward(self, x, mask):  # the reference's module is forward-only (test_ffn.py:41)
        return self.blend(x, mask)


def generate_mask(batch_size, seq_len, image_size, rng, device):
    """One contiguous visual span of `image_size` tokens at a seeded position (test_linear.py:15-21)."""
    mask = torch.zeros((batch_size, seq_len), dtype=torch.bool, device=device)
    mid = rng.randint(image_size // 2, seq_len - image_size // 2)
    mask[:, mid - image_size // 2: mid + image_size // 2] = True
    return mask


def _time(fn, trials=10):
    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(trials):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    ts.sort()
    return ts[len(ts) // 2]


def _rel(a, b):
    return (torch.dist(a.float(), b.float()) / b.float().norm().clamp_min(1e-30)).item()


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m ffn_kernel_amd.check")
    ap.add_argument("op", choices=["linear", "ffn"])
    ap.add_argument("--bsz", type=int, default=1)
    ap.add_argument("--check", action="store_true")
    ap.add_argument("--bwd", action="store_true", help="include the backward")
    ap.add_argument("--max-mult", type=int, default=31, help="sweep seq_len = 2048 * i for i = 1..max-mult")
    ap.add_argument("--d", type=int, default=1024)
    ap.add_argument("--h", type=int, default=2048)
    ap.add_argument("--image-size", type=int, default=1024)
    ap.add_argument("--tol", type=float, default=2e-2, help="relative L2 bound between two bf16 results")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("ffn_kernel_amd.check needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    rng = random.Random(0)
    torch.manual_seed(0)
    if args.op == "linear":
        ref = TorchLinear(args.d, args.d).to(dev).bfloat16()
        mod = MaskedLinearModule(args.d, args.d, device=dev)
    else:
        ref = TorchFFN(args.d, args.h).to(dev).bfloat16()
        mod = MaskedFFNModule(args.d, args.h, device=dev)
    mod.load_state_dict(ref.state_dict())
    bad = False
    for i in range(1, args.max_mult + 1):
        seq = 2048 * i
        x = torch.rand((args.bsz, seq, args.d), dtype=torch.bfloat16, device=dev)
        mask = generate_mask(args.bsz, seq, args.image_size, rng, dev)
        rec = {"op": args.op, "bsz": args.bsz, "seq_len": seq}
        if args.check:
            if args.op == "linear":
                xs = []
                outs = []
                for m in (ref, mod):
                    m.zero_grad(set_to_none=True)
                    xi = x.clone().requires_grad_(True)
                    o = m(xi, mask)
                    o.sum().backward()
                    xs.append(xi)
                    outs.append(o)
                rec["rel_l2_out"] = _rel(outs[1], outs[0])
                rec["rel_l2_dx"] = _rel(xs[1].grad, xs[0].grad)
                rec["rel_l2_dWv"] = _rel(mod.linear_v.weight.grad, ref.linear_v.weight.grad)
                rec["rel_l2_dWt"] = _rel(mod.linear_t.weight.grad, ref.linear_t.weight.grad)
            elif args.bwd:
                xs = []
                for m, fwd in ((ref, ref.blend), (mod, mod)):
                    m.zero_grad(set_to_none=True)
                    xi = x.clone().requires_grad_(True)
                    o = fwd(xi, mask)
                    o.sum().backward()
                    xs.append((xi, o))
                rec["rel_l2_out"] = _rel(xs[1][1], xs[0][1])
                rec["rel_l2_dx"] = _rel(xs[1][0].grad, xs[0][0].grad)
                for k in ("w1", "w2", "w3", "u1", "u2", "u3"):
                    rec[f"rel_l2_d{k}"] = _rel(getattr(mod, k).weight.grad, getattr(ref, k).weight.grad)
            else:
                rec["rel_l2_out"] = _rel(mod(x, mask), ref(x, mask))
            rec["ok"] = all(v <= args.tol for k, v in rec.items() if k.startswith("rel_l2"))
            bad |= not rec["ok"]
        else:
            def run(m):
                if args.bwd:
                    m.zero_grad(set_to_none=True)
                    xi = x.clone().requires_grad_(True)
                    (m.blend if isinstance(m, TorchFFN) else m)(xi, mask).sum().backward()
                else:
                    with torch.no_grad():
                        m(x, mask)
            rec["pytorch_ms"] = _time(lambda: run(ref))
            rec["hip_ms"] = _time(lambda: run(mod))
            rec["speedup"] = rec["pytorch_ms"] / rec["hip_ms"]
        print(json.dumps(rec), flush=True)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
