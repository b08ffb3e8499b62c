"""Shared helpers of the GPU parity tests: call the C ABI through the package's ops and compare
against the CPU oracle."""
from __future__ import annotations

import torch

from oracle import cref
from oracle import modules as om


def note(msg: str) -> None:
    """Name the case before a GPU step so that a lost box still tells which case ran."""
    print(f"[gpu-case] {msg}", flush=True)


def assert_close(got: torch.Tensor, ref: torch.Tensor, what: str, scale_with_magnitude: bool = True) -> dict:
    rep = om.error_report(got.detach().float().cpu(), ref)
    assert om.within_tolerance(rep, scale_with_magnitude), f"{what}: {rep}"
    return rep
