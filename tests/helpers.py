"""Shared helpers of the GPU parity tests: call the C ABI through the package's ops and compare
against the CPU oracle."""
from __future__ import annotations

import torch

from oracle import cref
from oracle import modules as om


def note(msg: str) -> None:
    """Name the case before a GPU step so that a lost box still tells which case ran."""
    print(f"[gpu-case] {msg}", flush=True)


def assert_close(got: torch.Tensor, ref: torch.Tensor, what: str) -> dict:
    """bf16 tolerance against a high-precision reference: every element within 2e-2 (or one bf16 ulp
    of the reference where that is larger) and rel-L2 <= 5e-3."""
    rep = om.error_report(got.detach().float().cpu(), ref)
    assert om.within_tolerance(rep), f"{what}: {rep}"
    return rep


def assert_close_pipeline(got: torch.Tensor, ref: torch.Tensor, what: str) -> dict:
    """Tolerance for results that sit behind several bf16-stored stages (the MaskedFFN backward keeps
    t1, t3, dh, dt1, dt3 and the intermediate in bf16 between its GEMMs).  The reference rounds at the
    same places, but a stored value that lands on a rounding boundary can round the other way on the
    GPU (fp32 accumulation, __expf), and a weight gradient sums such one-ulp flips over the rows of a
    group: its error scales with the size of the summed terms, not with the (possibly cancelled)
    element.  Bound: rel-L2 <= 5e-3 and every element within max(2e-2, 2^-7 of the largest reference
    magnitude), i.e. about two bf16 ulps of the tensor's scale."""
    rep = om.error_report(got.detach().float().cpu(), ref)
    bound = max(om.MAX_ABS_TOL, rep["ref_abs_max"] * 2.0 ** -7)
    assert rep["max_abs"] <= bound and rep["rel_l2"] <= om.REL_L2_TOL, f"{what}: {rep} (bound {bound})"
    return rep


def assert_close_bf16_pair(got: torch.Tensor, other_bf16: torch.Tensor, what: str) -> dict:
    """Two bf16 results of the same maths (e.g. the kernel and the reference's bf16 PyTorch modules,
    which round after every Linear / silu / product): each is within the bounds above of the exact
    value, so they may differ from one another by twice those bounds, and the module form adds its
    intermediate roundings on top (four for the FFN: both projections, silu, product).  Bound used:
    every element within 4x (2e-2 or one bf16 ulp), rel-L2 <= 1.5e-2.  This is a sanity check
    against the reference's own formulation; the tight check is the one against the exact oracle."""
    rep = om.error_report(got.detach().float().cpu(), other_bf16.double())
    ok = rep["max_excess"] <= 4.0 and rep["rel_l2"] <= 3 * om.REL_L2_TOL
    assert ok, f"{what}: {rep}"
    return rep
