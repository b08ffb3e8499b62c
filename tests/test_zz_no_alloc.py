"""ffnk_masked_ffn_fwd_static: the MaskedFFN forward whose scratch is a static device array inside the
library (for callers that cannot allocate).  Called through the C ABI and compared bit for bit with
ffnk_masked_ffn_fwd, which runs the same kernels on a caller-supplied workspace; two calls in a row,
the second on a smaller input, so that what the first call left in the shared array is shown not to
matter."""
import pytest
import torch

from ffn_kernel_amd import _lib
from ffn_kernel_amd import workloads as wl

from helpers import assert_close, note
from oracle import cref

pytestmark = pytest.mark.gpu


def _args(w, out):
    M, d = w.x.shape
    h = w.h
    W = w.W
    return (w.x.data_ptr(), w.x.stride(0), W["w1"].data_ptr(), W["w3"].data_ptr(), W["u1"].data_ptr(),
            W["u3"].data_ptr(), 1, d, W["w2"].data_ptr(), W["u2"].data_ptr(), 1, h, w.mask.data_ptr(),
            out.data_ptr(), d, M, d, h)


def _with_workspace(w):
    lib = _lib.load()
    M, d = w.x.shape
    out = torch.full((M, d), float("nan"), device=w.x.device, dtype=torch.bfloat16)
    ws = torch.empty(_lib.workspace_bytes(_lib.OP_FFN_FWD, M, d, w.h), dtype=torch.uint8, device=w.x.device)
    rc = lib.ffnk_masked_ffn_fwd(*_args(w, out), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "ffnk_masked_ffn_fwd")
    torch.cuda.synchronize()
    return out


def _static(w):
    lib = _lib.load()
    M, d = w.x.shape
    out = torch.full((M, d), float("nan"), device=w.x.device, dtype=torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream
    # Once untimed: the first call on a GPU looks the scratch array's address up, and the runtime loads a
    # kernel's code the first time it is launched.  The call that counts must leave both of torch's
    # counters and the device's own free-memory figure where they were - the latter also sees a hipMalloc
    # made inside the library, which torch's allocator statistics would not.
    _lib.check(lib.ffnk_masked_ffn_fwd_static(*_args(w, out), stream), "ffnk_masked_ffn_fwd_static")
    torch.cuda.synchronize()
    out.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    rc = lib.ffnk_masked_ffn_fwd_static(*_args(w, out), stream)
    _lib.check(rc, "ffnk_masked_ffn_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before, "device memory was allocated during the call"
    return out


# (first call, second and smaller call): decode kernels (dot-product and LDS-transposed streams, with
# split-K partials in the scratch) and the LDS-tiled GEMMs (perm, counts, intermediate, split-K partials)
PAIRS = [
    ((64, 1024, 2048), (24, 1024, 2048)),
    ((8, 1024, 4096), (3, 512, 1024)),
    ((700, 512, 1024), (300, 256, 512)),
    ((256, 4096, 14336), (33, 4096, 14336)),
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_scratch_forward_matches_workspace_forward(dev, first, second):
    for n, (M, d, h) in enumerate((first, second)):
        note(f"ffnk_masked_ffn_fwd_static call {n} M={M} d={d} h={h}")
        assert _lib.workspace_bytes(_lib.OP_FFN_FWD, M, d, h) <= _lib.STATIC_SCRATCH_BYTES
        mask = torch.rand(M, generator=torch.Generator().manual_seed(M + n)) < 0.5
        w_cpu = wl.make_ffn("t", M, d, h, mask, seed=17 + M, w_std=0.03)
        w = w_cpu.to(dev)
        got = _static(w)
        want = _with_workspace(w)
        assert torch.equal(got, want), f"call {n}: static-scratch forward differs from the workspace forward"
        if M * d * h <= 64 * 1024 * 2048:
            assert_close(got, cref.ffn_fwd(w_cpu.x, w_cpu.W, w_cpu.mask, round_mid=True), f"call {n} vs oracle")


def test_static_scratch_forward_rejects_what_does_not_fit(dev):
    note("ffnk_masked_ffn_fwd_static size limit")
    lib = _lib.load()
    M, d, h = 32768, 4096, 14336
    assert _lib.workspace_bytes(_lib.OP_FFN_FWD, M, d, h) > _lib.STATIC_SCRATCH_BYTES
    # the size check comes before any pointer is looked at: no tensors of that size are needed
    rc = lib.ffnk_masked_ffn_fwd_static(0, d, 0, 0, 0, 0, 1, d, 0, 0, 1, h, 0, 0, d, M, d, h, 0)
    assert rc == -5  # FFNK_E_WORKSPACE
    with pytest.raises(ValueError, match="static"):
        _lib.check(rc, "ffnk_masked_ffn_fwd_static")


def test_static_scratch_is_looked_up_on_the_device_of_the_output(dev):
    """The scratch array's address is taken on the GPU that holds `out`, whatever the calling thread's
    current device: an output that is not device memory is refused before anything is launched."""
    note("ffnk_masked_ffn_fwd_static with a host output pointer")
    lib = _lib.load()
    host = torch.empty(64, 64, dtype=torch.bfloat16)
    rc = lib.ffnk_masked_ffn_fwd_static(0, 64, 0, 0, 0, 0, 1, 64, 0, 0, 1, 64, 0, host.data_ptr(), 64, 64, 64, 64, 0)
    assert rc == -1  # FFNK_E_NULL
    torch.cuda.synchronize()  # the refused query left no error behind for the next call
    assert torch.zeros(4, device=dev).sum().item() == 0
