"""MaskedLinear / MaskedFFN — the torch.autograd.Function surface of the reference
(ffn_kernel/ops.py:9-38) on top of libffnk's HIP kernels.

Same class names, same positional signatures:
    MaskedLinear.apply(a, b1, b2, mask) -> c            b1 = W_v^T, b2 = W_t^T, views [K, N]
    MaskedFFN.apply(a, w1, w2, w3, u1, u2, u3, mask)    w1, w3, u1, u3 = [d, h]; w2, u2 = [h, d]
`mask` is a bool [M] tensor: True rows use b1 / w*, False rows use b2 / u*.
"""
from __future__ import annotations

import contextlib
import ctypes
import threading

import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import _lib


def _require_cuda_bf16(name: str, t: torch.Tensor, ndim: int) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if t.dim() != ndim:
        raise ValueError(f"{name} must be {ndim}-D, got shape {tuple(t.shape)}")
    if t.dtype != torch.bfloat16:
        raise ValueError(f"{name} must be torch.bfloat16, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on a GPU (got {t.device}); libffnk has no CPU path")


def _require_mask(mask: torch.Tensor, M: int, dev: torch.device) -> torch.Tensor:
    if not isinstance(mask, torch.Tensor) or mask.dtype != torch.bool:
        raise ValueError(f"mask must be a torch.bool tensor, got {getattr(mask, 'dtype', type(mask))}")
    if mask.dim() != 1 or mask.shape[0] != M:
        raise ValueError(f"mask must have shape [{M}], got {tuple(mask.shape)}")
    if mask.device != dev:
        raise ValueError(f"mask is on {mask.device}, inputs on {dev}")
    return mask if mask.stride(0) == 1 or M <= 1 else mask.contiguous()


def _rows_contiguous(t: torch.Tensor) -> torch.Tensor:
    """[M, K] rows the MFMA kernels can address: unit column stride, and - when K is a multiple of 8,
    i.e. when the fast path applies at all - a row stride that is a multiple of 8 elements on a
    16-byte aligned base.  Such views pass through without a copy; anything else is copied, as the
    reference's a.contiguous() / gd.contiguous() does for every input (linear.py:430, 463;
    ffn.py:533), so that an odd view never drops onto the slow any-stride kernels."""
    M, K = t.shape
    unit_cols = K <= 1 or t.stride(1) == 1
    rows_ok = M <= 1 or t.stride(0) >= K
    if unit_cols and rows_ok:
        if K % 8 != 0 or K == 0:
            return t  # the any-stride kernels take it as it is; a copy would not change the path
        if (M <= 1 or t.stride(0) % 8 == 0) and t.data_ptr() % 16 == 0:
            return t
    return t.contiguous()


def _k_major(w: torch.Tensor) -> torch.Tensor:
    """Logical [K, N] weight whose memory is [N, K] row-major (stride(0) == 1), the layout of
    nn.Linear.weight.T that the MFMA path reads directly.  Any other layout is re-laid once."""
    K, N = w.shape
    if (K <= 1 or w.stride(0) == 1) and (N <= 1 or w.stride(1) >= K):
        return w
    return w.t().contiguous().t()


def _same_device(dev, **tensors) -> None:
    for name, t in tensors.items():
        if t.device != dev:
            raise ValueError(f"{name} is on {t.device}, expected {dev}")


_NO_SWITCH = contextlib.nullcontext()


# The raw getters of torch's extension module: torch.cuda.current_device() / current_stream() wrap them in device
# look-ups and a Stream object that cost 1 and 4 us of a 20 us call.
_raw_device = getattr(torch._C, "_cuda_getDevice", None) or torch.cuda.current_device
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _on_device(dev: torch.device):
    """Context that makes `dev` the current device; nothing to enter when it already is (the usual case,
    and the device guard costs several microseconds of a 20 us call)."""
    return _NO_SWITCH if dev.index is None or _raw_device() == dev.index else torch.cuda.device(dev)


def _stream_ptr(dev: torch.device) -> int:
    """hipStream_t of torch's current stream on `dev`, as an integer."""
    if _raw_stream is not None:
        return _raw_stream(dev.index if dev.index is not None else _raw_device())
    return torch.cuda.current_stream(dev).cuda_stream


def _workspace(nbytes: int, dev: torch.device) -> torch.Tensor:
    # torch's caching allocator hands out 512-byte aligned blocks.
    return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)


def _wstrides(w: torch.Tensor):
    """(stride_k, stride_n) of a logical [K, N] weight with size-1 dimensions normalised."""
    K, N = w.shape
    sk = w.stride(0) if K > 1 else 1
    sn = w.stride(1) if N > 1 else max(K, 1)
    if sk == 1 and sn < K:  # both extents ambiguous only when a dimension is 1
        sn = K
    return sk, sn


class Routing:
    """A row partition on the device: perm int32[M] (visual rows first, each group ascending) and
    counts int32[2], as ffnk_route writes them.  One partition serves every operation that runs with the
    same mask - the projections of a layer, a forward and its backward - where the reference re-tests the
    mask inside every tile of every launch (linear.py:120-149, ffn.py:61-105)."""
    __slots__ = ("perm", "counts", "M", "_struct")

    def __init__(self, perm: torch.Tensor, counts: torch.Tensor):
        self.perm, self.counts, self.M = perm, counts, perm.shape[0]
        self._struct = _lib.RoutingStruct(perm.data_ptr(), counts.data_ptr())

    def ref(self):
        return ctypes.byref(self._struct)


def route(mask: torch.Tensor) -> Routing:
    """Partition the rows by mask on the mask's device and current stream (ffnk_route)."""
    if not isinstance(mask, torch.Tensor) or mask.dtype != torch.bool or mask.dim() != 1 or not mask.is_cuda:
        raise ValueError("route: mask must be a 1-D torch.bool tensor on a GPU")
    M, dev = mask.shape[0], mask.device
    mask = mask if mask.stride(0) == 1 or M <= 1 else mask.contiguous()
    buf = torch.empty(M + 2, dtype=torch.int32, device=dev)
    routing = Routing(buf[:M], buf[M:])
    with _on_device(dev):
        rc = _lib.load().ffnk_route(mask.data_ptr(), M, routing.perm.data_ptr(), routing.counts.data_ptr(), _stream_ptr(dev))
    _lib.check(rc, "ffnk_route")
    return routing


class _RouteCache(threading.local):
    """The last partition made on this thread and what it was made from."""
    enabled = True
    key = None
    mask = None     # keeps the mask's memory alive, so that its address cannot be handed to another tensor
    routing = None
    last = None     # the partition the last forward on this thread ran with (read back by the autograd functions)


_route_cache = _RouteCache()
_ROUTED_MIN_ROWS = 65  # up to 64 rows the weight-streaming kernels run, which read the mask themselves


def set_route_cache(enabled: bool) -> bool:
    """Switch the sharing of row partitions between calls on or off for this thread; returns the old setting."""
    old = _route_cache.enabled
    _route_cache.enabled = bool(enabled)
    if not enabled:
        _route_cache.key = _route_cache.mask = _route_cache.routing = None
    return old


def shared_routing(mask: torch.Tensor, M: int, stream: int | None = None):
    """The row partition for `mask` (contiguous, on a GPU), made once and shared by the calls that follow with
    the same mask: the operations of a transformer layer all route by one mask, and each would otherwise
    launch its own partition kernel ahead of its GEMM.  The one-entry cache is keyed on the address of the
    mask's first element (the entry keeps the tensor, so the memory cannot be handed to another one), the row
    count, the version counter - every in-place write through torch bumps it, so a mask changed in place is
    partitioned again - and the stream.  Returns None where no partition is shared: decode sizes, the cache
    switched off, tensors without a version counter, a stream under graph capture (a captured graph must not
    point at memory this cache may drop later)."""
    if M < _ROUTED_MIN_ROWS or not _route_cache.enabled:
        return None
    try:
        version = mask._version
    except RuntimeError:  # inference tensors keep no version counter
        return None
    if torch.cuda.is_current_stream_capturing():
        return None
    key = (mask.data_ptr(), M, version, _stream_ptr(mask.device) if stream is None else stream)
    if _route_cache.key == key:
        return _route_cache.routing
    routing = route(mask)
    _route_cache.key, _route_cache.mask, _route_cache.routing = key, mask, routing
    return routing


def _routing_arg(routing, mask: torch.Tensor, M: int, stream: int):
    """(Routing or None, its ffnk_routing_t* or None) for a call: the caller's, else the shared one."""
    if routing is None:
        routing = shared_routing(mask, M, stream)
    elif routing.M != M or routing.perm.device != mask.device:
        raise ValueError(f"routing is for {routing.M} rows on {routing.perm.device}, the call has {M} on {mask.device}")
    _route_cache.last = routing
    return routing, (routing.ref() if routing is not None else None)


def masked_linear_forward(a: torch.Tensor, b1: torch.Tensor, b2: torch.Tensor, mask: torch.Tensor,
                          routing: Routing | None = None) -> torch.Tensor:
    """c[m] = a[m] @ (b1 if mask[m] else b2).  Replaces _bf16_linear_forward (linear.py:418-452).
    routing: a partition of `mask` made by route(); None: the shared one (shared_routing)."""
    _require_cuda_bf16("a", a, 2)
    _require_cuda_bf16("b1", b1, 2)
    _require_cuda_bf16("b2", b2, 2)
    M, K = a.shape
    if b1.shape[0] != K or b2.shape != b1.shape:
        raise ValueError(f"weight shapes {tuple(b1.shape)}, {tuple(b2.shape)} do not match a {tuple(a.shape)}")
    N = b1.shape[1]
    dev = a.device
    _same_device(dev, b1=b1, b2=b2)
    mask = _require_mask(mask, M, dev)
    a = _rows_contiguous(a)
    if K > 1 and N > 1 and b1.stride() == (1, K) and b2.stride() == (1, K):
        sk, sn = 1, K  # nn.Linear.weight.T views: nothing to normalise
    else:
        b1, b2 = _k_major(b1), _k_major(b2)
        if _wstrides(b1) != _wstrides(b2):
            b2 = b2.t().contiguous().t()
            b1 = b1.t().contiguous().t()
        sk, sn = _wstrides(b1)
    c = torch.empty((M, N), device=dev, dtype=torch.bfloat16)
    if M == 0 or N == 0:
        return c
    lib = _lib.load()
    with _on_device(dev):
        stream = _stream_ptr(dev)
        routing, rt = _routing_arg(routing, mask, M, stream)
        ws_bytes = _lib.workspace_bytes(_lib.OP_LINEAR_FWD, M, K, N)
        ws = _workspace(ws_bytes, dev)
        rc = lib.ffnk_masked_linear_fwd_routed(a.data_ptr(), a.stride(0) if M > 1 else max(K, 1), b1.data_ptr(),
                                               b2.data_ptr(), sk, sn, mask.data_ptr(), c.data_ptr(), N, M, K, N,
                                               ws.data_ptr(), ws.numel(), stream, rt)
    _lib.check(rc, "ffnk_masked_linear_fwd")
    return c


def masked_linear_backward(grad: torch.Tensor, a: torch.Tensor, b1: torch.Tensor, b2: torch.Tensor,
                           mask: torch.Tensor, routing: Routing | None = None):
    """(da, db1, db2) of MaskedLinear.  Replaces _bf16_linear_backward (linear.py:455-496);
    db1/db2 keep b1's strides as the reference's empty_like(b1) does (linear.py:475)."""
    _require_cuda_bf16("grad", grad, 2)
    _require_cuda_bf16("a", a, 2)
    M, K = a.shape
    N = b1.shape[1]
    if grad.shape != (M, N):
        raise ValueError(f"grad shape {tuple(grad.shape)} != {(M, N)}")
    dev = a.device
    mask = _require_mask(mask, M, dev)
    grad = _rows_contiguous(grad)
    a = _rows_contiguous(a)
    if _wstrides(b1) != _wstrides(b2):
        b2 = b2.t().contiguous().t()
        b1 = b1.t().contiguous().t()
    sk, sn = _wstrides(b1)
    da = torch.empty((M, K), device=dev, dtype=torch.bfloat16)
    db1, db2 = torch.empty_like(b1), torch.empty_like(b2)
    if db1.stride() != db2.stride():
        db2 = torch.empty_strided(db1.shape, db1.stride(), device=dev, dtype=torch.bfloat16)
    dsk, dsn = _wstrides(db1)
    if K == 0:
        return da, db1, db2
    lib = _lib.load()
    with _on_device(dev):
        stream = _stream_ptr(dev)
        routing, rt = _routing_arg(routing, mask, M, stream)
        ws_bytes = _lib.workspace_bytes(_lib.OP_LINEAR_BWD, M, K, N)
        ws = _workspace(ws_bytes, dev)
        rc = lib.ffnk_masked_linear_bwd_routed(grad.data_ptr(), grad.stride(0) if M > 1 else max(N, 1), a.data_ptr(),
                                               a.stride(0) if M > 1 else max(K, 1), b1.data_ptr(), b2.data_ptr(), sk, sn,
                                               mask.data_ptr(), da.data_ptr(), K, db1.data_ptr(), db2.data_ptr(), dsk,
                                               dsn, M, K, N, ws.data_ptr(), ws.numel(), stream, rt)
    _lib.check(rc, "ffnk_masked_linear_bwd")
    return da, db1, db2


def masked_ffn_forward(a, w1, w2, w3, u1, u2, u3, mask, save_pre: bool = False, routing: Routing | None = None):
    """SwiGLU FFN routed by mask.  Replaces _bf16_ffn_forward + _bf16_linear_forward
    (ops.py:30-32, ffn.py:527-560).

    save_pre: also return the pre-activations [M, 2h] (routed order, gate | up) for
    masked_ffn_backward(..., pre=...), or None where the shape runs on a path that cannot keep them
    (decode sizes, d or h not a multiple of 8); the return value is then the pair (out, pre)."""
    _require_cuda_bf16("a", a, 2)
    for name, w in (("w1", w1), ("w2", w2), ("w3", w3), ("u1", u1), ("u2", u2), ("u3", u3)):
        _require_cuda_bf16(name, w, 2)
    M, d = a.shape
    h = w1.shape[1]
    for name, w in (("w1", w1), ("w3", w3), ("u1", u1), ("u3", u3)):
        if w.shape != (d, h):
            raise ValueError(f"{name} shape {tuple(w.shape)} != {(d, h)}")
    for name, w in (("w2", w2), ("u2", u2)):
        if w.shape[0] != h or w.shape != w2.shape:
            raise ValueError(f"{name} shape {tuple(w.shape)} does not match [h={h}, out]")
    d_out = w2.shape[1]
    if d_out != d:
        # The C entry point fuses both stages for the square case only; chain the two ops otherwise.
        raise ValueError(f"MaskedFFN needs w2/u2 of shape [{h}, {d}], got {tuple(w2.shape)}")
    dev = a.device
    _same_device(dev, w1=w1, w2=w2, w3=w3, u1=u1, u2=u2, u3=u3)
    mask = _require_mask(mask, M, dev)
    a = _rows_contiguous(a)
    ups = [_k_major(w) for w in (w1, w3, u1, u3)]
    if len({_wstrides(w) for w in ups}) != 1:
        ups = [w.t().contiguous().t() for w in ups]
    downs = [_k_major(w) for w in (w2, u2)]
    if len({_wstrides(w) for w in downs}) != 1:
        downs = [w.t().contiguous().t() for w in downs]
    usk, usn = _wstrides(ups[0])
    dsk, dsn = _wstrides(downs[0])
    out = torch.empty((M, d), device=dev, dtype=torch.bfloat16)
    if M == 0 or d == 0:
        return (out, None) if save_pre else out
    lib = _lib.load()
    pre = None
    if save_pre and h > 0 and lib.ffnk_masked_ffn_can_save(M, d, h) and usk == 1 and dsk == 1:
        pre = torch.empty((M, 2 * h), device=dev, dtype=torch.bfloat16)
    with _on_device(dev):
        stream = _stream_ptr(dev)
        routing, rt = _routing_arg(routing, mask, M, stream)
        ws_bytes = _lib.workspace_bytes(_lib.OP_FFN_FWD, M, d, h)
        ws = _workspace(ws_bytes, dev)
        head = (a.data_ptr(), a.stride(0) if M > 1 else max(d, 1), ups[0].data_ptr(), ups[1].data_ptr(),
                ups[2].data_ptr(), ups[3].data_ptr(), usk, usn, downs[0].data_ptr(), downs[1].data_ptr(), dsk, dsn,
                mask.data_ptr(), out.data_ptr(), d)
        tail = (M, d, h, ws.data_ptr(), ws.numel(), stream, rt)
        if pre is None:
            rc = lib.ffnk_masked_ffn_fwd_routed(*head, None, 0, *tail)
        else:
            rc = lib.ffnk_masked_ffn_fwd_routed(*head, pre.data_ptr(), 2 * h, *tail)
    _lib.check(rc, "ffnk_masked_ffn_fwd")
    return (out, pre) if save_pre else out


def masked_ffn_backward(grad, a, w1, w2, w3, u1, u2, u3, mask, pre=None, routing: Routing | None = None):
    """(da, dw1, dw2, dw3, du1, du2, du3) of MaskedFFN.  The reference stops at NotImplementedError
    here (ops.py:34-38); the decomposition follows its README sketch (README.md:159-172): routed
    GEMMs around one elementwise SwiGLU-gradient pass.  Weight gradients keep the strides of the
    weight views they belong to, as the linear backward's do.  pre: the pre-activations that
    masked_ffn_forward(..., save_pre=True) returned for the same inputs (read-only); None: they are
    recomputed."""
    _require_cuda_bf16("grad", grad, 2)
    _require_cuda_bf16("a", a, 2)
    for name, w in (("w1", w1), ("w2", w2), ("w3", w3), ("u1", u1), ("u2", u2), ("u3", u3)):
        _require_cuda_bf16(name, w, 2)
    M, d = a.shape
    h = w1.shape[1]
    if grad.shape != (M, d):
        raise ValueError(f"grad shape {tuple(grad.shape)} != {(M, d)}")
    for name, w in (("w1", w1), ("w3", w3), ("u1", u1), ("u3", u3)):
        if w.shape != (d, h):
            raise ValueError(f"{name} shape {tuple(w.shape)} != {(d, h)}")
    for name, w in (("w2", w2), ("u2", u2)):
        if w.shape != (h, d):
            raise ValueError(f"{name} shape {tuple(w.shape)} != {(h, d)}")
    if d % 8 or h % 8 or d == 0 or h == 0:
        raise ValueError(f"MaskedFFN backward needs d and h to be positive multiples of 8, got d={d}, h={h}")
    dev = a.device
    _same_device(dev, w1=w1, w2=w2, w3=w3, u1=u1, u2=u2, u3=u3, grad=grad)
    mask = _require_mask(mask, M, dev)
    grad = _rows_contiguous(grad)
    a = _rows_contiguous(a)
    # the up-projection weights must be K-contiguous ([h, d] memory, i.e. nn.Linear.weight.T views)
    ups = [w if _wstrides(w) == (1, d) else w.t().contiguous().t() for w in (w1, w3, u1, u3)]
    downs = [_k_major(w) for w in (w2, u2)]
    if len({_wstrides(w) for w in downs}) != 1:
        downs = [w.t().contiguous().t() for w in downs]
    usk, usn = _wstrides(ups[0])
    dsk, dsn = _wstrides(downs[0])
    da = torch.empty((M, d), device=dev, dtype=torch.bfloat16)
    dups = [torch.empty_strided(w1.shape, w1.stride(), device=dev, dtype=torch.bfloat16) for _ in range(4)]
    ddowns = [torch.empty_strided(w2.shape, w2.stride(), device=dev, dtype=torch.bfloat16) for _ in range(2)]
    gusk, gusn = _wstrides(dups[0])
    gdsk, gdsn = _wstrides(ddowns[0])
    lib = _lib.load()
    with _on_device(dev):
        # Sized for this layout when every weight is 16-byte aligned (what the lean query assumes), for any
        # layout otherwise: the usual views then skip the room for weight copies and transposed intermediates.
        if all(w.data_ptr() % 16 == 0 for w in (*ups, *downs)):
            ws_bytes = lib.ffnk_workspace_bytes_ffn_bwd(M, d, h, grad.stride(0) if M > 1 else d, usn, dsk, dsn, gusk, gdsk)
            if ws_bytes == (1 << 64) - 1:
                raise ValueError(f"ffnk_workspace_bytes_ffn_bwd: invalid extents M={M} d={d} h={h}")
        else:
            ws_bytes = _lib.workspace_bytes(_lib.OP_FFN_BWD, M, d, h)
        ws = _workspace(ws_bytes, dev)
        stream = _stream_ptr(dev)
        routing, rt = _routing_arg(routing, mask, M, stream)
        head = (grad.data_ptr(), grad.stride(0) if M > 1 else d, a.data_ptr(), a.stride(0) if M > 1 else d,
                ups[0].data_ptr(), ups[1].data_ptr(), ups[2].data_ptr(), ups[3].data_ptr(), usk, usn,
                downs[0].data_ptr(), downs[1].data_ptr(), dsk, dsn, mask.data_ptr())
        tail = (da.data_ptr(), d, dups[0].data_ptr(), dups[1].data_ptr(), dups[2].data_ptr(), dups[3].data_ptr(),
                gusk, gusn, ddowns[0].data_ptr(), ddowns[1].data_ptr(), gdsk, gdsn, M, d, h, ws.data_ptr(), ws.numel(),
                stream, rt)
        if pre is None:
            rc = lib.ffnk_masked_ffn_bwd_routed(*head, None, 0, *tail)
        else:
            if pre.shape != (M, 2 * h) or pre.dtype != torch.bfloat16 or pre.device != dev or pre.stride(1) != 1:
                raise ValueError(f"pre must be a bf16 [{M}, {2 * h}] tensor on {dev} with contiguous rows")
            rc = lib.ffnk_masked_ffn_bwd_routed(*head, pre.data_ptr(), pre.stride(0) if M > 1 else 2 * h, *tail)
    _lib.check(rc, "ffnk_masked_ffn_bwd")
    dw1, dw3, du1, du3 = dups
    dw2, du2 = ddowns
    return da, dw1, dw2, dw3, du1, du2, du3


class _GradMode(threading.local):
    enabled = True


_grad_mode = _GradMode()


class MaskedLinear(Function):
    """c = a @ (b1 where mask else b2), forward and backward (reference: ops.py:9-24)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, a, b1, b2, mask):
        ctx.save_for_backward(a, mask)
        ctx.b1, ctx.b2 = b1, b2
        _route_cache.last = None
        out = masked_linear_forward(a, b1, b2, mask)
        # the partition the forward ran with serves the backward too (autograd refuses a saved mask that
        # was changed in place, so it cannot go stale)
        ctx.routing = _route_cache.last
        return out

    @staticmethod
    @once_differentiable
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad):
        a, mask = ctx.saved_tensors
        da, db1, db2 = masked_linear_backward(grad, a, ctx.b1, ctx.b2, mask, routing=ctx.routing)
        return da, db1, db2, None


class MaskedFFN(Function):
    """Routed SwiGLU FFN (reference: ops.py:27-38).  The backward, which the reference leaves at
    NotImplementedError, uses the pre-activations that a forward with gradients requested keeps
    ([M, 2h] bf16; as the reference's unfinished training forward does, ffn.py:116-221), and
    recomputes them from the saved inputs where the forward could not keep them (decode sizes)."""

    @classmethod
    def apply(cls, *args, **kwargs):
        # forward() always runs with gradients switched off and ctx.needs_input_grad does not say whether
        # the caller is under torch.no_grad(): note it here, so that evaluation does not pay for keeping
        # the pre-activations
        _grad_mode.enabled = torch.is_grad_enabled()
        return super().apply(*args, **kwargs)

    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx, a, w1, w2, w3, u1, u2, u3, mask):
        ctx.weights = (w1, w2, w3, u1, u2, u3)
        _route_cache.last = None
        if _grad_mode.enabled and any(ctx.needs_input_grad):
            out, pre = masked_ffn_forward(a, w1, w2, w3, u1, u2, u3, mask, save_pre=True)
        else:
            out, pre = masked_ffn_forward(a, w1, w2, w3, u1, u2, u3, mask), None
        ctx.routing = _route_cache.last
        ctx.has_pre = pre is not None
        if pre is None:
            ctx.save_for_backward(a, mask)
        else:
            ctx.save_for_backward(a, mask, pre)
        return out

    @staticmethod
    @once_differentiable
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, grad):
        a, mask = ctx.saved_tensors[:2]
        pre = ctx.saved_tensors[2] if ctx.has_pre else None
        return (*masked_ffn_backward(grad, a, *ctx.weights, mask, pre=pre, routing=ctx.routing), None)
