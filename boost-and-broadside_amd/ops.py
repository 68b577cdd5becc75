"""Tensor-level front ends of the two HIP kernels.

``sdpa_masked`` stands in for the key-bias + ``F.scaled_dot_product_attention`` +
head-merge copy of the reference (models/yemong/attention.py:136-147,168);
``rglru_step`` stands in for the element-wise chain of ``RGLRU._step``
(models/yemong/griffin.py:179-185); ``conv_step`` for the padded ``cat``, the depthwise tap
loop and the buffer shift of the temporal block at T = 1 (griffin.py:127-139, 275-277).
All launch on torch's current stream, allocate their outputs with torch and never
synchronise.  They are forward-only and run on a ROCm device only: anything else raises.
"""

from __future__ import annotations

import os

import functools
import math

import torch

from . import _native

_DTYPE_CODE = {torch.float32: _native.F32, torch.bfloat16: _native.BF16}
def _outside_autocast(backward):
    """A custom Function's backward inherits the autocast state of the place ``.backward()`` is called
    from; inside it torch GEMMs would return bfloat16 tensors where the kernels are handed float32
    pointers.  Every backward here runs with autocast off and states its dtypes itself."""
    @functools.wraps(backward)
    def wrapped(ctx, *grads):
        with torch.autocast("cuda", enabled=False):
            return backward(ctx, *grads)
    return wrapped


_PATH_CODE = {"auto": _native.PATH_AUTO, "valu": _native.PATH_VALU, "mfma": _native.PATH_MFMA, "env": _native.PATH_ENV,
              "head": _native.PATH_HEAD}


def _need_device(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}; the attention/RG-LRU kernels only exist as HIP code for gfx950 "
            "and have no host fallback"
        )


def _code(t: torch.Tensor, name: str) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise TypeError(f"{name} must be float32 or bfloat16, got {t.dtype}") from None


_get_device = getattr(torch._C, "_cuda_getDevice", None)
_set_device = getattr(torch._C, "_cuda_setDevice", None)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """Raw handle of torch's current stream on the current device.  The direct query is what
    ``torch.cuda.current_stream().cuda_stream`` ends in, without building a Stream object on every launch
    (about 9 us of host time each; a small rollout step is bound by exactly that)."""
    if _raw_stream is not None and _get_device is not None:
        return _raw_stream(_get_device())
    return torch.cuda.current_stream().cuda_stream


class _on_device:
    """``with torch.cuda.device(d)`` that does nothing when ``d`` is already the current device, the usual case."""

    __slots__ = ("idx", "prev", "ctx")

    def __init__(self, device: torch.device) -> None:
        self.idx = device.index
        self.ctx = None

    def __enter__(self):
        if _get_device is None or _set_device is None or self.idx is None:
            self.ctx = torch.cuda.device(self.idx)
            return self.ctx.__enter__()
        self.prev = _get_device()
        if self.prev != self.idx:
            _set_device(self.idx)
        return None

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        if self.prev != self.idx:
            _set_device(self.prev)
        return False


def sdpa_masked(
    qkv: torch.Tensor,
    alive: torch.Tensor | None,
    n_heads: int,
    *,
    path: str = "auto",
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Masked multi-head attention over each environment's tokens.

    Args:
        qkv:     (B, NM, 3*D) packed projection, columns [Q | K | V], heads head-major
                 inside each third.  float32 or bfloat16; last dim contiguous, rows of an
                 environment and environments themselves evenly spaced (any row stride).
        alive:   (B, NM) bool (or uint8), True = the entity exists, or None for no mask.
                 Dead keys get weight 0; an environment with no live key averages V over
                 all keys; dead queries are still computed.
        n_heads: H; D must be divisible by it.
        path:    "auto" | "valu" | "mfma" | "env" — kernel selection, for tests and benchmarks ("mfma": one
                 work-group per (environment, head); "env": one per environment, heads streamed through LDS).
        out:     optional preallocated contiguous (B, NM, D) destination in qkv's dtype.

    Returns:
        (B, NM, D) in qkv's dtype, heads merged head-major (the input of ``out_proj``).
    """
    if qkv.dim() != 3 or qkv.shape[-1] % 3:
        raise ValueError(f"qkv must be (B, NM, 3*D), got {tuple(qkv.shape)}")
    _need_device(qkv, "qkv")
    dtype = _code(qkv, "qkv")
    B, NM, D3 = qkv.shape
    D = D3 // 3
    if n_heads < 1 or D % n_heads:
        raise ValueError(f"d_model={D} must be divisible by n_heads={n_heads}")
    if path not in _PATH_CODE:
        raise ValueError(f"path must be one of {sorted(_PATH_CODE)}, got {path!r}")
    if qkv.requires_grad and torch.is_grad_enabled():
        raise RuntimeError("sdpa_masked is forward-only; call it under torch.no_grad()")
    if B and NM and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NM * qkv.stride(1))):
        qkv = qkv.contiguous()
    mask_ptr = None
    if alive is not None:
        if alive.shape != (B, NM):
            raise ValueError(f"alive must be {(B, NM)}, got {tuple(alive.shape)}")
        if alive.dtype not in (torch.bool, torch.uint8):
            raise TypeError(f"alive must be bool or uint8, got {alive.dtype}")
        if alive.device != qkv.device:
            raise RuntimeError(f"alive is on {alive.device}, qkv on {qkv.device}")
        alive = alive.contiguous()
        mask_ptr = alive.data_ptr()
    if out is None:
        out = torch.empty((B, NM, D), dtype=qkv.dtype, device=qkv.device)
    elif out.shape != (B, NM, D) or out.dtype != qkv.dtype or out.device != qkv.device or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous {(B, NM, D)} {qkv.dtype} tensor on {qkv.device}")
    if B == 0 or NM == 0:
        return out
    with _on_device(qkv.device):
        rc = _native.load().bnb_sdpa_masked_fwd_path(
            qkv.data_ptr(), qkv.stride(1), mask_ptr, out.data_ptr(), B, NM, n_heads, D // n_heads, dtype,
            _PATH_CODE[path], _stream(),
        )
    _native.check(rc, "bnb_sdpa_masked_fwd")
    return out


def sdpa_train_supported(qkv: torch.Tensor, n_heads: int) -> bool:
    """Whether ``sdpa_train`` covers this input on the GPU: head size 32 and either at most 32 tokens and
    8 heads (float32 or bfloat16) or bfloat16 with at most 160 tokens."""
    if not (qkv.is_cuda and qkv.dim() == 3 and qkv.dtype in (torch.float32, torch.bfloat16) and qkv.shape[-1] % 3 == 0):
        return False
    D = qkv.shape[-1] // 3
    if D % n_heads or D // n_heads != 32 or qkv.shape[1] < 1:
        return False
    NM = qkv.shape[1]
    return (NM <= 32 and n_heads <= 8) or (qkv.dtype == torch.bfloat16 and NM <= 160)


def sdpa_masked_bwd(qkv: torch.Tensor, alive: torch.Tensor | None, n_heads: int, out: torch.Tensor,
                    dout: torch.Tensor, *, path: str = "auto") -> torch.Tensor:
    """Gradient of ``sdpa_masked`` with respect to ``qkv`` from the forward's result and its gradient.
    ``path``: "auto" | "valu" | "mfma" (kernel selection, for tests and benchmarks)."""
    B, NM, D3 = qkv.shape
    D = D3 // 3
    if out.shape != (B, NM, D) or dout.shape != (B, NM, D) or out.dtype != qkv.dtype:
        raise ValueError("out and dout must be (B, NM, D) in qkv's dtype")
    for name, t in (("qkv", qkv), ("out", out), ("dout", dout)):
        _need_device(t, name)
    if B and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NM * qkv.stride(1))):
        qkv = qkv.contiguous()
    out = out.contiguous()
    dout = dout.to(qkv.dtype).contiguous()
    mask_ptr = None
    if alive is not None:
        if alive.shape != (B, NM) or alive.dtype not in (torch.bool, torch.uint8):
            raise ValueError(f"alive must be a bool {(B, NM)} tensor")
        alive = alive.contiguous()
        mask_ptr = alive.data_ptr()
    dqkv = torch.empty((B, NM, D3), dtype=qkv.dtype, device=qkv.device)
    if B:
        with _on_device(qkv.device):
            rc = _native.load().bnb_sdpa_masked_bwd_path(qkv.data_ptr(), qkv.stride(1), mask_ptr, out.data_ptr(), dout.data_ptr(),
                                                         dqkv.data_ptr(), B, NM, n_heads, D // n_heads, _code(qkv, "qkv"),
                                                         _PATH_CODE[path], _stream())
        _native.check(rc, "bnb_sdpa_masked_bwd")
    return dqkv


class _SdpaTrain(torch.autograd.Function):
    """``sdpa_masked`` with its backward kernel."""

    @staticmethod
    def forward(ctx, qkv, alive, n_heads):
        with torch.no_grad():
            out = sdpa_masked(qkv, alive, n_heads)
        ctx.save_for_backward(qkv, out)
        ctx.alive = alive
        ctx.n_heads = n_heads
        return out

    @staticmethod
    @_outside_autocast
    def backward(ctx, dout):
        qkv, out = ctx.saved_tensors
        return sdpa_masked_bwd(qkv, ctx.alive, ctx.n_heads, out, dout), None, None


def sdpa_train(qkv: torch.Tensor, alive: torch.Tensor | None, n_heads: int) -> torch.Tensor:
    """Differentiable ``sdpa_masked`` (use where ``sdpa_train_supported`` holds)."""
    with torch.autocast("cuda", enabled=False):
        return _SdpaTrain.apply(qkv, alive, n_heads)


def cross_supported(q: torch.Tensor, kv: torch.Tensor, n_heads: int) -> bool:
    """Whether ``sdpa_cross`` covers these shapes: head size 32 and either bfloat16 with 1..2048 keys and
    at most 160 queries, or float32 with 1..4096 keys and at most 512 queries."""
    D = kv.shape[-1] // 2
    if not (q.is_cuda and q.dtype == kv.dtype and D % n_heads == 0 and D // n_heads == 32):
        return False
    if q.dtype == torch.bfloat16:
        return 1 <= kv.shape[1] <= 2048 and q.shape[1] <= 160
    return q.dtype == torch.float32 and 1 <= kv.shape[1] <= 4096 and q.shape[1] <= 512


def sdpa_cross(
    qkv: torch.Tensor,
    kv: torch.Tensor,
    key_mask: torch.Tensor | None,
    n_heads: int,
    *,
    accum: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Entity queries reading a second key/value set (the bullet read), on the matrix-core kernels
    (bfloat16, or float32 with true float32 products for evaluation without autocast).

    Args:
        qkv:      (B, NQ, 3*D) packed entity projection; only its Q third is read.
        kv:       (B, NK, 2*D) ``[K | V]`` of the other set (``kv_bullet``'s output).
        key_mask: (B, NK) bool, True = active, or None.  Inactive keys get weight 0; an
                  environment with no active key contributes exactly zero.
        accum:    optional (B, NQ, D) contiguous tensor the result is added to (and, unless
                  ``out`` is given, written into); default: the bare result in a new tensor.
        out:      optional (B, NQ, D) contiguous destination.

    Returns (B, NQ, D) in ``qkv``'s dtype.
    """
    B, NQ, D3 = qkv.shape
    D = D3 // 3
    NK = kv.shape[1]
    if kv.shape != (B, NK, 2 * D):
        raise ValueError(f"kv must be {(B, NK, 2 * D)}, got {tuple(kv.shape)}")
    if not cross_supported(qkv, kv, n_heads):
        raise RuntimeError("sdpa_cross covers head size 32 with bfloat16 (1..2048 keys, <= 160 queries) or "
                           "float32 (1..4096 keys, <= 512 queries), queries and keys in one dtype")
    if torch.is_grad_enabled() and (qkv.requires_grad or kv.requires_grad):
        raise RuntimeError("sdpa_cross is forward-only; call it under torch.no_grad()")
    if B and NQ and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NQ * qkv.stride(1))):
        qkv = qkv.contiguous()
    if B and (kv.stride(-1) != 1 or (B > 1 and kv.stride(0) != NK * kv.stride(1))):
        kv = kv.contiguous()
    mask_ptr = None
    if key_mask is not None:
        if key_mask.shape != (B, NK) or key_mask.dtype not in (torch.bool, torch.uint8):
            raise ValueError(f"key_mask must be a bool {(B, NK)} tensor")
        key_mask = key_mask.contiguous()
        mask_ptr = key_mask.data_ptr()
    if accum is not None and (accum.shape != (B, NQ, D) or accum.dtype != qkv.dtype or not accum.is_contiguous()):
        raise ValueError("accum must be a contiguous (B, NQ, D) tensor in qkv's dtype")
    if out is not None and (out.shape != (B, NQ, D) or out.dtype != qkv.dtype or not out.is_contiguous()):
        raise ValueError("out must be a contiguous (B, NQ, D) tensor in qkv's dtype")
    if out is None:
        out = accum if accum is not None else torch.empty((B, NQ, D), dtype=qkv.dtype, device=qkv.device)
    if B == 0 or NQ == 0:
        return out
    with _on_device(qkv.device):
        rc = _native.load().bnb_sdpa_cross_fwd(
            qkv.data_ptr(), qkv.stride(1), NQ, kv.data_ptr(), kv.data_ptr() + D * kv.element_size(), kv.stride(1), NK,
            mask_ptr, None if accum is None else accum.data_ptr(), out.data_ptr(), B, n_heads, D // n_heads,
            _code(qkv, "qkv"), _stream(),
        )
    _native.check(rc, "bnb_sdpa_cross_fwd")
    return out


def sdpa_cross_train_supported(qkv: torch.Tensor, kv: torch.Tensor, n_heads: int) -> bool:
    """Whether ``sdpa_cross_train`` covers these shapes: what ``sdpa_cross`` covers in bfloat16 (up to 2048 keys,
    160 queries)."""
    return cross_supported(qkv, kv, n_heads) and qkv.dtype == torch.bfloat16 and kv.dim() == 3 and qkv.dim() == 3


def sdpa_cross_stream_bwd(qkv, kv, rows: "CompactRows", n_heads, out, dout, *, indexed: bool, lse: torch.Tensor | None = None):
    """Gradients ``(dq (B, NQ, D), dkv)`` of the bullet read for any number of listed keys per environment.
    ``lse`` (B, n_heads, NQ) float32, optional: the log-sum-exp ``sdpa_cross_rows(..., lse=...)`` wrote in the forward
    pass over the same queries and keys; without it the first kernel recomputes it (a second pass over every key).

    ``indexed=False``: ``kv`` (capacity, 2D) holds ``[K | V]`` of the entries of ``rows`` in list order and
    ``dkv`` has that layout.  ``indexed=True``: ``kv`` is the (B, NK, 2D) buffer the mask of ``rows`` was
    taken over, read in place through the list; ``dkv`` (B, NK, 2D) is zero where the mask is."""
    B, NQ, D3 = qkv.shape
    D = D3 // 3
    for name, t in (("qkv", qkv), ("kv", kv), ("out", out), ("dout", dout)):
        _need_device(t, name)
        if t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be bfloat16")
    if rows.shape[0] != B or out.shape != (B, NQ, D) or dout.shape != (B, NQ, D) or NQ > 160 or D // n_heads != 32:
        raise ValueError("rows lists the keys of the B environments; out and dout are (B, NQ <= 160, D), heads of 32")
    if indexed:
        if kv.shape != (B, rows.shape[1], 2 * D):
            raise ValueError(f"kv must be {(B, rows.shape[1], 2 * D)}")
        if B and (kv.stride(-1) != 1 or kv.stride(1) != 2 * D or (B > 1 and kv.stride(0) != kv.shape[1] * 2 * D)):
            kv = kv.contiguous()
        dkv = torch.zeros_like(kv, memory_format=torch.contiguous_format)
        capacity = B * rows.shape[1]
    else:
        if kv.dim() != 2 or kv.shape[1] != 2 * D or not kv.is_contiguous():
            raise ValueError(f"kv must be a contiguous (capacity, {2 * D}) tensor")
        dkv = torch.empty_like(kv)
        capacity = kv.shape[0]
    if B and NQ and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NQ * qkv.stride(1))):
        qkv = qkv.contiguous()
    out, dout = out.contiguous(), dout.contiguous()
    dq = torch.empty((B, NQ, D), dtype=torch.bfloat16, device=qkv.device)
    if capacity == 0:
        return dq.zero_(), dkv
    if lse is not None and (lse.shape != (B, n_heads, NQ) or lse.dtype != torch.float32 or not lse.is_contiguous()
                            or lse.device != qkv.device):
        raise ValueError(f"lse must be a contiguous float32 {(B, n_heads, NQ)} tensor on the queries' device")
    if B and NQ:
        stats = torch.empty((B, n_heads, NQ, 2), dtype=torch.float32, device=qkv.device)
        lib = _native.load()
        with _on_device(qkv.device):
            if lse is None:
                rc = lib.bnb_sdpa_cross_stream_bwd(
                    qkv.data_ptr(), qkv.stride(1), NQ, kv.data_ptr(), 2 * D, rows.offsets.data_ptr(),
                    rows.index.data_ptr() if indexed else None, capacity, out.data_ptr(), dout.data_ptr(), dq.data_ptr(),
                    dkv.data_ptr(), stats.data_ptr(), B, n_heads, D // n_heads, _native.BF16, _stream())
            else:
                rc = lib.bnb_sdpa_cross_stream_bwd_lse(
                    qkv.data_ptr(), qkv.stride(1), NQ, kv.data_ptr(), 2 * D, rows.offsets.data_ptr(),
                    rows.index.data_ptr() if indexed else None, capacity, out.data_ptr(), dout.data_ptr(), lse.data_ptr(),
                    dq.data_ptr(), dkv.data_ptr(), stats.data_ptr(), B, n_heads, D // n_heads, _native.BF16, _stream())
        _native.check(rc, "bnb_sdpa_cross_stream_bwd")
    return dq, dkv


def sdpa_cross_bwd(qkv, kv, key_mask, n_heads, out, dout) -> tuple[torch.Tensor, torch.Tensor]:
    """Gradients ``(dq (B, NQ, D), dkv (B, NK, 2D))`` of ``sdpa_cross`` (without accumulator) from its
    result and that result's gradient; an environment without an active key gets zeros."""
    B, NQ, D3 = qkv.shape
    D = D3 // 3
    NK = kv.shape[1]
    for name, t in (("qkv", qkv), ("kv", kv), ("out", out), ("dout", dout)):
        _need_device(t, name)
        if t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be bfloat16")
    if kv.shape != (B, NK, 2 * D) or out.shape != (B, NQ, D) or dout.shape != (B, NQ, D):
        raise ValueError("kv must be (B, NK, 2D), out and dout (B, NQ, D)")
    if B and NQ and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NQ * qkv.stride(1))):
        qkv = qkv.contiguous()
    if B and (kv.stride(-1) != 1 or (B > 1 and kv.stride(0) != NK * kv.stride(1))):
        kv = kv.contiguous()
    out, dout = out.contiguous(), dout.contiguous()
    mask_ptr = None
    if key_mask is not None:
        if key_mask.shape != (B, NK) or key_mask.dtype not in (torch.bool, torch.uint8):
            raise ValueError(f"key_mask must be a bool {(B, NK)} tensor")
        key_mask = key_mask.contiguous()
        mask_ptr = key_mask.data_ptr()
    dq = torch.empty((B, NQ, D), dtype=torch.bfloat16, device=qkv.device)
    dkv = torch.empty((B, NK, 2 * D), dtype=torch.bfloat16, device=qkv.device)
    if B:
        with _on_device(qkv.device):
            rc = _native.load().bnb_sdpa_cross_bwd(qkv.data_ptr(), qkv.stride(1), NQ, kv.data_ptr(), kv.stride(1), NK, mask_ptr,
                                                   out.data_ptr(), dout.data_ptr(), dq.data_ptr(), dkv.data_ptr(), B, n_heads,
                                                   D // n_heads, _native.BF16, _stream())
        _native.check(rc, "bnb_sdpa_cross_bwd")
    return dq, dkv


class _SdpaCrossTrain(torch.autograd.Function):
    """``sdpa_cross`` (the read's own result, nothing accumulated) with its backward kernel."""

    @staticmethod
    def forward(ctx, qkv, kv, key_mask, n_heads):
        with torch.no_grad():
            out = sdpa_cross(qkv, kv, key_mask, n_heads)
        ctx.save_for_backward(qkv, kv, out)
        ctx.key_mask = key_mask
        ctx.n_heads = n_heads
        return out

    @staticmethod
    @_outside_autocast
    def backward(ctx, dout):
        qkv, kv, out = ctx.saved_tensors
        if kv.shape[1] <= 160:
            dq, dkv = sdpa_cross_bwd(qkv, kv, ctx.key_mask, ctx.n_heads, out, dout.to(torch.bfloat16))
        else:
            # long key axes: through the device-side list of the live slots (no copy to the host)
            mask = ctx.key_mask
            if mask is None:
                mask = torch.ones(kv.shape[:2], dtype=torch.bool, device=kv.device)
            dq, dkv = sdpa_cross_stream_bwd(qkv, kv, CompactRows(mask), ctx.n_heads, out, dout.to(torch.bfloat16), indexed=True)
        dqkv = torch.zeros_like(qkv)
        dqkv[..., : dq.shape[-1]] = dq
        return dqkv, dkv, None, None


def sdpa_cross_train(qkv: torch.Tensor, kv: torch.Tensor, key_mask: torch.Tensor | None, n_heads: int) -> torch.Tensor:
    """Differentiable ``sdpa_cross``: the entity queries' read of a second key/value set, (B, NQ, D)."""
    with torch.autocast("cuda", enabled=False):
        return _SdpaCrossTrain.apply(qkv, kv, key_mask, n_heads)


def sdpa_cross_rows_bwd(qkv, kv_rows, rows: "CompactRows", n_heads, out, dout, total: int, lse: torch.Tensor | None = None):
    """Gradients ``(dq (B, NQ, D), dkv_rows (total, 2D))`` of ``sdpa_cross_rows`` (without accumulator);
    ``total`` = ``rows.total_host()`` rows of ``kv_rows`` are valid.  ``lse``: what the forward wrote with
    ``sdpa_cross_rows(..., lse=...)``; used when some environment lists more than 160 keys (the streaming kernels)."""
    B, NQ, D3 = qkv.shape
    D = D3 // 3
    for name, t in (("qkv", qkv), ("kv_rows", kv_rows), ("out", out), ("dout", dout)):
        _need_device(t, name)
        if t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be bfloat16")
    if kv_rows.dim() != 2 or kv_rows.shape[1] != 2 * D or not kv_rows.is_contiguous() or kv_rows.shape[0] < total:
        raise ValueError(f"kv_rows must be a contiguous (>= {total}, {2 * D}) tensor")
    if rows.shape[0] != B or out.shape != (B, NQ, D) or dout.shape != (B, NQ, D):
        raise ValueError("rows must list the entries of the B environments; out and dout are (B, NQ, D)")
    if rows.max_count_host() > 160:
        return sdpa_cross_stream_bwd(qkv, kv_rows[:total], rows, n_heads, out, dout, indexed=False, lse=lse)
    if B and NQ and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NQ * qkv.stride(1))):
        qkv = qkv.contiguous()
    out, dout = out.contiguous(), dout.contiguous()
    dq = torch.empty((B, NQ, D), dtype=torch.bfloat16, device=qkv.device)
    dkv = torch.empty((total, 2 * D), dtype=torch.bfloat16, device=qkv.device)
    if total == 0:
        return dq.zero_(), dkv
    if B:
        with _on_device(qkv.device):
            rc = _native.load().bnb_sdpa_cross_ranges_bwd(qkv.data_ptr(), qkv.stride(1), NQ, kv_rows.data_ptr(), kv_rows.stride(0),
                                                          rows.offsets.data_ptr(), total, max(1, rows.max_count_host()), out.data_ptr(),
                                                          dout.data_ptr(),
                                                          dq.data_ptr(), dkv.data_ptr(), B, n_heads, D // n_heads, _native.BF16, _stream())
        _native.check(rc, "bnb_sdpa_cross_ranges_bwd")
    return dq, dkv


class _SdpaCrossRowsTrain(torch.autograd.Function):
    """``sdpa_cross_rows`` (nothing accumulated) with its backward kernel."""

    @staticmethod
    def forward(ctx, qkv, kv_rows, rows, n_heads, total):
        B, NQ, _ = qkv.shape
        # more keys than the single-tile backward takes: its streaming counterpart reuses the forward's log-sum-exp
        lse = (torch.empty((B, n_heads, NQ), dtype=torch.float32, device=qkv.device)
               if B and NQ and total and rows.max_count_host() > 160 else None)
        with torch.no_grad():
            out = sdpa_cross_rows(qkv, kv_rows, rows, n_heads, total=total, lse=lse)
        ctx.save_for_backward(qkv, kv_rows, out)
        ctx.rows, ctx.n_heads, ctx.total, ctx.lse = rows, n_heads, total, lse
        return out

    @staticmethod
    @_outside_autocast
    def backward(ctx, dout):
        qkv, kv_rows, out = ctx.saved_tensors
        dq, dkv = sdpa_cross_rows_bwd(qkv, kv_rows, ctx.rows, ctx.n_heads, out, dout.to(torch.bfloat16), ctx.total, ctx.lse)
        dqkv = torch.zeros_like(qkv)
        dqkv[..., : dq.shape[-1]] = dq
        return dqkv, dkv, None, None, None


def sdpa_cross_rows_train(qkv: torch.Tensor, kv_rows: torch.Tensor, rows: "CompactRows", n_heads: int) -> torch.Tensor:
    """Differentiable ``sdpa_cross_rows``: ``kv_rows`` holds exactly ``rows.total_host()`` rows, ``[K | V]`` of the
    listed entries in list order (bfloat16).  Needs head size 32 and at most 160 queries; any number of entries per
    row of the mask (up to 160 on the single-tile backward kernel, more on the streaming one)."""
    total = rows.total_host()
    if kv_rows.shape[0] != total:
        raise ValueError(f"kv_rows must hold the {total} listed rows")
    with torch.autocast("cuda", enabled=False):
        return _SdpaCrossRowsTrain.apply(qkv, kv_rows.contiguous(), rows, n_heads, total)


def rglru_step(
    x: torch.Tensor,
    gates_pre: torch.Tensor,
    log_lambda: torch.Tensor,
    c: float,
    h: torch.Tensor,
    *,
    h_out: torch.Tensor | None = None,
    y_dtype: torch.dtype | None = None,
    y_out: torch.Tensor | None = None,
    reset: torch.Tensor | None = None,
    rows_per_env: int = 1,
) -> tuple[torch.Tensor, torch.Tensor]:
    """One RG-LRU step given the two gate pre-activations.

    Args:
        x:          (R, D) input rows, float32 or bfloat16.
        gates_pre:  (R, 2*D): ``[linear_a(x) | linear_x(x)]`` with biases, float32 or bfloat16.
        log_lambda: (D,) float32 parameter.
        c:          exponent constant (8.0 in the reference).
        h:          (R, D) float32 previous state; rows may be strided (a view into the
                    packed (.., 4*D) hidden tensor works), the last dim must be contiguous.
        h_out:      optional float32 (R, D) destination (rows may be strided; may be ``h``
                    itself for an in-place update).  Default: a new contiguous tensor.
        y_dtype:    dtype of the returned layer output.  None or float32 returns the new
                    state itself; bfloat16 makes the kernel write a rounded copy as well.
        y_out:      optional preallocated destination of the layer output, float32 or bfloat16:
                    contiguous (R, D), or a (B, rows_per_env, D) view into a wider token tensor
                    (``tokens[:, :n]``), which the kernel then fills in place.
        reset:      optional (R / rows_per_env,) bool: environments whose previous state must
                    read as zero (``reset_hidden_for_envs`` folded into this step).
        rows_per_env: consecutive rows that belong to one environment (rows are env-major).

    Returns:
        (y, h_new): layer output and new state (the same tensor unless y_dtype is bfloat16).
    """
    if x.dim() != 2 or gates_pre.dim() != 2 or h.dim() != 2:
        raise ValueError("x, gates_pre and h must be 2-D (rows, channels)")
    R, D = x.shape
    if gates_pre.shape != (R, 2 * D) or h.shape != (R, D) or log_lambda.shape != (D,):
        raise ValueError(
            f"shape mismatch: x {tuple(x.shape)}, gates_pre {tuple(gates_pre.shape)}, h {tuple(h.shape)}, "
            f"log_lambda {tuple(log_lambda.shape)}"
        )
    for name, t in (("x", x), ("gates_pre", gates_pre), ("log_lambda", log_lambda), ("h", h)):
        _need_device(t, name)
    if h.dtype != torch.float32 or log_lambda.dtype != torch.float32:
        raise TypeError("h and log_lambda must be float32 (the recurrent state is never stored narrower)")
    if torch.is_grad_enabled() and (x.requires_grad or gates_pre.requires_grad or h.requires_grad):
        raise RuntimeError("rglru_step is forward-only; call it under torch.no_grad()")
    x_code, g_code = _code(x, "x"), _code(gates_pre, "gates_pre")
    x = x.contiguous()
    gates_pre = gates_pre.contiguous()
    log_lambda = log_lambda.detach().contiguous()
    if R and h.stride(-1) != 1:
        h = h.contiguous()
    if h_out is None:
        h_out = torch.empty((R, D), dtype=torch.float32, device=x.device)
    else:
        if h_out.shape != (R, D) or h_out.dtype != torch.float32 or h_out.device != x.device:
            raise ValueError("h_out must be a float32 (R, D) tensor on x's device")
        if R and h_out.stride(-1) != 1:
            raise ValueError("h_out must be contiguous in its last dim")
    y, y_group = None, 0
    if y_out is not None:
        # caller-owned destination in either dtype; a (B, n, D) view puts the rows of every
        # environment into a wider token tensor
        if y_out.dtype not in _DTYPE_CODE or y_out.device != x.device:
            raise ValueError("y_out must be a float32 or bfloat16 tensor on x's device")
        if y_dtype is not None and y_dtype != y_out.dtype:
            raise ValueError("y_dtype and y_out disagree")
        if y_out.dim() == 3:
            y_group, _ = _grouped_rows(y_out, R, D, rows_per_env, "y_out")
        elif y_out.shape != (R, D) or not y_out.is_contiguous():
            raise ValueError("y_out must be a contiguous (R, D) tensor or a (B, n, D) view")
        y = y_out
    elif y_dtype is not None and y_dtype != torch.float32:
        if y_dtype != torch.bfloat16:
            raise TypeError(f"y_dtype must be float32 or bfloat16, got {y_dtype}")
        y = torch.empty((R, D), dtype=torch.bfloat16, device=x.device)
    reset_ptr = _reset_pointer(reset, R, rows_per_env, x.device)
    if R == 0:
        return (h_out if y is None else y), h_out
    with _on_device(x.device):
        rc = _native.load().bnb_rglru_step_rows_fwd(
            x.data_ptr(), x_code, gates_pre.data_ptr(), g_code, log_lambda.data_ptr(), float(c),
            h.data_ptr(), h.stride(0), h_out.data_ptr(), h_out.stride(0),
            None if y is None else y.data_ptr(), _native.BF16 if y is None else _DTYPE_CODE[y.dtype], int(y_group),
            reset_ptr, int(rows_per_env), R, D, _stream(),
        )
    _native.check(rc, "bnb_rglru_step_fwd")
    return (h_out if y is None else y), h_out


def _grouped_rows(t: torch.Tensor, R: int, D: int, rows_per_env: int, name: str, pitch_ok: bool = False):
    """(group stride, row stride) in elements of a (B, n, D) view whose rows are the R = B*n rows
    of one environment after the other inside a wider tensor: ``t[b, i]`` at
    ``b * stride(0) + i * stride(1)``.  ``pitch_ok`` allows rows further apart than D (a column
    block of a wider matrix)."""
    if t.dim() != 3 or t.shape[2] != D or t.shape[0] * t.shape[1] != R:
        raise ValueError(f"{name} must be (R, D) or a (B, n, D) view with B*n == R")
    if t.shape[1] != rows_per_env:
        raise ValueError(f"{name} groups rows by {t.shape[1]}, rows_per_env is {rows_per_env}")
    row = t.stride(1) if t.shape[1] > 1 else D
    if R and (t.stride(2) != 1 or (row != D and not pitch_ok) or row < D or row % 8
              or (t.shape[0] > 1 and (t.stride(0) < t.shape[1] * row or t.stride(0) % 8))):
        raise ValueError(f"{name} must have contiguous rows at a regular pitch and a group stride that is a multiple of 8")
    return (t.stride(0) if t.shape[0] > 1 else t.shape[1] * row), row


def _reset_pointer(reset, R: int, rows_per_env: int, device) -> int | None:
    """Validate an optional per-environment reset mask and return its device address."""
    if reset is None:
        return None
    if rows_per_env < 1 or R % rows_per_env:
        raise ValueError(f"rows_per_env={rows_per_env} does not divide the {R} rows")
    if reset.shape != (R // rows_per_env,) or reset.dtype not in (torch.bool, torch.uint8):
        raise ValueError(f"reset must be a bool ({R // rows_per_env},) tensor, got {tuple(reset.shape)} {reset.dtype}")
    if reset.device != device or not reset.is_contiguous():
        raise ValueError("reset must be contiguous and on the same device as the rows")
    return reset.data_ptr()


def conv_step(
    b1: torch.Tensor,
    conv_buf: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    *,
    conv_out: torch.Tensor | None = None,
    reset: torch.Tensor | None = None,
    rows_per_env: int = 1,
    also_bf16: bool = False,
):
    """Causal depthwise conv of one timestep and the shift of the stored inputs.

    Args:
        b1:       (R, D) this step's ``linear1`` output, float32 or bfloat16; or a
                  (B, rows_per_env, D) view into a wider token tensor (``tokens[:, :n]``).
        conv_buf: (R, 3, D) float32 previous inputs, oldest first; each row's 3*D values must
                  be contiguous, rows may be strided (a view of the packed hidden works).
        weight:   (D, 4) or (D, 1, 4) float32 depthwise taps (``conv.weight``).
        bias:     (D,) float32 or None.
        conv_out: optional (R, 3, D) float32 destination with the same layout rules (may be
                  ``conv_buf`` itself).  Default: a new contiguous tensor.
        reset, rows_per_env: as in ``rglru_step``: environments whose stored inputs read as zero.
        also_bf16: also write a bfloat16 copy of the conv output (the input autocast would
                  feed the gate projections) and return it as a third value.

    Returns:
        (v, new_conv_buf[, v_bf16]): conv output (R, D) float32, the shifted buffer
        ``[p1, p2, b1]``, and the bfloat16 copy when asked for.
    """
    if b1.dim() not in (2, 3) or conv_buf.dim() != 3:
        raise ValueError("b1 must be (R, D) or a (B, rows_per_env, D) view, and conv_buf (R, 3, D)")
    D = b1.shape[-1]
    R = b1.numel() // D if D else 0
    if conv_buf.shape != (R, 3, D):
        raise ValueError(f"conv_buf must be {(R, 3, D)}, got {tuple(conv_buf.shape)}")
    for name, t in (("b1", b1), ("conv_buf", conv_buf), ("weight", weight)):
        _need_device(t, name)
    if conv_buf.dtype != torch.float32 or weight.dtype != torch.float32 or (bias is not None and bias.dtype != torch.float32):
        raise TypeError("conv_buf, weight and bias must be float32")
    if torch.is_grad_enabled() and (b1.requires_grad or conv_buf.requires_grad):
        raise RuntimeError("conv_step is forward-only; call it under torch.no_grad()")
    b_code = _code(b1, "b1")
    weight = weight.detach().reshape(D, 4).contiguous()
    bias_ptr = None
    if bias is not None:
        bias = bias.detach().contiguous()
        bias_ptr = bias.data_ptr()
    b1_group, b1_row = 0, 0
    if b1.dim() == 3 and not b1.is_contiguous():
        # rows of every environment inside a wider tensor (and possibly a column block of it)
        b1_group, b1_row = _grouped_rows(b1, R, D, rows_per_env, "b1", pitch_ok=True)
    else:
        b1 = b1.contiguous()

    def rows_ok(t):
        return R == 0 or (t.stride(2) == 1 and t.stride(1) == D)

    if not rows_ok(conv_buf):
        conv_buf = conv_buf.contiguous()
    if conv_out is None:
        conv_out = torch.empty((R, 3, D), dtype=torch.float32, device=b1.device)
    elif conv_out.shape != (R, 3, D) or conv_out.dtype != torch.float32 or conv_out.device != b1.device or not rows_ok(conv_out):
        raise ValueError("conv_out must be a float32 (R, 3, D) tensor on b1's device with contiguous rows")
    v = torch.empty((R, D), dtype=torch.float32, device=b1.device)
    v_lp = torch.empty((R, D), dtype=torch.bfloat16, device=b1.device) if also_bf16 else None
    reset_ptr = _reset_pointer(reset, R, rows_per_env, b1.device)
    if R:
        with _on_device(b1.device):
            rc = _native.load().bnb_conv_step_rows_fwd(
                b1.data_ptr(), b_code, int(b1_group), int(b1_row), conv_buf.data_ptr(), conv_buf.stride(0), weight.data_ptr(), bias_ptr,
                reset_ptr, int(rows_per_env), v.data_ptr(), None if v_lp is None else v_lp.data_ptr(),
                conv_out.data_ptr(), conv_out.stride(0), R, D, _stream(),
            )
        _native.check(rc, "bnb_conv_step_fwd")
    return (v, conv_out, v_lp) if also_bf16 else (v, conv_out)


def linear_wgrad_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether ``linear_wgrad`` covers this layer: GPU, both weight dimensions multiples of 128."""
    return x.is_cuda and weight.dim() == 2 and weight.shape[0] % 128 == 0 and weight.shape[1] % 128 == 0


def linear_wgrad(dy: torch.Tensor, x: torch.Tensor, out: torch.Tensor | None = None, accumulate: bool = False) -> torch.Tensor:
    """``dW = dy^T x`` for a Linear layer: ``dy`` (..., N) and ``x`` (..., K) bfloat16 with the same
    leading shape, result (N, K) float32 (``out`` is overwritten, or added to with ``accumulate``).
    Rows are reduced in a fixed order, so repeated calls give identical bits."""
    N, K = dy.shape[-1], x.shape[-1]
    if dy.dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
        raise TypeError("dy and x must be bfloat16")
    if dy.shape[:-1] != x.shape[:-1]:
        raise ValueError(f"dy {tuple(dy.shape)} and x {tuple(x.shape)} must share their leading shape")
    if N % 128 or K % 128:
        raise ValueError("linear_wgrad covers weight shapes whose dimensions are multiples of 128")
    _need_device(dy, "dy")
    _need_device(x, "x")
    dy2 = dy.reshape(-1, N) if _uniform_rows(dy, N) else dy.reshape(-1, N).contiguous()
    x2 = x.reshape(-1, K) if _uniform_rows(x, K) else x.reshape(-1, K).contiguous()
    R = dy2.shape[0]
    if out is None:
        if accumulate:
            raise ValueError("accumulate needs an existing out tensor")
        out = torch.empty((N, K), dtype=torch.float32, device=dy.device)
    elif out.shape != (N, K) or out.dtype != torch.float32 or not out.is_contiguous() or out.device != dy.device:
        raise ValueError("out must be a contiguous float32 (N, K) tensor on dy's device")
    lib = _native.load()
    slices = int(lib.bnb_linear_wgrad_slices(R, N, K))
    partials = torch.empty((slices, N, K), dtype=torch.float32, device=dy.device)
    with _on_device(dy.device):
        rc = lib.bnb_linear_wgrad_fwd(dy2.data_ptr(), dy2.stride(0) if R else N, x2.data_ptr(), x2.stride(0) if R else K,
                                      partials.data_ptr(), slices, out.data_ptr(), int(bool(accumulate)), R, N, K, _stream())
    _native.check(rc, "bnb_linear_wgrad_fwd")
    return out


def _linear_wgrad_tiled(dy_tiles: torch.Tensor, x_tiles: torch.Tensor, R: int) -> torch.Tensor:
    """``dW = dy^T x`` over the first R rows of operands stored tile by tile: ``dy_tiles`` (N/128, >= R, 128) and
    ``x_tiles`` (K/128, >= R, 128) contiguous bfloat16 (a plain (>= R, 128) matrix is one tile).  Returns (N, K) float32."""
    if dy_tiles.dim() == 2:
        dy_tiles = dy_tiles.unsqueeze(0)
    if x_tiles.dim() == 2:
        x_tiles = x_tiles.unsqueeze(0)
    for t, name in ((dy_tiles, "dy_tiles"), (x_tiles, "x_tiles")):
        _need_device(t, name)
        if t.dtype != torch.bfloat16 or not t.is_contiguous() or t.dim() != 3 or t.shape[2] != 128 or t.shape[1] < R:
            raise ValueError(f"{name} must be a contiguous bfloat16 (tiles, >= {R}, 128) tensor")
    N, K = 128 * dy_tiles.shape[0], 128 * x_tiles.shape[0]
    out = torch.empty((N, K), dtype=torch.float32, device=dy_tiles.device)
    lib = _native.load()
    slices = int(lib.bnb_linear_wgrad_slices(R, N, K))
    partials = torch.empty((slices, N, K), dtype=torch.float32, device=dy_tiles.device)
    with _on_device(dy_tiles.device):
        rc = lib.bnb_linear_wgrad_tiled_fwd(dy_tiles.data_ptr(), 128, max(dy_tiles.shape[1], 1) * 128, x_tiles.data_ptr(), 128,
                                            max(x_tiles.shape[1], 1) * 128, partials.data_ptr(), slices, out.data_ptr(), 0, R, N, K,
                                            _stream())
    _native.check(rc, "bnb_linear_wgrad_tiled_fwd")
    return out


def column_sums_supported(x: torch.Tensor) -> bool:
    """Whether ``column_sums`` covers this matrix: bfloat16 or float32 rows on the GPU, a width that is a
    multiple of 64 up to 2048, rows a multiple of 8 elements apart."""
    return (x.is_cuda and x.dim() == 2 and x.dtype in (torch.bfloat16, torch.float32) and x.shape[1] % 64 == 0
            and 0 < x.shape[1] <= 2048 and x.stride(1) == 1 and (x.shape[0] <= 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0)


def column_sums(x: torch.Tensor) -> torch.Tensor:
    """``x.sum(dim=0, dtype=float32)`` of a (R, N) matrix (a bias gradient) with the rows added in a fixed order."""
    if not column_sums_supported(x):
        raise ValueError(f"column_sums does not cover {x.dtype} {tuple(x.shape)} with strides {x.stride()}")
    R, N = x.shape
    lib = _native.load()
    slices = int(lib.bnb_column_sums_slices(R, N))
    partials = torch.empty((slices, N), dtype=torch.float32, device=x.device)
    out = torch.empty((N,), dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        rc = lib.bnb_column_sums(x.data_ptr(), _DTYPE_CODE[x.dtype], x.stride(0) if R > 1 else N, partials.data_ptr(), slices,
                                 out.data_ptr(), 0, R, N, _stream())
    _native.check(rc, "bnb_column_sums")
    return out


class _LinearTrain(torch.autograd.Function):
    """``F.linear`` under bfloat16 autocast whose weight gradient runs on ``linear_wgrad``."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        xb = x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)
        wb = weight.to(torch.bfloat16)
        ctx.save_for_backward(xb, wb)
        ctx.x_dtype = x.dtype
        ctx.has_bias = bias is not None
        return torch.nn.functional.linear(xb, wb, None if bias is None else bias.to(torch.bfloat16))

    @staticmethod
    @_outside_autocast
    def backward(ctx, dy):
        xb, wb = ctx.saved_tensors
        dy = dy.contiguous() if dy.stride(-1) != 1 else dy
        dyb = dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = torch.matmul(dyb, wb)
            if dx.dtype != ctx.x_dtype:
                dx = dx.to(ctx.x_dtype)
        if ctx.needs_input_grad[1]:
            dw = linear_wgrad(dyb, xb)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            rows = dyb.reshape(-1, dyb.shape[-1])
            db = column_sums(rows) if column_sums_supported(rows) else rows.sum(dim=0, dtype=torch.float32)
        return dx, dw, db


def linear_train(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
    """``F.linear(x, weight, bias)`` as bfloat16 autocast computes it, differentiable, with the weight
    gradient accumulated in float32 by ``linear_wgrad`` instead of a library GEMM that contracts
    over the (very long) row axis.  Use where ``linear_wgrad_supported`` holds."""
    with torch.autocast("cuda", enabled=False):
        return _LinearTrain.apply(x, weight, bias)


def pack_team_pool_weights(seeds: torch.Tensor, in_proj_weight: torch.Tensor, out_proj_weight: torch.Tensor,
                           n_heads: int) -> tuple[torch.Tensor, torch.Tensor]:
    """The constants ``team_pool`` needs, from TeamPMA's parameters (policy.py:88-92), float32:
    the 2H score vectors ``W_k[hs]^T (W_q seeds[t])[hs] * log2(e) / sqrt(dh)`` (row ``t*H + h``) and
    the (H*D, D) matrix whose rows ``h*D..`` are ``(out_proj.weight[:, hs] W_v[hs, :])^T``."""
    D = seeds.shape[-1]
    if seeds.shape != (2, D) or in_proj_weight.shape != (3 * D, D) or out_proj_weight.shape != (D, D) or D % n_heads:
        raise ValueError("expected seeds (2, D), in_proj_weight (3D, D), out_proj_weight (D, D), D divisible by n_heads")
    dh = D // n_heads
    with torch.no_grad(), torch.autocast(seeds.device.type, enabled=False):  # these constants stay float32
        w = in_proj_weight.detach().float()
        wq, wk, wv = w[:D], w[D:2 * D], w[2 * D:]
        q = (seeds.detach().float() @ wq.t()).view(2, n_heads, dh)                 # (t, h, dh)
        u = torch.einsum("thd,hdc->thc", q, wk.view(n_heads, dh, D)) * (math.log2(math.e) / math.sqrt(dh))
        wo = out_proj_weight.detach().float().view(D, n_heads, dh)                   # (o, h, dh)
        m = torch.einsum("ohd,hdc->hco", wo, wv.view(n_heads, dh, D))                # (h, c, o) = (W_o[:, hs] W_v[hs, :])^T
        return u.reshape(2 * n_heads, D).contiguous(), m.reshape(n_heads * D, D).contiguous()


def team_pool_supported(x: torch.Tensor, n_heads: int) -> bool:
    """Whether ``team_pool`` covers this input: float32 rows of 128 channels on the GPU, 2 or 4 heads."""
    return x.is_cuda and x.dtype == torch.float32 and x.dim() == 3 and x.shape[-1] == FFN_WIDTH and n_heads in (2, 4)


def team_pool(x: torch.Tensor, team_id: torch.Tensor, alive: torch.Tensor, score_vectors: torch.Tensor,
              folded_projection: torch.Tensor, norm_weight: torch.Tensor, eps: float | None, n_heads: int, *,
              broadcast: bool = True, intermediates: bool = False):
    """Per-team attention pooling of the ship rows (TeamPMA.forward, policy.py:94-120): a kernel
    that reads the ships once and leaves the weighted mean row per (team, head), one float32
    library GEMM with the folded value/output projection, a kernel for RMSNorm and the hand-out.

    Args:
        x:        (B, N, 128) float32 ship rows; a ``tokens[:, :N]`` view of a wider tensor works.
        team_id:  (B, N) integer team of every ship (0 / 1; anything else is nobody's key and
                  reads team ``clamp(id, 0, 1)``'s vector).
        alive:    (B, N) bool.
        score_vectors, folded_projection: from ``pack_team_pool_weights``.
        norm_weight: (128,) float32 RMSNorm weight; ``eps`` None means float32 machine epsilon.
        broadcast: also return the (B, N, 128) tensor in which every ship holds its team's vector.

    Returns:
        (ships or None, pool): ``pool`` is (B, 2, 128), zero for a team without an alive ship.  With
        ``intermediates`` also the attention-weighted mean rows ``z`` (B*2, H*128) and the projected
        rows before the norm (B*2, 128), which the backward needs.
    """
    if x.dim() != 3 or x.shape[-1] != FFN_WIDTH or x.dtype != torch.float32:
        raise ValueError("x must be float32 (B, N, 128)")
    B, N, D = x.shape
    if team_id.shape != (B, N) or alive.shape != (B, N):
        raise ValueError(f"team_id and alive must be {(B, N)}")
    if alive.dtype not in (torch.bool, torch.uint8):
        raise TypeError("alive must be bool")
    if score_vectors.shape != (2 * n_heads, D) or folded_projection.shape != (n_heads * D, D):
        raise ValueError("score_vectors / folded_projection must come from pack_team_pool_weights")
    for name, t in (("x", x), ("team_id", team_id), ("alive", alive), ("score_vectors", score_vectors),
                    ("folded_projection", folded_projection), ("norm_weight", norm_weight)):
        _need_device(t, name)
    for name, t in (("score_vectors", score_vectors), ("folded_projection", folded_projection), ("norm_weight", norm_weight)):
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32")
    if torch.is_grad_enabled() and x.requires_grad:
        raise RuntimeError("team_pool is forward-only; call it under torch.no_grad()")
    if N and (x.stride(2) != 1 or x.stride(1) % 4 or (B > 1 and x.stride(0) % 4)):
        x = x.contiguous()
    if team_id.dtype != torch.int32 or (N and team_id.stride(1) != 1):
        team_id = team_id.to(torch.int32).contiguous()
    if N and alive.stride(1) != 1:
        alive = alive.contiguous()
    dev = x.device
    pool = torch.empty((B, 2, D), dtype=torch.float32, device=dev)
    ships = torch.empty((B, N, D), dtype=torch.float32, device=dev) if broadcast else None
    if eps is None:
        eps = torch.finfo(torch.float32).eps
    z = pre = None
    if B:
        def env_stride(t):
            return t.stride(0) if B > 1 else t.shape[1] * (t.stride(1) if N else 1)

        z = torch.empty((B * 2, n_heads * D), dtype=torch.float32, device=dev)
        lib = _native.load()
        with _on_device(dev):
            rc = lib.bnb_team_attend_fwd(
                x.data_ptr(), env_stride(x), x.stride(1) if N else D, team_id.data_ptr(), env_stride(team_id) if N else 0,
                alive.data_ptr(), env_stride(alive) if N else 0, score_vectors.contiguous().data_ptr(), z.data_ptr(),
                B, N, int(n_heads), D, _stream(),
            )
            _native.check(rc, "bnb_team_attend_fwd")
            with torch.autocast("cuda", enabled=False):
                pre = torch.mm(z, folded_projection)
            rc = lib.bnb_team_norm_broadcast_fwd(
                pre.data_ptr(), norm_weight.detach().contiguous().data_ptr(), float(eps), team_id.data_ptr(),
                env_stride(team_id) if N else 0, pool.data_ptr(), None if ships is None else ships.data_ptr(), N * D, D,
                B, N, D, _stream(),
            )
            _native.check(rc, "bnb_team_norm_broadcast_fwd")
    if intermediates:
        if z is None:
            z = torch.zeros((0, n_heads * D), dtype=torch.float32, device=dev)
            pre = torch.zeros((0, D), dtype=torch.float32, device=dev)
        return ships, pool, z, pre
    return ships, pool


def team_pool_constants(seeds: torch.Tensor, in_proj_weight: torch.Tensor, out_proj_weight: torch.Tensor,
                        n_heads: int) -> tuple[torch.Tensor, torch.Tensor]:
    """``pack_team_pool_weights`` as differentiable float32 torch ops on the (small) parameters, for the
    update path: gradients of the two constants flow back to ``seeds`` and the attention weights."""
    D = seeds.shape[-1]
    dh = D // n_heads
    with torch.autocast(seeds.device.type, enabled=False):
        w = in_proj_weight.float()
        wq, wk, wv = w[:D], w[D:2 * D], w[2 * D:]
        q = (seeds.float() @ wq.t()).view(2, n_heads, dh)
        u = torch.einsum("thd,hdc->thc", q, wk.view(n_heads, dh, D)) * (math.log2(math.e) / math.sqrt(dh))
        wo = out_proj_weight.float().view(D, n_heads, dh)
        m = torch.einsum("ohd,hdc->hco", wo, wv.view(n_heads, dh, D))
        return u.reshape(2 * n_heads, D), m.reshape(n_heads * D, D)


class _TeamPoolTrain(torch.autograd.Function):
    """``team_pool`` (broadcast form) with a backward: the forward runs on the pooling kernels, the
    backward on the norm-backward kernel, two small float32 GEMMs with the folded projection and the
    attention-backward kernel (which recomputes the weights from the score vectors)."""

    @staticmethod
    def forward(ctx, x, team_id, alive, u, folded, norm_weight, eps, n_heads):
        with torch.no_grad():
            ships, _, z, pre = team_pool(x, team_id, alive, u, folded, norm_weight, eps, n_heads, intermediates=True)
        ctx.save_for_backward(x, team_id, alive, u, folded, norm_weight, z, pre)
        ctx.eps = eps
        ctx.n_heads = n_heads
        return ships

    @staticmethod
    @_outside_autocast
    def backward(ctx, dships):
        x, team_id, alive, u, folded, norm_weight, z, pre = ctx.saved_tensors
        B, N, D = x.shape
        H = ctx.n_heads
        dev = x.device
        u = u.float().contiguous()
        folded = folded.float()
        lib = _native.load()
        dships = dships.float().contiguous()
        if N and (x.stride(2) != 1 or x.stride(1) % 4 or (B > 1 and x.stride(0) % 4)):
            x = x.contiguous()
        if team_id.dtype != torch.int32 or (N and team_id.stride(1) != 1):
            team_id = team_id.to(torch.int32).contiguous()
        if N and alive.stride(1) != 1:
            alive = alive.contiguous()

        def env_stride(t):
            return t.stride(0) if B > 1 else t.shape[1] * (t.stride(1) if N else 1)

        dpool = torch.empty((B, 2, D), dtype=torch.float32, device=dev)
        with _on_device(dev):
            rc = lib.bnb_team_gather_bwd(dships.data_ptr(), team_id.data_ptr(), env_stride(team_id) if N else 0, alive.data_ptr(),
                                         env_stride(alive) if N else 0, dpool.data_ptr(), B, N, D, _stream())
        _native.check(rc, "bnb_team_gather_bwd")
        dpre, dnorm = rmsnorm_bwd(pre.view(B, 2, D), dpool, norm_weight, eps=ctx.eps)
        dpre = dpre.reshape(B * 2, D)
        dz = (dpre @ folded.t()).float().contiguous()  # (B*2, H*D) float32: the kernel reads it through a float pointer
        # z^T dpre contracts over 2B rows: batches of 1024 rows through the batched GEMM, then one sum
        rows = B * 2
        if rows >= 4096 and rows % 1024 == 0:
            dfolded = torch.bmm(z.view(rows // 1024, 1024, H * D).transpose(1, 2), dpre.view(rows // 1024, 1024, D)).sum(dim=0)
        else:
            dfolded = z.t() @ dpre

        for name, t, shape in (("z", z, (B * 2, H * D)), ("dz", dz, (B * 2, H * D)), ("score_vectors", u, (2 * H, D))):
            if t.dtype != torch.float32 or tuple(t.shape) != shape or not t.is_contiguous():
                raise TypeError(f"{name} must be a contiguous float32 {shape} tensor, got {t.dtype} {tuple(t.shape)}")
        dx = torch.empty((B, N, D), dtype=torch.float32, device=dev)
        ds = torch.empty((B * N, 2 * H), dtype=torch.float32, device=dev)
        du = torch.empty((2 * H, D), dtype=torch.float32, device=dev)
        partials = torch.empty((int(lib.bnb_team_attend_bwd_partial_rows()), 2 * H, D), dtype=torch.float32, device=dev)
        with _on_device(dev):
            rc = lib.bnb_team_attend_bwd(
                x.data_ptr(), env_stride(x) if N else 0, x.stride(1) if N else D, team_id.data_ptr(), env_stride(team_id) if N else 0,
                alive.data_ptr(), env_stride(alive) if N else 0, u.data_ptr(), z.data_ptr(), dz.data_ptr(),
                dx.data_ptr(), ds.data_ptr(), partials.data_ptr(), du.data_ptr(), B, N, H, D, _stream(),
            )
        _native.check(rc, "bnb_team_attend_bwd")
        return dx, None, None, du, dfolded, dnorm, None, None


def team_pool_train(x, team_id, alive, score_vectors, folded_projection, norm_weight, eps, n_heads) -> torch.Tensor:
    """Differentiable ``team_pool`` (the (B, N, 128) broadcast form); ``score_vectors`` and
    ``folded_projection`` from ``team_pool_constants`` so that their gradients reach the parameters."""
    with torch.autocast("cuda", enabled=False):
        return _TeamPoolTrain.apply(x, team_id, alive, score_vectors, folded_projection, norm_weight, eps, n_heads)


def pack_gate_weights(weight_a: torch.Tensor, weight_x: torch.Tensor) -> torch.Tensor:
    """``linear_a.weight`` and ``linear_x.weight`` (128, 128 each) as the bfloat16 operand stream
    of ``temporal_step``: ``[hf][q][ks][l][e]`` with the index meaning given in
    ``include/bnb_amd.h`` (every matrix-core operand one contiguous 1 KB run; a lane's 16 outputs
    per block of 32 channels are 16 consecutive channels)."""
    D = FFN_WIDTH
    if weight_a.shape != (D, D) or weight_x.shape != (D, D):
        raise ValueError("temporal_step covers (128, 128) gate weights")
    dev = weight_a.device
    w = torch.cat([weight_a.detach(), weight_x.detach()], dim=0).to(torch.bfloat16)
    hf = torch.arange(2, device=dev)[:, None, None, None, None]
    q = torch.arange(4, device=dev)[None, :, None, None, None]
    ks = torch.arange(8, device=dev)[None, None, :, None, None]
    lane = torch.arange(64, device=dev)[None, None, None, :, None]
    e = torch.arange(8, device=dev)[None, None, None, None, :]
    r = lane % 32
    rows = (q // 2) * D + 64 * hf + 32 * (q % 2) + 16 * ((r // 4) % 2) + 4 * (r // 8) + r % 4
    cols = 16 * ks + 8 * (lane // 32) + e
    rows, cols = torch.broadcast_tensors(rows, cols)
    return w[rows, cols].contiguous()


def temporal_step_supported(b1: torch.Tensor) -> bool:
    """Whether ``temporal_step`` covers these linear1 outputs: bfloat16, 128 channels."""
    return b1.is_cuda and b1.dtype == torch.bfloat16 and b1.shape[-1] == FFN_WIDTH


def temporal_step(
    b1: torch.Tensor,
    conv_buf: torch.Tensor,
    h: torch.Tensor,
    conv_weight: torch.Tensor,
    conv_bias: torch.Tensor | None,
    gate_weight_packed: torch.Tensor,
    gate_bias: torch.Tensor,
    log_lambda: torch.Tensor,
    c: float,
    *,
    conv_out: torch.Tensor | None = None,
    h_out: torch.Tensor | None = None,
    y_out: torch.Tensor | None = None,
    reset: torch.Tensor | None = None,
    rows_per_env: int = 1,
):
    """``conv_step`` -> gate projections -> ``rglru_step`` of one timestep as a single kernel
    (bfloat16 autocast flow; the conv output and the gate pre-activations never reach memory).

    Args:
        b1:        (R, 128) bfloat16 ``linear1`` outputs, or a (B, rows_per_env, 128) view into a
                   wider tensor (ship rows of a (B, N+M, ...) projection, possibly a column block).
        conv_buf, conv_out: (R, 3, 128) float32 stored inputs and their destination, as in ``conv_step``.
        h, h_out:  (R, 128) float32 state and its destination, as in ``rglru_step``.
        conv_weight (128, 4) or (128, 1, 4), conv_bias (128,) or None: float32.
        gate_weight_packed: ``pack_gate_weights(linear_a.weight, linear_x.weight)``.
        gate_bias: (256,) float32 ``[linear_a.bias | linear_x.bias]``.
        y_out:     optional bfloat16 destination of the layer output: contiguous (R, 128) or a
                   (B, rows_per_env, 128) view into a wider token tensor (possibly a column block).
        reset, rows_per_env: as in ``rglru_step``.

    Returns:
        (y, h_new, new_conv_buf).
    """
    D = FFN_WIDTH
    if b1.dim() not in (2, 3) or b1.shape[-1] != D or b1.dtype != torch.bfloat16:
        raise ValueError("b1 must be bfloat16 (R, 128) or a (B, rows_per_env, 128) view")
    R = b1.numel() // D
    if conv_buf.shape != (R, 3, D) or h.shape != (R, D):
        raise ValueError(f"conv_buf must be {(R, 3, D)} and h {(R, D)}, got {tuple(conv_buf.shape)}, {tuple(h.shape)}")
    if gate_weight_packed.shape != (2, 4, 8, 64, 8) or gate_weight_packed.dtype != torch.bfloat16:
        raise ValueError("gate_weight_packed must come from pack_gate_weights")
    if gate_bias.shape != (2 * D,) or log_lambda.shape != (D,):
        raise ValueError("gate_bias must be (256,) and log_lambda (128,)")
    for name, t in (("b1", b1), ("conv_buf", conv_buf), ("h", h), ("conv_weight", conv_weight),
                    ("gate_weight_packed", gate_weight_packed), ("gate_bias", gate_bias), ("log_lambda", log_lambda)):
        _need_device(t, name)
    for name, t in (("conv_buf", conv_buf), ("h", h), ("conv_weight", conv_weight), ("gate_bias", gate_bias),
                    ("log_lambda", log_lambda)):
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32")
    if conv_bias is not None and conv_bias.dtype != torch.float32:
        raise TypeError("conv_bias must be float32")
    if torch.is_grad_enabled() and (b1.requires_grad or conv_buf.requires_grad or h.requires_grad):
        raise RuntimeError("temporal_step is forward-only; call it under torch.no_grad()")
    dev = b1.device
    conv_weight = conv_weight.detach().reshape(D, 4).contiguous()
    conv_bias = None if conv_bias is None else conv_bias.detach().contiguous()
    gate_weight_packed = gate_weight_packed.contiguous()
    gate_bias = gate_bias.detach().contiguous()
    log_lambda = log_lambda.detach().contiguous()
    b1_group, b1_row = 0, D
    if b1.dim() == 3 and not b1.is_contiguous():
        b1_group, b1_row = _grouped_rows(b1, R, D, rows_per_env, "b1", pitch_ok=True)
    else:
        b1 = b1.contiguous()

    def conv_rows_ok(t):
        return R == 0 or (t.stride(2) == 1 and t.stride(1) == D)

    if not conv_rows_ok(conv_buf):
        conv_buf = conv_buf.contiguous()
    if R and h.stride(-1) != 1:
        h = h.contiguous()
    if conv_out is None:
        conv_out = torch.empty((R, 3, D), dtype=torch.float32, device=dev)
    elif conv_out.shape != (R, 3, D) or conv_out.dtype != torch.float32 or conv_out.device != dev or not conv_rows_ok(conv_out):
        raise ValueError("conv_out must be a float32 (R, 3, 128) tensor on b1's device with contiguous rows")
    if h_out is None:
        h_out = torch.empty((R, D), dtype=torch.float32, device=dev)
    elif h_out.shape != (R, D) or h_out.dtype != torch.float32 or h_out.device != dev or (R and h_out.stride(-1) != 1):
        raise ValueError("h_out must be a float32 (R, 128) tensor on b1's device, contiguous in its last dim")
    y_group, y_row = 0, D
    if y_out is None:
        y_out = torch.empty((R, D), dtype=torch.bfloat16, device=dev)
    else:
        if y_out.dtype != torch.bfloat16 or y_out.device != dev:
            raise ValueError("y_out must be a bfloat16 tensor on b1's device")
        if y_out.dim() == 3 and not y_out.is_contiguous():
            y_group, y_row = _grouped_rows(y_out, R, D, rows_per_env, "y_out", pitch_ok=True)
        elif y_out.shape not in ((R, D), (R // max(rows_per_env, 1), rows_per_env, D)) or not y_out.is_contiguous():
            raise ValueError("y_out must be a contiguous (R, 128) tensor or a (B, n, 128) view")
    reset_ptr = _reset_pointer(reset, R, rows_per_env, dev)
    if (b1_group or y_group) and (rows_per_env < 1 or R % rows_per_env):
        raise ValueError(f"rows_per_env={rows_per_env} does not divide the {R} rows")
    if R:
        with _on_device(dev):
            rc = _native.load().bnb_temporal_step_fwd(
                b1.data_ptr(), int(b1_group), int(b1_row), conv_buf.data_ptr(), conv_buf.stride(0),
                conv_out.data_ptr(), conv_out.stride(0), h.data_ptr(), h.stride(0), h_out.data_ptr(), h_out.stride(0),
                conv_weight.data_ptr(), None if conv_bias is None else conv_bias.data_ptr(),
                gate_weight_packed.data_ptr(), gate_bias.data_ptr(), log_lambda.data_ptr(), float(c),
                y_out.data_ptr(), int(y_group), int(y_row), reset_ptr, int(rows_per_env), R, D, _stream(),
            )
        _native.check(rc, "bnb_temporal_step_fwd")
    return y_out, h_out, conv_out


def _done_pointer(done, R, T, device):
    """Contiguous byte view of an optional (R, T) episode-end mask; returns (keepalive, pointer)."""
    if done is None:
        return None, None
    if done.shape != (R, T) or done.dtype not in (torch.bool, torch.uint8):
        raise ValueError(f"done must be a bool {(R, T)} tensor")
    if done.device != device:
        raise ValueError("done must live on the same device as the inputs")
    done = done.contiguous()
    return done, done.data_ptr()


def _token_rows(t: torch.Tensor, token_rows: int | None, time_major: bool, name: str):
    """``(rows_per_env, env_row_pitch, dense shape)`` of a kernel operand that may be a (T, B, NM, D) token tensor of
    which a call covers the first ``token_rows`` tokens per environment; (0, 0, t.shape) for a plain operand."""
    if token_rows is None:
        return 0, 0, tuple(t.shape)
    if not time_major or t.dim() != 4 or not 1 <= token_rows <= t.shape[2]:
        raise ValueError(f"token_rows needs time_major and a (T, B, NM, D) {name} with NM >= token_rows, got {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous when token_rows is given")
    T, B, NM, D = t.shape
    return int(token_rows), int(NM), (T, B * token_rows, D)


def conv_seq(
    b1: torch.Tensor,
    conv_buf: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    done: torch.Tensor | None = None,
    *,
    conv_out: torch.Tensor | None = None,
    also_bf16: bool = False,
    time_major: bool = False,
    token_rows: int | None = None,
):
    """Causal depthwise conv over a sequence, taps cut at episode ends (griffin.py:67-140).

    Args:
        b1:       (R, T, D) ``linear1`` outputs, float32 or bfloat16.
        conv_buf: (R, 3, D) float32 inputs stored before the sequence (rows may be strided).
        weight, bias: as in ``conv_step``.
        done:     optional (R, T) bool; True at t ends an episode at t.
        conv_out: optional (R, 3, D) float32 destination for the new stored inputs.
        also_bf16: also return a bfloat16 copy of the conv output.
        time_major: ``b1`` and the returned conv output are (T, R, D) instead of (R, T, D);
                  ``done`` stays (R, T).
        token_rows: with ``time_major``, ``b1`` is a (T, B, NM, D) token tensor and the conv runs over its first
                  ``token_rows`` tokens of every environment, read where they lie (R = B * token_rows, env-major);
                  the outputs are dense, (T, R, D).

    Returns:
        (v, new_conv_buf[, v_bf16]): conv output (R, T, D) float32 and the last three entries
        of ``[conv_buf, b1]``.
    """
    group, pitch, v_shape = _token_rows(b1, token_rows, time_major, "b1")
    if (b1.dim() != 3 and not group) or conv_buf.dim() != 3:
        raise ValueError("b1 must be (R, T, D) and conv_buf (R, 3, D)")
    R, T, D = v_shape
    if time_major:
        T, R = R, T
    if T < 1:
        raise ValueError("conv_seq needs at least one timestep")
    if conv_buf.shape != (R, 3, D):
        raise ValueError(f"conv_buf must be {(R, 3, D)}, got {tuple(conv_buf.shape)}")
    for name, t in (("b1", b1), ("conv_buf", conv_buf), ("weight", weight)):
        _need_device(t, name)
    if conv_buf.dtype != torch.float32 or weight.dtype != torch.float32 or (bias is not None and bias.dtype != torch.float32):
        raise TypeError("conv_buf, weight and bias must be float32")
    if torch.is_grad_enabled() and (b1.requires_grad or conv_buf.requires_grad):
        raise RuntimeError("conv_seq is forward-only; call it under torch.no_grad()")
    b_code = _code(b1, "b1")
    weight = weight.detach().reshape(D, 4).contiguous()
    bias_ptr = None
    if bias is not None:
        bias = bias.detach().contiguous()
        bias_ptr = bias.data_ptr()
    b1 = b1.contiguous()

    def rows_ok(t):
        return R == 0 or (t.stride(2) == 1 and t.stride(1) == D)

    if not rows_ok(conv_buf):
        conv_buf = conv_buf.contiguous()
    if conv_out is None:
        conv_out = torch.empty((R, 3, D), dtype=torch.float32, device=b1.device)
    elif conv_out.shape != (R, 3, D) or conv_out.dtype != torch.float32 or conv_out.device != b1.device or not rows_ok(conv_out):
        raise ValueError("conv_out must be a float32 (R, 3, D) tensor on b1's device with contiguous rows")
    v = torch.empty(v_shape, dtype=torch.float32, device=b1.device)
    v_lp = torch.empty(v_shape, dtype=torch.bfloat16, device=b1.device) if also_bf16 else None
    keep, done_ptr = _done_pointer(done, R, T, b1.device)
    if R:
        with _on_device(b1.device):
            rc = _native.load().bnb_conv_seq_fwd(
                b1.data_ptr(), b_code, conv_buf.data_ptr(), conv_buf.stride(0), weight.data_ptr(), bias_ptr, done_ptr,
                v.data_ptr(), None if v_lp is None else v_lp.data_ptr(), conv_out.data_ptr(), conv_out.stride(0),
                R, T, D, int(time_major), group, pitch, _stream(),
            )
        _native.check(rc, "bnb_conv_seq_fwd")
    del keep
    return (v, conv_out, v_lp) if also_bf16 else (v, conv_out)


_CONV_TRAIN_WIDTHS = (64, 128, 256, 512)


def conv_seq_bwd(b1, conv_buf, weight, done, dv, dconv_out=None, *, time_major: bool = False, dv_bf16=None,
                 token_rows: int | None = None, db1_out: torch.Tensor | None = None):
    """Backward of ``conv_seq``: returns ``(db1, dconv_buf, dweight (D, 4), dbias (D,))``.

    ``dv`` is the float32 gradient of the conv output (b1's layout), ``dconv_out`` the optional
    gradient of the returned stored inputs, ``dv_bf16`` the optional gradient of the output's bfloat16
    copy (added to ``dv`` in the kernel); ``db1`` has b1's dtype.  Sums run in a fixed order.

    ``token_rows`` as in ``conv_seq``: b1 is a (T, B, NM, D) token tensor, ``dv`` dense (T, B * token_rows, D), and
    ``db1`` is a token tensor like b1 (``db1_out`` if given) in which ONLY the first ``token_rows`` tokens of every
    environment are written."""
    group, pitch, v_shape = _token_rows(b1, token_rows, time_major, "b1")
    R, T, D = v_shape
    if time_major:
        T, R = R, T
    if D not in _CONV_TRAIN_WIDTHS:
        raise ValueError(f"conv_seq_bwd supports D in {_CONV_TRAIN_WIDTHS}, got {D}")
    if tuple(dv.shape) != v_shape or dv.dtype != torch.float32:
        raise ValueError("dv must be float32 with the conv output's shape")
    for name, t in (("b1", b1), ("conv_buf", conv_buf), ("weight", weight), ("dv", dv)):
        _need_device(t, name)
    b1 = b1.contiguous()
    dv = dv.contiguous()
    if dv_bf16 is not None:
        if tuple(dv_bf16.shape) != v_shape or dv_bf16.dtype != torch.bfloat16:
            raise ValueError("dv_bf16 must be bfloat16 with the conv output's shape")
        _need_device(dv_bf16, "dv_bf16")
        dv_bf16 = dv_bf16.contiguous()
    conv_buf = conv_buf if (R == 0 or (conv_buf.stride(2) == 1 and conv_buf.stride(1) == D)) else conv_buf.contiguous()
    weight = weight.detach().reshape(D, 4).contiguous()
    if dconv_out is not None:
        if dconv_out.shape != (R, 3, D):
            raise ValueError(f"dconv_out must be {(R, 3, D)}")
        dconv_out = dconv_out.to(torch.float32).contiguous()
    if db1_out is None:
        db1 = torch.empty_like(b1)
    elif db1_out.shape != b1.shape or db1_out.dtype != b1.dtype or db1_out.device != b1.device or not db1_out.is_contiguous():
        raise ValueError("db1_out must be a contiguous tensor like b1")
    else:
        db1 = db1_out
    dconv = torch.empty((R, 3, D), dtype=torch.float32, device=b1.device)
    dwb = torch.empty((5 * D,), dtype=torch.float32, device=b1.device)
    lib = _native.load()
    blocks = int(lib.bnb_conv_seq_bwd_blocks(R, T, D))
    partials = torch.empty((blocks, 5 * D), dtype=torch.float32, device=b1.device)
    keep, done_ptr = _done_pointer(done, R, T, b1.device)
    with _on_device(b1.device):
        rc = lib.bnb_conv_seq_bwd(b1.data_ptr(), _code(b1, "b1"), conv_buf.data_ptr(), conv_buf.stride(0) if R else 3 * D,
                                  weight.data_ptr(), done_ptr, dv.data_ptr(), None if dv_bf16 is None else dv_bf16.data_ptr(),
                                  None if dconv_out is None else dconv_out.data_ptr(), db1.data_ptr(), dconv.data_ptr(),
                                  partials.data_ptr(), blocks, dwb.data_ptr(), R, T, D, int(time_major), group, pitch, _stream())
    _native.check(rc, "bnb_conv_seq_bwd")
    del keep
    return db1, dconv, dwb[:4 * D].view(D, 4), dwb[4 * D:]


class _ConvSeqTrain(torch.autograd.Function):
    """``conv_seq`` with its backward kernel."""

    @staticmethod
    def forward(ctx, b1, conv_buf, weight, bias, done, time_major, also_bf16):
        with torch.no_grad():
            res = conv_seq(b1, conv_buf, weight, bias, done, time_major=time_major, also_bf16=also_bf16)
        ctx.save_for_backward(b1, conv_buf, weight)
        ctx.set_materialize_grads(False)
        ctx.done = done
        ctx.time_major = time_major
        ctx.has_bias = bias is not None
        return res[0], res[1], (res[2] if also_bf16 else None)

    @staticmethod
    @_outside_autocast
    def backward(ctx, dv, dbuf, dv_lp):
        b1, conv_buf, weight = ctx.saved_tensors
        if dv is None:
            dv = torch.zeros(b1.shape, dtype=torch.float32, device=b1.device)
        db1, dconv, dw, db = conv_seq_bwd(b1, conv_buf, weight, ctx.done, dv, dbuf, time_major=ctx.time_major, dv_bf16=dv_lp)
        return db1, dconv, dw.reshape(weight.shape), db if ctx.has_bias else None, None, None, None


def conv_seq_train_supported(b1: torch.Tensor) -> bool:
    """Whether ``conv_seq_train`` covers this input: a covered width on the GPU."""
    return b1.is_cuda and b1.dim() == 3 and b1.shape[-1] in _CONV_TRAIN_WIDTHS and b1.dtype in (torch.float32, torch.bfloat16)


def conv_seq_train(b1, conv_buf, weight, bias, done=None, *, time_major: bool = False, also_bf16: bool = False):
    """Differentiable ``conv_seq``: ``(v, new_conv_buf)`` with gradients for b1, conv_buf, weight and bias.

    ``also_bf16``: a third result, the bfloat16 rounding of ``v`` written by the same launch (what a bfloat16
    projection of ``v`` would cast for itself); its gradient is added to ``v``'s inside the backward kernel."""
    with torch.autocast("cuda", enabled=False):
        v, new_buf, v_lp = _ConvSeqTrain.apply(b1, conv_buf, weight, bias, done, time_major, also_bf16)
    return (v, new_buf, v_lp) if also_bf16 else (v, new_buf)


def rglru_scan(
    x: torch.Tensor,
    gates_pre: torch.Tensor,
    log_lambda: torch.Tensor,
    c: float,
    h0: torch.Tensor,
    done: torch.Tensor | None = None,
    *,
    y_dtype: torch.dtype = torch.float32,
    h_out: torch.Tensor | None = None,
    time_major: bool = False,
    y_tokens: tuple[torch.Tensor, int] | None = None,
):
    """RG-LRU over a whole sequence in one pass (griffin.py:188-219 without the log-depth scan).

    Args:
        x:          (R, T, D) float32 or bfloat16.
        gates_pre:  (R, T, 2*D) ``[linear_a(x) | linear_x(x)]``.
        log_lambda: (D,) float32.
        h0:         (R, D) float32 state before the sequence (rows may be strided).
        done:       optional (R, T) bool; True at t makes step t+1 start from a zero state.
        y_dtype:    dtype of the returned states.
        h_out:      optional (R, D) float32 destination of the final state.
        time_major: ``x``, ``gates_pre`` and the returned states are (T, R, .) instead of
                    (R, T, .); ``done`` stays (R, T).
        y_tokens:   ``(tokens, n)``: with ``time_major`` and no gradient, the states go into the first ``n`` tokens of
                    every environment of the (T, B, NM, D) tensor ``tokens`` (R = B * n, env-major), which is returned
                    in place of ``y``; its other tokens are left alone.

    Returns:
        (y, h_last): all states (R, T, D) in ``y_dtype`` and the final state (R, D) float32.
    """
    if x.dim() != 3:
        raise ValueError("x must be (R, T, D)")
    R, T, D = x.shape
    if gates_pre.shape != (R, T, 2 * D):
        raise ValueError(f"gates_pre must be {(R, T, 2 * D)}, got {tuple(gates_pre.shape)}")
    if time_major:
        T, R = R, T
    if h0.shape != (R, D) or h0.dtype != torch.float32:
        raise ValueError(f"h0 must be a float32 {(R, D)} tensor")
    if log_lambda.shape != (D,) or log_lambda.dtype != torch.float32:
        raise ValueError(f"log_lambda must be a float32 {(D,)} tensor")
    for name, t in (("x", x), ("gates_pre", gates_pre), ("h0", h0), ("log_lambda", log_lambda)):
        _need_device(t, name)
    if y_dtype not in _DTYPE_CODE:
        raise TypeError(f"y_dtype must be float32 or bfloat16, got {y_dtype}")
    if torch.is_grad_enabled() and (x.requires_grad or gates_pre.requires_grad or h0.requires_grad or log_lambda.requires_grad):
        # training: forward and backward kernels behind autograd
        if y_dtype != torch.float32 or h_out is not None or y_tokens is not None:
            raise RuntimeError("rglru_scan under autograd returns float32 states and owns its outputs")
        keep, _ = _done_pointer(done, R, T, x.device)
        return _RglruScan.apply(x, gates_pre, log_lambda, h0, keep, float(c), bool(time_major))
    x_code, g_code = _code(x, "x"), _code(gates_pre, "gates_pre")
    x = x.contiguous()
    gates_pre = gates_pre.contiguous()
    log_lambda = log_lambda.detach().contiguous()
    if R and h0.stride(1) != 1:
        h0 = h0.contiguous()
    if h_out is None:
        h_out = torch.empty((R, D), dtype=torch.float32, device=x.device)
    elif h_out.shape != (R, D) or h_out.dtype != torch.float32 or h_out.device != x.device or (R and h_out.stride(1) != 1):
        raise ValueError("h_out must be a float32 (R, D) tensor on x's device with contiguous rows")
    group = pitch = 0
    if y_tokens is None:
        y = torch.empty(x.shape, dtype=y_dtype, device=x.device)
    else:
        y, n = y_tokens
        group, pitch, dense = _token_rows(y, n, time_major, "y_tokens[0]")
        if dense != tuple(x.shape) or y.dtype != y_dtype or y.device != x.device:
            raise ValueError(f"y_tokens must hold {tuple(x.shape)} {y_dtype} states on x's device")
    keep, done_ptr = _done_pointer(done, R, T, x.device)
    if R:
        with _on_device(x.device):
            rc = _native.load().bnb_rglru_scan_fwd(
                x.data_ptr(), x_code, gates_pre.data_ptr(), g_code, log_lambda.data_ptr(), float(c), h0.data_ptr(),
                h0.stride(0), done_ptr, y.data_ptr(), _DTYPE_CODE[y_dtype], h_out.data_ptr(), h_out.stride(0),
                R, T, D, int(time_major), group, pitch, _stream(),
            )
        _native.check(rc, "bnb_rglru_scan_fwd")
    del keep
    return y, h_out


class _RglruScan(torch.autograd.Function):
    """``rglru_scan`` with a backward: one reverse-time kernel pass instead of autograd through
    the per-step coefficient chain and a log-depth scan."""

    @staticmethod
    def forward(ctx, x, gates_pre, log_lambda, h0, done, c, time_major):
        with torch.no_grad():
            y, h_last = rglru_scan(x, gates_pre, log_lambda, c, h0, done, time_major=time_major)
        ctx.save_for_backward(x, gates_pre, log_lambda, h0, y)
        ctx.set_materialize_grads(False)
        ctx.done, ctx.c, ctx.time_major = done, c, time_major
        return y, h_last

    @staticmethod
    @_outside_autocast
    def backward(ctx, dy, dh_last):
        x, gates_pre, log_lambda, h0, y = ctx.saved_tensors
        dx, dgates, dh0, dlam_rows = rglru_scan_bwd(x, gates_pre, log_lambda, ctx.c, h0, ctx.done, y, dy, dh_last,
                                                    time_major=ctx.time_major)
        return dx, dgates, dlam_rows.sum(dim=0), dh0, None, None, None


def rglru_scan_bwd(x, gates_pre, log_lambda, c, h0, done, y, dy, dh_last=None, *, time_major: bool = False,
                   token_rows: int | None = None):
    """Backward of ``rglru_scan``: ``(dx, dgates, dh0, dlog_lambda per row (R, D))`` from the saved inputs, the saved
    states ``y`` and the gradients of the states (``dy``, in y's dtype; None = zero) and of the final state.

    ``done`` is the (R, T) uint8/bool tensor the forward saw, or None.  ``token_rows``: with ``time_major``, ``y`` and
    ``dy`` are (T, B, NM, D) token tensors whose first ``token_rows`` tokens per environment are this call's rows."""
    group, pitch, dense = _token_rows(y, token_rows, time_major, "y")
    if dense != tuple(x.shape) or (dy is not None and dy.shape != y.shape):
        raise ValueError("y (and dy) must hold x's rows")
    T, R = (x.shape[0], x.shape[1]) if time_major else (x.shape[1], x.shape[0])
    D = x.shape[2]
    x_c, g_c = x.contiguous(), gates_pre.contiguous()
    h0_c = h0 if h0.stride(1) == 1 else h0.contiguous()
    y = y.contiguous()
    # the kernel reads dy in y's dtype and dh_last as float32; a gradient nobody produced arrives as None
    if dy is not None:
        dy = dy.to(y.dtype).contiguous()
    elif group:
        raise ValueError("dy is required with token_rows")
    else:
        dy = torch.zeros_like(y)
    if dh_last is not None:
        dh_last = dh_last.float().contiguous()
    dx = torch.empty_like(x_c)
    dgates = torch.empty_like(g_c)
    dh0 = torch.empty((R, D), dtype=torch.float32, device=x.device)
    dlam_rows = torch.empty((R, D), dtype=torch.float32, device=x.device)
    keep, done_ptr = _done_pointer(done, R, T, x.device)
    if R:
        with _on_device(x.device):
            rc = _native.load().bnb_rglru_scan_bwd(
                x_c.data_ptr(), _DTYPE_CODE[x.dtype], g_c.data_ptr(), _DTYPE_CODE[gates_pre.dtype],
                log_lambda.detach().contiguous().data_ptr(), float(c), h0_c.data_ptr(), h0_c.stride(0), done_ptr, y.data_ptr(),
                _DTYPE_CODE[y.dtype], dy.data_ptr(), None if dh_last is None else dh_last.data_ptr(),
                0 if dh_last is None else dh_last.stride(0), dx.data_ptr(), dgates.data_ptr(), dh0.data_ptr(),
                dlam_rows.data_ptr(), R, T, D, int(time_major), group, pitch, _stream(),
            )
        _native.check(rc, "bnb_rglru_scan_bwd")
    else:
        dlam_rows.zero_()
    del keep
    return dx, dgates, dh0, dlam_rows


class _TemporalMixTrain(torch.autograd.Function):
    """The middle of the temporal sublayer over a stored rollout's (T, B, NM, D) bfloat16 token tensor ``b1`` (the
    ``linear1`` outputs), as the update runs it under bfloat16 autocast: causal conv, the two gate projections and the
    RG-LRU over the first ``n`` tokens of every environment (griffin.py:267-283), a bias-free Linear ``field_w`` over
    the others (griffin.py:406-413), both results in ONE float32 (T, B, NM, D) tensor.

    The reference slices the tokens, runs the two branches and concatenates; here the conv and scan kernels read and
    write the ship rows where they lie in the token tensors (forward and backward), so neither the split, nor the
    concatenation, nor their backward copies exist.  Values and gradients equal those of the separate steps
    (``conv_seq_train`` with its bfloat16 copy, ``linear_train``, ``rglru_scan``, ``linear_train``, ``torch.cat``)."""

    @staticmethod
    def forward(ctx, b1, n, conv_buf, conv_w, conv_b, gate_w, gate_b, log_lambda, c, h0, done, field_w):
        T, B, NM, D = b1.shape
        bf16 = torch.bfloat16
        with torch.no_grad():
            v, new_buf, v_lp = conv_seq(b1, conv_buf, conv_w, conv_b, done, also_bf16=True, time_major=True, token_rows=n)
            wb = gate_w.to(bf16)
            gates = torch.nn.functional.linear(v_lp.view(-1, D), wb, gate_b.to(bf16)).view(T, B * n, 2 * D)
            y = torch.empty((T, B, NM, D), dtype=torch.float32, device=b1.device)
            _, h_last = rglru_scan(v, gates, log_lambda, c, h0, done, time_major=True, y_tokens=(y, n))
            fields = b1[:, :, n:].contiguous()
            fw = field_w.to(bf16)
            y[:, :, n:].copy_(torch.nn.functional.linear(fields, fw))  # bfloat16 values are exact in float32
        ctx.save_for_backward(b1, conv_buf, conv_w, wb, log_lambda, h0, v, v_lp, gates, y, fields, fw)
        ctx.set_materialize_grads(False)
        ctx.n, ctx.c, ctx.done = n, c, done
        ctx.conv_w_shape = conv_w.shape
        ctx.has_conv_bias = conv_b is not None
        return y, h_last, new_buf

    @staticmethod
    @_outside_autocast
    def backward(ctx, dy, dh_last, dbuf):
        b1, conv_buf, conv_w, wb, log_lambda, h0, v, v_lp, gates, y, fields, fw = ctx.saved_tensors
        T, B, NM, D = b1.shape
        n = ctx.n
        bf16 = torch.bfloat16
        dy = torch.zeros_like(y) if dy is None else dy.float().contiguous()
        dx, dgates, dh0, dlam_rows = rglru_scan_bwd(v, gates, log_lambda, ctx.c, h0, ctx.done, y, dy, dh_last, time_major=True,
                                                    token_rows=n)
        dg = dgates.view(-1, 2 * D)
        dv_lp = torch.matmul(dg, wb).view(T, B * n, D)
        d_gate_w = linear_wgrad(dg, v_lp.view(-1, D)) if ctx.needs_input_grad[5] else None
        d_gate_b = None
        if ctx.needs_input_grad[6]:
            d_gate_b = column_sums(dg) if column_sums_supported(dg) else dg.sum(dim=0, dtype=torch.float32)
        db1 = torch.empty_like(b1)
        _, dconv, dw, db = conv_seq_bwd(b1, conv_buf, conv_w, ctx.done, dx, dbuf, time_major=True, dv_bf16=dv_lp, token_rows=n,
                                        db1_out=db1)
        # the other tokens: one strided read of their gradient (rounded to bfloat16, as a bfloat16 Linear receives it),
        # the input-gradient GEMM, one strided write into the token tensor the conv backward filled the ship rows of
        dyf = torch.empty((T, B, NM - n, D), dtype=bf16, device=b1.device)
        dyf.copy_(dy[:, :, n:])
        db1[:, :, n:].copy_(torch.matmul(dyf.view(-1, D), fw).view(T, B, NM - n, D))
        d_field_w = linear_wgrad(dyf.view(-1, D), fields.view(-1, D)) if ctx.needs_input_grad[11] else None
        return (db1, None, dconv, dw.reshape(ctx.conv_w_shape), db if ctx.has_conv_bias else None, d_gate_w, d_gate_b,
                dlam_rows.sum(dim=0), None, dh0, None, d_field_w)


def temporal_mix_train_supported(b1: torch.Tensor, n: int, gate_w: torch.Tensor, field_w: torch.Tensor) -> bool:
    """Whether ``temporal_mix_train`` covers this token tensor: bfloat16 (T, B, NM, 128) on the GPU with recurrent and
    other tokens in every environment, float32 weights of the widths the weight-gradient kernel covers."""
    return (b1.is_cuda and b1.dim() == 4 and b1.dtype == torch.bfloat16 and b1.shape[-1] in _CONV_TRAIN_WIDTHS
            and 0 < n < b1.shape[2] and gate_w.dtype == field_w.dtype == torch.float32
            and linear_wgrad_supported(b1, gate_w) and linear_wgrad_supported(b1, field_w))


def temporal_mix_train(b1, n, conv_buf, conv_weight, conv_bias, gate_weight, gate_bias, log_lambda, c, h0, done, field_weight):
    """Differentiable conv + gate projections + RG-LRU over the first ``n`` tokens of every environment of the
    (T, B, NM, D) bfloat16 tensor ``b1`` and ``F.linear(., field_weight)`` over the others:
    ``(y (T, B, NM, D) float32, h_last (B*n, D), new_conv_buf (B*n, 3, D))``.

    ``gate_weight`` (2D, D) and ``gate_bias`` (2D,) are ``[linear_a | linear_x]``; ``h0`` (B*n, D), ``conv_buf``
    (B*n, 3, D) float32 and ``done`` ((B*n, T) or None) are env-major like the recurrent state."""
    with torch.autocast("cuda", enabled=False):
        return _TemporalMixTrain.apply(b1.contiguous(), int(n), conv_buf, conv_weight, conv_bias, gate_weight, gate_bias, log_lambda,
                                       float(c), h0, done, field_weight)


_F32_EPS = float(torch.finfo(torch.float32).eps)
_NORM_WIDTHS = (8, 16, 32, 64, 128, 256, 512)


def add_rmsnorm(
    x: torch.Tensor,
    weight: torch.Tensor,
    *,
    delta: torch.Tensor | None = None,
    eps: float | None = None,
    out_dtype: torch.dtype = torch.float32,
) -> tuple[torch.Tensor, torch.Tensor]:
    """``s = x + delta`` (if given) and ``rmsnorm(s) * weight`` in one pass.

    x (..., D) float32 with contiguous rows; delta same shape, float32 or bfloat16; weight (D,)
    float32; eps defaults to ``finfo(float32).eps`` (``nn.RMSNorm(D)`` with eps=None).
    Returns (s, normed): s is x itself when there is no delta; normed has ``out_dtype``.
    """
    D = x.shape[-1]
    if x.dtype != torch.float32 or weight.dtype != torch.float32 or weight.shape != (D,):
        raise TypeError("x and weight must be float32 and weight must be (D,)")
    if D not in _NORM_WIDTHS:
        raise ValueError(f"add_rmsnorm supports D in {_NORM_WIDTHS}, got {D}")
    _need_device(x, "x")
    if torch.is_grad_enabled() and (x.requires_grad or (delta is not None and delta.requires_grad)):
        raise RuntimeError("add_rmsnorm is forward-only; call it under torch.no_grad()")
    x2 = x.reshape(-1, D)
    if x2.numel() and x2.stride(-1) != 1:
        x2 = x2.contiguous()
    R = x2.shape[0]
    d_ptr, d_code, s_out = None, _native.F32, None
    if delta is not None:
        if delta.shape != x.shape:
            raise ValueError(f"delta must be {tuple(x.shape)}, got {tuple(delta.shape)}")
        delta = delta.reshape(-1, D).contiguous()
        d_ptr, d_code = delta.data_ptr(), _code(delta, "delta")
        s_out = torch.empty((R, D), dtype=torch.float32, device=x.device)
    normed = torch.empty((R, D), dtype=out_dtype, device=x.device)
    o_code = _code(normed, "out_dtype")
    if R:
        with _on_device(x.device):
            rc = _native.load().bnb_add_rmsnorm_fwd(
                x2.data_ptr(), x2.stride(0), d_ptr, d_code, weight.detach().contiguous().data_ptr(),
                _F32_EPS if eps is None else float(eps), None if s_out is None else s_out.data_ptr(),
                normed.data_ptr(), o_code, R, D, _stream(),
            )
        _native.check(rc, "bnb_add_rmsnorm_fwd")
    return (x if s_out is None else s_out.reshape(x.shape)), normed.reshape(x.shape)


_NORM_TRAIN_WIDTHS = (64, 128, 256, 512)


def rmsnorm_bwd(x: torch.Tensor, dy: torch.Tensor, weight: torch.Tensor, *, eps: float | None = None,
                grad_sum: torch.Tensor | None = None, also_bf16: bool = False):
    """Backward of ``y = rmsnorm(x) * weight``: returns ``(dx, dw)``, both float32, and with
    ``also_bf16`` a bfloat16 copy of dx as a third value (written by the same pass).

    x (..., D) float32 with contiguous rows; dy same shape, float32 or bfloat16; ``grad_sum`` (same
    shape, float32) is added to dx: the gradient reaching x on the branch that bypasses the norm.
    The rows are added into dw in a fixed order, so repeated calls give identical bits."""
    D = x.shape[-1]
    if x.dtype != torch.float32 or weight.dtype != torch.float32 or weight.shape != (D,):
        raise TypeError("x and weight must be float32 and weight must be (D,)")
    if D not in _NORM_TRAIN_WIDTHS:
        raise ValueError(f"rmsnorm_bwd supports D in {_NORM_TRAIN_WIDTHS}, got {D}")
    if dy.shape != x.shape or (grad_sum is not None and grad_sum.shape != x.shape):
        raise ValueError("dy and grad_sum must have x's shape")
    if grad_sum is not None and grad_sum.dtype != torch.float32:
        raise TypeError("grad_sum must be float32")
    _need_device(x, "x")
    _need_device(dy, "dy")
    x2 = x.reshape(-1, D) if _uniform_rows(x, D) else x.reshape(-1, D).contiguous()
    dy2 = dy.reshape(-1, D) if _uniform_rows(dy, D) else dy.reshape(-1, D).contiguous()
    gs = None if grad_sum is None else grad_sum.reshape(-1, D).contiguous()
    R = x2.shape[0]
    dx = torch.empty((R, D), dtype=torch.float32, device=x.device)
    dw = torch.empty((D,), dtype=torch.float32, device=x.device)
    dx_lp = torch.empty((R, D), dtype=torch.bfloat16, device=x.device) if also_bf16 else None
    lib = _native.load()
    blocks = int(lib.bnb_rmsnorm_bwd_blocks(R, D))
    partials = torch.empty((blocks, D), dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        rc = lib.bnb_rmsnorm_bwd(x2.data_ptr(), x2.stride(0) if R else D, dy2.data_ptr(), _code(dy2, "dy"),
                                 dy2.stride(0) if R else D, weight.detach().contiguous().data_ptr(),
                                 _F32_EPS if eps is None else float(eps), None if gs is None else gs.data_ptr(),
                                 dx.data_ptr(), None if dx_lp is None else dx_lp.data_ptr(), partials.data_ptr(), blocks,
                                 dw.data_ptr(), R, D, _stream())
    _native.check(rc, "bnb_rmsnorm_bwd")
    if also_bf16:
        return dx.reshape(x.shape), dw, dx_lp.reshape(x.shape)
    return dx.reshape(x.shape), dw


def rmsnorm_bwd_static(x: torch.Tensor, dy: torch.Tensor, weight: torch.Tensor, dx: torch.Tensor, dw: torch.Tensor, *,
                       eps: float | None = None, grad_sum: torch.Tensor | None = None,
                       dx_bf16: torch.Tensor | None = None) -> None:
    """``rmsnorm_bwd`` into the caller's ``dx`` (R, D) float32, ``dw`` (D,) float32 and optional ``dx_bf16``,
    allocating nothing: the partial weight gradients use the library's built-in buffer (one per GPU,
    shared by all calls on that GPU, so concurrent calls on one GPU must be ordered by the caller).
    For code that cannot allocate around the call, e.g. under HIP graph capture.  All tensors must
    have contiguous (R, D) rows already; nothing is copied."""
    D = x.shape[-1]
    R = x.numel() // D if D else 0
    for t, name, dt in ((x, "x", torch.float32), (weight, "weight", torch.float32), (dx, "dx", torch.float32),
                        (dw, "dw", torch.float32)):
        _need_device(t, name)
        if t.dtype != dt or not t.is_contiguous():
            raise TypeError(f"{name} must be contiguous {dt}")
    _need_device(dy, "dy")
    if not dy.is_contiguous() or dy.shape != x.shape or dx.shape != x.shape or weight.shape != (D,) or dw.shape != (D,):
        raise ValueError("dy and dx must be contiguous with x's shape, weight and dw (D,)")
    for t, name, dt in ((grad_sum, "grad_sum", torch.float32), (dx_bf16, "dx_bf16", torch.bfloat16)):
        if t is not None and (t.dtype != dt or not t.is_contiguous() or t.shape != x.shape or not t.is_cuda):
            raise TypeError(f"{name} must be a contiguous {dt} device tensor with x's shape")
    with _on_device(x.device):
        rc = _native.load().bnb_rmsnorm_bwd_static(
            x.data_ptr(), D, dy.data_ptr(), _code(dy, "dy"), D, weight.data_ptr(), _F32_EPS if eps is None else float(eps),
            None if grad_sum is None else grad_sum.data_ptr(), dx.data_ptr(), None if dx_bf16 is None else dx_bf16.data_ptr(),
            dw.data_ptr(), R, D, _stream())
    _native.check(rc, "bnb_rmsnorm_bwd_static")


class _RmsNormTrain(torch.autograd.Function):
    """``(x, rmsnorm(x) * weight)``: x is handed through so that the gradient arriving on the residual
    branch reaches the backward kernel, which adds it in the same pass."""

    @staticmethod
    def forward(ctx, x, weight, eps, out_dtype):
        with torch.no_grad():
            n = add_rmsnorm(x, weight, eps=eps, out_dtype=out_dtype)[1]
        ctx.save_for_backward(x, weight)
        ctx.set_materialize_grads(False)
        ctx.eps = eps
        return x.view_as(x), n

    @staticmethod
    @_outside_autocast
    def backward(ctx, ds, dn):
        x, weight = ctx.saved_tensors
        if dn is None:
            dn = torch.zeros_like(x)
        dx, dw = rmsnorm_bwd(x, dn, weight, eps=ctx.eps, grad_sum=ds)
        return dx, dw, None, None


class _AddRmsNormTrain(torch.autograd.Function):
    """``s = x + delta`` and ``rmsnorm(s) * weight``; the backward adds the gradient of ``s`` inside
    the norm-backward kernel and writes a bfloat16 delta's gradient in the same pass."""

    @staticmethod
    def forward(ctx, x, delta, weight, eps, out_dtype):
        with torch.no_grad():
            s, n = add_rmsnorm(x, weight, delta=delta, eps=eps, out_dtype=out_dtype)
        ctx.save_for_backward(s, weight)
        ctx.set_materialize_grads(False)
        ctx.eps = eps
        ctx.delta_dtype = delta.dtype
        return s, n

    @staticmethod
    @_outside_autocast
    def backward(ctx, ds, dn):
        s, weight = ctx.saved_tensors
        if dn is None:
            dn = torch.zeros_like(s)
        if ctx.delta_dtype == torch.bfloat16:
            dx, dw, ddelta = rmsnorm_bwd(s, dn, weight, eps=ctx.eps, grad_sum=ds, also_bf16=True)
        else:
            dx, dw = rmsnorm_bwd(s, dn, weight, eps=ctx.eps, grad_sum=ds)
            ddelta = dx
        return dx, ddelta, dw, None, None


class _NormLinearTrain(torch.autograd.Function):
    """``(x, linear(rmsnorm(x) * norm_weight), rmsnorm(x) * norm_weight)`` under bfloat16 autocast as one
    kernel forward: the projection's launch also writes the normalised rows, which are all the backward keeps
    besides x.  Backward: the library's input-gradient GEMM, the weight-gradient kernel and the norm's backward
    kernel, which adds the gradients reaching x (residual branch) and the normalised rows (their other users)
    in the same pass."""

    @staticmethod
    def forward(ctx, x, norm_weight, weight, eps, packed):
        D = x.shape[-1]
        x2 = x.reshape(-1, D)
        if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) % 4):
            x2 = x2.contiguous()
        R, N = x2.shape[0], weight.shape[0]
        y = torch.empty((R, N), dtype=torch.bfloat16, device=x.device)
        n = torch.empty((R, D), dtype=torch.bfloat16, device=x.device)
        if R:
            with _on_device(x.device):
                rc = _native.load().bnb_norm_linear_train_fwd(
                    x2.data_ptr(), x2.stride(0), norm_weight.detach().contiguous().data_ptr(),
                    float(_F32_EPS if eps is None else eps), packed.data_ptr(), y.data_ptr(), n.data_ptr(), R, D, N, _stream())
            _native.check(rc, "bnb_norm_linear_train_fwd")
        ctx.save_for_backward(x, norm_weight, weight, n)
        ctx.set_materialize_grads(False)
        ctx.eps = eps
        n_out = n.view(x.shape)
        return x.view_as(x), y.view(*x.shape[:-1], N), n_out

    @staticmethod
    @_outside_autocast
    def backward(ctx, ds, dy, dn_other):
        x, norm_weight, weight, n = ctx.saved_tensors
        D = x.shape[-1]
        dn = None
        d_weight = None
        if dn_other is not None:
            dn_other = dn_other.reshape(-1, D)
        if dy is not None:
            dy2 = dy.reshape(-1, dy.shape[-1])
            dyb = dy2 if dy2.dtype == torch.bfloat16 else dy2.to(torch.bfloat16)
            if dyb.stride(-1) != 1:
                dyb = dyb.contiguous()
            wb = weight.detach().to(torch.bfloat16)
            if dn_other is None:
                dn = torch.matmul(dyb, wb)
            else:
                # one rounding of (dy W + the other users' gradient) in the GEMM's epilogue instead of a second pass
                dn = torch.addmm(dn_other.to(torch.bfloat16), dyb, wb)
            if ctx.needs_input_grad[2]:
                d_weight = linear_wgrad(dyb, n)
        elif dn_other is not None:
            dn = dn_other
        if dn is None:
            dn = torch.zeros_like(n)
        dx, d_norm = rmsnorm_bwd(x, dn.view(x.shape), norm_weight, eps=ctx.eps, grad_sum=ds)
        return dx, d_norm, d_weight, None, None


def norm_linear_train_supported(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether ``norm_linear_train`` covers this projection: float32 (..., 128) rows on the GPU, a float32 (N, 128)
    weight with N a multiple of 64, enough rows for the weight-gradient kernel."""
    return (x.is_cuda and x.dtype == torch.float32 and x.shape[-1] == FFN_WIDTH and weight.dtype == torch.float32
            and weight.dim() == 2 and weight.shape[1] == FFN_WIDTH and weight.shape[0] % 64 == 0
            and linear_wgrad_supported(x, weight))


def norm_linear_train(x: torch.Tensor, norm_weight: torch.Tensor, weight: torch.Tensor, *, eps: float | None = None,
                      packed: torch.Tensor | None = None):
    """Differentiable ``norm_linear`` for the update under bfloat16 autocast: returns ``(x, y, n)`` with
    ``n = bf16(rmsnorm(x) * norm_weight)`` and ``y = n @ weight^T`` (bfloat16, float32 accumulation).  Use the returned
    x for the residual connection (its gradient is then added inside the norm's backward kernel) and ``n`` for any other
    projection of the same normalised rows.  ``packed``: ``pack_linear_weights(weight)``, if the caller caches it."""
    if packed is None:
        packed = pack_linear_weights(weight)
    with torch.autocast("cuda", enabled=False):
        return _NormLinearTrain.apply(x, norm_weight, weight, eps, packed)


def rmsnorm_train_supported(x: torch.Tensor) -> bool:
    """Whether ``rmsnorm_train`` covers this input: float32 rows of a covered width on the GPU."""
    return x.is_cuda and x.dtype == torch.float32 and x.shape[-1] in _NORM_TRAIN_WIDTHS


def rmsnorm_train(x: torch.Tensor, weight: torch.Tensor, *, delta: torch.Tensor | None = None, eps: float | None = None,
                  out_dtype: torch.dtype = torch.float32):
    """Differentiable ``add_rmsnorm``: returns ``(s, normed)`` with ``s = x + delta``, or ``s`` = x itself
    (an alias, to be used for the residual connection so that its gradient is added inside the backward
    kernel) without ``delta``.  ``normed`` is computed in float32 and rounded once to ``out_dtype`` (what
    ``nn.RMSNorm`` followed by autocast's cast in front of the next Linear gives)."""
    with torch.autocast("cuda", enabled=False):
        if delta is None:
            return _RmsNormTrain.apply(x, weight, eps, out_dtype)
        return _AddRmsNormTrain.apply(x, delta, weight, eps, out_dtype)


def gelu_mul(a: torch.Tensor, b: torch.Tensor, *, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``gelu(a) * b`` (erf GELU) for (..., H) tensors whose rows may be strided.

    The gelu is rounded to a's dtype (as ``F.gelu`` returns it), the product once to
    ``out_dtype`` (default: torch's promotion of a and b).
    """
    if a.shape != b.shape:
        raise ValueError(f"a {tuple(a.shape)} and b {tuple(b.shape)} differ")
    H = a.shape[-1]
    if H % 8:
        raise ValueError(f"gelu_mul needs a multiple of 8 channels, got {H}")
    _need_device(a, "a")
    _need_device(b, "b")
    if torch.is_grad_enabled() and (a.requires_grad or b.requires_grad):
        raise RuntimeError("gelu_mul is forward-only; call it under torch.no_grad()")
    if out_dtype is None:
        out_dtype = torch.promote_types(a.dtype, b.dtype)

    def rows(t):
        t2 = t.reshape(-1, H) if t.dim() != 2 else t
        if t2.numel() and t2.stride(-1) != 1:
            t2 = t2.contiguous()
        return t2

    a2, b2 = rows(a), rows(b)
    R = a2.shape[0]
    out = torch.empty((R, H), dtype=out_dtype, device=a.device)
    if R:
        with _on_device(a.device):
            rc = _native.load().bnb_gelu_mul_fwd(
                a2.data_ptr(), _code(a2, "a"), a2.stride(0), b2.data_ptr(), _code(b2, "b"), b2.stride(0),
                out.data_ptr(), _code(out, "out_dtype"), R, H, _stream(),
            )
        _native.check(rc, "bnb_gelu_mul_fwd")
    return out.reshape(a.shape)


def gelu_mul_bwd(a: torch.Tensor, b: torch.Tensor, dout: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Backward of ``gelu_mul``: ``(da, db)`` in a's and b's dtypes from the gradient of the product."""
    H = a.shape[-1]
    if a.shape != b.shape or dout.shape != a.shape or H % 8:
        raise ValueError("a, b and dout must share a shape with a multiple of 8 channels")
    for name, t in (("a", a), ("b", b), ("dout", dout)):
        _need_device(t, name)

    def rows(t):
        t2 = t.reshape(-1, H) if t.dim() != 2 else t
        if t2.numel() and t2.stride(-1) != 1:
            t2 = t2.contiguous()
        return t2

    a2, b2, g2 = rows(a), rows(b), rows(dout).contiguous()
    R = a2.shape[0]
    da = torch.empty((R, H), dtype=a.dtype, device=a.device)
    db = torch.empty((R, H), dtype=b.dtype, device=a.device)
    if R:
        with _on_device(a.device):
            rc = _native.load().bnb_gelu_mul_bwd(
                a2.data_ptr(), _code(a2, "a"), a2.stride(0), b2.data_ptr(), _code(b2, "b"), b2.stride(0),
                g2.data_ptr(), _code(g2, "dout"), da.data_ptr(), H, db.data_ptr(), H, R, H, _stream(),
            )
        _native.check(rc, "bnb_gelu_mul_bwd")
    return da.reshape(a.shape), db.reshape(a.shape)


class _GeluMulTrain(torch.autograd.Function):
    """``gelu(a) * b`` with one kernel forward and one backward."""

    @staticmethod
    def forward(ctx, a, b, out_dtype):
        with torch.no_grad():
            out = gelu_mul(a, b, out_dtype=out_dtype)
        ctx.save_for_backward(a, b)
        return out

    @staticmethod
    @_outside_autocast
    def backward(ctx, dout):
        a, b = ctx.saved_tensors
        da, db = gelu_mul_bwd(a, b, dout)
        return da, db, None


class _GeluMulPackedTrain(torch.autograd.Function):
    """``gelu(gu[..., :H]) * gu[..., H:]`` on one (..., 2H) projection output; the backward writes both
    halves of its gradient in place (no slices to stitch)."""

    @staticmethod
    def forward(ctx, gu, out_dtype):
        H = gu.shape[-1] // 2
        with torch.no_grad():
            out = gelu_mul(gu[..., :H], gu[..., H:], out_dtype=out_dtype)
        ctx.save_for_backward(gu)
        return out

    @staticmethod
    @_outside_autocast
    def backward(ctx, dout):
        (gu,) = ctx.saved_tensors
        H = gu.shape[-1] // 2
        g2 = gu.reshape(-1, 2 * H)
        if g2.numel() and g2.stride(-1) != 1:
            g2 = g2.contiguous()
        d2 = dout.reshape(-1, H).contiguous()
        R = g2.shape[0]
        dgu = torch.empty((R, 2 * H), dtype=gu.dtype, device=gu.device)
        if R:
            code = _code(g2, "gu")
            with _on_device(gu.device):
                rc = _native.load().bnb_gelu_mul_bwd(
                    g2.data_ptr(), code, g2.stride(0), g2.data_ptr() + H * g2.element_size(), code, g2.stride(0),
                    d2.data_ptr(), _code(d2, "dout"), dgu.data_ptr(), 2 * H, dgu.data_ptr() + H * dgu.element_size(), 2 * H,
                    R, H, _stream(),
                )
            _native.check(rc, "bnb_gelu_mul_bwd")
        return dgu.reshape(gu.shape), None


def gelu_mul_packed_train(gu: torch.Tensor, *, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Differentiable ``gelu(gate) * up`` for ``gu = [gate | up]`` (..., 2H), the output of one projection
    over concatenated weights.  Needs H % 8 == 0 and a float32 or bfloat16 tensor on the GPU."""
    H2 = gu.shape[-1]
    if H2 % 16 or gu.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("gu must be float32 or bfloat16 with 2H channels, H a multiple of 8")
    _need_device(gu, "gu")
    with torch.autocast("cuda", enabled=False):
        return _GeluMulPackedTrain.apply(gu, gu.dtype if out_dtype is None else out_dtype)


def gelu_mul_train_supported(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Whether ``gelu_mul_train`` covers these operands."""
    ok = (torch.float32, torch.bfloat16)
    return a.is_cuda and b.is_cuda and a.shape == b.shape and a.shape[-1] % 8 == 0 and a.dtype in ok and b.dtype in ok


def gelu_mul_train(a: torch.Tensor, b: torch.Tensor, *, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """Differentiable ``gelu_mul``."""
    with torch.autocast("cuda", enabled=False):
        return _GeluMulTrain.apply(a, b, out_dtype)


def copy_bytes(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Device copy through the library's 16-byte copy kernel (bandwidth yardstick)."""
    _need_device(src, "src")
    _need_device(dst, "dst")
    n = src.numel() * src.element_size()
    if n != dst.numel() * dst.element_size() or not (src.is_contiguous() and dst.is_contiguous()):
        raise ValueError("src and dst must be contiguous and of equal byte size")
    with _on_device(src.device):
        rc = _native.load().bnb_copy_bytes(src.data_ptr(), dst.data_ptr(), n, _stream())
    _native.check(rc, "bnb_copy_bytes")


def issue_probe(valu_per_mfma: int, *, mfma: bool = True, transcendentals: bool = False, waves_per_simd: int = 2,
                iters: int = 20000, device=None) -> float:
    """Issue time in nanoseconds of one slot = one 32x32x16 bfloat16 matrix product (``mfma``) followed by
    ``valu_per_mfma`` independent vector instructions (multiply-adds, every fifth one an exp2 with
    ``transcendentals``) on one SIMD carrying ``waves_per_simd`` waves: the yardstick for the kernels that are bound
    by instruction issue rather than by bandwidth (``bnb_issue_probe``).  Synchronises the device."""
    dev = torch.device(device if device is not None else "cuda")
    sink = torch.zeros(256, dtype=torch.float32, device=dev)
    lib = _native.load()
    with _on_device(sink.device):
        def launch(n):
            _native.check(lib.bnb_issue_probe(int(valu_per_mfma), int(mfma), int(transcendentals), int(waves_per_simd), n,
                                              sink.data_ptr(), _stream()), "bnb_issue_probe")
        launch(200)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        launch(iters)
        stop.record()
        stop.synchronize()
    return start.elapsed_time(stop) * 1e6 / (4.0 * iters * waves_per_simd)


FFN_WIDTH, FFN_HIDDEN = 128, 512


def pack_ffn_weights(gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor) -> torch.Tensor:
    """``gate_proj``/``up_proj`` (512, 128) and ``down_proj`` (128, 512) weights as the bfloat16
    operand stream of ``ffn_fused``: 16 chunks of 32 hidden units, each
    ``[gate (8, 64, 8) | up (8, 64, 8) | down (4, 2, 64, 8)]`` with the index meaning given in
    ``include/bnb_amd.h`` (every matrix-core operand is one contiguous 1 KB run)."""
    D, Hd = FFN_WIDTH, FFN_HIDDEN
    if gate_w.shape != (Hd, D) or up_w.shape != (Hd, D) or down_w.shape != (D, Hd):
        raise ValueError("ffn_fused covers d_model 128 with a hidden width of 512")
    dev = gate_w.device
    lane = torch.arange(64, device=dev)
    m, half = lane % 32, lane // 32
    e = torch.arange(8, device=dev)
    c = torch.arange(Hd // 32, device=dev)
    ks = torch.arange(8, device=dev)
    rows = (32 * c[:, None, None, None] + m[None, None, :, None]).expand(-1, 8, -1, 8)  # (16, 8, 64, 8)
    cols = (16 * ks[None, :, None, None] + 8 * (e // 4)[None, None, None, :] + 4 * half[None, None, :, None]
            + (e % 4)[None, None, None, :]).expand(16, -1, -1, -1)
    g = gate_w.detach().to(torch.bfloat16)[rows, cols]
    u = up_w.detach().to(torch.bfloat16)[rows, cols]
    cb = torch.arange(4, device=dev)
    t = torch.arange(2, device=dev)
    d_rows = (32 * cb[:, None] + m[None, :])[None, :, None, :, None].expand(16, -1, 2, -1, 8)  # (16, 4, 2, 64, 8)
    d_cols = (32 * c[:, None, None, None, None] + 16 * t[None, None, :, None, None]
              + 8 * (e // 4)[None, None, None, None, :] + 4 * half[None, None, None, :, None]
              + (e % 4)[None, None, None, None, :]).expand(-1, 4, -1, -1, -1)
    d = down_w.detach().to(torch.bfloat16)[d_rows, d_cols]
    return torch.cat([g.reshape(16, -1), u.reshape(16, -1), d.reshape(16, -1)], dim=1).contiguous()


def pack_proj_weights(weight: torch.Tensor) -> torch.Tensor:
    """A (128, 128) output-projection weight as the bfloat16 operand stream of the projection
    folded into ``ffn_fused``: ``[cb][ks][l][e] = W[32cb + l%32][16ks + 8(e/4) + 4(l/32) + e%4]``."""
    if weight.shape != (FFN_WIDTH, FFN_WIDTH):
        raise ValueError("the folded projection covers (128, 128) weights")
    dev = weight.device
    lane = torch.arange(64, device=dev)
    m, half = lane % 32, lane // 32
    e = torch.arange(8, device=dev)
    cb = torch.arange(4, device=dev)
    ks = torch.arange(8, device=dev)
    rows = (32 * cb[:, None, None, None] + m[None, None, :, None]).expand(-1, 8, -1, 8)
    cols = (16 * ks[None, :, None, None] + 8 * (e // 4)[None, None, None, :] + 4 * half[None, None, :, None]
            + (e % 4)[None, None, None, :]).expand(4, -1, -1, -1)
    return weight.detach().to(torch.bfloat16)[rows, cols].contiguous()


def pack_head_weights(weight: torch.Tensor) -> torch.Tensor:
    """A (N, 128) projection weight (N a multiple of 64, at least 128) as the bfloat16 operand stream of the
    next-sublayer head folded into ``ffn_fused``: chunks of 64 features,
    ``[c][b][ks][l][e] = W[64c + 32b + pi(l%32)][16ks + 8(e/4) + 4(l/32) + e%4]`` with
    ``pi(m) = 16(m/16) + 8((m/4)%2) + 4((m/8)%2) + m%4``."""
    N, D = weight.shape
    if D != FFN_WIDTH or N % 64 or N < 128:
        raise ValueError("the folded head covers (N, 128) weights with N a multiple of 64, at least 128")
    dev = weight.device
    lane = torch.arange(64, device=dev)
    m, half = lane % 32, lane // 32
    pi = 16 * (m // 16) + 8 * ((m // 4) % 2) + 4 * ((m // 8) % 2) + m % 4
    e = torch.arange(8, device=dev)
    blk = torch.arange(N // 32, device=dev)
    ks = torch.arange(8, device=dev)
    rows = (32 * blk[:, None, None, None] + pi[None, None, :, None]).expand(-1, 8, -1, 8)
    cols = (16 * ks[None, :, None, None] + 8 * (e // 4)[None, None, None, :] + 4 * half[None, None, :, None]
            + (e % 4)[None, None, None, :]).expand(N // 32, -1, -1, -1)
    return weight.detach().to(torch.bfloat16)[rows, cols].contiguous()


def pack_ffn_bwd_weights(gate_w: torch.Tensor, up_w: torch.Tensor, down_w: torch.Tensor) -> torch.Tensor:
    """The three GatedMLP weights as the bfloat16 operand stream of ``ffn_bwd``: 16 chunks of 32 hidden
    units, each ``[gate (8, 64, 8) | up (8, 64, 8) | down^T (8, 64, 8) | gate^T (4, 2, 64, 8) | up^T (4, 2, 64, 8)]``
    with the index meaning given in ``include/bnb_amd.h``."""
    D, Hd = FFN_WIDTH, FFN_HIDDEN
    if gate_w.shape != (Hd, D) or up_w.shape != (Hd, D) or down_w.shape != (D, Hd):
        raise ValueError("ffn_bwd covers d_model 128 with a hidden width of 512")
    dev = gate_w.device
    lane = torch.arange(64, device=dev)
    m, b = lane % 32, lane // 32
    pi = 16 * (m // 16) + 8 * ((m // 4) % 2) + 4 * ((m // 8) % 2) + m % 4  # unit that matrix-core row m stands for
    e = torch.arange(8, device=dev)
    c = torch.arange(Hd // 32, device=dev)
    ks = torch.arange(8, device=dev)
    # sections 0-2: (16, 8, 64, 8), rows = hidden unit, columns = channel
    hid = (32 * c[:, None, None, None] + pi[None, None, :, None]).expand(-1, 8, -1, 8)
    ch = (16 * ks[None, :, None, None] + 8 * b[None, None, :, None] + e[None, None, None, :]).expand(16, -1, -1, -1)
    wg, wu, wd = (w.detach().to(torch.bfloat16) for w in (gate_w, up_w, down_w))
    s0, s1, s2 = wg[hid, ch], wu[hid, ch], wd[ch, hid]
    # sections 3-4: (16, 4, 2, 64, 8), contraction over the chunk's hidden units, rows = channel
    cb = torch.arange(4, device=dev)
    t = torch.arange(2, device=dev)
    k_hid = (32 * c[:, None, None, None, None] + 16 * t[None, None, :, None, None] + 8 * b[None, None, None, :, None]
             + e[None, None, None, None, :]).expand(-1, 4, -1, -1, -1)
    r_ch = (32 * cb[None, :, None, None, None] + pi[None, None, None, :, None]).expand(16, -1, 2, -1, 8)
    s3, s4 = wg[k_hid, r_ch], wu[k_hid, r_ch]
    return torch.cat([x.reshape(16, -1) for x in (s0, s1, s2, s3, s4)], dim=1).contiguous()


def ffn_bwd(n: torch.Tensor, dy: torch.Tensor, weights_packed: torch.Tensor):
    """Backward of ``y = down(gelu(gate(n)) * up(n))`` with the gate/up activations recomputed on chip.

    n (R, 128) bfloat16 contiguous, dy (R, 128) float32 or bfloat16, ``weights_packed`` from
    ``pack_ffn_bwd_weights``.  Returns ``(dn, dgu, h, dy_bf16)``: dn (R, 128) bfloat16; ``dgu`` (8, Rp, 128) and
    ``h`` (4, Rp, 128) bfloat16, the tile-by-tile operands of the weight gradients (see ``ffn_weight_grads``;
    Rp is R rounded up to a multiple of 256, rows past R are don't-cares); dy rounded to bfloat16 (dy itself
    when it already is)."""
    D = FFN_WIDTH
    _need_device(n, "n")
    _need_device(dy, "dy")
    if n.dim() != 2 or n.shape[1] != D or n.dtype != torch.bfloat16 or not n.is_contiguous():
        raise ValueError("n must be a contiguous bfloat16 (R, 128) tensor")
    if dy.shape != n.shape or dy.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("dy must be a float32 or bfloat16 tensor of n's shape")
    if weights_packed.dtype != torch.bfloat16 or weights_packed.numel() != 5 * FFN_HIDDEN * D or not weights_packed.is_contiguous():
        raise ValueError("weights_packed must come from pack_ffn_bwd_weights")
    if not _uniform_rows(dy, D):
        dy = dy.contiguous()
    R = n.shape[0]
    Rp = (R + 255) // 256 * 256
    dev = n.device
    dn = torch.empty((Rp, D), dtype=torch.bfloat16, device=dev)
    dgu = torch.empty((8, Rp, 128), dtype=torch.bfloat16, device=dev)
    h = torch.empty((4, Rp, 128), dtype=torch.bfloat16, device=dev)
    dy_lp = torch.empty((Rp, D), dtype=torch.bfloat16, device=dev) if dy.dtype == torch.float32 else None
    if R:
        with _on_device(dev):
            rc = _native.load().bnb_ffn_bwd(n.data_ptr(), dy.data_ptr(), _code(dy, "dy"), dy.stride(0), weights_packed.data_ptr(),
                                            dn.data_ptr(), dgu.data_ptr(), h.data_ptr(),
                                            None if dy_lp is None else dy_lp.data_ptr(), R, Rp, D, FFN_HIDDEN, _stream())
        _native.check(rc, "bnb_ffn_bwd")
    return dn[:R], dgu, h, (dy if dy_lp is None else dy_lp[:R])


def ffn_weight_grads(n: torch.Tensor, dgu: torch.Tensor, h: torch.Tensor, dy_bf16: torch.Tensor):
    """``(d gate_proj.weight, d up_proj.weight, d down_proj.weight)`` (float32) from ``ffn_bwd``'s operands."""
    R = n.shape[0]
    dw = _linear_wgrad_tiled(dgu, n, R).view(8, 2, 2, 32, FFN_WIDTH)  # [pair][chunk in pair][gate, up][unit][channel]
    d_gate = dw[:, :, 0].reshape(FFN_HIDDEN, FFN_WIDTH)
    d_up = dw[:, :, 1].reshape(FFN_HIDDEN, FFN_WIDTH)
    return d_gate, d_up, _linear_wgrad_tiled(dy_bf16, h, R)


class _FfnTailTrain(torch.autograd.Function):
    """``s = x + d; s + mlp(rmsnorm(s) * w)`` for the update path, with ``d`` = ``delta`` or, with a projection weight,
    ``delta @ proj_w^T`` formed inside the kernel: forward on the fused sublayer-tail kernel (which also writes
    ``s`` and the normalised rows), backward on ``ffn_bwd``, the weight-gradient kernel and the norm's backward
    kernel.  Only ``s`` (float32), the normalised rows (bfloat16) and the projection's operand rows are kept."""

    @staticmethod
    def forward(ctx, x, delta, proj_w, norm_weight, gate_w, up_w, down_w, eps, packed_fwd, packed_bwd, proj_packed):
        D = x.shape[-1]
        x2 = x.reshape(-1, D)
        if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) % 4):
            x2 = x2.contiguous()
        R = x2.shape[0]
        dev = x.device
        out = torch.empty((R, D), dtype=torch.float32, device=dev)
        n = torch.empty((R, D), dtype=torch.bfloat16, device=dev)
        s, delta2 = None, None
        if delta is not None:
            delta2 = delta.reshape(-1, D)
            if proj_w is None or not _uniform_rows(delta2, D):
                delta2 = delta2.contiguous()
            s = torch.empty((R, D), dtype=torch.float32, device=dev)
        nw = norm_weight.detach().contiguous()
        if R:
            lib = _native.load()
            with _on_device(dev):
                if proj_w is None:
                    rc = lib.bnb_ffn_fused_train_fwd(
                        x2.data_ptr(), x2.stride(0), None if delta2 is None else delta2.data_ptr(), _native.BF16, nw.data_ptr(),
                        float(eps), packed_fwd.data_ptr(), out.data_ptr(), None if s is None else s.data_ptr(), n.data_ptr(), R, D,
                        FFN_HIDDEN, _stream())
                else:
                    rc = lib.bnb_ffn_fused_proj_train_fwd(
                        x2.data_ptr(), x2.stride(0), delta2.data_ptr(), delta2.stride(0), proj_packed.data_ptr(), nw.data_ptr(),
                        float(eps), packed_fwd.data_ptr(), out.data_ptr(), s.data_ptr(), n.data_ptr(), R, D, FFN_HIDDEN, _stream())
            _native.check(rc, "bnb_ffn_fused_train_fwd" if proj_w is None else "bnb_ffn_fused_proj_train_fwd")
        if proj_w is None:
            ctx.save_for_backward(x2 if s is None else s, n, nw, packed_bwd)
        else:
            ctx.save_for_backward(s, n, nw, packed_bwd, delta2, proj_w)
        ctx.eps = eps
        ctx.has_delta = delta is not None
        ctx.has_proj = proj_w is not None
        ctx.shape = x.shape
        return out.reshape(x.shape)

    @staticmethod
    @_outside_autocast
    def backward(ctx, dout):
        saved = ctx.saved_tensors  # read once: activation checkpointing unpacks on every access
        s, n, nw, packed_bwd = saved[:4]
        D = s.shape[-1]
        dout2 = dout.reshape(-1, D)
        if dout2.dtype != torch.float32:
            dout2 = dout2.float()
        dout2 = dout2.contiguous()
        dn, dgu, h, dy_lp = ffn_bwd(n, dout2, packed_bwd)
        need_w = ctx.needs_input_grad[4] or ctx.needs_input_grad[5] or ctx.needs_input_grad[6]
        d_gate = d_up = d_down = None
        if need_w:
            d_gate, d_up, d_down = ffn_weight_grads(n, dgu, h, dy_lp)
        del dgu, h
        ddelta = d_proj = None
        if ctx.has_delta:
            dx, dw, ds_lp = rmsnorm_bwd(s, dn, nw, eps=ctx.eps, grad_sum=dout2, also_bf16=True)
            if ctx.has_proj:
                # the projection's output gradient is the bfloat16 rounding of ds, as autograd hands it to a bf16 Linear
                rows, proj_w = saved[4:]
                if ctx.needs_input_grad[1]:
                    ddelta = torch.matmul(ds_lp, proj_w.to(torch.bfloat16)).reshape(ctx.shape)
                if ctx.needs_input_grad[2]:
                    d_proj = linear_wgrad(ds_lp, rows)
            else:
                ddelta = ds_lp.reshape(ctx.shape)
        else:
            dx, dw = rmsnorm_bwd(s, dn, nw, eps=ctx.eps, grad_sum=dout2)
        return dx.reshape(ctx.shape), ddelta, d_proj, dw, d_gate, d_up, d_down, None, None, None, None


def ffn_tail_train_supported(x: torch.Tensor, delta: torch.Tensor | None, hidden: int) -> bool:
    """Whether ``ffn_tail_train`` covers this sublayer tail: float32 (..., 128) residual stream on the GPU,
    hidden width 512, ``delta`` bfloat16 of x's shape or absent."""
    return ffn_supported(x, hidden) and (delta is None or (delta.dtype == torch.bfloat16 and delta.shape == x.shape))


def ffn_tail_train(x, delta, norm_weight, gate_w, up_w, down_w, *, eps: float | None, packed_fwd: torch.Tensor,
                   packed_bwd: torch.Tensor, proj_weight: torch.Tensor | None = None,
                   proj_packed: torch.Tensor | None = None) -> torch.Tensor:
    """Differentiable ``s = x + delta; s + down(gelu(gate(n)) * up(n))`` with ``n = rmsnorm(s) * norm_weight``, as
    bfloat16 autocast computes it, without saving the 512/1024-wide activations (``packed_fwd`` from
    ``pack_ffn_weights``, ``packed_bwd`` from ``pack_ffn_bwd_weights``, both of the current weights).

    With ``proj_weight`` (128, 128) and its ``pack_proj_weights`` arrangement, ``delta`` is the operand of a bias-free
    projection that runs inside the kernel: ``s = x + delta @ proj_weight^T`` (accumulated in float32 onto x, not
    rounded to bfloat16 first)."""
    if (proj_weight is None) != (proj_packed is None):
        raise ValueError("give proj_weight and proj_packed together")
    if proj_weight is not None and (delta is None or proj_weight.shape != (FFN_WIDTH, FFN_WIDTH) or proj_packed.dtype != torch.bfloat16
                                    or proj_packed.numel() != FFN_WIDTH * FFN_WIDTH or not proj_packed.is_contiguous()):
        raise ValueError("the folded projection needs its operand rows, a (128, 128) weight and pack_proj_weights' output")
    with torch.autocast("cuda", enabled=False):
        return _FfnTailTrain.apply(x, delta, proj_weight, norm_weight, gate_w, up_w, down_w, _F32_EPS if eps is None else float(eps),
                                   packed_fwd, packed_bwd, proj_packed)


def _uniform_rows(t: torch.Tensor, D: int) -> bool:
    """Whether ``t`` (..., D) can be viewed as rows at one regular pitch without a copy (a
    column block of a contiguous wider matrix qualifies)."""
    if t.stride(-1) != 1 or t.dim() < 2:
        return False
    try:
        v = t.view(-1, D)
    except RuntimeError:
        return False
    return v.stride(0) % 8 == 0 and v.stride(0) >= D and v.data_ptr() % 16 == 0


def ffn_supported(x: torch.Tensor, hidden: int) -> bool:
    """Whether ``ffn_fused`` covers this residual stream (fp32 on the GPU, width 128, hidden 512)."""
    return x.is_cuda and x.dtype == torch.float32 and x.shape[-1] == FFN_WIDTH and hidden == FFN_HIDDEN


def ffn_fused(
    x: torch.Tensor,
    delta: torch.Tensor | None,
    norm_weight: torch.Tensor,
    weights_packed: torch.Tensor,
    *,
    eps: float | None = None,
    out: torch.Tensor | None = None,
    proj: tuple | None = None,
    next_head: tuple | None = None,
):
    """``s = x + delta; s + down(gelu(gate(n)) * up(n))`` with ``n = rmsnorm(s) * norm_weight``,
    one matrix-core kernel with bfloat16 projections (what the sublayer tail computes under
    bfloat16 autocast).

    x (..., 128) float32 with contiguous rows; delta same shape, bfloat16, or None;
    ``weights_packed`` from ``pack_ffn_weights``.  Returns (..., 128) float32.

    ``proj`` folds the sublayer's output projection in (then ``delta`` must be None):
    ``(rows, wp)`` adds ``rows @ W^T``, ``(rows_g, rows_y, wp)`` adds
    ``(gelu(rows_g) * rows_y) @ W^T``; rows are bfloat16 with x's shape, ``wp`` from
    ``pack_proj_weights``.

    ``next_head = (next_norm_weight, next_eps, packed, N)`` (only with ``proj``) makes the same launch go on to
    the head of the next sublayer, ``bf16(rmsnorm(out) * next_norm_weight) @ Wh^T`` with ``packed`` from
    ``pack_head_weights`` (N features); the call then returns ``(out, head)`` with head (..., N) bfloat16.
    """
    D = x.shape[-1]
    if next_head is not None and proj is None:
        raise ValueError("next_head needs the folded projection form (proj=...)")
    if not ffn_supported(x, FFN_HIDDEN):
        raise RuntimeError("ffn_fused covers float32 (..., 128) residual streams on the GPU")
    _need_device(x, "x")
    if torch.is_grad_enabled() and (x.requires_grad or (delta is not None and delta.requires_grad)):
        raise RuntimeError("ffn_fused is forward-only; call it under torch.no_grad()")
    if weights_packed.dtype != torch.bfloat16 or weights_packed.numel() != 3 * FFN_HIDDEN * FFN_WIDTH or not weights_packed.is_contiguous():
        raise ValueError("weights_packed must come from pack_ffn_weights")
    if norm_weight.shape != (D,) or norm_weight.dtype != torch.float32:
        raise ValueError(f"norm_weight must be a float32 {(D,)} tensor")
    x2 = x.reshape(-1, D)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    R = x2.shape[0]
    delta_ptr = None
    if delta is not None:
        if delta.shape != x.shape or delta.dtype != torch.bfloat16:
            raise ValueError(f"delta must be a bfloat16 {tuple(x.shape)} tensor")
        delta = delta.reshape(-1, D).contiguous()
        delta_ptr = delta.data_ptr()
    if out is None:
        out = torch.empty((R, D), dtype=torch.float32, device=x.device)
    elif out.numel() != R * D or out.dtype != torch.float32 or not out.is_contiguous() or out.device != x.device:
        raise ValueError("out must be a contiguous float32 tensor of x's size on x's device")
    norm_weight = norm_weight.detach().contiguous()
    if proj is not None:
        if delta is not None:
            raise ValueError("give either delta or proj")
        *rows, wp = proj
        if len(rows) not in (1, 2) or wp.dtype != torch.bfloat16 or wp.numel() != D * D or not wp.is_contiguous():
            raise ValueError("proj must be (rows, packed) or (rows_g, rows_y, packed) with pack_proj_weights output")
        flat = []
        for k, t in enumerate(rows):
            if t.shape != x.shape or t.dtype != torch.bfloat16:
                raise ValueError(f"projection operand rows must be bfloat16 {tuple(x.shape)} tensors")
            if torch.is_grad_enabled() and t.requires_grad:
                raise RuntimeError("ffn_fused is forward-only; call it under torch.no_grad()")
            flat.append(t.view(-1, D) if _uniform_rows(t, D) else t.reshape(-1, D).contiguous())
        if next_head is not None:
            nw2, eps2, hp, N2 = next_head
            if (nw2.shape != (D,) or nw2.dtype != torch.float32 or hp.dtype != torch.bfloat16 or hp.numel() != N2 * D
                    or not hp.is_contiguous() or N2 % 64 or N2 < 128):
                raise ValueError("next_head must be (float32 (128,) norm weight, eps, pack_head_weights output, N)")
            Rp = (R + 127) // 128 * 128  # the head's stores are unconditional: room for whole work-groups
            head = torch.empty((Rp, N2), dtype=torch.bfloat16, device=x.device)
            if R:
                with _on_device(x.device):
                    rc = _native.load().bnb_ffn_fused_proj_next_fwd(
                        x2.data_ptr(), x2.stride(0), flat[0].data_ptr(), flat[0].stride(0),
                        flat[1].data_ptr() if len(flat) == 2 else None, flat[1].stride(0) if len(flat) == 2 else 0,
                        wp.data_ptr(), norm_weight.data_ptr(), float(_F32_EPS if eps is None else eps),
                        weights_packed.data_ptr(), out.data_ptr(), nw2.detach().contiguous().data_ptr(),
                        float(_F32_EPS if eps2 is None else eps2), hp.data_ptr(), head.data_ptr(), N2, Rp, R, D, FFN_HIDDEN,
                        _stream(),
                    )
                _native.check(rc, "bnb_ffn_fused_proj_next_fwd")
            return out.reshape(x.shape), head[:R].reshape(*x.shape[:-1], N2)
        if R:
            with _on_device(x.device):
                rc = _native.load().bnb_ffn_fused_proj_fwd(
                    x2.data_ptr(), x2.stride(0), flat[0].data_ptr(), flat[0].stride(0),
                    flat[1].data_ptr() if len(flat) == 2 else None, flat[1].stride(0) if len(flat) == 2 else 0,
                    wp.data_ptr(), norm_weight.data_ptr(), float(_F32_EPS if eps is None else eps),
                    weights_packed.data_ptr(), out.data_ptr(), R, D, FFN_HIDDEN, _stream(),
                )
            _native.check(rc, "bnb_ffn_fused_proj_fwd")
        return out.reshape(x.shape)
    if R:
        with _on_device(x.device):
            rc = _native.load().bnb_ffn_fused_fwd(
                x2.data_ptr(), x2.stride(0), delta_ptr, _native.BF16, norm_weight.data_ptr(),
                float(_F32_EPS if eps is None else eps), weights_packed.data_ptr(), out.data_ptr(), R, D, FFN_HIDDEN,
                _stream(),
            )
        _native.check(rc, "bnb_ffn_fused_fwd")
    return out.reshape(x.shape)


def pack_linear_f32(weight: torch.Tensor, up_weight: torch.Tensor | None = None) -> torch.Tensor:
    """A float32 Linear weight (N, K), N % 32 == 0, K % 128 == 0, as the operand stream of ``linear_f32``:
    ``[fb][s4][l][e] = W[32 fb + l%32][(l/32) K/2 + 4 s4 + e]`` (a lane's four next contraction steps are one
    16-byte piece of a 1 KB contiguous wave read).  With ``up_weight`` (same shape) the two matrices are
    interleaved in blocks of 32 rows, ``[gate block u, up block u]``, for the gated form."""
    w = weight.detach().float()
    N, K = w.shape
    if N % 32 or K % 128 or (up_weight is not None and up_weight.shape != weight.shape):
        raise ValueError("linear_f32 covers (N, K) weights with N % 32 == 0 and K % 128 == 0 (gate and up of one shape)")
    if up_weight is not None:
        u = up_weight.detach().float()
        w = torch.stack([w.view(N // 32, 32, K), u.view(N // 32, 32, K)], dim=1).reshape(2 * N, K)
        N = 2 * N
    dev = w.device
    lane = torch.arange(64, device=dev)
    rows = (32 * torch.arange(N // 32, device=dev)[:, None, None, None] + (lane % 32)[None, None, :, None]).expand(-1, K // 8, -1, 4)
    cols = ((lane // 32)[None, None, :, None] * (K // 2) + 4 * torch.arange(K // 8, device=dev)[None, :, None, None]
            + torch.arange(4, device=dev)[None, None, None, :]).expand(N // 32, -1, -1, -1)
    return w[rows, cols].contiguous()


def linear_f32_supported(x: torch.Tensor, n_features: int) -> bool:
    """Whether ``linear_f32`` covers this input: float32 rows on the GPU, K % 128 == 0, N % 32 == 0."""
    return (x.is_cuda and x.dtype == torch.float32 and x.shape[-1] % 128 == 0 and n_features % 32 == 0
            and x.stride(-1) == 1)


def linear_f32(x: torch.Tensor, weight_packed: torch.Tensor, *, bias: torch.Tensor | None = None,
               norm_weight: torch.Tensor | None = None, eps: float | None = None, gelu_times: torch.Tensor | None = None,
               gate: bool = False, resid: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    """A float32 Linear with its neighbours folded in, one kernel on the fp32 matrix cores.

    ``out = A W^T + bias (+ resid)`` with ``A = x``, or ``rmsnorm(x) * norm_weight`` (K = 128), or
    ``gelu(x) * gelu_times``; with ``gate`` the packed weight holds gate and up projections
    (``pack_linear_f32(gate_w, up_w)``) and ``out = gelu(A Wg^T) * (A Wu^T)``.  ``x`` (..., K) float32 with
    unit-stride channels and evenly spaced rows; ``resid`` / ``out`` (..., N_out) float32 contiguous."""
    K = x.shape[-1]
    _need_device(x, "x")
    if x.dtype != torch.float32 or weight_packed.dtype != torch.float32:
        raise TypeError("linear_f32 takes float32 rows and a float32 packed weight")
    n_blocks = weight_packed.shape[0]
    if weight_packed.dim() != 4 or weight_packed.shape[1:] != (K // 8, 64, 4) or not weight_packed.is_contiguous():
        raise ValueError("weight_packed must come from pack_linear_f32 for this contraction width")
    N = 32 * n_blocks
    n_out = N // 2 if gate else N
    if torch.is_grad_enabled() and x.requires_grad:
        raise RuntimeError("linear_f32 is forward-only; call it under torch.no_grad()")
    x2 = x.reshape(-1, K) if _uniform_rows(x, K) else x.reshape(-1, K).contiguous()
    R = x2.shape[0]
    y2 = None
    if gelu_times is not None:
        if gelu_times.shape != x.shape or gelu_times.dtype != torch.float32:
            raise ValueError("gelu_times must be float32 with x's shape")
        y2 = gelu_times.reshape(-1, K) if _uniform_rows(gelu_times, K) else gelu_times.reshape(-1, K).contiguous()
    lead = x.shape[:-1]
    if out is None:
        out = torch.empty((*lead, n_out), dtype=torch.float32, device=x.device)
    elif out.shape != (*lead, n_out) or out.dtype != torch.float32 or not out.is_contiguous():
        raise ValueError(f"out must be a contiguous float32 {(*lead, n_out)} tensor")
    r2 = None
    if resid is not None:
        if resid.shape != (*lead, n_out) or resid.dtype != torch.float32:
            raise ValueError(f"resid must be float32 {(*lead, n_out)}")
        r2 = resid.reshape(-1, n_out) if _uniform_rows(resid, n_out) else resid.reshape(-1, n_out).contiguous()
    if R == 0:
        return out
    with _on_device(x.device):
        rc = _native.load().bnb_linear_f32_fwd(
            x2.data_ptr(), x2.stride(0) if R > 1 else K, None if y2 is None else y2.data_ptr(),
            0 if y2 is None else (y2.stride(0) if R > 1 else K), None if norm_weight is None else norm_weight.detach().contiguous().data_ptr(),
            float(_F32_EPS if eps is None else eps), weight_packed.data_ptr(), None if bias is None else bias.detach().contiguous().data_ptr(),
            None if r2 is None else r2.data_ptr(), 0 if r2 is None else (r2.stride(0) if R > 1 else n_out), out.data_ptr(), n_out, R, K, N,
            1 if gate else 0, _stream())
    _native.check(rc, "bnb_linear_f32_fwd")
    return out


def pack_linear_weights(weight: torch.Tensor) -> torch.Tensor:
    """A Linear weight (N, 128), N a multiple of 64, as the bfloat16 operand stream of
    ``norm_linear``: ``[fb][ks][l][e]`` with the index meaning given in ``include/bnb_amd.h``
    (every matrix-core operand one contiguous 1 KB run; a lane's 16 outputs per block of 32
    features are two runs of 8 consecutive features)."""
    N, D = weight.shape
    if D != FFN_WIDTH or N % 64:
        raise ValueError("norm_linear covers (N, 128) weights with N a multiple of 64")
    dev = weight.device
    lane = torch.arange(64, device=dev)
    r, half = lane % 32, lane // 32
    e = torch.arange(8, device=dev)
    fb = torch.arange(N // 32, device=dev)
    ks = torch.arange(8, device=dev)
    feat = 16 * ((r // 8) // 2) + 8 * ((r // 4) % 2) + 4 * ((r // 8) % 2) + r % 4  # (64,)
    rows = (32 * fb[:, None, None, None] + feat[None, None, :, None]).expand(-1, 8, -1, 8)
    cols = (16 * ks[None, :, None, None] + 8 * (e // 4)[None, None, None, :] + 4 * half[None, None, :, None]
            + (e % 4)[None, None, None, :]).expand(N // 32, -1, -1, -1)
    return weight.detach().to(torch.bfloat16)[rows, cols].contiguous()


class CompactRows:
    """The set entries of a (B, n) bool mask as a device-side list: ``index`` (capacity B*n,
    int32 flat positions b*n + j, ascending, the first ``offsets[B]`` valid) and ``offsets``
    (B+1, int32 exclusive prefix of the per-row counts).  Built without any copy to the host.

    ``total`` / ``max_count`` (optional Python ints): the number of set entries and the largest count of
    one row, for a caller that knows them already (e.g. counted when the rollout was stored).  The
    update path sizes gathered tensors with them and picks the single-tile or the streaming backward by
    ``max_count``; without the hint ``total_host()`` copies them from the device once, which makes the host
    wait for everything queued before.  The hints are taken on trust: a ``total`` below the true count makes
    the gathered tensors too small for what the kernels write, a ``max_count`` below the true one sends a row with
    more than 160 entries to the single-tile backward, and either is undefined behaviour.  ``check_hints()``
    compares them with the device's counts (one copy to the host); with ``BNB_CHECK_HINTS=1`` in the environment
    every construction with hints does that."""

    def __init__(self, mask: torch.Tensor, *, total: int | None = None, max_count: int | None = None) -> None:
        if mask.dim() != 2 or mask.dtype not in (torch.bool, torch.uint8):
            raise ValueError("mask must be a bool (B, n) tensor")
        _need_device(mask, "mask")
        mask = mask.contiguous()
        B, n = mask.shape
        if B * n >= 2 ** 31:
            raise ValueError("mask too large for 32-bit row positions")
        self.shape = (B, n)
        self.mask = mask
        if (total is None) != (max_count is None):
            raise ValueError("give both total and max_count, or neither")
        self._host = None if total is None else (int(total), int(max_count))
        self._hinted = total is not None
        self.shared_kv = None  # set by the trunk: {id(layer): [K | V] rows of the listed entries}, one projection pass for all readers
        counts = torch.empty(B, dtype=torch.int32, device=mask.device)
        self.offsets = torch.zeros(B + 1, dtype=torch.int32, device=mask.device)
        self.index = torch.empty(max(B * n, 1), dtype=torch.int32, device=mask.device)
        if B and n:
            lib = _native.load()
            with _on_device(mask.device):
                _native.check(lib.bnb_mask_count(mask.data_ptr(), counts.data_ptr(), B, n, _stream()), "bnb_mask_count")
                torch.cumsum(counts, dim=0, dtype=torch.int32, out=self.offsets[1:])
                _native.check(lib.bnb_mask_fill(mask.data_ptr(), self.offsets.data_ptr(), self.index.data_ptr(), B, n,
                                                _stream()), "bnb_mask_fill")

        if self._hinted and os.environ.get("BNB_CHECK_HINTS") == "1":
            self.check_hints()

    def check_hints(self) -> None:
        """Raise ``ValueError`` unless the ``total`` / ``max_count`` given at construction equal the device's counts
        (``total``) or bound them from above (``max_count``).  Copies two integers to the host."""
        if not self._hinted:
            return
        B = self.shape[0]
        if B == 0:
            true_total, true_max = 0, 0
        else:
            per_row = self.offsets[1:] - self.offsets[:-1]
            true_total, true_max = (int(v) for v in torch.stack([self.offsets[-1], per_row.max()]).tolist())
        total, max_count = self._host
        if total != true_total or max_count < true_max:
            raise ValueError(f"CompactRows hints total={total}, max_count={max_count} do not fit the mask: it has "
                             f"{true_total} set entries, at most {true_max} in one row")

    @property
    def total(self) -> torch.Tensor:
        """Number of valid entries, as a one-element int32 device tensor."""
        return self.offsets[-1:]

    def _host_counts(self) -> tuple[int, int]:
        if getattr(self, "_host", None) is None:
            B = self.shape[0]
            if B == 0:
                self._host = (0, 0)
            else:
                per_row = self.offsets[1:] - self.offsets[:-1]
                both = torch.stack([self.offsets[-1], per_row.max()]).tolist()  # one device-to-host copy
                self._host = (int(both[0]), int(both[1]))
        return self._host

    def total_host(self) -> int:
        """Number of valid entries as a Python int (one device-to-host copy, cached): what torch ops
        over exactly the listed rows need to size their tensors."""
        return self._host_counts()[0]

    def max_count_host(self) -> int:
        """Largest number of entries in one row of the mask, as a Python int (same copy, cached)."""
        return self._host_counts()[1]


def norm_linear(
    x: torch.Tensor,
    norm_weight: torch.Tensor,
    weight_packed: torch.Tensor,
    bias: torch.Tensor | None = None,
    *,
    eps: float | None = None,
    rows: CompactRows | None = None,
) -> torch.Tensor:
    """``linear(rmsnorm(x) * norm_weight)`` in one matrix-core kernel with bfloat16 projection.

    x (..., 128) float32 with contiguous rows; ``weight_packed`` from ``pack_linear_weights``
    (N features).  With ``rows`` only the listed rows of the flattened x are projected, into
    the leading ``rows.total`` rows of a (capacity, N) result in list order; the remaining
    rows of the result are left unwritten.  Returns bfloat16 (..., N), or (capacity, N) with ``rows``.
    """
    D = x.shape[-1]
    if not (x.is_cuda and x.dtype == torch.float32 and D == FFN_WIDTH):
        raise RuntimeError("norm_linear covers float32 (..., 128) inputs on the GPU")
    if torch.is_grad_enabled() and x.requires_grad:
        raise RuntimeError("norm_linear is forward-only; call it under torch.no_grad()")
    if weight_packed.dtype != torch.bfloat16 or weight_packed.dim() != 4 or not weight_packed.is_contiguous():
        raise ValueError("weight_packed must come from pack_linear_weights")
    N = weight_packed.shape[0] * 32
    if norm_weight.shape != (D,) or norm_weight.dtype != torch.float32:
        raise ValueError(f"norm_weight must be a float32 {(D,)} tensor")
    x2 = x.reshape(-1, D)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    R = x2.shape[0]
    if rows is not None and rows.shape[0] * rows.shape[1] != R:
        raise ValueError("rows was built for a mask of a different size")
    bias_ptr = None
    if bias is not None:
        if bias.shape != (N,):
            raise ValueError(f"bias must have {N} entries")
        bias = bias.detach().float().contiguous()
        bias_ptr = bias.data_ptr()
    out = torch.empty((R, N), dtype=torch.bfloat16, device=x.device)
    norm_weight = norm_weight.detach().contiguous()
    if R:
        with _on_device(x.device):
            rc = _native.load().bnb_norm_linear_fwd(
                x2.data_ptr(), x2.stride(0), None if rows is None else rows.index.data_ptr(),
                None if rows is None else rows.total.data_ptr(), norm_weight.data_ptr(),
                float(_F32_EPS if eps is None else eps), weight_packed.data_ptr(), bias_ptr, out.data_ptr(), R, D, N,
                _stream(),
            )
        _native.check(rc, "bnb_norm_linear_fwd")
    return out if rows is not None else out.reshape(*x.shape[:-1], N)


def sdpa_cross_rows(
    qkv: torch.Tensor,
    kv_rows: torch.Tensor,
    rows: CompactRows,
    n_heads: int,
    *,
    accum: torch.Tensor | None = None,
    total: int | None = None,
    lse: torch.Tensor | None = None,
) -> torch.Tensor:
    """``sdpa_cross`` over key/value rows compacted beforehand: ``kv_rows`` (capacity, 2*D)
    holds ``[K | V]`` of the entries listed in ``rows`` (e.g. ``norm_linear(bullets, ..., rows=rows)``),
    environment b reading the rows ``rows.offsets[b] .. rows.offsets[b+1]-1``.  Same result as
    ``sdpa_cross`` with the mask the list was built from, without scanning the mask again.

    ``lse``: optional contiguous float32 (B, n_heads, NQ) tensor that receives the base-2 log-sum-exp of every
    query's scaled scores, which ``sdpa_cross_stream_bwd`` takes instead of recomputing it."""
    B, NQ, D3 = qkv.shape
    D = D3 // 3
    if not (qkv.is_cuda and qkv.dtype == torch.bfloat16 and kv_rows.dtype == torch.bfloat16 and D % n_heads == 0
            and D // n_heads == 32 and NQ <= 160):
        raise RuntimeError("sdpa_cross_rows covers bfloat16, head size 32 and at most 160 queries")
    if kv_rows.dim() != 2 or kv_rows.shape[1] != 2 * D or kv_rows.stride(1) != 1 or kv_rows.stride(0) % 8:
        raise ValueError(f"kv_rows must be a (capacity, {2 * D}) tensor with unit column stride (a column block of a wider one is fine)")
    need = rows.shape[0] * rows.shape[1] if total is None else total  # without the host-side count: room for every entry
    if rows.shape[0] != B or kv_rows.shape[0] < need:
        raise ValueError("rows was built for a different batch, or kv_rows is smaller than its capacity")
    if torch.is_grad_enabled() and (qkv.requires_grad or kv_rows.requires_grad):
        raise RuntimeError("sdpa_cross_rows is forward-only; call it under torch.no_grad()")
    if B and NQ and (qkv.stride(-1) != 1 or (B > 1 and qkv.stride(0) != NQ * qkv.stride(1))):
        qkv = qkv.contiguous()
    if accum is not None and (accum.shape != (B, NQ, D) or accum.dtype != torch.bfloat16 or not accum.is_contiguous()):
        raise ValueError("accum must be a contiguous bfloat16 (B, NQ, D) tensor")
    if lse is not None and (lse.shape != (B, n_heads, NQ) or lse.dtype != torch.float32 or not lse.is_contiguous()
                            or lse.device != qkv.device):
        raise ValueError(f"lse must be a contiguous float32 {(B, n_heads, NQ)} tensor on the queries' device")
    out = accum if accum is not None else torch.empty((B, NQ, D), dtype=torch.bfloat16, device=qkv.device)
    if B == 0 or NQ == 0:
        return out
    if kv_rows.shape[0] == 0:  # an empty list: every environment reads nothing
        return out if accum is not None else out.zero_()
    lib = _native.load()
    with _on_device(qkv.device):
        if lse is None:
            rc = lib.bnb_sdpa_cross_ranges_fwd(
                qkv.data_ptr(), qkv.stride(1), NQ, kv_rows.data_ptr(), kv_rows.stride(0), rows.offsets.data_ptr(),
                kv_rows.shape[0], None if accum is None else accum.data_ptr(), out.data_ptr(), B, n_heads, D // n_heads,
                _native.BF16, _stream(),
            )
        else:
            rc = lib.bnb_sdpa_cross_ranges_fwd_lse(
                qkv.data_ptr(), qkv.stride(1), NQ, kv_rows.data_ptr(), kv_rows.stride(0), rows.offsets.data_ptr(),
                kv_rows.shape[0], None if accum is None else accum.data_ptr(), out.data_ptr(), lse.data_ptr(), B, n_heads,
                D // n_heads, _native.BF16, _stream(),
            )
    _native.check(rc, "bnb_sdpa_cross_ranges_fwd")
    return out
