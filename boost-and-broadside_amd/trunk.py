"""Drop-in trunk layers for the Yemong policy, running on the gfx950 kernels.

Every class keeps the constructor arguments, method signatures, tensor layouts and
``state_dict`` keys of the layer it replaces, so a reference checkpoint loads with
``load_state_dict`` and a reference policy can swap its ``yemong_layers`` for these:

    TransformerBlock        models/yemong/attention.py:40-169
    GatedMLP                models/yemong/attention.py:21-37
    RGLRU                   models/yemong/griffin.py:143-219
    GriffinTemporalBlock    models/yemong/griffin.py:222-317
    YemongBlock             models/yemong/griffin.py:320-472
    TeamPMA                 models/yemong/policy.py:78-120
    ModelConfig             config/core.py:213-275
    YemongTrunk             the block loop and hidden-state handling of
                            models/yemong/policy.py:234-254, 268-285, 311-354

What runs where.  Without gradients (rollout, evaluation) every sublayer runs on the HIP
kernels in ``ops``: attention core, recurrence, conv taps with the buffer shift, and under
bfloat16 autocast at width 128 also the norms, projections and the gated MLP (fused kernels).
``YemongTrunk.forward`` steps the packed hidden tensor in place of the reference's unpack /
``cat`` / re-pack and can fold the done-environment reset into the same kernels.  With
gradients enabled (the PPO update) the same layers run on forward + backward kernels behind
``torch.autograd.Function``s, with the forward and input-gradient GEMMs on the library.
The layers refuse to run off-GPU.

Shapes outside what the kernels cover run the same mathematics through torch's library on the
device.  Every such dispatch is counted in ``library_dispatches`` and warned about once per
site (``LibraryDispatchWarning``); ``forbid_library_dispatch()`` turns them into errors.

Derived weights (bfloat16 copies, concatenations, matrix-core operand packings) are cached per
layer and rebuilt when a source parameter's version counter, address or device changes, when
the module is moved / cast (``.to()``), on ``load_state_dict`` and on ``train()`` / ``eval()``.
A write through ``param.data`` (``avg_parameter.data.copy_(...)``, train/rl/opponents.py:107-112)
leaves the version counter alone, so the layers hold their parameters as ``WatchedParameter``s:
every access to ``.data`` counts as a possible write and the caches that depend on that parameter
are rebuilt by the next forward.  No call by the trainer is needed.  What still escapes is a write
through an alias taken earlier and kept (``alias = p.data`` once, ``alias.copy_(...)`` many times):
``invalidate_weight_caches(module)`` covers that, and ``verify_weight_caches(module)`` finds it.
"""

from __future__ import annotations

import collections
import contextlib
import warnings
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F
import torch.utils.checkpoint

from . import _native, ops

CONV_KERNEL = 4  # taps of the causal depthwise conv; the state keeps the last CONV_KERNEL-1 inputs

_FUSED_WIDTHS = (8, 16, 32, 64, 128, 256, 512)  # d_model values the fused norm kernel covers
_WGRAD_MIN_ROWS = 8192  # below this many rows the library's weight-gradient GEMM is as fast as ops.linear_wgrad


def _projection_dtype() -> torch.dtype:
    """dtype a Linear computes in right now: the autocast dtype if autocast is on, else float32."""
    if torch.is_autocast_enabled("cuda"):
        return torch.get_autocast_dtype("cuda")
    return torch.float32


def _widen_tokens(x: torch.Tensor) -> tuple[torch.Tensor, bool]:
    """``(tokens for the kernels, whether they were widened)``.

    Under bfloat16 autocast the reference's encoder ends in ``Linear -> RMSNorm`` (models/yemong/encoder.py:82-101),
    which hands the trunk bfloat16 tokens, and its residual stream then stays bfloat16.  The kernels carry the
    residual stream in float32 (every sublayer adds its bfloat16 output onto float32 rows), so such tokens are
    widened once on entry and the result is rounded back to bfloat16 once on exit: the same function with fewer
    roundings in between, instead of torch's library composition for a bfloat16 stream."""
    if x.dtype == torch.bfloat16 and x.is_cuda and _projection_dtype() == torch.bfloat16:
        return x.float(), True
    return x, False


def _fused_ok(x: torch.Tensor, act: torch.dtype) -> bool:
    """Whether the fused norm / gelu kernels apply: fp32 residual stream on the GPU, a covered
    width, fp32 or bf16 projections.  Anything else takes the plain torch composition."""
    if torch.is_grad_enabled():
        return False
    ok = x.is_cuda and x.dtype == torch.float32 and x.shape[-1] in _FUSED_WIDTHS and act in (torch.float32, torch.bfloat16)
    if not ok and x.is_cuda:
        _note_library("norm_and_gate_kernels", f"rows {x.dtype} of width {x.shape[-1]}, projections in {act}")
    return ok


def _f32_fused_ok(x: torch.Tensor, act: torch.dtype, *layers: nn.Linear) -> bool:
    """Whether the float32 matrix-core Linear kernel applies: no gradients, float32 projections over float32 rows
    of width 128 on the GPU, float32 weights."""
    return (
        not torch.is_grad_enabled() and act == torch.float32 and x.is_cuda and x.dtype == torch.float32
        and x.shape[-1] == ops.FFN_WIDTH and all(l.weight.dtype == torch.float32 for l in layers)
    )


def _packed_f32(layer: nn.Module, slot: str, *weights: torch.Tensor) -> torch.Tensor:
    """The float32 operand stream of ``ops.linear_f32`` for one weight, or for a (gate, up) pair (cached)."""
    return _cached_cast(layer, slot, weights, torch.float32, lambda: ops.pack_linear_f32(*weights))


_HEAD_FUSION = True  # the sublayer tail also forms the next sublayer's norm + projection (bf16 inference, width 128)


@contextlib.contextmanager
def separate_heads():
    """Inside the block every sublayer forms its own norm + projection (one more launch per sublayer) instead of
    receiving it from the tail kernel of the sublayer before.  For comparisons."""
    global _HEAD_FUSION
    keep, _HEAD_FUSION = _HEAD_FUSION, False
    try:
        yield
    finally:
        _HEAD_FUSION = keep


_TRAIN_KERNELS = True  # grad-mode norms, gates, conv, attention and weight gradients on the library's own kernels when False


@contextlib.contextmanager
def library_update_path():
    """Inside the block the grad-mode path uses torch's own differentiable ops only (norms, gelu gates,
    conv taps, attention, weight-gradient GEMMs); the recurrence keeps its kernels.  For comparisons."""
    global _TRAIN_KERNELS
    keep, _TRAIN_KERNELS = _TRAIN_KERNELS, False
    try:
        yield
    finally:
        _TRAIN_KERNELS = keep


class LibraryDispatchWarning(UserWarning):
    """A shape outside what the kernels cover ran through torch's library on the device."""


library_dispatches: collections.Counter = collections.Counter()  # site -> calls that took the library path
_FORBID_LIBRARY = False


def _note_library(site: str, why: str) -> None:
    """Record that ``site`` runs on torch's library for this call (counter + one warning per site)."""
    if _FORBID_LIBRARY:
        raise RuntimeError(f"library dispatch at {site} ({why}) inside forbid_library_dispatch()")
    if not library_dispatches[site]:
        warnings.warn(f"{site}: {why}; running torch's library on the device instead of the gfx950 kernels",
                      LibraryDispatchWarning, stacklevel=3)
    library_dispatches[site] += 1


@contextlib.contextmanager
def forbid_library_dispatch():
    """Inside the block a call that would leave the kernels for torch's library raises instead."""
    global _FORBID_LIBRARY
    keep, _FORBID_LIBRARY = _FORBID_LIBRARY, True
    try:
        yield
    finally:
        _FORBID_LIBRARY = keep


_CACHE_PREFIX = "_bnb_"


class _DerivedWeight:
    """One cached tensor derived from parameters: the value, how to rebuild it, what it depends on."""

    __slots__ = ("key", "value", "build", "tensors", "dtype")

    def __init__(self, key, value, build, tensors, dtype):
        self.key, self.value, self.build, self.tensors, self.dtype = key, value, build, tensors, dtype

    def refresh(self) -> None:
        """Rebuild from the source tensors into the same memory (addresses stay valid)."""
        with torch.no_grad():
            _copy_into(self.value, self.build())
        self.key = _cache_key(self.tensors, self.dtype)


def _same_layout(a, b) -> bool:
    if isinstance(a, tuple) or isinstance(b, tuple):
        return (isinstance(a, tuple) and isinstance(b, tuple) and len(a) == len(b)
                and all(_same_layout(x, y) for x, y in zip(a, b)))
    return a.shape == b.shape and a.dtype == b.dtype and a.device == b.device


def _copy_into(dst, src) -> None:
    if isinstance(dst, tuple):
        for d, s in zip(dst, src):
            d.copy_(s)
    else:
        dst.copy_(src)


def _cache_key(tensors: tuple, dtype: torch.dtype):
    return (dtype,) + tuple((t._version, t.data_ptr(), t.device, getattr(t, "_bnb_touch", 0)) for t in tensors)


class WatchedParameter(nn.Parameter):
    """An ``nn.Parameter`` that counts accesses to ``.data``.

    ``p.data`` hands out an alias with a version counter of its own, so ``p.data.copy_(w)`` changes the weights
    without changing ``p._version``, and a cache keyed on the version would keep serving the old weights.  Here
    the ``.data`` attribute itself is the signal: reading or assigning it bumps ``_bnb_touch``, which is part
    of every derived weight's key.  A read that wrote nothing costs one rebuild of the copies derived from
    that parameter; optimizers and ``load_state_dict`` write under ``no_grad`` and do not come this way.
    Everything else (autograd, ``state_dict``, ``deepcopy``, ``.to()``) behaves as for ``nn.Parameter``."""

    __torch_function__ = torch._C._disabled_torch_function_impl

    def __new__(cls, data=None, requires_grad=True):
        if data is None:
            data = torch.empty(0)
        out = torch.Tensor._make_subclass(cls, data, requires_grad)
        out._bnb_touch = 0
        return out

    @property
    def data(self):
        self._bnb_touch = getattr(self, "_bnb_touch", 0) + 1
        return torch._C.TensorBase.data.__get__(self)

    @data.setter
    def data(self, value):
        self._bnb_touch = getattr(self, "_bnb_touch", 0) + 1
        torch._C.TensorBase.data.__set__(self, value)


def watch_parameters(module: nn.Module) -> None:
    """Replace every plain ``nn.Parameter`` below ``module`` by a ``WatchedParameter`` over the same memory."""
    for m in module.modules():
        for name, p in m._parameters.items():
            if p is not None and type(p) is nn.Parameter:
                watched = WatchedParameter(torch._C.TensorBase.data.__get__(p), p.requires_grad)
                if p.grad is not None:
                    watched.grad = p.grad
                m._parameters[name] = watched


def _cached_cast(owner: nn.Module, slot: str, tensors: tuple, dtype: torch.dtype, build):
    """``build()`` (a tensor derived from ``tensors`` in ``dtype``) cached on ``owner`` until one of the
    source tensors is modified in place, replaced or moved, or the cache is invalidated.  A rebuild
    of the same shape is written into the existing memory, so an address captured into a HIP graph
    stays valid.  Saves the per-step weight casts autocast would otherwise repeat."""
    key = _cache_key(tensors, dtype)
    hit = owner.__dict__.get(slot)
    if hit is not None and hit.key == key:
        return hit.value
    with torch.no_grad():
        value = build()
    if hit is not None and _same_layout(hit.value, value):
        _copy_into(hit.value, value)
        hit.key, hit.build, hit.tensors, hit.dtype = key, build, tensors, dtype
    else:
        hit = _DerivedWeight(key, value, build, tensors, dtype)
        owner.__dict__[slot] = hit
    return hit.value


def derived_weights(module: nn.Module) -> list:
    """Every cached derived-weight entry below ``module``."""
    return [v for m in module.modules() for k, v in m.__dict__.items()
            if k.startswith(_CACHE_PREFIX) and isinstance(v, _DerivedWeight)]


def invalidate_weight_caches(module: nn.Module, *, drop: bool = False) -> None:
    """Mark every cached derived weight below ``module`` stale, so the next forward rebuilds it.

    Only needed after a write the caches cannot see: one through an alias of the weights that was taken
    earlier and kept (``alias = p.data`` once, then ``alias.copy_(...)``), or through a view of the storage made
    outside autograd.  ``p.data.copy_(...)`` itself is seen (``WatchedParameter``).  ``drop=True`` frees the
    cached tensors instead of keeping their memory for the rebuild."""
    for m in module.modules():
        for k in [k for k, v in m.__dict__.items() if k.startswith(_CACHE_PREFIX) and isinstance(v, _DerivedWeight)]:
            if drop:
                del m.__dict__[k]
            else:
                m.__dict__[k].key = None


def verify_weight_caches(module: nn.Module) -> list[str]:
    """Names (``module path:slot``) of cached derived weights that no longer equal a fresh build from their
    sources although their key says they are current.  Compares on the device and copies one flag per entry
    to the host: a debugging aid for a trainer suspected of writing weights where the caches cannot see it."""
    stale = []
    for name, m in module.named_modules():
        for slot, entry in m.__dict__.items():
            if not (slot.startswith(_CACHE_PREFIX) and isinstance(entry, _DerivedWeight)):
                continue
            if entry.key != _cache_key(entry.tensors, entry.dtype):
                continue  # known to be stale: the next forward rebuilds it
            with torch.no_grad():
                fresh = entry.build()
            have = entry.value if isinstance(entry.value, tuple) else (entry.value,)
            want = fresh if isinstance(fresh, tuple) else (fresh,)
            if not all(torch.equal(a, b) for a, b in zip(have, want)):
                stale.append(f"{name}:{slot}")
    return stale


class _WeightCaches:
    """Mixin of the layers: keeps the derived-weight caches in step with what ``nn.Module`` does to
    the parameters behind the caches' back (moves and casts, state-dict loads, mode switches), and
    keeps the parameters below the layer ``WatchedParameter``s, so writes through ``.data`` are seen."""

    def invalidate_weight_caches(self, *, drop: bool = False) -> None:
        invalidate_weight_caches(self, drop=drop)

    def __setattr__(self, name, value):
        super().__setattr__(name, value)
        if isinstance(value, nn.Module):
            watch_parameters(value)
        elif type(value) is nn.Parameter:
            watch_parameters(self)

    def __setstate__(self, state):
        super().__setstate__(state)
        watch_parameters(self)  # unpickling rebuilds plain Parameters

    def _apply(self, fn, *args, **kwargs):
        out = super()._apply(fn, *args, **kwargs)
        watch_parameters(self)
        invalidate_weight_caches(self, drop=True)  # device or dtype may have changed
        return out

    def load_state_dict(self, *args, **kwargs):
        out = super().load_state_dict(*args, **kwargs)
        watch_parameters(self)  # assign=True swaps the Parameter objects
        invalidate_weight_caches(self)
        return out

    def train(self, mode: bool = True):
        out = super().train(mode)
        invalidate_weight_caches(self)
        return out


def _grad_linear(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None) -> torch.Tensor:
    """``F.linear`` in grad mode: under bf16 autocast with enough rows the weight gradient runs on the
    row-sliced kernel (``ops.linear_train``), otherwise autocast's own differentiable casts apply."""
    if (
        _TRAIN_KERNELS and w.requires_grad and w.dtype == torch.float32 and _projection_dtype() == torch.bfloat16
        and x.numel() >= _WGRAD_MIN_ROWS * x.shape[-1] and ops.linear_wgrad_supported(x, w)
    ):
        return ops.linear_train(x, w, b)
    return F.linear(x, w, b)


def _project(layer: nn.Linear, x: torch.Tensor) -> torch.Tensor:
    """``layer(x)`` for an activation that already has the projection dtype."""
    w, b = layer.weight, layer.bias
    if torch.is_grad_enabled():
        return _grad_linear(x, w, b)
    if x.dtype == w.dtype:
        return F.linear(x, w, b)
    dt = x.dtype  # the builders must not keep the activation alive
    wc = _cached_cast(layer, "_bnb_w", (w,), dt, lambda: w.detach().to(dt))
    bc = None if b is None else _cached_cast(layer, "_bnb_b", (b,), dt, lambda: b.detach().to(dt))
    return F.linear(x, wc, bc)


def _gelu_gate(gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """``gelu(gate) * value`` in grad mode: one kernel forward and one backward on the GPU (the product
    rounded once to the projection dtype, which is what the next Linear would cast it to), torch ops elsewhere."""
    act = _projection_dtype()
    if _TRAIN_KERNELS and ops.gelu_mul_train_supported(gate, value) and act in (torch.float32, torch.bfloat16):
        out_dtype = act if act == torch.bfloat16 else torch.promote_types(gate.dtype, value.dtype)
        return ops.gelu_mul_train(gate, value, out_dtype=out_dtype)
    return F.gelu(gate) * value


def _norm_linear_train_ok(x: torch.Tensor, act: torch.dtype, norm: nn.RMSNorm, layer: nn.Linear) -> bool:
    """Whether ``layer(norm(x))`` of the update runs as one forward kernel (``ops.norm_linear_train``)."""
    return (
        _TRAIN_KERNELS and torch.is_grad_enabled() and act == torch.bfloat16 and layer.bias is None
        and norm.weight is not None and norm.weight.dtype == torch.float32 and layer.weight.requires_grad
        and x.numel() >= _WGRAD_MIN_ROWS * x.shape[-1] and ops.norm_linear_train_supported(x, layer.weight)
    )


def _norm_linear_train(x: torch.Tensor, norm: nn.RMSNorm, layer: nn.Linear):
    """``(x, layer(norm(x)), norm(x))`` through ``ops.norm_linear_train``; use the returned x for the residual."""
    w = layer.weight
    pk = _cached_cast(layer, "_bnb_pack", (w,), torch.bfloat16, lambda: ops.pack_linear_weights(w))
    return ops.norm_linear_train(x, norm.weight, w, eps=norm.eps, packed=pk)


def _train_norm(norm: nn.RMSNorm, x: torch.Tensor, delta: torch.Tensor | None = None):
    """``(s, norm(s))`` with ``s = x + delta`` (``s`` = x without ``delta``), differentiable.  Use the
    returned ``s`` for the residual connection.

    On the GPU with float32 rows of a covered width the norm's output is rounded once to the
    projection dtype, forward and backward are one kernel each and the backward adds the residual
    branch's gradient in the same pass (``ops.rmsnorm_train``); anything else is the module itself."""
    act = _projection_dtype()
    if (
        _TRAIN_KERNELS and torch.is_grad_enabled() and act in (torch.float32, torch.bfloat16) and ops.rmsnorm_train_supported(x)
        and norm.weight is not None and norm.weight.dtype == torch.float32
        and (delta is None or (delta.shape == x.shape and delta.dtype in (torch.float32, torch.bfloat16)))
    ):
        return ops.rmsnorm_train(x, norm.weight, delta=delta, eps=norm.eps, out_dtype=act)
    if _TRAIN_KERNELS and torch.is_grad_enabled() and x.is_cuda:
        _note_library("rmsnorm_backward", f"rows {x.dtype} of width {x.shape[-1]}, projections in {act}")
    s = x if delta is None else x + delta
    return s, norm(s)


@dataclass(frozen=True)
class ModelConfig:
    """Trunk architecture; field names and checks follow config/core.py:213-275."""

    d_model: int
    n_heads: int
    n_yemong_blocks: int
    n_spatial_per_block: int = 1
    n_temporal_per_block: int = 1
    encoder_split: bool = False
    n_bullet_cross_per_block: int = 0
    bullet_encoder_hidden: int = 64
    grad_checkpoint: bool = False

    @property
    def n_hidden_layers(self) -> int:
        return self.n_yemong_blocks * self.n_temporal_per_block

    @property
    def reads_bullets(self) -> bool:
        return self.n_bullet_cross_per_block > 0 and self.n_yemong_blocks > 0

    def __post_init__(self) -> None:
        if self.d_model % self.n_heads:
            raise ValueError(f"d_model={self.d_model} must be divisible by n_heads={self.n_heads}")
        for name in ("n_yemong_blocks", "n_spatial_per_block", "n_temporal_per_block"):
            if getattr(self, name) < 0:
                raise ValueError(f"{name} must be >= 0, got {getattr(self, name)}")
        if not 0 <= self.n_bullet_cross_per_block <= self.n_spatial_per_block:
            raise ValueError(
                f"n_bullet_cross_per_block must lie in [0, {self.n_spatial_per_block}], "
                f"got {self.n_bullet_cross_per_block}"
            )


class GatedMLP(_WeightCaches, nn.Module):
    """``down_proj(gelu(gate_proj(x)) * up_proj(x))`` with a 4x hidden width by default."""

    def __init__(self, d_model: int, expand: int = 4) -> None:
        super().__init__()
        self.gate_proj = nn.Linear(d_model, expand * d_model, bias=False)
        self.up_proj = nn.Linear(d_model, expand * d_model, bias=False)
        self.down_proj = nn.Linear(expand * d_model, d_model, bias=False)

    def packed_weights(self) -> torch.Tensor:
        """The three weight matrices as the fused sublayer-tail kernel's bf16 operand stream (cached)."""
        ws = (self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight)
        return _cached_cast(self, "_bnb_ffn_pack", ws, torch.bfloat16, lambda: ops.pack_ffn_weights(*ws))

    def fused_tail_ok(self, x: torch.Tensor) -> bool:
        """Whether the one-kernel sublayer tail applies (bf16-autocast inference, width 128, hidden 512)."""
        return (
            not torch.is_grad_enabled() and _projection_dtype() == torch.bfloat16
            and ops.ffn_supported(x, self.gate_proj.out_features)
        )

    def fused_tail(self, x, delta, norm: nn.RMSNorm, *, proj_layer: nn.Linear | None = None, gate=None, next_head=None):
        """``s = x + d; s + self(norm(s))`` as one kernel, or None when it does not apply.

        ``d`` is ``delta`` itself, or with ``proj_layer`` (a bias-free 128 x 128 Linear)
        ``proj_layer(delta)``, or with ``gate`` as well ``proj_layer(gelu(gate) * delta)``,
        the projection then running inside the kernel.  With ``next_head`` (``head_spec`` of the sublayer that
        follows) and a folded projection the same launch also forms that sublayer's norm + projection, and the
        result is the pair ``(out, head)``."""
        if not self.fused_tail_ok(x) or (delta is not None and delta.dtype != torch.bfloat16):
            return None
        if proj_layer is None:
            return ops.ffn_fused(x, delta, norm.weight, self.packed_weights(), eps=norm.eps)
        w = proj_layer.weight
        if proj_layer.bias is not None or tuple(w.shape) != (ops.FFN_WIDTH, ops.FFN_WIDTH):
            return None
        if gate is not None and gate.dtype != torch.bfloat16:
            return None
        wp = _cached_cast(proj_layer, "_bnb_proj_pack", (w,), torch.bfloat16, lambda: ops.pack_proj_weights(w))
        proj = (delta, wp) if gate is None else (gate, delta, wp)
        return ops.ffn_fused(x, None, norm.weight, self.packed_weights(), eps=norm.eps, proj=proj, next_head=next_head)

    def train_tail(self, x: torch.Tensor, delta: torch.Tensor | None, norm: nn.RMSNorm, *,
                   proj_layer: nn.Linear | None = None) -> torch.Tensor | None:
        """``s = x + delta; s + self(norm(s))`` in grad mode under bfloat16 autocast as one kernel forward and one
        matrix-core kernel backward that recomputes the 512/1024-wide activations instead of saving them
        (plus the weight-gradient and norm-backward kernels); None when that does not apply.  With ``proj_layer``
        (a bias-free 128 x 128 Linear with float32 weights) ``s = x + proj_layer(delta)``, the projection inside the kernel."""
        ws = (self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight)
        if proj_layer is not None and (proj_layer.bias is not None or proj_layer.weight.dtype != torch.float32
                                       or tuple(proj_layer.weight.shape) != (ops.FFN_WIDTH, ops.FFN_WIDTH)):
            return None
        if not (
            _TRAIN_KERNELS and torch.is_grad_enabled() and _projection_dtype() == torch.bfloat16
            and ops.ffn_tail_train_supported(x, delta, self.gate_proj.out_features)
            and self.gate_proj.bias is None and self.up_proj.bias is None and self.down_proj.bias is None
            and norm.weight is not None and norm.weight.dtype == torch.float32 and all(w.dtype == torch.float32 for w in ws)
        ):
            return None
        packed_bwd = _cached_cast(self, "_bnb_ffn_bwd_pack", ws, torch.bfloat16, lambda: ops.pack_ffn_bwd_weights(*ws))
        if proj_layer is None:
            return ops.ffn_tail_train(x, delta, norm.weight, *ws, eps=norm.eps, packed_fwd=self.packed_weights(),
                                      packed_bwd=packed_bwd)
        w = proj_layer.weight
        wp = _cached_cast(proj_layer, "_bnb_proj_pack", (w,), torch.bfloat16, lambda: ops.pack_proj_weights(w))
        return ops.ffn_tail_train(x, delta, norm.weight, *ws, eps=norm.eps, packed_fwd=self.packed_weights(),
                                  packed_bwd=packed_bwd, proj_weight=w, proj_packed=wp)

    def tail_f32(self, x1: torch.Tensor, norm: nn.RMSNorm) -> torch.Tensor | None:
        """``x1 + self(norm(x1))`` in float32 as two kernels (norm + gate/up + gelu gate; down + residual), or None
        when that does not apply (other widths, biases)."""
        if (self.gate_proj.bias is not None or self.up_proj.bias is not None or self.down_proj.bias is not None
                or self.gate_proj.out_features % 128 or norm.weight is None
                or not _f32_fused_ok(x1, torch.float32, self.gate_proj, self.up_proj, self.down_proj)):
            return None
        gu = _packed_f32(self, "_bnb_f32_gate_up", self.gate_proj.weight, self.up_proj.weight)
        hid = ops.linear_f32(x1, gu, norm_weight=norm.weight, eps=norm.eps, gate=True)
        return ops.linear_f32(hid, _packed_f32(self.down_proj, "_bnb_f32_pack", self.down_proj.weight), resid=x1)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        hidden = self.gate_proj.out_features
        if not x.is_cuda or hidden % 8 or x.dtype not in (torch.float32, torch.bfloat16) or torch.is_grad_enabled():
            if (
                _TRAIN_KERNELS and torch.is_grad_enabled() and x.is_cuda and hidden % 8 == 0 and self.gate_proj.bias is None
                and self.up_proj.bias is None and _projection_dtype() == torch.bfloat16
            ):
                # one projection over [gate | up] (one pass over x forward, one GEMM for its gradient backward),
                # the gate product on its column blocks
                gu = _grad_linear(x, torch.cat([self.gate_proj.weight, self.up_proj.weight], dim=0), None)
                return _project(self.down_proj, ops.gelu_mul_packed_train(gu, out_dtype=torch.bfloat16))
            return _project(self.down_proj, _gelu_gate(_project(self.gate_proj, x), _project(self.up_proj, x)))
        # one GEMM for [gate | up], one kernel for gelu(gate) * up, one GEMM down
        wg, wu = self.gate_proj.weight, self.up_proj.weight
        dt = x.dtype
        w = _cached_cast(self, "_bnb_gate_up", (wg, wu), dt, lambda: torch.cat([wg, wu], dim=0).detach().to(dt))
        gu = F.linear(x, w)
        return _project(self.down_proj, ops.gelu_mul(gu[..., :hidden], gu[..., hidden:], out_dtype=x.dtype))


class TransformerBlock(_WeightCaches, nn.Module):
    """Pre-norm attention + FFN over the entity tokens of each environment.

    ``forward(x (B,N,D), alive_mask (B,N) bool | None, bullets, bullet_mask) -> (B,N,D)``.
    """

    def __init__(self, model_config: ModelConfig, reads_bullets: bool = False) -> None:
        super().__init__()
        D = model_config.d_model
        self.d_model = D
        self.n_heads = model_config.n_heads
        self.head_dim = D // model_config.n_heads
        self.reads_bullets = reads_bullets
        self.norm1 = nn.RMSNorm(D)
        self.qkv = nn.Linear(D, 3 * D, bias=False)
        self.out_proj = nn.Linear(D, D, bias=False)
        if reads_bullets:
            self.norm_bullet = nn.RMSNorm(D)
            self.kv_bullet = nn.Linear(D, 2 * D, bias=False)
        self.norm2 = nn.RMSNorm(D)
        self.ffn = GatedMLP(D)

    def head_spec(self, x: torch.Tensor):
        """``(norm weight, eps, packed weight, features)`` of this sublayer's head ``qkv(norm1(x))`` for the tail
        kernel of the sublayer before (``ops.ffn_fused(next_head=...)``), or None when this sublayer would not take
        the bfloat16 kernel path for rows like ``x``."""
        if not (_HEAD_FUSION and not torch.is_grad_enabled() and _projection_dtype() == torch.bfloat16 and x.is_cuda
                and x.dtype == torch.float32 and self.d_model == ops.FFN_WIDTH and self.qkv.bias is None
                and self.norm1.weight is not None and self.norm1.weight.dtype == torch.float32):
            return None
        w = self.qkv.weight
        hp = _cached_cast(self.qkv, "_bnb_head_pack", (w,), torch.bfloat16, lambda: ops.pack_head_weights(w))
        return (self.norm1.weight, self.norm1.eps, hp, 3 * self.d_model)

    def forward(self, x, alive_mask=None, bullets=None, bullet_mask=None, *, head=None, next_head=None):
        """``head``: this sublayer's ``qkv(norm1(x))`` when the sublayer before has already formed it;
        ``next_head``: the ``head_spec`` of the sublayer that follows: the result is then the pair
        ``(out, that head or None)``.  Both are internal to the trunk's step."""
        if next_head is not None:
            out = self._forward(x, alive_mask, bullets, bullet_mask, head, next_head)
            return out if isinstance(out, tuple) else (out, None)
        return self._forward(x, alive_mask, bullets, bullet_mask, head, None)

    def _forward(self, x, alive_mask, bullets, bullet_mask, head, next_head):
        act = _projection_dtype()
        if not _fused_ok(x, act):
            qkv = None
            if _norm_linear_train_ok(x, act, self.norm1, self.qkv):
                # the update: norm1 and qkv as one kernel that also leaves the normalised rows for the weight gradient
                x0, qkv, n1 = _norm_linear_train(x, self.norm1, self.qkv)
            else:
                x0, n1 = _train_norm(self.norm1, x)
            if torch.is_grad_enabled():
                # out_proj inside the tail kernel, on the merged heads, when the tail kernel applies
                merged = self._attn(n1, alive_mask, bullets, bullet_mask, qkv=qkv, project=False)
                tail = None
                if merged.dtype == torch.bfloat16:
                    tail = self.ffn.train_tail(x0, merged, self.norm2, proj_layer=self.out_proj)
                if tail is not None:
                    return tail
                attn = _project(self.out_proj, merged)
            else:
                attn = self._attn(n1, alive_mask, bullets, bullet_mask)
            tail = self.ffn.train_tail(x0, attn, self.norm2)
            if tail is not None:
                return tail
            x1, n2 = _train_norm(self.norm2, x0, attn)
            return x1 + self.ffn(n2)
        # norm + qkv (one kernel under bf16) -> attention kernel -> out_proj -> fused sublayer tail
        if act == torch.bfloat16 and self.d_model == ops.FFN_WIDTH and self.qkv.bias is None:
            w = self.qkv.weight
            if head is not None:
                qkv = head  # formed by the tail kernel of the sublayer before
            else:
                pk = _cached_cast(self.qkv, "_bnb_pack", (w,), torch.bfloat16, lambda: ops.pack_linear_weights(w))
                qkv = ops.norm_linear(x, self.norm1.weight, pk, eps=self.norm1.eps)
            if self.ffn.fused_tail_ok(x) and self.out_proj.bias is None:
                # the output projection runs inside the tail kernel, on the merged heads
                merged = self._attn(None, alive_mask, bullets, bullet_mask, qkv=qkv, project=False)
                fused = self.ffn.fused_tail(x, merged, self.norm2, proj_layer=self.out_proj, next_head=next_head)
                if fused is not None:
                    return fused
                attn = _project(self.out_proj, merged)
            else:
                attn = self._attn(None, alive_mask, bullets, bullet_mask, qkv=qkv)
        elif (_f32_fused_ok(x, act, self.qkv, self.out_proj) and self.qkv.bias is None and self.out_proj.bias is None
              and self.norm1.weight is not None):
            # float32 (evaluation without autocast): every Linear on the fp32 matrix cores with its norm, gate and
            # residual folded in: norm1 + qkv, attention, out_proj + residual, norm2 + gate/up + gelu gate, down + residual
            qkv = ops.linear_f32(x, _packed_f32(self.qkv, "_bnb_f32_pack", self.qkv.weight), norm_weight=self.norm1.weight,
                                 eps=self.norm1.eps)
            merged = self._attn(None, alive_mask, bullets, bullet_mask, qkv=qkv, project=False)
            x1 = ops.linear_f32(merged, _packed_f32(self.out_proj, "_bnb_f32_pack", self.out_proj.weight), resid=x)
            tail = self.ffn.tail_f32(x1, self.norm2)
            if tail is not None:
                return tail
            _, n2 = ops.add_rmsnorm(x1, self.norm2.weight, eps=self.norm2.eps, out_dtype=act)
            return x1 + self.ffn(n2)
        else:
            _, n1 = ops.add_rmsnorm(x, self.norm1.weight, eps=self.norm1.eps, out_dtype=act)
            attn = self._attn(n1, alive_mask, bullets, bullet_mask)
        fused = self.ffn.fused_tail(x, attn, self.norm2)
        if fused is not None:
            return fused
        x1, n2 = ops.add_rmsnorm(x, self.norm2.weight, delta=attn, eps=self.norm2.eps, out_dtype=act)
        return x1 + self.ffn(n2)

    def _attn(self, x, alive_mask, bullets=None, bullet_mask=None, qkv=None, project=True):
        """Attention sublayer without the residual; ``project=False`` returns the merged heads
        before ``out_proj``."""
        if qkv is None:
            qkv = _project(self.qkv, x)  # (B, N, 3D), fp32 or bf16 under autocast
        if torch.is_grad_enabled():
            # training: forward and backward kernels for the small token counts of the update,
            # torch's differentiable SDPA for the rest
            if _TRAIN_KERNELS and ops.sdpa_train_supported(qkv, self.n_heads):
                merged = ops.sdpa_train(qkv, alive_mask, self.n_heads)
            else:
                if _TRAIN_KERNELS and qkv.is_cuda:
                    _note_library("TransformerBlock.self_attention_backward",
                                  f"qkv {tuple(qkv.shape)} {qkv.dtype}, {self.n_heads} heads")
                merged = self._self_attention_autograd(qkv, alive_mask)
            if self.reads_bullets and bullets is not None:
                merged = merged + self._bullet_branch_autograd(qkv, bullets, bullet_mask)
            return _project(self.out_proj, merged) if project else merged
        try:
            merged = ops.sdpa_masked(qkv, alive_mask, self.n_heads)  # (B, N, D) head-major
        except _native.NativeLibraryError as err:
            if err.code != _native.ERR_UNSUPPORTED:
                raise
            # a shape the kernels do not cover (head sizes other than 8/16/32/64, more than 512
            # tokens, float32 keys beyond what fits LDS): the library's attention on the device
            _note_library("TransformerBlock.self_attention", f"qkv {tuple(qkv.shape)} {qkv.dtype}, {self.n_heads} heads")
            merged = self._self_attention_autograd(qkv, alive_mask)
        if self.reads_bullets and bullets is not None:
            rows = bullet_mask if isinstance(bullet_mask, ops.CompactRows) else None
            if rows is None and bullet_mask is not None and self._compact_read_ok(qkv, bullets):
                rows = ops.CompactRows(bullet_mask)
            if rows is not None and self._compact_read_ok(qkv, bullets):
                # only the bullets in flight are normalised and projected (one kernel over a
                # device-side list of them), and the read walks each environment's run of rows
                kv_rows = rows.shared_kv.get(id(self)) if rows.shared_kv is not None else None
                if kv_rows is None:
                    w = self.kv_bullet.weight
                    pk = _cached_cast(self.kv_bullet, "_bnb_pack", (w,), torch.bfloat16, lambda: ops.pack_linear_weights(w))
                    kv_rows = ops.norm_linear(bullets, self.norm_bullet.weight, pk, eps=self.norm_bullet.eps, rows=rows)
                merged = ops.sdpa_cross_rows(qkv, kv_rows, rows, self.n_heads, accum=merged)
                return _project(self.out_proj, merged) if project else merged
            if rows is not None:
                bullet_mask = rows.mask
            if (_f32_fused_ok(bullets, qkv.dtype, self.kv_bullet) and self.kv_bullet.bias is None
                    and self.norm_bullet.weight is not None):
                kv = ops.linear_f32(bullets, _packed_f32(self.kv_bullet, "_bnb_f32_pack", self.kv_bullet.weight),
                                    norm_weight=self.norm_bullet.weight, eps=self.norm_bullet.eps)
            else:
                kv = _project(self.kv_bullet, self._norm_bullets(bullets, qkv.dtype))
            if ops.cross_supported(qkv, kv, self.n_heads):
                merged = ops.sdpa_cross(qkv, kv, bullet_mask, self.n_heads, accum=merged)
            else:
                _note_library("TransformerBlock.bullet_read", f"queries {tuple(qkv.shape)} {qkv.dtype}, keys {tuple(kv.shape)}")
                merged = merged + self._bullet_read(qkv, kv, bullet_mask)
        return _project(self.out_proj, merged) if project else merged

    def _compact_read_ok(self, qkv, bullets) -> bool:
        """Whether the bullet read can run on the compacted list (bf16 projections, width 128,
        heads of 32, at most 160 entity tokens, float32 bullet tokens on the GPU)."""
        return (
            qkv.dtype == torch.bfloat16 and self.d_model == ops.FFN_WIDTH and self.head_dim == 32 and qkv.shape[1] <= 160
            and bullets.is_cuda and bullets.dtype == torch.float32 and self.kv_bullet.bias is None
            # the compacted [K | V] rows are addressed with 32-bit element offsets over the full slot capacity
            and bullets.shape[0] * bullets.shape[1] * 2 * self.d_model < 2 ** 32
        )

    def _bullet_branch_autograd(self, qkv, bullets, bullet_mask):
        """The bullet read in grad mode, (B, N, D) to be added to the self-attention output.

        With a mask, bf16 projections and at most 2048 slots per environment only the bullets in
        flight are normalised and projected: the list of live slots is built on the device, its
        length read back once (torch needs it to size the gathered rows), ``norm_bullet`` and
        ``kv_bullet`` run on the gathered rows and the read and its backward take the compacted
        ``[K | V]`` rows with per-environment ranges (a ``CompactRows`` built with ``total=`` /
        ``max_count=`` by a caller that knows the counts needs no read-back).  Otherwise every slot is projected and the
        read is the masked kernel pair, or torch's SDPA for the shapes the kernels do not cover."""
        rows = bullet_mask if isinstance(bullet_mask, ops.CompactRows) else None
        mask = rows.mask if rows is not None else bullet_mask
        B, NB, D = bullets.shape
        compact_ok = (
            _TRAIN_KERNELS and mask is not None and qkv.is_cuda and qkv.dtype == torch.bfloat16 and NB <= 2048
            and self.head_dim == 32 and qkv.shape[1] <= 160 and self.kv_bullet.bias is None and B * NB < 2 ** 31
        )
        if compact_ok:
            if rows is None:
                rows = ops.CompactRows(mask)
            total = rows.total_host()
            if total == 0:
                return torch.zeros_like(qkv[..., :D])
            live = bullets.reshape(B * NB, D).index_select(0, rows.index[:total].long())
            kv_rows = _project(self.kv_bullet, _train_norm(self.norm_bullet, live)[1])
            if kv_rows.dtype == torch.bfloat16:
                return ops.sdpa_cross_rows_train(qkv, kv_rows, rows, self.n_heads)
        kv = _project(self.kv_bullet, _train_norm(self.norm_bullet, bullets)[1])
        if _TRAIN_KERNELS and ops.sdpa_cross_train_supported(qkv, kv, self.n_heads):
            return ops.sdpa_cross_train(qkv, kv, mask, self.n_heads)
        if _TRAIN_KERNELS and qkv.is_cuda:
            _note_library("TransformerBlock.bullet_read_backward", f"queries {tuple(qkv.shape)} {qkv.dtype}, keys {tuple(kv.shape)}")
        return self._bullet_read(qkv, kv, mask)

    def _self_attention_autograd(self, qkv, alive_mask):
        """Masked self-attention as the reference composes it (attention.py:136-147,168)."""
        B, N, _ = qkv.shape
        H, dh, D = self.n_heads, self.head_dim, self.d_model
        q, k, v = (t.reshape(B, N, H, dh).transpose(1, 2) for t in qkv.split(D, dim=-1))
        bias = None
        if alive_mask is not None:
            keep = alive_mask.reshape(B, 1, 1, N).to(q.dtype)
            bias = (1.0 - keep) * (torch.finfo(q.dtype).min / 2)
        o = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, dropout_p=0.0)
        return o.transpose(1, 2).reshape(B, N, D)

    def _norm_bullets(self, bullets, act):
        """norm_bullet(bullets) in the projection dtype."""
        if _fused_ok(bullets, act):
            return ops.add_rmsnorm(bullets, self.norm_bullet.weight, eps=self.norm_bullet.eps, out_dtype=act)[1]
        n = self.norm_bullet(bullets)
        return n if n.dtype == act else n.to(act)

    def _bullet_read(self, qkv, kv, bullet_mask):
        """Cross-attention of the entity queries to bullet key/values (attention.py:149-166) for
        the shapes the matrix-core kernels do not cover (head sizes other than 32, more than 2048
        bullet slots in bf16 or 4096 in fp32): torch's SDPA on the device, with the reference's
        additive bias and its all-inactive gate.  ``kv`` is ``kv_bullet(norm_bullet(bullets))``."""
        B, N, _ = qkv.shape
        H, dh, D = self.n_heads, self.head_dim, self.d_model
        NB = kv.shape[1]
        q = qkv[..., :D].reshape(B, N, H, dh).transpose(1, 2)
        kb = kv[..., :D].reshape(B, NB, H, dh).transpose(1, 2)
        vb = kv[..., D:].reshape(B, NB, H, dh).transpose(1, 2)
        bias = None
        if bullet_mask is not None:
            keep = bullet_mask.reshape(B, 1, 1, NB).to(q.dtype)
            bias = (1.0 - keep) * (torch.finfo(q.dtype).min / 2)
        o = F.scaled_dot_product_attention(q, kb, vb, attn_mask=bias, dropout_p=0.0)
        if bullet_mask is not None:
            o = o * bullet_mask.any(dim=-1).reshape(B, 1, 1, 1).to(o.dtype)
        return o.transpose(1, 2).reshape(B, N, D)


class RGLRU(_WeightCaches, nn.Module):
    """Real-gated linear recurrent unit; parameters ``log_lambda``, ``linear_a``, ``linear_x``."""

    def __init__(self, d_model: int, c: float = 8.0) -> None:
        super().__init__()
        self.c = c
        self.log_lambda = nn.Parameter(torch.linspace(0.0, 4.0, d_model))
        self.linear_a = nn.Linear(d_model, d_model, bias=True)
        self.linear_x = nn.Linear(d_model, d_model, bias=True)

    def _gate_preactivations(self, x: torch.Tensor, x_act: torch.Tensor | None = None) -> torch.Tensor:
        """``[linear_a(x) | linear_x(x)]`` as one (R, 2D) GEMM over concatenated weights.

        ``x_act``: the same rows already in the projection dtype (saves the cast)."""
        if torch.is_grad_enabled():
            # the (small) weights are concatenated, not the activations: one cast of x, one GEMM, one weight gradient
            w = torch.cat([self.linear_a.weight, self.linear_x.weight], dim=0)
            b = torch.cat([self.linear_a.bias, self.linear_x.bias], dim=0)
            if x_act is not None and x_act.dtype == _projection_dtype():
                x = x_act  # the producer's own copy in the projection dtype: no cast here, no cast back in the backward
            return _grad_linear(x, w, b)
        act = _projection_dtype()
        wa, wx, ba, bx = self.linear_a.weight, self.linear_x.weight, self.linear_a.bias, self.linear_x.bias
        if _f32_fused_ok(x, act, self.linear_a, self.linear_x) and x.dim() == 2 and ba is not None and bx is not None:
            # float32: both gate projections and their biases as one kernel on the fp32 matrix cores
            pk = _cached_cast(self, "_bnb_f32_gates", (wa, wx), torch.float32,
                              lambda: ops.pack_linear_f32(torch.cat([wa.detach(), wx.detach()], dim=0)))
            bias = _cached_cast(self, "_bnb_f32_gate_bias", (ba, bx), torch.float32,
                                lambda: torch.cat([ba.detach(), bx.detach()], dim=0).float())
            return ops.linear_f32(x, pk, bias=bias)
        if x_act is None or x_act.dtype != act:
            x_act = x.to(act)
        w = _cached_cast(self, "_bnb_gw", (wa, wx), act, lambda: torch.cat([wa, wx], dim=0).detach().to(act))
        b = _cached_cast(self, "_bnb_gb", (ba, bx), act, lambda: torch.cat([ba, bx], dim=0).detach().to(act))
        return F.linear(x_act, w, b)

    def _step(self, x: torch.Tensor, h: torch.Tensor) -> torch.Tensor:
        """(R,D), (R,D) -> new state (R,D) float32 (also the layer output)."""
        return self.step(x, h)[1]

    def step(self, x, h, y_dtype=None, *, h_out=None, reset=None, rows_per_env=1, x_act=None, y_out=None):
        """One kernel launch: returns (output in ``y_dtype`` or the state itself, new state).

        ``h_out`` lets the new state land in place (e.g. in the RG-LRU columns of a packed
        hidden tensor); ``reset`` (one bool per environment of ``rows_per_env`` rows) makes the
        previous state of those environments read as zero.
        """
        return ops.rglru_step(
            x, self._gate_preactivations(x, x_act), self.log_lambda, self.c, h, y_dtype=y_dtype, h_out=h_out,
            reset=reset, rows_per_env=rows_per_env, y_out=y_out,
        )

    def forward_sequence(self, x_seq, h0, done_mask=None, *, time_major=False, y_dtype=torch.float32, x_act=None,
                         h_out=None):
        """(R,T,D), (R,D) -> ((R,T,D) states, (R,D) last state), one pass over the sequence.

        The gate projections run as one GEMM over all R*T rows and one kernel walks the
        recurrence in time order; ``done_mask[:, t]`` cuts the state after step t
        (griffin.py:213-218).  ``time_major``: ``x_seq`` and the states are (T,R,D).
        """
        D = x_seq.shape[-1]
        flat_act = None if x_act is None else x_act.reshape(-1, D)
        gates = self._gate_preactivations(x_seq.reshape(-1, D), flat_act).reshape(*x_seq.shape[:2], 2 * D)
        return ops.rglru_scan(x_seq, gates, self.log_lambda, self.c, h0, done_mask, y_dtype=y_dtype, h_out=h_out,
                              time_major=time_major)


class GriffinTemporalBlock(_WeightCaches, nn.Module):
    """norm -> (linear1 -> causal conv -> RG-LRU) * gelu(linear2) -> linear_out, then a gated MLP."""

    def __init__(self, d_model: int) -> None:
        super().__init__()
        self.norm1 = nn.RMSNorm(d_model)
        self.linear1 = nn.Linear(d_model, d_model, bias=False)
        self.conv = nn.Conv1d(d_model, d_model, kernel_size=CONV_KERNEL, groups=d_model, bias=True)
        self.rg_lru = RGLRU(d_model)
        self.linear2 = nn.Linear(d_model, d_model, bias=False)
        self.linear_out = nn.Linear(d_model, d_model, bias=False)
        self.norm2 = nn.RMSNorm(d_model)
        self.gated_mlp = GatedMLP(d_model)

    def forward_sequence(self, x_seq, h0, conv_buf, done_mask=None, *, time_major=False):
        """(R,T,D), (R,D), (R,3,D) [, (R,T) bool] -> (out (R,T,D), new_h (R,D), new_conv_buf (R,3,D)).

        ``time_major``: ``x_seq`` and ``out`` are (T,R,D), the layout stored rollouts have.
        """
        T = x_seq.shape[0] if time_major else x_seq.shape[1]
        if T == 1 and done_mask is None and not time_major and not torch.is_grad_enabled():
            # rollout: the conv taps and the buffer shift are one kernel, the recurrence another
            x = x_seq[:, 0]
            out, new_h, new_conv_buf = self._step(x, h0, conv_buf, None, None, None, 1)
            return out.unsqueeze(1), new_h, new_conv_buf
        if torch.is_grad_enabled():
            return self._sequence_autograd(x_seq, h0, conv_buf, done_mask, time_major)
        # two passes over the sequence: conv taps (cut at episode ends), then the recurrence;
        # the only tensors in between are the conv output and the gate pre-activations
        act = _projection_dtype()
        x_seq, normed = self._norm_in(x_seq)
        b1 = _project(self.linear1, normed)
        want_lp = act == torch.bfloat16
        res = ops.conv_seq(b1, conv_buf, self.conv.weight, self.conv.bias, done_mask, also_bf16=want_lp,
                           time_major=time_major)
        y, new_h = self.rg_lru.forward_sequence(res[0], h0, done_mask, time_major=time_major,
                                                y_dtype=act if _fused_ok(x_seq, act) else torch.float32,
                                                x_act=res[2] if want_lp else None)
        return self._finish(x_seq, normed, y), new_h, res[1]

    def _sequence_autograd(self, x_seq, h0, conv_buf, done_mask, time_major):
        """Training path: torch ops (differentiable) around the recurrence, which runs on its
        forward and backward kernels."""
        if _norm_linear_train_ok(x_seq, _projection_dtype(), self.norm1, self.linear1):
            x_seq, b1, normed = _norm_linear_train(x_seq, self.norm1, self.linear1)
        else:
            x_seq, normed = _train_norm(self.norm1, x_seq)
            b1 = _project(self.linear1, normed)
        if (_TRAIN_KERNELS and ops.conv_seq_train_supported(b1) and conv_buf.dtype == torch.float32
                and self.conv.weight.dtype == torch.float32):
            # conv forward and backward on their kernels (one pass each instead of a dozen element-wise ops per tap)
            want_lp = _projection_dtype() == torch.bfloat16
            res = ops.conv_seq_train(b1, conv_buf, self.conv.weight, self.conv.bias, done_mask, time_major=time_major,
                                     also_bf16=want_lp)
            y, new_h = self.rg_lru.forward_sequence(res[0], h0, done_mask, time_major=time_major,
                                                    x_act=res[2] if want_lp else None)
            return self._finish(x_seq, normed, y), new_h, res[1]
        rows_first = b1.transpose(0, 1) if time_major else b1  # (R, T, D) view
        T = rows_first.shape[1]
        padded = torch.cat([conv_buf, rows_first], dim=1)  # fp32 buffer promotes a bf16 b1
        v = _conv_within_episodes(padded, self.conv.weight.squeeze(1), self.conv.bias, done_mask)
        if time_major:
            v = v.transpose(0, 1).contiguous()
        y, new_h = self.rg_lru.forward_sequence(v, h0, done_mask, time_major=time_major)
        return self._finish(x_seq, normed, y), new_h, padded[:, T:]

    def sequence_tokens(self, x, n_rec, h0, conv_buf, done_rows, field_sub):
        """The update's form of this sublayer over ALL tokens of a stored rollout at once, or None when it does not apply.

        x (T, B, NM, D) float32, the first ``n_rec`` tokens of an environment recurrent (state rows env-major,
        ``h0`` (B*n_rec, D), ``conv_buf`` (B*n_rec, 3, D), ``done_rows`` (B*n_rec, T) or None), the rest going through
        ``field_sub`` instead of conv + RG-LRU (griffin.py:288-317, :406-413).  The reference runs the block twice, on the
        ship rows and on the field rows, and concatenates the results; every row-wise part (both norms, linear1,
        linear2, the gate, linear_out, the gated MLP and all their backward kernels) is the same function of a row
        either way, so here it runs once over all rows, and only conv + recurrence (ship rows) and ``field_sub``
        (field rows) see a part of them.  Returns ``(out (T, B, NM, D), new_h, new_conv_buf)``."""
        T, B, NM, D = x.shape
        if not (_TRAIN_KERNELS and torch.is_grad_enabled() and x.is_cuda and NM > n_rec and field_sub is not None
                and _projection_dtype() == torch.bfloat16 and conv_buf.dtype == torch.float32
                and self.conv.weight.dtype == torch.float32):
            return None
        if _norm_linear_train_ok(x, torch.bfloat16, self.norm1, self.linear1):
            x, b1, normed = _norm_linear_train(x, self.norm1, self.linear1)
        else:
            x, normed = _train_norm(self.norm1, x)
            b1 = _project(self.linear1, normed)
        if b1.dtype != torch.bfloat16 or b1.shape[-1] != ops.FFN_WIDTH:
            return None
        rows = T * B * min(n_rec, NM - n_rec)
        if (rows >= _WGRAD_MIN_ROWS and field_sub.bias is None and self.rg_lru.linear_a.bias is not None
                and self.rg_lru.linear_x.bias is not None):
            gate_w = torch.cat([self.rg_lru.linear_a.weight, self.rg_lru.linear_x.weight], dim=0)
            gate_b = torch.cat([self.rg_lru.linear_a.bias, self.rg_lru.linear_x.bias], dim=0)
            if ops.temporal_mix_train_supported(b1, n_rec, gate_w, field_sub.weight):
                # conv, gates, recurrence (ship tokens) and field_sub (the others) read and write the token tensors in place
                y, new_h, new_buf = ops.temporal_mix_train(b1, n_rec, conv_buf, self.conv.weight, self.conv.bias, gate_w, gate_b,
                                                           self.rg_lru.log_lambda, self.rg_lru.c, h0, done_rows, field_sub.weight)
                return self._finish(x, normed, y), new_h, new_buf
        ships_b1, fields_b1 = _SplitTokens.apply(b1, n_rec)
        ships_b1 = ships_b1.reshape(T, B * n_rec, D)
        if not ops.conv_seq_train_supported(ships_b1):
            return None
        # the conv launch also writes its output in bfloat16 for the gate projections (the backward kernel adds the two gradients)
        v, new_buf, v_lp = ops.conv_seq_train(ships_b1, conv_buf, self.conv.weight, self.conv.bias, done_rows, time_major=True,
                                              also_bf16=True)
        y_ships, new_h = self.rg_lru.forward_sequence(v, h0, done_rows, time_major=True, x_act=v_lp)
        y_fields = _project(field_sub, fields_b1)
        # the recurrence's output is float32 (the conv buffer promotes its input, griffin.py:275); the field rows'
        # bfloat16 values are exact in it, and the gate kernel rounds the product once either way
        y = torch.cat([y_ships.reshape(T, B, n_rec, D), y_fields.to(y_ships.dtype)], dim=2)
        return self._finish(x, normed, y), new_h, new_buf

    def _norm_in(self, x):
        """``(x, norm1(x))`` with the norm in the projection dtype (one kernel with the cast when the fused
        path applies); the returned x is the one to use for the residual connection."""
        act = _projection_dtype()
        if _fused_ok(x, act):
            return x, ops.add_rmsnorm(x, self.norm1.weight, eps=self.norm1.eps, out_dtype=act)[1]
        return _train_norm(self.norm1, x)

    def _finish(self, x, normed, y, gate_in=None, next_head=None):
        """Gate branch, output projection and the gated MLP, both residuals.  With ``next_head`` (the ``head_spec``
        of the sublayer that follows) the result is ``(out, that head or None)``."""
        if next_head is not None:
            out = self._finish_sublayer(x, normed, y, gate_in, next_head)
            return out if isinstance(out, tuple) else (out, None)
        return self._finish_sublayer(x, normed, y, gate_in, None)

    def _finish_sublayer(self, x, normed, y, gate_in, next_head):
        act = _projection_dtype()
        if gate_in is None:
            gate_in = _project(self.linear2, normed)
        if (_f32_fused_ok(x, act, self.linear_out) and self.linear_out.bias is None and gate_in.dtype == torch.float32
                and y.dtype == torch.float32 and y.shape == gate_in.shape):
            # float32: gelu(linear2) * y, linear_out and the residual in one kernel, then the gated MLP's two
            x1 = ops.linear_f32(gate_in, _packed_f32(self.linear_out, "_bnb_f32_pack", self.linear_out.weight), gelu_times=y,
                                resid=x)
            tail = self.gated_mlp.tail_f32(x1, self.norm2)
            if tail is not None:
                return tail
            _, n2 = ops.add_rmsnorm(x1, self.norm2.weight, eps=self.norm2.eps, out_dtype=act)
            return x1 + self.gated_mlp(n2)
        if _fused_ok(x, act) and gate_in.dtype == act:
            if y.dtype == torch.bfloat16 and y.shape == gate_in.shape:
                # gelu(linear2) * y, linear_out, both residual adds, norm2 and the gated MLP in one kernel
                fused = self.gated_mlp.fused_tail(x, y, self.norm2, proj_layer=self.linear_out, gate=gate_in,
                                                  next_head=next_head)
                if fused is not None:
                    return fused
            # gelu(linear2) * y in one kernel, residual add + norm2 (+ cast) in one kernel
            r = _project(self.linear_out, ops.gelu_mul(gate_in, y, out_dtype=act))
            fused = self.gated_mlp.fused_tail(x, r, self.norm2)
            if fused is not None:
                return fused
            x1, n2 = ops.add_rmsnorm(x, self.norm2.weight, delta=r, eps=self.norm2.eps, out_dtype=act)
            return x1 + self.gated_mlp(n2)
        r = _project(self.linear_out, _gelu_gate(gate_in, y))
        tail = self.gated_mlp.train_tail(x, r, self.norm2)
        if tail is not None:
            return tail
        x1, n2 = _train_norm(self.norm2, x, r)
        return x1 + self.gated_mlp(n2)

    def _step(self, x, h_in, conv_in, h_out, conv_out, reset, rows_per_env):
        """One timestep: x (R,D), h_in (R,D), conv_in (R,3,D) -> (out, new_h, new_conv_buf)."""
        act = _projection_dtype()
        x, normed = self._norm_in(x)
        b1 = _project(self.linear1, normed)
        want_lp = act == torch.bfloat16
        res = ops.conv_step(b1, conv_in, self.conv.weight, self.conv.bias, conv_out=conv_out, reset=reset,
                            rows_per_env=rows_per_env, also_bf16=want_lp)
        v, new_conv_buf = res[0], res[1]
        y, new_h = self.rg_lru.step(v, h_in, h_out=h_out, reset=reset, rows_per_env=rows_per_env,
                                    x_act=res[2] if want_lp else None)
        return self._finish(x, normed, y), new_h, new_conv_buf

    def step_packed(self, x, state_in, state_out, reset=None, rows_per_env=1):
        """One timestep on packed state rows, written where they live.

        x (R, D); ``state_in`` / ``state_out`` (R, 4*D) float32 rows ``[h | p0 | p1 | p2]`` of the
        policy's packed hidden tensor (rows may be strided).  The conv kernel writes the shifted
        inputs into ``state_out[:, D:]`` and the RG-LRU kernel writes the new state into
        ``state_out[:, :D]``: no ``cat`` builds the padded sequence or re-packs the state, and a
        ``reset`` mask (one bool per environment) stands in for zeroing the state beforehand.
        Returns the sublayer output (R, D).
        """
        R, D = x.shape
        return self._step(
            x, state_in[:, :D], state_in[:, D:].view(R, CONV_KERNEL - 1, D), state_out[:, :D],
            state_out[:, D:].view(R, CONV_KERNEL - 1, D), reset, rows_per_env,
        )[0]

    def _head_weights(self, NM, n_rec, field_sub):
        """``(fold, weights)`` of the bfloat16 head ``[linear1 | linear2 (| field_sub . linear1)](norm1(x))``:
        with field tokens a third block carries field_sub(linear1(.)) as ONE projection (exact while field_sub is
        the identity it starts as, a bf16 rounding of b1 apart otherwise)."""
        rg = self.rg_lru
        fold = (NM > n_rec and field_sub is not None and field_sub.bias is None
                and rg.linear_a.bias is not None and rg.linear_x.bias is not None)
        return fold, (self.linear1.weight, self.linear2.weight) + ((field_sub.weight,) if fold else ())

    @staticmethod
    def _head_matrix(ws):
        blocks = [ws[0].detach().float(), ws[1].detach().float()]
        if len(ws) == 3:
            with torch.autocast("cuda", enabled=False):  # the folded product is formed in float32
                blocks.append(ws[2].detach().float() @ blocks[0])
        return torch.cat(blocks, dim=0)

    def head_spec(self, x: torch.Tensor, n_rec: int, field_sub):
        """``(norm weight, eps, packed weight, features)`` of this sublayer's head as ``step_tokens`` forms it, for the
        tail kernel of the sublayer before (``ops.ffn_fused(next_head=...)``), or None when ``step_tokens`` would not
        take the bfloat16 kernel path for tokens like ``x`` (B, NM, D)."""
        if not (_HEAD_FUSION and not torch.is_grad_enabled() and _projection_dtype() == torch.bfloat16 and x.is_cuda
                and x.dtype == torch.float32 and x.shape[-1] == ops.FFN_WIDTH and self.linear1.bias is None
                and self.linear2.bias is None and self.norm1.weight is not None and self.norm1.weight.dtype == torch.float32):
            return None
        fold, ws = self._head_weights(x.shape[1], n_rec, field_sub)
        hp = _cached_cast(self, "_bnb_l12f_head_pack" if fold else "_bnb_l12_head_pack", ws, torch.bfloat16,
                          lambda: ops.pack_head_weights(self._head_matrix(ws)))
        return (self.norm1.weight, self.norm1.eps, hp, len(ws) * ops.FFN_WIDTH)

    def step_tokens(self, x, n_rec, state_in, state_out, reset, field_sub, *, head=None, next_head=None):
        """One timestep over all tokens of every environment at once.

        x (B, NM, D): the first ``n_rec`` tokens of an environment are recurrent (state rows
        ``state_in`` / ``state_out`` (B*n_rec, 4*D) as in ``step_packed``), the rest go through
        ``field_sub`` instead of conv + RG-LRU.  Norms, projections, gate and the sublayer tail
        run once over all rows; the conv kernel reads its rows out of the (B, NM, D) projection
        and the recurrence writes its output into the (B, NM, D) gate operand in place, so the
        reference's slicing and concatenation of ship and field tokens (griffin.py:390-417)
        costs nothing.  Returns (B, NM, D).

        ``head``: this sublayer's head (``head_spec``) when the sublayer before has already formed it;
        ``next_head``: the ``head_spec`` of the sublayer that follows: the result is then ``(out, that head or None)``.
        """
        B, NM, D = x.shape
        R = B * n_rec
        act = _projection_dtype()
        gate_in = normed = None
        y = None
        if act == torch.bfloat16 and D == ops.FFN_WIDTH and self.linear1.bias is None and self.linear2.bias is None:
            # norm1, linear1 and linear2 as one kernel: [b1 | gate_in] side by side, read in place.
            # With field tokens the third block (field_sub . linear1) gives the field rows of y; the recurrence
            # then writes the ship rows of the same block, and no gather, GEMM and scatter of the field rows remain.
            fold, ws = self._head_weights(NM, n_rec, field_sub)
            if head is not None:
                both = head  # formed by the tail kernel of the sublayer before
            else:
                pk = _cached_cast(self, "_bnb_l12f_pack" if fold else "_bnb_l12_pack", ws, torch.bfloat16,
                                  lambda: ops.pack_linear_weights(self._head_matrix(ws)))
                both = ops.norm_linear(x, self.norm1.weight, pk, eps=self.norm1.eps)  # (B, NM, 2D or 3D)
            b1, gate_in = both[..., :D], both[..., D:2 * D]
            if fold:
                y = both[..., 2 * D:]
        elif (_f32_fused_ok(x, act, self.linear1, self.linear2) and self.linear1.bias is None and self.linear2.bias is None
              and self.norm1.weight is not None):
            # float32: norm1 and [linear1 | linear2] as one kernel; with field tokens field_sub(linear1(.)) is one more
            # projection of the same normed rows (field_sub . linear1 folded in float32), written for every token and
            # then overwritten on the ship rows by the recurrence
            w12 = (self.linear1.weight, self.linear2.weight)
            pk = _cached_cast(self, "_bnb_f32_l12", w12, torch.float32,
                              lambda: ops.pack_linear_f32(torch.cat([w12[0].detach(), w12[1].detach()], dim=0)))
            both = ops.linear_f32(x, pk, norm_weight=self.norm1.weight, eps=self.norm1.eps)  # (B, NM, 2D)
            b1, gate_in = both[..., :D], both[..., D:]
            if NM > n_rec and field_sub is not None and field_sub.bias is None and field_sub.weight.dtype == torch.float32:
                ws = (field_sub.weight, self.linear1.weight)
                pf = _cached_cast(self, "_bnb_f32_fsub", ws, torch.float32,
                                  lambda: ops.pack_linear_f32(ws[0].detach().float() @ ws[1].detach().float()))
                y = ops.linear_f32(x, pf, norm_weight=self.norm1.weight, eps=self.norm1.eps)  # (B, NM, D)
        else:
            x, normed = self._norm_in(x)
            b1 = _project(self.linear1, normed)
        want_lp = act == torch.bfloat16
        fields_done = y is not None
        if y is None:
            y = torch.empty((B, NM, D), dtype=act, device=x.device)
        ships_b1 = b1[:, :n_rec] if (NM > n_rec or gate_in is not None) else b1.reshape(R, D)
        rg = self.rg_lru
        if ops.temporal_step_supported(b1) and rg.linear_a.bias is not None and rg.linear_x.bias is not None:
            # conv taps + buffer shift, both gate projections and the recurrence as one kernel:
            # the conv output and the gate pre-activations never reach memory
            gw = (rg.linear_a.weight, rg.linear_x.weight)
            gb = (rg.linear_a.bias, rg.linear_x.bias)
            gpk = _cached_cast(rg, "_bnb_gate_pack", gw, torch.bfloat16, lambda: ops.pack_gate_weights(*gw))
            gbias = _cached_cast(rg, "_bnb_gate_bias", gb, torch.float32,
                                 lambda: torch.cat([gb[0], gb[1]], dim=0).detach().float())
            ops.temporal_step(ships_b1, state_in[:, D:].view(R, CONV_KERNEL - 1, D), state_in[:, :D],
                              self.conv.weight, self.conv.bias, gpk, gbias, rg.log_lambda, rg.c,
                              conv_out=state_out[:, D:].view(R, CONV_KERNEL - 1, D), h_out=state_out[:, :D],
                              y_out=y[:, :n_rec] if NM > n_rec else y.view(R, D), reset=reset, rows_per_env=n_rec)
            if NM > n_rec and not fields_done:
                y[:, n_rec:] = _project(field_sub, b1[:, n_rec:].reshape(-1, D)).view(B, NM - n_rec, D)
            return self._finish(x, normed, y, gate_in, next_head)
        res = ops.conv_step(ships_b1, state_in[:, D:].view(R, CONV_KERNEL - 1, D),
                            self.conv.weight, self.conv.bias, conv_out=state_out[:, D:].view(R, CONV_KERNEL - 1, D),
                            reset=reset, rows_per_env=n_rec, also_bf16=want_lp)
        self.rg_lru.step(res[0], state_in[:, :D], h_out=state_out[:, :D], reset=reset, rows_per_env=n_rec,
                         x_act=res[2] if want_lp else None, y_out=y[:, :n_rec] if NM > n_rec else y.view(R, D))
        if NM > n_rec and not fields_done:
            # gathered into one (B*M, D) matrix first: on the strided view the library would run a
            # batch of B tiny GEMMs
            y[:, n_rec:] = _project(field_sub, b1[:, n_rec:].reshape(-1, D)).view(B, NM - n_rec, D)
        return self._finish(x, normed, y, gate_in, next_head)

    def forward_nonrecurrent(self, x, sub):
        """Same block with ``sub`` (a Linear) in place of conv + RG-LRU; no state."""
        act = _projection_dtype()
        x, normed = self._norm_in(x)
        b1 = _project(sub, _project(self.linear1, normed))
        gate_in = _project(self.linear2, normed)
        if _fused_ok(x, act) and gate_in.dtype == act:
            r = _project(self.linear_out, ops.gelu_mul(gate_in, b1, out_dtype=act))
            fused = self.gated_mlp.fused_tail(x, r, self.norm2)
            if fused is not None:
                return fused
            x1, n2 = ops.add_rmsnorm(x, self.norm2.weight, delta=r, eps=self.norm2.eps, out_dtype=act)
            return x1 + self.gated_mlp(n2)
        r = _project(self.linear_out, _gelu_gate(gate_in, b1))
        tail = self.gated_mlp.train_tail(x, r, self.norm2)
        if tail is not None:
            return tail
        x1, n2 = _train_norm(self.norm2, x, r)
        return x1 + self.gated_mlp(n2)


def _conv_within_episodes(padded, w, bias, done_mask):
    """Depthwise causal conv whose taps stop at episode ends (griffin.py:67-140), in torch ops.

    ``padded`` (R, T+3, D), ``w`` (D, 4).  ``done_mask[:, t]`` ends an episode at t.  A tap
    contributes to output t only if the input it reads lies in the same episode as t; the
    stored buffer counts as belonging to the episode running at t = 0.
    """
    T = padded.shape[1] - (CONV_KERNEL - 1)
    if done_mask is None:
        return sum(padded[:, k:k + T] * w[:, k] for k in range(CONV_KERNEL)) + bias
    R = done_mask.shape[0]
    starts = torch.zeros_like(done_mask, dtype=torch.long)
    starts[:, 1:] = done_mask[:, :-1].long()
    episode = torch.cat([starts.new_zeros(R, CONV_KERNEL - 1), starts.cumsum(dim=1)], dim=1)  # (R, T+3)
    here = episode[:, CONV_KERNEL - 1:]
    out = 0
    for k in range(CONV_KERNEL):
        same = (episode[:, k:k + T] == here).to(padded.dtype).unsqueeze(-1)
        out = out + padded[:, k:k + T] * w[:, k] * same
    return out + bias


class TeamPMA(_WeightCaches, nn.Module):
    """Pooling by multi-head attention over each team's alive ships (policy.py:78-120).

    Parameters and ``state_dict`` keys as in the reference: ``seeds`` (2, D), ``attn``
    (``nn.MultiheadAttention``, bias-free, only its weights are used) and ``norm``.  ``forward``
    returns (B, N, D): every ship holds the pooled, normalised vector of team
    ``clamp(team_id, 0, 1)``; a team without an alive ship pools to zero.

    Float32 rows of width 128 on the GPU without gradients run as one kernel (``ops.team_pool``),
    which reads ``x`` once and never projects the ships to keys and values.  Everything else
    (training, other widths) is one library attention call with both seeds as queries.
    """

    def __init__(self, d_model: int, n_heads: int) -> None:
        super().__init__()
        self.n_heads = n_heads
        self.seeds = nn.Parameter(torch.zeros(2, d_model))
        self.attn = nn.MultiheadAttention(d_model, n_heads, batch_first=True, bias=False)
        self.norm = nn.RMSNorm(d_model)

    def _folded(self):
        srcs = (self.seeds, self.attn.in_proj_weight, self.attn.out_proj.weight)
        return _cached_cast(self, "_bnb_pool_pack", srcs, torch.float32,
                            lambda: ops.pack_team_pool_weights(*srcs, self.n_heads))

    def pooled(self, x: torch.Tensor, team_id: torch.Tensor, alive: torch.Tensor) -> torch.Tensor:
        """(B, 2, D) pooled team vectors without the broadcast back to the ships."""
        x, widened = _widen_tokens(x)
        if widened:
            return self.pooled(x, team_id, alive).to(torch.bfloat16)
        if not torch.is_grad_enabled() and ops.team_pool_supported(x, self.n_heads):
            return ops.team_pool(x, team_id, alive, *self._folded(), self.norm.weight, self.norm.eps, self.n_heads,
                                 broadcast=False)[1]
        return self._pooled_library(x, team_id, alive)

    def _pooled_library(self, x, team_id, alive):
        B, N, D = x.shape
        keys = torch.stack([(team_id == 0) & alive, (team_id == 1) & alive], dim=1)  # (B, 2, N)
        has_ship = keys.any(dim=-1, keepdim=True)
        # a team without a ship may look at every row (keeps the softmax finite); its result is gated off
        blocked = ~keys & has_ship
        out, _ = self.attn(self.seeds.unsqueeze(0).expand(B, 2, D), x, x,
                           attn_mask=blocked.repeat_interleave(self.n_heads, dim=0), need_weights=False)
        out = out * has_ship.to(out.dtype)
        return self.norm(out).to(x.dtype)

    def forward(self, x: torch.Tensor, team_id: torch.Tensor, alive: torch.Tensor) -> torch.Tensor:
        x, widened = _widen_tokens(x)
        if widened:  # a bfloat16 stream under autocast: the kernels read float32 rows, the result is rounded back
            return self.forward(x, team_id, alive).to(torch.bfloat16)
        if ops.team_pool_supported(x, self.n_heads):
            if not torch.is_grad_enabled():
                return ops.team_pool(x, team_id, alive, *self._folded(), self.norm.weight, self.norm.eps, self.n_heads)[0]
            if _TRAIN_KERNELS and self.norm.weight.dtype == torch.float32:
                # update path: the same kernels forward, gradients through the score vectors and the folded projection
                u, folded = ops.team_pool_constants(self.seeds, self.attn.in_proj_weight, self.attn.out_proj.weight, self.n_heads)
                return ops.team_pool_train(x, team_id, alive, u, folded, self.norm.weight, self.norm.eps, self.n_heads)
        B, N, D = x.shape
        if x.is_cuda and _TRAIN_KERNELS:
            _note_library("TeamPMA.forward", f"rows {tuple(x.shape)} {x.dtype}, {self.n_heads} heads")
        pool = self._pooled_library(x, team_id, alive)
        return pool.gather(1, team_id.clamp(0, 1).long().unsqueeze(-1).expand(B, N, D))


class _SplitTokens(torch.autograd.Function):
    """``(x[:, :, :n], x[:, :, n:])`` of a (T, B, NM, D) tensor as two contiguous tensors.  The backward is one
    concatenation; autograd's own slicing would fill two full-size zero tensors, copy a slice into each and
    add them."""

    @staticmethod
    def forward(ctx, x, n):
        ctx.n = n
        ctx.shape = x.shape
        ctx.set_materialize_grads(False)
        return x[:, :, :n].contiguous(), x[:, :, n:].contiguous()

    @staticmethod
    def backward(ctx, d_first, d_rest):
        T, B, NM, D = ctx.shape
        if d_first is None and d_rest is None:
            return None, None
        like = d_first if d_first is not None else d_rest
        if d_first is None:
            d_first = like.new_zeros(T, B, ctx.n, D)
        if d_rest is None:
            d_rest = like.new_zeros(T, B, NM - ctx.n, D)
        return torch.cat([d_first, d_rest], dim=2), None


class YemongBlock(_WeightCaches, nn.Module):
    """``n_spatial_per_block`` attention sublayers, then ``n_temporal_per_block`` recurrent ones."""

    def __init__(self, model_config: ModelConfig) -> None:
        super().__init__()
        D = model_config.d_model
        self.spatial = nn.ModuleList(
            TransformerBlock(model_config, reads_bullets=i < model_config.n_bullet_cross_per_block)
            for i in range(model_config.n_spatial_per_block)
        )
        self.temporal = nn.ModuleList(GriffinTemporalBlock(D) for _ in range(model_config.n_temporal_per_block))
        self.field_sub = nn.ModuleList(nn.Linear(D, D, bias=False) for _ in range(model_config.n_temporal_per_block))
        for sub in self.field_sub:
            nn.init.eye_(sub.weight)

    @property
    def n_temporal(self) -> int:
        return len(self.temporal)

    def step(self, x, alive, h, conv_buf, num_recurrent=None, bullets=None, bullet_mask=None):
        """One timestep.

        x (B,NM,D); alive (B,NM) bool; h (n_temporal, B*n_rec, D); conv_buf
        (n_temporal, B*n_rec, 3, D).  The first ``num_recurrent`` tokens of every
        environment are recurrent (state row b*n_rec + n), the rest take the state-free
        path.  Returns (x, new_h, new_conv_buf) as new tensors.
        """
        B, NM, D = x.shape
        n_rec = NM if num_recurrent is None else num_recurrent
        x, widened = _widen_tokens(x)
        if widened:
            out, new_h, new_cb = self.step(x, alive, h, conv_buf, num_recurrent, bullets, bullet_mask)
            return out.to(torch.bfloat16), new_h, new_cb
        for layer in self.spatial:
            x = layer(x, alive, bullets, bullet_mask)
        new_h, new_cb = [], []
        for j, layer in enumerate(self.temporal):
            ships = x[:, :n_rec].reshape(B * n_rec, 1, D)
            out, h_j, cb_j = layer.forward_sequence(ships, h[j], conv_buf[j])
            parts = [out.reshape(B, n_rec, D)]
            if NM > n_rec:
                parts.append(layer.forward_nonrecurrent(x[:, n_rec:], self.field_sub[j]))
            x = torch.cat(parts, dim=1) if len(parts) > 1 else parts[0]
            new_h.append(h_j)
            new_cb.append(cb_j)
        if not new_h:
            return x, h[:0], conv_buf[:0]
        return x, torch.stack(new_h), torch.stack(new_cb)

    def first_head_spec(self, x, num_recurrent):
        """``head_spec`` of this block's first sublayer for tokens like ``x`` (B, NM, D), or None."""
        if len(self.spatial):
            return self.spatial[0].head_spec(x)
        if len(self.temporal):
            return self.temporal[0].head_spec(x, num_recurrent, self.field_sub[0] if x.shape[1] > num_recurrent else None)
        return None

    def step_packed(self, x, alive, state_in, state_out, num_recurrent, reset=None, bullets=None,
                    bullet_mask=None, *, head=None, after=None):
        """``step`` on this block's slots of the packed hidden tensor.

        ``state_in`` / ``state_out`` are (n_temporal, B*n_rec, 4*D) views; the new state is
        written into ``state_out`` by the kernels.  Returns the updated tokens (B, NM, D).

        Under bfloat16 autocast each sublayer's tail kernel also forms the norm + projection the next sublayer
        starts with.  Across blocks: ``head`` is that product for this block's first sublayer when the block before
        has formed it, and ``after`` (the next block's ``first_head_spec``) asks the last sublayer here for the next
        block's; with ``after`` the result is ``(tokens, that head or None)``.
        """
        B, NM, D = x.shape
        n_rec = num_recurrent
        x, widened = _widen_tokens(x)
        if widened:
            out = self.step_packed(x, alive, state_in, state_out, num_recurrent, reset, bullets, bullet_mask, head=head,
                                   after=after)
            return (out[0].to(torch.bfloat16), out[1]) if after is not None else out.to(torch.bfloat16)
        act = _projection_dtype()
        n_s, n_t = len(self.spatial), len(self.temporal)

        def spec_of(k, x):  # head_spec of sublayer k of this block (spatial first), of the next block's first past the end
            if k < n_s:
                return self.spatial[k].head_spec(x)
            if k < n_s + n_t:
                return self.temporal[k - n_s].head_spec(x, n_rec, self.field_sub[k - n_s] if NM > n_rec else None)
            return after(x) if after is not None else None

        for k, layer in enumerate(self.spatial):
            nxt = spec_of(k + 1, x)
            out = layer(x, alive, bullets, bullet_mask, head=head, next_head=nxt)
            x, head = out if nxt is not None else (out, None)
        for j, layer in enumerate(self.temporal):
            if _fused_ok(x, act):
                fsub = self.field_sub[j] if NM > n_rec else None
                nxt = spec_of(n_s + j + 1, x)
                out = layer.step_tokens(x, n_rec, state_in[j], state_out[j], reset, fsub, head=head, next_head=nxt)
                x, head = out if nxt is not None else (out, None)
                continue
            head = None
            ships = layer.step_packed(x[:, :n_rec].reshape(B * n_rec, D), state_in[j], state_out[j], reset, n_rec)
            parts = [ships.reshape(B, n_rec, D)]
            if NM > n_rec:
                parts.append(layer.forward_nonrecurrent(x[:, n_rec:], self.field_sub[j]))
            x = torch.cat(parts, dim=1) if len(parts) > 1 else parts[0]
        return (x, head) if after is not None else x

    def sequence(self, x, alive_mask, h0, conv_buf0, done_mask=None, num_recurrent=None, bullets=None,
                 bullet_mask=None):
        """(T,B,NM,D) variant of ``step`` for re-evaluating a stored rollout.

        Under ``torch.no_grad()`` every sublayer runs on the inference kernels.  With gradients
        enabled (the PPO update) the recurrence, the conv, the norms, the gelu gates, the attention
        and the Linear weight gradients run on forward and backward kernels; the forward and
        input-gradient GEMMs stay with the library."""
        T, B, NM, D = x.shape
        n_rec = NM if num_recurrent is None else num_recurrent
        x, widened = _widen_tokens(x)
        if widened:
            out, new_h, new_cb = self.sequence(x, alive_mask, h0, conv_buf0, done_mask, num_recurrent, bullets, bullet_mask)
            return out.to(torch.bfloat16), new_h, new_cb
        for layer in self.spatial:
            x = layer(x.reshape(T * B, NM, D), alive_mask.reshape(T * B, NM), bullets, bullet_mask)
            x = x.reshape(T, B, NM, D)
        done_rows = None if done_mask is None else done_mask.t().repeat_interleave(n_rec, dim=0)  # (B*n_rec, T)
        new_h, new_cb = [], []
        for j, layer in enumerate(self.temporal):
            if NM > n_rec and torch.is_grad_enabled():
                # the update: every row-wise part of the sublayer once over all tokens
                whole = layer.sequence_tokens(x, n_rec, h0[j], conv_buf0[j], done_rows, self.field_sub[j])
                if whole is not None:
                    x = whole[0]
                    new_h.append(whole[1])
                    new_cb.append(whole[2])
                    continue
            # the sequence kernels read (T, rows, D) as stored: no transposed copies of the rollout
            if NM > n_rec and x.requires_grad:
                ships, fields = _SplitTokens.apply(x, n_rec)
            else:
                ships, fields = x[:, :, :n_rec], x[:, :, n_rec:]
            out, h_j, cb_j = layer.forward_sequence(ships.reshape(T, B * n_rec, D), h0[j], conv_buf0[j], done_rows,
                                                    time_major=True)
            parts = [out.reshape(T, B, n_rec, D)]
            if NM > n_rec:
                parts.append(layer.forward_nonrecurrent(fields, self.field_sub[j]))
            x = torch.cat(parts, dim=2) if len(parts) > 1 else parts[0]
            new_h.append(h_j)
            new_cb.append(cb_j)
        if not new_h:
            return x, h0[:0], conv_buf0[:0]
        return x, torch.stack(new_h), torch.stack(new_cb)


def _byte_range(t: torch.Tensor) -> tuple[int, int]:
    """[first, last) byte addresses a (possibly strided) tensor can touch."""
    if t.numel() == 0:
        return (0, 0)
    span = sum((n - 1) * abs(st) for n, st in zip(t.shape, t.stride())) + 1
    return t.data_ptr(), t.data_ptr() + span * t.element_size()


def _overlap(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Whether the address ranges of two tensors intersect (a view at another offset included)."""
    (a0, a1), (b0, b1) = _byte_range(a), _byte_range(b)
    return a0 < b1 and b0 < a1


class YemongTrunk(_WeightCaches, nn.Module):
    """The recurrent trunk: ``forward(tokens, alive_mask, recurrent_state) -> (hidden, new_state)``.

    ``recurrent_state`` is the packed tensor (n_layers, B*n_rec, 4*D) float32 of the
    reference policy: ``[..., :D]`` is the RG-LRU state, ``[..., D:]`` the last three conv
    inputs, oldest first.  ``n_rec`` is read off its row count, so a state sized with N
    sends the trailing M tokens down the state-free path and one sized with N+M makes every
    token recurrent.  The submodule list is named ``yemong_layers`` as in the policy.
    """

    def __init__(self, model_config: ModelConfig) -> None:
        super().__init__()
        self.config = model_config
        self.yemong_layers = nn.ModuleList(YemongBlock(model_config) for _ in range(model_config.n_yemong_blocks))

    @property
    def n_hidden_layers(self) -> int:
        return self.config.n_hidden_layers

    def initial_hidden(self, num_envs: int, num_recurrent_tokens: int, device) -> torch.Tensor:
        return torch.zeros(
            self.n_hidden_layers, num_envs * num_recurrent_tokens, CONV_KERNEL * self.config.d_model, device=device
        )

    @staticmethod
    def reset_hidden_for_envs(hidden: torch.Tensor, done_mask: torch.Tensor, num_recurrent_tokens: int):
        """Zero all rows of finished environments (rows are env-major)."""
        keep = (~done_mask.repeat_interleave(num_recurrent_tokens)).to(hidden.dtype)
        return hidden * keep[None, :, None]

    def sequence(self, x, alive_mask, initial_hidden, done_mask=None, bullets=None, bullet_mask=None, *,
                 grad_checkpoint: bool = False) -> torch.Tensor:
        """The trunk part of the rollout re-evaluation of the PPO update (policy.py:424-477): every block's
        ``sequence`` over (T, B, NM, D) tokens from the rollout-start state, ``done_mask`` (T, B) resetting
        the recurrence after an episode end.  ``initial_hidden`` is the packed (n_layers, B*n_rec, 4*D)
        state; the final states are not needed by the update and not returned.  ``grad_checkpoint``
        recomputes each block in the backward pass instead of keeping its activations, as the
        reference's ``grad_checkpoint`` option does."""
        T, B, NM, D = x.shape
        x, widened = _widen_tokens(x)
        if widened:
            return self.sequence(x, alive_mask, initial_hidden, done_mask, bullets, bullet_mask,
                                 grad_checkpoint=grad_checkpoint).to(torch.bfloat16)
        n_layers, rows = initial_hidden.shape[0], initial_hidden.shape[1]
        if n_layers != self.n_hidden_layers or rows % B:
            raise ValueError(f"initial_hidden must be ({self.n_hidden_layers}, B*n_rec, {CONV_KERNEL * D})")
        n_rec = rows // B
        if (bullets is not None and isinstance(bullet_mask, torch.Tensor) and bullet_mask.is_cuda
                and bullet_mask.dtype == torch.bool and bullet_mask.dim() == 2):
            bullet_mask = ops.CompactRows(bullet_mask)  # one list of the bullets in flight for every bullet-reading layer
        h_all = initial_hidden[:, :, :D]
        cb_all = initial_hidden[:, :, D:].reshape(n_layers, rows, CONV_KERNEL - 1, D)
        slot = 0
        for layer in self.yemong_layers:
            own = slice(slot, slot + layer.n_temporal)
            slot += layer.n_temporal

            def run(x_in, layer=layer, own=own):
                return layer.sequence(x_in, alive_mask, h_all[own], cb_all[own], done_mask, n_rec, bullets, bullet_mask)[0]

            if grad_checkpoint and torch.is_grad_enabled():
                x = torch.utils.checkpoint.checkpoint(run, x, use_reentrant=False)
            else:
                x = run(x)
        return x

    def _bullet_kv_of_all_layers(self, bullets, rows):
        """``{id(layer): [K | V] rows}`` of every bullet-reading sublayer of the step from ONE pass over the bullets in
        flight, or None when there are fewer than two such sublayers (or their norms differ in eps).

        Every reading sublayer normalises the same bullet tokens with its own ``norm_bullet`` weight and projects them
        with its own ``kv_bullet`` (attention.py:149-151).  The normalised row is the same up to that weight, which
        folds into the projection's columns: ``(x^ * w) W^T = x^ (W * w)^T``.  So the live bullets are gathered and
        normalised once and projected onto the folded weights of all layers side by side; a layer reads its column
        block.  (The operand is then ``bf16(x^)`` against ``bf16(W * w)`` instead of ``bf16(x^ * w)`` against
        ``bf16(W)``: a bfloat16 rounding apart, like the other folded products.)"""
        readers = [layer for block in self.yemong_layers for layer in block.spatial if layer.reads_bullets]
        if (len(readers) < 2 or torch.is_grad_enabled() or any(l.kv_bullet.bias is not None for l in readers)
                or any(l.norm_bullet.weight is None or l.norm_bullet.eps != readers[0].norm_bullet.eps for l in readers)):
            return None
        D = self.config.d_model
        # a layer's column block is addressed with 32-bit element offsets over the full slot capacity
        if bullets.shape[0] * bullets.shape[1] * 2 * D * len(readers) >= 2 ** 32:
            return None
        ws = tuple(t for l in readers for t in (l.kv_bullet.weight, l.norm_bullet.weight))

        def folded():
            with torch.autocast("cuda", enabled=False):
                return ops.pack_linear_weights(torch.cat(
                    [l.kv_bullet.weight.detach().float() * l.norm_bullet.weight.detach().float()[None, :] for l in readers], dim=0))

        pk = _cached_cast(self, "_bnb_bullet_kv_pack", ws, torch.bfloat16, folded)
        ones = _cached_cast(self, "_bnb_unit_norm", (readers[0].norm_bullet.weight,), torch.float32,
                            lambda: torch.ones(D, dtype=torch.float32, device=bullets.device))
        kv = ops.norm_linear(bullets, ones, pk, eps=readers[0].norm_bullet.eps, rows=rows)  # (capacity, 2 D x layers)
        return {id(l): kv[:, 2 * D * i:2 * D * (i + 1)] for i, l in enumerate(readers)}

    @torch.no_grad()
    def forward(self, tokens, alive_mask, recurrent_state, bullets=None, bullet_mask=None, *, reset_mask=None,
                out_state=None):
        """tokens (B,NM,D), alive_mask (B,NM) bool, recurrent_state (L, B*n_rec, 4D) -> (hidden, new_state).

        ``reset_mask`` (B,) bool, optional: environments whose incoming state is to be read as
        zero, i.e. ``forward(x, a, reset_hidden_for_envs(state, reset_mask, n_rec))`` without the
        extra pass over the state.  ``out_state``: optional preallocated destination for the new
        state (must not alias ``recurrent_state``); by default a new tensor is returned and the
        input state is left untouched, as in the reference.
        """
        B, NM, D = tokens.shape
        L, rows, width = recurrent_state.shape
        if L != self.n_hidden_layers or width != CONV_KERNEL * D or (B and rows % B):
            raise ValueError(
                f"recurrent_state {tuple(recurrent_state.shape)} does not fit {self.n_hidden_layers} layers, "
                f"{B} environments and d_model {D}"
            )
        if recurrent_state.dtype != torch.float32:
            raise TypeError("the recurrent state is float32")
        n_rec = rows // B if B else 0
        n_t = self.config.n_temporal_per_block
        if out_state is None:
            out_state = torch.empty_like(recurrent_state)
        elif out_state.shape != recurrent_state.shape or out_state.dtype != torch.float32 or _overlap(out_state, recurrent_state):
            raise ValueError("out_state must be a float32 tensor shaped like recurrent_state that shares no memory with it")
        if reset_mask is not None:
            reset_mask = reset_mask.contiguous()
        # the list of bullets in flight is built once and shared by every layer that reads them
        bullet_rows = bullet_mask
        if (
            bullets is not None and bullet_mask is not None and self.config.reads_bullets and bullets.is_cuda
            and bullets.dtype == torch.float32 and _projection_dtype() == torch.bfloat16 and D == ops.FFN_WIDTH
            and D // self.config.n_heads == 32 and NM <= 160
        ):
            bullet_rows = ops.CompactRows(bullet_mask)
            bullet_rows.shared_kv = self._bullet_kv_of_all_layers(bullets, bullet_rows)
        x, widened = _widen_tokens(tokens)
        blocks = list(self.yemong_layers)
        head = None
        for i, block in enumerate(blocks):
            sl = slice(i * n_t, (i + 1) * n_t)
            if i + 1 < len(blocks):
                # the last sublayer of this block also forms the norm + projection the next block starts with
                nxt = blocks[i + 1]
                x, head = block.step_packed(x, alive_mask, recurrent_state[sl], out_state[sl], n_rec, reset_mask, bullets,
                                            bullet_rows, head=head, after=lambda t, nxt=nxt: nxt.first_head_spec(t, n_rec))
            else:
                x = block.step_packed(x, alive_mask, recurrent_state[sl], out_state[sl], n_rec, reset_mask, bullets,
                                      bullet_rows, head=head)
        return (x.to(torch.bfloat16) if widened else x), out_state


def _bullet_buffers(trunk, num_envs: int, num_bullet_slots: int | None, dev, dtype):
    """Static ``(bullets, bullet_mask)`` inputs of a stepper, or ``(None, None)`` for a trunk that reads none.

    A trunk whose configuration reads bullets skips the read silently when it is handed none
    (attention.py:149), which is a different policy: a stepper over such a trunk therefore wants the slot
    count spelled out, 0 meaning that the policy has no bullet encoder and steps without them on purpose."""
    if not trunk.config.reads_bullets:
        if num_bullet_slots:
            raise ValueError("this trunk has no bullet-reading sublayer")
        return None, None
    if num_bullet_slots is None:
        raise ValueError("the trunk reads bullets: pass num_bullet_slots (0 to step without them on purpose)")
    if num_bullet_slots == 0:
        return None, None
    bullets = torch.zeros(num_envs, num_bullet_slots, trunk.config.d_model, device=dev, dtype=dtype)
    return bullets, torch.zeros(num_envs, num_bullet_slots, dtype=torch.bool, device=dev)


def _weights_stamp(params) -> int:
    """Changes whenever a parameter is written in place or touched through ``.data``."""
    return sum(p._version + getattr(p, "_bnb_touch", 0) for p in params)


class GraphedTrunk:
    """``YemongTrunk.forward`` for one fixed shape, captured into two HIP graphs and replayed.

    At rollout scale of a few thousand tokens a trunk step is ~100 short launches and the
    host, not the GPU, sets the pace (the reference notes the same of its own rollout).
    Capturing the step removes that: ``step(tokens, alive_mask, reset_mask, bullets, bullet_mask)`` copies
    the inputs into static buffers, replays one graph and returns the static output and state tensors.
    The packed state lives in two buffers that alternate as input and output, hence two
    graphs.  Outputs are overwritten by the next ``step``; clone what must outlive it.

    Weights: the captured kernels read the parameters themselves (norm weights, float32 GEMM operands)
    and the derived copies the layers cache (bfloat16 casts, concatenations, operand packings) at the
    addresses they had at capture time.  A replay runs no Python, so ``step`` first compares a stamp of the
    parameters (version counters and ``.data`` accesses) with the one of the last step and, when it moved
    (optimizer step, ``load_state_dict``, a write through ``.data``), rebuilds the derived copies whose
    sources changed into the same memory; ``refresh_weights()`` rebuilds all of them unconditionally.
    This object keeps those copies alive, so nothing the graphs read is ever returned to the allocator.
    Replacing parameter tensors, moving or casting the module requires a new capture.

    Args:
        trunk: the module to capture.
        num_envs, num_tokens, num_recurrent: B, N+M and n_rec of every later call.
        autocast_dtype: ``torch.bfloat16`` to capture under autocast, None for fp32.
        use_reset: capture with a ``reset_mask`` input (all-False masks are then cheap no-ops).
        num_bullet_slots: length of the bullet axis (ships x ring-buffer slots); required for a trunk whose
            configuration reads bullets, 0 to step such a trunk without bullets on purpose.
        bullet_dtype: dtype of the bullet tokens the caller's encoder emits (float32 by default).
    """

    def __init__(self, trunk: YemongTrunk, num_envs: int, num_tokens: int, num_recurrent: int, *,
                 autocast_dtype: torch.dtype | None = None, use_reset: bool = True, device=None,
                 num_bullet_slots: int | None = None, bullet_dtype: torch.dtype = torch.float32) -> None:
        dev = torch.device(device) if device is not None else next(trunk.parameters()).device
        D = trunk.config.d_model
        self.trunk, self.autocast_dtype = trunk, autocast_dtype
        self.tokens = torch.zeros(num_envs, num_tokens, D, device=dev)
        self.alive = torch.ones(num_envs, num_tokens, dtype=torch.bool, device=dev)
        self.reset = torch.zeros(num_envs, dtype=torch.bool, device=dev) if use_reset else None
        self.bullets, self.bullet_mask = _bullet_buffers(trunk, num_envs, num_bullet_slots, dev, bullet_dtype)
        self.states = [trunk.initial_hidden(num_envs, num_recurrent, dev) for _ in range(2)]
        self.cur = 0  # index of the buffer holding the current state
        self.graphs, self.outputs = [], []
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(3):  # warm-up outside capture: weight caches, GEMM heuristics, code loading
                self._run(0)
                self._run(1)
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        for src in (0, 1):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                out = self._run(src)
            self.graphs.append(graph)
            self.outputs.append(out)
        for s in self.states:
            s.zero_()
        # the derived weights the captured kernels read: held here so their memory outlives any cache
        # invalidation on the module, and rebuilt in place when their sources change
        self._derived = derived_weights(trunk)
        self._params = list(trunk.parameters())
        self._stamp = _weights_stamp(self._params)

    def refresh_weights(self) -> None:
        """Rebuild every derived weight copy the graphs read from the current parameters, in place."""
        for entry in self._derived:
            entry.refresh()
        self._stamp = _weights_stamp(self._params)

    def _follow_weights(self) -> None:
        stamp = _weights_stamp(self._params)
        if stamp != self._stamp:
            for entry in self._derived:
                if entry.key != _cache_key(entry.tensors, entry.dtype):
                    entry.refresh()
            self._stamp = stamp

    def _run(self, src: int) -> torch.Tensor:
        with torch.autocast("cuda", dtype=self.autocast_dtype or torch.bfloat16, enabled=self.autocast_dtype is not None):
            out, _ = self.trunk(self.tokens, self.alive, self.states[src], self.bullets, self.bullet_mask,
                                reset_mask=self.reset, out_state=self.states[1 - src])
        return out

    @property
    def state(self) -> torch.Tensor:
        """The current packed recurrent state (a static buffer)."""
        return self.states[self.cur]

    def load_state(self, state: torch.Tensor) -> None:
        self.states[self.cur].copy_(state)

    @torch.no_grad()
    def step(self, tokens, alive_mask, reset_mask=None, bullets=None, bullet_mask=None):
        """One trunk step on the captured shape; returns (hidden, new_state) static tensors.

        The inputs are copied into the static buffers ``self.tokens`` / ``self.alive`` / ``self.reset`` /
        ``self.bullets`` / ``self.bullet_mask``; a producer that writes its result straight into those buffers
        passes the buffers themselves and no copy is made (at 4096 environments x 160 tokens the token copy
        alone is 0.13 ms of a 4.5 ms step).  A capture with bullet inputs needs them at every step;
        ``bullet_mask=None`` then means every slot holds a bullet, as in the reference."""
        if tokens is not self.tokens:
            self.tokens.copy_(tokens)
        if alive_mask is not self.alive:
            self.alive.copy_(alive_mask)
        if self.reset is not None:
            if reset_mask is None:
                self.reset.fill_(False)
            elif reset_mask is not self.reset:
                self.reset.copy_(reset_mask)
        elif reset_mask is not None:
            raise ValueError("this capture was made without a reset input")
        if self.bullets is not None:
            if bullets is None:
                raise ValueError("this capture reads bullets: pass bullets (and bullet_mask) at every step")
            if bullets is not self.bullets:
                self.bullets.copy_(bullets)
            if bullet_mask is None:
                self.bullet_mask.fill_(True)
            elif bullet_mask is not self.bullet_mask:
                self.bullet_mask.copy_(bullet_mask)
        elif bullets is not None:
            raise ValueError("this capture was made without bullet inputs")
        self._follow_weights()
        self.graphs[self.cur].replay()
        out = self.outputs[self.cur]
        self.cur = 1 - self.cur
        return out, self.states[self.cur]


class EagerTrunkStepper:
    """``GraphedTrunk``'s interface on plain launches: the packed state alternates between two buffers it owns and
    ``step(tokens, alive_mask, reset_mask, bullets, bullet_mask)`` returns ``(hidden, new_state)``.  For batches
    large enough that the kernels, not their launches, set the pace of a step."""

    def __init__(self, trunk: YemongTrunk, num_envs: int, num_tokens: int, num_recurrent: int, *,
                 autocast_dtype: torch.dtype | None = None, device=None, num_bullet_slots: int | None = None,
                 bullet_dtype: torch.dtype = torch.float32) -> None:
        dev = torch.device(device) if device is not None else next(trunk.parameters()).device
        self.trunk, self.autocast_dtype = trunk, autocast_dtype
        if trunk.config.reads_bullets and num_bullet_slots is None:
            raise ValueError("the trunk reads bullets: pass num_bullet_slots (0 to step without them on purpose)")
        if num_bullet_slots and not trunk.config.reads_bullets:
            raise ValueError("this trunk has no bullet-reading sublayer")
        self.reads_bullets = bool(num_bullet_slots)
        self.states = [trunk.initial_hidden(num_envs, num_recurrent, dev) for _ in range(2)]
        self.cur = 0

    def refresh_weights(self) -> None:
        """Nothing to do: every step looks the weights up (the derived copies follow the parameters' version counters)."""

    @property
    def state(self) -> torch.Tensor:
        return self.states[self.cur]

    def load_state(self, state: torch.Tensor) -> None:
        self.states[self.cur].copy_(state)

    @torch.no_grad()
    def step(self, tokens, alive_mask, reset_mask=None, bullets=None, bullet_mask=None):
        if self.reads_bullets and bullets is None:
            raise ValueError("this stepper reads bullets: pass bullets (and bullet_mask) at every step")
        if not self.reads_bullets and bullets is not None:
            raise ValueError("this stepper was made without bullet inputs")
        with torch.autocast("cuda", dtype=self.autocast_dtype or torch.bfloat16, enabled=self.autocast_dtype is not None):
            out, new_state = self.trunk(tokens, alive_mask, self.states[self.cur], bullets, bullet_mask,
                                        reset_mask=reset_mask, out_state=self.states[1 - self.cur])
        self.cur = 1 - self.cur
        return out, new_state


# tokens per step below which a captured step beats plain launches (measured on MI355X with the default trunk of
# 2 blocks x (2 attention + 1 temporal sublayer)): the launches of a step take the host ~0.4 ms
GRAPH_BELOW_TOKENS = {torch.float32: 10_000, torch.bfloat16: 40_000}


def trunk_stepper(trunk: YemongTrunk, num_envs: int, num_tokens: int, num_recurrent: int, *,
                  autocast_dtype: torch.dtype | None = None, graph: bool | None = None, device=None,
                  num_bullet_slots: int | None = None, bullet_dtype: torch.dtype = torch.float32):
    """The rollout's way to step the trunk for one fixed shape: a ``GraphedTrunk`` (the step captured into HIP graphs)
    when ``num_envs * num_tokens`` is small enough that launches set the pace (``GRAPH_BELOW_TOKENS``), an
    ``EagerTrunkStepper`` above that; ``graph`` forces either.  Both own the packed state and share
    ``step`` / ``state`` / ``load_state`` / ``refresh_weights``.  A trunk whose configuration reads bullets needs
    ``num_bullet_slots`` (the length of the bullet axis; 0 to step without bullets on purpose)."""
    if graph is None:
        graph = num_envs * num_tokens < GRAPH_BELOW_TOKENS[torch.float32 if autocast_dtype is None else torch.bfloat16]
    if graph:
        return GraphedTrunk(trunk, num_envs, num_tokens, num_recurrent, autocast_dtype=autocast_dtype, device=device,
                            num_bullet_slots=num_bullet_slots, bullet_dtype=bullet_dtype)
    return EagerTrunkStepper(trunk, num_envs, num_tokens, num_recurrent, autocast_dtype=autocast_dtype, device=device,
                             num_bullet_slots=num_bullet_slots, bullet_dtype=bullet_dtype)
