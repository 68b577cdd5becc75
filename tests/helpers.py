"""Shared test utilities: seeded weights keyed by the reference's state_dict names, error metrics."""

from __future__ import annotations

import math
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _xavier(gen: torch.Generator, out_f: int, in_f: int) -> torch.Tensor:
    bound = math.sqrt(6.0 / (in_f + out_f))
    return (torch.rand(out_f, in_f, generator=gen) * 2 - 1) * bound


def _uniform(gen: torch.Generator, n: int, fan_in: int) -> torch.Tensor:
    bound = 1.0 / math.sqrt(fan_in)
    return (torch.rand(n, generator=gen) * 2 - 1) * bound


def spatial_params(gen: torch.Generator, prefix: str, D: int) -> dict:
    """Weights of one spatial sublayer (names: models/yemong/attention.py:60-74)."""
    return {
        prefix + "norm1.weight": 1.0 + 0.1 * torch.randn(D, generator=gen),
        prefix + "qkv.weight": _xavier(gen, 3 * D, D),
        prefix + "out_proj.weight": _xavier(gen, D, D),
        prefix + "norm2.weight": 1.0 + 0.1 * torch.randn(D, generator=gen),
        prefix + "ffn.gate_proj.weight": _xavier(gen, 4 * D, D),
        prefix + "ffn.up_proj.weight": _xavier(gen, 4 * D, D),
        prefix + "ffn.down_proj.weight": _xavier(gen, D, 4 * D),
    }


def temporal_params(gen: torch.Generator, prefix: str, D: int) -> dict:
    """Weights of one temporal sublayer (names: models/yemong/griffin.py:165-167,238-247)."""
    return {
        prefix + "norm1.weight": 1.0 + 0.1 * torch.randn(D, generator=gen),
        prefix + "linear1.weight": _xavier(gen, D, D),
        prefix + "conv.weight": 0.5 * torch.randn(D, 1, 4, generator=gen),
        prefix + "conv.bias": 0.1 * torch.randn(D, generator=gen),
        prefix + "rg_lru.log_lambda": torch.linspace(0.0, 4.0, D),
        prefix + "rg_lru.linear_a.weight": _xavier(gen, D, D),
        prefix + "rg_lru.linear_a.bias": _uniform(gen, D, D),
        prefix + "rg_lru.linear_x.weight": _xavier(gen, D, D),
        prefix + "rg_lru.linear_x.bias": _uniform(gen, D, D),
        prefix + "linear2.weight": _xavier(gen, D, D),
        prefix + "linear_out.weight": _xavier(gen, D, D),
        prefix + "norm2.weight": 1.0 + 0.1 * torch.randn(D, generator=gen),
        prefix + "gated_mlp.gate_proj.weight": _xavier(gen, 4 * D, D),
        prefix + "gated_mlp.up_proj.weight": _xavier(gen, 4 * D, D),
        prefix + "gated_mlp.down_proj.weight": _xavier(gen, D, 4 * D),
    }


def block_params(gen: torch.Generator, prefix: str, D: int, n_spatial: int, n_temporal: int) -> dict:
    """Weights of one Yemong block (names: models/yemong/griffin.py:340-368)."""
    p: dict = {}
    for s in range(n_spatial):
        p.update(spatial_params(gen, f"{prefix}spatial.{s}.", D))
    for j in range(n_temporal):
        p.update(temporal_params(gen, f"{prefix}temporal.{j}.", D))
        # the reference starts field_sub at identity; perturb it so a wrong wiring shows
        p[f"{prefix}field_sub.{j}.weight"] = torch.eye(D) + 0.05 * torch.randn(D, D, generator=gen)
    return p


def trunk_params(seed: int, D: int, n_blocks: int, n_spatial: int, n_temporal: int) -> dict:
    gen = torch.Generator().manual_seed(seed)
    p: dict = {}
    for i in range(n_blocks):
        p.update(block_params(gen, f"yemong_layers.{i}.", D, n_spatial, n_temporal))
    return p


def max_rel(y: torch.Tensor, ref: torch.Tensor) -> float:
    """max|y - ref| / max|ref| over the whole tensor (the parity metric of the step)."""
    y, ref = y.double(), ref.double()
    return float((y - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def team_pool_params(gen: torch.Generator, prefix: str, D: int) -> dict:
    """Weights of the team pooling layer (names: models/yemong/policy.py:88-92; scales as initialised at :218-220)."""
    return {
        prefix + "seeds": 0.5 * torch.randn(2, D, generator=gen),
        prefix + "attn.in_proj_weight": torch.randn(3 * D, D, generator=gen) * math.sqrt(2.0 / D),
        prefix + "attn.out_proj.weight": torch.randn(D, D, generator=gen) / math.sqrt(D),
        prefix + "norm.weight": 1.0 + 0.1 * torch.randn(D, generator=gen),
    }


def team_case(seed: int, B: int, N: int, p_alive: float = 0.7):
    """Seeded (team_id int32, alive bool) with the edge cases in the first environments: one team
    absent, everybody dead, everybody alive, a single ship alive."""
    g = torch.Generator().manual_seed(seed)
    team = torch.randint(0, 2, (B, N), generator=g, dtype=torch.int32)
    alive = torch.rand(B, N, generator=g) < p_alive
    if B > 0 and N > 0:
        team[0] = 0
    if B > 1:
        alive[1] = False
    if B > 2:
        alive[2] = True
    if B > 3 and N > 0:
        alive[3] = False
        alive[3, N - 1] = True
    return team, alive


F32_COMPOSED_TOL = 1e-5  # the float32 bar of the step, applied to compositions through ``assert_float32_bar``


def as_float64(p: dict) -> dict:
    return {k: v.double() for k, v in p.items()}


def float64_truth(fn, *args, **kwargs):
    """``fn`` of the torch oracle evaluated in float64 on the same (float32) numbers, with the float32 module's
    norm eps: the exact value of the function the float32 module computes, up to float64 rounding."""
    from oracle import torch_ref

    def widen(a):
        if isinstance(a, dict):
            return as_float64(a)
        if isinstance(a, torch.Tensor) and a.is_floating_point():
            return a.double()
        return a

    with torch_ref.norm_eps_of(torch.float32):
        return fn(*[widen(a) for a in args], **{k: widen(v) for k, v in kwargs.items()})


def assert_float32_bar(got: torch.Tensor, ref32: torch.Tensor, ref64: torch.Tensor, what, tol: float = F32_COMPOSED_TOL):
    """The bar of a float32 composition several sublayers deep.

    ``ref64`` is the exact value (``float64_truth``), ``ref32`` what the float32 torch oracle makes of the same
    inputs.  The kernels pass when they are within ``tol`` (max |error| / max |value|) of the exact value, or
    no further from it than the float32 oracle is: a composition cannot be asked to round better than the
    reference's own arithmetic does.  Both errors are printed (``pytest -s`` shows them)."""
    scale = ref64.abs().max().clamp_min(1e-30)
    err_kernels = float((got.double() - ref64).abs().max() / scale)
    err_oracle = float((ref32.double() - ref64).abs().max() / scale)
    print(f"float32 bar [{what}]: kernels vs float64 {err_kernels:.2e}, float32 oracle vs float64 {err_oracle:.2e}", flush=True)
    assert err_kernels <= max(tol, err_oracle), (what, err_kernels, err_oracle)
