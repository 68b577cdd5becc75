"""Benchmark workloads, their algorithmic HBM traffic, and the minimal measured step.

The five workloads are the configurations the step is quoted on (4v4 on CPU-sized and
rollout-sized batches, 8v11, 32v48, 64v88).  ``AttnRglruStep`` is the smallest
composition of the reference's operations that contains both kernels:

    qkv = tokens W_qkv^T -> masked attention -> u = o W_o^T           (attention.py:135-169)
    ships = u[:, :N] -> [W_a ships + b_a | W_x ships + b_x] -> RG-LRU  (griffin.py:179-186)
    hidden = cat(y, u[:, N:])   (fields skip the recurrence, griffin.py:406-413)
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

D_MODEL = 128
N_HEADS = 4
HBM_PEAK_BYTES_PER_S = 8.0e12  # MI355X HBM3E


@dataclass(frozen=True)
class Workload:
    """One benchmark configuration: B environments of N ship + M field tokens."""

    name: str
    index: int  # position in the list of quoted configurations; seeds derive from it
    B: int
    N: int
    M: int
    dtype: torch.dtype
    steps: int  # timesteps the recurrent state is carried for
    alive: str  # "bernoulli:<p>" | "dying:<p per step>" | "uniform_live:<lo>:<hi>"

    @property
    def NM(self) -> int:
        return self.N + self.M

    @property
    def tokens_per_step(self) -> int:
        return self.B * self.NM

    @property
    def seed(self) -> int:
        return 1234 + self.index


WORKLOADS = {
    w.name: w
    for w in (
        Workload("c0_4v4_fp32", 0, 1024, 8, 4, torch.float32, 1, "bernoulli:0.85"),
        Workload("c1_4v4_rollout_bf16", 1, 8192, 8, 4, torch.bfloat16, 128, "dying:0.01"),
        Workload("c2_8v11_bf16", 2, 4096, 19, 4, torch.bfloat16, 1, "bernoulli:0.8"),
        Workload("c3_32v48_bf16", 3, 4096, 80, 4, torch.bfloat16, 1, "bernoulli:0.7"),
        Workload("c4_64v88_bf16", 4, 4096, 152, 8, torch.bfloat16, 64, "uniform_live:16:160"),
    )
}
HEADLINE = "c4_64v88_bf16"


def algorithmic_bytes(w: Workload, d_model: int = D_MODEL) -> dict:
    """HBM bytes one step must move, counting every token, dead or alive.

    attention: read Q, K, V and one alive byte per token, write O once.
    RG-LRU:    read x and both gate pre-activations, read and write the fp32 state, and in
               bf16 mode write the bf16 copy of the output as well.
    """
    s = 2 if w.dtype == torch.bfloat16 else 4
    attn = w.NM * (4 * d_model * s + 1)
    rglru = w.N * (3 * d_model * s + 2 * d_model * 4 + (d_model * s if s == 2 else 0))
    return {
        "attn_per_env": attn,
        "rglru_per_env": rglru,
        "attn": w.B * attn,
        "rglru": w.B * rglru,
        "step": w.B * (attn + rglru),
        # what a single kernel fused with its projections could not go below
        "contract_boundary": w.B * (w.NM * (2 * d_model * s + 1) + w.N * 2 * d_model * 4),
    }


def attention_flops(w: Workload, d_model: int = D_MODEL) -> int:
    return w.B * 4 * w.NM * w.NM * d_model


# ----------------------------------------------------------------------------- inputs


def make_weights(seed: int, dtype: torch.dtype, d_model: int = D_MODEL) -> dict:
    """Xavier-uniform projections, U(+-1/sqrt(D)) biases, log_lambda = linspace(0, 4, D); CPU tensors."""
    g = torch.Generator().manual_seed(seed)

    def xavier(out_f, in_f):
        bound = math.sqrt(6.0 / (in_f + out_f))
        return ((torch.rand(out_f, in_f, generator=g) * 2 - 1) * bound).to(dtype)

    def bias(n):
        return ((torch.rand(n, generator=g) * 2 - 1) / math.sqrt(d_model)).to(dtype)

    return {
        "qkv.weight": xavier(3 * d_model, d_model),
        "out_proj.weight": xavier(d_model, d_model),
        "linear_a.weight": xavier(d_model, d_model),
        "linear_a.bias": bias(d_model),
        "linear_x.weight": xavier(d_model, d_model),
        "linear_x.bias": bias(d_model),
        "log_lambda": torch.linspace(0.0, 4.0, d_model),
    }


def make_alive(w: Workload, steps: int | None = None, B: int | None = None) -> torch.Tensor:
    """(steps, B, NM) bool alive masks on the CPU, seeded; field tokens are always alive."""
    steps = w.steps if steps is None else steps
    B = w.B if B is None else B
    g = torch.Generator().manual_seed(w.seed * 7919 + 1)
    kind, *args = w.alive.split(":")
    alive = torch.ones(steps, B, w.NM, dtype=torch.bool)
    if kind == "bernoulli":
        p = float(args[0])
        alive[:, :, : w.N] = (torch.rand(B, w.N, generator=g) < p).unsqueeze(0)
    elif kind == "dying":
        p = float(args[0])
        cur = torch.ones(B, w.N, dtype=torch.bool)
        for t in range(steps):
            if t:
                cur = cur & (torch.rand(B, w.N, generator=g) >= p)
            alive[t, :, : w.N] = cur
    elif kind == "uniform_live":
        lo, hi = int(args[0]), int(args[1])
        live = torch.randint(lo, hi + 1, (B,), generator=g)  # live tokens per env, fields included
        ships_live = (live - w.M).clamp_(0, w.N)
        rank = torch.rand(B, w.N, generator=g).argsort(dim=1).argsort(dim=1)  # random permutation rank
        alive[:, :, : w.N] = (rank < ships_live.unsqueeze(1)).unsqueeze(0)
    else:
        raise ValueError(f"unknown alive spec {w.alive!r}")
    return alive


def make_inputs(w: Workload, B: int | None = None, d_model: int = D_MODEL):
    """Seeded CPU inputs for one step: tokens (B,NM,D) ~ N(0,1) in w.dtype, state (B*N,D) ~ N(0,0.5) fp32."""
    B = w.B if B is None else B
    g = torch.Generator().manual_seed(w.seed)
    tokens = torch.randn(B, w.NM, d_model, generator=g).to(w.dtype)
    state = 0.5 * torch.randn(B * w.N, d_model, generator=g)
    return tokens, state


# ----------------------------------------------------------------------------- measured step


class AttnRglruStep(nn.Module):
    """``forward(tokens, alive_mask, recurrent_state) -> (hidden, new_state)`` on the two kernels.

    tokens (B, NM, D); alive_mask (B, NM) bool; recurrent_state (B*N, D) float32 for the
    first N tokens of each environment.  hidden is (B, NM, D) in tokens' dtype, new_state
    (B*N, D) float32.
    """

    def __init__(self, d_model: int = D_MODEL, n_heads: int = N_HEADS, c: float = 8.0) -> None:
        super().__init__()
        self.n_heads = n_heads
        self.c = c
        self.qkv = nn.Linear(d_model, 3 * d_model, bias=False)
        self.out_proj = nn.Linear(d_model, d_model, bias=False)
        self.gates = nn.Linear(d_model, 2 * d_model, bias=True)  # rows [linear_a ; linear_x]
        self.log_lambda = nn.Parameter(torch.linspace(0.0, 4.0, d_model))

    @classmethod
    def from_weights(cls, p: dict, device, n_heads: int = N_HEADS) -> "AttnRglruStep":
        d_model = p["out_proj.weight"].shape[0]
        m = cls(d_model, n_heads)
        dtype = p["qkv.weight"].dtype
        with torch.no_grad():
            m.to(dtype)
            m.qkv.weight.copy_(p["qkv.weight"])
            m.out_proj.weight.copy_(p["out_proj.weight"])
            m.gates.weight.copy_(torch.cat([p["linear_a.weight"], p["linear_x.weight"]], dim=0))
            m.gates.bias.copy_(torch.cat([p["linear_a.bias"], p["linear_x.bias"]], dim=0))
            m.log_lambda.data = p["log_lambda"].float().clone()
        return m.to(device).eval()

    @torch.no_grad()
    def forward(self, tokens, alive_mask, recurrent_state):
        B, NM, D = tokens.shape
        N = recurrent_state.shape[0] // B if B else 0
        merged = ops.sdpa_masked(self.qkv(tokens), alive_mask, self.n_heads)
        u = self.out_proj(merged)
        ships = u[:, :N].reshape(B * N, D)
        y, new_state = ops.rglru_step(
            ships, self.gates(ships), self.log_lambda, self.c, recurrent_state, y_dtype=tokens.dtype
        )
        hidden = y.reshape(B, N, D) if NM == N else torch.cat([y.reshape(B, N, D), u[:, N:]], dim=1)
        return hidden, new_state
