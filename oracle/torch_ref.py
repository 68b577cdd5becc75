"""CPU oracle for the attention + RG-LRU step, restated with plain torch ops.

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the package, its kernels, its
modules) may import this file; it exists so that tests, the smoke check and the
CPU-baseline leg of the benchmark have an independent statement of what the
reference computes.  Every function is written from the text of the reference
and cites the lines it follows (paths relative to the reference checkout,
``src/boost_and_broadside/``).

All functions are pure: weights come in as a flat ``dict`` keyed by the
reference's ``state_dict`` names, so the oracle shares no module code with the
product.  Dtype behaviour is whatever torch's own type promotion gives for the
dtypes passed in, which is exactly how the reference behaves under autocast:
feed bf16 gate pre-activations and the sigmoids come out bf16, the decay
``sigmoid(log_lambda) ** (c * r)`` promotes to fp32, and so on.

How each function is pinned (see tests/test_oracle_pins.py):

* ``sdpa_masked``      library routine (torch SDPA) + fp64 brute force
                       (oracle/bruteforce.py) + closed forms (all-alive,
                       single alive key, all dead => mean of V, dead-key
                       perturbation invariance, permutation equivariance).
* ``sdpa_masked_softmax``  the same function written out, for gradients: values and
                       gradients equal ``sdpa_masked``'s wherever an environment has a live
                       key, closed form (uniform weights) where it has none.
* ``rglru_step``       closed forms from the recurrence (x=0, h=0, lambda=0
                       with r=1, r=0 => clamp floor) + the C restatement.
* ``conv_sequence``    library ``F.conv1d`` (no boundaries) and per-episode ``F.conv1d`` on
                       zero history (with boundaries).
* ``rglru_sequence``   the log-depth scan == a plain loop of the pinned ``rglru_step`` with
                       the state zeroed after each episode end; fp64 agreement to 1e-12.
* ``team_pool``        library ``nn.MultiheadAttention`` + ``nn.RMSNorm`` composed as the
                       reference's forward does + fp64 brute force + closed forms (one
                       ship alive => that ship's projected row, empty team => zeros,
                       other-team / dead perturbation invariance).
* ``temporal_step``    step == sequence, with the sequence path built on the
                       library ``F.conv1d`` (fixes tap order and buffer order).
* ``field_step``, ``block_step``, ``pack/unpack/reset``  invariants the
                       reference's own tests state (fields ignore state, reset
                       zeroes exactly the done environments, env-major rows).
"""

from __future__ import annotations

import contextlib
import math

import torch
import torch.nn.functional as F

CONV_TAPS = 4  # models/yemong/griffin.py:22


# --------------------------------------------------------------------------
# Level K: the two operations the HIP kernels replace
# --------------------------------------------------------------------------

def key_bias(alive: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Additive key bias (B,1,1,NM) in ``dtype``: 0 where alive, finfo.min/2 where dead.

    Follows models/yemong/attention.py:101-112.
    """
    keep = alive.reshape(alive.shape[0], 1, 1, alive.shape[-1]).to(dtype)
    return (1.0 - keep) * (torch.finfo(dtype).min / 2)


def sdpa_masked(qkv: torch.Tensor, alive: torch.Tensor | None, n_heads: int) -> torch.Tensor:
    """Masked multi-head attention over one packed projection buffer.

    ``qkv`` is (B, NM, 3*D) with columns [Q | K | V], each third split head-major
    into ``n_heads`` runs of D/n_heads columns.  Returns (B, NM, D) with the heads
    merged back head-major, i.e. the tensor the reference hands to ``out_proj``.
    Follows models/yemong/attention.py:136-147 and :168.
    """
    B, NM, D3 = qkv.shape
    D = D3 // 3
    dh = D // n_heads
    q, k, v = (t.reshape(B, NM, n_heads, dh).transpose(1, 2) for t in qkv.split(D, dim=-1))
    bias = None if alive is None else key_bias(alive, q.dtype)
    o = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, dropout_p=0.0)
    return o.transpose(1, 2).reshape(B, NM, D)


def sdpa_masked_softmax(qkv: torch.Tensor, alive: torch.Tensor | None, n_heads: int) -> torch.Tensor:
    """``sdpa_masked`` with the attention written out (scores, bias, softmax, weighted sum) instead
    of the library call of models/yemong/attention.py:147: the statement whose autograd is the
    gradient truth.

    The forward values are the same.  The gradients are the same wherever an environment has a
    live key.  For an environment without one, the fused library backward recomputes the weights
    from ``scores + bias - logsumexp`` with the finfo.min/2 bias absorbing ``log(NM)``, which turns
    every weight into 1 instead of 1/NM (an artefact of that kernel, NM times the gradient of
    the function it evaluated); this statement keeps the weights it used in the forward.
    """
    B, NM, D3 = qkv.shape
    D = D3 // 3
    dh = D // n_heads
    q, k, v = (t.reshape(B, NM, n_heads, dh).transpose(1, 2) for t in qkv.split(D, dim=-1))
    scores = q @ k.transpose(-1, -2) / (dh ** 0.5)
    if alive is not None:
        scores = scores + key_bias(alive, q.dtype)
    o = torch.softmax(scores, dim=-1) @ v
    return o.transpose(1, 2).reshape(B, NM, D)


def bullet_read(qkv: torch.Tensor, kv: torch.Tensor, bullet_mask: torch.Tensor | None, n_heads: int) -> torch.Tensor:
    """Cross-attention of the entity queries to bullet key/values, merged head-major.

    ``qkv`` (B, N, 3D) is the entity projection (only its Q third is used), ``kv`` (B, NB, 2D)
    is ``kv_bullet(norm_bullet(bullets))`` = [K | V].  Inactive bullets get the additive
    finfo.min/2 bias; an environment with no active bullet is gated to exactly zero instead of
    the uniform average the bias alone would give.  Follows models/yemong/attention.py:149-165.
    """
    B, N, D3 = qkv.shape
    D = D3 // 3
    dh = D // n_heads
    NB = kv.shape[1]
    q = qkv[..., :D].reshape(B, N, n_heads, dh).transpose(1, 2)
    kb = kv[..., :D].reshape(B, NB, n_heads, dh).transpose(1, 2)
    vb = kv[..., D:].reshape(B, NB, n_heads, dh).transpose(1, 2)
    bias = None if bullet_mask is None else key_bias(bullet_mask, q.dtype)
    o = F.scaled_dot_product_attention(q, kb, vb, attn_mask=bias, dropout_p=0.0)
    if bullet_mask is not None:
        o = o * bullet_mask.any(dim=-1).reshape(B, 1, 1, 1).to(o.dtype)
    return o.transpose(1, 2).reshape(B, N, D)


def rglru_step(
    x: torch.Tensor,
    gates_pre: torch.Tensor,
    log_lambda: torch.Tensor,
    c: float,
    h: torch.Tensor,
) -> torch.Tensor:
    """One RG-LRU update given the two gate pre-activations.

    ``gates_pre`` is (R, 2*D): columns [0,D) are ``linear_a(x)``, columns [D,2D)
    are ``linear_x(x)`` (bias included).  Returns the new state, which is also the
    layer output.  Follows models/yemong/griffin.py:179-186 (identical to the T=1
    scan, griffin.py:206-212 with :45-64 degenerating to ``a*h0 + b``).
    """
    D = x.shape[-1]
    r = torch.sigmoid(gates_pre[..., :D])
    i = torch.sigmoid(gates_pre[..., D:])
    a = torch.sigmoid(log_lambda) ** (c * r)
    g = torch.sqrt(torch.clamp((1.0 - a) * (1.0 + a), min=1e-6))
    return a * h + g * (i * x)


# --------------------------------------------------------------------------
# Level M pieces (torch library ops around the two kernels)
# --------------------------------------------------------------------------

_NORM_EPS_DTYPE = None  # set by norm_eps_of(): the dtype whose eps the norms use, whatever dtype they compute in


@contextlib.contextmanager
def norm_eps_of(dtype: torch.dtype):
    """Inside the block every ``rms_norm`` uses ``finfo(dtype).eps`` instead of the eps of the dtype it is handed.

    ``nn.RMSNorm(D)`` takes its eps from the input's dtype, so the float32 module and the same formulas typed in
    float64 are two slightly different functions.  A float64 evaluation that is to serve as the exact value of the
    float32 module (the yardstick of the composed float32 tests) keeps the float32 eps: ``norm_eps_of(torch.float32)``."""
    global _NORM_EPS_DTYPE
    keep, _NORM_EPS_DTYPE = _NORM_EPS_DTYPE, dtype
    try:
        yield
    finally:
        _NORM_EPS_DTYPE = keep


def rms_norm(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``nn.RMSNorm(D)`` with its default ``eps=None`` (=> finfo(x.dtype).eps)."""
    eps = None if _NORM_EPS_DTYPE is None else torch.finfo(_NORM_EPS_DTYPE).eps
    return F.rms_norm(x, (x.shape[-1],), weight, eps)


def gated_mlp(p: dict, prefix: str, x: torch.Tensor) -> torch.Tensor:
    """down(gelu(gate(x)) * up(x)); models/yemong/attention.py:21-37."""
    gate = F.gelu(F.linear(x, p[prefix + "gate_proj.weight"]))
    return F.linear(gate * F.linear(x, p[prefix + "up_proj.weight"]), p[prefix + "down_proj.weight"])


def spatial_sublayer(p: dict, prefix: str, x: torch.Tensor, alive: torch.Tensor | None, n_heads: int,
                     bullets: torch.Tensor | None = None, bullet_mask: torch.Tensor | None = None) -> torch.Tensor:
    """Pre-norm attention (+ optional bullet read) + FFN block; models/yemong/attention.py:76-99,114-169."""
    n = rms_norm(x, p[prefix + "norm1.weight"])
    qkv = F.linear(n, p[prefix + "qkv.weight"])
    merged = sdpa_masked(qkv, alive, n_heads)
    if bullets is not None and (prefix + "kv_bullet.weight") in p:
        kv = F.linear(rms_norm(bullets, p[prefix + "norm_bullet.weight"]), p[prefix + "kv_bullet.weight"])
        merged = merged + bullet_read(qkv, kv, bullet_mask, n_heads)
    x = x + F.linear(merged, p[prefix + "out_proj.weight"])
    return x + gated_mlp(p, prefix + "ffn.", rms_norm(x, p[prefix + "norm2.weight"]))


def rglru_gates(p: dict, prefix: str, x: torch.Tensor) -> torch.Tensor:
    """[linear_a(x) | linear_x(x)] as one (R, 2D) tensor; models/yemong/griffin.py:166-167."""
    return torch.cat(
        [
            F.linear(x, p[prefix + "linear_a.weight"], p[prefix + "linear_a.bias"]),
            F.linear(x, p[prefix + "linear_x.weight"], p[prefix + "linear_x.bias"]),
        ],
        dim=-1,
    )


def temporal_step(p: dict, prefix: str, x: torch.Tensor, h: torch.Tensor, conv_buf: torch.Tensor):
    """Griffin temporal sublayer for one timestep.

    x (R,D), h (R,D), conv_buf (R,3,D) oldest -> newest.  Returns
    (x_out, h_new, conv_buf_new).  Follows models/yemong/griffin.py:269-286 with
    T=1 and done_mask=None; the tap at weight index k multiplies padded[:, k]
    (griffin.py:131-137), so the current input meets weight index 3.
    """
    n = rms_norm(x, p[prefix + "norm1.weight"])
    b1 = F.linear(n, p[prefix + "linear1.weight"])
    w = p[prefix + "conv.weight"].squeeze(1)  # (D, 4)
    padded = torch.cat([conv_buf, b1.unsqueeze(1)], dim=1)  # (R, 4, D)
    v = (padded * w.t().unsqueeze(0)).sum(dim=1) + p[prefix + "conv.bias"]
    lam = p[prefix + "rg_lru.log_lambda"]
    h_new = rglru_step(v, rglru_gates(p, prefix + "rg_lru.", v), lam, 8.0, h)
    b2 = F.gelu(F.linear(n, p[prefix + "linear2.weight"]))
    x1 = x + F.linear(h_new * b2, p[prefix + "linear_out.weight"])
    x2 = x1 + gated_mlp(p, prefix + "gated_mlp.", rms_norm(x1, p[prefix + "norm2.weight"]))
    return x2, h_new, padded[:, 1:, :]


def conv_sequence(b1: torch.Tensor, conv_buf: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None,
                  done: torch.Tensor | None = None):
    """Causal depthwise conv over (R,T,D) with the stored buffer as left padding.

    Tap k of the (D,1,4) weight meets padded[:, t+k], i.e. the input ``3-k`` steps back
    (griffin.py:127-139).  ``done[:, t]`` ends an episode at t: a tap is dropped when an
    episode started between the input it reads and the output step; the stored buffer belongs
    to the episode running at t = 0 (griffin.py:67-93).  Returns (v (R,T,D), last three
    entries of the padded sequence), griffin.py:275-277.
    """
    R, T, D = b1.shape
    padded = torch.cat([conv_buf, b1], dim=1)
    w = weight.reshape(D, CONV_TAPS)
    v = torch.zeros(R, T, D, dtype=padded.dtype)
    if done is not None:
        begins = torch.zeros(R, T + CONV_TAPS - 1, dtype=torch.long)  # 1 where a padded position opens an episode
        begins[:, CONV_TAPS:] = done[:, :-1].long()
        opened = begins.cumsum(dim=1)  # episodes opened up to and including each padded position
    for k in range(CONV_TAPS):
        tap = padded[:, k:k + T] * w[:, k]
        if done is not None:
            inside = opened[:, k:k + T] == opened[:, CONV_TAPS - 1:CONV_TAPS - 1 + T]
            tap = tap * inside.unsqueeze(-1).to(tap.dtype)
        v = v + tap
    if bias is not None:
        v = v + bias
    return v, padded[:, -(CONV_TAPS - 1):, :]


def rglru_sequence(x: torch.Tensor, gates_pre: torch.Tensor, log_lambda: torch.Tensor, c: float, h0: torch.Tensor,
                   done: torch.Tensor | None = None):
    """RG-LRU over (R,T,D) the way the reference evaluates it: per-step a_t, b_t, then a
    log-depth inclusive scan of the pairs under (a2,b2)o(a1,b1) = (a2 a1, a2 b1 + b2).

    Follows griffin.py:206-219 (coefficients; ``a`` is zeroed at the step after an episode
    end) and :25-64 (the scan: pad T to a power of two with the identity (1,0), log2 rounds
    of shifted combines, h_t = A_t h0 + B_t).  Returns (all states (R,T,D), last state).
    """
    R, T, D = x.shape
    r = torch.sigmoid(gates_pre[..., :D])
    i = torch.sigmoid(gates_pre[..., D:])
    a = torch.sigmoid(log_lambda) ** (c * r)
    b = torch.sqrt(torch.clamp((1.0 - a) * (1.0 + a), min=1e-6)) * (i * x)
    if done is not None:
        fresh = torch.zeros(R, T, dtype=torch.bool)
        fresh[:, 1:] = done[:, :-1]
        a = a.masked_fill(fresh.unsqueeze(-1), 0.0)
    width = 1
    while width < T:
        width *= 2
    A = torch.ones(R, width, D, dtype=a.dtype)
    Bc = torch.zeros(R, width, D, dtype=b.dtype)
    A[:, :T], Bc[:, :T] = a, b
    span = 1
    while span < width:
        A_prev = torch.ones_like(A)
        B_prev = torch.zeros_like(Bc)
        A_prev[:, span:], B_prev[:, span:] = A[:, :-span], Bc[:, :-span]
        Bc = A * B_prev + Bc  # uses the not yet updated A
        A = A * A_prev
        span *= 2
    states = (A * h0.unsqueeze(1) + Bc)[:, :T]
    return states, states[:, -1]


def temporal_sequence(
    p: dict,
    prefix: str,
    x_seq: torch.Tensor,
    h0: torch.Tensor,
    conv_buf: torch.Tensor,
    done: torch.Tensor | None = None,
):
    """Same sublayer over (R,T,D), written independently of ``temporal_step``.

    The depthwise causal conv goes through the library ``F.conv1d`` (the reference
    states its tap loop is that cross-correlation, griffin.py:131-134) and the
    recurrence is a plain loop over T, so a wrong tap or buffer order in
    ``temporal_step`` cannot hide here.  ``done`` (R,T) follows griffin.py:213-218:
    done at t cuts the state (and the conv taps reaching back across it,
    griffin.py:67-93) for steps after t.
    """
    R, T, D = x_seq.shape
    n = rms_norm(x_seq, p[prefix + "norm1.weight"])
    b1 = F.linear(n, p[prefix + "linear1.weight"])
    padded = torch.cat([conv_buf, b1], dim=1)  # (R, T+3, D)
    if done is None:
        v = F.conv1d(padded.transpose(1, 2), p[prefix + "conv.weight"], p[prefix + "conv.bias"], groups=D)
        v = v.transpose(1, 2)
    else:
        # episode id of every padded position; a tap contributes only inside one episode
        starts = torch.zeros(R, T, dtype=torch.long)
        starts[:, 1:] = done[:, :-1].long()
        epi = torch.cat([torch.zeros(R, CONV_TAPS - 1, dtype=torch.long), starts.cumsum(1)], dim=1)
        w = p[prefix + "conv.weight"].squeeze(1)
        v = torch.zeros_like(b1)
        for t in range(T):
            for k in range(CONV_TAPS):
                same = (epi[:, t + k] == epi[:, t + CONV_TAPS - 1]).to(b1.dtype).unsqueeze(-1)
                v[:, t] = v[:, t] + padded[:, t + k] * w[:, k] * same
        v = v + p[prefix + "conv.bias"]
    lam = p[prefix + "rg_lru.log_lambda"]
    gates = rglru_gates(p, prefix + "rg_lru.", v)
    h, ys = h0, []
    for t in range(T):
        if done is not None and t > 0:
            h = h * (~done[:, t - 1]).to(h.dtype).unsqueeze(-1)
        h = rglru_step(v[:, t], gates[:, t], lam, 8.0, h)
        ys.append(h)
    y = torch.stack(ys, dim=1)
    b2 = F.gelu(F.linear(n, p[prefix + "linear2.weight"]))
    x1 = x_seq + F.linear(y * b2, p[prefix + "linear_out.weight"])
    x2 = x1 + gated_mlp(p, prefix + "gated_mlp.", rms_norm(x1, p[prefix + "norm2.weight"]))
    return x2, h, padded[:, -(CONV_TAPS - 1):, :]


def field_step(p: dict, prefix: str, sub_weight: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """Temporal sublayer for state-free (field) tokens; models/yemong/griffin.py:288-317."""
    n = rms_norm(x, p[prefix + "norm1.weight"])
    b1 = F.linear(F.linear(n, p[prefix + "linear1.weight"]), sub_weight)
    b2 = F.gelu(F.linear(n, p[prefix + "linear2.weight"]))
    x1 = x + F.linear(b1 * b2, p[prefix + "linear_out.weight"])
    return x1 + gated_mlp(p, prefix + "gated_mlp.", rms_norm(x1, p[prefix + "norm2.weight"]))


def block_step(
    p: dict,
    prefix: str,
    n_spatial: int,
    n_temporal: int,
    n_heads: int,
    x: torch.Tensor,
    alive: torch.Tensor,
    h: torch.Tensor,
    conv_buf: torch.Tensor,
    n_rec: int | None = None,
    bullets: torch.Tensor | None = None,
    bullet_mask: torch.Tensor | None = None,
):
    """One Yemong block for one timestep; models/yemong/griffin.py:376-417.

    x (B,NM,D), alive (B,NM), h (n_temporal, B*n_rec, D), conv_buf
    (n_temporal, B*n_rec, 3, D).  Recurrent rows are env-major (b*n_rec + n).  ``bullets``
    (B,NB,D) / ``bullet_mask`` (B,NB) reach every spatial sublayer (griffin.py:400-401); the
    ones that own ``kv_bullet`` weights read them (attention.py:149).
    """
    B, NM, D = x.shape
    n_rec = NM if n_rec is None else n_rec
    for s in range(n_spatial):
        x = spatial_sublayer(p, f"{prefix}spatial.{s}.", x, alive, n_heads, bullets, bullet_mask)
    hs, cbs = [], []
    for j in range(n_temporal):
        tp = f"{prefix}temporal.{j}."
        ships = x[:, :n_rec].reshape(B * n_rec, D)
        out, h_new, cb_new = temporal_step(p, tp, ships, h[j], conv_buf[j])
        parts = [out.reshape(B, n_rec, D)]
        if NM > n_rec:
            parts.append(field_step(p, tp, p[f"{prefix}field_sub.{j}.weight"], x[:, n_rec:]))
        x = torch.cat(parts, dim=1)
        hs.append(h_new)
        cbs.append(cb_new)
    if not hs:
        return x, h[:0], conv_buf[:0]
    return x, torch.stack(hs), torch.stack(cbs)


def unpack_hidden(hidden: torch.Tensor, d_model: int):
    """(L, R, 4D) -> h (L,R,D), conv_buf (L,R,3,D); models/yemong/policy.py:323-324."""
    L, R, _ = hidden.shape
    return hidden[:, :, :d_model], hidden[:, :, d_model:].reshape(L, R, CONV_TAPS - 1, d_model)


def pack_hidden(h: torch.Tensor, conv_buf: torch.Tensor) -> torch.Tensor:
    """Inverse of ``unpack_hidden``; models/yemong/policy.py:346-354."""
    L, R, D = h.shape
    return torch.cat([h, conv_buf.reshape(L, R, (CONV_TAPS - 1) * D)], dim=-1)


def reset_hidden(hidden: torch.Tensor, done: torch.Tensor, n_rec: int) -> torch.Tensor:
    """Zero every recurrent row of finished environments; models/yemong/policy.py:268-285."""
    keep = (~done.repeat_interleave(n_rec)).to(hidden.dtype)
    return hidden * keep[None, :, None]


def trunk_step(
    p: dict,
    n_blocks: int,
    n_spatial: int,
    n_temporal: int,
    n_heads: int,
    x: torch.Tensor,
    alive: torch.Tensor,
    hidden: torch.Tensor,
    bullets: torch.Tensor | None = None,
    bullet_mask: torch.Tensor | None = None,
):
    """The block loop of ``get_action_and_value``; models/yemong/policy.py:311-354 (bullets handed to
    every block, :327-340)."""
    B, NM, D = x.shape
    n_rec = hidden.shape[1] // B
    h_all, cb_all = unpack_hidden(hidden, D)
    hs, cbs = [], []
    for i in range(n_blocks):
        sl = slice(i * n_temporal, (i + 1) * n_temporal)
        x, h_new, cb_new = block_step(
            p, f"yemong_layers.{i}.", n_spatial, n_temporal, n_heads, x, alive, h_all[sl], cb_all[sl], n_rec,
            bullets, bullet_mask,
        )
        hs.append(h_new)
        cbs.append(cb_new)
    if not hs or hs[0].shape[0] == 0:
        return x, hidden
    return x, pack_hidden(torch.cat(hs), torch.cat(cbs))


# --------------------------------------------------------------------------
# The measured composition (two kernels + the four projections around them)
# --------------------------------------------------------------------------

def harness_step(p: dict, tokens: torch.Tensor, alive: torch.Tensor, state: torch.Tensor, n_heads: int = 4):
    """Minimal attention + RG-LRU step on (B,NM,D) tokens.

    ``p`` holds ``qkv.weight`` (3D,D), ``out_proj.weight`` (D,D), ``linear_a.*``,
    ``linear_x.*`` and ``log_lambda``; ``state`` is (B*N, D) fp32 for the first N
    tokens of every environment (ships); the trailing NM-N tokens (fields) skip
    the recurrence as in models/yemong/griffin.py:406-413.
    Returns (hidden (B,NM,D), new_state (B*N,D)).
    """
    B, NM, D = tokens.shape
    N = state.shape[0] // B
    u = F.linear(sdpa_masked(F.linear(tokens, p["qkv.weight"]), alive, n_heads), p["out_proj.weight"])
    ships = u[:, :N].reshape(B * N, D)
    h_new = rglru_step(ships, rglru_gates(p, "", ships), p["log_lambda"], 8.0, state)
    y = h_new.to(u.dtype).reshape(B, N, D)
    return torch.cat([y, u[:, N:]], dim=1), h_new


def team_pool(p: dict, prefix: str, x: torch.Tensor, team_id: torch.Tensor, alive: torch.Tensor, n_heads: int):
    """Pooling by multi-head attention per team, broadcast back to the ships.

    Follows models/yemong/policy.py:78-120: for team t in {0, 1} the learned seed ``seeds[t]`` is
    the single query of a bias-free multi-head attention whose keys and values are the ship
    rows ``x``, keys restricted to the alive ships of team t; a team without such a ship pools
    to zero; the pooled vector goes through RMSNorm; every ship receives the pooled vector of
    team ``clamp(team_id, 0, 1)``.  Weights: ``{prefix}seeds`` (2, D), ``{prefix}attn.in_proj_weight``
    (3D, D) = [W_q; W_k; W_v], ``{prefix}attn.out_proj.weight`` (D, D), ``{prefix}norm.weight`` (D).
    Returns (ships (B, N, D), pool (B, 2, D)).
    """
    B, N, D = x.shape
    dh = D // n_heads
    w_in = p[prefix + "attn.in_proj_weight"]
    wq, wk, wv = w_in[:D], w_in[D:2 * D], w_in[2 * D:]
    k = F.linear(x, wk).view(B, N, n_heads, dh)
    v = F.linear(x, wv).view(B, N, n_heads, dh)
    pool = x.new_zeros(B, 2, D)
    for t in range(2):
        keys = (team_id == t) & alive  # (B, N)
        q = F.linear(p[prefix + "seeds"][t], wq).view(n_heads, dh)
        scores = torch.einsum("hd,bnhd->bhn", q, k) / math.sqrt(dh)
        scores = scores.masked_fill(~keys[:, None, :], float("-inf"))
        weights = torch.softmax(scores, dim=-1).nan_to_num(0.0)  # no key at all: nothing is pooled
        merged = torch.einsum("bhn,bnhd->bhd", weights, v).reshape(B, D)
        out = F.linear(merged, p[prefix + "attn.out_proj.weight"])
        out = out * keys.any(dim=1, keepdim=True).to(out.dtype)
        pool[:, t] = rms_norm(out, p[prefix + "norm.weight"])
    idx = team_id.clamp(0, 1).long().unsqueeze(-1).expand(B, N, D)
    return pool.gather(1, idx), pool


def sigma_lambda_reference(d_model: int) -> torch.Tensor:
    """log_lambda as the reference initialises it; models/yemong/griffin.py:165."""
    return torch.linspace(0.0, 4.0, d_model)


def softplus_neg(x: float) -> float:
    """log(sigmoid(x)) for a python float, used by closed-form checks."""
    return -math.log1p(math.exp(-x))
