"""Textbook fp64 statements of the two kernels, loops only, for tiny inputs.

TEST INFRASTRUCTURE ONLY (never imported by the product).  These do not call
any attention or recurrence routine: they spell the definitions out with
python loops over numpy float64 scalars so that the torch restatement in
``oracle/torch_ref.py`` and the C restatement in ``oracle/bnb_oracle.c`` can be
checked against something that shares no code with either.
"""

from __future__ import annotations

import math

import numpy as np

F32_MIN_HALF = float(np.finfo(np.float32).min) / 2.0  # additive bias for dead keys, fp32 flavour


def sdpa_masked_loops(qkv: np.ndarray, alive: np.ndarray | None, n_heads: int, neg: float = F32_MIN_HALF) -> np.ndarray:
    """softmax_j(q_i.k_j/sqrt(dh) + bias_j) v_j per (env, head), bias_j = 0 | neg.

    Definition being restated: models/yemong/attention.py:101-112,136-147,168.
    The addition ``score + neg`` is carried out in float32 when ``neg`` is the
    fp32 constant, because that rounding (|score| << ulp(1.7e38)) is what makes
    an all-dead environment come out exactly uniform in the reference.
    """
    qkv = np.asarray(qkv, dtype=np.float64)
    B, NM, D3 = qkv.shape
    D = D3 // 3
    dh = D // n_heads
    out = np.zeros((B, NM, D), dtype=np.float64)
    for b in range(B):
        for hd in range(n_heads):
            lo = hd * dh
            for i in range(NM):
                q = qkv[b, i, lo:lo + dh]
                scores = []
                for j in range(NM):
                    k = qkv[b, j, D + lo:D + lo + dh]
                    s = float(np.dot(q, k)) / math.sqrt(dh)
                    if alive is not None and not alive[b, j]:
                        s = float(np.float32(s) + np.float32(neg))
                    scores.append(s)
                m = max(scores)
                w = [math.exp(s - m) for s in scores]
                z = sum(w)
                for j in range(NM):
                    out[b, i, lo:lo + dh] += (w[j] / z) * qkv[b, j, 2 * D + lo:2 * D + lo + dh]
    return out


def rglru_step_loops(x, gates_pre, log_lambda, c, h) -> np.ndarray:
    """h' = a*h + sqrt(max((1-a)(1+a),1e-6)) * (i*x), a = sigmoid(lambda)^(c*r).

    Definition being restated: models/yemong/griffin.py:150-153,179-186.
    """
    x = np.asarray(x, dtype=np.float64)
    g = np.asarray(gates_pre, dtype=np.float64)
    lam = np.asarray(log_lambda, dtype=np.float64)
    h = np.asarray(h, dtype=np.float64)
    R, D = x.shape
    out = np.zeros((R, D), dtype=np.float64)
    for row in range(R):
        for d in range(D):
            r = 1.0 / (1.0 + math.exp(-g[row, d]))
            i = 1.0 / (1.0 + math.exp(-g[row, D + d]))
            sig = 1.0 / (1.0 + math.exp(-lam[d]))
            a = sig ** (c * r)
            gate = math.sqrt(max((1.0 - a) * (1.0 + a), 1e-6))
            out[row, d] = a * h[row, d] + gate * (i * x[row, d])
    return out


def bullet_read_loops(q: np.ndarray, kv: np.ndarray, active: np.ndarray | None, n_heads: int) -> np.ndarray:
    """Entity queries over bullet keys/values: softmax over the active bullets only, and an
    environment without an active bullet contributes zero.

    Definition being restated: models/yemong/attention.py:149-165.  ``q`` (B, N, D),
    ``kv`` (B, NB, 2D) = [K | V].  With at least one active bullet the finfo.min/2 bias gives
    inactive bullets weight exactly 0, which is what dropping them states.
    """
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    B, N, D = q.shape
    NB = kv.shape[1]
    dh = D // n_heads
    out = np.zeros((B, N, D), dtype=np.float64)
    for b in range(B):
        keys = [j for j in range(NB) if active is None or active[b, j]]
        if not keys:
            continue
        for hd in range(n_heads):
            lo = hd * dh
            for i in range(N):
                scores = [float(np.dot(q[b, i, lo:lo + dh], kv[b, j, lo:lo + dh])) / math.sqrt(dh) for j in keys]
                m = max(scores)
                w = [math.exp(s - m) for s in scores]
                z = sum(w)
                for wj, j in zip(w, keys):
                    out[b, i, lo:lo + dh] += (wj / z) * kv[b, j, D + lo:D + lo + dh]
    return out


def conv_sequence_loops(b1, conv_buf, weight, bias, done) -> np.ndarray:
    """out[r,t] = bias + sum_j w[:,3-j] * input[r,t-j] over the lags j that stay inside the
    episode of step t; inputs before t = 0 come from the stored buffer (same episode as t = 0).

    Definition being restated: models/yemong/griffin.py:67-93 (validity), :127-139 (taps).
    """
    b1 = np.asarray(b1, dtype=np.float64)
    buf = np.asarray(conv_buf, dtype=np.float64)
    w = np.asarray(weight, dtype=np.float64).reshape(b1.shape[-1], 4)
    R, T, D = b1.shape
    out = np.zeros((R, T, D), dtype=np.float64)
    for r in range(R):
        seq = [buf[r, 0], buf[r, 1], buf[r, 2]] + [b1[r, t] for t in range(T)]  # position p holds time p - 3
        for t in range(T):
            acc = np.zeros(D) if bias is None else np.asarray(bias, dtype=np.float64).copy()
            for j in range(4):
                # input at time t-j is in the episode of t iff no episode ended at t-j .. t-1
                crossed = any(done is not None and 0 <= s < T and done[r, s] for s in range(t - j, t))
                if not crossed:
                    acc = acc + w[:, 3 - j] * seq[t - j + 3]
            out[r, t] = acc
    return out


def rglru_sequence_loops(x, gates_pre, log_lambda, c, h0, done) -> np.ndarray:
    """All states of the recurrence over T steps; the state is zero after an episode end.

    Definition being restated: models/yemong/griffin.py:188-219.
    """
    x = np.asarray(x, dtype=np.float64)
    R, T, D = x.shape
    h = np.asarray(h0, dtype=np.float64).copy()
    out = np.zeros((R, T, D), dtype=np.float64)
    for t in range(T):
        if t > 0 and done is not None:
            for r in range(R):
                if done[r, t - 1]:
                    h[r] = 0.0
        h = rglru_step_loops(x[:, t], np.asarray(gates_pre)[:, t], log_lambda, c, h)
        out[:, t] = h
    return out


def ffn_tail_loops(x, delta, norm_w, gate_w, up_w, down_w, eps) -> np.ndarray:
    """s = x + delta; s + Wd (gelu(Wg n) * (Wu n)), n = s / sqrt(mean(s^2) + eps) * norm_w, erf GELU.

    Definition being restated: models/yemong/attention.py:21-37,97-99.
    """
    x = np.asarray(x, dtype=np.float64)
    s = x if delta is None else x + np.asarray(delta, dtype=np.float64)
    R, D = s.shape
    gw, uw, dw = (np.asarray(a, dtype=np.float64) for a in (gate_w, up_w, down_w))
    out = np.zeros((R, D), dtype=np.float64)
    for r in range(R):
        n = s[r] / math.sqrt(float(np.mean(s[r] * s[r])) + eps) * np.asarray(norm_w, dtype=np.float64)
        hidden = np.zeros(gw.shape[0])
        for j in range(gw.shape[0]):
            g = float(np.dot(gw[j], n))
            hidden[j] = 0.5 * g * (1.0 + math.erf(g / math.sqrt(2.0))) * float(np.dot(uw[j], n))
        out[r] = s[r] + dw @ hidden
    return out


def team_pool_loops(x, team_id, alive, seeds, in_proj_weight, out_proj_weight, norm_weight, n_heads, eps) -> np.ndarray:
    """Per team t in {0, 1}: softmax over the alive ships j of team t of (W_q seed_t)_h . (W_k x_j)_h / sqrt(dh),
    weighted sum of (W_v x_j)_h, heads concatenated, W_o, RMSNorm; no such ship: zeros.  Returns the
    pooled vectors (B, 2, D).

    Definition being restated: models/yemong/policy.py:104-116 with torch's multi-head attention
    (packed in-projection [W_q; W_k; W_v], heads = consecutive slices of the projected vectors).
    """
    x = np.asarray(x, dtype=np.float64)
    B, N, D = x.shape
    dh = D // n_heads
    w_in = np.asarray(in_proj_weight, dtype=np.float64)
    wq, wk, wv = w_in[:D], w_in[D:2 * D], w_in[2 * D:]
    wo = np.asarray(out_proj_weight, dtype=np.float64)
    pool = np.zeros((B, 2, D), dtype=np.float64)
    for b in range(B):
        for t in range(2):
            keys = [j for j in range(N) if int(team_id[b, j]) == t and bool(alive[b, j])]
            if not keys:
                continue
            q = wq @ np.asarray(seeds[t], dtype=np.float64)
            merged = np.zeros(D)
            for hd in range(n_heads):
                lo, hi = hd * dh, (hd + 1) * dh
                scores = [float(np.dot(q[lo:hi], (wk @ x[b, j])[lo:hi])) / math.sqrt(dh) for j in keys]
                m = max(scores)
                w = [math.exp(sc - m) for sc in scores]
                z = sum(w)
                for wj, j in zip(w, keys):
                    merged[lo:hi] += (wj / z) * (wv @ x[b, j])[lo:hi]
            out = wo @ merged
            pool[b, t] = out / math.sqrt(float(np.mean(out * out)) + eps) * np.asarray(norm_weight, dtype=np.float64)
    return pool


# --------------------------------------------------------------------------
# gradients of the update path, written out (not differentiated by a library)
# --------------------------------------------------------------------------

def sdpa_masked_grad_loops(qkv: np.ndarray, alive: np.ndarray | None, n_heads: int, dout: np.ndarray) -> np.ndarray:
    """d(qkv) of ``sdpa_masked_loops`` for the output gradient ``dout`` (B, NM, D), float64.

    Per environment and head, with P the weights the forward used (masked softmax; 1/NM for
    every key when no key is alive, which is what equal biases on all keys evaluate to):
        dV = P^T dO,  dP = dO V^T,  dS = P * (dP - rowsum(P * dP)),
        dQ = dS K / sqrt(dh),  dK = dS^T Q / sqrt(dh).
    Chain rule through models/yemong/attention.py:136-147 written out by hand.
    """
    qkv = np.asarray(qkv, dtype=np.float64)
    dout = np.asarray(dout, dtype=np.float64)
    B, NM, D3 = qkv.shape
    D = D3 // 3
    dh = D // n_heads
    grad = np.zeros_like(qkv)
    for b in range(B):
        live = np.ones(NM, dtype=bool) if alive is None else np.asarray(alive[b], dtype=bool)
        uniform = not live.any()
        for h in range(n_heads):
            cols = slice(h * dh, (h + 1) * dh)
            Q, K, V = qkv[b, :, cols], qkv[b, :, D:][:, cols], qkv[b, :, 2 * D:][:, cols]
            dO = dout[b, :, cols]
            P = np.zeros((NM, NM))
            for i in range(NM):
                if uniform:
                    P[i, :] = 1.0 / NM
                    continue
                s = np.array([np.dot(Q[i], K[j]) / math.sqrt(dh) if live[j] else -np.inf for j in range(NM)])
                e = np.exp(s - s[live].max())
                e[~live] = 0.0
                P[i] = e / e.sum()
            dP = dO @ V.T
            dS = P * (dP - (P * dP).sum(axis=1, keepdims=True))
            grad[b, :, cols] = dS @ K / math.sqrt(dh)
            grad[b, :, D:][:, cols] = dS.T @ Q / math.sqrt(dh)
            grad[b, :, 2 * D:][:, cols] = P.T @ dO
    return grad


def conv_sequence_grad_loops(b1, conv_buf, weight, done, dv, dtail=None):
    """Gradients ``(db1, dconv_buf, dweight (D, 4), dbias (D,))`` of ``conv_sequence_loops`` for the output
    gradient ``dv`` (R, T, D) and the gradient ``dtail`` (R, 3, D) of the three inputs handed on
    (the last three of [conv_buf, b1], models/yemong/griffin.py:277), float64: every term
    ``w[:, 3-j] * input[t-j]`` of the forward sends ``dv[t] * w`` to its input and ``dv[t] * input``
    to its tap."""
    b1 = np.asarray(b1, dtype=np.float64)
    buf = np.asarray(conv_buf, dtype=np.float64)
    dv = np.asarray(dv, dtype=np.float64)
    R, T, D = b1.shape
    w = np.asarray(weight, dtype=np.float64).reshape(D, 4)
    dseq = np.zeros((R, T + 3, D))  # position p = time p - 3
    dw = np.zeros((D, 4))
    for r in range(R):
        seq = np.concatenate([buf[r], b1[r]], axis=0)
        for t in range(T):
            for j in range(4):
                crossed = any(done is not None and 0 <= s < T and done[r, s] for s in range(t - j, t))
                if not crossed:
                    dseq[r, t - j + 3] += dv[r, t] * w[:, 3 - j]
                    dw[:, 3 - j] += dv[r, t] * seq[t - j + 3]
        if dtail is not None:
            dseq[r, T:] += np.asarray(dtail[r], dtype=np.float64)
    return dseq[:, 3:], dseq[:, :3], dw, dv.sum(axis=(0, 1))


def rms_norm_grad_loops(x, weight, eps, dy):
    """``(dx, dweight)`` of ``y = x * rsqrt(mean(x^2) + eps) * weight`` (nn.RMSNorm, attention.py:60,73), float64,
    row by row from the quotient rule."""
    x = np.asarray(x, dtype=np.float64)
    w = np.asarray(weight, dtype=np.float64)
    dy = np.asarray(dy, dtype=np.float64)
    R, D = x.shape
    dx = np.zeros_like(x)
    dw = np.zeros(D)
    for r in range(R):
        ms = float(np.dot(x[r], x[r])) / D + eps
        rstd = 1.0 / math.sqrt(ms)
        g = dy[r] * w
        dx[r] = g * rstd - x[r] * (float(np.dot(g, x[r])) / D) * rstd ** 3
        dw += dy[r] * x[r] * rstd
    return dx, dw


def bullet_read_grad_loops(q: np.ndarray, kv: np.ndarray, active: np.ndarray | None, n_heads: int, dout: np.ndarray):
    """``(dq (B, N, D), dkv (B, NB, 2D))`` of ``bullet_read_loops`` for the output gradient ``dout``, float64: the same
    chain rule as ``sdpa_masked_grad_loops`` over the active bullets only; an environment without an active bullet
    was gated to zero (models/yemong/attention.py:161-164), so nothing flows back from it."""
    q = np.asarray(q, dtype=np.float64)
    kv = np.asarray(kv, dtype=np.float64)
    dout = np.asarray(dout, dtype=np.float64)
    B, N, D = q.shape
    dh = D // n_heads
    dq = np.zeros_like(q)
    dkv = np.zeros_like(kv)
    for b in range(B):
        keys = [j for j in range(kv.shape[1]) if active is None or active[b, j]]
        if not keys:
            continue
        for hd in range(n_heads):
            cols = slice(hd * dh, (hd + 1) * dh)
            Q, K, V, dO = q[b, :, cols], kv[b, keys][:, cols], kv[b, keys][:, D:][:, cols], dout[b, :, cols]
            S = Q @ K.T / math.sqrt(dh)
            E = np.exp(S - S.max(axis=1, keepdims=True))
            P = E / E.sum(axis=1, keepdims=True)
            dP = dO @ V.T
            dS = P * (dP - (P * dP).sum(axis=1, keepdims=True))
            dq[b, :, cols] = dS @ K / math.sqrt(dh)
            dK, dV = dS.T @ Q / math.sqrt(dh), P.T @ dO
            for n, j in enumerate(keys):
                dkv[b, j, cols] = dK[n]
                dkv[b, j, D:][cols] = dV[n]
    return dq, dkv
