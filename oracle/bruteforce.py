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
