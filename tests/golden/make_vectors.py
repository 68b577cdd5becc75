"""Writes tests/golden/step_vectors.npz, widened_vectors.npz, team_pool_vectors.npz and update_vectors.npz:
small seeded inputs and their expected outputs (update_vectors: expected gradients).

The reference keeps no stored numeric vectors for this path (its tests are property tests and
its one golden file needs weights that are not in the checkout), and the reference was not
imported.  These vectors come from the fp64 loop-only statements in oracle/bruteforce.py, so
they freeze the checked oracle's answers: a later change to the oracle, the kernels or the
host code that moves a result shows up against committed data, not against itself.

Run from the repository root:  python tests/golden/make_vectors.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import bruteforce  # noqa: E402


def main() -> None:
    rng = np.random.default_rng(20240601)
    out = {}
    # masked attention: (B, NM, H, dh) with mixed masks, one all-dead and one single-live environment
    for tag, (B, NM, H, dh) in {"attn_4v4": (4, 12, 4, 32), "attn_8v11": (3, 23, 4, 32), "attn_odd": (2, 7, 2, 16)}.items():
        D = H * dh
        qkv = rng.standard_normal((B, NM, 3 * D)).astype(np.float32)
        alive = rng.random((B, NM)) < 0.7
        alive[0] = False
        alive[1] = False
        alive[1, NM // 2] = True
        out[f"{tag}_qkv"] = qkv
        out[f"{tag}_alive"] = alive
        out[f"{tag}_heads"] = np.int64(H)
        out[f"{tag}_out"] = bruteforce.sdpa_masked_loops(qkv, alive, H)
    # RG-LRU step: D = 128 reference initialisation of log_lambda, gates spanning saturation
    R, D = 6, 128
    x = rng.standard_normal((R, D)).astype(np.float32)
    gates = (3.0 * rng.standard_normal((R, 2 * D))).astype(np.float32)
    gates[0, :D] = -40.0  # r -> 0: a = 1, clamp floor
    gates[1, :D] = 40.0   # r -> 1
    h = (0.5 * rng.standard_normal((R, D))).astype(np.float32)
    lam = np.linspace(0.0, 4.0, D, dtype=np.float32)
    out["rglru_x"], out["rglru_gates"], out["rglru_h"], out["rglru_lambda"] = x, gates, h, lam
    out["rglru_out"] = bruteforce.rglru_step_loops(x, gates, lam, 8.0, h)
    np.savez_compressed(os.path.join(HERE, "step_vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "step_vectors.npz"), {k: v.shape for k, v in out.items()})
    widened()
    team_pool()
    update()


def widened() -> None:
    """tests/golden/widened_vectors.npz: bullet read, sequence path and the sublayer tail."""
    rng = np.random.default_rng(20240602)
    out = {}

    def bf16(a):
        """Round to bfloat16 (nearest even), returned as float32."""
        u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
        u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
        return u.view(np.float32)

    def bits(a):
        """bfloat16-exact float32 array -> its 16-bit patterns (halves the file)."""
        return (np.ascontiguousarray(a, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)

    # bullet read: env 0 has nothing in flight, env 1 a single bullet; 176 slots exercise the streamed path
    for tag, (B, N, NB, H, dh) in {"read_small": (3, 6, 20, 4, 32), "read_long": (3, 5, 176, 4, 32)}.items():
        D = H * dh
        q = bf16(rng.standard_normal((B, N, D)))
        kv = bf16(rng.standard_normal((B, NB, 2 * D)))
        active = rng.random((B, NB)) < 0.4
        active[0] = False
        active[1] = False
        active[1, NB - 1] = True
        out[f"{tag}_q_bf16"], out[f"{tag}_kv_bf16"], out[f"{tag}_active"] = bits(q), bits(kv), active
        out[f"{tag}_heads"] = np.int64(H)
        out[f"{tag}_out"] = bruteforce.bullet_read_loops(q, kv, active, H)
    # sequence path: conv with episode ends, recurrence with resets (T = 9 crosses the 4-step load groups)
    R, T, D = 4, 9, 128
    done = rng.random((R, T)) < 0.25
    done[0] = False
    done[1, 0] = True
    b1 = rng.standard_normal((R, T, D)).astype(np.float32)
    buf = rng.standard_normal((R, 3, D)).astype(np.float32)
    w = (0.5 * rng.standard_normal((D, 1, 4))).astype(np.float32)
    bias = (0.1 * rng.standard_normal(D)).astype(np.float32)
    out["seq_done"], out["conv_b1"], out["conv_buf"], out["conv_w"], out["conv_bias"] = done, b1, buf, w, bias
    out["conv_out"] = bruteforce.conv_sequence_loops(b1, buf, w, bias, done)
    x = rng.standard_normal((R, T, D)).astype(np.float32)
    gates = (2.0 * rng.standard_normal((R, T, 2 * D))).astype(np.float32)
    h0 = (0.5 * rng.standard_normal((R, D))).astype(np.float32)
    lam = np.linspace(0.0, 4.0, D, dtype=np.float32)
    out["scan_x"], out["scan_gates"], out["scan_h0"], out["scan_lambda"] = x, gates, h0, lam
    out["scan_out"] = bruteforce.rglru_sequence_loops(x, gates, lam, 8.0, h0, done)
    # sublayer tail: weights already rounded to bf16 so that fp32 and bf16 paths see the same numbers
    R, D, Hd = 5, 128, 512
    out["ffn_x"] = rng.standard_normal((R, D)).astype(np.float32)
    delta = bf16(0.5 * rng.standard_normal((R, D)))
    out["ffn_norm_w"] = (1.0 + 0.1 * rng.standard_normal(D)).astype(np.float32)
    gw = bf16(rng.standard_normal((Hd, D)) / np.sqrt(D))
    uw = bf16(rng.standard_normal((Hd, D)) / np.sqrt(D))
    dw = bf16(rng.standard_normal((D, Hd)) / np.sqrt(Hd))
    out["ffn_delta_bf16"], out["ffn_gate_w_bf16"], out["ffn_up_w_bf16"], out["ffn_down_w_bf16"] = (
        bits(delta), bits(gw), bits(uw), bits(dw))
    out["ffn_out"] = bruteforce.ffn_tail_loops(out["ffn_x"], delta, out["ffn_norm_w"], gw, uw, dw,
                                               float(np.finfo(np.float32).eps))
    np.savez_compressed(os.path.join(HERE, "widened_vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "widened_vectors.npz"), {k: v.shape for k, v in out.items()})


def team_pool() -> None:
    """tests/golden/team_pool_vectors.npz: per-team attention pooling (policy.py:78-120)."""
    rng = np.random.default_rng(20240603)
    B, N, D, H = 4, 9, 128, 4
    out = {
        "x": rng.standard_normal((B, N, D)).astype(np.float32),
        "team_id": rng.integers(0, 2, (B, N)).astype(np.int32),
        "alive": rng.random((B, N)) < 0.7,
        "seeds": (0.5 * rng.standard_normal((2, D))).astype(np.float32),
        "in_proj_weight": (rng.standard_normal((3 * D, D)) * np.sqrt(2.0 / D)).astype(np.float32),
        "out_proj_weight": (rng.standard_normal((D, D)) / np.sqrt(D)).astype(np.float32),
        "norm_weight": (1.0 + 0.1 * rng.standard_normal(D)).astype(np.float32),
        "heads": np.int64(H),
    }
    out["team_id"][0] = 0       # nobody on team 1
    out["alive"][1] = False     # everybody dead
    out["alive"][2] = False
    out["alive"][2, 4] = True   # a single ship alive
    out["team_id"][3, 0] = 2    # a field id among the ships: nobody's key, reads team 1's vector
    out["pool"] = bruteforce.team_pool_loops(out["x"], out["team_id"], out["alive"], out["seeds"], out["in_proj_weight"],
                                             out["out_proj_weight"], out["norm_weight"], H, float(np.finfo(np.float32).eps))
    np.savez_compressed(os.path.join(HERE, "team_pool_vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "team_pool_vectors.npz"), {k: v.shape for k, v in out.items()})




def update() -> None:
    """tests/golden/update_vectors.npz: gradients of the update path from the hand-written chain rules."""
    rng = np.random.default_rng(20240604)
    out = {}

    def bf16(a):
        u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
        return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)  # round to nearest even

    # attention backward: inputs already bf16-representable so that both dtypes see the same numbers
    for tag, (B, NM, H) in {"attn_4v4": (4, 12, 4), "attn_8v11": (3, 23, 4), "attn_wide": (2, 40, 4)}.items():
        D = 32 * H
        qkv = bf16(1.2 * rng.standard_normal((B, NM, 3 * D)))
        alive = rng.random((B, NM)) < 0.7
        alive[0] = False
        alive[1] = False
        alive[1, NM // 2] = True
        dout = bf16(rng.standard_normal((B, NM, D)))
        out[f"{tag}_qkv"], out[f"{tag}_alive"], out[f"{tag}_heads"], out[f"{tag}_dout"] = qkv, alive, np.int64(H), dout
        out[f"{tag}_dqkv"] = bruteforce.sdpa_masked_grad_loops(qkv, alive, H, dout)
    # bullet read backward: one environment without an active bullet, one with a single one
    for tag, (B, N, NB, H) in {"cross_4v4": (4, 12, 80, 4), "cross_wide": (2, 40, 33, 4)}.items():
        D = 32 * H
        qkv = bf16(1.2 * rng.standard_normal((B, N, 3 * D)))
        kv = bf16(1.2 * rng.standard_normal((B, NB, 2 * D)))
        active = rng.random((B, NB)) < 0.3
        active[0] = False
        active[1] = False
        active[1, NB // 3] = True
        dout = bf16(rng.standard_normal((B, N, D)))
        dq, dkv = bruteforce.bullet_read_grad_loops(qkv[..., :D], kv, active, H, dout)
        out.update({f"{tag}_qkv": qkv, f"{tag}_kv": kv, f"{tag}_active": active, f"{tag}_heads": np.int64(H), f"{tag}_dout": dout,
                    f"{tag}_dq": dq, f"{tag}_dkv": dkv})
    # the same over a long slot axis (more live bullets than one 160-key tile of the backward kernels), from its
    # own generator so that the vectors above and below do not depend on it
    rng_long = np.random.default_rng(20260)
    B, N, NB, H = 3, 12, 200, 1
    D = 32 * H
    qkv = bf16(1.2 * rng_long.standard_normal((B, N, 3 * D)))
    kv = bf16(1.2 * rng_long.standard_normal((B, NB, 2 * D)))
    active = rng_long.random((B, NB)) < 0.9
    active[0] = False
    active[1] = False
    active[1, NB // 3] = True
    dout = bf16(rng_long.standard_normal((B, N, D)))
    dq, dkv = bruteforce.bullet_read_grad_loops(qkv[..., :D], kv, active, H, dout)
    out.update({"cross_long_qkv": qkv, "cross_long_kv": kv, "cross_long_active": active, "cross_long_heads": np.int64(H),
                "cross_long_dout": dout, "cross_long_dq": dq, "cross_long_dkv": dkv})
    # sequence conv backward with episode ends and a gradient on the handed-on inputs
    R, T, D = 5, 11, 128
    b1 = bf16(rng.standard_normal((R, T, D)))
    buf = rng.standard_normal((R, 3, D)).astype(np.float32)
    w = (0.5 * rng.standard_normal((D, 1, 4))).astype(np.float32)
    done = rng.random((R, T)) < 0.25
    dv = rng.standard_normal((R, T, D)).astype(np.float32)
    dtail = rng.standard_normal((R, 3, D)).astype(np.float32)
    g = bruteforce.conv_sequence_grad_loops(b1, buf, w, done, dv, dtail)
    out.update(conv_b1=b1, conv_buf=buf, conv_w=w, conv_done=done, conv_dv=dv, conv_dtail=dtail,
               conv_db1=g[0], conv_dbuf=g[1], conv_dw=g[2], conv_dbias=g[3])
    # RMSNorm backward
    R, D = 9, 128
    x = (rng.standard_normal((R, D)) * (0.2 + 3.0 * rng.random((R, 1)))).astype(np.float32)
    nw = (1.0 + 0.3 * rng.standard_normal(D)).astype(np.float32)
    dy = bf16(rng.standard_normal((R, D)))
    eps = float(np.finfo(np.float32).eps)
    gx, gw = bruteforce.rms_norm_grad_loops(x, nw, eps, dy)
    out.update(norm_x=x, norm_w=nw, norm_dy=dy, norm_dx=gx, norm_dw=gw)
    np.savez_compressed(os.path.join(HERE, "update_vectors.npz"), **out)
    print("wrote", os.path.join(HERE, "update_vectors.npz"), {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
