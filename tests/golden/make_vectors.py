"""Writes tests/golden/step_vectors.npz: small seeded inputs and their expected outputs.

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


if __name__ == "__main__":
    main()
