"""Committed vectors (tests/golden/step_vectors.npz) against the oracle on the CPU and against
the HIP kernels on the GPU.  The vectors are fp64 answers of the loop-only statements for small
seeded inputs, including an all-dead and a single-live-key environment and saturated gates."""

import os

import numpy as np
import pytest
import torch

from helpers import ROOT, max_rel
from oracle import c_ref, torch_ref

GOLD = np.load(os.path.join(ROOT, "tests", "golden", "step_vectors.npz"))
ATTN = ("attn_4v4", "attn_8v11", "attn_odd")


@pytest.mark.parametrize("tag", ATTN)
def test_oracles_reproduce_attention_vectors(tag):
    qkv, alive, H = GOLD[f"{tag}_qkv"], GOLD[f"{tag}_alive"], int(GOLD[f"{tag}_heads"])
    want = GOLD[f"{tag}_out"]
    got_t = torch_ref.sdpa_masked(torch.from_numpy(qkv), torch.from_numpy(alive), H).double().numpy()
    got_c = c_ref.sdpa_masked(qkv, alive, H).astype(np.float64)
    assert np.abs(got_t - want).max() <= 5e-6 and np.abs(got_c - want).max() <= 5e-7
    D = qkv.shape[-1] // 3
    assert np.abs(want[0] - qkv[0, :, 2 * D:].astype(np.float64).mean(0)).max() <= 1e-6  # all dead: mean of V
    assert np.abs(want[1] - qkv[1, qkv.shape[1] // 2, 2 * D:]).max() <= 1e-6  # single live key: its V row


def test_oracles_reproduce_rglru_vectors():
    x, g, h, lam = (GOLD[k] for k in ("rglru_x", "rglru_gates", "rglru_h", "rglru_lambda"))
    want = GOLD["rglru_out"]
    got_t = torch_ref.rglru_step(*(torch.from_numpy(a) for a in (x, g, lam)), 8.0, torch.from_numpy(h)).double().numpy()
    assert np.abs(got_t - want).max() <= 5e-6
    assert np.abs(c_ref.rglru_step(x, g, lam, 8.0, h) - want).max() <= 5e-7
    assert np.abs(want[0] - (h[0] + 1e-3 * x[0] / (1 + np.exp(-g[0, 128:].astype(np.float64))))).max() <= 1e-6  # clamp floor row


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ATTN)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_kernels_reproduce_attention_vectors(tag, dtype):
    from boost_and_broadside_amd import ops

    qkv = torch.from_numpy(GOLD[f"{tag}_qkv"]).to(dtype)
    alive, H = torch.from_numpy(GOLD[f"{tag}_alive"]), int(GOLD[f"{tag}_heads"])
    got = ops.sdpa_masked(qkv.cuda(), alive.cuda(), H).float().cpu()
    if dtype == torch.float32:
        assert max_rel(got, torch.from_numpy(GOLD[f"{tag}_out"])) <= 1e-5
    else:  # bf16 inputs differ from the stored fp32 ones by their rounding: compare on the rounded inputs
        truth = torch_ref.sdpa_masked(qkv.float(), alive, H)
        assert max_rel(got, truth) <= 2e-2
        assert max_rel(got, torch.from_numpy(GOLD[f"{tag}_out"]).float()) <= 3e-2


@pytest.mark.gpu
def test_kernels_reproduce_rglru_vectors():
    from boost_and_broadside_amd import ops

    x, g, h, lam = (torch.from_numpy(GOLD[k]).cuda() for k in ("rglru_x", "rglru_gates", "rglru_h", "rglru_lambda"))
    _, got = ops.rglru_step(x, g, lam, 8.0, h)
    assert max_rel(got.cpu(), torch.from_numpy(GOLD["rglru_out"])) <= 1e-5
