"""Parity of the two HIP kernels (through the C ABI) against the CPU oracle.

Bars: float32 max relative error <= 1e-5, bfloat16 <= 2e-2 (both as max|y-ref|/max|ref|
against the float32 oracle evaluated on the same, already rounded, inputs), identical
alive-masking behaviour (dead keys weigh exactly nothing, an all-dead environment is the
mean of V, dead queries are computed).
"""

import math

import numpy as np
import pytest
import torch

from helpers import max_rel, team_case, team_pool_params
from oracle import bruteforce, c_ref, torch_ref

from boost_and_broadside_amd import harness, ops

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 2e-2
DEV = "cuda:0"


def _qkv(seed, B, NM, D, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(B, NM, 3 * D, generator=g)).to(dtype)


def _alive(seed, B, NM, p):
    g = torch.Generator().manual_seed(seed + 99)
    return torch.rand(B, NM, generator=g) < p


def _run_sdpa(qkv, alive, H, path="auto"):
    out = ops.sdpa_masked(qkv.to(DEV), None if alive is None else alive.to(DEV), H, path=path)
    torch.cuda.synchronize()
    return out.cpu()


# ------------------------------------------------------------------ masked attention, fp32


@pytest.mark.parametrize(
    "B,NM,H,dh",
    [(3, 12, 4, 32), (5, 23, 4, 32), (2, 1, 4, 32), (7, 8, 4, 32), (2, 31, 4, 32), (3, 84, 4, 32),
     (2, 160, 4, 32), (1, 200, 4, 32), (4, 9, 4, 16), (4, 6, 4, 8), (2, 10, 2, 64), (65, 12, 4, 32)],
)
def test_sdpa_fp32_matches_oracle(B, NM, H, dh):
    qkv = _qkv(B * 1000 + NM, B, NM, H * dh, torch.float32)
    alive = _alive(NM, B, NM, 0.75)
    alive[:, 0] = True
    got = _run_sdpa(qkv, alive, H)
    ref = torch_ref.sdpa_masked(qkv, alive, H)
    assert max_rel(got, ref) <= F32_TOL
    assert torch.allclose(got, ref, rtol=1e-4, atol=2e-6)
    if B * NM * NM <= 40000:  # the plain-C statement as a second, torch-free witness
        cc = torch.from_numpy(c_ref.sdpa_masked(qkv.numpy(), alive.numpy(), H))
        assert max_rel(got, cc) <= F32_TOL


@pytest.mark.parametrize("NM", [33, 63, 64, 65, 100, 160, 161, 255, 320, 512])
def test_sdpa_fp32_matrix_core_kernel_matches_oracle_and_the_vector_kernel(NM):
    # fp32 with head size 32 and more than 32 tokens runs on the fp32 matrix-core kernel (AUTO);
    # path="valu" forces the vector kernel on the same inputs
    B, H, D = 5, 4, 128
    qkv = _qkv(NM * 3, B, NM, D, torch.float32, scale=1.5)
    alive = _alive(NM, B, NM, 0.6)
    alive[0] = True
    alive[1] = False            # nobody alive: mean of V
    alive[2] = False
    alive[2, NM - 1] = True     # a single key
    got = _run_sdpa(qkv, alive, H)
    ref = torch_ref.sdpa_masked(qkv, alive, H)
    assert max_rel(got, ref) <= F32_TOL
    assert torch.allclose(got, ref, rtol=1e-4, atol=2e-6)
    assert max_rel(got, _run_sdpa(qkv, alive, H, "valu")) <= F32_TOL
    assert (got[1] - qkv[1, :, 2 * D:].mean(dim=0, keepdim=True)).abs().max() <= 2e-6
    assert torch.allclose(got[2], qkv[2, NM - 1, 2 * D:].expand(NM, D), atol=1e-6)
    # dead keys weigh exactly nothing
    pert = qkv.clone()
    dead = ~alive
    dead[1] = False
    pert[..., D:][dead] = pert[..., D:][dead] * -3.0 + 17.0
    assert torch.equal(_run_sdpa(pert, alive, H), got)
    # padded rows (a view of a wider buffer) and no mask at all
    wide = torch.zeros(B, NM, 3 * D + 64)
    wide[..., : 3 * D] = qkv
    view = wide.to(DEV)[..., : 3 * D]
    assert torch.equal(ops.sdpa_masked(view, alive.to(DEV), H).cpu(), got)
    assert max_rel(_run_sdpa(qkv, None, H), torch_ref.sdpa_masked(qkv, None, H)) <= F32_TOL


def test_sdpa_fp32_large_scores_stay_exact():
    # scores of magnitude ~50 exercise the running-max rescaling
    qkv = _qkv(5, 4, 23, 128, torch.float32, scale=3.0)
    alive = _alive(5, 4, 23, 0.6)
    alive[:, 3] = True
    assert max_rel(_run_sdpa(qkv, alive, 4), torch_ref.sdpa_masked(qkv, alive, 4)) <= F32_TOL


def test_sdpa_no_mask_equals_all_alive():
    qkv = _qkv(6, 3, 12, 128, torch.float32)
    a = _run_sdpa(qkv, None, 4)
    b = _run_sdpa(qkv, torch.ones(3, 12, dtype=torch.bool), 4)
    assert torch.equal(a, b)
    assert max_rel(a, torch_ref.sdpa_masked(qkv, None, 4)) <= F32_TOL


@pytest.mark.parametrize("dtype,path,NM", [(torch.float32, "valu", 12), (torch.bfloat16, "valu", 12),
                                          (torch.bfloat16, "mfma", 84), (torch.bfloat16, "mfma", 160)])
def test_all_dead_environment_is_mean_of_values(dtype, path, NM):
    B, H, D = 3, 4, 128
    qkv = _qkv(7, B, NM, D, dtype)
    alive = torch.ones(B, NM, dtype=torch.bool)
    alive[1] = False  # everyone dead in env 1
    got = _run_sdpa(qkv, alive, H, path).float()
    assert torch.isfinite(got).all()
    mean_v = qkv[1, :, 2 * D:].float().mean(dim=0, keepdim=True).expand(NM, D)
    tol = 2e-6 if dtype == torch.float32 else 1.6e-2
    assert (got[1] - mean_v).abs().max() <= tol
    ref = torch_ref.sdpa_masked(qkv.float(), alive, H)
    assert max_rel(got, ref) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)


@pytest.mark.parametrize("dtype,path,NM", [(torch.float32, "valu", 12), (torch.bfloat16, "valu", 23),
                                          (torch.bfloat16, "mfma", 84), (torch.bfloat16, "mfma", 33)])
def test_dead_keys_have_exactly_zero_weight(dtype, path, NM):
    B, H, D = 4, 4, 128
    qkv = _qkv(8, B, NM, D, dtype)
    alive = _alive(8, B, NM, 0.6)
    alive[:, 1] = True
    base = _run_sdpa(qkv, alive, H, path)
    pert = qkv.clone()
    dead = ~alive
    pert[..., D:][dead] = pert[..., D:][dead] * -3.0 + 17.0  # K and V rows of dead tokens only
    again = _run_sdpa(pert, alive, H, path)
    assert torch.equal(base, again)
    assert base[dead].float().abs().max() > 0  # dead queries still produce rows


def test_single_live_key_broadcasts_its_value_row():
    B, NM, H, D = 2, 12, 4, 128
    qkv = _qkv(9, B, NM, D, torch.float32)
    alive = torch.zeros(B, NM, dtype=torch.bool)
    alive[0, 7] = True
    alive[1, 0] = True
    got = _run_sdpa(qkv, alive, H)
    assert torch.allclose(got[0], qkv[0, 7, 2 * D:].expand(NM, D), atol=1e-6)
    assert torch.allclose(got[1], qkv[1, 0, 2 * D:].expand(NM, D), atol=1e-6)


def test_sdpa_accepts_padded_rows_and_uint8_mask():
    B, NM, H, D = 3, 12, 4, 128
    qkv = _qkv(10, B, NM, D, torch.float32)
    wide = torch.zeros(B, NM, 3 * D + 64)
    wide[..., : 3 * D] = qkv
    alive = _alive(10, B, NM, 0.7)
    alive[:, 2] = True
    view = wide.to(DEV)[..., : 3 * D]  # row stride 448 elements
    got = ops.sdpa_masked(view, alive.to(DEV).to(torch.uint8), H).cpu()
    assert max_rel(got, torch_ref.sdpa_masked(qkv, alive, H)) <= F32_TOL


def test_sdpa_empty_and_rejected_inputs():
    assert ops.sdpa_masked(torch.zeros(0, 12, 384, device=DEV), None, 4).shape == (0, 12, 128)
    assert ops.sdpa_masked(torch.zeros(2, 0, 384, device=DEV), None, 4).shape == (2, 0, 128)
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.sdpa_masked(torch.zeros(1, 4, 3 * 4 * 24, device=DEV), None, 4)  # head_dim 24
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.sdpa_masked(torch.zeros(1, 600, 384, device=DEV), None, 4)  # more tokens than supported
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.sdpa_masked(torch.zeros(1, 12, 384, device=DEV), None, 4, path="mfma")  # fp32 on the bf16 kernel
    with pytest.raises(TypeError):
        ops.sdpa_masked(torch.zeros(1, 4, 384, device=DEV, dtype=torch.float16), None, 4)


# ------------------------------------------------------------------ masked attention, bf16


@pytest.mark.parametrize(
    "B,NM,path",
    [(5, 12, "valu"), (4, 23, "valu"), (3, 31, "valu"), (3, 12, "mfma"), (3, 23, "mfma"), (3, 32, "mfma"),
     (3, 33, "mfma"), (4, 84, "mfma"), (3, 96, "mfma"), (2, 129, "mfma"), (3, 160, "mfma"), (2, 160, "valu"),
     (3, 84, "auto"), (9, 12, "auto")],
)
def test_sdpa_bf16_matches_fp32_oracle(B, NM, path):
    H, D = 4, 128
    qkv = _qkv(B * 77 + NM, B, NM, D, torch.bfloat16)
    alive = _alive(NM + 1, B, NM, 0.7)
    alive[:, NM // 2] = True
    got = _run_sdpa(qkv, alive, H, path)
    assert got.dtype == torch.bfloat16
    truth = torch_ref.sdpa_masked(qkv.float(), alive, H)
    assert max_rel(got.float(), truth) <= BF16_TOL
    # no worse than the reference's own bf16 path (library SDPA on bf16 tensors) by more than rounding
    lib16 = torch_ref.sdpa_masked(qkv, alive, H).float()
    assert max_rel(got.float(), truth) <= max_rel(lib16, truth) + 8e-3


@pytest.mark.parametrize("NM,path", [(12, "mfma"), (12, "auto"), (84, "mfma"), (160, "mfma"), (84, "env"), (84, "head"), (160, "head")])
@pytest.mark.parametrize("case", ["large", "huge", "all_negative", "mixed"])
def test_sdpa_bf16_scores_beyond_the_exponent_range_take_the_shifted_sweep(NM, path, case):
    """The matrix-core kernels first form the weights without subtracting the maximum; scores whose weights leave
    float32's safe range (|score| / sqrt(dh) beyond ~40) must fall back to the shifted form and stay at the bar."""
    B, H, D = 4, 4, 128
    g = torch.Generator().manual_seed(NM + len(case))
    qkv = torch.randn(B, NM, 3 * D, generator=g)
    if case == "large":        # weights up to 2^150: overflow without the shift
        qkv[..., : 2 * D] *= 6.0
    elif case == "huge":       # nearly one-hot rows
        qkv[..., : 2 * D] *= 40.0
    elif case == "all_negative":
        # every key points against every query: all weights underflow without the shift, yet they differ by O(1)
        u = torch.randn(H, 32, generator=g)
        u = u / u.norm(dim=-1, keepdim=True)
        k = 30.0 * u.view(1, 1, H, 32) + 0.3 * torch.randn(B, NM, H, 32, generator=g)
        qkv[..., D:2 * D] = k.reshape(B, NM, D)
        qkv[..., :D] = (-30.0 * u.view(1, 1, H, 32) + 0.3 * torch.randn(B, NM, H, 32, generator=g)).reshape(B, NM, D)
    else:                      # one environment out of range, the others ordinary: the choice is made per wave
        qkv[1, :, : 2 * D] *= 25.0
    qkv = qkv.bfloat16()
    alive = _alive(NM, B, NM, 0.7)
    alive[:, NM // 3] = True
    got = _run_sdpa(qkv, alive, H, path).float()
    assert torch.isfinite(got).all()
    truth = torch_ref.sdpa_masked(qkv.double(), alive, H).float()
    for b in range(B):
        assert max_rel(got[b], truth[b]) <= BF16_TOL, (case, b)
    lib16 = torch_ref.sdpa_masked(qkv, alive, H).float()
    assert max_rel(got, truth) <= max_rel(lib16, truth) + 8e-3


def test_sdpa_bf16_one_live_key_returns_its_value_row_exactly_on_every_kernel():
    # the normaliser is the sum of the weights as the matrix product sees them, so a single weight cancels exactly
    B, NM, H, D = 3, 84, 4, 128
    qkv = _qkv(5, B, NM, D, torch.bfloat16, scale=2.0)
    alive = torch.zeros(B, NM, dtype=torch.bool)
    alive[0, 7], alive[1, NM - 1], alive[2, 40] = True, True, True
    for path in ("mfma", "env", "head"):
        got = _run_sdpa(qkv, alive, H, path)
        for b, key in enumerate((7, NM - 1, 40)):
            assert torch.equal(got[b], qkv[b, key, 2 * D:].expand(NM, D)), (path, b)
    small = _qkv(6, B, 12, D, torch.bfloat16, scale=2.0)
    one = torch.zeros(B, 12, dtype=torch.bool)
    one[:, 5] = True
    assert torch.equal(_run_sdpa(small, one, H, "auto"), small[:, 5:6, 2 * D:].expand(B, 12, D))


def test_sdpa_bf16_both_kernels_agree():
    B, NM, H, D = 6, 84, 4, 128
    qkv = _qkv(21, B, NM, D, torch.bfloat16)
    alive = _alive(21, B, NM, 0.7)
    alive[:, 0] = True
    a = _run_sdpa(qkv, alive, H, "valu").float()
    b = _run_sdpa(qkv, alive, H, "mfma").float()
    assert max_rel(a, b) <= 1.2e-2


def test_sdpa_mfma_live_counts_across_block_edges():
    # live keys 1, 31, 32, 33, 64, 65, 159, 160 of NM = 160: every padding/compaction edge
    NM, H, D = 160, 4, 128
    counts = [1, 31, 32, 33, 64, 65, 159, 160]
    B = len(counts)
    qkv = _qkv(22, B, NM, D, torch.bfloat16)
    g = torch.Generator().manual_seed(22)
    alive = torch.zeros(B, NM, dtype=torch.bool)
    for b, c in enumerate(counts):
        alive[b, torch.randperm(NM, generator=g)[:c]] = True
    got = _run_sdpa(qkv, alive, H, "mfma").float()
    truth = torch_ref.sdpa_masked(qkv.float(), alive, H)
    for b in range(B):
        assert max_rel(got[b], truth[b]) <= BF16_TOL, counts[b]


@pytest.mark.parametrize("NM", [1, 7, 12, 23, 31, 32, 33, 64, 65, 84, 96, 97, 128, 129, 159, 160])
@pytest.mark.parametrize("groups", [24, 7, 3])
def test_sdpa_environment_kernel_matches_oracle_and_the_per_head_kernel(NM, groups, monkeypatch):
    # groups = work-groups the 24 environments are dealt to (each walks its environments with the next one's
    # set-up overlapped with the current one's arithmetic): one each, 3-4 each (ragged), 8 each
    monkeypatch.setenv("BNB_ENV_GROUP", str(groups))
    # one work-group per environment, K/V rows straight into LDS, V read through the transposing LDS load.
    # Per environment: mixed, all alive, all dead, only the first and only the last token alive, then
    # random live counts that cross every key-block edge
    B, H, D = 24, 4, 128
    qkv = _qkv(700 + NM, B, NM, D, torch.bfloat16)
    g = torch.Generator().manual_seed(700 + NM)
    alive = _alive(701 + NM, B, NM, 0.6)
    alive[0] = True
    alive[1] = False
    alive[2] = False
    alive[2, 0] = True
    alive[3] = False
    alive[3, NM - 1] = True
    for b in range(4, B):
        alive[b] = False
        alive[b, torch.randperm(NM, generator=g)[: int(torch.randint(1, NM + 1, (1,), generator=g))]] = True
    got = _run_sdpa(qkv, alive, H, "env").float()
    truth = torch_ref.sdpa_masked(qkv.float(), alive, H)
    assert torch.isfinite(got).all()
    for b in range(B):
        assert max_rel(got[b], truth[b]) <= BF16_TOL, (b, int(alive[b].sum()))
    mean_v = qkv[1, :, 2 * D:].float().mean(dim=0, keepdim=True).expand(NM, D)
    assert (got[1] - mean_v).abs().max() <= 1.6e-2
    assert torch.equal(got[3], qkv[3, NM - 1, 2 * D:].float().expand(NM, D))  # one live key: its V row, exactly
    # the same arithmetic in the same order as the per-head kernel: identical bits
    assert torch.equal(got, _run_sdpa(qkv, alive, H, "mfma").float())
    # dead keys weigh exactly nothing: rewriting their K and V rows changes no output bit
    pert = qkv.clone()
    dead = ~alive
    dead[~alive.any(dim=1)] = False  # an all-dead environment averages every row
    pert[..., D:][dead] = pert[..., D:][dead] * -3.0 + 17.0
    assert torch.equal(_run_sdpa(pert, alive, H, "env").float(), got)
    # heads do not leak into each other
    other = qkv.clone()
    for part in range(3):
        other[..., part * D + 64: part * D + 96] = other[..., part * D + 64: part * D + 96] * 2.0 + 1.0
    again = _run_sdpa(other, alive, H, "env").float()
    keep = torch.ones(D, dtype=torch.bool)
    keep[64:96] = False
    assert torch.equal(again[..., keep], got[..., keep]) and not torch.equal(again[..., 64:96], got[..., 64:96])
    # no mask, and rows that are a view of a wider buffer
    wide = torch.zeros(B, NM, 3 * D + 64, dtype=torch.bfloat16)
    wide[..., : 3 * D] = qkv
    view = wide.to(DEV)[..., : 3 * D]
    assert torch.equal(ops.sdpa_masked(view, alive.to(DEV), H, path="env").float().cpu(), got)
    assert max_rel(ops.sdpa_masked(view, None, H, path="env").float().cpu(), torch_ref.sdpa_masked(qkv.float(), None, H)) <= BF16_TOL
    # a batch that does not fill the last run
    assert torch.equal(_run_sdpa(qkv[: B - 1], alive[: B - 1], H, "env").float(), got[: B - 1])


@pytest.mark.parametrize("NM", [1, 12, 23, 32, 33, 84, 97, 129, 160])
@pytest.mark.parametrize("H", [4, 2, 8, 3])
def test_sdpa_head_kernel_with_rows_loaded_straight_into_lds_matches_oracle_and_the_staged_kernel(NM, H):
    # one work-group per (environment, head) like the staged kernel, but K/V rows go global -> LDS directly, the key
    # list comes from the alive row per wave, V is read through the transposing LDS load: same arithmetic, same bits
    B, D = 21, 32 * H
    qkv = _qkv(900 + NM + H, B, NM, D, torch.bfloat16)
    g = torch.Generator().manual_seed(900 + NM)
    alive = _alive(901 + NM, B, NM, 0.6)
    alive[0] = True
    alive[1] = False
    alive[2] = False
    alive[2, 0] = True
    alive[3] = False
    alive[3, NM - 1] = True
    for b in range(4, B):
        alive[b] = False
        alive[b, torch.randperm(NM, generator=g)[: int(torch.randint(1, NM + 1, (1,), generator=g))]] = True
    got = _run_sdpa(qkv, alive, H, "head").float()
    truth = torch_ref.sdpa_masked(qkv.float(), alive, H)
    assert torch.isfinite(got).all()
    for b in range(B):
        assert max_rel(got[b], truth[b]) <= BF16_TOL, (b, int(alive[b].sum()))
    assert torch.equal(got, _run_sdpa(qkv, alive, H, "mfma").float())
    assert torch.equal(got[3], qkv[3, NM - 1, 2 * D:].float().expand(NM, D))
    pert = qkv.clone()
    dead = ~alive
    dead[~alive.any(dim=1)] = False
    pert[..., D:][dead] = pert[..., D:][dead] * -3.0 + 17.0
    assert torch.equal(_run_sdpa(pert, alive, H, "head").float(), got)
    wide = torch.zeros(B, NM, 3 * D + 64, dtype=torch.bfloat16)
    wide[..., : 3 * D] = qkv
    view = wide.to(DEV)[..., : 3 * D]
    assert torch.equal(ops.sdpa_masked(view, alive.to(DEV), H, path="head").float().cpu(), got)
    assert max_rel(ops.sdpa_masked(view, None, H, path="head").float().cpu(), torch_ref.sdpa_masked(qkv.float(), None, H)) <= BF16_TOL


def test_sdpa_environment_kernel_limits():
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.sdpa_masked(torch.zeros(1, 12, 192, device=DEV, dtype=torch.bfloat16), None, 2, path="env")  # two heads
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.sdpa_masked(torch.zeros(1, 161, 384, device=DEV, dtype=torch.bfloat16), None, 4, path="env")
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.sdpa_masked(torch.zeros(1, 12, 384, device=DEV), None, 4, path="env")  # float32


@pytest.mark.parametrize("NM", [1, 2, 5, 12, 15, 16])
@pytest.mark.parametrize("H", [2, 4, 8, 3])
def test_sdpa_two_heads_per_wave_for_up_to_16_tokens(NM, H):
    # up to 16 tokens and an even head count take the kernel that shares one matrix-core tile
    # between two heads (an odd head count keeps one head per wave); per environment: mixed,
    # all alive, all dead, only the first and only the last token alive
    B, D = 37, 32 * H
    qkv = _qkv(300 + NM + H, B, NM, D, torch.bfloat16)
    alive = _alive(300 + NM, B, NM, 0.6)
    alive[0] = True
    alive[1] = False
    alive[2] = False
    alive[2, 0] = True
    alive[3] = False
    alive[3, NM - 1] = True
    got = _run_sdpa(qkv, alive, H, "mfma").float()
    truth = torch_ref.sdpa_masked(qkv.float(), alive, H)
    assert torch.isfinite(got).all()
    for b in range(B):
        assert max_rel(got[b], truth[b]) <= BF16_TOL, (b, alive[b])
    mean_v = qkv[1, :, 2 * D:].float().mean(dim=0, keepdim=True).expand(NM, D)
    assert (got[1] - mean_v).abs().max() <= 1.6e-2
    assert torch.equal(got[3], qkv[3, NM - 1, 2 * D:].float().expand(NM, D))
    # dead keys weigh exactly nothing: rewriting their K and V rows changes no output bit
    pert = qkv.clone()
    dead = ~alive
    dead[~alive.any(dim=1)] = False  # an all-dead environment averages every row
    pert[..., D:][dead] = pert[..., D:][dead] * -3.0 + 17.0
    assert torch.equal(_run_sdpa(pert, alive, H, "mfma").float(), got)
    # heads do not leak into each other: changing one head's inputs leaves the others' outputs alone
    other = qkv.clone()
    for part in range(3):
        other[..., part * D: part * D + 32] = other[..., part * D: part * D + 32] * 2.0 + 1.0
    again = _run_sdpa(other, alive, H, "mfma").float()
    assert torch.equal(again[..., 32:], got[..., 32:])
    assert not torch.equal(again[..., :32], got[..., :32])


@pytest.mark.parametrize("NM,path", [(161, "auto"), (200, "auto"), (320, "auto")])
def test_sdpa_bf16_beyond_matrix_core_range_uses_the_vector_kernel(NM, path):
    # crossover evaluation reaches 320 ships (modes/crossover.py:92); more than 160 tokens in bf16
    # falls back to the vector-ALU kernel
    B, H, D = 2, 4, 128
    qkv = _qkv(NM, B, NM, D, torch.bfloat16)
    alive = _alive(NM, B, NM, 0.6)
    alive[:, 5] = True
    got = _run_sdpa(qkv, alive, H, path).float()
    assert max_rel(got, torch_ref.sdpa_masked(qkv.float(), alive, H)) <= BF16_TOL
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        _run_sdpa(qkv, alive, H, "mfma")


@pytest.mark.parametrize("NM", [12, 84])
def test_sdpa_mfma_padded_rows_no_mask_and_uint8_mask(NM):
    B, H, D = 5, 4, 128
    qkv = _qkv(31 + NM, B, NM, D, torch.bfloat16)
    wide = torch.zeros(B, NM, 3 * D + 64, dtype=torch.bfloat16)
    wide[..., : 3 * D] = qkv
    view = wide.to(DEV)[..., : 3 * D]  # row stride 448 elements
    truth = torch_ref.sdpa_masked(qkv.float(), None, H)
    assert max_rel(ops.sdpa_masked(view, None, H, path="mfma").float().cpu(), truth) <= BF16_TOL
    alive = _alive(NM, B, NM, 0.5)
    alive[:, 0] = True
    a = ops.sdpa_masked(view, alive.to(DEV).to(torch.uint8), H, path="mfma")
    b = ops.sdpa_masked(qkv.to(DEV), alive.to(DEV), H, path="mfma")
    assert torch.equal(a, b)


def test_sdpa_small_batches_fp32():
    # one and a handful of environments (crossover runs 48..256, modes/crossover.py:37-47)
    for B in (1, 2, 48):
        qkv = _qkv(B, B, 12, 128, torch.float32)
        alive = _alive(B, B, 12, 0.8)
        alive[:, 0] = True
        assert max_rel(_run_sdpa(qkv, alive, 4), torch_ref.sdpa_masked(qkv, alive, 4)) <= F32_TOL


def test_sdpa_environment_permutation_is_bitwise_equivariant_at_full_size():
    # full 64v88 batch: shuffling environments must shuffle outputs bit for bit
    w = harness.WORKLOADS["c4_64v88_bf16"]
    g = torch.Generator(device=DEV).manual_seed(3)
    qkv = torch.randn(w.B, w.NM, 384, device=DEV, generator=g).bfloat16()
    alive = harness.make_alive(w, steps=1)[0].to(DEV)
    perm = torch.randperm(w.B, device=DEV)
    a = ops.sdpa_masked(qkv, alive, 4)
    b = ops.sdpa_masked(qkv[perm].contiguous(), alive[perm].contiguous(), 4)
    assert torch.equal(a[perm], b)
    # and a sample of environments against the CPU oracle
    pick = torch.arange(0, w.B, 257)
    truth = torch_ref.sdpa_masked(qkv[pick].float().cpu(), alive[pick].cpu(), 4)
    assert max_rel(a[pick].float().cpu(), truth) <= BF16_TOL


# ------------------------------------------------------------------ bullet read (cross-attention)


@pytest.mark.parametrize("B,NQ,NK", [(4, 12, 80), (3, 20, 160), (5, 12, 7), (2, 84, 40), (3, 33, 33), (2, 160, 1)])
def test_sdpa_cross_matches_oracle(B, NQ, NK):
    H, D = 4, 128
    g = torch.Generator().manual_seed(NQ * 200 + NK)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16()
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16()
    mask = torch.rand(B, NK, generator=g) < 0.5
    mask[0] = False  # nothing active in env 0
    mask[1, 0] = True
    merged = torch.randn(B, NQ, D, generator=g).bfloat16()
    truth = torch_ref.bullet_read(qkv.float(), kv.float(), mask, H)
    bare = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H).float().cpu()
    assert bare[0].abs().max() == 0  # gated off exactly
    assert max_rel(bare, truth) <= BF16_TOL
    acc = merged.to(DEV).clone()
    out = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H, accum=acc)
    assert out.data_ptr() == acc.data_ptr()
    want = (merged + bare.bfloat16()).float()  # bf16 + bf16 as torch adds them
    assert torch.equal(out.float().cpu(), want)
    assert torch.equal(out[0].cpu(), merged[0])  # env 0 untouched
    # inactive slots cannot influence the result
    kv2 = kv.clone()
    kv2[~mask] = kv2[~mask] * -2.0 + 9.0
    assert torch.equal(ops.sdpa_cross(qkv.to(DEV), kv2.to(DEV), mask.to(DEV), H).float().cpu(), bare)
    no_mask = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), None, H).float().cpu()
    assert max_rel(no_mask, torch_ref.bullet_read(qkv.float(), kv.float(), None, H)) <= BF16_TOL


@pytest.mark.parametrize("B,NQ,NK,p_live", [(4, 12, 161, 0.5), (3, 84, 800, 0.3), (2, 156, 1520, 1.0), (3, 156, 1520, 0.1),
                                           (2, 33, 2048, 0.7), (3, 20, 500, 0.02), (2, 160, 193, 0.17),
                                           # a fifth block of queries, shared by the waves: 2 rows of it, few keys, many keys
                                           (3, 130, 700, 0.3), (3, 129, 300, 0.05), (2, 145, 2048, 0.9)])
def test_sdpa_cross_streams_long_key_axes(B, NQ, NK, p_live):
    # more keys than fit in LDS at once: tiles of live keys with an online softmax across them
    H, D = 4, 128
    g = torch.Generator().manual_seed(NQ * 3000 + NK)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16()
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16()
    kv[:, :, :D] *= 3.0  # peaked softmax rows: the running maximum has to move between tiles
    mask = torch.rand(B, NK, generator=g) < p_live
    mask[0] = False
    mask[1, NK - 1] = True
    merged = torch.randn(B, NQ, D, generator=g).bfloat16()
    truth = torch_ref.bullet_read(qkv.float(), kv.float(), mask, H)
    bare = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H).float().cpu()
    assert bare[0].abs().max() == 0
    assert max_rel(bare, truth) <= BF16_TOL
    acc = merged.to(DEV).clone()
    out = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H, accum=acc)
    assert out.data_ptr() == acc.data_ptr()
    assert torch.equal(out.float().cpu(), (merged + bare.bfloat16()).float())
    other = torch.empty_like(acc)  # accum != out: environments without a live key copy accum through
    got = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H, accum=merged.to(DEV), out=other)
    assert torch.equal(got.cpu(), out.cpu())
    kv2 = kv.clone()
    kv2[~mask] = kv2[~mask] * -2.0 + 9.0
    assert torch.equal(ops.sdpa_cross(qkv.to(DEV), kv2.to(DEV), mask.to(DEV), H).float().cpu(), bare)
    no_mask = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), None, H).float().cpu()
    assert max_rel(no_mask, torch_ref.bullet_read(qkv.float(), kv.float(), None, H)) <= BF16_TOL


@pytest.mark.parametrize("B,NQ,NK,p_live", [(4, 12, 80, 0.5), (3, 20, 160, 0.25), (5, 12, 7, 0.5), (2, 84, 800, 0.3),
                                           (2, 160, 1520, 1.0), (3, 160, 1520, 0.1), (2, 320, 3200, 0.25), (2, 33, 4096, 0.7),
                                           (3, 20, 500, 0.02), (2, 160, 1, 1.0), (2, 512, 97, 0.6)])
def test_sdpa_cross_fp32_matches_oracle(B, NQ, NK, p_live):
    # evaluation without autocast: the same read on the fp32 matrix cores, float32 bar
    H, D = 4, 128
    g = torch.Generator().manual_seed(NQ * 5000 + NK)
    qkv = torch.randn(B, NQ, 3 * D, generator=g)
    kv = torch.randn(B, NK, 2 * D, generator=g)
    kv[:, :, :D] *= 2.0  # peaked rows: the running maximum moves between tiles
    mask = torch.rand(B, NK, generator=g) < p_live
    mask[0] = False  # nothing active in env 0
    mask[1, NK - 1] = True
    merged = torch.randn(B, NQ, D, generator=g)
    truth = torch_ref.bullet_read(qkv, kv, mask, H)
    bare = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H).cpu()
    assert bare.dtype == torch.float32 and bare[0].abs().max() == 0  # gated off exactly
    assert max_rel(bare, truth) <= F32_TOL
    if NK <= 200:  # the float64 loop statement on a few queries
        brute = bruteforce.bullet_read_loops(qkv[1:2, :3, :D].numpy(), kv[1:2].numpy(), mask[1:2].numpy(), H)
        assert max_rel(bare[1:2, :3].double(), torch.as_tensor(brute)) <= F32_TOL
    acc = merged.to(DEV).clone()
    out = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H, accum=acc)
    assert out.data_ptr() == acc.data_ptr()
    assert torch.equal(out.cpu(), merged + bare)  # one float32 addition
    assert torch.equal(out[0].cpu(), merged[0])  # env 0 untouched
    other = torch.empty_like(acc)
    got = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), mask.to(DEV), H, accum=merged.to(DEV), out=other)
    assert torch.equal(got.cpu(), out.cpu())
    # inactive slots cannot influence the result; strided views of wider buffers work
    kv2 = kv.clone()
    kv2[~mask] = kv2[~mask] * -2.0 + 9.0
    assert torch.equal(ops.sdpa_cross(qkv.to(DEV), kv2.to(DEV), mask.to(DEV), H).cpu(), bare)
    no_mask = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), None, H).cpu()
    assert max_rel(no_mask, torch_ref.bullet_read(qkv, kv, None, H)) <= F32_TOL


def test_sdpa_cross_limits():
    qkv = torch.zeros(1, 12, 384, device=DEV, dtype=torch.bfloat16)
    assert not ops.cross_supported(qkv, torch.zeros(1, 2049, 256, device=DEV, dtype=torch.bfloat16), 4)
    assert ops.cross_supported(qkv.float(), torch.zeros(1, 80, 256, device=DEV), 4)  # float32 has its own kernel
    assert not ops.cross_supported(qkv.float(), torch.zeros(1, 80, 256, device=DEV, dtype=torch.bfloat16), 4)  # one dtype
    assert not ops.cross_supported(qkv.float(), torch.zeros(1, 4097, 256, device=DEV), 4)
    with pytest.raises(RuntimeError):
        ops.sdpa_cross(qkv, torch.zeros(1, 2100, 256, device=DEV, dtype=torch.bfloat16), None, 4)


# ------------------------------------------------------------------ RG-LRU step


def _rglru_inputs(seed, R, D, xdt, gdt):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(R, D, generator=g).to(xdt)
    gates = (1.5 * torch.randn(R, 2 * D, generator=g)).to(gdt)
    h = 0.5 * torch.randn(R, D, generator=g)
    return x, gates, torch.linspace(0.0, 4.0, D), h


@pytest.mark.parametrize("R,D", [(1, 128), (17, 128), (1000, 128), (4097, 128), (33, 32), (9, 64), (5, 12), (3, 136)])
def test_rglru_fp32_matches_oracle(R, D):
    x, gates, lam, h = _rglru_inputs(R + D, R, D, torch.float32, torch.float32)
    y, h_new = ops.rglru_step(x.to(DEV), gates.to(DEV), lam.to(DEV), 8.0, h.to(DEV))
    assert y is h_new and h_new.dtype == torch.float32
    ref = torch_ref.rglru_step(x, gates, lam, 8.0, h)
    assert max_rel(h_new.cpu(), ref) <= F32_TOL
    assert torch.allclose(h_new.cpu(), ref, rtol=2e-5, atol=2e-6)
    cc = torch.from_numpy(c_ref.rglru_step(x.numpy(), gates.numpy(), lam.numpy(), 8.0, h.numpy()))
    assert max_rel(h_new.cpu(), cc) <= F32_TOL


def test_rglru_known_answers_on_device():
    D = 128
    lam = torch.linspace(0.0, 4.0, D)
    h = torch.full((2, D), 2.0)
    x = torch.full((2, D), 0.5)
    big = 40.0
    gates = torch.cat([torch.full((2, D), -big), torch.full((2, D), big)], dim=-1)  # r -> 0, i -> 1
    _, out = ops.rglru_step(x.to(DEV), gates.to(DEV), lam.to(DEV), 8.0, h.to(DEV))
    assert torch.allclose(out.cpu(), h + 1e-3 * x, rtol=1e-6)  # a = 1, clamp floor => gate = 1e-3
    gates = torch.full((2, 2 * D), big)  # r -> 1
    _, out = ops.rglru_step(torch.zeros(2, D, device=DEV), gates.to(DEV), lam.to(DEV), 8.0, h.to(DEV))
    assert float(out[0, 0]) == pytest.approx(2.0 * 0.5 ** 8, rel=1e-6)  # lambda = 0 => a = 0.5^8


def test_rglru_reads_and_writes_the_packed_hidden_in_place():
    # state rows live inside a (R, 4D) tensor, as in the policy's packed hidden (policy.py:323)
    R, D = 50, 128
    x, gates, lam, h = _rglru_inputs(3, R, D, torch.float32, torch.float32)
    packed = torch.randn(R, 4 * D)
    packed[:, :D] = h
    dev = packed.to(DEV)
    view = dev[:, :D]
    y, h_new = ops.rglru_step(x.to(DEV), gates.to(DEV), lam.to(DEV), 8.0, view, h_out=view)
    ref = torch_ref.rglru_step(x, gates, lam, 8.0, h)
    assert h_new.data_ptr() == dev.data_ptr()
    assert max_rel(dev[:, :D].cpu(), ref) <= F32_TOL
    assert torch.equal(dev[:, D:].cpu(), packed[:, D:])  # conv-buffer columns untouched


@pytest.mark.parametrize("xdt,gdt", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16),
                                     (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("R,D", [(257, 128), (6, 20)])
def test_rglru_bf16_follows_autocast_dtype_flow(xdt, gdt, R, D):
    x, gates, lam, h = _rglru_inputs(R, R, D, xdt, gdt)
    y, h_new = ops.rglru_step(x.to(DEV), gates.to(DEV), lam.to(DEV), 8.0, h.to(DEV), y_dtype=torch.bfloat16)
    assert y.dtype == torch.bfloat16 and h_new.dtype == torch.float32
    truth = torch_ref.rglru_step(x.float(), gates.float(), lam, 8.0, h)
    assert max_rel(h_new.cpu(), truth) <= BF16_TOL
    assert max_rel(y.float().cpu(), truth) <= BF16_TOL
    # same operations in the same dtypes on the CPU: only transcendental rounding may differ
    mirror = torch_ref.rglru_step(x, gates, lam, 8.0, h)
    assert mirror.dtype == torch.float32
    assert max_rel(h_new.cpu(), mirror) <= 4e-3
    assert torch.equal(y.cpu(), h_new.cpu().bfloat16())


def test_rglru_empty_and_rejected_inputs():
    lam = torch.linspace(0, 4, 128, device=DEV)
    y, h = ops.rglru_step(torch.zeros(0, 128, device=DEV), torch.zeros(0, 256, device=DEV), lam, 8.0,
                          torch.zeros(0, 128, device=DEV))
    assert h.shape == (0, 128)
    with pytest.raises(TypeError):
        ops.rglru_step(torch.zeros(2, 128, device=DEV), torch.zeros(2, 256, device=DEV), lam, 8.0,
                       torch.zeros(2, 128, device=DEV, dtype=torch.bfloat16))


def test_rglru_rollout_of_full_size_state_matches_oracle_on_sampled_rows():
    # 64v88 state (622,592 rows), 4 carried steps; rows sampled across the tensor go through the oracle
    w = harness.WORKLOADS["c4_64v88_bf16"]
    R, D, T = w.B * w.N, 128, 4
    g = torch.Generator(device=DEV).manual_seed(11)
    lam = torch.linspace(0, 4, D, device=DEV)
    h = 0.5 * torch.randn(R, D, device=DEV, generator=g)
    pick = torch.arange(0, R, 9973, device=DEV)
    h_ref = h[pick].cpu()
    for t in range(T):
        x = torch.randn(R, D, device=DEV, generator=g).bfloat16()
        gates = torch.randn(R, 2 * D, device=DEV, generator=g).bfloat16()
        y, h = ops.rglru_step(x, gates, lam, 8.0, h, y_dtype=torch.bfloat16)
        h_ref = torch_ref.rglru_step(x[pick].float().cpu(), gates[pick].float().cpu(), lam.cpu(), 8.0, h_ref)
        assert max_rel(h[pick].cpu(), h_ref) <= BF16_TOL, t
    assert torch.isfinite(h).all()


# ------------------------------------------------------------------ conv step and folded reset


def _conv_ref(b1, conv_buf, weight, bias):
    """padded = [p0,p1,p2,b1]; v = sum_k padded[k] * w[:,k] + bias; buffer shifts (griffin.py:127-139,275-277)."""
    padded = torch.cat([conv_buf, b1.float().unsqueeze(1)], dim=1)
    v = (padded * weight.reshape(-1, 4).t().unsqueeze(0)).sum(dim=1)
    return (v + bias if bias is not None else v), padded[:, 1:]


@pytest.mark.parametrize("R,D,dtype", [(1, 128, torch.float32), (77, 128, torch.bfloat16), (5000, 128, torch.bfloat16),
                                       (9, 32, torch.float32), (7, 12, torch.bfloat16), (3, 136, torch.float32)])
def test_conv_step_matches_tap_formula(R, D, dtype):
    g = torch.Generator().manual_seed(R + D)
    b1 = torch.randn(R, D, generator=g).to(dtype)
    buf = torch.randn(R, 3, D, generator=g)
    w = 0.5 * torch.randn(D, 1, 4, generator=g)
    bias = 0.1 * torch.randn(D, generator=g)
    v, new_buf = ops.conv_step(b1.to(DEV), buf.to(DEV), w.to(DEV), bias.to(DEV))
    ref_v, ref_buf = _conv_ref(b1, buf, w, bias)
    assert v.dtype == torch.float32 and new_buf.shape == (R, 3, D)
    assert max_rel(v.cpu(), ref_v) <= F32_TOL
    assert torch.equal(new_buf.cpu(), ref_buf)  # a pure shift: bit exact
    # the library depthwise conv as an independent statement of the tap order
    lib = torch.nn.functional.conv1d(torch.cat([buf, b1.float().unsqueeze(1)], 1).transpose(1, 2), w, bias, groups=D)[:, :, 0]
    assert max_rel(v.cpu(), lib) <= F32_TOL
    v2, _ = ops.conv_step(b1.to(DEV), buf.to(DEV), w.to(DEV), None)
    assert max_rel(v2.cpu(), ref_v - bias) <= F32_TOL


def test_conv_and_rglru_step_update_the_packed_state_in_place_with_reset():
    # rows of the policy's packed hidden (R, 4D) = [h | p0 | p1 | p2]; environments 1 and 3 were reset
    B, n_rec, D = 5, 3, 128
    R = B * n_rec
    g = torch.Generator().manual_seed(9)
    state = torch.randn(R, 4 * D, generator=g)
    b1 = torch.randn(R, D, generator=g).bfloat16()
    w, bias = 0.5 * torch.randn(D, 1, 4, generator=g), 0.1 * torch.randn(D, generator=g)
    gates = torch.randn(R, 2 * D, generator=g).bfloat16()
    lam = torch.linspace(0, 4, D)
    done = torch.tensor([False, True, False, True, False])
    dev_in, dev_out = state.to(DEV), torch.full((R, 4 * D), float("nan"), device=DEV)
    v, _ = ops.conv_step(b1.to(DEV), dev_in[:, D:].view(R, 3, D), w.to(DEV), bias.to(DEV),
                         conv_out=dev_out[:, D:].view(R, 3, D), reset=done.to(DEV), rows_per_env=n_rec)
    y, _ = ops.rglru_step(v, gates.to(DEV), lam.to(DEV), 8.0, dev_in[:, :D], h_out=dev_out[:, :D],
                          reset=done.to(DEV), rows_per_env=n_rec)
    assert torch.equal(dev_in.cpu(), state)  # the incoming state is never written
    zeroed = torch_ref.reset_hidden(state.unsqueeze(0), done, n_rec)[0]
    ref_v, ref_buf = _conv_ref(b1, zeroed[:, D:].reshape(R, 3, D), w, bias)
    ref_h = torch_ref.rglru_step(ref_v, gates, lam, 8.0, zeroed[:, :D])
    assert max_rel(v.cpu(), ref_v) <= F32_TOL
    assert torch.equal(dev_out[:, D:].cpu(), ref_buf.reshape(R, 3 * D))
    assert max_rel(dev_out[:, :D].cpu(), ref_h) <= 4e-3  # bf16 gate flow, fp32 oracle of the same dtypes
    assert y.data_ptr() == dev_out.data_ptr()


def test_conv_step_full_size_rows_sampled_against_formula():
    w_ = harness.WORKLOADS["c4_64v88_bf16"]
    R, D = w_.B * w_.N, 128
    g = torch.Generator(device=DEV).manual_seed(4)
    state = torch.randn(R, 4 * D, device=DEV, generator=g)
    b1 = torch.randn(R, D, device=DEV, generator=g).bfloat16()
    w = 0.5 * torch.randn(D, 1, 4, device=DEV, generator=g)
    bias = 0.1 * torch.randn(D, device=DEV, generator=g)
    new_state = torch.empty_like(state)
    v, _ = ops.conv_step(b1, state[:, D:].view(R, 3, D), w, bias, conv_out=new_state[:, D:].view(R, 3, D))
    pick = torch.arange(0, R, 7919, device=DEV)
    ref_v, ref_buf = _conv_ref(b1[pick].cpu(), state[pick, D:].reshape(-1, 3, D).cpu(), w.cpu(), bias.cpu())
    assert max_rel(v[pick].cpu(), ref_v) <= F32_TOL
    assert torch.equal(new_state[pick, D:].cpu(), ref_buf.reshape(-1, 3 * D))
    assert torch.equal(new_state[:, D:2 * D], state[:, 2 * D:3 * D])  # whole-tensor shift property


# ------------------------------------------------------------------ fused norm and gelu-gate kernels


@pytest.mark.parametrize("R,D", [(1, 128), (37, 128), (3000, 128), (9, 64), (5, 32), (4, 512), (6, 8)])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_add_rmsnorm_matches_library_rms_norm(R, D, out_dtype):
    g = torch.Generator().manual_seed(R * 7 + D)
    x = 2.0 * torch.randn(R, D, generator=g)
    w = 1.0 + 0.1 * torch.randn(D, generator=g)
    delta = torch.randn(R, D, generator=g).bfloat16()
    tol = F32_TOL if out_dtype == torch.float32 else 4e-3
    # norm only: nn.RMSNorm(D) semantics (eps = finfo(float32).eps)
    same, n = ops.add_rmsnorm(x.to(DEV), w.to(DEV), out_dtype=out_dtype)
    assert same.data_ptr() != 0 and n.dtype == out_dtype
    ref = torch.nn.functional.rms_norm(x, (D,), w, None)
    assert max_rel(n.float().cpu(), ref) <= tol
    assert torch.allclose(n.float().cpu(), ref.to(out_dtype).float(), rtol=1e-2 if out_dtype == torch.bfloat16 else 1e-5, atol=1e-5)
    # add + norm: fp32 residual + bf16 branch output
    s_, n2 = ops.add_rmsnorm(x.to(DEV), w.to(DEV), delta=delta.to(DEV), out_dtype=out_dtype)
    ref_s = x + delta
    assert torch.equal(s_.cpu(), ref_s)  # fp32 + bf16 -> fp32, one rounding: bit exact
    assert max_rel(n2.float().cpu(), torch.nn.functional.rms_norm(ref_s, (D,), w, None)) <= tol


def test_add_rmsnorm_keeps_leading_shape_and_rejects_uncovered_widths():
    x = torch.randn(3, 5, 128, device=DEV)
    w = torch.ones(128, device=DEV)
    s_, n = ops.add_rmsnorm(x, w, delta=torch.zeros_like(x))
    assert s_.shape == x.shape and n.shape == x.shape and torch.equal(s_, x)
    with pytest.raises(ValueError):
        ops.add_rmsnorm(torch.randn(2, 24, device=DEV), torch.ones(24, device=DEV))


@pytest.mark.parametrize("adt,bdt,odt", [(torch.float32, torch.float32, torch.float32),
                                         (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                         (torch.bfloat16, torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("R,H", [(3, 512), (1000, 512), (7, 128), (5, 8)])
def test_gelu_mul_matches_torch_with_its_rounding_points(adt, bdt, odt, R, H):
    g = torch.Generator().manual_seed(R + H)
    both = (2.0 * torch.randn(R, 2 * H, generator=g)).to(adt)
    a = both[:, :H]  # the two halves of one projection output: row stride 2H
    b = both[:, H:].to(bdt) if bdt == adt else torch.randn(R, H, generator=g).to(bdt)
    dev_both = both.to(DEV)
    dev_b = dev_both[:, H:] if bdt == adt else b.to(DEV)
    out = ops.gelu_mul(dev_both[:, :H], dev_b, out_dtype=odt)
    assert out.dtype == odt and out.is_contiguous()
    ref = (torch.nn.functional.gelu(a) * b).to(odt)  # torch rounds gelu to a's dtype, then the product
    truth = torch.nn.functional.gelu(a.double()) * b.double()
    assert max_rel(out.float().cpu(), truth.float()) <= (F32_TOL if odt == torch.float32 else BF16_TOL)
    if odt == torch.float32:
        assert torch.allclose(out.cpu(), ref, rtol=1e-5, atol=2e-6)
    else:
        # identical rounding points: at most one bf16 ulp apart where erf rounding differs
        assert (out.float().cpu() - ref.float()).abs().max() <= 2 ** -7 * ref.float().abs().max()


# ------------------------------------------------------------------ the measured step


@pytest.mark.parametrize("name,B", [("c0_4v4_fp32", None), ("c1_4v4_rollout_bf16", 256), ("c2_8v11_bf16", 128),
                                    ("c3_32v48_bf16", 32), ("c4_64v88_bf16", 16)])
def test_step_matches_oracle_on_benchmark_workloads(name, B):
    w = harness.WORKLOADS[name]
    B = w.B if B is None else B
    p = harness.make_weights(w.seed, w.dtype)
    tokens, state = harness.make_inputs(w, B=B)
    alive = harness.make_alive(w, steps=1, B=B)[0]
    step = harness.AttnRglruStep.from_weights(p, DEV)
    hidden, new_state = step(tokens.to(DEV), alive.to(DEV), state.to(DEV))
    p32 = {k: v.float() for k, v in p.items()}
    ref_hidden, ref_state = torch_ref.harness_step(p32, tokens.float(), alive, state)
    tol = F32_TOL if w.dtype == torch.float32 else BF16_TOL
    assert hidden.dtype == w.dtype and new_state.dtype == torch.float32
    assert max_rel(hidden.float().cpu(), ref_hidden) <= tol
    assert max_rel(new_state.cpu(), ref_state) <= tol


def test_step_carried_rollout_with_dying_ships():
    # 4v4 rollout shape, 12 carried steps, ships dying along the way
    w = harness.WORKLOADS["c1_4v4_rollout_bf16"]
    B, T = 64, 12
    p = harness.make_weights(w.seed, w.dtype)
    step = harness.AttnRglruStep.from_weights(p, DEV)
    p32 = {k: v.float() for k, v in p.items()}
    alive = harness.make_alive(w, steps=T, B=B)
    _, state = harness.make_inputs(w, B=B)
    dev_state, ref_state = state.to(DEV), state
    g = torch.Generator().manual_seed(5)
    for t in range(T):
        tokens = torch.randn(B, w.NM, 128, generator=g).bfloat16()
        hidden, dev_state = step(tokens.to(DEV), alive[t].to(DEV), dev_state)
        ref_hidden, ref_state = torch_ref.harness_step(p32, tokens.float(), alive[t], ref_state)
        assert max_rel(hidden.float().cpu(), ref_hidden) <= BF16_TOL, t
    assert max_rel(dev_state.cpu(), ref_state) <= BF16_TOL


# ------------------------------------------------------------------ sequence path: conv + recurrence over T


def _seq_inputs(seed, R, T, D, x_dtype, g_dtype, p_done):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(R, T, D, generator=g).to(x_dtype)
    gates = (2.0 * torch.randn(R, T, 2 * D, generator=g)).to(g_dtype)
    h0 = torch.randn(R, D, generator=g)
    done = (torch.rand(R, T, generator=g) < p_done) if p_done > 0 else None
    return x, gates, h0, done


# R * D/8 >= 131072 lanes takes the 8-channels-per-lane kernel, smaller inputs one lane per channel
@pytest.mark.parametrize("R,T,D", [(5, 1, 128), (7, 2, 128), (9, 3, 64), (33, 7, 128), (16, 128, 128), (3, 130, 40),
                                   (8192, 5, 128), (8200, 9, 128)])
@pytest.mark.parametrize("p_done", [0.0, 0.2])
def test_rglru_scan_fp32_matches_oracle(R, T, D, p_done):
    x, gates, h0, done = _seq_inputs(R + T, R, T, D, torch.float32, torch.float32, p_done)
    lam = torch.linspace(0.0, 4.0, D)
    want, want_last = torch_ref.rglru_sequence(x, gates, lam, 8.0, h0, done)
    y, last = ops.rglru_scan(x.to(DEV), gates.to(DEV), lam.to(DEV), 8.0, h0.to(DEV), None if done is None else done.to(DEV))
    assert y.dtype == torch.float32 and y.shape == (R, T, D)
    assert max_rel(y.cpu(), want) <= F32_TOL
    assert max_rel(last.cpu(), want_last) <= F32_TOL
    assert torch.equal(last.cpu(), y[:, -1].cpu())


@pytest.mark.parametrize("R,T", [(6, 4), (40, 128), (8192, 6)])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
def test_rglru_scan_bf16_gates_match_oracle(R, T, x_dtype):
    D = 128
    x, gates, h0, done = _seq_inputs(R * 3 + T, R, T, D, x_dtype, torch.bfloat16, 0.1)
    lam = torch.linspace(0.0, 4.0, D)
    want, want_last = torch_ref.rglru_sequence(x, gates, lam, 8.0, h0, done)  # torch's own promotion, as under autocast
    assert want.dtype == torch.float32
    for y_dtype in (torch.float32, torch.bfloat16):
        y, last = ops.rglru_scan(x.to(DEV), gates.to(DEV), lam.to(DEV), 8.0, h0.to(DEV), done.to(DEV), y_dtype=y_dtype)
        assert y.dtype == y_dtype
        assert max_rel(y.float().cpu(), want) <= BF16_TOL
        assert max_rel(last.cpu(), want_last) <= BF16_TOL


def test_rglru_scan_equals_the_step_kernel_applied_t_times():
    # same element arithmetic in both kernels: bit-identical states
    R, T, D = 64, 12, 128
    x, gates, h0, done = _seq_inputs(5, R, T, D, torch.float32, torch.bfloat16, 0.25)
    lam = torch.linspace(0.0, 4.0, D).to(DEV)
    xd, gd, dd = x.to(DEV), gates.to(DEV), done.to(DEV)
    y, last = ops.rglru_scan(xd, gd, lam, 8.0, h0.to(DEV), dd)
    h = h0.to(DEV)
    for t in range(T):
        reset = dd[:, t - 1].contiguous() if t > 0 else None
        _, h = ops.rglru_step(xd[:, t].contiguous(), gd[:, t].contiguous(), lam, 8.0, h, reset=reset, rows_per_env=1)
        assert torch.equal(h, y[:, t])
    assert torch.equal(h, last)


def test_rglru_scan_strided_state_and_in_place_final_state():
    R, T, D = 10, 6, 128
    x, gates, h0, _ = _seq_inputs(8, R, T, D, torch.float32, torch.float32, 0.0)
    lam = torch.linspace(0.0, 4.0, D).to(DEV)
    packed = torch.randn(R, 4 * D, device=DEV)
    packed[:, :D] = h0.to(DEV)
    before = packed.clone()
    y, last = ops.rglru_scan(x.to(DEV), gates.to(DEV), lam, 8.0, packed[:, :D], h_out=packed[:, :D])
    want, want_last = torch_ref.rglru_sequence(x, gates, lam.cpu(), 8.0, h0)
    assert last.data_ptr() == packed.data_ptr()
    assert max_rel(packed[:, :D].cpu(), want_last) <= F32_TOL
    assert torch.equal(packed[:, D:], before[:, D:])


@pytest.mark.parametrize("R,T,D", [(5, 1, 128), (7, 2, 128), (6, 3, 64), (33, 9, 128), (12, 128, 128), (3, 20, 40),
                                   (8192, 5, 128)])
@pytest.mark.parametrize("p_done", [0.0, 0.3])
@pytest.mark.parametrize("b_dtype", [torch.float32, torch.bfloat16])
def test_conv_seq_matches_oracle(R, T, D, p_done, b_dtype):
    g = torch.Generator().manual_seed(R * 7 + T)
    b1 = torch.randn(R, T, D, generator=g).to(b_dtype)
    buf = torch.randn(R, 3, D, generator=g)
    w = 0.5 * torch.randn(D, 1, 4, generator=g)
    bias = 0.1 * torch.randn(D, generator=g)
    done = (torch.rand(R, T, generator=g) < p_done) if p_done > 0 else None
    want, want_tail = torch_ref.conv_sequence(b1.float(), buf, w, bias, done)
    v, tail, v_lp = ops.conv_seq(b1.to(DEV), buf.to(DEV), w.to(DEV), bias.to(DEV), None if done is None else done.to(DEV),
                                 also_bf16=True)
    assert v.dtype == torch.float32 and v_lp.dtype == torch.bfloat16
    assert max_rel(v.cpu(), want) <= F32_TOL
    assert torch.equal(tail.cpu(), want_tail)
    assert torch.equal(v_lp.cpu(), v.cpu().bfloat16())


def test_conv_seq_equals_the_step_kernel_applied_t_times():
    R, T, D = 32, 7, 128
    g = torch.Generator().manual_seed(3)
    b1 = torch.randn(R, T, D, generator=g).bfloat16().to(DEV)
    buf = torch.randn(R, 3, D, generator=g).to(DEV)
    w = (0.5 * torch.randn(D, 1, 4, generator=g)).to(DEV)
    bias = (0.1 * torch.randn(D, generator=g)).to(DEV)
    done = (torch.rand(R, T, generator=g) < 0.3).to(DEV)
    v, tail = ops.conv_seq(b1, buf, w, bias, done)
    cur = buf
    for t in range(T):
        reset = done[:, t - 1].contiguous() if t > 0 else None
        vt, cur = ops.conv_step(b1[:, t].contiguous(), cur, w, bias, reset=reset, rows_per_env=1)
        assert torch.equal(vt, v[:, t])
    # the step path zeroes the stored inputs of a finished episode, the sequence path keeps the raw tail
    raw_tail = torch.cat([buf, b1.float()], dim=1)[:, -3:]
    assert torch.equal(tail, raw_tail)


@pytest.mark.parametrize("R,T", [(12, 9), (8192, 4)])
def test_sequence_kernels_time_major_layout_gives_the_same_numbers(R, T):
    D = 128
    x, gates, h0, done = _seq_inputs(77 + R, R, T, D, torch.float32, torch.bfloat16, 0.2)
    lam = torch.linspace(0.0, 4.0, D).to(DEV)
    xd, gd, dd, hd = x.to(DEV), gates.to(DEV), done.to(DEV), h0.to(DEV)
    y, last = ops.rglru_scan(xd, gd, lam, 8.0, hd, dd, y_dtype=torch.bfloat16)
    yt, last_t = ops.rglru_scan(xd.transpose(0, 1).contiguous(), gd.transpose(0, 1).contiguous(), lam, 8.0, hd, dd,
                                y_dtype=torch.bfloat16, time_major=True)
    assert yt.shape == (T, R, D)
    assert torch.equal(yt.transpose(0, 1), y) and torch.equal(last_t, last)
    g = torch.Generator().manual_seed(1)
    buf = torch.randn(R, 3, D, generator=g).to(DEV)
    w = torch.randn(D, 1, 4, generator=g).to(DEV)
    bias = torch.randn(D, generator=g).to(DEV)
    v, tail, v_lp = ops.conv_seq(xd, buf, w, bias, dd, also_bf16=True)
    vt, tail_t, vt_lp = ops.conv_seq(xd.transpose(0, 1).contiguous(), buf, w, bias, dd, also_bf16=True, time_major=True)
    assert torch.equal(vt.transpose(0, 1), v) and torch.equal(tail_t, tail) and torch.equal(vt_lp.transpose(0, 1), v_lp)


# ------------------------------------------------------------------ recurrence backward


def _scan_grads_oracle(x, gates, lam, h0, done, wy, wl, dtype64=True):
    """Gradients of sum(y*wy) + sum(h_last*wl) through the oracle's scan, by torch autograd."""
    up = (lambda t: t.double()) if dtype64 else (lambda t: t.clone())
    leaves = [up(t).requires_grad_(True) for t in (x, gates, lam, h0)]
    y, last = torch_ref.rglru_sequence(leaves[0], leaves[1], leaves[2], 8.0, leaves[3], done)
    ((y * up(wy)).sum() + (last * up(wl)).sum()).backward()
    return [t.grad for t in leaves]


@pytest.mark.parametrize("R,T,D", [(4, 1, 128), (6, 5, 64), (9, 128, 128), (3, 7, 40), (8192, 6, 128)])
@pytest.mark.parametrize("p_done", [0.0, 0.2])
@pytest.mark.parametrize("time_major", [False, True])
def test_rglru_scan_backward_fp32_matches_autograd_of_the_oracle(R, T, D, p_done, time_major):
    x, gates, h0, done = _seq_inputs(R * 5 + T, R, T, D, torch.float32, torch.float32, p_done)
    g = torch.Generator().manual_seed(T)
    wy, wl = torch.randn(R, T, D, generator=g), torch.randn(R, D, generator=g)
    lam = torch.linspace(0.0, 4.0, D)
    want = _scan_grads_oracle(x, gates, lam, h0, done, wy, wl)
    lay = (lambda t: t.transpose(0, 1).contiguous()) if time_major else (lambda t: t)
    leaves = [t.to(DEV).requires_grad_(True) for t in (lay(x), lay(gates), lam, h0)]
    y, last = ops.rglru_scan(leaves[0], leaves[1], leaves[2], 8.0, leaves[3], None if done is None else done.to(DEV),
                             time_major=time_major)
    ((y * lay(wy).to(DEV)).sum() + (last * wl.to(DEV)).sum()).backward()
    got = [t.grad.cpu() for t in leaves]
    assert max_rel(lay(got[0]) if time_major else got[0], want[0]) <= 2e-5
    assert max_rel(lay(got[1]) if time_major else got[1], want[1]) <= 2e-5
    assert max_rel(got[2], want[2]) <= 2e-5
    assert max_rel(got[3], want[3]) <= 2e-5


def test_rglru_scan_backward_with_bf16_gates():
    # the update path's dtypes: fp32 conv output, bf16 gate pre-activations
    R, T, D = 32, 64, 128
    x, gates, h0, done = _seq_inputs(9, R, T, D, torch.float32, torch.bfloat16, 0.05)
    g = torch.Generator().manual_seed(2)
    wy, wl = torch.randn(R, T, D, generator=g), torch.randn(R, D, generator=g)
    lam = torch.linspace(0.0, 4.0, D)
    want = _scan_grads_oracle(x, gates.float(), lam, h0, done, wy, wl)  # exact gradients at the rounded inputs
    leaves = [t.to(DEV).requires_grad_(True) for t in (x, gates, lam, h0)]
    y, last = ops.rglru_scan(leaves[0], leaves[1], leaves[2], 8.0, leaves[3], done.to(DEV))
    ((y * wy.to(DEV)).sum() + (last * wl.to(DEV)).sum()).backward()
    assert leaves[1].grad.dtype == torch.bfloat16
    for got, ref in zip((t.grad for t in leaves), want):
        assert max_rel(got.float().cpu(), ref) <= BF16_TOL


# ------------------------------------------------------------------ fused sublayer tail (add + norm + gated MLP + add)


def _ffn_case(seed, R):
    g = torch.Generator().manual_seed(seed)
    D, Hd = 128, 512
    x = torch.randn(R, D, generator=g)
    delta = (0.5 * torch.randn(R, D, generator=g)).bfloat16()
    nw = 1.0 + 0.1 * torch.randn(D, generator=g)
    p = {"f.gate_proj.weight": torch.randn(Hd, D, generator=g) / D ** 0.5,
         "f.up_proj.weight": torch.randn(Hd, D, generator=g) / D ** 0.5,
         "f.down_proj.weight": torch.randn(D, Hd, generator=g) / Hd ** 0.5}
    return x, delta, nw, p


@pytest.mark.parametrize("R", [1, 31, 128, 129, 1000, 40000])
@pytest.mark.parametrize("with_delta", [True, False])
def test_ffn_fused_matches_oracle(R, with_delta):
    x, delta, nw, p = _ffn_case(R, R)
    rounded = {k: v.bfloat16().float() for k, v in p.items()}  # the projections run on bf16 weights
    s = x + delta.float() if with_delta else x
    want = s + torch_ref.gated_mlp(rounded, "f.", torch_ref.rms_norm(s, nw))
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    got = ops.ffn_fused(x.to(DEV), delta.to(DEV) if with_delta else None, nw.to(DEV), pk)
    assert got.shape == (R, 128) and got.dtype == torch.float32
    assert max_rel(got.cpu(), want) <= BF16_TOL
    # the MLP contribution alone (the residual would otherwise hide an error in it)
    assert max_rel(got.cpu() - s, want - s) <= BF16_TOL


def test_ffn_fused_every_weight_reaches_its_output():
    # one-hot weights: hidden unit j and output channel k are hit exactly where the layout says
    D, Hd = 128, 512
    x = torch.zeros(64, D)
    x[:, 5] = 1.0  # after the norm every channel but 5 is zero
    nw = torch.ones(D)
    for j, k in [(0, 0), (37, 100), (511, 127), (300, 9)]:
        wg, wu, wd = torch.zeros(Hd, D), torch.zeros(Hd, D), torch.zeros(D, Hd)
        wg[j, 5], wu[j, 5], wd[k, j] = 1.0, 2.0, 3.0
        pk = ops.pack_ffn_weights(wg.to(DEV), wu.to(DEV), wd.to(DEV))
        got = ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk).cpu() - x
        n5 = torch_ref.rms_norm(x, nw)[0, 5].bfloat16().float()
        h = (torch.nn.functional.gelu(n5).bfloat16().float() * (2.0 * n5).bfloat16().float()).bfloat16().float()
        want = torch.zeros(D)
        want[k] = 3.0 * h
        assert torch.allclose(got[0], want, rtol=1e-2, atol=1e-6), (j, k)
        assert torch.equal(got[0], got[63])


# ------------------------------------------------------------------ the gated MLP in the update: fused forward, recompute-backward


def _ffn_bwd_reference(n, dy, p):
    """float64 autograd through the oracle's gated MLP on the bf16-rounded operands the kernel sees."""
    w = {k: v.bfloat16().double().requires_grad_() for k, v in p.items()}
    nd = n.double().requires_grad_()
    a = torch.nn.functional.linear(nd, w["f.gate_proj.weight"])
    b = torch.nn.functional.linear(nd, w["f.up_proj.weight"])
    a.retain_grad(), b.retain_grad()
    hid = torch.nn.functional.gelu(a) * b
    y = torch.nn.functional.linear(hid, w["f.down_proj.weight"])
    assert torch.allclose(y, torch_ref.gated_mlp({k: v.detach() for k, v in w.items()}, "f.", nd.detach()), rtol=1e-12, atol=1e-12)
    y.backward(dy.bfloat16().double())
    return hid.detach(), a.grad, b.grad, nd.grad, w


@pytest.mark.parametrize("R", [1, 31, 256, 257, 1000, 20000])
@pytest.mark.parametrize("dy_dtype", [torch.float32, torch.bfloat16])
def test_ffn_bwd_matches_autograd_of_the_oracle(R, dy_dtype):
    _, _, _, p = _ffn_case(R + 3, R)
    g = torch.Generator().manual_seed(R)
    n = torch.randn(R, 128, generator=g).bfloat16()
    dy = torch.randn(R, 128, generator=g).to(dy_dtype)
    hid, da, db, dn_ref, w = _ffn_bwd_reference(n, dy.float(), p)
    pk = ops.pack_ffn_bwd_weights(*(p[k].to(DEV) for k in ("f.gate_proj.weight", "f.up_proj.weight", "f.down_proj.weight")))
    dn, dgu, h, dy_lp = ops.ffn_bwd(n.to(DEV), dy.to(DEV), pk)
    assert dn.shape == (R, 128) and dn.dtype == torch.bfloat16 and dgu.shape[0] == 8 and h.shape[0] == 4
    assert torch.equal(dy_lp.cpu(), dy.bfloat16())
    h_rows = h[:, :R].permute(1, 0, 2).reshape(R, 512).float().cpu()
    t = dgu[:, :R].permute(1, 0, 2).reshape(R, 8, 2, 2, 32).float().cpu()  # [row][pair][chunk in pair][gate, up][unit]
    assert max_rel(h_rows, hid.float()) <= BF16_TOL
    assert max_rel(t[:, :, :, 0].reshape(R, 512), da.float()) <= BF16_TOL
    assert max_rel(t[:, :, :, 1].reshape(R, 512), db.float()) <= BF16_TOL
    assert max_rel(dn.float().cpu(), dn_ref.float()) <= BF16_TOL
    d_gate, d_up, d_down = ops.ffn_weight_grads(n.to(DEV), dgu, h, dy_lp)
    assert max_rel(d_gate.cpu(), w["f.gate_proj.weight"].grad.float()) <= BF16_TOL
    assert max_rel(d_up.cpu(), w["f.up_proj.weight"].grad.float()) <= BF16_TOL
    assert max_rel(d_down.cpu(), w["f.down_proj.weight"].grad.float()) <= BF16_TOL
    # fixed-order reductions: repeated calls give identical bits
    again = ops.ffn_bwd(n.to(DEV), dy.to(DEV), pk)
    assert torch.equal(again[0], dn) and torch.equal(again[1][:, :R], dgu[:, :R]) and torch.equal(again[2][:, :R], h[:, :R])


def test_ffn_bwd_at_update_size_on_sampled_rows():
    # the update's row count at 4v4 (128 steps x 256 environments x 12 tokens): six rounds of resident work-groups
    R = 128 * 256 * 12
    _, _, _, p = _ffn_case(77, 1)
    g = torch.Generator(device=DEV).manual_seed(78)
    n = torch.randn(R, 128, device=DEV, generator=g).bfloat16()
    dy = torch.randn(R, 128, device=DEV, generator=g)
    pk = ops.pack_ffn_bwd_weights(*(p[k].to(DEV) for k in ("f.gate_proj.weight", "f.up_proj.weight", "f.down_proj.weight")))
    dn, dgu, h, dy_lp = ops.ffn_bwd(n, dy, pk)
    pick = torch.arange(0, R, 3001, device=DEV)
    hid, da, db, dn_ref, _ = _ffn_bwd_reference(n[pick].cpu(), dy[pick].cpu(), p)
    P = pick.numel()
    assert max_rel(h[:, pick].permute(1, 0, 2).reshape(P, 512).float().cpu(), hid.float()) <= BF16_TOL
    t = dgu[:, pick].permute(1, 0, 2).reshape(P, 8, 2, 2, 32).float().cpu()
    assert max_rel(t[:, :, :, 0].reshape(P, 512), da.float()) <= BF16_TOL
    assert max_rel(t[:, :, :, 1].reshape(P, 512), db.float()) <= BF16_TOL
    assert max_rel(dn[pick].float().cpu(), dn_ref.float()) <= BF16_TOL
    assert torch.isfinite(dn.float()).all()
    # a row's results do not depend on where or when it is computed: bit for bit under a row permutation
    perm = torch.randperm(R, device=DEV, generator=g)
    dn_p, dgu_p, h_p, _ = ops.ffn_bwd(n[perm], dy[perm], pk)
    assert torch.equal(dn_p, dn[perm]) and torch.equal(dgu_p[:, :R], dgu[:, perm]) and torch.equal(h_p[:, :R], h[:, perm])
    # weight gradients against float32 products of the very operands the kernel stored
    d_gate, d_up, d_down = ops.ffn_weight_grads(n, dgu, h, dy_lp)
    tt = dgu[:, :R].permute(1, 0, 2).reshape(R, 8, 2, 2, 32).float()
    nf = n.float()
    assert max_rel(d_gate, tt[:, :, :, 0].reshape(R, 512).t() @ nf) <= 1e-3
    assert max_rel(d_up, tt[:, :, :, 1].reshape(R, 512).t() @ nf) <= 1e-3
    assert max_rel(d_down, dy_lp.float().t() @ h[:, :R].permute(1, 0, 2).reshape(R, 512).float()) <= 1e-3


def test_ffn_bwd_every_weight_reaches_its_gradient():
    # one-hot weights: the packed operand order, the tile layout of the results and the weight-gradient un-permutation
    # must each put hidden unit j and channel k where the layout says
    D, Hd, R = 128, 512, 64
    n = torch.zeros(R, D)
    n[:, 5] = 1.5
    dy = torch.zeros(R, D)
    for j, k in [(0, 0), (37, 100), (511, 127), (300, 9), (140, 64)]:
        wg, wu, wd = torch.zeros(Hd, D), torch.zeros(Hd, D), torch.zeros(D, Hd)
        wg[j, 5], wu[j, 5], wd[k, j] = 1.0, 2.0, 3.0
        dy.zero_()
        dy[:, k] = 0.5
        pk = ops.pack_ffn_bwd_weights(wg.to(DEV), wu.to(DEV), wd.to(DEV))
        dn, dgu, h, dy_lp = ops.ffn_bwd(n.bfloat16().to(DEV), dy.to(DEV), pk)
        a, b, dh = 1.5, 3.0, 1.5  # gate, up, gradient of the hidden unit
        cdf = 0.5 * (1.0 + math.erf(a / 2 ** 0.5))
        pdf = math.exp(-a * a / 2) / (2 * math.pi) ** 0.5
        h_rows = h[:, :R].permute(1, 0, 2).reshape(R, Hd).float().cpu()
        want_h = torch.zeros(Hd)
        want_h[j] = a * cdf * b
        assert torch.allclose(h_rows[0], want_h, rtol=1e-2, atol=1e-6), (j, k)
        t = dgu[:, :R].permute(1, 0, 2).reshape(R, 8, 2, 2, 32).float().cpu()
        want_g, want_u = torch.zeros(Hd), torch.zeros(Hd)
        want_g[j], want_u[j] = dh * b * (cdf + a * pdf), dh * a * cdf
        assert torch.allclose(t[0, :, :, 0].reshape(Hd), want_g, rtol=1e-2, atol=1e-6), (j, k)
        assert torch.allclose(t[0, :, :, 1].reshape(Hd), want_u, rtol=1e-2, atol=1e-6), (j, k)
        want_n = torch.zeros(D)
        want_n[5] = float(want_g[j]) * 1.0 + float(want_u[j]) * 2.0
        assert torch.allclose(dn[0].float().cpu(), want_n, rtol=2e-2, atol=1e-6), (j, k)
        assert torch.equal(dn[0], dn[R - 1])
        d_gate, d_up, d_down = ops.ffn_weight_grads(n.bfloat16().to(DEV), dgu, h, dy_lp)
        hot = torch.zeros(Hd, D)
        hot[j, 5] = 1.0
        got_g = t[0, :, :, 0].reshape(Hd)[j].item()
        assert torch.allclose(d_gate.cpu(), hot * (R * 1.5 * got_g), rtol=1e-2, atol=1e-5), (j, k)
        assert d_down.cpu()[k, j] != 0 and d_down.cpu().count_nonzero() == 1, (j, k)


@pytest.mark.parametrize("R", [1, 300, 5000])
@pytest.mark.parametrize("with_delta", [True, False])
def test_ffn_tail_train_matches_the_inference_kernel_and_autograd_of_the_oracle(R, with_delta):
    x, delta, nw, p = _ffn_case(R + 11, R)
    names = ("f.gate_proj.weight", "f.up_proj.weight", "f.down_proj.weight")
    ws = [p[k].to(DEV).requires_grad_() for k in names]
    pf, pb = ops.pack_ffn_weights(*ws), ops.pack_ffn_bwd_weights(*ws)
    xg = x.to(DEV).requires_grad_()
    dg = delta.to(DEV).requires_grad_() if with_delta else None
    nwg = nw.to(DEV).requires_grad_()
    out = ops.ffn_tail_train(xg, dg, nwg, *ws, eps=None, packed_fwd=pf, packed_bwd=pb)
    with torch.no_grad():
        assert torch.equal(out, ops.ffn_fused(x.to(DEV), delta.to(DEV) if with_delta else None, nw.to(DEV), pf))
    g = torch.Generator().manual_seed(R + 1)
    up = torch.randn(R, 128, generator=g)
    out.backward(up.to(DEV))
    # float64 autograd through the oracle on the bf16-rounded weights
    wd = {k: p[k].bfloat16().double().requires_grad_() for k in names}
    xd = x.double().requires_grad_()
    dd = delta.double().requires_grad_()
    nwd = nw.double().requires_grad_()
    s = xd + dd if with_delta else xd
    (s + torch_ref.gated_mlp(wd, "f.", torch_ref.rms_norm(s, nwd))).backward(up.double())
    assert max_rel(xg.grad.cpu(), xd.grad.float()) <= BF16_TOL
    if with_delta:
        assert dg.grad.dtype == torch.bfloat16 and max_rel(dg.grad.float().cpu(), dd.grad.float()) <= BF16_TOL
    assert max_rel(nwg.grad.cpu(), nwd.grad.float()) <= BF16_TOL
    for w_, k in zip(ws, names):
        assert max_rel(w_.grad.cpu(), wd[k].grad.float()) <= BF16_TOL, k


@pytest.mark.parametrize("R", [1, 300, 5000])
def test_ffn_tail_train_with_the_output_projection_inside_matches_autograd_of_the_oracle(R):
    x, _, nw, p = _ffn_case(R + 17, R)
    g = torch.Generator().manual_seed(R + 2)
    names = ("f.gate_proj.weight", "f.up_proj.weight", "f.down_proj.weight")
    Wp = torch.randn(128, 128, generator=g) / 128 ** 0.5
    rows = torch.randn(R, 128, generator=g).bfloat16()
    ws = [p[k].to(DEV).requires_grad_() for k in names]
    wp = Wp.to(DEV).requires_grad_()
    pf, pb, pp = ops.pack_ffn_weights(*ws), ops.pack_ffn_bwd_weights(*ws), ops.pack_proj_weights(wp)
    xg, rg, nwg = x.to(DEV).requires_grad_(), rows.to(DEV).requires_grad_(), nw.to(DEV).requires_grad_()
    out = ops.ffn_tail_train(xg, rg, nwg, *ws, eps=None, packed_fwd=pf, packed_bwd=pb, proj_weight=wp, proj_packed=pp)
    with torch.no_grad():
        assert torch.equal(out, ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pf, proj=(rows.to(DEV), pp)))
    up = torch.randn(R, 128, generator=g)
    out.backward(up.to(DEV))
    wd = {k: p[k].bfloat16().double().requires_grad_() for k in names}
    xd, rd, nwd = x.double().requires_grad_(), rows.double().requires_grad_(), nw.double().requires_grad_()
    wpd = Wp.bfloat16().double().requires_grad_()
    s = xd + rd @ wpd.t()
    (s + torch_ref.gated_mlp(wd, "f.", torch_ref.rms_norm(s, nwd))).backward(up.double())
    assert max_rel(xg.grad.cpu(), xd.grad.float()) <= BF16_TOL
    assert rg.grad.dtype == torch.bfloat16 and max_rel(rg.grad.float().cpu(), rd.grad.float()) <= BF16_TOL
    assert max_rel(wp.grad.cpu(), wpd.grad.float()) <= BF16_TOL
    assert max_rel(nwg.grad.cpu(), nwd.grad.float()) <= BF16_TOL
    for w_, k in zip(ws, names):
        assert max_rel(w_.grad.cpu(), wd[k].grad.float()) <= BF16_TOL, k


# ------------------------------------------------------------------ rows addressed inside a wider (B, N+M, D) token tensor


@pytest.mark.parametrize("B,n,NM", [(3, 8, 12), (5, 19, 23), (1, 4, 9), (600, 8, 12)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_state_kernels_address_ship_rows_inside_the_token_tensor(B, n, NM, dtype):
    D = 128
    g = torch.Generator().manual_seed(B * 31 + NM)
    tokens = torch.randn(B, NM, D, generator=g).to(dtype).to(DEV)   # linear1 outputs of all tokens
    buf = torch.randn(B * n, 3, D, generator=g).to(DEV)
    w = (0.5 * torch.randn(D, 1, 4, generator=g)).to(DEV)
    bias = (0.1 * torch.randn(D, generator=g)).to(DEV)
    reset = (torch.rand(B, generator=g) < 0.4).to(DEV)
    view = tokens[:, :n]
    v_a, buf_a = ops.conv_step(view, buf, w, bias, reset=reset, rows_per_env=n)
    v_b, buf_b = ops.conv_step(view.reshape(B * n, D).contiguous(), buf, w, bias, reset=reset, rows_per_env=n)
    assert torch.equal(v_a, v_b) and torch.equal(buf_a, buf_b)
    # recurrence output written into the first n tokens of a wider tensor, the rest untouched
    gates = torch.randn(B * n, 2 * D, generator=g).to(dtype).to(DEV)
    h = torch.randn(B * n, D, generator=g).to(DEV)
    lam = torch.linspace(0.0, 4.0, D).to(DEV)
    for y_dtype in (torch.float32, torch.bfloat16):
        wide = torch.full((B, NM, D), 7.0, dtype=y_dtype, device=DEV)
        y, h_new = ops.rglru_step(v_a, gates, lam, 8.0, h, reset=reset, rows_per_env=n, y_out=wide[:, :n])
        y_ref, h_ref = ops.rglru_step(v_a, gates, lam, 8.0, h, reset=reset, rows_per_env=n, y_dtype=y_dtype)
        assert torch.equal(h_new, h_ref)
        assert torch.equal(wide[:, :n].reshape(B * n, D), y_ref.to(y_dtype))
        assert (wide[:, n:] == 7.0).all()
    # no reset mask: the grouping alone still needs rows_per_env
    wide = torch.zeros((B, NM, D), dtype=torch.float32, device=DEV)
    ops.rglru_step(v_a, gates, lam, 8.0, h, rows_per_env=n, y_out=wide[:, :n])
    assert torch.equal(wide[:, :n].reshape(B * n, D), ops.rglru_step(v_a, gates, lam, 8.0, h)[1])
    with pytest.raises(ValueError):
        ops.rglru_step(v_a, gates, lam, 8.0, h, rows_per_env=n + 1, y_out=wide[:, :n])


# ------------------------------------------------------------------ conv + gate projections + recurrence in one kernel


def _temporal_inputs(seed, R, D=128):
    g = torch.Generator().manual_seed(seed)
    return dict(
        b1=torch.randn(R, D, generator=g).to(torch.bfloat16),
        buf=torch.randn(R, 3, D, generator=g),
        h=0.5 * torch.randn(R, D, generator=g),
        cw=0.5 * torch.randn(D, 1, 4, generator=g),
        cb=0.1 * torch.randn(D, generator=g),
        wa=torch.randn(D, D, generator=g) / D ** 0.5,
        wx=torch.randn(D, D, generator=g) / D ** 0.5,
        ba=0.3 * torch.randn(D, generator=g),
        bx=0.3 * torch.randn(D, generator=g),
        lam=torch.linspace(0.0, 4.0, D),
    )


def _temporal_truth(t, reset=None, rows_per_env=1):
    """fp32 statement on the same (already rounded) inputs: conv taps, gate projections of the
    unrounded conv output, recurrence.  Returns (h', shifted buffer)."""
    b1 = t["b1"].float()
    buf, h = t["buf"].clone(), t["h"].clone()
    if reset is not None:
        rows = reset.repeat_interleave(rows_per_env)
        buf[rows] = 0.0
        h[rows] = 0.0
    w = t["cw"].reshape(-1, 4)
    v = buf[:, 0] * w[:, 0] + buf[:, 1] * w[:, 1] + buf[:, 2] * w[:, 2] + b1 * w[:, 3] + t["cb"]
    wa, wx = t["wa"].to(torch.bfloat16).float(), t["wx"].to(torch.bfloat16).float()
    gates = torch.cat([v @ wa.t() + t["ba"], v @ wx.t() + t["bx"]], dim=1)
    h_new = torch_ref.rglru_step(v, gates, t["lam"], 8.0, h)
    return h_new, torch.stack([buf[:, 1], buf[:, 2], b1], dim=1)


@pytest.mark.parametrize("R", [1, 31, 32, 33, 257, 5000, 70001])
@pytest.mark.parametrize("with_reset", [False, True])
def test_temporal_step_matches_oracle_and_the_three_kernel_composition(R, with_reset):
    t = _temporal_inputs(R, R)
    d = {k: v.to(DEV) for k, v in t.items()}
    reset = None
    if with_reset:
        reset = torch.rand(R, generator=torch.Generator().manual_seed(R)) < 0.3
    rdev = None if reset is None else reset.to(DEV)
    pk = ops.pack_gate_weights(d["wa"], d["wx"])
    gb = torch.cat([d["ba"], d["bx"]])
    y, h_new, buf_new = ops.temporal_step(d["b1"], d["buf"], d["h"], d["cw"], d["cb"], pk, gb, d["lam"], 8.0, reset=rdev)
    torch.cuda.synchronize()
    h_true, buf_true = _temporal_truth(t, reset)
    assert torch.equal(buf_new.cpu(), buf_true)  # the buffer shift only moves values
    assert max_rel(h_new.cpu(), h_true) <= BF16_TOL
    assert torch.equal(y, h_new.to(torch.bfloat16))
    # the composition it replaces: conv kernel, library GEMM on the bf16 conv output, recurrence kernel
    v, buf_c, v_lp = ops.conv_step(d["b1"], d["buf"], d["cw"], d["cb"], reset=rdev, also_bf16=True)
    gates = torch.nn.functional.linear(v_lp, torch.cat([d["wa"], d["wx"]]).to(torch.bfloat16), gb.to(torch.bfloat16))
    y_c, h_c = ops.rglru_step(v, gates, d["lam"], 8.0, d["h"], reset=rdev, y_dtype=torch.bfloat16)
    assert torch.equal(buf_new, buf_c)
    # same rounding points; the conv arithmetic may differ in the last fp32 bit and the summation
    # order inside the projections now and then moves a pre-activation by one bf16 ulp
    assert max_rel(h_new, h_c) <= 8e-3
    assert (y == y_c).float().mean().item() >= 0.999
    off = ((h_new - h_c).abs() > 1e-5 * h_c.abs().clamp_min(1e-2)).float().mean().item()
    assert off <= 1e-3, off
    assert max_rel(h_c.cpu(), h_true) <= BF16_TOL


def test_temporal_step_every_gate_weight_reaches_its_channel():
    # one-hot gate weights: channel j of gate g sees exactly conv-output channel perm[j]; any
    # slip in the operand packing or in the channel order of the exchange shows as a mismatch
    R, D = 64, 128
    t = _temporal_inputs(5, R)
    g = torch.Generator().manual_seed(6)
    pa, px = torch.randperm(D, generator=g), torch.randperm(D, generator=g)
    t["wa"] = torch.zeros(D, D)
    t["wa"][torch.arange(D), pa] = 2.0
    t["wx"] = torch.zeros(D, D)
    t["wx"][torch.arange(D), px] = -1.5
    d = {k: v.to(DEV) for k, v in t.items()}
    _, h_new, _ = ops.temporal_step(d["b1"], d["buf"], d["h"], d["cw"], d["cb"], ops.pack_gate_weights(d["wa"], d["wx"]),
                                    torch.cat([d["ba"], d["bx"]]), d["lam"], 8.0)
    h_true, _ = _temporal_truth(t)
    assert max_rel(h_new.cpu(), h_true) <= BF16_TOL
    # elementwise too: a swapped pair of channels would hide inside a max-norm bound less easily here
    assert torch.allclose(h_new.cpu(), h_true, rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("B,n,NM", [(3, 8, 12), (5, 19, 23), (600, 8, 12), (7, 152, 160)])
def test_temporal_step_reads_and_writes_ship_rows_inside_wider_tensors(B, n, NM):
    D, R = 128, B * n
    t = _temporal_inputs(B + NM, R)
    d = {k: v.to(DEV) for k, v in t.items()}
    g = torch.Generator().manual_seed(B)
    both = torch.randn(B, NM, 2 * D, generator=g).to(torch.bfloat16).to(DEV)  # [linear1 | linear2] of all tokens
    both[:, :n, :D] = d["b1"].view(B, n, D)
    reset = (torch.rand(B, generator=g) < 0.4).to(DEV)
    pk, gb = ops.pack_gate_weights(d["wa"], d["wx"]), torch.cat([d["ba"], d["bx"]])
    # packed state rows [h | p0 | p1 | p2], read from one tensor and written into another
    state_in = torch.cat([d["h"], d["buf"].reshape(R, 3 * D)], dim=1)
    state_out = torch.full_like(state_in, 3.0)
    wide = torch.full((B, NM, D), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.temporal_step(both[:, :n, :D], state_in[:, D:].view(R, 3, D), state_in[:, :D], d["cw"], d["cb"], pk, gb, d["lam"], 8.0,
                      conv_out=state_out[:, D:].view(R, 3, D), h_out=state_out[:, :D], y_out=wide[:, :n], reset=reset,
                      rows_per_env=n)
    y_ref, h_ref, buf_ref = ops.temporal_step(d["b1"], d["buf"], d["h"], d["cw"], d["cb"], pk, gb, d["lam"], 8.0, reset=reset,
                                              rows_per_env=n)
    assert torch.equal(state_out[:, :D], h_ref) and torch.equal(state_out[:, D:].view(R, 3, D), buf_ref)
    assert torch.equal(wide[:, :n].reshape(R, D), y_ref)
    assert (wide[:, n:] == 7.0).all()
    # in place: the state may be updated where it lives
    ops.temporal_step(d["b1"], state_in[:, D:].view(R, 3, D), state_in[:, :D], d["cw"], d["cb"], pk, gb, d["lam"], 8.0,
                      conv_out=state_in[:, D:].view(R, 3, D), h_out=state_in[:, :D], reset=reset, rows_per_env=n)
    assert torch.equal(state_in, state_out)


def test_temporal_step_rejects_what_it_does_not_cover():
    t = {k: v.to(DEV) for k, v in _temporal_inputs(1, 4).items()}
    pk, gb = ops.pack_gate_weights(t["wa"], t["wx"]), torch.cat([t["ba"], t["bx"]])
    with pytest.raises(ValueError):
        ops.temporal_step(t["b1"].float(), t["buf"], t["h"], t["cw"], t["cb"], pk, gb, t["lam"], 8.0)
    with pytest.raises(ValueError):
        ops.temporal_step(t["b1"], t["buf"][:3], t["h"], t["cw"], t["cb"], pk, gb, t["lam"], 8.0)
    with pytest.raises(ValueError):
        ops.temporal_step(t["b1"], t["buf"], t["h"], t["cw"], t["cb"], pk.reshape(-1), gb, t["lam"], 8.0)
    with pytest.raises(ValueError):
        ops.pack_gate_weights(torch.zeros(64, 64, device=DEV), torch.zeros(64, 64, device=DEV))
    empty = ops.temporal_step(t["b1"][:0], t["buf"][:0], t["h"][:0], t["cw"], t["cb"], pk, gb, t["lam"], 8.0)
    assert empty[0].shape == (0, 128) and empty[1].shape == (0, 128) and empty[2].shape == (0, 3, 128)


# ------------------------------------------------------------------ RMSNorm + Linear, compact row lists


@pytest.mark.parametrize("R,N", [(1, 64), (33, 128), (128, 256), (1000, 384), (70000, 256)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_norm_linear_matches_oracle(R, N, with_bias):
    g = torch.Generator().manual_seed(R + N)
    D = 128
    x = 2.0 * torch.randn(R, D, generator=g)
    nw = 1.0 + 0.1 * torch.randn(D, generator=g)
    W = torch.randn(N, D, generator=g) / D ** 0.5
    bias = 0.2 * torch.randn(N, generator=g) if with_bias else None
    want = torch.nn.functional.linear(torch_ref.rms_norm(x, nw), W.bfloat16().float(), bias)
    got = ops.norm_linear(x.to(DEV), nw.to(DEV), ops.pack_linear_weights(W.to(DEV)), None if bias is None else bias.to(DEV))
    assert got.shape == (R, N) and got.dtype == torch.bfloat16
    assert max_rel(got.float().cpu(), want) <= BF16_TOL


def test_norm_linear_one_hot_weights_hit_the_documented_positions():
    D, N = 128, 128
    x = torch.zeros(40, D)
    x[:, 77] = 3.0
    nw = torch.ones(D)
    for f in (0, 5, 31, 64, 127):
        W = torch.zeros(N, D)
        W[f, 77] = 1.0
        got = ops.norm_linear(x.to(DEV), nw.to(DEV), ops.pack_linear_weights(W.to(DEV))).float().cpu()
        n77 = float(torch_ref.rms_norm(x, nw)[0, 77])
        want = torch.zeros(N)
        want[f] = n77
        assert torch.allclose(got[0], want, rtol=1e-2, atol=1e-6), f
        assert torch.equal(got[0], got[39])


@pytest.mark.parametrize("B,n,p", [(1, 1, 1.0), (5, 80, 0.3), (7, 190, 0.0), (40, 1520, 0.25), (3, 2048, 1.0)])
def test_compact_rows_and_gathered_projection(B, n, p):
    g = torch.Generator().manual_seed(B * 7 + n)
    mask = torch.rand(B, n, generator=g) < p
    rows = ops.CompactRows(mask.to(DEV))
    counts = mask.sum(1)
    offs = torch.cat([torch.zeros(1, dtype=torch.long), counts.cumsum(0)])
    assert torch.equal(rows.offsets.cpu().long(), offs)
    total = int(offs[-1])
    assert torch.equal(rows.index[:total].cpu().long(), mask.flatten().nonzero().flatten())
    # projection over the listed rows only
    D, N = 128, 256
    x = torch.randn(B, n, D, generator=g)
    nw = 1.0 + 0.1 * torch.randn(D, generator=g)
    W = torch.randn(N, D, generator=g) / D ** 0.5
    out = ops.norm_linear(x.to(DEV), nw.to(DEV), ops.pack_linear_weights(W.to(DEV)), rows=rows)
    assert out.shape == (B * n, N)
    if total:
        want = torch.nn.functional.linear(torch_ref.rms_norm(x.reshape(-1, D)[mask.flatten()], nw), W.bfloat16().float())
        assert max_rel(out[:total].float().cpu(), want) <= BF16_TOL


@pytest.mark.parametrize("B,NQ,NK,p", [(4, 12, 80, 0.5), (3, 84, 800, 0.3), (3, 156, 1520, 0.1), (2, 33, 3000, 0.6), (5, 20, 190, 0.0),
                                       (3, 131, 900, 0.4), (4, 160, 1520, 0.02)])
def test_sdpa_cross_over_compacted_rows_equals_the_masked_form(B, NQ, NK, p):
    H, D = 4, 128
    g = torch.Generator().manual_seed(NQ * 13 + NK)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16().to(DEV)
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16().to(DEV)
    mask = torch.rand(B, NK, generator=g) < p
    mask[0] = False
    if p > 0:
        mask[1, NK - 1] = True
    mask = mask.to(DEV)
    rows = ops.CompactRows(mask)
    kv_rows = torch.zeros(B * NK, 2 * D, dtype=torch.bfloat16, device=DEV)
    total = int(rows.total.item())
    kv_rows[:total] = kv.reshape(B * NK, 2 * D)[rows.index[:total].long()]
    bare = ops.sdpa_cross_rows(qkv, kv_rows, rows, H)
    truth = torch_ref.bullet_read(qkv.float().cpu(), kv.float().cpu(), mask.cpu(), H)
    assert bare[0].abs().max() == 0
    if truth.abs().max() > 0:
        assert max_rel(bare.float().cpu(), truth) <= BF16_TOL
    merged = torch.randn(B, NQ, D, generator=g).bfloat16().to(DEV)
    got = ops.sdpa_cross_rows(qkv, kv_rows, rows, H, accum=merged.clone())
    assert torch.equal(got, merged + bare)
    if 160 < NK <= 2048:  # the masked form on the same kernel: same keys in the same order, bit for bit
        assert torch.equal(got, ops.sdpa_cross(qkv, kv, mask, H, accum=merged.clone()))


@pytest.mark.parametrize("R", [1, 130, 5000])
@pytest.mark.parametrize("gated", [False, True])
def test_ffn_fused_with_folded_projection_matches_oracle(R, gated):
    x, _, nw, p = _ffn_case(R + 7, R)
    g = torch.Generator().manual_seed(R)
    D = 128
    Wp = torch.randn(D, D, generator=g) / D ** 0.5
    rows_a = torch.randn(R, D, generator=g).bfloat16()
    rows_y = torch.randn(R, D, generator=g).bfloat16()
    rounded = {k: v.bfloat16().float() for k, v in p.items()}
    operand = rows_a.float()
    if gated:
        operand = (torch.nn.functional.gelu(rows_a.float()).bfloat16().float() * rows_y.float()).bfloat16().float()
    s = x + operand @ Wp.bfloat16().float().t()
    want = s + torch_ref.gated_mlp(rounded, "f.", torch_ref.rms_norm(s, nw))
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    wp = ops.pack_proj_weights(Wp.to(DEV))
    proj = (rows_a.to(DEV), rows_y.to(DEV), wp) if gated else (rows_a.to(DEV), wp)
    got = ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, proj=proj)
    assert max_rel(got.cpu(), want) <= BF16_TOL
    assert max_rel(got.cpu() - x, want - x) <= BF16_TOL
    # the folded projection against the same projection done outside (bf16 GEMM output as delta)
    delta = (operand @ Wp.bfloat16().float().t()).bfloat16()
    two_step = ops.ffn_fused(x.to(DEV), delta.to(DEV), nw.to(DEV), pk)
    assert max_rel(got.cpu(), two_step.cpu()) <= 1e-2


@pytest.mark.parametrize("R,N", [(1, 128), (37, 384), (128, 256), (130, 384), (5000, 256), (4096, 384), (700, 192), (3000, 320),
                                 (260, 640)])
@pytest.mark.parametrize("gated", [False, True])
def test_ffn_fused_with_the_next_sublayers_head_matches_oracle(R, N, gated):
    # the same launch goes on to rmsnorm(out) * w2 -> bf16 -> @ Wh^T, the projection the next sublayer starts with
    x, _, nw, p = _ffn_case(R + N, R)
    g = torch.Generator().manual_seed(R * 3 + N)
    D = 128
    Wp = torch.randn(D, D, generator=g) / D ** 0.5
    Wh = torch.randn(N, D, generator=g) / D ** 0.5
    nw2 = 1.0 + 0.2 * torch.randn(D, generator=g)
    rows_a = torch.randn(R, D, generator=g).bfloat16()
    rows_y = torch.randn(R, D, generator=g).bfloat16()
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    wp = ops.pack_proj_weights(Wp.to(DEV))
    proj = (rows_a.to(DEV), rows_y.to(DEV), wp) if gated else (rows_a.to(DEV), wp)
    plain = ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, proj=proj)
    out, head = ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, proj=proj,
                              next_head=(nw2.to(DEV), None, ops.pack_head_weights(Wh.to(DEV)), N))
    assert torch.equal(out, plain)  # the tail itself is the same arithmetic
    assert head.shape == (R, N) and head.dtype == torch.bfloat16 and head.is_contiguous()
    # the oracle's norm + Linear on the rows the kernel produced
    want = torch.nn.functional.linear(torch_ref.rms_norm(plain.cpu(), nw2), Wh.bfloat16().float())
    assert max_rel(head.float().cpu(), want) <= BF16_TOL
    # and against the stand-alone norm + projection kernel on the same rows: two bf16 roundings of one product
    alone = ops.norm_linear(plain, nw2.to(DEV), ops.pack_linear_weights(Wh.to(DEV)))
    assert max_rel(head.float().cpu(), alone.float().cpu()) <= BF16_TOL


def test_next_head_one_hot_weights_hit_the_documented_positions():
    D, N, R = 128, 384, 70
    x, _, nw, p = _ffn_case(11, R)
    g = torch.Generator().manual_seed(5)
    rows_a = torch.randn(R, D, generator=g).bfloat16().to(DEV)
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    wp = ops.pack_proj_weights((torch.randn(D, D, generator=g) / D ** 0.5).to(DEV))
    nw2 = torch.ones(D)
    plain = ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, proj=(rows_a, wp)).cpu()
    normed = torch_ref.rms_norm(plain, nw2).bfloat16().float()
    for f, k in ((0, 0), (5, 77), (63, 127), (64, 3), (200, 64), (383, 31)):
        Wh = torch.zeros(N, D)
        Wh[f, k] = 1.0
        _, head = ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, proj=(rows_a, wp),
                                next_head=(nw2.to(DEV), None, ops.pack_head_weights(Wh.to(DEV)), N))
        head = head.float().cpu()
        assert torch.allclose(head[:, f], normed[:, k], rtol=1e-2, atol=1e-6), (f, k)
        head[:, f] = 0
        assert head.abs().max() == 0, (f, k)


def test_next_head_refuses_what_the_kernel_does_not_cover():
    x, _, nw, p = _ffn_case(2, 16)
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    nw2 = torch.ones(128, device=DEV)
    hp = ops.pack_head_weights(torch.zeros(256, 128, device=DEV))
    with pytest.raises(ValueError):  # only with the folded projection
        ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, next_head=(nw2, None, hp, 256))
    wp = ops.pack_proj_weights(torch.zeros(128, 128, device=DEV))
    rows = torch.zeros(16, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):  # feature count and pack disagree
        ops.ffn_fused(x.to(DEV), None, nw.to(DEV), pk, proj=(rows, wp), next_head=(nw2, None, hp, 384))
    with pytest.raises(ValueError):
        ops.pack_head_weights(torch.zeros(96, 128, device=DEV))
    from boost_and_broadside_amd import _native

    lib = _native.load()
    out = torch.empty(16, 128, device=DEV)
    head = torch.empty(128, 256, dtype=torch.bfloat16, device=DEV)
    args = lambda feats, rows_out: (x.to(DEV).data_ptr(), 128, rows.data_ptr(), 128, None, 0, wp.data_ptr(), nw.to(DEV).data_ptr(),
                                    1e-6, pk.data_ptr(), out.data_ptr(), nw2.data_ptr(), 1e-6, hp.data_ptr(), head.data_ptr(),
                                    feats, rows_out, 16, 128, 512, None)
    bad_shape = 10003  # BNB_ERR_BAD_SHAPE
    assert lib.bnb_ffn_fused_proj_next_fwd(*args(96, 128)) == bad_shape  # not a multiple of 64
    assert lib.bnb_ffn_fused_proj_next_fwd(*args(256, 16)) == bad_shape  # the head needs whole work-groups of rows
    assert lib.bnb_ffn_fused_proj_next_fwd(*args(256, 128)) == 0


def test_column_block_operands_are_read_in_place():
    # [linear1 | linear2] outputs side by side: the conv reads the left block, the tail's gate the right one
    B, n, NM, D = 6, 8, 12, 128
    g = torch.Generator().manual_seed(4)
    both = torch.randn(B, NM, 2 * D, generator=g).bfloat16().to(DEV)
    b1, gate = both[..., :D], both[..., D:]
    buf = torch.randn(B * n, 3, D, generator=g).to(DEV)
    w = (0.5 * torch.randn(D, 1, 4, generator=g)).to(DEV)
    bias = (0.1 * torch.randn(D, generator=g)).to(DEV)
    v_a, buf_a = ops.conv_step(b1[:, :n], buf, w, bias, rows_per_env=n)
    v_b, buf_b = ops.conv_step(b1[:, :n].reshape(B * n, D).contiguous(), buf, w, bias)
    assert torch.equal(v_a, v_b) and torch.equal(buf_a, buf_b)
    x, _, nw, p = _ffn_case(3, B * NM)
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    wp = ops.pack_proj_weights((torch.randn(D, D, generator=g) / D ** 0.5).to(DEV))
    y = torch.randn(B, NM, D, generator=g).bfloat16().to(DEV)
    xd = x.to(DEV).view(B, NM, D)
    in_place = ops.ffn_fused(xd, None, nw.to(DEV), pk, proj=(gate, y, wp))
    copied = ops.ffn_fused(xd, None, nw.to(DEV), pk, proj=(gate.contiguous(), y, wp))
    assert torch.equal(in_place, copied)


def test_three_column_blocks_share_one_projection_output():
    # [linear1 | linear2 | recurrence output] in one (B, NM, 3D) tensor: the fused state kernel
    # writes the ship rows of the third block, the tail reads its gate and y operands in place
    B, n, NM, D = 7, 8, 12, 128
    t = {k: v.to(DEV) for k, v in _temporal_inputs(9, B * n).items()}
    g = torch.Generator().manual_seed(5)
    wide = torch.randn(B, NM, 3 * D, generator=g).bfloat16().to(DEV)
    wide[:, :n, :D] = t["b1"].view(B, n, D)
    before = wide.clone()
    pk, gb = ops.pack_gate_weights(t["wa"], t["wx"]), torch.cat([t["ba"], t["bx"]])
    y_ref, h_ref, buf_ref = ops.temporal_step(t["b1"], t["buf"], t["h"], t["cw"], t["cb"], pk, gb, t["lam"], 8.0, rows_per_env=n)
    _, h_new, buf_new = ops.temporal_step(wide[:, :n, :D], t["buf"], t["h"], t["cw"], t["cb"], pk, gb, t["lam"], 8.0,
                                          y_out=wide[:, :n, 2 * D:], rows_per_env=n)
    assert torch.equal(h_new, h_ref) and torch.equal(buf_new, buf_ref)
    assert torch.equal(wide[:, :n, 2 * D:].reshape(B * n, D), y_ref)
    assert torch.equal(wide[..., :2 * D], before[..., :2 * D]) and torch.equal(wide[:, n:], before[:, n:])
    x, _, nw, p = _ffn_case(6, B * NM)
    ffn = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    wp = ops.pack_proj_weights((torch.randn(D, D, generator=g) / D ** 0.5).to(DEV))
    xd = x.to(DEV).view(B, NM, D)
    gate, y = wide[..., D:2 * D], wide[..., 2 * D:]
    in_place = ops.ffn_fused(xd, None, nw.to(DEV), ffn, proj=(gate, y, wp))
    copied = ops.ffn_fused(xd, None, nw.to(DEV), ffn, proj=(gate.contiguous(), y.contiguous(), wp))
    assert torch.equal(in_place, copied)


# ------------------------------------------------------------------ team pooling


def _team_pool_run(p, x, team, alive, H, broadcast=True):
    consts = ops.pack_team_pool_weights(p["tp.seeds"].to(DEV), p["tp.attn.in_proj_weight"].to(DEV),
                                        p["tp.attn.out_proj.weight"].to(DEV), H)
    ships, pool = ops.team_pool(x.to(DEV), team.to(DEV), alive.to(DEV), *consts, p["tp.norm.weight"].to(DEV), None, H,
                                broadcast=broadcast)
    torch.cuda.synchronize()
    return (None if ships is None else ships.cpu()), pool.cpu()


@pytest.mark.parametrize("B,N", [(1, 1), (5, 8), (6, 19), (9, 64), (7, 65), (4, 152), (3, 320), (1030, 8)])
@pytest.mark.parametrize("H", [4, 2])
def test_team_pool_matches_oracle(B, N, H):
    D = 128
    g = torch.Generator().manual_seed(B * 7 + N)
    p = team_pool_params(g, "tp.", D)
    x = torch.randn(B, N, D, generator=g)
    team, alive = team_case(B + N, B, N)
    ships, pool = _team_pool_run(p, x, team, alive, H)
    ref_ships, ref_pool = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    assert max_rel(pool, ref_pool) <= F32_TOL
    assert torch.allclose(pool, ref_pool, rtol=1e-4, atol=2e-5)
    # which teams are empty is reproduced exactly, and every ship carries its team's vector bit for bit
    assert torch.equal(pool == 0, ref_pool == 0)
    idx = team.clamp(0, 1).long().unsqueeze(-1).expand(B, N, D)
    assert torch.equal(ships, pool.gather(1, idx))
    if B * N <= 200:  # loop-only fp64 statement as a second witness
        from oracle import bruteforce
        loops = bruteforce.team_pool_loops(x.numpy(), team.numpy(), alive.numpy(), p["tp.seeds"].numpy(),
                                           p["tp.attn.in_proj_weight"].numpy(), p["tp.attn.out_proj.weight"].numpy(),
                                           p["tp.norm.weight"].numpy(), H, float(torch.finfo(torch.float32).eps))
        assert max_rel(pool, torch.from_numpy(loops).float()) <= F32_TOL


def test_team_pool_large_scores_and_masking_invariances():
    B, N, D, H = 6, 40, 128, 4
    g = torch.Generator().manual_seed(11)
    p = team_pool_params(g, "tp.", D)
    p["tp.seeds"] = 6.0 * torch.randn(2, D, generator=g)  # scores of magnitude ~50: the running maximum matters
    x = 2.0 * torch.randn(B, N, D, generator=g)
    team, alive = team_case(12, B, N)
    _, pool = _team_pool_run(p, x, team, alive, H, broadcast=False)
    _, ref = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    assert max_rel(pool, ref) <= F32_TOL
    # dead ships are nobody's keys: rewriting their rows changes no bit
    pert = x.clone()
    pert[~alive] = pert[~alive] * -3.0 + 5.0
    assert torch.equal(_team_pool_run(p, pert, team, alive, H, broadcast=False)[1], pool)
    # team 0's vector does not depend on team 1's ships
    pert = x.clone()
    pert[team == 1] += 1.0
    again = _team_pool_run(p, pert, team, alive, H, broadcast=False)[1]
    assert torch.equal(again[:, 0], pool[:, 0]) and not torch.equal(again[:, 1], pool[:, 1])
    # an id outside {0, 1} is no key and reads team 1's vector
    odd = team.clone()
    odd[2, 0] = 2
    ships, pool_odd = _team_pool_run(p, x, odd, alive, H)
    assert torch.equal(ships[2, 0], pool_odd[2, 1])
    stay = alive.clone()
    stay[2, 0] = False
    assert torch.equal(_team_pool_run(p, x, team, stay, H, broadcast=False)[1][2], pool_odd[2])


def test_team_pool_reads_ship_rows_inside_the_token_tensor_and_other_id_types():
    B, N, M, D, H = 9, 8, 4, 128, 4
    g = torch.Generator().manual_seed(13)
    p = team_pool_params(g, "tp.", D)
    tokens = torch.randn(B, N + M, D, generator=g).to(DEV)
    team_all = torch.full((B, N + M), 2, dtype=torch.int32)
    alive_all = torch.ones(B, N + M, dtype=torch.bool)
    team_all[:, :N], alive_all[:, :N] = team_case(14, B, N)
    team_all, alive_all = team_all.to(DEV), alive_all.to(DEV)
    consts = ops.pack_team_pool_weights(p["tp.seeds"].to(DEV), p["tp.attn.in_proj_weight"].to(DEV),
                                        p["tp.attn.out_proj.weight"].to(DEV), H)
    nw = p["tp.norm.weight"].to(DEV)
    a = ops.team_pool(tokens[:, :N], team_all[:, :N], alive_all[:, :N], *consts, nw, None, H)
    b = ops.team_pool(tokens[:, :N].contiguous(), team_all[:, :N].long(), alive_all[:, :N].contiguous(), *consts, nw, None, H)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    with pytest.raises(ValueError):
        ops.team_pool(tokens[:, :N], team_all, alive_all[:, :N], *consts, nw, None, H)
    with pytest.raises(ValueError):
        ops.team_pool(tokens[:, :N].bfloat16(), team_all[:, :N], alive_all[:, :N], *consts, nw, None, H)
    empty = ops.team_pool(tokens[:0, :N], team_all[:0, :N], alive_all[:0, :N], *consts, nw, None, H)
    assert empty[0].shape == (0, N, D) and empty[1].shape == (0, 2, D)


# ------------------------------------------------------------------ widened kernels at the headline size


def test_full_size_temporal_step_on_sampled_rows_and_environment_permutation():
    # 64v88: 4096 environments x 152 ships = 622,592 state rows, two carried steps on the packed state;
    # sampled rows go through the fp32 statement, and permuting the environments permutes the result bit for bit
    w = harness.WORKLOADS["c4_64v88_bf16"]
    B, n, D = w.B, w.N, 128
    R = B * n
    g = torch.Generator(device=DEV).manual_seed(17)
    small = {k: v.to(DEV) for k, v in _temporal_inputs(17, 4).items()}  # weights only
    pk, gb = ops.pack_gate_weights(small["wa"], small["wx"]), torch.cat([small["ba"], small["bx"]])
    state = torch.randn(R, 4 * D, device=DEV, generator=g) * 0.5
    nxt = torch.empty_like(state)
    y = torch.empty(R, D, device=DEV, dtype=torch.bfloat16)
    pick = torch.arange(0, R, 7919, device=DEV)
    ref = {"h": state[pick, :D].cpu(), "buf": state[pick, D:].view(-1, 3, D).cpu()}
    cpu_w = {k: small[k].cpu() for k in ("cw", "cb", "wa", "wx", "ba", "bx", "lam")}
    for t in range(2):
        b1 = torch.randn(R, D, device=DEV, generator=g).bfloat16()
        ops.temporal_step(b1, state[:, D:].view(R, 3, D), state[:, :D], small["cw"], small["cb"], pk, gb, small["lam"], 8.0,
                          conv_out=nxt[:, D:].view(R, 3, D), h_out=nxt[:, :D], y_out=y)
        h_true, buf_true = _temporal_truth({**cpu_w, "b1": b1[pick].cpu(), "h": ref["h"], "buf": ref["buf"]})
        assert torch.equal(nxt[pick, D:].view(-1, 3, D).cpu(), buf_true), t
        assert max_rel(nxt[pick, :D].cpu(), h_true) <= BF16_TOL, t
        if t == 0:
            perm = torch.randperm(B, device=DEV, generator=g)
            rows = (perm[:, None] * n + torch.arange(n, device=DEV)[None, :]).reshape(-1)
            st_p, nxt_p, y_p = state[rows].contiguous(), torch.empty_like(state), torch.empty_like(y)
            ops.temporal_step(b1[rows].contiguous(), st_p[:, D:].view(R, 3, D), st_p[:, :D], small["cw"], small["cb"], pk, gb,
                              small["lam"], 8.0, conv_out=nxt_p[:, D:].view(R, 3, D), h_out=nxt_p[:, :D], y_out=y_p)
            assert torch.equal(nxt_p, nxt[rows]) and torch.equal(y_p, y[rows])
            del st_p, nxt_p, y_p
        ref = {"h": h_true, "buf": buf_true}  # carry the oracle's own state: errors must not need a reset to stay bounded
        state, nxt = nxt, state
    assert torch.isfinite(state).all()


def test_full_size_sublayer_tail_and_projection_on_sampled_rows():
    # 64v88: 655,360 token rows through the fused tail and through norm + qkv projection
    w = harness.WORKLOADS["c4_64v88_bf16"]
    R, D = w.B * w.NM, 128
    g = torch.Generator(device=DEV).manual_seed(19)
    _, _, nw, p = _ffn_case(19, 1)
    x = torch.randn(R, D, device=DEV, generator=g)
    delta = torch.randn(R, D, device=DEV, generator=g).bfloat16()
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    out = ops.ffn_fused(x, delta, nw.to(DEV), pk)
    pick = torch.arange(0, R, 6007, device=DEV)
    rounded = {k: v.bfloat16().float() for k, v in p.items()}
    s = x[pick].cpu() + delta[pick].float().cpu()
    want = s + torch_ref.gated_mlp(rounded, "f.", torch_ref.rms_norm(s, nw))
    assert max_rel(out[pick].cpu(), want) <= BF16_TOL
    assert torch.isfinite(out).all()
    # row permutation equivariance, bit for bit (every row is computed on its own)
    perm = torch.randperm(R, device=DEV, generator=g)
    assert torch.equal(ops.ffn_fused(x[perm], delta[perm], nw.to(DEV), pk), out[perm])
    wq = torch.randn(3 * D, D, generator=torch.Generator().manual_seed(20)) / D ** 0.5
    qkv = ops.norm_linear(x, nw.to(DEV), ops.pack_linear_weights(wq.to(DEV)))
    want = torch_ref.rms_norm(x[pick].cpu(), nw) @ wq.bfloat16().float().t()
    assert max_rel(qkv[pick].float().cpu(), want) <= BF16_TOL


@pytest.mark.parametrize("gated,N", [(False, 384), (True, 256)])
def test_full_size_tail_with_the_next_sublayers_head_on_sampled_rows(gated, N):
    # 64v88: 655,360 token rows, ten rounds of resident work-groups: every weight buffer is recycled many times
    w = harness.WORKLOADS["c4_64v88_bf16"]
    R, D = w.B * w.NM, 128
    g = torch.Generator(device=DEV).manual_seed(29 + N)
    cg = torch.Generator().manual_seed(30 + N)
    _, _, nw, p = _ffn_case(29, 1)
    x = torch.randn(R, D, device=DEV, generator=g)
    rows_a = torch.randn(R, D, device=DEV, generator=g).bfloat16()
    rows_y = torch.randn(R, D, device=DEV, generator=g).bfloat16()
    Wp = torch.randn(D, D, generator=cg) / D ** 0.5
    Wh = torch.randn(N, D, generator=cg) / D ** 0.5
    nw2 = 1.0 + 0.2 * torch.randn(D, generator=cg)
    pk = ops.pack_ffn_weights(p["f.gate_proj.weight"].to(DEV), p["f.up_proj.weight"].to(DEV), p["f.down_proj.weight"].to(DEV))
    wp = ops.pack_proj_weights(Wp.to(DEV))
    spec = (nw2.to(DEV), None, ops.pack_head_weights(Wh.to(DEV)), N)
    proj = (rows_a, rows_y, wp) if gated else (rows_a, wp)
    out, head = ops.ffn_fused(x, None, nw.to(DEV), pk, proj=proj, next_head=spec)
    assert torch.equal(out, ops.ffn_fused(x, None, nw.to(DEV), pk, proj=proj))
    assert torch.isfinite(head.float()).all()
    pick = torch.arange(0, R, 5003, device=DEV)
    want = torch.nn.functional.linear(torch_ref.rms_norm(out[pick].cpu(), nw2), Wh.bfloat16().float())
    assert max_rel(head[pick].float().cpu(), want) <= BF16_TOL
    alone = ops.norm_linear(out, nw2.to(DEV), ops.pack_linear_weights(Wh.to(DEV)))
    assert max_rel(head.float(), alone.float()) <= BF16_TOL
    # row permutation equivariance, bit for bit: a row's result does not depend on where or when it is computed
    perm = torch.randperm(R, device=DEV, generator=g)
    proj_p = (rows_a[perm], rows_y[perm], wp) if gated else (rows_a[perm], wp)
    out_p, head_p = ops.ffn_fused(x[perm], None, nw.to(DEV), pk, proj=proj_p, next_head=spec)
    assert torch.equal(out_p, out[perm]) and torch.equal(head_p, head[perm])


def test_full_size_team_pool_on_sampled_environments():
    w = harness.WORKLOADS["c4_64v88_bf16"]
    B, N, D, H = w.B, w.N, 128, 4
    g = torch.Generator().manual_seed(23)
    p = team_pool_params(g, "tp.", D)
    gd = torch.Generator(device=DEV).manual_seed(23)
    x = torch.randn(B, w.NM, D, device=DEV, generator=gd)
    team, alive = team_case(24, B, N, p_alive=0.6)
    consts = ops.pack_team_pool_weights(p["tp.seeds"].to(DEV), p["tp.attn.in_proj_weight"].to(DEV),
                                        p["tp.attn.out_proj.weight"].to(DEV), H)
    ships, pool = ops.team_pool(x[:, :N], team.to(DEV), alive.to(DEV), *consts, p["tp.norm.weight"].to(DEV), None, H)
    pick = torch.arange(0, B, 97)
    _, ref = torch_ref.team_pool(p, "tp.", x[pick, :N].cpu(), team[pick], alive[pick], H)
    assert max_rel(pool[pick].cpu(), ref) <= F32_TOL
    idx = team.clamp(0, 1).long().unsqueeze(-1).expand(B, N, D).to(DEV)
    assert torch.equal(ships, pool.gather(1, idx))


# ------------------------------------------------------------------ Linear weight gradient


def _wgrad_case(seed, R, N, K):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(R, N, generator=g).bfloat16(), torch.randn(R, K, generator=g).bfloat16()


@pytest.fixture(params=["dma", "staged"])
def wgrad_path(request):
    """Both kernels behind bnb_linear_wgrad_fwd: operand rows global -> LDS directly with the transposing LDS
    read (the default), and through registers with the transpose in registers."""
    from boost_and_broadside_amd import _native

    lib = _native.load()
    assert lib.bnb_linear_wgrad_path(_native.WGRAD_PATH_DMA if request.param == "dma" else _native.WGRAD_PATH_STAGED) == 0
    yield request.param
    assert lib.bnb_linear_wgrad_path(_native.WGRAD_PATH_AUTO) == 0


@pytest.mark.parametrize("R", [0, 1, 31, 33, 63, 64, 65, 1000, 20011, 140000])
@pytest.mark.parametrize("N,K", [(128, 128), (384, 128), (128, 512), (256, 256)])
def test_linear_wgrad_matches_float64_product(R, N, K, wgrad_path):
    """dW = dy^T x is fixed by the mathematics: the float64 product of the same bf16 operands is the truth
    (what nn.Linear's backward, reference models/yemong/attention.py:60-74, computes for its weight)."""
    if R == 140000 and (N, K) != (128, 128):
        pytest.skip("the long case runs once")
    dy, x = _wgrad_case(R + N + K, R, N, K)
    got = ops.linear_wgrad(dy.to(DEV), x.to(DEV))
    torch.cuda.synchronize()
    ref = dy.double().t() @ x.double()
    assert got.shape == (N, K) and got.dtype == torch.float32
    if R == 0:
        assert not got.any()
        return
    assert max_rel(got.cpu().double(), ref) <= F32_TOL
    again = ops.linear_wgrad(dy.to(DEV), x.to(DEV))
    assert torch.equal(got, again)  # fixed summation order


def test_linear_wgrad_single_entries_land_where_the_definition_puts_them():
    R, N, K = 777, 256, 128
    dy = torch.zeros(R, N).bfloat16()
    x = torch.zeros(R, K).bfloat16()
    picks = [(0, 0, 0, 1.0), (63, 5, 127, 2.0), (64, 255, 1, -3.0), (776, 131, 64, 0.5), (400, 33, 97, 4.0), (401, 33, 97, 8.0)]
    want = torch.zeros(N, K)
    for r, n, k, v in picks:
        dy[r, n] = v
        x[r, k] = 1.0
        want[n, k] += v
    # every other product of the chosen rows that is not zero belongs to the truth too
    want = dy.float().t() @ x.float()
    assert want[33, 97] == 12.0 and want[255, 1] == -3.0 and want[5, 127] == 2.0
    got = ops.linear_wgrad(dy.to(DEV), x.to(DEV)).cpu()
    assert torch.equal(got, want)


def test_linear_wgrad_reads_strided_rows_and_accumulates():
    R, N, K = 5000, 128, 256
    g = torch.Generator().manual_seed(5)
    wide_dy = torch.randn(R, 3 * N, generator=g).bfloat16().to(DEV)
    wide_x = torch.randn(R, K + 64, generator=g).bfloat16().to(DEV)
    dy, x = wide_dy[:, N:2 * N], wide_x[:, 64:]
    ref = dy.double().t() @ x.double()
    out = torch.full((N, K), 2.0, device=DEV)
    ops.linear_wgrad(dy, x, out=out)
    assert max_rel(out.double(), ref) <= F32_TOL
    ops.linear_wgrad(dy, x, out=out, accumulate=True)
    assert max_rel(out.double(), 2 * ref) <= F32_TOL
    lead = ops.linear_wgrad(dy.view(50, 100, N), x.view(50, 100, K))
    assert torch.equal(lead, ops.linear_wgrad(dy, x))


def test_linear_wgrad_rejects_what_it_does_not_cover():
    dy, x = _wgrad_case(1, 10, 128, 128)
    with pytest.raises(TypeError):
        ops.linear_wgrad(dy.float().to(DEV), x.to(DEV))
    with pytest.raises(ValueError):
        ops.linear_wgrad(dy.to(DEV), x[:9].to(DEV))
    with pytest.raises(ValueError):
        ops.linear_wgrad(dy.to(DEV)[:, :64], x.to(DEV))
    with pytest.raises(ValueError):
        ops.linear_wgrad(dy.to(DEV), x.to(DEV), accumulate=True)
    assert not ops.linear_wgrad_supported(x.to(DEV), torch.zeros(128, 96))


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("x_dtype", [torch.float32, torch.bfloat16])
def test_linear_train_gradients_match_autograd_of_the_same_bf16_linear(with_bias, x_dtype):
    R, N, K = 9000, 256, 128
    g = torch.Generator().manual_seed(11)
    x0 = torch.randn(30, 300, K, generator=g).to(x_dtype)
    w0 = torch.randn(N, K, generator=g) / K ** 0.5
    b0 = torch.randn(N, generator=g) if with_bias else None
    up = torch.randn(30, 300, N, generator=g)

    x = x0.to(DEV).requires_grad_()
    w = w0.to(DEV).requires_grad_()
    b = b0.to(DEV).requires_grad_() if with_bias else None
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = ops.linear_train(x, w, b)
    assert y.dtype == torch.bfloat16
    (y.float() * up.to(DEV)).sum().backward()

    # truth: the same bf16-rounded operands, float64 arithmetic
    xd = x0.bfloat16().double().requires_grad_()
    wd = w0.bfloat16().double().requires_grad_()
    bd = b0.bfloat16().double().requires_grad_() if with_bias else None
    yd = torch.nn.functional.linear(xd, wd, bd)
    assert max_rel(y.detach().float().cpu().double(), yd.detach()) <= BF16_TOL
    dyb = up.bfloat16().double()  # the gradient reaching the layer is rounded to its bf16 output
    (yd * dyb).sum().backward()
    assert x.grad.dtype == x_dtype and w.grad.dtype == torch.float32
    assert max_rel(w.grad.cpu().double(), wd.grad) <= F32_TOL
    assert max_rel(x.grad.float().cpu().double(), xd.grad) <= BF16_TOL
    if with_bias:
        assert max_rel(b.grad.cpu().double(), bd.grad) <= F32_TOL


@pytest.mark.parametrize("R,N", [(1, 64), (7, 256), (300, 384), (9001, 256), (70000, 128), (513, 2048), (0, 256)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_column_sums_match_the_float64_sums_and_repeat_exactly(R, N, dtype):
    g = torch.Generator().manual_seed(R + N)
    x = (torch.randn(R, N, generator=g) + 0.25).to(dtype)
    xd = x.to(DEV)
    got = ops.column_sums(xd)
    torch.cuda.synchronize()
    assert got.dtype == torch.float32 and got.shape == (N,)
    want = x.double().sum(dim=0)
    scale = max(float(x.double().abs().sum(dim=0).max()), 1.0)  # float32 sums of R terms: error against the terms' size
    assert float((got.cpu().double() - want).abs().max()) / scale <= F32_TOL
    assert torch.equal(got, ops.column_sums(xd))
    # rows further apart than their width (a column slice of a wider matrix)
    if R:
        wide = torch.zeros(R, N + 64, dtype=dtype, device=DEV)
        wide[:, :N] = xd
        assert torch.equal(ops.column_sums(wide[:, :N]), got)


def test_column_sums_find_a_single_entry_in_its_column_and_refuse_other_shapes():
    x = torch.zeros(5000, 256, dtype=torch.bfloat16, device=DEV)
    x[4321, 77] = 3.0
    x[0, 255] = -2.0
    got = ops.column_sums(x).cpu()
    want = torch.zeros(256)
    want[77], want[255] = 3.0, -2.0
    assert torch.equal(got, want)
    for bad in (torch.zeros(10, 100, device=DEV), torch.zeros(10, 4096, device=DEV), torch.zeros(10, 128, device=DEV).half(),
                torch.zeros(10, 128, 2, device=DEV)):
        assert not ops.column_sums_supported(bad)
        with pytest.raises(ValueError):
            ops.column_sums(bad)
    from boost_and_broadside_amd import _native

    lib = _native.load()
    out = torch.zeros(256, device=DEV)
    part = torch.zeros(4, 256, device=DEV)
    assert lib.bnb_column_sums(None, _native.BF16, 256, part.data_ptr(), 4, out.data_ptr(), 0, 10, 256, None) == 10001
    assert lib.bnb_column_sums(x.data_ptr(), _native.BF16, 256, part.data_ptr(), 4, out.data_ptr(), 0, 10, 100, None) != 0
    assert lib.bnb_column_sums(x.data_ptr(), _native.BF16, 100, part.data_ptr(), 4, out.data_ptr(), 0, 10, 256, None) == 10003


# ------------------------------------------------------------------ RMSNorm backward


def _norm_truth(x, dy, w, eps, grad_sum=None):
    """Autograd through the float64 definition (attention.py:60,73 use nn.RMSNorm(d_model), eps = finfo(float32).eps)."""
    xd = x.double().requires_grad_()
    wd = w.double().requires_grad_()
    y = xd * torch.rsqrt(xd.square().mean(dim=-1, keepdim=True) + eps) * wd
    (y * dy.double()).sum().backward()
    dx = xd.grad if grad_sum is None else xd.grad + grad_sum.double()
    return dx, wd.grad


@pytest.mark.parametrize("D", [64, 128, 256, 512])
@pytest.mark.parametrize("R", [0, 1, 31, 257, 5000, 70001])
@pytest.mark.parametrize("dy_dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_bwd_matches_autograd_of_the_definition(D, R, dy_dtype):
    if R == 70001 and D != 128:
        pytest.skip("the long case runs at the trunk's width")
    g = torch.Generator().manual_seed(R * 7 + D)
    x = torch.randn(R, D, generator=g) * (0.2 + 3.0 * torch.rand(R, 1, generator=g))
    dy = torch.randn(R, D, generator=g).to(dy_dtype)
    w = 1.0 + 0.3 * torch.randn(D, generator=g)
    eps = float(torch.finfo(torch.float32).eps)
    dx, dw = ops.rmsnorm_bwd(x.to(DEV), dy.to(DEV), w.to(DEV))
    torch.cuda.synchronize()
    assert dx.shape == (R, D) and dw.shape == (D,) and dx.dtype == dw.dtype == torch.float32
    if R == 0:
        assert not dw.any()
        return
    ref_dx, ref_dw = _norm_truth(x, dy, w, eps)
    assert max_rel(dx.cpu().double(), ref_dx) <= F32_TOL
    assert max_rel(dw.cpu().double(), ref_dw) <= F32_TOL
    dx2, dw2 = ops.rmsnorm_bwd(x.to(DEV), dy.to(DEV), w.to(DEV))
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)


def test_rmsnorm_bwd_adds_the_bypass_gradient_and_reads_strided_rows():
    R, D = 3001, 128
    g = torch.Generator().manual_seed(3)
    wide = torch.randn(R, 3 * D, generator=g).to(DEV)
    x = wide[:, D:2 * D]
    dy = torch.randn(R, 2 * D, generator=g).bfloat16().to(DEV)[:, :D]
    gs = torch.randn(R, D, generator=g).to(DEV)
    w = (1.0 + 0.3 * torch.randn(D, generator=g)).to(DEV)
    dx, dw, dx_lp = ops.rmsnorm_bwd(x, dy, w, eps=1e-5, grad_sum=gs, also_bf16=True)
    assert torch.equal(dx_lp, dx.bfloat16())
    ref_dx, ref_dw = _norm_truth(x.cpu(), dy.cpu(), w.cpu(), 1e-5, gs.cpu())
    assert max_rel(dx.cpu().double(), ref_dx) <= F32_TOL and max_rel(dw.cpu().double(), ref_dw) <= F32_TOL
    lead_dx, lead_dw = ops.rmsnorm_bwd(x.reshape(3001, 1, D), dy.reshape(3001, 1, D), w, eps=1e-5, grad_sum=gs.reshape(3001, 1, D))
    assert torch.equal(lead_dx.reshape(R, D), dx) and torch.equal(lead_dw, dw)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("with_delta", [False, True])
def test_rmsnorm_train_gradients_match_autograd_of_torch_rms_norm(out_dtype, with_delta):
    R, D = 4000, 128
    g = torch.Generator().manual_seed(17)
    x0 = torch.randn(8, R // 8, D, generator=g)
    d0 = torch.randn(8, R // 8, D, generator=g).bfloat16() if with_delta else None
    w0 = 1.0 + 0.2 * torch.randn(D, generator=g)
    up_n = torch.randn(8, R // 8, D, generator=g).to(out_dtype)
    up_s = torch.randn(8, R // 8, D, generator=g)

    x = x0.to(DEV).requires_grad_()
    w = w0.to(DEV).requires_grad_()
    d = d0.to(DEV).requires_grad_() if with_delta else None
    with torch.autocast("cuda", dtype=torch.bfloat16):
        s, n = ops.rmsnorm_train(x, w, delta=d, out_dtype=out_dtype)
    if not with_delta:
        assert torch.equal(s, x)  # x handed through for the residual connection
    loss = (n.float() * up_n.to(DEV).float()).sum() + (s * up_s.to(DEV)).sum()
    assert n.dtype == out_dtype
    loss.backward()

    xr = x0.double().requires_grad_()
    wr = w0.double().requires_grad_()
    dr = d0.double().requires_grad_() if with_delta else None
    sr = xr + dr if with_delta else xr
    nr = torch.nn.functional.rms_norm(sr, (D,), wr, float(torch.finfo(torch.float32).eps))
    lr = (nr * up_n.double()).sum() + (sr * up_s.double()).sum()
    lr.backward()
    tol = F32_TOL if out_dtype == torch.float32 else BF16_TOL
    assert max_rel(n.detach().float().cpu().double(), nr.detach()) <= tol
    assert max_rel(x.grad.cpu().double(), xr.grad) <= F32_TOL
    assert max_rel(w.grad.cpu().double(), wr.grad) <= F32_TOL
    if with_delta:
        assert d.grad.dtype == torch.bfloat16
        assert max_rel(d.grad.float().cpu().double(), dr.grad) <= BF16_TOL


# ------------------------------------------------------------------ sequence conv backward


def _conv_truth_grads(b1, buf, w, bias, done, up_v, up_tail):
    """Autograd through the pinned oracle statement of the conv, float64."""
    leaves = [t.double().requires_grad_() for t in (b1, buf, w, bias)]
    v, tail = torch_ref.conv_sequence(leaves[0], leaves[1], leaves[2], leaves[3], done)
    loss = (v * up_v.double()).sum()
    if up_tail is not None:
        loss = loss + (tail * up_tail.double()).sum()
    loss.backward()
    return [t.grad for t in leaves]


@pytest.mark.parametrize("R,T,D", [(5, 1, 128), (7, 2, 128), (6, 3, 64), (33, 13, 128), (12, 128, 128), (9, 35, 256),
                                   (3, 16, 512), (2100, 29, 128)])
@pytest.mark.parametrize("p_done", [0.0, 0.35])
@pytest.mark.parametrize("b_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("time_major", [False, True])
def test_conv_seq_bwd_matches_autograd_of_the_oracle(R, T, D, p_done, b_dtype, time_major):
    g = torch.Generator().manual_seed(R * 11 + T + D)
    b1 = torch.randn(R, T, D, generator=g).to(b_dtype)
    buf = torch.randn(R, 3, D, generator=g)
    w = 0.5 * torch.randn(D, 1, 4, generator=g)
    bias = 0.1 * torch.randn(D, generator=g)
    done = (torch.rand(R, T, generator=g) < p_done) if p_done > 0 else None
    up_v = torch.randn(R, T, D, generator=g)
    up_tail = torch.randn(R, 3, D, generator=g) if (R + T) % 2 else None
    want = _conv_truth_grads(b1.float(), buf, w, bias, done, up_v, up_tail)

    def lay(t):
        return t.transpose(0, 1).contiguous() if time_major else t

    db1, dbuf, dw, dbias = ops.conv_seq_bwd(lay(b1).to(DEV), buf.to(DEV), w.to(DEV), None if done is None else done.to(DEV),
                                            lay(up_v).to(DEV), None if up_tail is None else up_tail.to(DEV),
                                            time_major=time_major)
    torch.cuda.synchronize()
    assert db1.dtype == b_dtype and dbuf.dtype == dw.dtype == dbias.dtype == torch.float32
    got_b1 = db1.float().cpu()
    got_b1 = got_b1.transpose(0, 1) if time_major else got_b1
    assert max_rel(got_b1.double(), want[0]) <= (F32_TOL if b_dtype == torch.float32 else BF16_TOL)
    assert max_rel(dbuf.cpu().double(), want[1]) <= F32_TOL
    assert max_rel(dw.cpu().double(), want[2].reshape(D, 4)) <= F32_TOL
    assert max_rel(dbias.cpu().double(), want[3]) <= F32_TOL
    again = ops.conv_seq_bwd(lay(b1).to(DEV), buf.to(DEV), w.to(DEV), None if done is None else done.to(DEV),
                             lay(up_v).to(DEV), None if up_tail is None else up_tail.to(DEV), time_major=time_major)
    assert all(torch.equal(a, b) for a, b in zip((db1, dbuf, dw, dbias), again))


def test_conv_seq_train_is_differentiable_and_equals_the_forward_kernel():
    R, T, D = 40, 24, 128
    g = torch.Generator().manual_seed(21)
    b1 = torch.randn(T, R, D, generator=g).bfloat16().to(DEV).requires_grad_()
    buf = torch.randn(R, 3, D, generator=g).to(DEV).requires_grad_()
    w = (0.5 * torch.randn(D, 1, 4, generator=g)).to(DEV).requires_grad_()
    bias = (0.1 * torch.randn(D, generator=g)).to(DEV).requires_grad_()
    done = (torch.rand(R, T, generator=g) < 0.2).to(DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        v, tail = ops.conv_seq_train(b1, buf, w, bias, done, time_major=True)
    with torch.no_grad():
        v0, tail0 = ops.conv_seq(b1.detach(), buf.detach(), w.detach(), bias.detach(), done, time_major=True)
    assert torch.equal(v, v0) and torch.equal(tail, tail0)
    up_v = torch.randn(T, R, D, generator=g).to(DEV)
    (v * up_v).sum().backward()  # the handed-on inputs carry no gradient here
    want = _conv_truth_grads(b1.detach().float().cpu().transpose(0, 1), buf.detach().cpu(), w.detach().cpu(),
                             bias.detach().cpu(), done.cpu(), up_v.cpu().transpose(0, 1), None)
    assert b1.grad.dtype == torch.bfloat16 and w.grad.shape == w.shape
    assert max_rel(b1.grad.float().cpu().transpose(0, 1).double(), want[0]) <= BF16_TOL
    assert max_rel(buf.grad.cpu().double(), want[1]) <= F32_TOL
    assert max_rel(w.grad.cpu().double(), want[2]) <= F32_TOL
    assert max_rel(bias.grad.cpu().double(), want[3]) <= F32_TOL


@pytest.mark.parametrize("R,T,time_major", [(40, 24, True), (9, 35, False), (2100, 29, True)])
def test_conv_seq_bwd_adds_the_gradient_of_the_bfloat16_copy_in_the_same_pass(R, T, time_major):
    D = 128
    g = torch.Generator().manual_seed(R + T)
    shape = (T, R, D) if time_major else (R, T, D)
    b1 = torch.randn(shape, generator=g).bfloat16().to(DEV)
    buf = torch.randn(R, 3, D, generator=g).to(DEV)
    w = (0.5 * torch.randn(D, 1, 4, generator=g)).to(DEV)
    done = (torch.rand(R, T, generator=g) < 0.2).to(DEV)
    dv = torch.randn(shape, generator=g).to(DEV)
    dv_lp = torch.randn(shape, generator=g).bfloat16().to(DEV)
    got = ops.conv_seq_bwd(b1, buf, w, done, dv, None, time_major=time_major, dv_bf16=dv_lp)
    want = ops.conv_seq_bwd(b1, buf, w, done, dv + dv_lp.float(), None, time_major=time_major)
    assert all(torch.equal(a, b) for a, b in zip(got, want))  # the same float32 addition, inside the kernel
    with pytest.raises(ValueError):
        ops.conv_seq_bwd(b1, buf, w, done, dv, None, time_major=time_major, dv_bf16=dv_lp.float())


def test_conv_seq_train_hands_out_a_bfloat16_copy_whose_gradient_reaches_the_input():
    R, T, D = 40, 24, 128
    g = torch.Generator().manual_seed(22)
    b1 = torch.randn(T, R, D, generator=g).bfloat16().to(DEV).requires_grad_()
    buf = torch.randn(R, 3, D, generator=g).to(DEV).requires_grad_()
    w = (0.5 * torch.randn(D, 1, 4, generator=g)).to(DEV).requires_grad_()
    bias = (0.1 * torch.randn(D, generator=g)).to(DEV).requires_grad_()
    done = (torch.rand(R, T, generator=g) < 0.2).to(DEV)
    up_v = torch.randn(T, R, D, generator=g).to(DEV)
    up_lp = torch.randn(T, R, D, generator=g).bfloat16().to(DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        v, tail, v_lp = ops.conv_seq_train(b1, buf, w, bias, done, time_major=True, also_bf16=True)
    assert v_lp.dtype == torch.bfloat16 and torch.equal(v_lp, v.detach().bfloat16())
    ((v * up_v).sum() + (v_lp.float() * up_lp.float()).sum()).backward()
    got = [t.grad.clone() for t in (b1, buf, w, bias)]
    for t in (b1, buf, w, bias):
        t.grad = None
    # the same loss with the copy made by autograd's own cast
    with torch.autocast("cuda", dtype=torch.bfloat16):
        v2, _ = ops.conv_seq_train(b1, buf, w, bias, done, time_major=True)
    ((v2 * up_v).sum() + (v2.bfloat16().float() * up_lp.float()).sum()).backward()
    for a, t in zip(got, (b1, buf, w, bias)):
        assert torch.equal(a, t.grad)
    # only the copy used: the float32 output's gradient is absent, not a tensor of zeros
    for t in (b1, buf, w, bias):
        t.grad = None
    with torch.autocast("cuda", dtype=torch.bfloat16):
        _, _, v_lp3 = ops.conv_seq_train(b1, buf, w, bias, done, time_major=True, also_bf16=True)
    (v_lp3.float() * up_lp.float()).sum().backward()
    want = ops.conv_seq_bwd(b1.detach(), buf.detach(), w.detach(), done, up_lp.float(), None, time_major=True)
    assert torch.equal(b1.grad, want[0]) and torch.equal(buf.grad, want[1])


# ------------------------------------------------------------------ gelu(a) * b backward


@pytest.mark.parametrize("R,H", [(1, 8), (37, 128), (1000, 512), (4099, 136)])
@pytest.mark.parametrize("a_dtype,b_dtype,o_dtype", [(torch.float32, torch.float32, torch.float32),
                                                     (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                                     (torch.bfloat16, torch.float32, torch.bfloat16)])
def test_gelu_mul_train_gradients_match_autograd_of_erf_gelu(R, H, a_dtype, b_dtype, o_dtype):
    g = torch.Generator().manual_seed(R + H)
    a0 = (2.0 * torch.randn(R, H, generator=g)).to(a_dtype)
    b0 = torch.randn(R, H, generator=g).to(b_dtype)
    up = torch.randn(R, H, generator=g).to(o_dtype)
    a = a0.to(DEV).requires_grad_()
    b = b0.to(DEV).requires_grad_()
    out = ops.gelu_mul_train(a, b, out_dtype=o_dtype)
    with torch.no_grad():
        assert torch.equal(out, ops.gelu_mul(a.detach(), b.detach(), out_dtype=o_dtype))
    out.backward(up.to(DEV))
    ad = a0.double().requires_grad_()
    bd = b0.double().requires_grad_()
    (torch.nn.functional.gelu(ad) * bd * up.double()).sum().backward()
    assert a.grad.dtype == a_dtype and b.grad.dtype == b_dtype
    assert max_rel(a.grad.float().cpu().double(), ad.grad) <= (F32_TOL if a_dtype == torch.float32 else BF16_TOL)
    assert max_rel(b.grad.float().cpu().double(), bd.grad) <= (F32_TOL if a_dtype == b_dtype == torch.float32 else BF16_TOL)


def test_gelu_mul_bwd_reads_column_blocks_of_one_projection_output():
    R, H = 300, 256
    g = torch.Generator().manual_seed(9)
    gu = torch.randn(R, 2 * H, generator=g).bfloat16().to(DEV)
    dout = torch.randn(R, H, generator=g).bfloat16().to(DEV)
    da, db = ops.gelu_mul_bwd(gu[:, :H], gu[:, H:], dout)
    da2, db2 = ops.gelu_mul_bwd(gu[:, :H].contiguous(), gu[:, H:].contiguous(), dout)
    assert torch.equal(da, da2) and torch.equal(db, db2)


# ------------------------------------------------------------------ masked attention backward


def _sdpa_truth_grad(qkv, alive, H, up):
    """Autograd through the oracle's written-out statement of attention.py:136-147, float64 (pinned against the
    library call in tests/test_oracle_pins.py; they differ only in the gradient of environments without a live key)."""
    x = qkv.double().requires_grad_()
    out = torch_ref.sdpa_masked_softmax(x, alive, H)
    (out * up.double()).sum().backward()
    return out.detach(), x.grad


@pytest.mark.parametrize("B,NM,H", [(3, 12, 4), (70, 12, 4), (5, 27, 4), (4, 1, 4), (6, 32, 4), (9, 7, 2), (3, 20, 8), (1000, 12, 4)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p_alive", [1.0, 0.7, 0.0])
def test_sdpa_masked_bwd_matches_autograd_of_the_oracle(B, NM, H, dtype, p_alive):
    D = 32 * H
    qkv = _qkv(B * 31 + NM, B, NM, D, dtype, scale=1.5)
    alive = None if p_alive == 1.0 else _alive(NM + B, B, NM, p_alive)
    if alive is not None and p_alive > 0 and B > 2:
        alive[1] = False  # one environment without a live key among live ones
    g = torch.Generator().manual_seed(B + NM)
    up = torch.randn(B, NM, D, generator=g).to(dtype)
    ref_out, ref_grad = _sdpa_truth_grad(qkv, alive, H, up)
    out = ops.sdpa_masked(qkv.to(DEV), None if alive is None else alive.to(DEV), H)
    dqkv = ops.sdpa_masked_bwd(qkv.to(DEV), None if alive is None else alive.to(DEV), H, out, up.to(DEV))
    torch.cuda.synchronize()
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    assert dqkv.dtype == dtype and dqkv.shape == qkv.shape
    assert max_rel(out.float().cpu().double(), ref_out) <= tol
    # the bf16 forward result enters the backward (rowsum(dO * O)), so compare per third
    for name, cols in (("dQ", slice(0, D)), ("dK", slice(D, 2 * D)), ("dV", slice(2 * D, 3 * D))):
        if NM == 1 and name != "dV":  # a single key: the softmax is constant, dQ = dK = 0 up to float64 noise
            assert dqkv[..., cols].float().abs().max() <= 1e-6 * ref_grad.abs().max(), name
            continue
        assert max_rel(dqkv[..., cols].float().cpu().double(), ref_grad[..., cols]) <= tol, name
    if alive is not None and p_alive > 0:
        dead = ~alive & alive.any(dim=1, keepdim=True)  # dead keys of environments that have live ones
        assert not dqkv.cpu()[..., D:][dead].any()  # dead keys receive exactly nothing
    again = ops.sdpa_masked_bwd(qkv.to(DEV), None if alive is None else alive.to(DEV), H, out, up.to(DEV))
    assert torch.equal(dqkv, again)


def test_sdpa_train_is_differentiable_and_reads_strided_rows():
    B, NM, H, D = 33, 12, 4, 128
    g = torch.Generator().manual_seed(4)
    wide = (torch.randn(B, NM, 3 * D + 64, generator=g)).bfloat16().to(DEV).requires_grad_()
    alive = (torch.rand(B, NM, generator=g) < 0.8).to(DEV)
    up = torch.randn(B, NM, D, generator=g).to(DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = ops.sdpa_train(wide[..., 64:], alive, H)
    (out.float() * up).sum().backward()
    ref_out, ref_grad = _sdpa_truth_grad(wide.detach()[..., 64:].float().cpu(), alive.cpu(), H, up.bfloat16().cpu())
    assert max_rel(out.detach().float().cpu().double(), ref_out) <= BF16_TOL
    assert not wide.grad[..., :64].any()
    assert max_rel(wide.grad[..., 64:].float().cpu().double(), ref_grad) <= BF16_TOL
    assert not ops.sdpa_train_supported(torch.zeros(2, 40, 384, device=DEV), 4)
    assert not ops.sdpa_train_supported(torch.zeros(2, 12, 192, device=DEV), 4)


def test_gelu_mul_packed_train_equals_the_two_operand_form():
    R, H = 700, 512
    g = torch.Generator().manual_seed(13)
    gu0 = torch.randn(R, 2 * H, generator=g).bfloat16().to(DEV)
    up = torch.randn(R, H, generator=g).bfloat16().to(DEV)
    gu = gu0.clone().requires_grad_()
    out = ops.gelu_mul_packed_train(gu.view(7, 100, 2 * H), out_dtype=torch.bfloat16)
    out.backward(up.view(7, 100, H))
    a = gu0[:, :H].clone().requires_grad_()
    b = gu0[:, H:].clone().requires_grad_()
    ref = ops.gelu_mul_train(a, b, out_dtype=torch.bfloat16)
    ref.backward(up)
    assert torch.equal(out.reshape(R, H), ref)
    assert torch.equal(gu.grad[:, :H], a.grad) and torch.equal(gu.grad[:, H:], b.grad)


@pytest.mark.parametrize("B,NM,H", [(3, 12, 4), (5, 27, 4), (4, 1, 4), (6, 32, 4), (5, 33, 4), (4, 64, 4), (3, 84, 4), (2, 152, 4),
                                    (2, 160, 4), (3, 100, 2), (300, 40, 4),
                                    # two heads per tile (up to 16 tokens, even head count) and its neighbours
                                    (70, 12, 4), (9, 7, 2), (5, 16, 4), (3, 15, 8), (4, 17, 4), (6, 12, 3), (1001, 12, 4)])
@pytest.mark.parametrize("p_alive", [1.0, 0.7, 0.0])
def test_sdpa_masked_bwd_on_the_matrix_cores_matches_autograd_of_the_oracle(B, NM, H, p_alive):
    D = 32 * H
    qkv = _qkv(B * 17 + NM, B, NM, D, torch.bfloat16, scale=1.5)
    alive = None if p_alive == 1.0 else _alive(NM + B, B, NM, p_alive)
    if alive is not None and p_alive > 0 and B > 2:
        alive[1] = False
    g = torch.Generator().manual_seed(B + NM)
    up = torch.randn(B, NM, D, generator=g).bfloat16()
    ref_out, ref_grad = _sdpa_truth_grad(qkv, alive, H, up)
    mask = None if alive is None else alive.to(DEV)
    out = ops.sdpa_masked(qkv.to(DEV), mask, H)
    dqkv = ops.sdpa_masked_bwd(qkv.to(DEV), mask, H, out, up.to(DEV), path="mfma")
    torch.cuda.synchronize()
    for name, cols in (("dQ", slice(0, D)), ("dK", slice(D, 2 * D)), ("dV", slice(2 * D, 3 * D))):
        if NM == 1 and name != "dV":
            assert dqkv[..., cols].float().abs().max() <= 1e-6 * ref_grad.abs().max(), name
            continue
        assert max_rel(dqkv[..., cols].float().cpu().double(), ref_grad[..., cols]) <= BF16_TOL, name
    if alive is not None and p_alive > 0:
        dead = ~alive & alive.any(dim=1, keepdim=True)
        assert not dqkv.cpu()[..., D:][dead].any()
    assert torch.equal(dqkv, ops.sdpa_masked_bwd(qkv.to(DEV), mask, H, out, up.to(DEV), path="mfma"))
    if NM <= 32:  # the two kernels against each other
        other = ops.sdpa_masked_bwd(qkv.to(DEV), mask, H, out, up.to(DEV), path="valu")
        assert max_rel(dqkv.float().cpu(), other.float().cpu()) <= BF16_TOL


# ------------------------------------------------------------------ bullet read backward


@pytest.mark.parametrize("B,NQ,NK,H", [(3, 12, 80, 4), (5, 23, 160, 4), (4, 1, 1, 4), (2, 84, 33, 4), (3, 160, 10, 4), (6, 12, 31, 2),
                                       (200, 12, 80, 4)])
@pytest.mark.parametrize("p_live", [1.0, 0.25, 0.0])
def test_sdpa_cross_bwd_matches_autograd_of_the_oracle(B, NQ, NK, H, p_live):
    D = 32 * H
    g = torch.Generator().manual_seed(B * 13 + NQ + NK)
    qkv = (1.2 * torch.randn(B, NQ, 3 * D, generator=g)).bfloat16()
    kv = (1.2 * torch.randn(B, NK, 2 * D, generator=g)).bfloat16()
    mask = None if p_live == 1.0 else torch.rand(B, NK, generator=g) < p_live
    if mask is not None and p_live > 0 and B > 2:
        mask[1] = False  # an environment without an active bullet among active ones
        mask[0, 0] = True
    up = torch.randn(B, NQ, D, generator=g).bfloat16()
    xq = qkv.double().requires_grad_()
    xkv = kv.double().requires_grad_()
    ref = torch_ref.bullet_read(xq, xkv, mask, H)
    (ref * up.double()).sum().backward()
    dmask = None if mask is None else mask.to(DEV)
    out = ops.sdpa_cross(qkv.to(DEV), kv.to(DEV), dmask, H)
    dq, dkv = ops.sdpa_cross_bwd(qkv.to(DEV), kv.to(DEV), dmask, H, out, up.to(DEV))
    torch.cuda.synchronize()
    assert max_rel(out.float().cpu().double(), ref.detach()) <= BF16_TOL or not ref.detach().any()
    for name, got, want in (("dQ", dq, xq.grad[..., :D]), ("dK", dkv[..., :D], xkv.grad[..., :D]), ("dV", dkv[..., D:], xkv.grad[..., D:])):
        if want.abs().max() < 1e-12:  # gated-off environments only, or a single key
            assert got.float().abs().max() <= 1e-6 * max(1.0, float(xkv.grad.abs().max())), name
            continue
        assert max_rel(got.float().cpu().double(), want) <= BF16_TOL, name
    assert not xq.grad[..., D:].any()  # the read never touches the entity keys and values
    if mask is not None:
        off = ~mask.any(dim=1)
        assert not dq.cpu()[off].any() and not dkv.cpu()[off].any()  # gated off: exactly nothing
        dead = ~mask & mask.any(dim=1, keepdim=True)
        assert not dkv.cpu()[dead].any()
    again = ops.sdpa_cross_bwd(qkv.to(DEV), kv.to(DEV), dmask, H, out, up.to(DEV))
    assert torch.equal(dq, again[0]) and torch.equal(dkv, again[1])


def test_sdpa_cross_train_is_differentiable():
    B, NQ, NK, H, D = 9, 12, 80, 4, 128
    g = torch.Generator().manual_seed(2)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16().to(DEV).requires_grad_()
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16().to(DEV).requires_grad_()
    mask = (torch.rand(B, NK, generator=g) < 0.3).to(DEV)
    up = torch.randn(B, NQ, D, generator=g).to(DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = ops.sdpa_cross_train(qkv, kv, mask, H)
        (out.float() * up).sum().backward()  # backward called inside autocast on purpose
    xq = qkv.detach().cpu().double().requires_grad_()
    xkv = kv.detach().cpu().double().requires_grad_()
    (torch_ref.bullet_read(xq, xkv, mask.cpu(), H) * up.bfloat16().cpu().double()).sum().backward()
    assert max_rel(qkv.grad.float().cpu().double(), xq.grad) <= BF16_TOL
    assert max_rel(kv.grad.float().cpu().double(), xkv.grad) <= BF16_TOL
    assert ops.sdpa_cross_train_supported(qkv, torch.zeros(B, 200, 2 * D, device=DEV, dtype=torch.bfloat16), H)
    assert not ops.sdpa_cross_train_supported(qkv, torch.zeros(B, 2049, 2 * D, device=DEV, dtype=torch.bfloat16), H)
    assert not ops.sdpa_cross_train_supported(qkv.float(), torch.zeros(B, 80, 2 * D, device=DEV), H)


@pytest.mark.parametrize("B,NQ,NK,p_live", [
    (3, 12, 200, 0.5), (4, 23, 480, 0.3), (2, 160, 1520, 0.25), (3, 84, 800, 1.0), (5, 152, 2048, 0.05), (3, 33, 161, 1.0),
    (4, 12, 80, 0.25), (6, 64, 1520, 0.02), (2, 97, 2048, 1.0),
])
def test_sdpa_cross_streaming_backward_matches_autograd_of_the_oracle(B, NQ, NK, p_live):
    """The bullet read's backward over long slot axes (10 slots per ship: 1520 at 64v88), in both forms: the
    (B, NK, 2D) buffer read in place through the list of its live slots, and rows compacted beforehand."""
    H, D = 4, 128
    g = torch.Generator().manual_seed(B * 17 + NQ + NK)
    qkv = (1.2 * torch.randn(B, NQ, 3 * D, generator=g)).bfloat16()
    kv = (1.2 * torch.randn(B, NK, 2 * D, generator=g)).bfloat16()
    mask = torch.rand(B, NK, generator=g) < p_live
    if B > 2:
        mask[1] = False  # an environment without an active bullet among active ones
    mask[0, 0] = True
    mask[0, NK - 1] = True
    up = torch.randn(B, NQ, D, generator=g).bfloat16()
    xq = qkv.double().requires_grad_()
    xkv = kv.double().requires_grad_()
    ref = torch_ref.bullet_read(xq, xkv, mask, H)
    (ref * up.double()).sum().backward()
    dmask = mask.to(DEV)
    dqkv, dkv_in, dup = qkv.to(DEV), kv.to(DEV), up.to(DEV)
    out = ops.sdpa_cross(dqkv, dkv_in, dmask, H)
    rows = ops.CompactRows(dmask)
    dq, dkv = ops.sdpa_cross_stream_bwd(dqkv, dkv_in, rows, H, out, dup, indexed=True)
    torch.cuda.synchronize()
    for name, got, want in (("dQ", dq, xq.grad[..., :D]), ("dK", dkv[..., :D], xkv.grad[..., :D]), ("dV", dkv[..., D:], xkv.grad[..., D:])):
        assert max_rel(got.float().cpu().double(), want) <= BF16_TOL, name
    off = ~mask.any(dim=1)
    assert not dq.cpu()[off].any() and not dkv.cpu()[off].any()  # gated off: exactly nothing
    assert not dkv.cpu()[~mask].any()  # dead slots receive exact zeros
    # rows compacted beforehand: the same keys in the same order, so the same numbers
    total = rows.total_host()
    kv_rows = dkv_in.reshape(B * NK, 2 * D)[dmask.reshape(-1)].contiguous()
    dq_r, dkv_r = ops.sdpa_cross_stream_bwd(dqkv, kv_rows, rows, H, out, dup, indexed=False)
    assert torch.equal(dq_r, dq)
    assert torch.equal(dkv_r, dkv.reshape(B * NK, 2 * D)[dmask.reshape(-1)])
    if rows.max_count_host() > 160:  # what the rows form of the update path dispatches to above one tile of keys
        dq_d, dkv_d = ops.sdpa_cross_rows_bwd(dqkv, kv_rows, rows, H, out, dup, total)
        assert torch.equal(dq_d, dq) and torch.equal(dkv_d, dkv_r)
    elif NK <= 160:  # one tile: the single-tile kernel answers the same question
        dq_s, dkv_s = ops.sdpa_cross_bwd(dqkv, dkv_in, dmask, H, out, dup)
        assert max_rel(dq_s.float().cpu(), dq.float().cpu()) <= BF16_TOL
        assert max_rel(dkv_s.float().cpu(), dkv.float().cpu()) <= BF16_TOL
    again = ops.sdpa_cross_stream_bwd(dqkv, dkv_in, rows, H, out, dup, indexed=True)
    assert torch.equal(dq, again[0]) and torch.equal(dkv, again[1])


def test_sdpa_cross_train_over_a_long_slot_axis_is_differentiable():
    B, NQ, NK, H, D = 5, 84, 800, 4, 128
    g = torch.Generator().manual_seed(3)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16().to(DEV).requires_grad_()
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16().to(DEV).requires_grad_()
    mask = (torch.rand(B, NK, generator=g) < 0.3).to(DEV)
    up = torch.randn(B, NQ, D, generator=g).to(DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = ops.sdpa_cross_train(qkv, kv, mask, H)
        (out.float() * up).sum().backward()
    xq = qkv.detach().cpu().double().requires_grad_()
    xkv = kv.detach().cpu().double().requires_grad_()
    (torch_ref.bullet_read(xq, xkv, mask.cpu(), H) * up.bfloat16().cpu().double()).sum().backward()
    assert max_rel(qkv.grad.float().cpu().double(), xq.grad) <= BF16_TOL
    assert max_rel(kv.grad.float().cpu().double(), xkv.grad) <= BF16_TOL
    # rows form with more than one tile of keys per environment
    rows = ops.CompactRows(mask)
    kv_rows = kv.detach().reshape(B * NK, 2 * D)[mask.reshape(-1)].clone().requires_grad_()
    q2 = qkv.detach().clone().requires_grad_()
    (ops.sdpa_cross_rows_train(q2, kv_rows, rows, H).float() * up).sum().backward()
    assert max_rel(q2.grad.float().cpu().double(), xq.grad) <= BF16_TOL
    assert max_rel(kv_rows.grad.float().cpu().double(), xkv.grad.reshape(B * NK, 2 * D)[mask.cpu().reshape(-1)]) <= BF16_TOL


@pytest.mark.parametrize("B,NQ,NK,p_live", [(4, 12, 80, 0.25), (3, 23, 160, 0.1), (5, 12, 40, 1.0), (6, 84, 33, 0.5), (300, 12, 80, 0.25)])
def test_sdpa_cross_rows_bwd_equals_the_masked_form(B, NQ, NK, p_live):
    H, D = 4, 128
    g = torch.Generator().manual_seed(B + NQ + NK)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16().to(DEV)
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16().to(DEV)
    mask = (torch.rand(B, NK, generator=g) < p_live).to(DEV)
    if B > 2:
        mask[1] = False
    up = torch.randn(B, NQ, D, generator=g).bfloat16().to(DEV)
    rows = ops.CompactRows(mask)
    total = rows.total_host()
    assert total == int(mask.sum())
    kv_rows = kv.reshape(B * NK, 2 * D)[mask.reshape(-1)].contiguous()
    out = ops.sdpa_cross(qkv, kv, mask, H)
    out_rows = ops.sdpa_cross_rows(qkv, kv_rows, rows, H, total=total)
    assert max_rel(out_rows.float().cpu(), out.float().cpu()) <= BF16_TOL  # two forward kernels (tile vs streamed keys)
    dq, dkv = ops.sdpa_cross_bwd(qkv, kv, mask, H, out, up)
    dq_r, dkv_r = ops.sdpa_cross_rows_bwd(qkv, kv_rows, rows, H, out, up, total)
    # same keys, in the same order per environment: the live rows' gradients and dq agree to rounding of the
    # sums' order (compaction moves keys to other accumulator rows), well inside the bf16 bar
    assert max_rel(dq_r.float().cpu(), dq.float().cpu()) <= BF16_TOL
    assert max_rel(dkv_r.float().cpu(), dkv.reshape(B * NK, 2 * D)[mask.reshape(-1)].float().cpu()) <= BF16_TOL
    off = ~mask.any(dim=1)
    assert not dq_r[off].any()


def test_sdpa_cross_rows_train_matches_autograd_of_the_oracle():
    B, NQ, NK, H, D = 7, 12, 80, 4, 128
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16().to(DEV).requires_grad_()
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16()
    mask = torch.rand(B, NK, generator=g) < 0.3
    up = torch.randn(B, NQ, D, generator=g)
    rows = ops.CompactRows(mask.to(DEV))
    kv_rows = kv.reshape(B * NK, 2 * D)[mask.reshape(-1)].to(DEV).requires_grad_()
    out = ops.sdpa_cross_rows_train(qkv, kv_rows, rows, H)
    (out.float() * up.to(DEV)).sum().backward()
    xq = qkv.detach().cpu().double().requires_grad_()
    xkv = kv.double().requires_grad_()
    (torch_ref.bullet_read(xq, xkv, mask, H) * up.bfloat16().double()).sum().backward()
    assert max_rel(qkv.grad.float().cpu().double(), xq.grad) <= BF16_TOL
    assert max_rel(kv_rows.grad.float().cpu().double(), xkv.grad.reshape(B * NK, 2 * D)[mask.reshape(-1)]) <= BF16_TOL


@pytest.mark.parametrize("B,NQ,NK,p_live", [(5, 12, 400, 0.6), (4, 84, 800, 0.3), (3, 156, 1520, 0.25), (3, 130, 700, 0.5)])
def test_streamed_read_hands_its_log_sum_exp_to_the_backward(B, NQ, NK, p_live):
    """More than 160 listed keys per environment: the forward writes every query's log2-sum-exp, the backward takes it
    instead of passing over the keys twice.  Pinned three ways: the values against float64 scores of the same
    bfloat16 operands, the gradients against the backward that recomputes them, and, through autograd, against the
    oracle's."""
    H, D = 4, 128
    g = torch.Generator().manual_seed(B * 1000 + NQ + NK)
    qkv = torch.randn(B, NQ, 3 * D, generator=g).bfloat16()
    kv = torch.randn(B, NK, 2 * D, generator=g).bfloat16()
    kv[:, :, :D] *= 2.0
    mask = torch.rand(B, NK, generator=g) < p_live
    mask[1] = False
    up = torch.randn(B, NQ, D, generator=g).bfloat16()
    rows = ops.CompactRows(mask.to(DEV))
    total = rows.total_host()
    assert rows.max_count_host() > 160
    kv_rows = kv.reshape(B * NK, 2 * D)[mask.reshape(-1)].contiguous().to(DEV)
    q_d = qkv.to(DEV)
    lse = torch.full((B, H, NQ), float("nan"), device=DEV)
    out = ops.sdpa_cross_rows(q_d, kv_rows, rows, H, total=total, lse=lse)
    assert torch.equal(out, ops.sdpa_cross_rows(q_d, kv_rows, rows, H, total=total))  # the same forward either way
    # log2 sum_k exp2(q.k log2(e) / sqrt(32)) over the live keys
    qh = qkv[..., :D].double().reshape(B, NQ, H, 32).transpose(1, 2)
    kh = kv[..., :D].double().reshape(B, NK, H, 32).transpose(1, 2)
    scores = (qh @ kh.transpose(-1, -2)) / 32 ** 0.5
    scores = scores.masked_fill(~mask[:, None, None, :], float("-inf"))
    want = torch.logsumexp(scores, dim=-1) / math.log(2.0)
    live = mask.any(dim=1)
    assert (lse[live.to(DEV)].double().cpu() - want[live]).abs().max() <= 1e-4

    dq0, dkv0 = ops.sdpa_cross_rows_bwd(q_d, kv_rows, rows, H, out, up.to(DEV), total)
    dq1, dkv1 = ops.sdpa_cross_rows_bwd(q_d, kv_rows, rows, H, out, up.to(DEV), total, lse=lse)
    assert max_rel(dq1.float().cpu(), dq0.float().cpu()) <= 2e-3 and max_rel(dkv1.float().cpu(), dkv0.float().cpu()) <= 2e-3
    assert not dq1[~live.to(DEV)].any()

    qg = q_d.clone().requires_grad_()
    kvg = kv_rows.clone().requires_grad_()
    (ops.sdpa_cross_rows_train(qg, kvg, rows, H).float() * up.to(DEV).float()).sum().backward()
    xq = qkv.double().requires_grad_()
    xkv = kv.double().requires_grad_()
    (torch_ref.bullet_read(xq, xkv, mask, H) * up.double()).sum().backward()
    assert max_rel(qg.grad.float().cpu().double(), xq.grad) <= BF16_TOL
    assert max_rel(kvg.grad.float().cpu().double(), xkv.grad.reshape(B * NK, 2 * D)[mask.reshape(-1)]) <= BF16_TOL
    with pytest.raises(ValueError):
        ops.sdpa_cross_rows(q_d, kv_rows, rows, H, total=total, lse=lse[:, :, :-1])


# ------------------------------------------------------------------ element offsets past 2^31


def _slices_of(n, width=2048):
    return (slice(0, width), slice(n // 2, n // 2 + width), slice(n - width, n))


def test_update_path_kernels_index_rows_whose_element_offsets_pass_2_31():
    """Rollout-sized inputs (millions of token rows): the last rows must be as right as the first.

    Every check compares a window at the start, the middle and the end of the rows against torch
    on the same values; the weight gradient, a sum over all rows, against float64 in chunks.
    """
    import torch.nn.functional as F

    gen = torch.Generator(device=DEV).manual_seed(11)
    R = 2_300_000  # 1024 columns: offsets up to 2.36e9 elements
    gu = torch.randn(R, 1024, device=DEV, generator=gen).bfloat16().requires_grad_()
    out = ops.gelu_mul_packed_train(gu)
    dout = torch.randn(R, 512, device=DEV, generator=gen).bfloat16()
    out.backward(dout)
    for sl in _slices_of(R):
        g = gu.detach()[sl].float().requires_grad_()
        ref = F.gelu(g[:, :512]).bfloat16().float() * g[:, 512:]
        ref.backward(dout[sl].float())
        assert max_rel(out[sl].detach().float(), ref.detach()) <= BF16_TOL
        assert max_rel(gu.grad[sl].float(), g.grad) <= BF16_TOL

    x = torch.randn(R, 128, device=DEV, generator=gen).bfloat16()
    dy = gu.detach()[:, 512:]  # strided rows of the same buffer
    got = ops.linear_wgrad(dy, x)
    ref = torch.zeros(512, 128, device=DEV, dtype=torch.float64)
    for s in range(0, R, 1 << 18):
        ref += dy[s:s + (1 << 18)].double().t() @ x[s:s + (1 << 18)].double()
    assert max_rel(got, ref) <= F32_TOL
    del gu, out, dout, dy, x
    torch.cuda.empty_cache()

    R2 = 17_000_000  # 128 columns: offsets up to 2.18e9 elements
    xs = torch.randn(R2, 128, device=DEV, generator=gen).requires_grad_()
    w = (1 + 0.1 * torch.randn(128, device=DEV, generator=gen)).requires_grad_()
    _, n = ops.rmsnorm_train(xs, w)
    dn = torch.randn(R2, 128, device=DEV, generator=gen).to(n.dtype)
    n.backward(dn)
    eps = torch.finfo(torch.float32).eps
    for sl in _slices_of(R2):
        xr = xs.detach()[sl].clone().requires_grad_()
        nr = F.rms_norm(xr, (128,), w.detach(), eps)
        nr.backward(dn[sl].float())
        assert max_rel(n[sl].detach().float(), nr.detach()) <= (BF16_TOL if n.dtype == torch.bfloat16 else F32_TOL)
        assert max_rel(xs.grad[sl], xr.grad) <= F32_TOL
    dw = torch.zeros(128, device=DEV, dtype=torch.float64)
    for s in range(0, R2, 1 << 20):
        xr = xs.detach()[s:s + (1 << 20)].double()
        dw += (xr * torch.rsqrt(xr.square().mean(-1, keepdim=True) + eps) * dn[s:s + (1 << 20)].double()).sum(0)
    assert max_rel(w.grad, dw) <= F32_TOL
    del xs, n, dn
    torch.cuda.empty_cache()

    B, NM, H = 480_000, 12, 4  # 5.76 million token rows x 384 columns = 2.2e9 elements
    qkv = torch.randn(B, NM, 384, device=DEV, generator=gen).bfloat16().requires_grad_()
    alive = torch.rand(B, NM, device=DEV, generator=gen) < 0.8
    o = ops.sdpa_train(qkv, alive, H)
    do = torch.randn(B, NM, 128, device=DEV, generator=gen).bfloat16()
    o.backward(do)
    for sl in _slices_of(B, 256):
        q = qkv.detach()[sl].float().cpu().requires_grad_()
        r = torch_ref.sdpa_masked_softmax(q, alive[sl].cpu(), H)
        r.backward(do[sl].float().cpu())
        assert max_rel(o[sl].detach().float().cpu(), r.detach()) <= BF16_TOL
        assert max_rel(qkv.grad[sl].float().cpu(), q.grad) <= BF16_TOL


def test_rollout_and_inference_kernels_index_rows_whose_element_offsets_pass_2_31():
    """The same check for the sequence kernels, the bullet read (mask and list form), the sublayer tail
    and norm + projection: a window at the start and one at the end of the rows against the oracle."""
    import torch.nn.functional as F

    gen = torch.Generator(device=DEV).manual_seed(12)

    def randn(*shape):
        return torch.randn(*shape, device=DEV, generator=gen)

    R, T, D = 140_000, 128, 128  # 2.29e9 elements per (R, T, D) tensor
    b1 = randn(R, T, D).bfloat16().requires_grad_()
    cb = randn(R, 3, D).requires_grad_()
    w, bias = randn(D, 4).requires_grad_(), randn(D).requires_grad_()
    done = torch.rand(R, T, device=DEV, generator=gen) < 0.05
    v, _ = ops.conv_seq_train(b1, cb, w, bias, done)
    dv = randn(R, T, D)
    v.backward(dv)
    for sl in (slice(0, 48), slice(R - 48, R)):
        b = b1.detach()[sl].float().cpu().requires_grad_()
        c = cb.detach()[sl].cpu().requires_grad_()
        r, _ = torch_ref.conv_sequence(b, c, w.detach().cpu(), bias.detach().cpu(), done[sl].cpu())
        r.backward(dv[sl].cpu())
        assert max_rel(v[sl].detach().cpu(), r.detach()) <= F32_TOL
        assert max_rel(b1.grad[sl].float().cpu(), b.grad) <= BF16_TOL
        assert max_rel(cb.grad[sl].cpu(), c.grad) <= F32_TOL
    del b1, v, dv
    torch.cuda.empty_cache()

    x, gates = randn(R, T, D), randn(R, T, 2 * D)
    lam, h0 = torch.linspace(0, 4, D, device=DEV), randn(R, D)
    y, h_last = ops.rglru_scan(x, gates, lam, 8.0, h0, done)
    for sl in (slice(0, 24), slice(R - 24, R)):
        r, rh = torch_ref.rglru_sequence(x[sl].cpu(), gates[sl].cpu(), lam.cpu(), 8.0, h0[sl].cpu(), done[sl].cpu())
        assert max_rel(y[sl].cpu(), r) <= 2e-5
        assert max_rel(h_last[sl].cpu(), rh) <= 2e-5
    del x, gates, y, h_last
    torch.cuda.empty_cache()

    B, NQ, NK, H = 6000, 12, 1520, 4  # keys and values: 2.33e9 elements
    qkv, kv = randn(B, NQ, 384).bfloat16(), randn(B, NK, 256).bfloat16()
    mask = torch.rand(B, NK, device=DEV, generator=gen) < 0.1
    o = ops.sdpa_cross(qkv, kv, mask, H)
    rows = ops.CompactRows(mask)
    kv_rows = torch.zeros(B * NK, 256, device=DEV, dtype=torch.bfloat16)
    kv_rows[: rows.total_host()] = kv.reshape(B * NK, 256)[mask.reshape(-1)]
    o2 = ops.sdpa_cross_rows(qkv, kv_rows, rows, H)
    for sl in (slice(0, 16), slice(B - 16, B)):
        r = torch_ref.bullet_read(qkv[sl].float().cpu(), kv[sl].float().cpu(), mask[sl].cpu(), H)
        assert max_rel(o[sl].float().cpu(), r) <= BF16_TOL
        assert max_rel(o2[sl].float().cpu(), r) <= BF16_TOL
    del qkv, kv, o, o2, kv_rows
    torch.cuda.empty_cache()

    R2 = 17_000_000  # 2.18e9 elements per (R2, 128) tensor
    xs, delta, nw = randn(R2, 128), randn(R2, 128).bfloat16(), 1 + 0.1 * randn(128)
    gw, uw, dw = randn(512, 128) / 11, randn(512, 128) / 11, randn(128, 512) / 22
    wq = randn(384, 128) / 11
    out = ops.ffn_fused(xs, delta, nw, ops.pack_ffn_weights(gw, uw, dw))
    q = ops.norm_linear(xs, nw, ops.pack_linear_weights(wq))
    eps = torch.finfo(torch.float32).eps
    for sl in (slice(0, 2048), slice(R2 - 2048, R2)):
        s = xs[sl] + delta[sl].float()
        n = F.rms_norm(s, (128,), nw, eps).bfloat16()
        hidden = F.gelu(F.linear(n, gw.bfloat16())) * F.linear(n, uw.bfloat16())
        assert max_rel(out[sl], s + F.linear(hidden, dw.bfloat16()).float()) <= BF16_TOL
        r = F.linear(F.rms_norm(xs[sl], (128,), nw, eps).bfloat16(), wq.bfloat16())
        assert max_rel(q[sl].float(), r.float()) <= BF16_TOL


# ------------------------------------------------------------------ float32 Linear layers with their neighbours folded in


def _gelu64(t):
    return 0.5 * t * (1.0 + torch.erf(t / 2 ** 0.5))


@pytest.mark.parametrize("R", [1, 31, 32, 33, 1000, 12288])
@pytest.mark.parametrize("mode", ["plain", "bias_resid", "norm", "norm_gate", "mulgelu_resid", "gate", "k512_resid"])
def test_linear_f32_matches_the_float64_statement(R, mode):
    # every float32 Linear of the trunk as evaluation runs it (no autocast), with the passes around it folded in
    g = torch.Generator().manual_seed(R * 13 + len(mode))
    K = 512 if mode == "k512_resid" else 128
    N = {"plain": 384, "bias_resid": 256, "norm": 384, "norm_gate": 512, "mulgelu_resid": 128, "gate": 512, "k512_resid": 128}[mode]
    x = torch.randn(R, K, generator=g) * (0.3 + 2.0 * torch.rand(R, 1, generator=g))
    w = torch.randn(N, K, generator=g) / K ** 0.5
    xd, wd = x.double(), w.double()
    kw, ref = {}, None
    if mode == "plain":
        ref = xd @ wd.t()
        packed = ops.pack_linear_f32(w.to(DEV))
    elif mode == "bias_resid":
        b, res = torch.randn(N, generator=g), torch.randn(R, N, generator=g)
        ref = xd @ wd.t() + b.double() + res.double()
        packed = ops.pack_linear_f32(w.to(DEV))
        kw = dict(bias=b.to(DEV), resid=res.to(DEV))
    elif mode in ("norm", "norm_gate"):
        nw = 1.0 + 0.2 * torch.randn(K, generator=g)
        eps = float(torch.finfo(torch.float32).eps)
        n = xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + eps) * nw.double()
        kw = dict(norm_weight=nw.to(DEV))
        if mode == "norm":
            ref = n @ wd.t()
            packed = ops.pack_linear_f32(w.to(DEV))
        else:
            up = torch.randn(N, K, generator=g) / K ** 0.5
            ref = _gelu64(n @ wd.t()) * (n @ up.double().t())
            packed = ops.pack_linear_f32(w.to(DEV), up.to(DEV))
            kw["gate"] = True
    elif mode == "gate":
        up = torch.randn(N, K, generator=g) / K ** 0.5
        ref = _gelu64(xd @ wd.t()) * (xd @ up.double().t())
        packed = ops.pack_linear_f32(w.to(DEV), up.to(DEV))
        kw = dict(gate=True)
    elif mode == "mulgelu_resid":
        y, res = torch.randn(R, K, generator=g), torch.randn(R, N, generator=g)
        ref = (_gelu64(xd) * y.double()) @ wd.t() + res.double()
        packed = ops.pack_linear_f32(w.to(DEV))
        kw = dict(gelu_times=y.to(DEV), resid=res.to(DEV))
    else:
        res = torch.randn(R, N, generator=g)
        ref = xd @ wd.t() + res.double()
        packed = ops.pack_linear_f32(w.to(DEV))
        kw = dict(resid=res.to(DEV))
    got = ops.linear_f32(x.to(DEV), packed, **kw)
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert max_rel(got.cpu().double(), ref) <= F32_TOL
    # repeated calls give identical bits; a leading shape is kept
    again = ops.linear_f32(x.to(DEV).reshape(R, 1, K), packed, **{k: (v.reshape(R, 1, -1) if k in ("resid", "gelu_times") else v) for k, v in kw.items()})
    assert torch.equal(again.reshape(got.shape), got)


def test_linear_f32_reads_column_blocks_in_place_and_writes_into_the_residual():
    g = torch.Generator().manual_seed(5)
    R, K = 777, 128
    wide = torch.randn(R, 3 * K, generator=g).to(DEV)
    w = (torch.randn(K, K, generator=g) / K ** 0.5).to(DEV)
    packed = ops.pack_linear_f32(w)
    x = wide[:, K:2 * K]  # a column block: no copy is made
    res = torch.randn(R, K, generator=g).to(DEV)
    want = (x.double() @ w.double().t() + res.double()).cpu()
    got = ops.linear_f32(x, packed, resid=res, out=res)  # in place on the residual stream
    assert got.data_ptr() == res.data_ptr() and max_rel(got.cpu().double(), want) <= F32_TOL
    with pytest.raises(RuntimeError, match="outside what the kernels cover"):
        ops.linear_f32(torch.zeros(4, 256, device=DEV), ops.pack_linear_f32(torch.zeros(32, 256, device=DEV)),
                       norm_weight=torch.ones(256, device=DEV))  # the norm prologue is for width 128
    with pytest.raises(ValueError):
        ops.pack_linear_f32(torch.zeros(48, 128))


# ------------------------------------------------------------------ norm + projection of the update (forward kernel writes n)


@pytest.mark.parametrize("R,N", [(1, 128), (130, 384), (8192, 384), (20000, 128)])
def test_norm_linear_train_forward_and_gradients_match_autograd_of_the_oracle(R, N):
    g = torch.Generator().manual_seed(R + N)
    D = 128
    x = 2.0 * torch.randn(R, D, generator=g)
    nw = 1.0 + 0.1 * torch.randn(D, generator=g)
    W = torch.randn(N, D, generator=g) / D ** 0.5
    dy = torch.randn(R, N, generator=g).bfloat16()
    ds = torch.randn(R, D, generator=g)
    dn_other = torch.randn(R, D, generator=g).bfloat16()
    xd, nwd, Wd = x.to(DEV).requires_grad_(), nw.to(DEV).requires_grad_(), W.to(DEV).requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        x_out, y, n = ops.norm_linear_train(xd, nwd, Wd)
    assert y.dtype == torch.bfloat16 and n.dtype == torch.bfloat16 and x_out.data_ptr() == xd.data_ptr()
    # forward: the inference kernel bit for bit; n the bf16 rows of the oracle's norm
    with torch.no_grad():
        assert torch.equal(y, ops.norm_linear(xd.detach(), nwd.detach(), ops.pack_linear_weights(Wd.detach())))
    n_ref = torch_ref.rms_norm(x, nw)
    assert max_rel(n.float().cpu(), n_ref) <= BF16_TOL
    # backward against float64 autograd through the oracle on the bf16-rounded weight
    xr, nwr = x.double().requires_grad_(), nw.double().requires_grad_()
    Wr = W.bfloat16().double().requires_grad_()
    nr = torch_ref.rms_norm(xr, nwr)
    yr = nr @ Wr.t()
    (yr * dy.double()).sum().add((xr * ds.double()).sum()).add((nr * dn_other.double()).sum()).backward()
    torch.autograd.backward([x_out, y, n], [ds.to(DEV), dy.to(DEV), dn_other.to(DEV)])
    assert max_rel(xd.grad.cpu(), xr.grad.float()) <= BF16_TOL
    assert max_rel(Wd.grad.cpu(), Wr.grad.float()) <= BF16_TOL
    assert max_rel(nwd.grad.cpu(), nwr.grad.float()) <= BF16_TOL


def test_norm_linear_train_refuses_what_the_kernel_does_not_cover():
    from boost_and_broadside_amd import _native

    lib = _native.load()
    x = torch.zeros(16, 128, device=DEV)
    w = torch.ones(128, device=DEV)
    pk = ops.pack_linear_weights(torch.zeros(128, 128, device=DEV))
    y = torch.empty(16, 128, dtype=torch.bfloat16, device=DEV)
    n = torch.empty(16, 128, dtype=torch.bfloat16, device=DEV)
    args = lambda D, N, n_ptr: (x.data_ptr(), 128, w.data_ptr(), 1e-6, pk.data_ptr(), y.data_ptr(), n_ptr, 16, D, N, None)
    assert lib.bnb_norm_linear_train_fwd(*args(128, 128, n.data_ptr())) == 0
    assert lib.bnb_norm_linear_train_fwd(*args(64, 128, n.data_ptr())) == _native.ERR_UNSUPPORTED
    assert lib.bnb_norm_linear_train_fwd(*args(128, 96, n.data_ptr())) == _native.ERR_UNSUPPORTED
    assert lib.bnb_norm_linear_train_fwd(*args(128, 128, None)) == 10001  # BNB_ERR_NULL_POINTER
    assert not ops.norm_linear_train_supported(x, torch.zeros(64, 128, device=DEV))  # the weight-gradient kernel wants 128s


def test_issue_probe_reports_a_plausible_matrix_product_time_and_rejects_bad_arguments():
    # the yardstick of the issue-bound kernels: a 32x32x16 bf16 matrix product occupies a SIMD's matrix core for 32
    # cycles, i.e. 13-20 ns at the clocks this part runs at; vector work added to it can only make a slot longer
    from boost_and_broadside_amd import _native

    alone = ops.issue_probe(0, iters=4000)
    with_valu = ops.issue_probe(16, iters=4000)
    valu_alone = ops.issue_probe(16, mfma=False, iters=4000)
    assert 8.0 < alone < 40.0, alone
    assert with_valu >= alone and with_valu >= valu_alone
    assert with_valu <= 1.2 * (alone + valu_alone)
    lib = _native.load()
    sink = torch.zeros(256, device=DEV)
    assert lib.bnb_issue_probe(3, 1, 0, 2, 10, sink.data_ptr(), None) == _native.ERR_UNSUPPORTED
    assert lib.bnb_issue_probe(8, 1, 0, 3, 10, sink.data_ptr(), None) == 10003  # BNB_ERR_BAD_SHAPE
    assert lib.bnb_issue_probe(8, 1, 0, 2, 10, None, None) == 10001  # BNB_ERR_NULL_POINTER
    assert not sink.any()


def test_compact_rows_hints_are_checked_on_request(monkeypatch):
    # a caller that counted the live bullets when the rollout was stored hands the counts over; wrong ones are
    # undefined behaviour in the kernels, so there is a way to find them
    gen = torch.Generator().manual_seed(5)
    mask = (torch.rand(9, 40, generator=gen) < 0.3).to(DEV)
    total, most = int(mask.sum()), int(mask.sum(dim=1).max())
    ops.CompactRows(mask, total=total, max_count=most).check_hints()
    ops.CompactRows(mask, total=total, max_count=most + 7).check_hints()  # an upper bound on the row count is fine
    ops.CompactRows(mask).check_hints()  # nothing to check without hints
    for bad_total, bad_most in ((total - 1, most), (total + 1, most), (total, most - 1)):
        with pytest.raises(ValueError, match="do not fit the mask"):
            ops.CompactRows(mask, total=bad_total, max_count=bad_most).check_hints()
    monkeypatch.setenv("BNB_CHECK_HINTS", "1")
    with pytest.raises(ValueError, match="do not fit the mask"):
        ops.CompactRows(mask, total=total - 1, max_count=most)
    ops.CompactRows(mask, total=total, max_count=most)
