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


# ---------------------------------------------------------------- bullet read, sequence path, sublayer tail

WIDE = np.load(os.path.join(ROOT, "tests", "golden", "widened_vectors.npz"))


def _from_bits(name):
    """bfloat16 bit patterns stored as uint16 -> float32 tensor."""
    return torch.from_numpy((WIDE[name].astype(np.uint32) << 16).view(np.float32).copy())


@pytest.mark.parametrize("tag", ["read_small", "read_long"])
def test_oracle_reproduces_bullet_read_vectors(tag):
    q, kv, active = _from_bits(f"{tag}_q_bf16"), _from_bits(f"{tag}_kv_bf16"), torch.from_numpy(WIDE[f"{tag}_active"])
    H, want = int(WIDE[f"{tag}_heads"]), WIDE[f"{tag}_out"]
    qkv = torch.cat([q, torch.zeros(*q.shape[:2], 2 * q.shape[-1])], dim=-1)  # only the Q third is read
    got = torch_ref.bullet_read(qkv, kv, active, H).double().numpy()
    assert np.abs(got - want).max() <= 5e-6
    assert np.abs(want[0]).max() == 0  # nothing in flight
    D = q.shape[-1]
    assert np.abs(want[1] - kv[1, -1, D:].double().numpy()).max() <= 1e-12  # one bullet: its V row


def test_oracle_reproduces_sequence_vectors():
    done = torch.from_numpy(WIDE["seq_done"])
    v, _ = torch_ref.conv_sequence(*(torch.from_numpy(WIDE[k]) for k in ("conv_b1", "conv_buf", "conv_w", "conv_bias")), done)
    assert np.abs(v.double().numpy() - WIDE["conv_out"]).max() <= 5e-6
    y, _ = torch_ref.rglru_sequence(torch.from_numpy(WIDE["scan_x"]), torch.from_numpy(WIDE["scan_gates"]),
                                    torch.from_numpy(WIDE["scan_lambda"]), 8.0, torch.from_numpy(WIDE["scan_h0"]), done)
    assert np.abs(y.double().numpy() - WIDE["scan_out"]).max() <= 5e-6


def test_oracle_reproduces_sublayer_tail_vectors():
    p = {"f.gate_proj.weight": _from_bits("ffn_gate_w_bf16"), "f.up_proj.weight": _from_bits("ffn_up_w_bf16"),
         "f.down_proj.weight": _from_bits("ffn_down_w_bf16")}
    s = torch.from_numpy(WIDE["ffn_x"]) + _from_bits("ffn_delta_bf16")
    got = s + torch_ref.gated_mlp(p, "f.", torch_ref.rms_norm(s, torch.from_numpy(WIDE["ffn_norm_w"])))
    assert np.abs(got.double().numpy() - WIDE["ffn_out"]).max() <= 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["read_small", "read_long"])
def test_kernels_reproduce_bullet_read_vectors(tag):
    from boost_and_broadside_amd import ops

    q, kv, active = _from_bits(f"{tag}_q_bf16"), _from_bits(f"{tag}_kv_bf16"), torch.from_numpy(WIDE[f"{tag}_active"])
    qkv = torch.cat([q, torch.zeros(*q.shape[:2], 2 * q.shape[-1])], dim=-1).bfloat16()
    got = ops.sdpa_cross(qkv.cuda(), kv.bfloat16().cuda(), active.cuda(), int(WIDE[f"{tag}_heads"])).float().cpu()
    assert got[0].abs().max() == 0
    assert max_rel(got, torch.from_numpy(WIDE[f"{tag}_out"])) <= 2e-2


@pytest.mark.gpu
def test_kernels_reproduce_sequence_vectors():
    from boost_and_broadside_amd import ops

    done = torch.from_numpy(WIDE["seq_done"]).cuda()
    v, _ = ops.conv_seq(*(torch.from_numpy(WIDE[k]).cuda() for k in ("conv_b1", "conv_buf", "conv_w", "conv_bias")), done)
    assert max_rel(v.cpu(), torch.from_numpy(WIDE["conv_out"])) <= 1e-5
    y, last = ops.rglru_scan(torch.from_numpy(WIDE["scan_x"]).cuda(), torch.from_numpy(WIDE["scan_gates"]).cuda(),
                             torch.from_numpy(WIDE["scan_lambda"]).cuda(), 8.0, torch.from_numpy(WIDE["scan_h0"]).cuda(), done)
    assert max_rel(y.cpu(), torch.from_numpy(WIDE["scan_out"])) <= 1e-5
    assert torch.equal(last, y[:, -1])


@pytest.mark.gpu
def test_kernels_reproduce_sublayer_tail_vectors():
    from boost_and_broadside_amd import ops

    pk = ops.pack_ffn_weights(_from_bits("ffn_gate_w_bf16").cuda(), _from_bits("ffn_up_w_bf16").cuda(),
                              _from_bits("ffn_down_w_bf16").cuda())
    got = ops.ffn_fused(torch.from_numpy(WIDE["ffn_x"]).cuda(), _from_bits("ffn_delta_bf16").bfloat16().cuda(),
                        torch.from_numpy(WIDE["ffn_norm_w"]).cuda(), pk).cpu()
    assert max_rel(got, torch.from_numpy(WIDE["ffn_out"])) <= 2e-2


# ---------------------------------------------------------------- team pooling

TEAM = np.load(os.path.join(ROOT, "tests", "golden", "team_pool_vectors.npz"))


def _team_inputs():
    p = {"tp.seeds": TEAM["seeds"], "tp.attn.in_proj_weight": TEAM["in_proj_weight"],
         "tp.attn.out_proj.weight": TEAM["out_proj_weight"], "tp.norm.weight": TEAM["norm_weight"]}
    p = {k: torch.from_numpy(v) for k, v in p.items()}
    return p, torch.from_numpy(TEAM["x"]), torch.from_numpy(TEAM["team_id"]), torch.from_numpy(TEAM["alive"]), int(TEAM["heads"])


def test_oracle_reproduces_team_pool_vectors():
    p, x, team, alive, H = _team_inputs()
    ships, pool = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    want = TEAM["pool"]
    assert np.abs(pool.double().numpy() - want).max() <= 2e-5
    assert np.abs(want[0, 1]).max() == 0 and np.abs(want[1]).max() == 0  # empty teams
    assert torch.equal(ships[3, 0], pool[3, 1])  # the field id reads team 1's vector


@pytest.mark.gpu
def test_kernels_reproduce_team_pool_vectors():
    from boost_and_broadside_amd import ops

    p, x, team, alive, H = _team_inputs()
    consts = ops.pack_team_pool_weights(p["tp.seeds"].cuda(), p["tp.attn.in_proj_weight"].cuda(),
                                        p["tp.attn.out_proj.weight"].cuda(), H)
    ships, pool = ops.team_pool(x.cuda(), team.cuda(), alive.cuda(), *consts, p["tp.norm.weight"].cuda(), None, H)
    want = torch.from_numpy(TEAM["pool"]).float()
    assert max_rel(pool.cpu(), want) <= 1e-5
    assert torch.equal(pool.cpu() == 0, want == 0)
    assert torch.equal(ships[3, 0], pool[3, 1])


# ---------------------------------------------------------------- gradients of the update path

UPD = np.load(os.path.join(ROOT, "tests", "golden", "update_vectors.npz"))
UPD_ATTN = ("attn_4v4", "attn_8v11", "attn_wide")


@pytest.mark.parametrize("tag", UPD_ATTN)
def test_autograd_of_the_oracle_reproduces_attention_gradient_vectors(tag):
    # the hand-written chain rule (oracle/bruteforce.py) and torch's differentiation of the written-out oracle agree
    qkv = torch.from_numpy(UPD[f"{tag}_qkv"]).double().requires_grad_()
    alive, H = torch.from_numpy(UPD[f"{tag}_alive"]), int(UPD[f"{tag}_heads"])
    (torch_ref.sdpa_masked_softmax(qkv, alive, H) * torch.from_numpy(UPD[f"{tag}_dout"]).double()).sum().backward()
    assert np.abs(qkv.grad.numpy() - UPD[f"{tag}_dqkv"]).max() <= 1e-10


def test_autograd_of_the_oracle_reproduces_conv_and_norm_gradient_vectors():
    lv = [torch.from_numpy(UPD[k]).double().requires_grad_() for k in ("conv_b1", "conv_buf", "conv_w")]
    bias = torch.zeros(lv[0].shape[-1], dtype=torch.float64, requires_grad=True)
    v, tail = torch_ref.conv_sequence(lv[0], lv[1], lv[2], bias, torch.from_numpy(UPD["conv_done"]))
    ((v * torch.from_numpy(UPD["conv_dv"]).double()).sum() + (tail * torch.from_numpy(UPD["conv_dtail"]).double()).sum()).backward()
    for t, key in zip(lv + [bias], ("conv_db1", "conv_dbuf", "conv_dw", "conv_dbias")):
        assert np.abs(t.grad.numpy().reshape(UPD[key].shape) - UPD[key]).max() <= 1e-10, key
    x = torch.from_numpy(UPD["norm_x"]).double().requires_grad_()
    w = torch.from_numpy(UPD["norm_w"]).double().requires_grad_()
    y = torch.nn.functional.rms_norm(x, (x.shape[-1],), w, float(np.finfo(np.float32).eps))
    (y * torch.from_numpy(UPD["norm_dy"]).double()).sum().backward()
    assert np.abs(x.grad.numpy() - UPD["norm_dx"]).max() <= 1e-10 and np.abs(w.grad.numpy() - UPD["norm_dw"]).max() <= 1e-10


@pytest.mark.gpu
@pytest.mark.parametrize("tag", UPD_ATTN)
@pytest.mark.parametrize("dtype,path", [(torch.float32, "valu"), (torch.bfloat16, "valu"), (torch.bfloat16, "mfma")])
def test_kernels_reproduce_attention_gradient_vectors(tag, dtype, path):
    from boost_and_broadside_amd import ops

    qkv = torch.from_numpy(UPD[f"{tag}_qkv"]).to(dtype)  # stored values are bf16-representable: both dtypes see the same numbers
    alive, H = torch.from_numpy(UPD[f"{tag}_alive"]), int(UPD[f"{tag}_heads"])
    if path == "valu" and qkv.shape[1] > 32:
        pytest.skip("the vector kernel covers up to 32 tokens")
    dout = torch.from_numpy(UPD[f"{tag}_dout"]).to(dtype)
    out = ops.sdpa_masked(qkv.cuda(), alive.cuda(), H)
    got = ops.sdpa_masked_bwd(qkv.cuda(), alive.cuda(), H, out, dout.cuda(), path=path).float().cpu()
    want = torch.from_numpy(UPD[f"{tag}_dqkv"])
    D = qkv.shape[-1] // 3
    for third in range(3):
        cols = slice(third * D, (third + 1) * D)
        assert max_rel(got[..., cols].double(), want[..., cols]) <= (1e-5 if dtype == torch.float32 else 2e-2), third


@pytest.mark.gpu
@pytest.mark.parametrize("b_dtype", [torch.float32, torch.bfloat16])
def test_kernels_reproduce_conv_and_norm_gradient_vectors(b_dtype):
    from boost_and_broadside_amd import ops

    b1 = torch.from_numpy(UPD["conv_b1"]).to(b_dtype).cuda()
    got = ops.conv_seq_bwd(b1, torch.from_numpy(UPD["conv_buf"]).cuda(), torch.from_numpy(UPD["conv_w"]).cuda(),
                           torch.from_numpy(UPD["conv_done"]).cuda(), torch.from_numpy(UPD["conv_dv"]).cuda(),
                           torch.from_numpy(UPD["conv_dtail"]).cuda())
    assert max_rel(got[0].float().cpu().double(), torch.from_numpy(UPD["conv_db1"])) <= (1e-5 if b_dtype == torch.float32 else 2e-2)
    for g, key in zip(got[1:], ("conv_dbuf", "conv_dw", "conv_dbias")):
        assert max_rel(g.cpu().double(), torch.from_numpy(UPD[key])) <= 1e-5, key
    dx, dw = ops.rmsnorm_bwd(torch.from_numpy(UPD["norm_x"]).cuda(), torch.from_numpy(UPD["norm_dy"]).to(b_dtype).cuda(),
                             torch.from_numpy(UPD["norm_w"]).cuda())
    assert max_rel(dx.cpu().double(), torch.from_numpy(UPD["norm_dx"])) <= 1e-5
    assert max_rel(dw.cpu().double(), torch.from_numpy(UPD["norm_dw"])) <= 1e-5


UPD_CROSS = ("cross_4v4", "cross_wide", "cross_long")


@pytest.mark.parametrize("tag", UPD_CROSS)
def test_autograd_of_the_oracle_reproduces_bullet_read_gradient_vectors(tag):
    xq = torch.from_numpy(UPD[f"{tag}_qkv"]).double().requires_grad_()
    xkv = torch.from_numpy(UPD[f"{tag}_kv"]).double().requires_grad_()
    act, H = torch.from_numpy(UPD[f"{tag}_active"]), int(UPD[f"{tag}_heads"])
    (torch_ref.bullet_read(xq, xkv, act, H) * torch.from_numpy(UPD[f"{tag}_dout"]).double()).sum().backward()
    D = xkv.shape[-1] // 2
    assert np.abs(xq.grad.numpy()[..., :D] - UPD[f"{tag}_dq"]).max() <= 1e-10 and not xq.grad[..., D:].any()
    assert np.abs(xkv.grad.numpy() - UPD[f"{tag}_dkv"]).max() <= 1e-10


@pytest.mark.gpu
@pytest.mark.parametrize("tag", UPD_CROSS)
@pytest.mark.parametrize("form", ["mask", "ranges"])
def test_kernels_reproduce_bullet_read_gradient_vectors(tag, form):
    from boost_and_broadside_amd import ops

    qkv = torch.from_numpy(UPD[f"{tag}_qkv"]).bfloat16().cuda()
    kv = torch.from_numpy(UPD[f"{tag}_kv"]).bfloat16().cuda()
    act, H = torch.from_numpy(UPD[f"{tag}_active"]).cuda(), int(UPD[f"{tag}_heads"])
    dout = torch.from_numpy(UPD[f"{tag}_dout"]).bfloat16().cuda()
    want_dq, want_dkv = torch.from_numpy(UPD[f"{tag}_dq"]), torch.from_numpy(UPD[f"{tag}_dkv"])
    B, NB, D2 = kv.shape
    if form == "mask":
        out = ops.sdpa_cross(qkv, kv, act, H)
        if NB <= 160:
            dq, dkv = ops.sdpa_cross_bwd(qkv, kv, act, H, out, dout)
        else:  # long slot axes: the streaming pair, reading the buffer in place through the list of live slots
            dq, dkv = ops.sdpa_cross_stream_bwd(qkv, kv, ops.CompactRows(act), H, out, dout, indexed=True)
        dkv = dkv.float().cpu()
    else:
        rows = ops.CompactRows(act)
        total = rows.total_host()
        kv_rows = kv.reshape(B * NB, D2)[act.reshape(-1)].contiguous()
        out = ops.sdpa_cross_rows(qkv, kv_rows, rows, H, total=total)
        dq, dkv_rows = ops.sdpa_cross_rows_bwd(qkv, kv_rows, rows, H, out, dout, total)
        dkv = torch.zeros(B * NB, D2)
        dkv[act.reshape(-1).cpu()] = dkv_rows.float().cpu()
        dkv = dkv.reshape(B, NB, D2)
    scale = float(want_dkv.abs().max())
    # with a single active bullet the weights are constant and dq is zero up to float64 noise: measure against the
    # gradients' common scale rather than dq's own maximum
    assert float((dq.float().cpu().double() - want_dq).abs().max()) <= 2e-2 * max(float(want_dq.abs().max()), 1e-2 * scale)
    assert max_rel(dkv.double(), want_dkv) <= 2e-2
    assert not dq[0].any()  # no active bullet: gated off
