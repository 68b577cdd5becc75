"""Pins the CPU oracle before anything is compared against it.

The reference ships no stored numeric vectors for this path (its tests are
property tests, tests/models/test_encoder.py:106-268, :408-589, :1041-1203), so the
oracle is pinned by (1) the library routine the reference itself calls, (2) fp64
loop-only brute force, (3) hand-computed known answers and (4) the invariants the
reference's tests assert.  Each check is chosen so that a dropped term, a wrong
sign, a transposed operand or a swapped index fails it.
"""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import block_params, temporal_params, trunk_params
from oracle import bruteforce, c_ref, torch_ref


def _qkv(seed, B, NM, D, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, NM, 3 * D, generator=g).to(dtype)


# ---------------------------------------------------------------- masked attention


def test_bias_constants_per_dtype():
    alive = torch.tensor([[True, False]])
    b32 = torch_ref.key_bias(alive, torch.float32)
    b16 = torch_ref.key_bias(alive, torch.bfloat16)
    assert b32.shape == (1, 1, 1, 2) and b32.dtype == torch.float32 and b16.dtype == torch.bfloat16
    assert b32[0, 0, 0, 0] == 0 and b16[0, 0, 0, 0] == 0
    assert float(b32[0, 0, 0, 1]) == pytest.approx(-1.7014117331926443e38, rel=1e-7)
    assert float(b16[0, 0, 0, 1]) == pytest.approx(-1.6947656946257677e38, rel=1e-7)


def test_written_out_attention_pins_values_and_gradients_of_the_library_call():
    """The gradient truth of the attention-backward tests: same values as the library call everywhere,
    same gradients wherever an environment has a live key; without one the library's fused backward
    returns NM times the gradient of the function it evaluated (weights 1 instead of 1/NM)."""
    B, NM, H, D = 6, 9, 4, 128
    qkv = _qkv(5, B, NM, D, torch.float64)
    g = torch.Generator().manual_seed(6)
    alive = torch.rand(B, NM, generator=g) < 0.6
    alive[:, 0] = True
    alive[2] = False
    up = torch.randn(B, NM, D, generator=g, dtype=torch.float64)
    grads = []
    for fn in (torch_ref.sdpa_masked, torch_ref.sdpa_masked_softmax):
        x = qkv.clone().requires_grad_()
        out = fn(x, alive, H)
        (out * up).sum().backward()
        grads.append((out.detach(), x.grad))
    assert torch.allclose(grads[0][0], grads[1][0], rtol=1e-12, atol=1e-13)
    some = alive.any(dim=1)
    assert torch.allclose(grads[0][1][some], grads[1][1][some], rtol=1e-10, atol=1e-12)
    # the all-dead environment, against the closed form with uniform weights 1/NM
    q, k, v = (t.reshape(NM, H, 32).transpose(0, 1) for t in qkv[2].split(D, dim=-1))
    do = up[2].reshape(NM, H, 32).transpose(0, 1)
    P = torch.full((H, NM, NM), 1.0 / NM, dtype=torch.float64)
    dP = do @ v.transpose(-1, -2)
    dS = P * (dP - (P * dP).sum(-1, keepdim=True))
    want = torch.cat([(dS @ k / 32 ** 0.5).transpose(0, 1).reshape(NM, D),
                      (dS.transpose(-1, -2) @ q / 32 ** 0.5).transpose(0, 1).reshape(NM, D),
                      (P.transpose(-1, -2) @ do).transpose(0, 1).reshape(NM, D)], dim=-1)
    assert torch.allclose(grads[1][1][2], want, rtol=1e-10, atol=1e-12)
    # and no-mask gradients agree as well
    x0, x1 = qkv.clone().requires_grad_(), qkv.clone().requires_grad_()
    (torch_ref.sdpa_masked(x0, None, H) * up).sum().backward()
    (torch_ref.sdpa_masked_softmax(x1, None, H) * up).sum().backward()
    assert torch.allclose(x0.grad, x1.grad, rtol=1e-10, atol=1e-12)


def test_hand_computed_two_key_case():
    # one head, dh=2; scores 0 and ln 3 => weights 1/4, 3/4; V rows (4,0),(0,8) => (1,6)
    D = 2
    qkv = torch.zeros(1, 2, 3 * D)
    qkv[0, 0, 0:2] = torch.tensor([1.0, 0.0])  # q0
    qkv[0, 1, 0:2] = torch.tensor([1.0, 0.0])  # q1 (same row => same answer)
    qkv[0, 1, 2:4] = torch.tensor([math.sqrt(2.0) * math.log(3.0), 5.0])  # k1; second comp ignored by q
    qkv[0, 0, 4:6] = torch.tensor([4.0, 0.0])
    qkv[0, 1, 4:6] = torch.tensor([0.0, 8.0])
    want = torch.tensor([[[1.0, 6.0], [1.0, 6.0]]])
    got = torch_ref.sdpa_masked(qkv, torch.ones(1, 2, dtype=torch.bool), 1)
    assert torch.allclose(got, want, atol=1e-6)
    assert np.allclose(bruteforce.sdpa_masked_loops(qkv.numpy(), None, 1), want.numpy(), atol=1e-12)
    assert np.allclose(c_ref.sdpa_masked(qkv.numpy(), None, 1), want.numpy(), atol=1e-6)
    # killing key 1 leaves only V row 0
    dead1 = torch.tensor([[True, False]])
    assert torch.allclose(torch_ref.sdpa_masked(qkv, dead1, 1), torch.tensor([[[4.0, 0.0], [4.0, 0.0]]]), atol=1e-6)


@pytest.mark.parametrize("B,NM,H,dh,p_alive", [(2, 5, 2, 4, 0.6), (1, 7, 4, 8, 0.8), (3, 12, 4, 32, 0.85)])
def test_three_statements_agree(B, NM, H, dh, p_alive):
    D = H * dh
    qkv = _qkv(10 + NM, B, NM, D)
    g = torch.Generator().manual_seed(NM)
    alive = torch.rand(B, NM, generator=g) < p_alive
    alive[0, 0] = True
    brute = bruteforce.sdpa_masked_loops(qkv.numpy(), alive.numpy(), H)
    lib = torch_ref.sdpa_masked(qkv, alive, H).double().numpy()
    cc = c_ref.sdpa_masked(qkv.numpy(), alive.numpy(), H).astype(np.float64)
    assert np.abs(lib - brute).max() < 5e-6
    assert np.abs(cc - brute).max() < 5e-7
    # fp64 through the library routine as well
    lib64 = torch_ref.sdpa_masked(qkv.double(), alive, H).numpy()
    assert np.abs(lib64 - brute).max() < 1e-12


def test_head_split_is_head_major_and_qkv_order():
    # make head 1's V the only non-zero V: output must be non-zero only in head 1's columns
    B, NM, H, dh = 1, 4, 4, 8
    D = H * dh
    qkv = _qkv(3, B, NM, D)
    qkv[..., 2 * D:] = 0
    qkv[..., 2 * D + dh:2 * D + 2 * dh] = 1.0
    out = torch_ref.sdpa_masked(qkv, None, H)
    assert torch.allclose(out[..., dh:2 * dh], torch.ones(B, NM, dh), atol=1e-6)
    assert out[..., :dh].abs().max() == 0 and out[..., 2 * dh:].abs().max() == 0


def test_all_alive_equals_unmasked_library_call():
    B, NM, H, dh = 2, 9, 4, 16
    qkv = _qkv(4, B, NM, H * dh)
    a = torch_ref.sdpa_masked(qkv, torch.ones(B, NM, dtype=torch.bool), H)
    b = torch_ref.sdpa_masked(qkv, None, H)
    assert torch.allclose(a, b, atol=1e-6)


def test_single_alive_key_returns_its_value_row():
    B, NM, H, dh = 2, 6, 2, 8
    D = H * dh
    qkv = _qkv(5, B, NM, D)
    alive = torch.zeros(B, NM, dtype=torch.bool)
    alive[0, 4] = True
    alive[1, 1] = True
    out = torch_ref.sdpa_masked(qkv, alive, H)
    assert torch.allclose(out[0], qkv[0, 4, 2 * D:].expand(NM, D), atol=1e-6)
    assert torch.allclose(out[1], qkv[1, 1, 2 * D:].expand(NM, D), atol=1e-6)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 1.6e-2)])
def test_all_dead_is_uniform_mean_and_finite(dtype, tol):
    # tests/models/test_encoder.py:130-140: an all-dead mask must not produce NaN
    B, NM, H, dh = 2, 5, 2, 8
    D = H * dh
    qkv = _qkv(6, B, NM, D, dtype)
    alive = torch.zeros(B, NM, dtype=torch.bool)
    out = torch_ref.sdpa_masked(qkv, alive, H)
    assert torch.isfinite(out).all()
    mean_v = qkv[..., 2 * D:].float().mean(dim=1, keepdim=True).expand(B, NM, D)
    assert (out.float() - mean_v).abs().max() < tol
    if dtype == torch.float32:
        assert np.abs(c_ref.sdpa_masked(qkv.numpy(), alive.numpy(), H) - mean_v.numpy()).max() < tol


def test_dead_keys_cannot_influence_anything_but_their_own_query_row():
    B, NM, H, dh = 2, 8, 4, 8
    D = H * dh
    qkv = _qkv(7, B, NM, D)
    alive = torch.ones(B, NM, dtype=torch.bool)
    alive[:, 2] = False
    alive[:, 5] = False
    base = torch_ref.sdpa_masked(qkv, alive, H)
    pert = qkv.clone()
    pert[:, [2, 5], D:] += 100.0  # K and V of the dead tokens only
    again = torch_ref.sdpa_masked(pert, alive, H)
    assert torch.equal(base, again)
    # dead queries are still evaluated: their rows are ordinary softmax rows, not zeros
    assert base[:, 2].abs().max() > 0


def test_token_permutation_equivariance():
    B, NM, H, dh = 1, 7, 2, 8
    qkv = _qkv(8, B, NM, H * dh)
    alive = torch.tensor([[True, False, True, True, False, True, True]])
    perm = torch.tensor([3, 0, 6, 1, 5, 2, 4])
    a = torch_ref.sdpa_masked(qkv, alive, H)[:, perm]
    b = torch_ref.sdpa_masked(qkv[:, perm], alive[:, perm], H)
    assert torch.allclose(a, b, atol=1e-6)


def test_mask_dtype_follows_query_dtype(monkeypatch):
    # tests/models/test_encoder.py:142-176
    seen = {}
    real = F.scaled_dot_product_attention

    def spy(q, k, v, attn_mask=None, **kw):
        seen["q"], seen["m"] = q.dtype, attn_mask.dtype
        return real(q, k, v, attn_mask=attn_mask, **kw)

    monkeypatch.setattr(torch_ref.F, "scaled_dot_product_attention", spy)
    qkv = _qkv(9, 2, 4, 16, torch.bfloat16)
    alive = torch.tensor([[True, True, False, True], [True] * 4])
    torch_ref.sdpa_masked(qkv, alive, 4)
    assert seen["q"] == torch.bfloat16 and seen["m"] == torch.bfloat16


def test_bullet_read_is_masked_softmax_over_bullets_with_an_empty_gate():
    # attention.py:149-165: separate softmax over bullet keys; all-inactive environment => exactly 0
    B, N, NB, H, dh = 3, 4, 6, 2, 8
    D = H * dh
    g = torch.Generator().manual_seed(11)
    qkv = torch.randn(B, N, 3 * D, generator=g)
    kv = torch.randn(B, NB, 2 * D, generator=g)
    mask = torch.tensor([[True, False, True, True, False, True], [False] * 6, [False, False, False, True, False, False]])
    got = torch_ref.bullet_read(qkv, kv, mask, H)
    assert got[1].abs().max() == 0  # nothing in flight: gated off, not a uniform average
    assert torch.allclose(got[2], kv[2, 3, D:].expand(N, D), atol=1e-6)  # single active bullet: its V row
    # fp64 loops: same definition as masked attention with Q from one buffer and K/V from the other
    fake = torch.zeros(1, max(N, NB), 3 * D, dtype=torch.float64)
    fake[0, :N, :D] = qkv[0, :, :D]
    fake[0, :NB, D:] = kv[0]
    alive = torch.zeros(1, max(N, NB), dtype=torch.bool)
    alive[0, :NB] = mask[0]
    brute = bruteforce.sdpa_masked_loops(fake.numpy(), alive.numpy(), H)[0, :N]
    assert np.abs(got[0].double().numpy() - brute).max() < 5e-6
    # inactive slots cannot influence anything (tests/models/test_encoder.py:700-720)
    kv2 = kv.clone()
    kv2[~mask] += 500.0
    assert torch.equal(torch_ref.bullet_read(qkv, kv2, mask, H), got)
    assert torch.allclose(torch_ref.bullet_read(qkv, kv, None, H), torch_ref.bullet_read(qkv, kv, torch.ones(B, NB, dtype=torch.bool), H))


# ---------------------------------------------------------------- RG-LRU step


def test_log_lambda_init_is_linspace_0_4():
    lam = torch_ref.sigma_lambda_reference(128)
    for k in (0, 1, 64, 127):
        assert float(lam[k]) == pytest.approx(4.0 * k / 127.0, abs=1e-6)


def test_rglru_closed_forms():
    D = 4
    lam = torch.tensor([0.0, 1.0, 2.0, 4.0])
    h = torch.tensor([[1.0, -2.0, 3.0, 0.5]])
    x = torch.tensor([[0.3, 0.7, -1.1, 2.0]])
    big = 40.0
    # r -> 1, lambda = 0: a = 0.5 ** 8
    g = torch.full((1, 2 * D), big)
    out = torch_ref.rglru_step(torch.zeros(1, D), g, lam, 8.0, h)
    assert float(out[0, 0]) == pytest.approx(0.00390625 * 1.0, rel=1e-6)
    # x = 0: h' = a h with a = sigmoid(lambda)^(8 r), r = sigmoid(0.5)
    g = torch.full((1, 2 * D), 0.5)
    r = 1.0 / (1.0 + math.exp(-0.5))
    out = torch_ref.rglru_step(torch.zeros(1, D), g, lam, 8.0, h)
    for d in range(D):
        a = math.exp(8.0 * r * torch_ref.softplus_neg(float(lam[d])))
        assert float(out[0, d]) == pytest.approx(a * float(h[0, d]), rel=2e-6)
    # h = 0: h' = sqrt(1 - a^2) * i * x
    out = torch_ref.rglru_step(x, g, lam, 8.0, torch.zeros(1, D))
    for d in range(D):
        a = math.exp(8.0 * r * torch_ref.softplus_neg(float(lam[d])))
        assert float(out[0, d]) == pytest.approx(math.sqrt(1 - a * a) * r * float(x[0, d]), rel=2e-6)
    # r -> 0: a = 1, the clamp floor gives gate = 1e-3 (not 0); i -> 1
    g = torch.cat([torch.full((1, D), -big), torch.full((1, D), big)], dim=-1)
    out = torch_ref.rglru_step(x, g, lam, 8.0, h)
    assert torch.allclose(out, h + 1e-3 * x, rtol=1e-6, atol=1e-9)


def test_rglru_gate_columns_are_not_interchangeable():
    # swapping the two halves of gates_pre must change the answer (r drives a, i scales x)
    g = torch.Generator().manual_seed(0)
    x, h = torch.randn(3, 8, generator=g), torch.randn(3, 8, generator=g)
    gates = torch.randn(3, 16, generator=g)
    lam = torch.linspace(0, 4, 8)
    a = torch_ref.rglru_step(x, gates, lam, 8.0, h)
    b = torch_ref.rglru_step(x, torch.cat([gates[:, 8:], gates[:, :8]], -1), lam, 8.0, h)
    assert not torch.allclose(a, b, atol=1e-3)


def test_rglru_three_statements_agree():
    g = torch.Generator().manual_seed(1)
    R, D = 5, 16
    x, h = torch.randn(R, D, generator=g), 0.5 * torch.randn(R, D, generator=g)
    gates = 2.0 * torch.randn(R, 2 * D, generator=g)
    lam = torch.linspace(0, 4, D)
    brute = bruteforce.rglru_step_loops(x.numpy(), gates.numpy(), lam.numpy(), 8.0, h.numpy())
    t32 = torch_ref.rglru_step(x, gates, lam, 8.0, h).double().numpy()
    t64 = torch_ref.rglru_step(x.double(), gates.double(), lam.double(), 8.0, h.double()).numpy()
    cc = c_ref.rglru_step(x.numpy(), gates.numpy(), lam.numpy(), 8.0, h.numpy()).astype(np.float64)
    assert np.abs(t64 - brute).max() < 1e-13
    assert np.abs(t32 - brute).max() < 2e-6
    assert np.abs(cc - brute).max() < 2e-7


def test_rglru_bf16_gate_flow_keeps_state_fp32():
    # under autocast the gate pre-activations are bf16 and everything downstream of the
    # power is fp32 (griffin.py:181 promotes through the fp32 log_lambda parameter)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(4, 8, generator=g)
    gates = torch.randn(4, 16, generator=g).bfloat16()
    out = torch_ref.rglru_step(x, gates, torch.linspace(0, 4, 8), 8.0, torch.zeros(4, 8))
    assert out.dtype == torch.float32 and torch.isfinite(out).all()


# ---------------------------------------------------------------- temporal sublayer, block, packing


def _temporal(seed=0, D=16):
    gen = torch.Generator().manual_seed(seed)
    return temporal_params(gen, "t.", D), gen


def test_temporal_step_equals_sequence():
    # tests/models/test_encoder.py:466-514 (step path == sequence path, atol 1e-5)
    D, R, T = 16, 5, 7
    p, gen = _temporal()
    x_seq = torch.randn(R, T, D, generator=gen)
    h0 = 0.5 * torch.randn(R, D, generator=gen)
    cb0 = torch.randn(R, 3, D, generator=gen)
    seq_out, seq_h, seq_cb = torch_ref.temporal_sequence(p, "t.", x_seq, h0, cb0)
    h, cb, outs = h0, cb0, []
    for t in range(T):
        o, h, cb = torch_ref.temporal_step(p, "t.", x_seq[:, t], h, cb)
        outs.append(o)
    assert torch.allclose(torch.stack(outs, 1), seq_out, atol=1e-5)
    assert torch.allclose(h, seq_h, atol=1e-5) and torch.allclose(cb, seq_cb, atol=1e-6)


def test_temporal_step_equals_sequence_across_episode_boundary():
    # tests/models/test_encoder.py:516-569: reset of the packed state after done == done-aware sequence
    D, R, T = 16, 4, 8
    p, gen = _temporal(1)
    x_seq = torch.randn(R, T, D, generator=gen)
    h0 = 0.5 * torch.randn(R, D, generator=gen)
    cb0 = torch.randn(R, 3, D, generator=gen)
    done = torch.zeros(R, T, dtype=torch.bool)
    done[:2, 3] = True
    seq_out, seq_h, _ = torch_ref.temporal_sequence(p, "t.", x_seq, h0, cb0, done)
    h, cb, outs = h0, cb0, []
    for t in range(T):
        o, h, cb = torch_ref.temporal_step(p, "t.", x_seq[:, t], h, cb)
        outs.append(o)
        keep = (~done[:, t]).float()
        h, cb = h * keep[:, None], cb * keep[:, None, None]
    assert torch.allclose(torch.stack(outs, 1), seq_out, atol=1e-5)


def test_conv_buffer_is_shifted_oldest_to_newest():
    D, R = 16, 3
    p, gen = _temporal(2)
    x = torch.randn(R, D, generator=gen)
    cb = torch.randn(R, 3, D, generator=gen)
    _, _, cb_new = torch_ref.temporal_step(p, "t.", x, torch.zeros(R, D), cb)
    b1 = F.linear(torch_ref.rms_norm(x, p["t.norm1.weight"]), p["t.linear1.weight"])
    assert torch.equal(cb_new[:, 0], cb[:, 1]) and torch.equal(cb_new[:, 1], cb[:, 2])
    assert torch.allclose(cb_new[:, 2], b1)


def test_field_path_is_the_manual_composition_and_ignores_state():
    # tests/models/test_encoder.py:1070-1090, :1107-1131
    D, B, N, M = 16, 2, 3, 2
    gen = torch.Generator().manual_seed(3)
    p = block_params(gen, "b.", D, 1, 1)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    h_a, cb_a = torch.zeros(1, B * N, D), torch.zeros(1, B * N, 3, D)
    h_b, cb_b = torch.randn(1, B * N, D, generator=gen), torch.randn(1, B * N, 3, D, generator=gen)
    xa, _, _ = torch_ref.block_step(p, "b.", 1, 1, 4, x, alive, h_a, cb_a, N)
    xb, _, _ = torch_ref.block_step(p, "b.", 1, 1, 4, x, alive, h_b, cb_b, N)
    assert torch.equal(xa[:, N:], xb[:, N:])  # fields do not see recurrent state
    assert not torch.allclose(xa[:, :N], xb[:, :N])  # ships do
    after_spatial = torch_ref.spatial_sublayer(p, "b.spatial.0.", x, alive, 4)
    fields = after_spatial[:, N:]
    n = torch_ref.rms_norm(fields, p["b.temporal.0.norm1.weight"])
    b1 = F.linear(F.linear(n, p["b.temporal.0.linear1.weight"]), p["b.field_sub.0.weight"])
    b2 = F.gelu(F.linear(n, p["b.temporal.0.linear2.weight"]))
    x1 = fields + F.linear(b1 * b2, p["b.temporal.0.linear_out.weight"])
    manual = x1 + torch_ref.gated_mlp(p, "b.temporal.0.gated_mlp.", torch_ref.rms_norm(x1, p["b.temporal.0.norm2.weight"]))
    assert torch.allclose(xa[:, N:], manual, atol=1e-6)


def test_block_rows_are_env_major():
    # state row b*n_rec + n belongs to token n of environment b (griffin.py:408)
    D, B, N = 16, 3, 2
    gen = torch.Generator().manual_seed(4)
    p = block_params(gen, "b.", D, 0, 1)
    x = torch.randn(B, N, D, generator=gen)
    alive = torch.ones(B, N, dtype=torch.bool)
    h = torch.zeros(1, B * N, D)
    cb = torch.zeros(1, B * N, 3, D)
    base, _, _ = torch_ref.block_step(p, "b.", 0, 1, 4, x, alive, h, cb)
    h2 = h.clone()
    h2[0, 1 * N + 1] = 5.0  # env 1, token 1
    out, _, _ = torch_ref.block_step(p, "b.", 0, 1, 4, x, alive, h2, cb)
    changed = (out - base).abs().amax(-1) > 0
    want = torch.zeros(B, N, dtype=torch.bool)
    want[1, 1] = True
    assert torch.equal(changed, want)


def test_pack_unpack_roundtrip_and_reset():
    # tests/models/test_encoder.py:272-303, :384-405
    D, B, N, L = 8, 4, 3, 2
    g = torch.Generator().manual_seed(5)
    hidden = torch.randn(L, B * N, 4 * D, generator=g)
    h, cb = torch_ref.unpack_hidden(hidden, D)
    assert h.shape == (L, B * N, D) and cb.shape == (L, B * N, 3, D)
    assert torch.equal(cb[:, :, 0], hidden[:, :, D:2 * D]) and torch.equal(cb[:, :, 2], hidden[:, :, 3 * D:])
    assert torch.equal(torch_ref.pack_hidden(h, cb), hidden)
    done = torch.tensor([True, False, True, False])
    out = torch_ref.reset_hidden(hidden, done, N)
    for b in range(B):
        rows = out[:, b * N:(b + 1) * N]
        if done[b]:
            assert (rows == 0).all()
        else:
            assert torch.equal(rows, hidden[:, b * N:(b + 1) * N])


def test_trunk_step_shapes_and_hidden_layout():
    D, B, N, M = 16, 2, 3, 2
    p = trunk_params(0, D, 2, 2, 1)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(B, N + M, D, generator=g)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    hidden = torch.zeros(2, B * N, 4 * D)
    out, new_hidden = torch_ref.trunk_step(p, 2, 2, 1, 4, x, alive, hidden)
    assert out.shape == x.shape and new_hidden.shape == hidden.shape
    # the newest conv-buffer slot of layer 0 holds this step's linear1 output, older slots the shifted zeros
    assert (new_hidden[0, :, D:3 * D] == 0).all() and new_hidden[0, :, 3 * D:].abs().max() > 0


def test_harness_step_matches_its_parts():
    D, B, N, M = 16, 3, 2, 1
    g = torch.Generator().manual_seed(7)
    p = {
        "qkv.weight": torch.randn(3 * D, D, generator=g) * 0.2,
        "out_proj.weight": torch.randn(D, D, generator=g) * 0.2,
        "linear_a.weight": torch.randn(D, D, generator=g) * 0.2,
        "linear_a.bias": torch.randn(D, generator=g) * 0.1,
        "linear_x.weight": torch.randn(D, D, generator=g) * 0.2,
        "linear_x.bias": torch.randn(D, generator=g) * 0.1,
        "log_lambda": torch.linspace(0, 4, D),
    }
    tokens = torch.randn(B, N + M, D, generator=g)
    alive = torch.tensor([[True, False, True], [True, True, True], [False, False, True]])
    state = 0.5 * torch.randn(B * N, D, generator=g)
    hidden, new_state = torch_ref.harness_step(p, tokens, alive, state, 4)
    u = F.linear(torch_ref.sdpa_masked(F.linear(tokens, p["qkv.weight"]), alive, 4), p["out_proj.weight"])
    assert torch.equal(hidden[:, N:], u[:, N:])  # fields pass through un-recurred
    assert torch.equal(hidden[:, :N].reshape(B * N, D), new_state)
    ships = u[:, :N].reshape(B * N, D)
    want = torch_ref.rglru_step(ships, torch_ref.rglru_gates(p, "", ships), p["log_lambda"], 8.0, state)
    assert torch.equal(new_state, want)


# ---------------------------------------------------------------- sequence path (conv + scan over T)


def _episode_conv_bruteforce(b1, conv_buf, weight, bias, done):
    """Per row, per episode: library conv1d on that episode's inputs with zero history
    (the stored buffer is the history of the episode running at t = 0)."""
    R, T, D = b1.shape
    out = torch.zeros(R, T, D, dtype=b1.dtype)
    for r in range(R):
        start = 0
        hist = conv_buf[r]
        for t in range(T):
            last = t == T - 1 or bool(done[r, t])
            if last:
                seg = torch.cat([hist, b1[r, start:t + 1]], dim=0)  # (3 + len, D)
                y = F.conv1d(seg.t().unsqueeze(0), weight, bias, groups=D)[0].t()
                out[r, start:t + 1] = y
                start = t + 1
                hist = torch.zeros(3, D, dtype=b1.dtype)
    return out


@pytest.mark.parametrize("T", [1, 2, 3, 4, 9, 33])
def test_conv_sequence_is_the_library_conv_without_boundaries(T):
    g = torch.Generator().manual_seed(T)
    R, D = 3, 8
    b1 = torch.randn(R, T, D, generator=g, dtype=torch.float64)
    buf = torch.randn(R, 3, D, generator=g, dtype=torch.float64)
    w = torch.randn(D, 1, 4, generator=g, dtype=torch.float64)
    bias = torch.randn(D, generator=g, dtype=torch.float64)
    v, tail = torch_ref.conv_sequence(b1, buf, w, bias)
    lib = F.conv1d(torch.cat([buf, b1], 1).transpose(1, 2), w, bias, groups=D).transpose(1, 2)
    assert (v - lib).abs().max() < 1e-12
    assert torch.equal(tail, torch.cat([buf, b1], 1)[:, -3:])
    none_done = torch.zeros(R, T, dtype=torch.bool)
    assert torch.equal(torch_ref.conv_sequence(b1, buf, w, bias, none_done)[0], v)


@pytest.mark.parametrize("T,p", [(1, 0.5), (2, 0.5), (5, 0.4), (16, 0.3), (40, 0.1), (12, 1.0)])
def test_conv_sequence_cuts_taps_at_episode_ends(T, p):
    g = torch.Generator().manual_seed(100 + T)
    R, D = 4, 6
    b1 = torch.randn(R, T, D, generator=g, dtype=torch.float64)
    buf = torch.randn(R, 3, D, generator=g, dtype=torch.float64)
    w = torch.randn(D, 1, 4, generator=g, dtype=torch.float64)
    bias = torch.randn(D, generator=g, dtype=torch.float64)
    done = torch.rand(R, T, generator=g) < p
    v, tail = torch_ref.conv_sequence(b1, buf, w, bias, done)
    assert (v - _episode_conv_bruteforce(b1, buf, w, bias, done)).abs().max() < 1e-12
    assert torch.equal(tail, torch.cat([buf, b1], 1)[:, -3:])  # the stored inputs are not cut
    # a done flag at the last step changes nothing inside the sequence
    d2 = done.clone()
    d2[:, -1] = ~d2[:, -1]
    assert torch.equal(torch_ref.conv_sequence(b1, buf, w, bias, d2)[0], v)


def _loop_of_steps(x, gates, lam, c, h0, done):
    h, ys = h0, []
    for t in range(x.shape[1]):
        if done is not None and t > 0:
            h = h * (~done[:, t - 1]).to(h.dtype).unsqueeze(-1)
        h = torch_ref.rglru_step(x[:, t], gates[:, t], lam, c, h)
        ys.append(h)
    return torch.stack(ys, dim=1)


@pytest.mark.parametrize("T,p", [(1, 0.0), (2, 0.5), (3, 0.0), (7, 0.3), (128, 0.05), (130, 0.0), (64, 1.0)])
def test_rglru_sequence_scan_equals_the_step_loop(T, p):
    # tests/models/test_encoder.py:179-268 asserts the same at T = 1 and T = 128
    g = torch.Generator().manual_seed(200 + T)
    R, D = 3, 16
    x = torch.randn(R, T, D, generator=g, dtype=torch.float64)
    gates = 2.0 * torch.randn(R, T, 2 * D, generator=g, dtype=torch.float64)
    lam = torch.linspace(0.0, 4.0, D, dtype=torch.float64)
    h0 = torch.randn(R, D, generator=g, dtype=torch.float64)
    done = (torch.rand(R, T, generator=g) < p) if p > 0 else None
    ys, last = torch_ref.rglru_sequence(x, gates, lam, 8.0, h0, done)
    want = _loop_of_steps(x, gates, lam, 8.0, h0, done)
    assert (ys - want).abs().max() < 1e-12
    assert torch.equal(last, ys[:, -1])
    ys32, _ = torch_ref.rglru_sequence(x.float(), gates.float(), lam.float(), 8.0, h0.float(), done)
    assert (ys32.double() - want).abs().max() < 2e-5


def test_rglru_sequence_forgets_everything_after_an_episode_end():
    g = torch.Generator().manual_seed(7)
    R, T, D = 2, 10, 8
    x = torch.randn(R, T, D, generator=g)
    gates = torch.randn(R, T, 2 * D, generator=g)
    lam = torch.linspace(0.0, 4.0, D)
    done = torch.zeros(R, T, dtype=torch.bool)
    done[:, 4] = True
    a, _ = torch_ref.rglru_sequence(x, gates, lam, 8.0, torch.randn(R, D, generator=g), done)
    x2 = x.clone()
    x2[:, :5] += 3.0
    b, _ = torch_ref.rglru_sequence(x2, gates, lam, 8.0, torch.randn(R, D, generator=g), done)
    assert torch.equal(a[:, 5:], b[:, 5:]) and not torch.equal(a[:, :5], b[:, :5])


# ---------------------------------------------------------------- team pooling (policy.py:78-120)


def _team_case(seed, B=4, N=7, D=32, H=4, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    p = {
        "tp.seeds": 0.5 * torch.randn(2, D, generator=g, dtype=dtype),
        "tp.attn.in_proj_weight": torch.randn(3 * D, D, generator=g, dtype=dtype) / D ** 0.5,
        "tp.attn.out_proj.weight": torch.randn(D, D, generator=g, dtype=dtype) / D ** 0.5,
        "tp.norm.weight": 1.0 + 0.2 * torch.randn(D, generator=g, dtype=dtype),
    }
    x = torch.randn(B, N, D, generator=g, dtype=dtype)
    team = torch.randint(0, 2, (B, N), generator=g, dtype=torch.int32)
    alive = torch.rand(B, N, generator=g) < 0.7
    team[0] = 0            # env 0: nobody on team 1
    alive[1] = False       # env 1: everyone dead
    alive[2] = True
    return p, x, team, alive, H


def _reference_forward_with_library_modules(p, x, team_id, alive, H):
    """The text of policy.py:94-120 on torch's own nn.MultiheadAttention / nn.RMSNorm."""
    B, N, D = x.shape
    attn = torch.nn.MultiheadAttention(D, H, batch_first=True, bias=False, dtype=x.dtype)
    norm = torch.nn.RMSNorm(D, dtype=x.dtype)
    with torch.no_grad():
        attn.in_proj_weight.copy_(p["tp.attn.in_proj_weight"])
        attn.out_proj.weight.copy_(p["tp.attn.out_proj.weight"])
        norm.weight.copy_(p["tp.norm.weight"])
        pool = x.new_zeros(B, 2, D)
        for t in range(2):
            mask = (team_id == t) & alive
            seed = p["tp.seeds"][t].view(1, 1, D).expand(B, 1, D)
            out, _ = attn(seed, x, x, key_padding_mask=~mask, need_weights=False)
            out = out.squeeze(1).nan_to_num(0.0)
            out = out * mask.any(dim=1).unsqueeze(1).to(out.dtype)
            pool[:, t] = norm(out)
        idx = team_id.clamp(0, 1).long().unsqueeze(-1).expand(B, N, D)
        return pool.gather(1, idx), pool


@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-12), (torch.float32, 2e-6)])
def test_team_pool_is_the_library_attention_composition(dtype, tol):
    p, x, team, alive, H = _team_case(3, dtype=dtype)
    ships, pool = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    ships_lib, pool_lib = _reference_forward_with_library_modules(p, x, team, alive, H)
    assert torch.allclose(pool, pool_lib, rtol=tol, atol=tol)
    assert torch.allclose(ships, ships_lib, rtol=tol, atol=tol)


def test_team_pool_matches_brute_force_and_closed_forms():
    p, x, team, alive, H = _team_case(4)
    ships, pool = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    eps = torch.finfo(torch.float64).eps
    loops = bruteforce.team_pool_loops(x.numpy(), team.numpy(), alive.numpy(), p["tp.seeds"].numpy(),
                                       p["tp.attn.in_proj_weight"].numpy(), p["tp.attn.out_proj.weight"].numpy(),
                                       p["tp.norm.weight"].numpy(), H, eps)
    assert np.allclose(pool.numpy(), loops, rtol=1e-10, atol=1e-12)
    # empty teams pool to exactly zero; every ship carries the pooled vector of its (clamped) team
    assert (pool[0, 1] == 0).all() and (pool[1] == 0).all()
    B, N, D = x.shape
    for b in range(B):
        for n in range(N):
            assert torch.equal(ships[b, n], pool[b, int(team[b, n].clamp(0, 1))])
    # one alive ship on a team: softmax over one key is 1 whatever the seed says, so the pooled
    # vector is RMSNorm(W_o W_v x_j)
    one = alive.clone()
    one[3] = False
    one[3, 2] = True
    t = int(team[3, 2])
    _, pool_one = torch_ref.team_pool(p, "tp.", x, team, one, H)
    D = x.shape[-1]
    direct = p["tp.attn.out_proj.weight"] @ (p["tp.attn.in_proj_weight"][2 * D:] @ x[3, 2])
    assert torch.allclose(pool_one[3, t], torch_ref.rms_norm(direct, p["tp.norm.weight"]), rtol=1e-10, atol=1e-12)
    assert (pool_one[3, 1 - t] == 0).all()


def test_team_pool_ignores_dead_ships_other_teams_and_field_ids():
    p, x, team, alive, H = _team_case(5)
    _, base = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    pert = x.clone()
    pert[~alive] = pert[~alive] * -3.0 + 5.0  # dead ships are no keys of either team
    _, again = torch_ref.team_pool(p, "tp.", pert, team, alive, H)
    assert torch.equal(base, again)
    # team 0's pool does not move when only team-1 ships change, and the other way round
    pert = x.clone()
    pert[team == 1] += 1.0
    _, again = torch_ref.team_pool(p, "tp.", pert, team, alive, H)
    assert torch.equal(base[:, 0], again[:, 0]) and not torch.equal(base[:, 1], again[:, 1])
    # an id outside {0, 1} (field tokens carry 2) is nobody's key but reads team 1's pool
    odd = team.clone()
    odd[2, 0] = 2
    ships, pool = torch_ref.team_pool(p, "tp.", x, odd, alive, H)
    assert torch.equal(ships[2, 0], pool[2, 1])
    stay = alive.clone()
    stay[2, 0] = False
    _, without = torch_ref.team_pool(p, "tp.", x, team, stay, H)
    assert torch.allclose(pool[2], without[2], rtol=1e-12, atol=1e-12)
    # ship order inside an environment does not matter for the pools
    perm = torch.randperm(x.shape[1], generator=torch.Generator().manual_seed(1))
    _, shuffled = torch_ref.team_pool(p, "tp.", x[:, perm], team[:, perm], alive[:, perm], H)
    assert torch.allclose(base, shuffled, rtol=1e-10, atol=1e-12)
