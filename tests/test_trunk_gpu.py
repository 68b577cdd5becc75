"""The drop-in trunk layers on the GPU against the CPU oracle fed the same state_dict.

These mirror the reference's own layer tests (tests/models/test_encoder.py): shape and
finiteness of the attention block incl. the all-dead mask (:106-140), the RG-LRU sequence
against its step loop (:198-268), step == sequence across sublayer layouts and an episode
boundary (:466-569), the field path (:1041-1203) and hidden-state handling (:272-303,
:384-405).  Numeric bars: float32 1e-5, bf16 autocast 2e-2 (max|y-ref|/max|ref|); GEMMs,
norms and GELUs are library calls on both sides.
"""

import pytest
import torch

from helpers import (assert_float32_bar, block_params, float64_truth, max_rel, team_case, team_pool_params, temporal_params,
                     trunk_params)
from oracle import torch_ref

import boost_and_broadside_amd as bnb

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32_TOL = 1e-5
BF16_TOL = 2e-2


def _strip(p, prefix):
    return {k[len(prefix):]: v for k, v in p.items() if k.startswith(prefix)}


def _cfg(D=64, H=4, blocks=1, spatial=1, temporal=1, bullets=0):
    return bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=blocks, n_spatial_per_block=spatial,
                           n_temporal_per_block=temporal, n_bullet_cross_per_block=bullets)


# ------------------------------------------------------------------ TransformerBlock


@pytest.mark.parametrize("D,H,B,N", [(64, 4, 3, 8), (128, 4, 5, 12), (128, 4, 2, 23), (32, 4, 2, 4)])
def test_transformer_block_matches_oracle_fp32(D, H, B, N):
    gen = torch.Generator().manual_seed(D + N)
    p = block_params(gen, "b.", D, 1, 0)
    layer = bnb.TransformerBlock(_cfg(D, H)).eval()
    layer.load_state_dict(_strip(p, "b.spatial.0."))
    layer.to(DEV)
    x = torch.randn(B, N, D, generator=gen)
    alive = torch.rand(B, N, generator=gen) < 0.7
    alive[:, 0] = True
    with torch.no_grad():
        got = layer(x.to(DEV), alive_mask=alive.to(DEV)).cpu()
        got_nomask = layer(x.to(DEV)).cpu()
    assert got.shape == (B, N, D)
    assert max_rel(got, torch_ref.spatial_sublayer(p, "b.spatial.0.", x, alive, H)) <= F32_TOL
    assert max_rel(got_nomask, torch_ref.spatial_sublayer(p, "b.spatial.0.", x, None, H)) <= F32_TOL


def test_transformer_block_all_dead_mask_is_finite():
    layer = bnb.TransformerBlock(_cfg()).to(DEV).eval()
    x = torch.randn(1, 4, 64, device=DEV)
    with torch.no_grad():
        out = layer(x, alive_mask=torch.zeros(1, 4, dtype=torch.bool, device=DEV))
    assert not torch.isnan(out).any() and torch.isfinite(out).all()


def test_transformer_block_under_bf16_autocast_feeds_bf16_to_the_kernel(monkeypatch):
    # under autocast the qkv Linear emits bf16 while the norm keeps x fp32 (test_encoder.py:142-176):
    # the kernel must see the bf16 projection and the residual stream must stay fp32
    gen = torch.Generator().manual_seed(3)
    D, H, B, N = 128, 4, 4, 12
    p = block_params(gen, "b.", D, 1, 0)
    layer = bnb.TransformerBlock(_cfg(D, H)).eval()
    layer.load_state_dict(_strip(p, "b.spatial.0."))
    layer.to(DEV)
    seen = {}
    real = bnb.ops.sdpa_masked

    def spy(qkv, alive, n_heads, **kw):
        seen["dtype"] = qkv.dtype
        return real(qkv, alive, n_heads, **kw)

    monkeypatch.setattr(bnb.trunk.ops, "sdpa_masked", spy)
    x = torch.randn(B, N, D, generator=gen)
    alive = torch.rand(B, N, generator=gen) < 0.8
    alive[:, 1] = True
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        got = layer(x.to(DEV), alive_mask=alive.to(DEV))
    assert seen["dtype"] == torch.bfloat16 and got.dtype == torch.float32
    assert max_rel(got.cpu(), torch_ref.spatial_sublayer(p, "b.spatial.0.", x, alive, H)) <= BF16_TOL


def test_layers_train_through_torch_ops_and_refuse_host_tensors():
    layer = bnb.TransformerBlock(_cfg()).to(DEV)
    x = torch.randn(2, 4, 64, device=DEV)
    alive = torch.tensor([[True, True, False, True], [True, False, False, True]], device=DEV)
    with torch.no_grad():
        want = layer(x, alive)
    got = layer(x, alive)  # grad mode on, parameters require grad: the differentiable composition
    assert got.requires_grad and max_rel(got.detach().cpu(), want.cpu()) <= 2e-5
    got.sum().backward()
    assert all(p.grad is not None for p in layer.parameters())
    qkv = torch.randn(1, 4, 192, device=DEV, requires_grad=True)
    with pytest.raises(RuntimeError, match="forward-only"):
        bnb.sdpa_masked(qkv, None, 4)  # the kernels themselves have no backward
    with pytest.raises(RuntimeError, match="no host fallback"):
        with torch.no_grad():
            bnb.TransformerBlock(_cfg())(torch.randn(1, 4, 64))


def test_bullet_cross_attention_matches_manual_composition():
    # attention.py:149-166: separate softmax over bullet keys, gated off when no bullet is active
    gen = torch.Generator().manual_seed(5)
    D, H, B, N, NB = 64, 4, 3, 6, 10
    layer = bnb.TransformerBlock(_cfg(D, H, spatial=1, bullets=1), reads_bullets=True).to(DEV).eval()
    x = torch.randn(B, N, D, generator=gen).to(DEV)
    alive = torch.ones(B, N, dtype=torch.bool, device=DEV)
    bullets = torch.randn(B, NB, D, generator=gen).to(DEV)
    bmask = (torch.rand(B, NB, generator=gen) < 0.5).to(DEV)
    bmask[0] = False  # nothing in flight in env 0: contribution must vanish there
    with torch.no_grad():
        with_b = layer(x, alive, bullets, bmask)
        without = layer(x, alive)
    assert torch.allclose(with_b[0], without[0], atol=1e-6)
    assert not torch.allclose(with_b[1], without[1], atol=1e-4)


# ------------------------------------------------------------------ RG-LRU and temporal block


def test_rglru_sequence_equals_step_loop_and_oracle():
    # test_encoder.py:198-225 at D=32, T=1 and T=16
    torch.manual_seed(0)
    D, R = 32, 8
    unit = bnb.RGLRU(D).to(DEV).eval()
    p = {k: v.detach().cpu() for k, v in unit.state_dict().items()}
    gen = torch.Generator().manual_seed(2)
    for T in (1, 16):
        x_seq = torch.randn(R, T, D, generator=gen)
        h0 = torch.randn(R, D, generator=gen)
        with torch.no_grad():
            out, h_last = unit.forward_sequence(x_seq.to(DEV), h0.to(DEV))
        assert out.shape == (R, T, D)
        h = h0
        for t in range(T):
            h = torch_ref.rglru_step(x_seq[:, t], torch_ref.rglru_gates(p, "", x_seq[:, t]), p["log_lambda"], 8.0, h)
            assert torch.allclose(out[:, t].cpu(), h, atol=1e-5)
        assert torch.allclose(h_last.cpu(), h, atol=1e-5)


def test_rglru_done_mask_cuts_the_state():
    # test_encoder.py:227-256
    torch.manual_seed(0)
    D, R, T = 32, 2, 8
    unit = bnb.RGLRU(D).to(DEV).eval()
    gen = torch.Generator().manual_seed(4)
    x_seq = torch.randn(R, T, D, generator=gen).to(DEV)
    h0 = torch.randn(R, D, generator=gen).to(DEV)
    done = torch.zeros(R, T, dtype=torch.bool, device=DEV)
    done[0, 3] = True
    with torch.no_grad():
        with_done, _ = unit.forward_sequence(x_seq, h0, done)
        no_done, _ = unit.forward_sequence(x_seq, h0)
        fresh, _ = unit.forward_sequence(x_seq[:, 4:], torch.zeros(R, D, device=DEV))
    assert torch.allclose(with_done[0, :4], no_done[0, :4], atol=1e-6)
    assert not torch.allclose(with_done[0, 4:], no_done[0, 4:], atol=1e-6)
    assert torch.allclose(with_done[1], no_done[1], atol=1e-6)
    assert torch.allclose(with_done[0, 4:], fresh[0], atol=1e-5)


@pytest.mark.parametrize("D,R", [(64, 10), (128, 33)])
def test_temporal_block_step_matches_oracle(D, R):
    gen = torch.Generator().manual_seed(D)
    p = temporal_params(gen, "t.", D)
    layer = bnb.GriffinTemporalBlock(D).eval()
    layer.load_state_dict(_strip(p, "t."))
    layer.to(DEV)
    x = torch.randn(R, D, generator=gen)
    h0 = 0.5 * torch.randn(R, D, generator=gen)
    cb = torch.randn(R, 3, D, generator=gen)
    with torch.no_grad():
        out, h1, cb1 = layer.forward_sequence(x.unsqueeze(1).to(DEV), h0.to(DEV), cb.to(DEV))
    ref_out, ref_h, ref_cb = torch_ref.temporal_step(p, "t.", x, h0, cb)
    assert out.shape == (R, 1, D) and cb1.shape == (R, 3, D)
    assert max_rel(out[:, 0].cpu(), ref_out) <= F32_TOL
    assert max_rel(h1.cpu(), ref_h) <= F32_TOL
    assert max_rel(cb1.cpu(), ref_cb) <= F32_TOL


def test_temporal_block_sequence_with_done_matches_oracle_sequence():
    D, R, T = 64, 6, 7
    gen = torch.Generator().manual_seed(8)
    p = temporal_params(gen, "t.", D)
    layer = bnb.GriffinTemporalBlock(D).eval()
    layer.load_state_dict(_strip(p, "t."))
    layer.to(DEV)
    x_seq = torch.randn(R, T, D, generator=gen)
    h0 = 0.5 * torch.randn(R, D, generator=gen)
    cb = torch.randn(R, 3, D, generator=gen)
    done = torch.zeros(R, T, dtype=torch.bool)
    done[:3, 2] = True
    with torch.no_grad():
        out, h1, cb1 = layer.forward_sequence(x_seq.to(DEV), h0.to(DEV), cb.to(DEV), done.to(DEV))
    ref_out, ref_h, ref_cb = torch_ref.temporal_sequence(p, "t.", x_seq, h0, cb, done)
    t_out, t_h, t_cb = float64_truth(torch_ref.temporal_sequence, p, "t.", x_seq, h0, cb, done)
    assert_float32_bar(out.cpu(), ref_out, t_out, "temporal sequence, output")
    assert_float32_bar(h1.cpu(), ref_h, t_h, "temporal sequence, state")
    assert_float32_bar(cb1.cpu(), ref_cb, t_cb, "temporal sequence, conv inputs")


@pytest.mark.parametrize("time_major", [False, True])
def test_temporal_block_sequence_under_autocast_matches_oracle(time_major):
    # the update path's precision: bf16 projections around fp32 conv and recurrence, T = 128
    D, R, T = 128, 24, 128
    gen = torch.Generator().manual_seed(18)
    p = temporal_params(gen, "t.", D)
    layer = bnb.GriffinTemporalBlock(D).eval()
    layer.load_state_dict(_strip(p, "t."))
    layer.to(DEV)
    x_seq = torch.randn(R, T, D, generator=gen)
    h0 = 0.5 * torch.randn(R, D, generator=gen)
    cb = torch.randn(R, 3, D, generator=gen)
    done = torch.rand(R, T, generator=gen) < 0.03
    xin = x_seq.transpose(0, 1).contiguous() if time_major else x_seq
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        out, h1, cb1 = layer.forward_sequence(xin.to(DEV), h0.to(DEV), cb.to(DEV), done.to(DEV), time_major=time_major)
    if time_major:
        out = out.transpose(0, 1)
    ref_out, ref_h, ref_cb = torch_ref.temporal_sequence(p, "t.", x_seq, h0, cb, done)
    assert max_rel(out.float().cpu(), ref_out) <= BF16_TOL
    assert max_rel(h1.cpu(), ref_h) <= BF16_TOL
    assert max_rel(cb1.cpu(), ref_cb) <= BF16_TOL


# ------------------------------------------------------------------ block and trunk


@pytest.mark.parametrize("spatial,temporal,N,M", [(1, 1, 3, 2), (2, 1, 8, 4), (3, 2, 5, 0), (2, 0, 4, 2)])
def test_block_step_matches_oracle(spatial, temporal, N, M):
    D, H, B = 64, 4, 3
    gen = torch.Generator().manual_seed(spatial * 10 + temporal)
    p = block_params(gen, "b.", D, spatial, temporal)
    block = bnb.YemongBlock(_cfg(D, H, 1, spatial, temporal)).eval()
    block.load_state_dict(_strip(p, "b."))
    block.to(DEV)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.rand(B, N + M, generator=gen) < 0.8
    alive[:, N:] = True
    alive[:, 0] = True
    h = 0.5 * torch.randn(temporal, B * N, D, generator=gen)
    cb = torch.randn(temporal, B * N, 3, D, generator=gen)
    with torch.no_grad():
        out, h1, cb1 = block.step(x.to(DEV), alive.to(DEV), h.to(DEV), cb.to(DEV), N)
    ref_out, ref_h, ref_cb = torch_ref.block_step(p, "b.", spatial, temporal, H, x, alive, h, cb, N)
    t_out, t_h, t_cb = float64_truth(torch_ref.block_step, p, "b.", spatial, temporal, H, x, alive, h, cb, N)
    assert out.shape == x.shape and h1.shape == h.shape and cb1.shape == cb.shape
    assert_float32_bar(out.cpu(), ref_out, t_out, f"block step {spatial}+{temporal}, output")
    if temporal:
        assert_float32_bar(h1.cpu(), ref_h, t_h, f"block step {spatial}+{temporal}, state")
        assert_float32_bar(cb1.cpu(), ref_cb, t_cb, f"block step {spatial}+{temporal}, conv inputs")


@pytest.mark.parametrize("blocks,spatial,temporal", [(2, 1, 1), (2, 2, 1), (1, 3, 2)])
def test_trunk_step_equals_sequence_and_oracle(blocks, spatial, temporal):
    # the load-bearing property of the trunk (test_encoder.py:466-514): rolling out step by step
    # and re-evaluating the stored sequence agree
    D, H, B, N, M, T = 64, 4, 2, 3, 2, 6
    p = trunk_params(blocks * 7 + spatial, D, blocks, spatial, temporal)
    trunk = bnb.YemongTrunk(_cfg(D, H, blocks, spatial, temporal)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    gen = torch.Generator().manual_seed(7)
    xs = torch.randn(T, B, N + M, D, generator=gen)
    alive = torch.ones(T, B, N + M, dtype=torch.bool)
    alive[2:, 0, 1] = False
    hidden0 = trunk.initial_hidden(B, N, DEV)
    assert hidden0.shape == (blocks * temporal, B * N, 4 * D)

    hidden, ref_hidden, true_hidden, outs = hidden0, hidden0.cpu(), hidden0.cpu().double(), []
    for t in range(T):
        out, hidden = trunk(xs[t].to(DEV), alive[t].to(DEV), hidden)
        ref_out, ref_hidden = torch_ref.trunk_step(p, blocks, spatial, temporal, H, xs[t], alive[t], ref_hidden)
        true_out, true_hidden = float64_truth(torch_ref.trunk_step, p, blocks, spatial, temporal, H, xs[t], alive[t], true_hidden)
        assert_float32_bar(out.cpu(), ref_out, true_out, f"trunk {blocks}x({spatial}+{temporal}) step {t}, output")
        outs.append(out)
    assert_float32_bar(hidden.cpu(), ref_hidden, true_hidden, f"trunk {blocks}x({spatial}+{temporal}) after {T} steps, state")

    # sequence path over the same inputs
    x = xs.to(DEV)
    h_all, cb_all = hidden0[:, :, :D], hidden0[:, :, D:].reshape(blocks * temporal, B * N, 3, D)
    with torch.no_grad():
        for i, block in enumerate(trunk.yemong_layers):
            sl = slice(i * temporal, (i + 1) * temporal)
            x, _, _ = block.sequence(x, alive.to(DEV), h_all[sl], cb_all[sl], None, N)
    assert torch.allclose(x, torch.stack(outs), atol=1e-4)


def test_trunk_reset_between_steps_equals_done_aware_sequence():
    # test_encoder.py:516-569: zeroing the packed state after a done env == sequence path with done_mask
    D, H, B, N, M, T = 64, 4, 2, 3, 2, 8
    p = trunk_params(11, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    gen = torch.Generator().manual_seed(11)
    xs = torch.randn(T, B, N + M, D, generator=gen).to(DEV)
    alive = torch.ones(T, B, N + M, dtype=torch.bool, device=DEV)
    done = torch.zeros(T, B, dtype=torch.bool, device=DEV)
    done[3] = True
    hidden0 = trunk.initial_hidden(B, N, DEV)
    hidden, outs = hidden0, []
    for t in range(T):
        out, hidden = trunk(xs[t], alive[t], hidden)
        outs.append(out)
        hidden = trunk.reset_hidden_for_envs(hidden, done[t], N)
    x = xs
    h_all, cb_all = hidden0[:, :, :D], hidden0[:, :, D:].reshape(2, B * N, 3, D)
    with torch.no_grad():
        for i, block in enumerate(trunk.yemong_layers):
            x, _, _ = block.sequence(x, alive, h_all[i:i + 1], cb_all[i:i + 1], done, N)
    assert torch.allclose(x, torch.stack(outs), atol=1e-4)


def test_state_sized_with_all_tokens_makes_fields_recurrent():
    # policy.py:318-322: n_rec is read off the hidden tensor
    D, H, B, N, M = 64, 4, 2, 3, 2
    p = trunk_params(3, D, 1, 1, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 1, 1, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    hidden = torch.randn(1, B * (N + M), 4 * D, generator=gen)
    out, new_hidden = trunk(x.to(DEV), alive.to(DEV), hidden.to(DEV))
    ref_out, ref_hidden = torch_ref.trunk_step(p, 1, 1, 1, H, x, alive, hidden)
    true_out, true_hidden = float64_truth(torch_ref.trunk_step, p, 1, 1, 1, H, x, alive, hidden)
    assert new_hidden.shape == hidden.shape
    assert_float32_bar(out.cpu(), ref_out, true_out, "trunk with recurrent fields, output")
    assert_float32_bar(new_hidden.cpu(), ref_hidden, true_hidden, "trunk with recurrent fields, state")


def test_trunk_under_autocast_matches_oracle_within_bf16_bar():
    # rollout configuration: 2 blocks x (2 spatial + 1 temporal), d_model 128, bf16 autocast
    D, H, B, N, M = 128, 4, 16, 8, 4
    p = trunk_params(21, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    gen = torch.Generator().manual_seed(21)
    hidden, ref_hidden = trunk.initial_hidden(B, N, DEV), torch.zeros(2, B * N, 4 * D)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    for t in range(4):
        x = torch.randn(B, N + M, D, generator=gen)
        alive[:, :N] &= torch.rand(B, N, generator=gen) > 0.1
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, hidden = trunk(x.to(DEV), alive.to(DEV), hidden)
        ref_out, ref_hidden = torch_ref.trunk_step(p, 2, 2, 1, H, x, alive, ref_hidden)
        assert hidden.dtype == torch.float32
        assert max_rel(out.float().cpu(), ref_out) <= BF16_TOL, t
        assert max_rel(hidden.cpu(), ref_hidden) <= BF16_TOL, t


def test_trunk_folded_reset_equals_reset_then_step_and_leaves_input_state_alone():
    # policy.py:268-285 zeroes the packed state of finished environments in a separate pass;
    # reset_mask folds that into the step kernels
    D, H, B, N, M = 128, 4, 6, 8, 4
    p = trunk_params(31, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    gen = torch.Generator().manual_seed(31)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    alive[2, 3] = False
    hidden = torch.randn(2, B * N, 4 * D, generator=gen)
    done = torch.tensor([False, True, False, False, True, False])
    dev_hidden = hidden.to(DEV)
    out_a, state_a = trunk(x.to(DEV), alive.to(DEV), dev_hidden, reset_mask=done.to(DEV))
    assert torch.equal(dev_hidden.cpu(), hidden)
    out_b, state_b = trunk(x.to(DEV), alive.to(DEV), trunk.reset_hidden_for_envs(dev_hidden, done.to(DEV), N))
    assert torch.equal(out_a, out_b) and torch.equal(state_a, state_b)
    ref_out, ref_state = torch_ref.trunk_step(p, 2, 2, 1, H, x, alive, torch_ref.reset_hidden(hidden, done, N))
    true_out, true_state = float64_truth(torch_ref.trunk_step, p, 2, 2, 1, H, x, alive, torch_ref.reset_hidden(hidden, done, N))
    assert_float32_bar(out_a.cpu(), ref_out, true_out, "trunk with folded reset, output")
    assert_float32_bar(state_a.cpu(), ref_state, true_state, "trunk with folded reset, state")
    # preallocated destination
    dest = torch.empty_like(dev_hidden)
    _, state_c = trunk(x.to(DEV), alive.to(DEV), dev_hidden, reset_mask=done.to(DEV), out_state=dest)
    assert state_c.data_ptr() == dest.data_ptr() and torch.equal(dest, state_a)
    with pytest.raises(ValueError):
        trunk(x.to(DEV), alive.to(DEV), dev_hidden, out_state=dev_hidden)


@pytest.mark.parametrize("autocast_dtype", [None, torch.bfloat16])
def test_graphed_trunk_replays_match_eager_steps(autocast_dtype):
    # every replay is checked against the eager step, with eager work and synchronisations in between
    D, H, B, N, M = 128, 4, 32, 8, 4
    p = trunk_params(41, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    graphed = bnb.GraphedTrunk(trunk, B, N + M, N, autocast_dtype=autocast_dtype)
    gen = torch.Generator().manual_seed(41)
    eager_state = trunk.initial_hidden(B, N, DEV)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    for t in range(6):
        x = torch.randn(B, N + M, D, generator=gen).to(DEV)
        alive[:, :N] &= torch.rand(B, N, generator=gen) > 0.1
        done = torch.rand(B, generator=gen) < 0.2 if t in (2, 4) else None
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast_dtype is not None):
            ref_out, eager_state = trunk(x, alive.to(DEV), eager_state,
                                         reset_mask=None if done is None else done.to(DEV))
        torch.cuda.synchronize()
        out, state = graphed.step(x, alive.to(DEV), None if done is None else done.to(DEV))
        assert torch.equal(out, ref_out), t
        assert torch.equal(state, eager_state), t
        assert state.data_ptr() == graphed.state.data_ptr()


@pytest.mark.parametrize("autocast", [False, True])
def test_bullet_reading_block_matches_oracle(autocast):
    # fp32 goes through the library SDPA path, bf16 autocast through the matrix-core cross kernel
    D, H, B, N, NB = 128, 4, 4, 12, 80
    gen = torch.Generator().manual_seed(17)
    p = block_params(gen, "b.", D, 1, 0)
    p["b.spatial.0.norm_bullet.weight"] = 1.0 + 0.1 * torch.randn(D, generator=gen)
    p["b.spatial.0.kv_bullet.weight"] = 0.1 * torch.randn(2 * D, D, generator=gen)
    layer = bnb.TransformerBlock(_cfg(D, H, spatial=1, bullets=1), reads_bullets=True).eval()
    layer.load_state_dict(_strip(p, "b.spatial.0."))
    layer.to(DEV)
    x = torch.randn(B, N, D, generator=gen)
    alive = torch.rand(B, N, generator=gen) < 0.8
    alive[:, 0] = True
    bullets = torch.randn(B, NB, D, generator=gen)
    bmask = torch.rand(B, NB, generator=gen) < 0.3
    bmask[0] = False
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        got = layer(x.to(DEV), alive.to(DEV), bullets.to(DEV), bmask.to(DEV))
    ref = torch_ref.spatial_sublayer(p, "b.spatial.0.", x, alive, H, bullets, bmask)
    assert max_rel(got.float().cpu(), ref) <= (BF16_TOL if autocast else F32_TOL)


# ------------------------------------------------------------------ training path (gradients)


def test_temporal_block_sequence_gradients_match_autograd_of_the_oracle():
    D, R, T = 64, 5, 9
    gen = torch.Generator().manual_seed(21)
    p = temporal_params(gen, "t.", D)
    layer = bnb.GriffinTemporalBlock(D)
    layer.load_state_dict(_strip(p, "t."))
    layer.to(DEV)
    x_seq = torch.randn(R, T, D, generator=gen)
    h0 = 0.5 * torch.randn(R, D, generator=gen)
    cb = torch.randn(R, 3, D, generator=gen)
    done = torch.zeros(R, T, dtype=torch.bool)
    done[:2, 3] = True
    wo = torch.randn(R, T, D, generator=gen)
    xd = x_seq.to(DEV).requires_grad_(True)
    out, h1, cb1 = layer.forward_sequence(xd, h0.to(DEV), cb.to(DEV), done.to(DEV))
    ((out * wo.to(DEV)).sum() + h1.sum() + cb1.sum()).backward()
    pr = {k: v.clone().double().requires_grad_(True) for k, v in p.items()}
    xr = x_seq.double().requires_grad_(True)
    ro, rh, rcb = torch_ref.temporal_sequence(pr, "t.", xr, h0.double(), cb.double(), done)
    ((ro * wo.double()).sum() + rh.sum() + rcb.sum()).backward()
    assert max_rel(xd.grad.cpu(), xr.grad) <= 5e-5
    for name, param in layer.named_parameters():
        assert max_rel(param.grad.cpu(), pr["t." + name].grad) <= 5e-5, name


def test_block_sequence_trains_and_matches_the_no_grad_path():
    cfg = _cfg(64, 4, spatial=1, temporal=1)
    torch.manual_seed(5)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, N, M, D = 6, 3, 4, 2, 64
    gen = torch.Generator().manual_seed(6)
    x = torch.randn(T, B, N + M, D, generator=gen).to(DEV)
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.8).to(DEV)
    alive[..., 0] = True
    h0 = torch.randn(1, B * N, D, generator=gen).to(DEV)
    cb0 = torch.randn(1, B * N, 3, D, generator=gen).to(DEV)
    done = (torch.rand(T, B, generator=gen) < 0.2).to(DEV)
    with torch.no_grad():
        want, want_h, want_cb = block.sequence(x, alive, h0, cb0, done, N)
    got, got_h, got_cb = block.sequence(x, alive, h0, cb0, done, N)
    assert max_rel(got.detach().cpu(), want.cpu()) <= 2e-5
    assert max_rel(got_h.detach().cpu(), want_h.cpu()) <= 2e-5 and max_rel(got_cb.detach().cpu(), want_cb.cpu()) <= 2e-5
    got.square().mean().backward()
    grads = [p.grad for p in block.parameters()]
    assert all(g is not None and torch.isfinite(g).all() for g in grads)
    assert block.temporal[0].rg_lru.log_lambda.grad.abs().max() > 0


@pytest.mark.parametrize("N,M", [(4, 2), (5, 0)])
def test_block_sequence_gradients_match_autograd_through_the_oracle_step_loop(N, M):
    """Gradients of every parameter, of x and of the initial state through ``YemongBlock.sequence`` (float32: norm,
    conv, gelu-gate, attention and recurrence backward kernels, ship/field split) against autograd in float64 through
    the oracle's one-step block applied T times with the state carried and cut at episode ends."""
    D, H, T, B, spatial, temporal = 128, 4, 7, 3, 2, 1
    gen = torch.Generator().manual_seed(41 + N)
    p = block_params(gen, "b.", D, spatial, temporal)
    block = bnb.YemongBlock(_cfg(D, H, 1, spatial, temporal))
    block.load_state_dict(_strip(p, "b."))
    block.to(DEV)
    x = torch.randn(T, B, N + M, D, generator=gen)
    alive = torch.rand(T, B, N + M, generator=gen) < 0.8
    alive[..., 0] = True
    h0 = 0.5 * torch.randn(temporal, B * N, D, generator=gen)
    cb0 = torch.randn(temporal, B * N, 3, D, generator=gen)
    done = torch.rand(T, B, generator=gen) < 0.3
    # the sequence form returns the last three conv inputs as they are (griffin.py:275-277), the step loop the buffer
    # it zeroed at an episode end: the two agree once three steps have followed the last end
    done[T - 3:] = False
    done[1, 0] = True
    up = torch.randn(T, B, N + M, D, generator=gen)

    xg, hg, cg = (t.to(DEV).requires_grad_() for t in (x, h0, cb0))
    out, h1, cb1 = block.sequence(xg, alive.to(DEV), hg, cg, done.to(DEV), N)
    ((out * up.to(DEV)).sum() + h1.square().sum() + cb1.sum()).backward()

    pd = {k: v.double().requires_grad_() for k, v in p.items()}
    xr, hr, cr = (t.double().requires_grad_() for t in (x, h0, cb0))
    h, cb, outs = hr, cr, []
    for t in range(T):
        if t > 0:  # a step that follows the end of an episode starts from the zero state (policy.py:268-285)
            keep = (~done[t - 1]).double().repeat_interleave(N)
            h, cb = h * keep[None, :, None], cb * keep[None, :, None, None]
        o, h, cb = torch_ref.block_step(pd, "b.", spatial, temporal, H, xr[t], alive[t], h, cb, N)
        outs.append(o)
    ref = torch.stack(outs)
    ((ref * up.double()).sum() + h.square().sum() + cb.sum()).backward()

    assert max_rel(out.detach().cpu(), ref.detach()) <= 2e-5
    assert max_rel(xg.grad.cpu(), xr.grad) <= 1e-4
    assert max_rel(hg.grad.cpu(), hr.grad) <= 1e-4 and max_rel(cg.grad.cpu(), cr.grad) <= 1e-4
    for name, param in block.named_parameters():
        want = pd["b." + name].grad
        if want is None:  # without field tokens their projection takes no part
            assert M == 0 and name.startswith("field_sub") and (param.grad is None or not param.grad.any()), name
            continue
        assert max_rel(param.grad.cpu(), want) <= 2e-4, name


@pytest.mark.parametrize("autocast", [False, True])
@pytest.mark.parametrize("D,H", [(128, 4), (64, 4)])
def test_team_pooling_layer_matches_oracle(autocast, D, H):
    # width 128 runs on the kernel, width 64 on the library attention call; both must state the same function
    B, N = 12, 19
    g = torch.Generator().manual_seed(D + autocast)
    p = team_pool_params(g, "tp.", D)
    layer = bnb.TeamPMA(D, H).to(DEV).eval()
    layer.load_state_dict(_strip(p, "tp."))
    x = torch.randn(B, N, D, generator=g)
    team, alive = team_case(3, B, N)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        got = layer(x.to(DEV), team.to(DEV), alive.to(DEV))
        pooled = layer.pooled(x.to(DEV), team.to(DEV), alive.to(DEV))
    ref, ref_pool = torch_ref.team_pool(p, "tp.", x, team, alive, H)
    assert got.shape == (B, N, D) and got.dtype == torch.float32
    tol = 2e-2 if (autocast and D != 128) else 1e-5  # the kernel computes in fp32 whatever autocast says
    assert max_rel(got.cpu(), ref) <= tol
    assert max_rel(pooled.cpu(), ref_pool) <= tol
    assert (got.cpu()[1] == 0).all()  # everybody dead in environment 1


@pytest.mark.parametrize("kernels", [True, False])
def test_team_pooling_layer_trains_and_matches_autograd_of_the_oracle(kernels):
    from boost_and_broadside_amd import trunk

    D, H, B, N = 128, 4, 37, 8
    g = torch.Generator().manual_seed(21)
    p = team_pool_params(g, "tp.", D)
    layer = bnb.TeamPMA(D, H).to(DEV)
    layer.load_state_dict(_strip(p, "tp."))
    x = torch.randn(B, N, D, generator=g).to(DEV).requires_grad_()
    # both teams present everywhere: with an empty team the oracle's softmax over no key is NaN
    # and so is autograd through it, which leaves nothing to compare with
    team = (torch.arange(N, dtype=torch.int32) % 2).repeat(B, 1)
    alive = torch.rand(B, N, generator=g) < 0.6
    alive[:, :2] = True
    up = torch.randn(B, N, D, generator=g)

    def run():
        out = layer(x, team.to(DEV), alive.to(DEV))
        (out * up.to(DEV)).sum().backward()
        return out

    if kernels:
        out = run()
    else:
        with trunk.library_update_path():
            out = run()
    assert torch.isfinite(x.grad).all() and all(torch.isfinite(q.grad).all() for q in layer.parameters())
    with torch.no_grad():
        assert max_rel(layer(x.detach(), team.to(DEV), alive.to(DEV)), out.detach()) <= 1e-5
    xr = x.detach().cpu().double().requires_grad_()
    pr = {k: v.double().requires_grad_() for k, v in p.items()}
    ref, _ = torch_ref.team_pool(pr, "tp.", xr, team, alive, H)
    (ref * up.double()).sum().backward()
    assert max_rel(x.grad.cpu(), xr.grad.float()) <= 1e-4
    for name, q in layer.named_parameters():
        assert max_rel(q.grad.cpu().double(), pr["tp." + name].grad) <= 1e-4, name


def test_team_pooling_gradients_with_empty_teams_are_finite_and_skip_them():
    D, H, B, N = 128, 4, 16, 8
    g = torch.Generator().manual_seed(23)
    p = team_pool_params(g, "tp.", D)
    layer = bnb.TeamPMA(D, H).to(DEV)
    layer.load_state_dict(_strip(p, "tp."))
    x = torch.randn(B, N, D, generator=g).to(DEV).requires_grad_()
    team = torch.randint(0, 2, (B, N), generator=g, dtype=torch.int32)
    alive = torch.rand(B, N, generator=g) < 0.5
    team[0] = 0            # team 1 absent
    alive[1] = False       # nobody alive
    layer(x, team.to(DEV), alive.to(DEV)).square().sum().backward()
    assert torch.isfinite(x.grad).all() and all(torch.isfinite(q.grad).all() for q in layer.parameters())
    assert not x.grad[1].any()  # no key, no gradient


def test_attention_block_outside_kernel_coverage_uses_the_library_on_the_device():
    # head size 24 is not one the kernels cover: the block must still compute the reference's function
    D, H, B, N = 96, 4, 3, 10
    g = torch.Generator().manual_seed(31)
    blk = bnb.TransformerBlock(_cfg(D=D, H=H)).to(DEV).eval()
    x = torch.randn(B, N, D, generator=g)
    alive = torch.rand(B, N, generator=g) < 0.7
    alive[0] = False
    with torch.no_grad():
        got = blk(x.to(DEV), alive.to(DEV)).cpu()
    sd = {"s." + k: v.detach().cpu() for k, v in blk.state_dict().items()}
    ref = torch_ref.spatial_sublayer(sd, "s.", x, alive, H)
    assert max_rel(got, ref) <= 1e-5
    from boost_and_broadside_amd import _native
    with pytest.raises(_native.NativeLibraryError) as err:
        bnb.ops.sdpa_masked(torch.zeros(1, 4, 3 * D, device=DEV), None, H)
    assert err.value.code == _native.ERR_UNSUPPORTED


def test_update_path_gradients_agree_between_the_kernels_and_the_library_ops(monkeypatch):
    """Under bf16 autocast with gradients on, the block runs its norms, gates, conv, attention and Linear
    weight gradients on the training kernels; every parameter gradient must agree with the same update
    computed through torch's own differentiable ops."""
    from boost_and_broadside_amd import ops, trunk

    cfg = _cfg(128, 4, spatial=1, temporal=1)
    torch.manual_seed(7)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, N, M, D = 16, 48, 8, 4, 128  # 9,216 token rows, 6,144 recurrent rows
    gen = torch.Generator().manual_seed(8)
    x = torch.randn(T, B, N + M, D, generator=gen).to(DEV)
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    h0 = torch.zeros(1, B * N, D, device=DEV)
    cb0 = torch.zeros(1, B * N, 3, D, device=DEV)
    done = (torch.rand(T, B, generator=gen) < 0.1).to(DEV)

    calls = []
    real = ops.linear_wgrad
    monkeypatch.setattr(ops, "linear_wgrad", lambda *a, **k: (calls.append(a[0].shape), real(*a, **k))[1])

    monkeypatch.setattr(trunk, "_WGRAD_MIN_ROWS", 4096)

    def grads():
        block.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, h, cb = block.sequence(x, alive, h0, cb0, done, N)
        (out.float().square().mean() + h.float().square().mean()).backward()
        return {n: p.grad.detach().clone() for n, p in block.named_parameters()}

    routed = grads()
    assert calls, "no Linear layer took the row-sliced weight gradient"
    n_calls = len(calls)
    with trunk.library_update_path():
        library = grads()
    assert len(calls) == n_calls
    for name, g in routed.items():
        assert torch.isfinite(g).all(), name
        assert max_rel(g.cpu(), library[name].cpu()) <= BF16_TOL, name


def test_update_path_kernels_compose_with_activation_checkpointing():
    """The reference can wrap each block's sequence pass in torch.utils.checkpoint (policy.py:452-466); the
    training kernels' autograd Functions must give the same gradients when recomputed that way."""
    from torch.utils.checkpoint import checkpoint

    cfg = _cfg(128, 4, spatial=1, temporal=1)
    torch.manual_seed(9)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, N, M, D = 12, 64, 8, 4, 128
    gen = torch.Generator().manual_seed(10)
    x = torch.randn(T, B, N + M, D, generator=gen).to(DEV).requires_grad_()
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    h0 = torch.zeros(1, B * N, D, device=DEV)
    cb0 = torch.zeros(1, B * N, 3, D, device=DEV)
    done = (torch.rand(T, B, generator=gen) < 0.1).to(DEV)

    def run(x_in):
        return block.sequence(x_in, alive, h0, cb0, done, N)[0]

    def grads(wrapped):
        block.zero_grad(set_to_none=True)
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = checkpoint(run, x, use_reentrant=False) if wrapped else run(x)
        out.float().square().mean().backward()
        return [x.grad.clone()] + [p.grad.clone() for p in block.parameters()]

    plain, recomputed = grads(False), grads(True)
    for a, b in zip(plain, recomputed):
        assert torch.equal(a, b)  # same kernels, same order: identical bits


def test_backward_called_inside_autocast_matches_backward_called_outside():
    """``loss.backward()`` inside the autocast block hands its autocast state to every custom backward; the
    kernels' backward code must not let a GEMM of its own turn bfloat16 there (a float32 pointer is what the
    kernels are given).  Same gradients as with backward called outside."""
    cfg = _cfg(128, 4, spatial=1, temporal=1)
    torch.manual_seed(11)
    block = bnb.YemongBlock(cfg).to(DEV)
    pma = bnb.TeamPMA(128, 4).to(DEV)
    with torch.no_grad():
        pma.seeds.normal_(0.0, 0.02)
    T, B, N, M, D = 8, 40, 8, 4, 128
    gen = torch.Generator().manual_seed(12)
    x = torch.randn(T, B, N + M, D, generator=gen).to(DEV).requires_grad_()
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    team = torch.randint(0, 2, (T * B, N), generator=gen, dtype=torch.int32).to(DEV)
    h0 = torch.zeros(1, B * N, D, device=DEV)
    cb0 = torch.zeros(1, B * N, 3, D, device=DEV)
    done = (torch.rand(T, B, generator=gen) < 0.1).to(DEV)
    params = list(block.parameters()) + list(pma.parameters())

    def grads(inside):
        for q in params:
            q.grad = None
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block.sequence(x, alive, h0, cb0, done, N)[0]
            pooled = pma(out[:, :, :N].reshape(T * B, N, D), team, alive[:, :, :N].reshape(T * B, N))
            loss = out.float().square().mean() + pooled.float().square().mean()
            if inside:
                loss.backward()
        if not inside:
            loss.backward()
        return [x.grad.clone()] + [q.grad.clone() for q in params]

    for a, b in zip(grads(False), grads(True)):
        # torch's own backward GEMMs (the small parameter einsums, F.linear) do change precision with the autocast
        # state, so the comparison is at the bf16 bar, not bitwise
        assert torch.isfinite(b).all()
        assert max_rel(b.float().cpu(), a.float().cpu()) <= BF16_TOL


@pytest.mark.parametrize("blocks,temporal", [(1, 1), (2, 1), (2, 2)])
def test_trunk_sequence_is_the_loop_over_blocks_and_trains_with_and_without_checkpointing(blocks, temporal):
    # the trunk part of policy.py:424-477: per block the slots [i*n_temporal, (i+1)*n_temporal) of the packed state
    D, H, B, N, M, T = 128, 4, 6, 8, 4, 10
    torch.manual_seed(31)
    trunk = bnb.YemongTrunk(_cfg(D, H, blocks, 1, temporal)).to(DEV)
    gen = torch.Generator().manual_seed(32)
    xs = torch.randn(T, B, N + M, D, generator=gen).to(DEV)
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    done = (torch.rand(T, B, generator=gen) < 0.15).to(DEV)
    hidden0 = 0.3 * torch.randn(blocks * temporal, B * N, 4 * D, generator=gen).to(DEV)

    with torch.no_grad():
        got = trunk.sequence(xs, alive, hidden0, done)
        x = xs
        h_all, cb_all = hidden0[:, :, :D], hidden0[:, :, D:].reshape(blocks * temporal, B * N, 3, D)
        for i, block in enumerate(trunk.yemong_layers):
            sl = slice(i * temporal, (i + 1) * temporal)
            x = block.sequence(x, alive, h_all[sl], cb_all[sl], done, N)[0]
        assert torch.equal(got, x)
        # and step by step with the state reset after an episode end
        hidden, outs = hidden0, []
        for t in range(T):
            out, hidden = trunk(xs[t], alive[t], hidden)
            hidden = trunk.reset_hidden_for_envs(hidden, done[t], N)
            outs.append(out)
        assert max_rel(got, torch.stack(outs)) <= 5e-5

    def grads(ckpt):
        trunk.zero_grad(set_to_none=True)
        xin = xs.clone().requires_grad_()
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = trunk.sequence(xin, alive, hidden0, done, grad_checkpoint=ckpt)
        out.float().square().mean().backward()
        return [xin.grad] + [q.grad.clone() for q in trunk.parameters()]

    plain, recomputed = grads(False), grads(True)
    assert all(torch.isfinite(g).all() for g in plain)
    for a, b in zip(plain, recomputed):
        assert torch.equal(a, b)
    with pytest.raises(ValueError):
        trunk.sequence(xs, alive, hidden0[:, :-1], done)


@pytest.mark.parametrize("p_live", [0.25, 0.0])
def test_update_path_with_the_bullet_read_agrees_with_the_library_ops(p_live):
    """Grad mode with bullets: only the bullets in flight are normalised and projected and the read runs on
    its kernels; every gradient (parameters, tokens, bullets) must agree with torch's own differentiable ops."""
    from boost_and_broadside_amd import trunk

    cfg = _cfg(128, 4, spatial=2, temporal=1, bullets=1)
    torch.manual_seed(13)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, N, M, D = 8, 80, 8, 4, 128
    NB = N * 10
    gen = torch.Generator().manual_seed(14)
    x = torch.randn(T, B, N + M, D, generator=gen).to(DEV).requires_grad_()
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    bullets = torch.randn(T * B, NB, D, generator=gen).to(DEV).requires_grad_()
    bmask = (torch.rand(T * B, NB, generator=gen) < p_live).to(DEV)
    if p_live > 0:
        bmask[3] = False
    h0 = torch.zeros(1, B * N, D, device=DEV)
    cb0 = torch.zeros(1, B * N, 3, D, device=DEV)
    done = (torch.rand(T, B, generator=gen) < 0.1).to(DEV)

    def grads():
        block.zero_grad(set_to_none=True)
        x.grad = bullets.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block.sequence(x, alive, h0, cb0, done, N, bullets, bmask)[0]
        out.float().square().mean().backward()
        named = {n: p.grad for n, p in block.named_parameters() if p.grad is not None}
        named["x"] = x.grad
        if bullets.grad is not None:
            named["bullets"] = bullets.grad
        return {k: v.detach().clone() for k, v in named.items()}

    fast = grads()
    with trunk.library_update_path():
        slow = grads()
    assert ("bullets" in fast) == (p_live > 0) or "bullets" in fast
    for name, g in slow.items():
        if name not in fast:
            assert not g.any(), name  # e.g. the bullet layers without any bullet in flight
            continue
        assert torch.isfinite(fast[name]).all(), name
        if g.abs().max() == 0:
            assert fast[name].abs().max() == 0, name
        else:
            assert max_rel(fast[name].float().cpu(), g.float().cpu()) <= BF16_TOL, name
    if p_live > 0:
        dead_rows = ~bmask.reshape(-1)
        assert not fast["bullets"].reshape(-1, D)[dead_rows].any()  # bullets that are not in flight receive nothing


def test_update_path_reads_more_than_one_tile_of_bullets_on_the_kernels():
    """32 ships = 320 bullet slots with most of them in flight: more live keys per environment than one tile
    of the attention backward holds.  The read and its backward stay on the kernels (no library dispatch is
    recorded) and every gradient agrees with torch's own differentiable ops."""
    from boost_and_broadside_amd import trunk

    cfg = _cfg(128, 4, spatial=2, temporal=1, bullets=1)
    torch.manual_seed(21)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, N, M, D = 3, 6, 32, 4, 128
    NB = N * 10
    gen = torch.Generator().manual_seed(22)
    x = torch.randn(T, B, N + M, D, generator=gen).to(DEV).requires_grad_()
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    bullets = torch.randn(T * B, NB, D, generator=gen).to(DEV).requires_grad_()
    bmask = (torch.rand(T * B, NB, generator=gen) < 0.7).to(DEV)
    bmask[2] = False
    bmask[4, 40:] = False  # one environment with few bullets among crowded ones
    assert int(bmask.sum(dim=1).max()) > 160
    h0 = torch.zeros(1, B * N, D, device=DEV)
    cb0 = torch.zeros(1, B * N, 3, D, device=DEV)
    done = torch.zeros(T, B, dtype=torch.bool, device=DEV)

    def grads():
        block.zero_grad(set_to_none=True)
        x.grad = bullets.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block.sequence(x, alive, h0, cb0, done, N, bullets, bmask)[0]
        out.float().square().mean().backward()
        named = {n: p.grad for n, p in block.named_parameters() if p.grad is not None}
        named["x"], named["bullets"] = x.grad, bullets.grad
        return {k: v.detach().clone() for k, v in named.items()}

    before = sum(trunk.library_dispatches.values())
    with trunk.forbid_library_dispatch():
        fast = grads()
    assert sum(trunk.library_dispatches.values()) == before
    with trunk.library_update_path():
        slow = grads()
    for name, g in slow.items():
        assert torch.isfinite(fast[name]).all(), name
        assert max_rel(fast[name].float().cpu(), g.float().cpu()) <= BF16_TOL, name
    assert not fast["bullets"].reshape(-1, D)[~bmask.reshape(-1)].any()


def test_trunk_sequence_with_bullets_shares_one_list_and_matches_the_block_loop():
    D, H, B, N, M, T = 128, 4, 10, 8, 4, 6
    torch.manual_seed(41)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1, bullets=1)).to(DEV)
    gen = torch.Generator().manual_seed(42)
    xs = torch.randn(T, B, N + M, D, generator=gen).to(DEV)
    alive = (torch.rand(T, B, N + M, generator=gen) < 0.85).to(DEV)
    alive[..., 0] = True
    bullets = torch.randn(T * B, N * 10, D, generator=gen).to(DEV)
    bmask = (torch.rand(T * B, N * 10, generator=gen) < 0.3).to(DEV)
    done = (torch.rand(T, B, generator=gen) < 0.15).to(DEV)
    hidden0 = torch.zeros(2, B * N, 4 * D, device=DEV)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        got = trunk.sequence(xs, alive, hidden0, done, bullets, bmask)
        x = xs
        for i, block in enumerate(trunk.yemong_layers):
            x = block.sequence(x, alive, hidden0[i:i + 1, :, :D], hidden0[i:i + 1, :, D:].reshape(1, B * N, 3, D), done, N,
                               bullets, bmask)[0]
    assert max_rel(got.float().cpu(), x.float().cpu()) <= BF16_TOL
    xin = xs.clone().requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = trunk.sequence(xin, alive, hidden0, done, bullets, bmask, grad_checkpoint=True)
    out.float().square().mean().backward()
    assert torch.isfinite(xin.grad).all() and all(q.grad is not None and torch.isfinite(q.grad).all() for q in trunk.parameters())


# ------------------------------------------------------------------ weights that change after the first forward


def _rollout_trunk(seed=51, D=128, H=4):
    p = trunk_params(seed, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    return trunk.to(DEV), p


@pytest.mark.parametrize("autocast", [False, True])
def test_weight_updates_after_the_first_forward_reach_the_cached_copies(autocast):
    # the averaged-opponent policy is overwritten through .data every update (train/rl/opponents.py:112);
    # the live policy by an optimizer step: after either, a no-grad forward must use the new weights
    D, H, B, N, M = 128, 4, 8, 8, 4
    trunk, _ = _rollout_trunk()
    gen = torch.Generator().manual_seed(52)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    hidden = torch.randn(2, B * N, 4 * D, generator=gen)

    def run_and_check(p_now):
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            out, new_hidden = trunk(x.to(DEV), alive.to(DEV), hidden.to(DEV))
        ref_out, ref_hidden = torch_ref.trunk_step(p_now, 2, 2, 1, H, x, alive, hidden)
        if autocast:
            assert max_rel(out.cpu(), ref_out) <= BF16_TOL and max_rel(new_hidden.cpu(), ref_hidden) <= BF16_TOL
        else:
            true_out, true_hidden = float64_truth(torch_ref.trunk_step, p_now, 2, 2, 1, H, x, alive, hidden)
            assert_float32_bar(out.cpu(), ref_out, true_out, "trunk after a weight update, output")
            assert_float32_bar(new_hidden.cpu(), ref_hidden, true_hidden, "trunk after a weight update, state")
        return out

    first = run_and_check({k: v.detach().cpu() for k, v in trunk.state_dict().items()})

    # 1. a write through .data exactly as the trainer's running average does it, and no call after it
    other = trunk_params(77, D, 2, 2, 1)
    cumsum = [2.0 * other[name].to(DEV) for name, _ in trunk.named_parameters()]
    for avg_parameter, cumulative in zip(trunk.parameters(), cumsum):
        avg_parameter.data.copy_(cumulative / 2)
    assert bnb.trunk.verify_weight_caches(trunk) == []  # every cache already knows it is out of date
    second = run_and_check(other)
    assert not torch.equal(first, second)
    assert bnb.trunk.verify_weight_caches(trunk) == []

    # 1b. a write the layers cannot see (through an alias taken earlier) is what verify_weight_caches reports
    #     and invalidate_weight_caches repairs
    aliases = [param.data for param in trunk.parameters()]
    run_and_check(other)  # the caches are rebuilt once more (the .data reads above) and are current again
    stale_free = trunk_params(79, D, 2, 2, 1)
    for (name, _), alias in zip(trunk.named_parameters(), aliases):
        alias.copy_(stale_free[name])
    assert bnb.trunk.verify_weight_caches(trunk) != []
    trunk.invalidate_weight_caches()
    run_and_check(stale_free)

    # 2. an optimizer step (in-place on the parameters: seen without any call)
    opt = torch.optim.SGD(trunk.parameters(), lr=0.05)
    for param in trunk.parameters():
        param.grad = torch.randn(param.shape, generator=gen).to(DEV)
    opt.step()
    third = run_and_check({k: v.detach().cpu() for k, v in trunk.state_dict().items()})
    assert not torch.equal(second, third)

    # 3. load_state_dict, also through a parent module that is not one of these layers
    holder = torch.nn.Module()
    holder.trunk = trunk
    holder.load_state_dict({"trunk." + k: v for k, v in trunk_params(78, D, 2, 2, 1).items()})
    run_and_check(trunk_params(78, D, 2, 2, 1))


@pytest.mark.parametrize("autocast_dtype", [None, torch.bfloat16])
def test_graphed_trunk_sees_new_weights_after_refresh(autocast_dtype):
    D, H, B, N, M = 128, 4, 16, 8, 4
    trunk, _ = _rollout_trunk(61)
    graphed = bnb.GraphedTrunk(trunk, B, N + M, N, autocast_dtype=autocast_dtype)
    gen = torch.Generator().manual_seed(62)
    alive = torch.ones(B, N + M, dtype=torch.bool, device=DEV)
    eager_state = trunk.initial_hidden(B, N, DEV)

    def both(t):
        nonlocal eager_state
        x = torch.randn(B, N + M, D, generator=gen).to(DEV)
        out, state = graphed.step(x, alive)
        out, state = out.clone(), state.clone()
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast_dtype is not None):
            ref_out, eager_state = trunk(x, alive, eager_state)
        assert torch.equal(out, ref_out) and torch.equal(state, eager_state), t

    both(0)
    # an optimizer-style in-place update and a write through .data, with no eager forward in between
    other = trunk_params(63, D, 2, 2, 1)
    for i, (name, param) in enumerate(trunk.named_parameters()):
        if i % 2:
            param.data.copy_(other[name])
        else:
            with torch.no_grad():
                param.copy_(other[name])
    both(1)  # no refresh_weights(), no invalidate call: the step follows the parameters by itself
    both(2)
    # the trainer's running average once more, between two replays
    for param in trunk.parameters():
        param.data.copy_(0.5 * param.detach() + 0.01)
    both(21)
    # and the explicit call still works
    with torch.no_grad():
        for param in trunk.parameters():
            param.mul_(1.01)
    graphed.refresh_weights()
    both(22)
    # the module dropping its caches must not take away memory the graphs read
    trunk.invalidate_weight_caches(drop=True)
    torch.cuda.empty_cache()
    scratch = [torch.randn(1 << 16, device=DEV) for _ in range(64)]  # reuses whatever was freed
    both(3)
    del scratch


def _bullet_trunk(seed, D=128, H=4):
    p = trunk_params(seed, D, 2, 2, 1)
    gen = torch.Generator().manual_seed(seed + 1000)
    for b in range(2):
        p[f"yemong_layers.{b}.spatial.0.norm_bullet.weight"] = 1.0 + 0.1 * torch.randn(D, generator=gen)
        p[f"yemong_layers.{b}.spatial.0.kv_bullet.weight"] = 0.1 * torch.randn(2 * D, D, generator=gen)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1, bullets=1)).eval()
    trunk.load_state_dict(p)
    return trunk.to(DEV), p


@pytest.mark.parametrize("graph", [True, False])
@pytest.mark.parametrize("autocast_dtype", [None, torch.bfloat16])
def test_steppers_over_a_bullet_reading_trunk_take_the_bullets_and_match_the_plain_forward(graph, autocast_dtype):
    # the shipped default reads bullets (config/defaults.py:29): a stepper that dropped them would step another policy
    D, H, B, N, M, K = 128, 4, 16, 8, 4, 10
    trunk, p = _bullet_trunk(91)
    with pytest.raises(ValueError, match="num_bullet_slots"):
        bnb.trunk_stepper(trunk, B, N + M, N, autocast_dtype=autocast_dtype, graph=graph)
    stepper = bnb.trunk_stepper(trunk, B, N + M, N, autocast_dtype=autocast_dtype, graph=graph, num_bullet_slots=N * K)
    gen = torch.Generator().manual_seed(92)
    eager_state = trunk.initial_hidden(B, N, DEV)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    with pytest.raises(ValueError, match="bullets"):
        stepper.step(torch.zeros(B, N + M, D, device=DEV), alive.to(DEV))
    for t in range(5):
        x = torch.randn(B, N + M, D, generator=gen).to(DEV)
        alive[:, :N] &= torch.rand(B, N, generator=gen) > 0.1
        bullets = torch.randn(B, N * K, D, generator=gen).to(DEV)
        bmask = torch.rand(B, N * K, generator=gen) < (0.0 if t == 1 else 0.3)  # one step with nothing in flight
        bmask[3] = False
        done = torch.rand(B, generator=gen) < 0.2 if t == 2 else None
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast_dtype is not None):
            ref_out, eager_state = trunk(x, alive.to(DEV), eager_state, bullets, bmask.to(DEV),
                                         reset_mask=None if done is None else done.to(DEV))
            no_read, _ = trunk(x, alive.to(DEV), stepper.state.clone(), reset_mask=None if done is None else done.to(DEV))
        torch.cuda.synchronize()
        out, state = stepper.step(x, alive.to(DEV), None if done is None else done.to(DEV), bullets, bmask.to(DEV))
        assert torch.equal(out, ref_out), t
        assert torch.equal(state, eager_state), t
        if t != 1:
            assert not torch.equal(out, no_read), t  # the read does change the result
    # and against the oracle on the last step's inputs
    hidden0 = torch.randn(2, B * N, 4 * D, generator=gen)
    stepper.load_state(hidden0.to(DEV))
    out, state = stepper.step(x, alive.to(DEV), None, bullets, bmask.to(DEV))
    ref_out, ref_hidden = torch_ref.trunk_step(p, 2, 2, 1, H, x.cpu(), alive, hidden0, bullets=bullets.cpu(), bullet_mask=bmask)
    if autocast_dtype is not None:
        assert max_rel(out.float().cpu(), ref_out) <= BF16_TOL and max_rel(state.cpu(), ref_hidden) <= BF16_TOL
    else:
        true_out, true_hidden = float64_truth(torch_ref.trunk_step, p, 2, 2, 1, H, x.cpu(), alive, hidden0, bullets=bullets.cpu(),
                                              bullet_mask=bmask)
        assert_float32_bar(out.cpu(), ref_out, true_out, "stepper with bullets, output")
        assert_float32_bar(state.cpu(), ref_hidden, true_hidden, "stepper with bullets, state")
    # a stepper without bullets over a trunk that reads none keeps its old signature
    plain_trunk, _ = _rollout_trunk(93)
    with pytest.raises(ValueError, match="no bullet-reading"):
        bnb.trunk_stepper(plain_trunk, B, N + M, N, graph=False, num_bullet_slots=80)


def test_block_step_and_single_step_sequence_work_in_grad_mode_and_match_autograd_through_the_oracle():
    # griffin.py:376-417 is differentiable in the reference; a T = 1 sequence in grad mode must not take
    # the inference kernels
    D, H, B, N, M = 64, 4, 3, 4, 2
    gen = torch.Generator().manual_seed(71)
    p = block_params(gen, "b.", D, 1, 1)
    block = bnb.YemongBlock(_cfg(D, H, 1, 1, 1))
    block.load_state_dict(_strip(p, "b."))
    block.to(DEV)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.rand(B, N + M, generator=gen) < 0.8
    alive[:, N:] = True
    h = 0.5 * torch.randn(1, B * N, D, generator=gen)
    cb = torch.randn(1, B * N, 3, D, generator=gen)
    wo = torch.randn(B, N + M, D, generator=gen)
    xd = x.to(DEV).requires_grad_(True)
    out, h1, cb1 = block.step(xd, alive.to(DEV), h.to(DEV), cb.to(DEV), N)
    assert out.requires_grad
    ((out * wo.to(DEV)).sum() + h1.sum() + 0.5 * cb1.sum()).backward()
    pr = {k: v.clone().double().requires_grad_(True) for k, v in p.items()}
    xr = x.double().requires_grad_(True)
    ro, rh, rcb = torch_ref.block_step(pr, "b.", 1, 1, H, xr, alive, h.double(), cb.double(), N)
    ((ro * wo.double()).sum() + rh.sum() + 0.5 * rcb.sum()).backward()
    assert max_rel(out.detach().cpu(), ro.detach()) <= 5e-5
    assert max_rel(xd.grad.cpu(), xr.grad) <= 2e-4
    for name, param in block.named_parameters():
        assert param.grad is not None, name
        assert max_rel(param.grad.cpu(), pr["b." + name].grad) <= 2e-4, name
    # the temporal layer alone, T = 1
    layer = block.temporal[0]
    xs = torch.randn(5, 1, D, generator=gen).to(DEV).requires_grad_(True)
    o, _, _ = layer.forward_sequence(xs, torch.zeros(5, D, device=DEV), torch.zeros(5, 3, D, device=DEV))
    o.sum().backward()
    assert xs.grad is not None and torch.isfinite(xs.grad).all()


def test_out_state_overlapping_the_input_state_at_an_offset_is_refused():
    D, H, B, N, M = 128, 4, 4, 8, 4
    trunk, _ = _rollout_trunk(81)
    x = torch.randn(B, N + M, D, device=DEV)
    alive = torch.ones(B, N + M, dtype=torch.bool, device=DEV)
    rows = B * N
    big = torch.zeros(2 * 2 * rows + 2 * rows, 4 * D, device=DEV)
    state = big[: 2 * rows].view(2, rows, 4 * D)
    shifted = big[rows: 3 * rows].view(2, rows, 4 * D)  # same storage, one layer's worth of rows further on
    with pytest.raises(ValueError, match="shares no memory"):
        trunk(x, alive, state, out_state=shifted)
    apart = big[2 * rows: 4 * rows].view(2, rows, 4 * D)
    _, new_state = trunk(x, alive, state, out_state=apart)  # adjacent but disjoint: fine
    assert new_state.data_ptr() == apart.data_ptr()


def test_a_policy_around_the_trunk_runs_under_torch_compile():
    """The reference wraps its policies in torch.compile (train/rl/ppo.py:396-400, policy_io.py:354-358).  The
    kernels are reached through ctypes, which the tracer cannot follow: it must break the graph there, run the
    trunk as it is and give the eager result, for the rollout step and for the update (gradients included).
    The encoder ends in Linear -> RMSNorm as the reference's does (encoder.py:82-101), so under autocast the trunk
    is handed bfloat16 tokens."""
    import torch._dynamo

    from boost_and_broadside_amd import trunk as trunk_module

    cfg = _cfg(128, 4, blocks=2, spatial=2, temporal=1)
    torch.manual_seed(21)
    trunk = bnb.YemongTrunk(cfg).to(DEV)

    class Policy(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.enc = torch.nn.Sequential(torch.nn.Linear(20, 128), torch.nn.RMSNorm(128))
            self.trunk = trunk
            self.head = torch.nn.Linear(128, 6)

        def forward(self, obs, alive, state):  # rollout step
            hidden, new_state = self.trunk(self.enc(obs), alive, state)
            return self.head(hidden), new_state

    class Evaluate(torch.nn.Module):  # the update's re-evaluation of a stored rollout
        def __init__(self, policy):
            super().__init__()
            self.policy = policy

        def forward(self, obs_seq, alive_seq, state, done):
            return self.policy.head(self.policy.trunk.sequence(self.policy.enc(obs_seq), alive_seq, state, done))

    policy = Policy().to(DEV)
    B, N, M, T = 24, 8, 4, 6
    g = torch.Generator().manual_seed(22)
    obs = torch.randn(T, B, N + M, 20, generator=g).to(DEV)
    alive = (torch.rand(T, B, N + M, generator=g) < 0.8).to(DEV)
    alive[..., N:] = True
    done = (torch.rand(T, B, generator=g) < 0.1).to(DEV)
    state = trunk.initial_hidden(B, N, DEV)
    torch._dynamo.reset()
    compiled = torch.compile(policy, backend="aot_eager")
    evaluate = Evaluate(policy)
    compiled_evaluate = torch.compile(evaluate, backend="aot_eager")
    try:
        with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16), trunk_module.forbid_library_dispatch():
            want = policy(obs[0], alive[0], state)
            got = compiled(obs[0], alive[0], state)
            again = compiled(obs[0], alive[0], state)
        for a, b, c in zip(want, got, again):
            assert torch.equal(a, b) and torch.equal(a, c)

        def grads(fn):
            policy.zero_grad(set_to_none=True)
            with torch.autocast("cuda", dtype=torch.bfloat16):
                logits = fn(obs, alive, state, done)
            logits.float().square().mean().backward()
            return [q.grad.clone() for q in policy.parameters()]

        for a, b in zip(grads(evaluate), grads(compiled_evaluate)):
            assert torch.isfinite(b).all() and max_rel(b.float().cpu(), a.float().cpu()) <= BF16_TOL
    finally:
        torch._dynamo.reset()


@pytest.mark.parametrize("bullets", [0, 1])
def test_bfloat16_tokens_under_autocast_run_on_the_kernels_and_match_the_oracle(bullets):
    """Linear -> RMSNorm at the end of the reference's encoder (encoder.py:82-101) emits bfloat16 under bf16 autocast,
    so that is what the trunk is handed there.  The tokens are widened on entry, every sublayer runs on the kernels
    (no library dispatch) and the result comes back in bfloat16, within the bf16 bar of the oracle's float32 evaluation
    of the same (already rounded) tokens."""
    from boost_and_broadside_amd import trunk as trunk_module

    D, H, B, N, M = 128, 4, 12, 8, 4
    p = trunk_params(33, D, 2, 2, 1)
    if bullets:
        pg = torch.Generator().manual_seed(35)
        for i in range(2):
            p[f"yemong_layers.{i}.spatial.0.norm_bullet.weight"] = 1.0 + 0.1 * torch.randn(D, generator=pg)
            p[f"yemong_layers.{i}.spatial.0.kv_bullet.weight"] = 0.15 * torch.randn(2 * D, D, generator=pg)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1, bullets=bullets)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    gen = torch.Generator().manual_seed(34)
    hidden, ref_hidden = trunk.initial_hidden(B, N, DEV), torch.zeros(2, B * N, 4 * D)
    alive = torch.ones(B, N + M, dtype=torch.bool)
    for t in range(3):
        x = torch.randn(B, N + M, D, generator=gen).bfloat16()
        alive[:, :N] &= torch.rand(B, N, generator=gen) > 0.1
        kw, ref_kw = {}, {}
        if bullets:
            bul = torch.randn(B, 10 * N, D, generator=gen)
            bm = torch.rand(B, 10 * N, generator=gen) < 0.3
            kw = {"bullets": bul.to(DEV), "bullet_mask": bm.to(DEV)}
            ref_kw = {"bullets": bul, "bullet_mask": bm}
        with torch.autocast("cuda", dtype=torch.bfloat16), trunk_module.forbid_library_dispatch():
            out, hidden = trunk(x.to(DEV), alive.to(DEV), hidden, **kw)
        assert out.dtype == torch.bfloat16 and hidden.dtype == torch.float32
        ref_out, ref_hidden = torch_ref.trunk_step(p, 2, 2, 1, H, x.float(), alive, ref_hidden, **ref_kw)
        assert max_rel(out.float().cpu(), ref_out) <= BF16_TOL, t
        assert max_rel(hidden.cpu(), ref_hidden) <= BF16_TOL, t
    # the update's re-evaluation takes the same tokens, differentiably
    xs = torch.randn(4, B, N + M, D, generator=gen).bfloat16().to(DEV).requires_grad_()
    al = torch.ones(4, B, N + M, dtype=torch.bool, device=DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        seq = trunk.sequence(xs, al, trunk.initial_hidden(B, N, DEV))
    assert seq.dtype == torch.bfloat16
    seq.float().square().mean().backward()
    assert xs.grad.dtype == torch.bfloat16 and torch.isfinite(xs.grad).all() and xs.grad.abs().max() > 0


def test_team_pooling_takes_a_bfloat16_stream_under_autocast_on_the_kernels():
    from boost_and_broadside_amd import trunk as trunk_module

    D, H, B, N = 128, 4, 40, 8
    torch.manual_seed(41)
    layer = bnb.TeamPMA(D, H).to(DEV)
    with torch.no_grad():
        layer.seeds.normal_(0.0, 0.02)
    g = torch.Generator().manual_seed(42)
    x = torch.randn(B, N, D, generator=g).bfloat16().to(DEV)
    team = torch.randint(0, 2, (B, N), generator=g, dtype=torch.int32).to(DEV)
    alive = (torch.rand(B, N, generator=g) < 0.8).to(DEV)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        with trunk_module.forbid_library_dispatch():
            got = layer(x, team, alive)
            pooled = layer.pooled(x, team, alive)
        want = layer(x.float(), team, alive)
    assert got.dtype == torch.bfloat16 and pooled.dtype == torch.bfloat16
    assert torch.equal(got, want.to(torch.bfloat16))
    xg = x.clone().requires_grad_()
    with torch.autocast("cuda", dtype=torch.bfloat16), trunk_module.forbid_library_dispatch():
        layer(xg, team, alive).float().square().mean().backward()
    assert xg.grad.dtype == torch.bfloat16 and torch.isfinite(xg.grad).all()


@pytest.mark.parametrize("blocks,spatial,temporal,M,bullets", [
    (2, 2, 1, 4, 0), (2, 2, 1, 0, 0), (2, 2, 1, 4, 1), (2, 1, 2, 4, 0), (1, 0, 2, 0, 0), (3, 1, 0, 4, 0), (2, 0, 1, 4, 0),
])
def test_sublayer_tails_hand_the_next_sublayer_its_projection(monkeypatch, blocks, spatial, temporal, M, bullets):
    """Under bf16 autocast the tail kernel of every sublayer but the last also forms the norm + projection the next
    sublayer starts with (within a block and across blocks): one stand-alone norm + projection launch is left, the
    first sublayer's.  Same result as with every sublayer forming its own, within the bf16 bar, and as the oracle."""
    from boost_and_broadside_amd import trunk as trunk_module

    D, H, B, N = 128, 4, 11, 8
    p = trunk_params(50 + blocks + 3 * spatial + 7 * temporal, D, blocks, spatial, temporal)
    pg = torch.Generator().manual_seed(51)
    for i in range(blocks):
        for j in range(temporal):  # field tokens' stand-in for the recurrence away from the identity it starts as
            p[f"yemong_layers.{i}.field_sub.{j}.weight"] = torch.eye(D) + 0.05 * torch.randn(D, D, generator=pg)
        if bullets:
            p[f"yemong_layers.{i}.spatial.0.norm_bullet.weight"] = 1.0 + 0.1 * torch.randn(D, generator=pg)
            p[f"yemong_layers.{i}.spatial.0.kv_bullet.weight"] = 0.15 * torch.randn(2 * D, D, generator=pg)
    trunk = bnb.YemongTrunk(_cfg(D, H, blocks, spatial, temporal, bullets=bullets)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    calls = []
    ops = trunk_module.ops
    real = ops.norm_linear
    monkeypatch.setattr(ops, "norm_linear", lambda x, *a, **k: (calls.append(k.get("rows") is None), real(x, *a, **k))[1])
    gen = torch.Generator().manual_seed(52)
    L = blocks * temporal
    state_a = state_b = torch.randn(L, B * N, 4 * D, generator=gen).to(DEV)
    ref_state = state_a.cpu()
    alive = torch.ones(B, N + M, dtype=torch.bool)
    for t in range(3):
        x = torch.randn(B, N + M, D, generator=gen)
        alive[:, :N] &= torch.rand(B, N, generator=gen) > 0.1
        reset = torch.rand(B, generator=gen) < 0.2
        kw, ref_kw = {}, {}
        if bullets:
            bul = torch.randn(B, 10 * N, D, generator=gen)
            bm = torch.rand(B, 10 * N, generator=gen) < 0.3
            kw = {"bullets": bul.to(DEV), "bullet_mask": bm.to(DEV)}
            ref_kw = {"bullets": bul, "bullet_mask": bm}
        with torch.autocast("cuda", dtype=torch.bfloat16), trunk_module.forbid_library_dispatch():
            calls.clear()
            out_a, state_a = trunk(x.to(DEV), alive.to(DEV), state_a, reset_mask=reset.to(DEV), **kw)
            handed_over = sum(calls)  # launches over all rows of the residual stream (the bullets' own do not count)
            with trunk_module.separate_heads():
                calls.clear()
                out_b, state_b = trunk(x.to(DEV), alive.to(DEV), state_b, reset_mask=reset.to(DEV), **kw)
                on_their_own = sum(calls)
        assert handed_over == 1 and on_their_own == blocks * (spatial + temporal)
        assert max_rel(out_a.cpu(), out_b.cpu()) <= BF16_TOL, t
        if L:
            assert max_rel(state_a.cpu(), state_b.cpu()) <= BF16_TOL, t
        ref_out, ref_state = torch_ref.trunk_step(p, blocks, spatial, temporal, H, x, alive,
                                                  torch_ref.reset_hidden(ref_state, reset, N), **ref_kw)
        assert max_rel(out_a.cpu(), ref_out) <= BF16_TOL, t
        if L:
            assert max_rel(state_a.cpu(), ref_state) <= BF16_TOL, t


def test_graphed_trunk_with_handed_over_projections_replays_like_the_eager_step():
    from boost_and_broadside_amd import trunk as trunk_module

    D, H, B, N, M = 128, 4, 24, 8, 4
    p = trunk_params(61, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    graphed = bnb.GraphedTrunk(trunk, B, N + M, N, autocast_dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(62)
    state = trunk.initial_hidden(B, N, DEV)
    alive = torch.ones(B, N + M, dtype=torch.bool, device=DEV)
    for t in range(4):
        x = torch.randn(B, N + M, D, generator=gen).to(DEV)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            eager, state = trunk(x, alive, state)
            with trunk_module.separate_heads():
                apart, _ = trunk(x, alive, graphed.state.clone())
        torch.cuda.synchronize()
        if t % 2:  # a producer that fills the capture's input buffers in place hands over the buffers themselves
            graphed.tokens.copy_(x)
            graphed.alive.copy_(alive)
            out, new_state = graphed.step(graphed.tokens, graphed.alive)
        else:
            out, new_state = graphed.step(x, alive)
        assert torch.equal(out, eager) and torch.equal(new_state, state), t
        assert max_rel(out.cpu(), apart.cpu()) <= BF16_TOL


@pytest.mark.parametrize("bullets", [0, 1])
def test_update_path_at_the_rollouts_size_agrees_with_the_library_ops(bullets):
    """One block forward + backward at the size of a stored 4v4 rollout (128 steps x 256 environments x 12 tokens:
    393,216 token rows, every update kernel several rounds of resident work-groups deep): every parameter gradient and
    the input gradient agree with the same update through torch's own differentiable ops, twice in a row bit for bit."""
    from boost_and_broadside_amd import trunk

    cfg = _cfg(128, 4, spatial=2, temporal=1, bullets=bullets)
    torch.manual_seed(70 + bullets)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, N, M, D = 128, 256, 8, 4, 128
    gen = torch.Generator(device=DEV).manual_seed(71)
    x = torch.randn(T, B, N + M, D, device=DEV, generator=gen).requires_grad_()
    alive = torch.rand(T, B, N + M, device=DEV, generator=gen) < 0.9
    alive[..., 0] = True
    h0 = torch.zeros(1, B * N, D, device=DEV)
    cb0 = torch.zeros(1, B * N, 3, D, device=DEV)
    done = torch.rand(T, B, device=DEV, generator=gen) < 0.02
    go = torch.randn(T, B, N + M, D, device=DEV, generator=gen)
    kw = {}
    if bullets:
        kw = {"bullets": torch.randn(T * B, N * 10, D, device=DEV, generator=gen),
              "bullet_mask": torch.rand(T * B, N * 10, device=DEV, generator=gen) < 0.25}

    def grads():
        block.zero_grad(set_to_none=True)
        x.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out = block.sequence(x, alive, h0, cb0, done, N, **kw)[0]
        out.backward(go)
        found = {n: p.grad.detach().clone() for n, p in block.named_parameters() if p.grad is not None}
        found["tokens"] = x.grad.detach().clone()
        return found

    with trunk.forbid_library_dispatch():
        routed = grads()
        again = grads()
    with trunk.library_update_path():
        library = grads()
    assert set(routed) == set(library)
    for name, g in routed.items():
        assert torch.isfinite(g).all(), name
        assert torch.equal(g, again[name]), name  # fixed-order reductions everywhere
        assert max_rel(g, library[name]) <= BF16_TOL, name


@pytest.mark.parametrize("N,M,with_done", [(8, 4, True), (8, 4, False), (3, 9, True)])
def test_temporal_mix_in_place_of_split_and_concatenation_gives_the_same_bits(N, M, with_done, monkeypatch):
    """The update's temporal sublayer reads the ship rows of the token tensor where they lie and writes its states (and
    their gradients) back into token tensors; with that switched off the same kernels run on split copies and the
    results are concatenated.  Same arithmetic either way: outputs, states and every gradient must be identical."""
    from boost_and_broadside_amd import ops

    cfg = _cfg(128, 4, spatial=1, temporal=1)
    torch.manual_seed(90 + N)
    block = bnb.YemongBlock(cfg).to(DEV)
    T, B, D = 32, 96, 128
    gen = torch.Generator(device=DEV).manual_seed(91)
    x = torch.randn(T, B, N + M, D, device=DEV, generator=gen).requires_grad_()
    alive = torch.rand(T, B, N + M, device=DEV, generator=gen) < 0.9
    alive[..., 0] = True
    h0 = torch.randn(1, B * N, D, device=DEV, generator=gen).requires_grad_()
    cb0 = torch.randn(1, B * N, 3, D, device=DEV, generator=gen).requires_grad_()
    done = (torch.rand(T, B, device=DEV, generator=gen) < 0.05) if with_done else None
    go = torch.randn(T, B, N + M, D, device=DEV, generator=gen)
    gh = torch.randn(1, B * N, D, device=DEV, generator=gen)
    gc = torch.randn(1, B * N, 3, D, device=DEV, generator=gen)

    used = []
    real = ops.temporal_mix_train
    monkeypatch.setattr(ops, "temporal_mix_train", lambda *a, **k: (used.append(1), real(*a, **k))[1])

    def run():
        block.zero_grad(set_to_none=True)
        for t in (x, h0, cb0):
            t.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, h, cb = block.sequence(x, alive, h0, cb0, done, N)
        torch.autograd.backward([out, h, cb], [go, gh, gc])
        found = {n: p.grad.detach().clone() for n, p in block.named_parameters() if p.grad is not None}
        found.update(tokens=x.grad.clone(), h0=h0.grad.clone(), cb0=cb0.grad.clone(), out=out.detach().clone(),
                     h=h.detach().clone(), cb=cb.detach().clone())
        return found

    in_place = run()
    assert used, "the token-tensor form did not run"
    n_used = len(used)
    monkeypatch.setattr(ops, "temporal_mix_train_supported", lambda *a, **k: False)
    apart = run()
    assert len(used) == n_used
    assert set(in_place) == set(apart)
    for name, g in in_place.items():
        assert torch.equal(g, apart[name]), name


@pytest.mark.parametrize("T,B,n,NM,D", [(5, 2048, 8, 12, 128), (3, 4100, 5, 6, 128), (6, 1100, 3, 4, 256), (7, 33, 2, 9, 64)])
def test_kernels_over_token_tensors_equal_the_dense_calls_on_the_wide_lane_forms_too(T, B, n, NM, D):
    """Enough rows for the eight-channels-per-lane kernels (and a few shapes of the one-lane-per-channel ones): the four
    sequence kernels over the ship rows of a token tensor give the bits of the same calls on sliced copies."""
    from boost_and_broadside_amd import ops

    gen = torch.Generator(device=DEV).manual_seed(T * B + n)
    R = B * n
    b1 = torch.randn(T, B, NM, D, device=DEV, generator=gen).bfloat16()
    buf = torch.randn(R, 3, D, device=DEV, generator=gen)
    w = 0.5 * torch.randn(D, 1, 4, device=DEV, generator=gen)
    bias = 0.1 * torch.randn(D, device=DEV, generator=gen)
    done = torch.rand(R, T, device=DEV, generator=gen) < 0.2
    ships = b1[:, :, :n].reshape(T, R, D).contiguous()
    want = ops.conv_seq(ships, buf, w, bias, done, time_major=True, also_bf16=True)
    got = ops.conv_seq(b1, buf, w, bias, done, time_major=True, also_bf16=True, token_rows=n)
    assert all(torch.equal(a, b) for a, b in zip(got, want))
    gates = torch.randn(T, R, 2 * D, device=DEV, generator=gen).bfloat16()
    lam = torch.linspace(0, 4, D, device=DEV)
    h0 = torch.randn(R, D, device=DEV, generator=gen)
    y_want, h_want = ops.rglru_scan(want[0], gates, lam, 8.0, h0, done, time_major=True)
    tokens = torch.full((T, B, NM, D), -3.0, device=DEV)
    _, h_got = ops.rglru_scan(want[0], gates, lam, 8.0, h0, done, time_major=True, y_tokens=(tokens, n))
    assert torch.equal(h_got, h_want) and torch.equal(tokens[:, :, :n].reshape(T, R, D), y_want)
    assert bool((tokens[:, :, n:] == -3.0).all())
    dy_tok = torch.randn(T, B, NM, D, device=DEV, generator=gen)
    dh = torch.randn(R, D, device=DEV, generator=gen)
    a = ops.rglru_scan_bwd(want[0], gates, lam, 8.0, h0, done, tokens, dy_tok, dh, time_major=True, token_rows=n)
    b = ops.rglru_scan_bwd(want[0], gates, lam, 8.0, h0, done, y_want, dy_tok[:, :, :n].reshape(T, R, D).contiguous(), dh,
                           time_major=True)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    dv = torch.randn(T, R, D, device=DEV, generator=gen)
    dv_lp = torch.randn(T, R, D, device=DEV, generator=gen).bfloat16()
    db1_tok = torch.full((T, B, NM, D), 3.0, device=DEV).bfloat16()
    c = ops.conv_seq_bwd(b1, buf, w, done, dv, None, time_major=True, dv_bf16=dv_lp, token_rows=n, db1_out=db1_tok)
    d = ops.conv_seq_bwd(ships, buf, w, done, dv, None, time_major=True, dv_bf16=dv_lp)
    assert torch.equal(db1_tok[:, :, :n].reshape(T, R, D), d[0]) and bool((db1_tok[:, :, n:] == 3.0).all())
    assert all(torch.equal(p, q) for p, q in zip(c[1:], d[1:]))


def test_kernels_over_token_tensors_touch_only_their_rows_and_refuse_other_layouts():
    from boost_and_broadside_amd import ops

    T, B, n, NM, D = 9, 5, 3, 7, 128
    gen = torch.Generator(device=DEV).manual_seed(5)
    b1 = torch.randn(T, B, NM, D, device=DEV, generator=gen).bfloat16()
    buf = torch.randn(B * n, 3, D, device=DEV, generator=gen)
    w = 0.5 * torch.randn(D, 1, 4, device=DEV, generator=gen)
    bias = 0.1 * torch.randn(D, device=DEV, generator=gen)
    done = torch.rand(B * n, T, device=DEV, generator=gen) < 0.2
    ships = b1[:, :, :n].reshape(T, B * n, D).contiguous()
    want = ops.conv_seq(ships, buf, w, bias, done, time_major=True, also_bf16=True)
    got = ops.conv_seq(b1, buf, w, bias, done, time_major=True, also_bf16=True, token_rows=n)
    assert all(torch.equal(a, b) for a, b in zip(got, want))
    # the recurrence writes its states into the first n tokens and leaves the others as they were
    gates = torch.randn(T, B * n, 2 * D, device=DEV, generator=gen).bfloat16()
    lam = torch.linspace(0, 4, D, device=DEV)
    h0 = torch.randn(B * n, D, device=DEV, generator=gen)
    y_want, h_want = ops.rglru_scan(want[0], gates, lam, 8.0, h0, done, time_major=True)
    tokens = torch.full((T, B, NM, D), 7.0, device=DEV)
    y_got, h_got = ops.rglru_scan(want[0], gates, lam, 8.0, h0, done, time_major=True, y_tokens=(tokens, n))
    assert y_got is tokens and torch.equal(h_got, h_want)
    assert torch.equal(tokens[:, :, :n].reshape(T, B * n, D), y_want) and bool((tokens[:, :, n:] == 7.0).all())
    # backward kernels: gradients of the ship rows from / into token tensors, the other rows untouched
    dy_tok = torch.randn(T, B, NM, D, device=DEV, generator=gen)
    dh = torch.randn(B * n, D, device=DEV, generator=gen)
    a = ops.rglru_scan_bwd(want[0], gates, lam, 8.0, h0, done, tokens, dy_tok, dh, time_major=True, token_rows=n)
    b = ops.rglru_scan_bwd(want[0], gates, lam, 8.0, h0, done, y_want, dy_tok[:, :, :n].reshape(T, B * n, D).contiguous(), dh,
                           time_major=True)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    dv = torch.randn(T, B * n, D, device=DEV, generator=gen)
    db1_tok = torch.full((T, B, NM, D), 3.0, device=DEV).bfloat16()
    c = ops.conv_seq_bwd(b1, buf, w, done, dv, None, time_major=True, token_rows=n, db1_out=db1_tok)
    d = ops.conv_seq_bwd(ships, buf, w, done, dv, None, time_major=True)
    assert c[0] is db1_tok and torch.equal(db1_tok[:, :, :n].reshape(T, B * n, D), d[0]) and bool((db1_tok[:, :, n:] == 3.0).all())
    assert all(torch.equal(p, q) for p, q in zip(c[1:], d[1:]))
    with pytest.raises(ValueError):
        ops.conv_seq(b1, buf, w, bias, done, token_rows=n)  # batch-major
    with pytest.raises(ValueError):
        ops.conv_seq(b1, buf, w, bias, done, time_major=True, token_rows=NM + 1)
    with pytest.raises(ValueError):
        ops.conv_seq(b1.transpose(1, 2), buf, w, bias, done, time_major=True, token_rows=n)
    # the C entry points refuse a placement that is not time-major, a pitch below the group, rows that are no multiple of it
    from boost_and_broadside_amd import _native

    lib = _native.load()
    v = torch.empty(T, B * n, D, device=DEV)
    nb = torch.empty(B * n, 3, D, device=DEV)
    w4 = w.reshape(D, 4).contiguous()

    def conv(time_major, group, pitch, rows=B * n):
        return lib.bnb_conv_seq_fwd(b1.data_ptr(), _native.BF16, buf.data_ptr(), 3 * D, w4.data_ptr(), bias.data_ptr(), None,
                                    v.data_ptr(), None, nb.data_ptr(), 3 * D, rows, T, D, time_major, group, pitch, None)

    assert conv(1, n, NM) == 0
    for bad in ((0, n, NM), (1, n, n - 1), (1, 0, NM), (1, 2, NM)):  # B * n = 15 rows are no multiple of 2
        assert conv(*bad) == 10003, bad


def test_trunk_stepper_picks_the_captured_step_for_small_batches_and_both_kinds_agree():
    D, H, N, M = 128, 4, 8, 4
    p = trunk_params(81, D, 2, 2, 1)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    small = bnb.trunk_stepper(trunk, 16, N + M, N, autocast_dtype=torch.bfloat16)
    assert isinstance(small, bnb.GraphedTrunk)
    assert isinstance(bnb.trunk_stepper(trunk, 4096, N + M, N, autocast_dtype=torch.bfloat16), bnb.EagerTrunkStepper)
    assert isinstance(bnb.trunk_stepper(trunk, 1024, N + M, N), bnb.EagerTrunkStepper)  # 12,288 tokens in float32
    plain = bnb.trunk_stepper(trunk, 16, N + M, N, autocast_dtype=torch.bfloat16, graph=False)
    assert isinstance(plain, bnb.EagerTrunkStepper)
    gen = torch.Generator().manual_seed(82)
    alive = torch.ones(16, N + M, dtype=torch.bool, device=DEV)
    for t in range(4):
        x = torch.randn(16, N + M, D, generator=gen).to(DEV)
        done = (torch.rand(16, generator=gen) < 0.3).to(DEV) if t == 2 else None
        out_a, state_a = small.step(x, alive, done)
        out_b, state_b = plain.step(x, alive, done)
        assert torch.equal(out_a, out_b) and torch.equal(state_a, state_b), t
        assert torch.equal(plain.state, state_b)
    plain.load_state(torch.zeros_like(plain.state))
    assert plain.state.abs().max() == 0


def test_bullet_reading_layers_share_one_projection_pass_over_the_live_bullets(monkeypatch):
    """Two blocks, each with one bullet-reading sublayer: the live bullets are gathered, normalised and projected once
    per step (the layers' norm weights folded into their projections), and the result stays within the bf16 bar of the
    oracle and of the step in which every layer projects for itself."""
    from boost_and_broadside_amd import trunk as trunk_module

    D, H, B, N, M = 128, 4, 9, 8, 4
    p = trunk_params(91, D, 2, 2, 1)
    pg = torch.Generator().manual_seed(92)
    for i in range(2):
        p[f"yemong_layers.{i}.spatial.0.norm_bullet.weight"] = 1.0 + 0.3 * torch.randn(D, generator=pg)
        p[f"yemong_layers.{i}.spatial.0.kv_bullet.weight"] = 0.15 * torch.randn(2 * D, D, generator=pg)
    trunk = bnb.YemongTrunk(_cfg(D, H, 2, 2, 1, bullets=1)).eval()
    trunk.load_state_dict(p)
    trunk.to(DEV)
    ops = trunk_module.ops
    calls = []
    real = ops.norm_linear
    monkeypatch.setattr(ops, "norm_linear", lambda x, *a, **k: (calls.append(k.get("rows") is not None), real(x, *a, **k))[1])
    gen = torch.Generator().manual_seed(93)
    x = torch.randn(B, N + M, D, generator=gen)
    alive = torch.rand(B, N + M, generator=gen) < 0.9
    alive[:, 0] = True
    bul = torch.randn(B, 10 * N, D, generator=gen)
    bm = torch.rand(B, 10 * N, generator=gen) < 0.3
    bm[2] = False  # an environment with nothing in flight
    hidden = trunk.initial_hidden(B, N, DEV)
    shared = bnb.YemongTrunk._bullet_kv_of_all_layers
    with torch.autocast("cuda", dtype=torch.bfloat16), trunk_module.forbid_library_dispatch():
        out, state = trunk(x.to(DEV), alive.to(DEV), hidden, bul.to(DEV), bm.to(DEV))
        assert sum(calls) == 1  # one pass over the bullets in flight for both readers
        calls.clear()
        monkeypatch.setattr(bnb.YemongTrunk, "_bullet_kv_of_all_layers", lambda self, bullets, rows: None)
        apart, state_b = trunk(x.to(DEV), alive.to(DEV), hidden, bul.to(DEV), bm.to(DEV))
        assert sum(calls) == 2
    ref_out, ref_state = torch_ref.trunk_step(p, 2, 2, 1, H, x, alive, torch.zeros(2, B * N, 4 * D), bullets=bul, bullet_mask=bm)
    assert max_rel(out.cpu(), ref_out) <= BF16_TOL and max_rel(state.cpu(), ref_state) <= BF16_TOL
    assert max_rel(out.cpu(), apart.cpu()) <= BF16_TOL and max_rel(state.cpu(), state_b.cpu()) <= BF16_TOL

    # an optimizer-style update of one reader's bullet weights: the folded matrix is rebuilt for the next step
    monkeypatch.setattr(bnb.YemongTrunk, "_bullet_kv_of_all_layers", shared)
    with torch.no_grad():
        trunk.yemong_layers[1].spatial[0].norm_bullet.weight.mul_(-0.5)
        trunk.yemong_layers[0].spatial[0].kv_bullet.weight.add_(0.05)
    p2 = {k: v.detach().cpu().clone() for k, v in trunk.state_dict().items()}
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out2, state2 = trunk(x.to(DEV), alive.to(DEV), hidden, bul.to(DEV), bm.to(DEV))
    ref2, ref_state2 = torch_ref.trunk_step(p2, 2, 2, 1, H, x, alive, torch.zeros(2, B * N, 4 * D), bullets=bul, bullet_mask=bm)
    assert max_rel(out2.cpu(), ref2) <= BF16_TOL and max_rel(state2.cpu(), ref_state2) <= BF16_TOL
    assert max_rel(ref2, ref_out) > 10 * BF16_TOL  # the update did change the result
