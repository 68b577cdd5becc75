"""CPU-side checks: the C ABI library loads and exports what the header declares, the host
wrappers validate their arguments, the layer classes keep the reference's state_dict names,
and the workload generators / traffic model give the documented figures.  No kernel runs."""

import os
import re

import pytest
import torch

from helpers import ROOT, trunk_params

import boost_and_broadside_amd as bnb
from boost_and_broadside_amd import _native, harness, ops


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "bnb_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bnb_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _native.load()
    names = _declared_functions()
    assert {"bnb_sdpa_masked_fwd", "bnb_rglru_step_fwd", "bnb_abi_version"} <= set(names)
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(_native.SIGNATURES) == names  # the ctypes table covers the header exactly


def test_library_identity_and_error_names():
    lib = _native.load()
    assert lib.bnb_abi_version() == _native.ABI_VERSION  # the header's value is checked below
    assert lib.bnb_build_arch() == b"gfx950"
    assert lib.bnb_error_string(0) == b"success"
    assert b"NULL" in lib.bnb_error_string(10001)
    assert b"alignment" in lib.bnb_error_string(10005)


def test_header_constants_match_loader():
    text = open(os.path.join(ROOT, "include", "bnb_amd.h")).read()
    consts = dict(re.findall(r"#define\s+(BNB_[A-Z0-9_]+)\s+(\d+)", text))
    assert int(consts["BNB_ABI_VERSION"]) == _native.ABI_VERSION
    assert int(consts["BNB_ERR_UNSUPPORTED"]) == _native.ERR_UNSUPPORTED
    assert (int(consts["BNB_F32"]), int(consts["BNB_BF16"])) == (_native.F32, _native.BF16)
    assert [int(consts[f"BNB_SDPA_PATH_{n}"]) for n in ("AUTO", "VALU", "MFMA")] == [0, 1, 2]
    assert [int(consts[f"BNB_WGRAD_PATH_{n}"]) for n in ("AUTO", "STAGED", "DMA")] == [
        _native.WGRAD_PATH_AUTO, _native.WGRAD_PATH_STAGED, _native.WGRAD_PATH_DMA]


def test_ops_refuse_host_tensors_and_bad_arguments():
    with pytest.raises(RuntimeError, match="no host fallback"):
        ops.sdpa_masked(torch.zeros(1, 2, 48), None, 4)
    with pytest.raises(ValueError):
        ops.sdpa_masked(torch.zeros(1, 2, 50), None, 4)  # not 3*D
    with pytest.raises(RuntimeError, match="no host fallback"):
        ops.rglru_step(torch.zeros(2, 8), torch.zeros(2, 16), torch.zeros(8), 8.0, torch.zeros(2, 8))
    with pytest.raises(ValueError):
        ops.rglru_step(torch.zeros(2, 8), torch.zeros(2, 8), torch.zeros(8), 8.0, torch.zeros(2, 8))


def test_model_config_validation_matches_reference_rules():
    # config/core.py:262-275 and tests/models/test_encoder.py:571-589
    cfg = bnb.ModelConfig(d_model=64, n_heads=4, n_yemong_blocks=2)
    assert (cfg.n_spatial_per_block, cfg.n_temporal_per_block, cfg.n_hidden_layers) == (1, 1, 2)
    for kwargs in ({"n_yemong_blocks": -1}, {"n_spatial_per_block": -1}, {"n_temporal_per_block": -1}):
        kw = {"n_yemong_blocks": 2, **kwargs}
        with pytest.raises(ValueError):
            bnb.ModelConfig(d_model=64, n_heads=4, **kw)
    with pytest.raises(ValueError):
        bnb.ModelConfig(d_model=66, n_heads=4, n_yemong_blocks=1)
    with pytest.raises(ValueError):
        bnb.ModelConfig(d_model=64, n_heads=4, n_yemong_blocks=1, n_spatial_per_block=1, n_bullet_cross_per_block=2)


@pytest.mark.parametrize("n_blocks,n_spatial,n_temporal", [(2, 1, 1), (2, 2, 1), (1, 4, 2), (2, 2, 0)])
def test_state_dict_keys_are_the_reference_names(n_blocks, n_spatial, n_temporal):
    cfg = bnb.ModelConfig(d_model=32, n_heads=4, n_yemong_blocks=n_blocks, n_spatial_per_block=n_spatial,
                          n_temporal_per_block=n_temporal)
    trunk = bnb.YemongTrunk(cfg)
    want = trunk_params(0, 32, n_blocks, n_spatial, n_temporal)
    have = trunk.state_dict()
    assert sorted(have) == sorted(want)
    for k in want:
        assert tuple(have[k].shape) == tuple(want[k].shape), k
    trunk.load_state_dict(want, strict=True)
    for block in trunk.yemong_layers:
        assert len(block.spatial) == n_spatial and len(block.temporal) == n_temporal


def test_bullet_reading_layers_carry_the_extra_reference_parameters():
    cfg = bnb.ModelConfig(d_model=32, n_heads=4, n_yemong_blocks=1, n_spatial_per_block=2, n_bullet_cross_per_block=1)
    keys = set(bnb.YemongBlock(cfg).state_dict())
    assert {"spatial.0.norm_bullet.weight", "spatial.0.kv_bullet.weight"} <= keys
    assert "spatial.1.kv_bullet.weight" not in keys


def test_fresh_layers_follow_reference_initialisation():
    cfg = bnb.ModelConfig(d_model=32, n_heads=4, n_yemong_blocks=1)
    block = bnb.YemongBlock(cfg)
    assert torch.equal(block.field_sub[0].weight, torch.eye(32))  # griffin.py:365-368
    assert torch.allclose(block.temporal[0].rg_lru.log_lambda, torch.linspace(0, 4, 32))  # griffin.py:165
    assert block.temporal[0].conv.weight.shape == (32, 1, 4) and block.temporal[0].rg_lru.c == 8.0


def test_hidden_state_shape_and_reset_are_env_major():
    # tests/models/test_encoder.py:272-303, :384-405
    cfg = bnb.ModelConfig(d_model=16, n_heads=4, n_yemong_blocks=2, n_temporal_per_block=2)
    trunk = bnb.YemongTrunk(cfg)
    B, N = 3, 4
    hidden = trunk.initial_hidden(B, N, torch.device("cpu"))
    assert hidden.shape == (4, B * N, 4 * 16) and hidden.dtype == torch.float32 and not hidden.any()
    hidden = torch.randn_like(hidden)
    done = torch.tensor([False, True, False])
    out = trunk.reset_hidden_for_envs(hidden, done, N)
    assert (out[:, N:2 * N] == 0).all()
    assert torch.equal(out[:, :N], hidden[:, :N]) and torch.equal(out[:, 2 * N:], hidden[:, 2 * N:])


def test_workloads_and_traffic_model():
    w = harness.WORKLOADS
    assert [x.tokens_per_step for x in w.values()] == [12288, 98304, 94208, 344064, 655360]
    got = {k: harness.algorithmic_bytes(v)["step"] for k, v in w.items()}
    assert got == {
        "c0_4v4_fp32": 1024 * (24588 + 20480),
        "c1_4v4_rollout_bf16": 8192 * (12300 + 16384),
        "c2_8v11_bf16": 4096 * (23575 + 38912),
        "c3_32v48_bf16": 4096 * (86100 + 163840),
        "c4_64v88_bf16": 4096 * (164000 + 311296),
    }
    assert harness.attention_flops(w["c4_64v88_bf16"]) == 4096 * 4 * 160 * 160 * 128


def test_alive_generators():
    w = harness.WORKLOADS
    a0 = harness.make_alive(w["c0_4v4_fp32"])
    assert a0.shape == (1, 1024, 12) and a0[..., 8:].all()
    assert 0.8 < a0[..., :8].float().mean() < 0.9
    a1 = harness.make_alive(w["c1_4v4_rollout_bf16"], steps=16, B=512)
    assert a1[0].all()
    assert (a1[1:] <= a1[:-1]).all()  # monotone dying
    assert a1[-1].float().mean() < 1.0
    a4 = harness.make_alive(w["c4_64v88_bf16"], steps=2, B=2048)
    live = a4[0].sum(-1)
    assert live.min() >= 16 and live.max() <= 160 and a4[0, :, 152:].all() and torch.equal(a4[0], a4[1])
    assert torch.equal(harness.make_alive(w["c2_8v11_bf16"]), harness.make_alive(w["c2_8v11_bf16"]))  # seeded


def test_inputs_are_seeded_and_typed():
    w = harness.WORKLOADS["c1_4v4_rollout_bf16"]
    t1, s1 = harness.make_inputs(w, B=8)
    t2, s2 = harness.make_inputs(w, B=8)
    assert torch.equal(t1, t2) and torch.equal(s1, s2)
    assert t1.dtype == torch.bfloat16 and s1.dtype == torch.float32 and s1.shape == (64, 128)
    p = harness.make_weights(w.seed, w.dtype)
    assert p["qkv.weight"].shape == (384, 128) and p["log_lambda"].dtype == torch.float32


@pytest.mark.parametrize("use", ["both", "first", "rest"])
def test_token_split_has_the_gradient_of_plain_slicing(use):
    """The ship/field split of the update path (one concatenation in its backward) against autograd's own slicing."""
    from boost_and_broadside_amd.trunk import _SplitTokens

    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 2, 5, 4, generator=g, dtype=torch.float64)
    wa, wb = torch.randn(3, 2, 3, 4, generator=g, dtype=torch.float64), torch.randn(3, 2, 2, 4, generator=g, dtype=torch.float64)

    def loss(first, rest):
        total = x.new_zeros(())
        if use in ("both", "first"):
            total = total + (first * wa).sum()
        if use in ("both", "rest"):
            total = total + (rest.square() * wb).sum()
        return total

    xs = x.clone().requires_grad_()
    first, rest = _SplitTokens.apply(xs, 3)
    assert first.is_contiguous() and rest.is_contiguous()
    assert torch.equal(first, x[:, :, :3]) and torch.equal(rest, x[:, :, 3:])
    loss(first, rest).backward()
    xr = x.clone().requires_grad_()
    loss(xr[:, :, :3], xr[:, :, 3:]).backward()
    assert torch.equal(xs.grad, xr.grad)


def test_backward_weight_pack_follows_the_documented_operand_order():
    # include/bnb_amd.h, bnb_ffn_bwd: sampled entries of the five sections against the index formulas written out
    from boost_and_broadside_amd import ops

    g = torch.Generator().manual_seed(3)
    wg, wu, wd = torch.randn(512, 128, generator=g), torch.randn(512, 128, generator=g), torch.randn(128, 512, generator=g)
    pk = ops.pack_ffn_bwd_weights(wg, wu, wd).view(16, 5, 4096).float()

    def pi(m):
        return 16 * (m // 16) + 8 * ((m // 4) % 2) + 4 * ((m // 8) % 2) + m % 4

    assert sorted(pi(m) for m in range(32)) == list(range(32))
    rnd = torch.randint(0, 1 << 30, (200, 5), generator=g).tolist()
    for a, b_, c_, d, e_ in rnd:
        c, ks, l, e = a % 16, b_ % 8, c_ % 64, d % 8
        m, b = l % 32, l // 32
        at = (ks * 64 + l) * 8 + e
        assert pk[c, 0, at] == wg.bfloat16().float()[32 * c + pi(m), 16 * ks + 8 * b + e]
        assert pk[c, 1, at] == wu.bfloat16().float()[32 * c + pi(m), 16 * ks + 8 * b + e]
        assert pk[c, 2, at] == wd.bfloat16().float()[16 * ks + 8 * b + e, 32 * c + pi(m)]
        cb, t = ks // 2, ks % 2
        at = ((cb * 2 + t) * 64 + l) * 8 + e
        assert pk[c, 3, at] == wg.bfloat16().float()[32 * c + 16 * t + 8 * b + e, 32 * cb + pi(m)]
        assert pk[c, 4, at] == wu.bfloat16().float()[32 * c + 16 * t + 8 * b + e, 32 * cb + pi(m)]


def test_layer_parameters_notice_writes_through_data_and_stay_ordinary_parameters():
    # train/rl/opponents.py:107-112 overwrites the averaged policy with avg_parameter.data.copy_(...), which
    # leaves the version counter alone: the layers' parameters count .data accesses instead
    import copy
    import io

    from boost_and_broadside_amd import trunk as trunk_module

    cfg = bnb.ModelConfig(d_model=32, n_heads=4, n_yemong_blocks=2, n_spatial_per_block=2, n_bullet_cross_per_block=1)
    trunk = bnb.YemongTrunk(cfg)
    params = dict(trunk.named_parameters())
    assert params and all(type(p) is trunk_module.WatchedParameter for p in params.values())
    assert all(isinstance(p, torch.nn.Parameter) and p.is_leaf and p.requires_grad for p in params.values())
    w = params["yemong_layers.0.spatial.0.qkv.weight"]
    key = trunk_module._cache_key((w,), torch.bfloat16)
    w.data.copy_(torch.ones_like(w))
    assert w._version == 0 and float(w.detach()[0, 0]) == 1.0
    assert trunk_module._cache_key((w,), torch.bfloat16) != key  # the write is seen although the version is not
    key = trunk_module._cache_key((w,), torch.bfloat16)
    with torch.no_grad():
        w.mul_(2.0)
    assert trunk_module._cache_key((w,), torch.bfloat16) != key
    # state_dict, deepcopy, pickling, casts and assign-loading keep the names, the values and the watching
    assert sorted(trunk.state_dict()) == sorted(params)
    for other in (copy.deepcopy(trunk), torch.load(_pickled(trunk), weights_only=False), copy.deepcopy(trunk).double()):
        assert all(type(p) is trunk_module.WatchedParameter for p in other.parameters())
        assert all(torch.equal(a.float(), b) for a, b in zip(other.parameters(), trunk.parameters()))
    fresh = bnb.YemongTrunk(cfg)
    fresh.load_state_dict({k: v.clone() for k, v in trunk.state_dict().items()}, assign=True)
    assert all(type(p) is trunk_module.WatchedParameter for p in fresh.parameters())
    assert float(fresh.yemong_layers[0].spatial[0].qkv.weight.detach()[0, 0]) == 2.0
    # gradients and optimizers see ordinary leaves
    lin = trunk.yemong_layers[0].spatial[0].out_proj
    lin(torch.ones(2, 32)).sum().backward()
    assert lin.weight.grad is not None and type(lin.weight.grad) is torch.Tensor
    torch.optim.SGD(trunk.parameters(), lr=0.1).step()


def _pickled(module):
    import io

    buf = io.BytesIO()
    torch.save(module, buf)
    buf.seek(0)
    return buf


def test_steppers_refuse_to_drop_the_bullets_of_a_bullet_reading_trunk():
    from boost_and_broadside_amd import trunk as trunk_module

    cfg = bnb.ModelConfig(d_model=32, n_heads=4, n_yemong_blocks=1, n_spatial_per_block=1, n_bullet_cross_per_block=1)
    trunk = bnb.YemongTrunk(cfg)
    with pytest.raises(ValueError, match="num_bullet_slots"):
        trunk_module._bullet_buffers(trunk, 4, None, "cpu", torch.float32)
    assert trunk_module._bullet_buffers(trunk, 4, 0, "cpu", torch.float32) == (None, None)
    bullets, mask = trunk_module._bullet_buffers(trunk, 4, 80, "cpu", torch.float32)
    assert bullets.shape == (4, 80, 32) and mask.shape == (4, 80) and mask.dtype == torch.bool and not mask.any()
    plain = bnb.YemongTrunk(bnb.ModelConfig(d_model=32, n_heads=4, n_yemong_blocks=1))
    with pytest.raises(ValueError, match="no bullet-reading"):
        trunk_module._bullet_buffers(plain, 4, 80, "cpu", torch.float32)
    assert trunk_module._bullet_buffers(plain, 4, None, "cpu", torch.float32) == (None, None)
