"""Benchmark of the attention + RG-LRU step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One "step" is one pass of the two kernels over one batch of synthetic input that is already
resident in HBM: masked attention over every environment's packed q/k/v rows, then the
RG-LRU update of every ship row with the recurrent state carried from step to step.  The
projections around the kernels (4 GEMMs) are torch library calls and are reported
separately (``module``), as are the same two regions run through eager PyTorch on the GPU
(``torch_gpu_baseline``) and on the host cores (``cpu_baseline``).  Rank 0 prints one JSON
line.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch
import torch.nn.functional as F

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "entity-tokens/sec through attention+RG-LRU step; % of HBM roofline"
POOL = 4  # distinct input batches cycled through the timed steps


def parse_args():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None, help="timed steps (default: the workload's rollout length, at least 32)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--repeats", type=int, default=9, help="the K-step loop is run this many times after the warm-up; the median loop is reported")
    ap.add_argument("--workload", default=None, help="one of the harness workloads (default: the 64v88 headline)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU-baseline leg; 0 skips it")
    ap.add_argument("--no-graph", action="store_true", help="time the step loop as eager launches only (no HIP graph replay)")
    ap.add_argument("--no-torch-baseline", action="store_true")
    ap.add_argument("--no-module", action="store_true")
    ap.add_argument("--no-issue-probe", action="store_true", help="skip the matrix-core / vector-ALU issue-rate yardstick")
    ap.add_argument("--no-ffn", action="store_true", help="skip the fused sublayer-tail leg")
    ap.add_argument("--no-bullets", action="store_true", help="skip the bullet-read leg")
    ap.add_argument("--no-sequence", action="store_true", help="skip the update-path (T = 128) recurrence leg")
    ap.add_argument("--no-team-pool", action="store_true", help="skip the team pooling leg")
    ap.add_argument("--no-fp32-attention", action="store_true", help="skip the float32 attention leg")
    ap.add_argument("--no-trunk", action="store_true", help="skip the whole-trunk leg (2 blocks x (2 spatial + 1 temporal))")
    ap.add_argument("--only-update-step", action="store_true",
                    help="run nothing but the update-path block step (forward + backward from a given gradient, T = 128 x 256 "
                         "environments of 4v4) a few times and print its time: the command a kernel trace of one step is taken from")
    return ap.parse_args()


# ---------------------------------------------------------------------------------------------
# reference-style eager PyTorch statements of the two regions (the GPU baseline being beaten);
# written out here so that the benchmark's GPU legs do not touch the CPU checker
# ---------------------------------------------------------------------------------------------


def torch_attention_region(qkv, alive, n_heads):
    B, NM, D3 = qkv.shape
    D = D3 // 3
    dh = D // n_heads
    q, k, v = qkv.chunk(3, dim=-1)
    q = q.view(B, NM, n_heads, dh).permute(0, 2, 1, 3)
    k = k.view(B, NM, n_heads, dh).permute(0, 2, 1, 3)
    v = v.view(B, NM, n_heads, dh).permute(0, 2, 1, 3)
    keep = alive.view(B, 1, 1, NM).to(q.dtype)
    bias = (1.0 - keep) * (torch.finfo(q.dtype).min / 2)
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=bias, dropout_p=0.0)
    return out.permute(0, 2, 1, 3).reshape(B, NM, D)


def torch_rglru_region(x, gates, log_lambda, c, h):
    D = x.shape[-1]
    r = torch.sigmoid(gates[:, :D])
    i = torch.sigmoid(gates[:, D:])
    a = torch.sigmoid(log_lambda) ** (c * r)
    gate = torch.sqrt(torch.clamp((1.0 - a) * (1.0 + a), min=1e-6))
    return a * h + gate * (i * x)


def torch_scan_region(x, gates, log_lambda, c, h0, done):
    """The reference's sequence recurrence in torch ops (griffin.py:206-219 and the log-depth
    scan :25-64): coefficients, reset of a after an episode end, shifted combines."""
    D = x.shape[-1]
    r = torch.sigmoid(gates[..., :D])
    i = torch.sigmoid(gates[..., D:])
    a = torch.sigmoid(log_lambda) ** (c * r)
    b = torch.sqrt(torch.clamp((1.0 - a) * (1.0 + a), min=1e-6)) * (i * x)
    fresh = done.roll(1, dims=1)
    fresh[:, 0] = False
    a = a.masked_fill(fresh.unsqueeze(-1), 0.0)
    T = a.shape[1]
    width = 1 << (T - 1).bit_length()
    if width > T:
        a = torch.nn.functional.pad(a, (0, 0, 0, width - T), value=1.0)
        b = torch.nn.functional.pad(b, (0, 0, 0, width - T), value=0.0)
    span = 1
    while span < width:
        a_prev = torch.nn.functional.pad(a[:, : width - span], (0, 0, span, 0), value=1.0)
        b_prev = torch.nn.functional.pad(b[:, : width - span], (0, 0, span, 0), value=0.0)
        b = a * b_prev + b
        a = a * a_prev
        span *= 2
    out = (a * h0.unsqueeze(1) + b)[:, :T]
    return out, out[:, -1]


def torch_conv_region(b1, conv_buf, weight, bias):
    padded = torch.cat([conv_buf, b1.unsqueeze(1)], dim=1)
    w = weight.reshape(-1, 4)
    out = torch.zeros_like(padded[:, :1])
    for k in range(4):
        out = out + padded[:, k:k + 1] * w[:, k]
    return (out + bias)[:, 0], padded[:, 1:]


class eager_kernels:
    """Context manager: the trunk layers run the reference-style eager PyTorch regions above
    instead of the HIP kernels (same modules, same weights) - the GPU baseline of the trunk leg."""

    def __enter__(self):
        from boost_and_broadside_amd import ops

        self.ops = ops
        self.saved = (ops.sdpa_masked, ops.rglru_step, ops.conv_step, ops.add_rmsnorm, ops.gelu_mul, ops.ffn_supported,
                      ops.FFN_WIDTH)

        def sdpa(qkv, alive, n_heads, **kw):
            if alive is None:
                alive = torch.ones(qkv.shape[:2], dtype=torch.bool, device=qkv.device)
            return torch_attention_region(qkv, alive, n_heads)

        def rglru(x, gates, lam, c, h, **kw):
            out = torch_rglru_region(x, gates, lam, c, h)
            return out, out

        def conv(b1, conv_buf, weight, bias, also_bf16=False, **kw):
            v, buf = torch_conv_region(b1, conv_buf, weight, bias)
            return (v, buf, v.to(torch.bfloat16)) if also_bf16 else (v, buf)

        def add_rmsnorm(x, weight, delta=None, eps=None, out_dtype=torch.float32):
            s = x if delta is None else x + delta
            return s, F.rms_norm(s, (s.shape[-1],), weight, eps).to(out_dtype)

        def gelu_mul(a, b, out_dtype=None):
            out = F.gelu(a) * b
            return out if out_dtype is None else out.to(out_dtype)

        ops.sdpa_masked, ops.rglru_step, ops.conv_step, ops.add_rmsnorm, ops.gelu_mul = sdpa, rglru, conv, add_rmsnorm, gelu_mul
        # the matrix-core kernels (sublayer tail, norm + projection) fall back to their library compositions
        ops.ffn_supported = lambda x, hidden: False
        ops.FFN_WIDTH = -1
        return self

    def __exit__(self, *exc):
        o = self.ops
        o.sdpa_masked, o.rglru_step, o.conv_step, o.add_rmsnorm, o.gelu_mul, o.ffn_supported, o.FFN_WIDTH = self.saved
        return False


def reference_style_trunk_step(trunk, x, alive, hidden, n_rec):
    """The block loop as the reference writes it: unpack views, per-block step, cat and re-pack
    (models/yemong/policy.py:316-354)."""
    L, rows, width = hidden.shape
    D = width // 4
    n_t = trunk.config.n_temporal_per_block
    h_all, cb_all = hidden[:, :, :D], hidden[:, :, D:].reshape(L, rows, 3, D)
    hs, cbs = [], []
    for i, block in enumerate(trunk.yemong_layers):
        sl = slice(i * n_t, (i + 1) * n_t)
        x, h_i, cb_i = block.step(x, alive, h_all[sl], cb_all[sl], n_rec)
        hs.append(h_i)
        cbs.append(cb_i)
    return x, torch.cat([torch.cat(hs, 0), torch.cat(cbs, 0).reshape(L, rows, 3 * D)], dim=-1)


# ---------------------------------------------------------------------------------------------


def timed_loop(fn, steps, warmup):
    """Run fn(t) for warmup + steps iterations; wall-clock seconds of the timed part."""
    for t in range(warmup):
        fn(t)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for t in range(steps):
        fn(warmup + t)
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def median_loop(fn, steps, warmup, repeats):
    """``warmup`` untimed iterations, then ``repeats`` loops of exactly ``steps`` iterations, each bracketed by a
    device synchronisation on both sides: (median loop seconds, all loop seconds in run order).  The step index keeps
    counting through the loops, so carried state and the input rotation go on as in one long rollout."""
    for t in range(warmup):
        fn(t)
    walls = []
    t = warmup
    for _ in range(max(1, repeats)):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn(t)
            t += 1
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
    return sorted(walls)[len(walls) // 2], walls


def event_split(launch_a, launch_b, steps, warmup, repeats=1):
    """Device time of the two launches, from events on the stream they run on: (mean a, mean b, median a, median b)
    of the round of ``steps`` steps whose a + b is the median of ``repeats`` such rounds (the first round after a pause
    of the device reads up to 15 % high on the issue-bound kernel: the device clock is still on its way up)."""
    for t in range(warmup):
        launch_a(t)
        launch_b(t)
    rounds = []
    t0 = warmup
    for _ in range(max(1, repeats)):
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
        torch.cuda.synchronize()
        for t in range(steps):
            ev[t][0].record()
            launch_a(t0 + t)
            ev[t][1].record()
            launch_b(t0 + t)
            ev[t][2].record()
        torch.cuda.synchronize()
        t0 += steps
        a = sorted(e[0].elapsed_time(e[1]) * 1e-3 for e in ev)
        b = sorted(e[1].elapsed_time(e[2]) * 1e-3 for e in ev)
        rounds.append((sum(a) / steps, sum(b) / steps, a[steps // 2], b[steps // 2]))
    rounds.sort(key=lambda r: r[0] + r[1])
    return rounds[len(rounds) // 2]


def cpu_baseline(w, p, budget_s):
    """The CPU checker (torch restatement of the reference ops) timed on the host cores.

    Same two regions as the GPU figure (attention incl. bias and head merge; RG-LRU
    element-wise chain), float32, on a slice of the workload's environments sized so the
    leg stays within ``budget_s`` seconds.
    """
    from oracle import torch_ref

    from boost_and_broadside_amd import harness

    threads = torch.get_num_threads()
    B = min(w.B, 256)
    p32 = {k: v.float() for k, v in p.items()}
    tokens, state = harness.make_inputs(w, B=B)
    alive = harness.make_alive(w, steps=1, B=B)[0]
    tokens = tokens.float()
    qkv = F.linear(tokens, p32["qkv.weight"])
    u = F.linear(torch_ref.sdpa_masked(qkv, alive, harness.N_HEADS), p32["out_proj.weight"])
    ships = u[:, : w.N].reshape(B * w.N, -1).contiguous()
    gates = torch_ref.rglru_gates(p32, "", ships)

    def once():
        torch_ref.sdpa_masked(qkv, alive, harness.N_HEADS)
        return torch_ref.rglru_step(ships, gates, p32["log_lambda"], 8.0, state)

    once()
    t0 = time.perf_counter()
    once()
    one = max(time.perf_counter() - t0, 1e-6)
    reps = int(max(3, min(5000, budget_s / one)))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        once()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": B * w.NM / med,
        "unit": "entity-tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{B} of {w.B} environments of {w.name}, float32, {reps} repetitions of the two regions "
                  f"(torch SDPA with additive key bias + head merge; RG-LRU element-wise chain), median",
        "ms_per_step_sample": med * 1e3,
        "cpu_model": _cpu_model(),
    }


def _cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def load_traffic(kernel, workload):
    """Measured HBM bytes per launch, if a counter summary has been recorded for this pair."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        table = json.load(open(path))
    except (OSError, ValueError):
        return None
    entry = table.get(f"{kernel}:{workload}")
    return None if entry is None else entry["total_bytes"]


def only_update_step():
    """One YemongBlock (2 attention + 1 temporal sublayer) forward + backward over a stored 4v4 rollout, as the
    `update_path` leg times it, and nothing else: `--only-update-step` under a kernel trace lists one step's launches."""
    import boost_and_broadside_amd as bnb
    from boost_and_broadside_amd import harness

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    H, D = harness.N_HEADS, harness.D_MODEL
    gen = torch.Generator(device=dev).manual_seed(1234)
    torch.manual_seed(1234)
    blk = bnb.YemongBlock(bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=1, n_spatial_per_block=2,
                                          n_temporal_per_block=1)).to(dev)
    Tu, Bu, Nu, Mu = 128, 256, 8, 4
    xu = torch.randn(Tu, Bu, Nu + Mu, D, device=dev, generator=gen)
    au = torch.rand(Tu, Bu, Nu + Mu, device=dev, generator=gen) < 0.9
    hu = torch.zeros(1, Bu * Nu, D, device=dev)
    cu = torch.zeros(1, Bu * Nu, 3, D, device=dev)
    du = torch.rand(Tu, Bu, device=dev, generator=gen) < 0.02
    go = torch.randn(Tu, Bu, Nu + Mu, D, device=dev, generator=gen)

    def step(t):
        blk.zero_grad(set_to_none=True)
        with torch.enable_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
            out = blk.sequence(xu, au, hu, cu, du, num_recurrent=Nu)[0]
        out.backward(go)

    ms = timed_loop(step, 4, 3) / 4 * 1e3
    print(json.dumps({"leg": "update_step", "rows": Tu * Bu * (Nu + Mu), "block_fwd_bwd_given_grad_ms": ms, "steps": 4, "warmup": 3}))


def main():
    args = parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        print(
            "bench.py measures one GPU: environments are independent, so more GPUs would only shard the batch "
            f"with no exchange; run it with --gpus 1 (got --gpus {args.gpus}, WORLD_SIZE {world}).",
            file=sys.stderr,
        )
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU (the kernels have no host fallback)", file=sys.stderr)
        sys.exit(2)

    import boost_and_broadside_amd as bnb
    from boost_and_broadside_amd import harness, ops

    bnb._native.load()
    if args.only_update_step:
        only_update_step()
        return
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = harness.WORKLOADS[args.workload or harness.HEADLINE]
    steps = args.steps if args.steps is not None else max(w.steps, 32)
    warmup = args.warmup
    H, D = harness.N_HEADS, harness.D_MODEL
    bf16 = w.dtype == torch.bfloat16

    # ---- synthetic inputs, resident in HBM before anything is timed ----
    p = harness.make_weights(w.seed, w.dtype)
    step_module = harness.AttnRglruStep.from_weights(p, dev)
    alive_steps = harness.make_alive(w, steps=min(max(w.steps, 1), warmup + steps)).to(dev)
    n_alive = alive_steps.shape[0]
    # tokens and state are drawn on the host from seeded generators (seed = 1234 + workload index for the first
    # batch, as the parity tests use) and moved to the device once; the later legs' auxiliary tensors come from a
    # device generator
    first_tokens, state0 = harness.make_inputs(w)
    tokens_pool = [first_tokens.to(dev)]
    for i in range(1, POOL):
        g_host = torch.Generator().manual_seed(w.seed + 7919 * i)
        tokens_pool.append(torch.randn(w.B, w.NM, D, generator=g_host).to(w.dtype).to(dev))
    del first_tokens
    state0 = state0.to(dev)
    gen = torch.Generator(device=dev).manual_seed(w.seed)
    lam = step_module.log_lambda.detach()

    # kernel inputs exactly as the projections produce them
    qkv_pool, x_pool, gates_pool = [], [], []
    with torch.no_grad():
        for i in range(POOL):
            qkv = step_module.qkv(tokens_pool[i])
            merged = ops.sdpa_masked(qkv, alive_steps[0], H)
            ships = step_module.out_proj(merged)[:, : w.N].reshape(w.B * w.N, D).contiguous()
            qkv_pool.append(qkv)
            x_pool.append(ships)
            gates_pool.append(step_module.gates(ships))
    o_buf = torch.empty(w.B, w.NM, D, dtype=w.dtype, device=dev)
    y_buf = torch.empty(w.B * w.N, D, dtype=torch.bfloat16, device=dev) if bf16 else None
    h_bufs = [state0.clone(), torch.empty_like(state0)]
    y_dtype = torch.bfloat16 if bf16 else None

    def launch_attn(t):
        ops.sdpa_masked(qkv_pool[t % POOL], alive_steps[t % n_alive], H, out=o_buf)

    def launch_rglru(t):
        ops.rglru_step(x_pool[t % POOL], gates_pool[t % POOL], lam, 8.0, h_bufs[t & 1], h_out=h_bufs[(t + 1) & 1],
                       y_dtype=y_dtype, y_out=y_buf)

    def kernel_step(t):
        launch_attn(t)
        launch_rglru(t)

    # `value` is the median of `repeats` loops of exactly K steps: one loop of a few milliseconds reads the device
    # clock wherever it happens to be on its ramp, and a short run then reports less than a long one
    wall_eager, walls_eager = median_loop(kernel_step, steps, warmup, args.repeats)
    # The same K steps (same inputs, masks and state buffers in the same order) recorded once into a HIP graph and
    # replayed: the 2 K launches reach the GPU as one submission, without the 8 us between two launches that the
    # host-side launch path leaves at the long shapes.  `value` is the faster of the two ways to launch the K steps;
    # both times are reported.
    wall_graph, walls_graph = None, None
    if not args.no_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for t in range(steps):
                    kernel_step(warmup + t)
            wall_graph, walls_graph = median_loop(lambda t: graph.replay(), 1, 1, args.repeats)
            del graph
        except RuntimeError as err:  # capture refused: the eager figure stands
            print(f"bench: HIP graph capture of the step loop failed ({err}); timing eager launches", file=sys.stderr)
            torch.cuda.synchronize()
    wall = wall_eager if wall_graph is None else min(wall_eager, wall_graph)
    launch_mode = "hip_graph_replay" if wall_graph is not None and wall_graph <= wall_eager else "eager_launches"
    t_attn, t_rglru, med_attn, med_rglru = event_split(launch_attn, launch_rglru, steps, warmup, args.repeats)
    assert torch.isfinite(h_bufs[0]).all() and torch.isfinite(o_buf.float()).all()

    tokens = w.tokens_per_step
    ab = harness.algorithmic_bytes(w)
    peak = harness.HBM_PEAK_BYTES_PER_S

    def roof(kernel, nbytes, seconds, median):
        traffic = load_traffic(kernel, w.name)
        return {
            "kernel": kernel, "bound": "hbm", "achieved": nbytes / seconds / 1e9, "peak": peak / 1e9, "unit": "GB/s",
            "frac": nbytes / seconds / peak, "algorithmic_bytes_per_launch": nbytes, "avg_launch_us": seconds * 1e6,
            "median_launch_us": median * 1e6, "traffic": traffic,
            # a stored figure (two counter runs of this kernel at this workload), not something this run measured
            "traffic_source": None if traffic is None else "profiles/hbm_traffic.json",
            # the same fraction on the bytes the kernel actually moves (dead K/V rows are never read)
            "frac_of_measured_traffic": None if traffic is None else traffic / seconds / peak,
        }

    attn_kernel = "sdpa_mfma_f32_kernel" if D // H == 32 else "sdpa_valu_kernel"
    if bf16 and w.NM <= 160:
        attn_kernel = "sdpa_mfma_pair_kernel" if (w.NM <= 16 and H % 2 == 0) else "sdpa_mfma_kernel"
    roofs = {"attention": roof(attn_kernel, ab["attn"], t_attn, med_attn),
             # the lane map with dense memory instructions covers the widths that divide 512
             "rglru": roof("rglru_step_dense_kernel" if 512 % D == 0 else "rglru_step_vec8_kernel", ab["rglru"], t_rglru, med_rglru)}
    dominant = "attention" if t_attn >= t_rglru else "rglru"

    result = {
        "metric": METRIC,
        "value": tokens * steps / wall,
        "unit": "entity-tokens/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": wall / steps * 1e3,
        "launch": launch_mode,
        "eager_launch_ms_per_step": wall_eager / steps * 1e3,
        "hip_graph_ms_per_step": None if wall_graph is None else wall_graph / steps * 1e3,
        "repeats": len(walls_eager),
        "loops_ms_per_step": {"eager_launches": [round(x / steps * 1e3, 5) for x in walls_eager],
                              "hip_graph_replay": None if walls_graph is None else [round(x / steps * 1e3, 5) for x in walls_graph],
                              "reported": "median of each list; `value` is from the faster of the two medians"},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: {w.B} environments x ({w.N} ship + {w.M} field tokens), d_model {D}, "
                        f"{H} heads x {D // H}, alive mask '{w.alive}', fp32 recurrent state carried over the steps",
            "region": "masked attention kernel + RG-LRU step kernel (the 4 projections are reported under 'module'); the K timed "
                      "steps are launched one by one and, recorded once, as one HIP graph replay, `repeats` loops of K steps each way: "
                      "`value` is the median loop of the faster way",
            "tokens_per_step": tokens,
        },
        "roofline": roofs[dominant],
        "roofline_step": {
            "bound": "hbm", "achieved": ab["step"] / (t_attn + t_rglru) / 1e9, "peak": peak / 1e9, "unit": "GB/s",
            "frac": ab["step"] / (t_attn + t_rglru) / peak, "algorithmic_bytes_per_step": ab["step"],
            "kernel_us_per_step": (t_attn + t_rglru) * 1e6, "median_kernel_us_per_step": (med_attn + med_rglru) * 1e6,
            # the same bytes over the wall-clock step of the timed region above (what `value` and `ms_per_step` are from);
            # the event figures carry the two event records per launch as well, which shows on launches of ~20 us
            "wall_us_per_step": wall / steps * 1e6, "frac_by_wall_clock": ab["step"] / (wall / steps) / peak,
        },
        "kernels": roofs,
    }

    # ---- yardstick: plain copy through the library's copy kernel ----
    n_copy = 1 << 30
    src = torch.empty(n_copy, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    t_copy = timed_loop(lambda t: ops.copy_bytes(src, dst), 20, 3) / 20
    result["copy_kernel"] = {"GBps_read_plus_write": 2 * n_copy / t_copy / 1e9, "bytes": n_copy}
    del src, dst

    # ---- yardstick of the issue-bound kernels: how a SIMD's issue is shared by matrix products and vector arithmetic ----
    if not args.no_issue_probe:
        mfma_only = ops.issue_probe(0)
        fma16 = ops.issue_probe(16, mfma=False)
        sweep = {str(m): ops.issue_probe(m) for m in (2, 4, 8, 12, 16)}
        mixed = ops.issue_probe(10, transcendentals=True)
        mixed_alone = ops.issue_probe(10, mfma=False, transcendentals=True)
        result["issue_probe"] = {
            "ns_per_slot": {"mfma_only": mfma_only, "16_fma_only": fma16, "mfma_plus_n_fma": sweep,
                            "mfma_plus_8_fma_2_exp": mixed, "8_fma_2_exp_only": mixed_alone},
            # 1 = the matrix product and the vector work take as long together as one after the other, 0 = the shorter
            # of the two disappears under the longer
            "serial_fraction_mfma_plus_16_fma": (sweep["16"] - max(mfma_only, fma16)) / min(mfma_only, fma16),
            "what": "bnb_issue_probe at two waves per SIMD: one 32x32x16 bf16 matrix product followed by n independent "
                    "vector instructions, order pinned; nanoseconds per such slot on one SIMD",
        }

    # ---- the same two regions through eager PyTorch on the GPU ----
    if not args.no_torch_baseline:
        hb = [state0.clone()]

        def torch_step(t):
            torch_attention_region(qkv_pool[t % POOL], alive_steps[t % n_alive], H)
            hb[0] = torch_rglru_region(x_pool[t % POOL], gates_pool[t % POOL], lam, 8.0, hb[0])

        n_t = max(4, min(steps, 16))
        wall_t = timed_loop(torch_step, n_t, 2)
        # no published number exists for this metric, so "vs_baseline" stays null; the ratio to the reference-style
        # eager path on the same GPU is reported under its own name
        result["vs_torch_gpu_baseline"] = (tokens * steps / wall_eager) / (tokens * n_t / wall_t)  # eager launches on both sides
        result["torch_gpu_baseline"] = {
            "value": tokens * n_t / wall_t, "unit": "entity-tokens/s", "ms_per_step": wall_t / n_t * 1e3,
            "steps": n_t, "speedup_of_this_build": (tokens * steps / wall_eager) / (tokens * n_t / wall_t),
            "what": "F.scaled_dot_product_attention with additive key bias + head-merge copy, and the eager "
                    "RG-LRU element-wise chain, same inputs, same dtype",
        }

    # ---- whole module step: 4 projections + the two kernels ----
    if not args.no_module:
        st = [state0.clone()]

        def module_step(t):
            _, st[0] = step_module(tokens_pool[t % POOL], alive_steps[t % n_alive], st[0])

        wall_m = timed_loop(module_step, steps, warmup)
        result["module"] = {"value": tokens * steps / wall_m, "unit": "entity-tokens/s", "ms_per_step": wall_m / steps * 1e3}

    # ---- conv-step kernel (temporal block's causal conv + buffer shift on the packed state) ----
    R = w.B * w.N
    packed = [torch.randn(R, 4 * D, device=dev, generator=gen), None]
    packed[1] = torch.empty_like(packed[0])
    b1_pool = [x_pool[i] for i in range(POOL)]  # same shape and dtype as linear1's output
    conv_w = 0.5 * torch.randn(D, 1, 4, device=dev, generator=gen)
    conv_b = 0.1 * torch.randn(D, device=dev, generator=gen)

    def launch_conv(t):
        src, dst = packed[t & 1], packed[(t + 1) & 1]
        ops.conv_step(b1_pool[t % POOL], src[:, D:].view(R, 3, D), conv_w, conv_b, conv_out=dst[:, D:].view(R, 3, D))

    t_conv = timed_loop(launch_conv, steps, warmup) / steps
    s_act = 2 if bf16 else 4
    conv_bytes = R * (D * s_act + 3 * D * 4 + D * 4 + 3 * D * 4)
    result["conv_step_kernel"] = {
        "avg_launch_us": t_conv * 1e6, "algorithmic_bytes_per_launch": conv_bytes, "achieved_GBps": conv_bytes / t_conv / 1e9,
        "frac_of_hbm_peak": conv_bytes / t_conv / peak,
        "what": "read linear1 output + 3 stored inputs, write conv output + shifted inputs into the packed state",
    }
    # ---- conv + gate projections + recurrence as one kernel, beside the three-kernel composition ----
    if bf16:
        gw_a = torch.randn(D, D, device=dev, generator=gen) / D ** 0.5
        gw_x = torch.randn(D, D, device=dev, generator=gen) / D ** 0.5
        g_bias = 0.3 * torch.randn(2 * D, device=dev, generator=gen)
        g_pack = ops.pack_gate_weights(gw_a, gw_x)
        g_w16, g_b16 = torch.cat([gw_a, gw_x]).to(torch.bfloat16), g_bias.to(torch.bfloat16)
        y_ts = torch.empty(R, D, device=dev, dtype=torch.bfloat16)

        def launch_fused(t):
            src, dst = packed[t & 1], packed[(t + 1) & 1]
            ops.temporal_step(b1_pool[t % POOL], src[:, D:].view(R, 3, D), src[:, :D], conv_w, conv_b, g_pack, g_bias, lam, 8.0,
                              conv_out=dst[:, D:].view(R, 3, D), h_out=dst[:, :D], y_out=y_ts)

        def launch_three(t):
            src, dst = packed[t & 1], packed[(t + 1) & 1]
            v, _, v16 = ops.conv_step(b1_pool[t % POOL], src[:, D:].view(R, 3, D), conv_w, conv_b,
                                      conv_out=dst[:, D:].view(R, 3, D), also_bf16=True)
            ops.rglru_step(v, F.linear(v16, g_w16, g_b16), lam, 8.0, src[:, :D], h_out=dst[:, :D], y_out=y_ts)

        t_ts = timed_loop(launch_fused, steps, warmup) / steps
        t_three = timed_loop(launch_three, steps, warmup) / steps
        ts_bytes = R * (D * 2 + 2 * 3 * D * 4 + 2 * D * 4 + D * 2)
        result["temporal_step_kernel"] = {
            "rows": R, "avg_launch_us": t_ts * 1e6, "algorithmic_bytes_per_launch": ts_bytes, "achieved_GBps": ts_bytes / t_ts / 1e9,
            "frac_of_hbm_peak": ts_bytes / t_ts / peak, "traffic": load_traffic("temporal_step_kernel", w.name),
            "three_kernel_composition_us": t_three * 1e6,
            "what": "conv taps + buffer shift, both gate projections (matrix cores) and the recurrence in one kernel: "
                    "bf16 linear1 output, packed fp32 state in, packed fp32 state and bf16 layer output out; "
                    "composition = conv kernel, library GEMM, recurrence kernel",
        }
    del packed

    # ---- fused sublayer tail: add + RMSNorm + gated MLP + add on the matrix cores ----
    if bf16 and not args.no_ffn:
        Rf = w.B * w.NM
        mlp = bnb.GatedMLP(D).to(dev).eval()
        nw = torch.ones(D, device=dev)
        pk = mlp.packed_weights()
        xf = torch.randn(Rf, D, device=dev, generator=gen)
        df = torch.randn(Rf, D, device=dev, generator=gen).to(torch.bfloat16)
        of = torch.empty_like(xf)
        n_f = max(4, min(steps, 16))
        t_ffn = timed_loop(lambda t: ops.ffn_fused(xf, df, nw, pk, out=of), n_f, 3) / n_f

        def ffn_library(t):
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                s = xf + df
                n = F.rms_norm(s, (D,), nw, None)
                return s + mlp.down_proj(F.gelu(mlp.gate_proj(n)) * mlp.up_proj(n))

        t_ffn_lib = None if args.no_torch_baseline else timed_loop(ffn_library, n_f, 3) / n_f
        ffn_flops = Rf * 2 * (D * 2 * 4 * D + 4 * D * D)
        ffn_bytes = Rf * (4 * D + 2 * D + 4 * D)
        result["ffn_fused_kernel"] = {
            "rows": Rf, "avg_launch_us": t_ffn * 1e6, "tflops": ffn_flops / t_ffn / 1e12,
            "frac_of_bf16_mfma_peak": ffn_flops / t_ffn / 2.5e15,
            "algorithmic_bytes_per_launch": ffn_bytes, "achieved_GBps": ffn_bytes / t_ffn / 1e9,
            "eager_torch_us": None if t_ffn_lib is None else t_ffn_lib * 1e6,
            "what": "x + delta, RMSNorm, gate/up projections, gelu * up, down projection, residual add in one kernel; "
                    "x fp32 and delta bf16 in, fp32 out; eager = the same composition in torch ops under bf16 autocast",
        }
        del xf, df, of, mlp

    # ---- bullet read (entity queries attending to the bullets in flight; 10 slots per ship) ----
    if bf16 and not args.no_bullets:
        NB = w.N * 10
        live_p = 0.25
        kv_b = (0.7 * torch.randn(w.B, NB, 2 * D, device=dev, generator=gen)).to(w.dtype)
        b_mask = torch.rand(w.B, NB, device=dev, generator=gen) < live_p
        merged = [torch.zeros(w.B, w.NM, D, device=dev, dtype=w.dtype) for _ in range(2)]
        qkv_b = qkv_pool[0]
        n_b = max(4, min(steps, 16))
        t_read = timed_loop(lambda t: ops.sdpa_cross(qkv_b, kv_b, b_mask, H, accum=merged[t & 1]), n_b, 3) / n_b

        def torch_read(t):
            q = qkv_b[..., :D].reshape(w.B, w.NM, H, D // H).transpose(1, 2)
            kb = kv_b[..., :D].reshape(w.B, NB, H, D // H).transpose(1, 2)
            vb = kv_b[..., D:].reshape(w.B, NB, H, D // H).transpose(1, 2)
            bias = (1.0 - b_mask.reshape(w.B, 1, 1, NB).to(q.dtype)) * (torch.finfo(q.dtype).min / 2)
            o = torch.nn.functional.scaled_dot_product_attention(q, kb, vb, attn_mask=bias)
            o = o * b_mask.any(-1).reshape(w.B, 1, 1, 1).to(o.dtype)
            merged[t & 1] += o.transpose(1, 2).reshape(w.B, w.NM, D)

        t_read_torch = None if args.no_torch_baseline else timed_loop(torch_read, 3, 1) / 3
        live = int(b_mask.sum().item())

        # the whole bullet branch of a layer, from raw bullet tokens: list of the bullets in flight,
        # norm + kv projection over that list, read over per-environment row ranges ...
        bullets_f = torch.randn(w.B, NB, D, device=dev, generator=gen)
        layer_b = bnb.TransformerBlock(bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=1, n_spatial_per_block=1, n_bullet_cross_per_block=1),
                                       reads_bullets=True).to(dev).eval()
        pk_kv = ops.pack_linear_weights(layer_b.kv_bullet.weight)

        def branch_compact(t):
            rows = ops.CompactRows(b_mask)
            kv_rows = ops.norm_linear(bullets_f, layer_b.norm_bullet.weight, pk_kv, rows=rows)
            ops.sdpa_cross_rows(qkv_b, kv_rows, rows, H, accum=merged[t & 1])

        # ... against the same branch over every slot (norm kernel, library GEMM, masked read)
        def branch_all_slots(t):
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                n = ops.add_rmsnorm(bullets_f, layer_b.norm_bullet.weight, out_dtype=torch.bfloat16)[1]
                ops.sdpa_cross(qkv_b, layer_b.kv_bullet(n), b_mask, H, accum=merged[t & 1])

        t_branch = timed_loop(branch_compact, n_b, 3) / n_b
        t_branch_all = timed_loop(branch_all_slots, 4, 2) / 4
        del bullets_f, layer_b

        # the read over rows compacted beforehand (what the trunk calls), and its backward (the PPO update's
        # kernels for this read: one tile of keys up to 160 live bullets per environment, the streaming pair above)
        rows_b = ops.CompactRows(b_mask)
        total_b = rows_b.total_host()
        kv_rows_b = kv_b.reshape(w.B * NB, 2 * D)[b_mask.reshape(-1)].contiguous()
        t_rows = timed_loop(lambda t: ops.sdpa_cross_rows(qkv_b, kv_rows_b, rows_b, H, accum=merged[t & 1], total=total_b), n_b, 3) / n_b
        # as the update runs it: the forward hands its log-sum-exp to the backward when the streaming kernels apply
        lse_b = torch.empty((w.B, H, w.NM), dtype=torch.float32, device=dev) if rows_b.max_count_host() > 160 else None
        out_b = ops.sdpa_cross_rows(qkv_b, kv_rows_b, rows_b, H, total=total_b, lse=lse_b)
        dout_b = (0.5 * torch.randn(w.B, w.NM, D, device=dev, generator=gen)).to(w.dtype)
        t_bwd = timed_loop(lambda t: ops.sdpa_cross_rows_bwd(qkv_b, kv_rows_b, rows_b, H, out_b, dout_b, total_b, lse=lse_b), n_b, 3) / n_b
        t_bwd_alone = timed_loop(lambda t: ops.sdpa_cross_rows_bwd(qkv_b, kv_rows_b, rows_b, H, out_b, dout_b, total_b), n_b, 3) / n_b
        del kv_rows_b, out_b, dout_b, lse_b
        read_bytes = live * 2 * D * 2 + w.B * NB + 3 * w.B * w.NM * D * 2
        result["bullet_read"] = {
            "avg_launch_us": t_read * 1e6, "slots_per_env": NB, "live_fraction": live_p,
            "algorithmic_bytes_per_launch": read_bytes, "achieved_GBps": read_bytes / t_read / 1e9,
            "frac_of_hbm_peak": read_bytes / t_read / peak,
            "tflops": 4 * live * w.NM * D / t_read / 1e12,
            "eager_torch_us": None if t_read_torch is None else t_read_torch * 1e6,
            "rows_form_us": t_rows * 1e6, "rows_form_backward_us": t_bwd * 1e6,
            "rows_form_backward_recomputing_lse_us": t_bwd_alone * 1e6, "max_live_per_env": rows_b.max_count_host(),
            "branch_compact_us": t_branch * 1e6, "branch_all_slots_us": t_branch_all * 1e6,
            "branch_what": "norm_bullet + kv_bullet + read from fp32 bullet tokens: compact = device-side list of the "
                           "live bullets, bnb_norm_linear_fwd over it, bnb_sdpa_cross_ranges_fwd; all_slots = "
                           "bnb_add_rmsnorm_fwd + library GEMM over every slot + bnb_sdpa_cross_fwd with the mask",
            "what": "bnb_sdpa_cross_fwd added into the self-attention output: K/V rows of the live bullets, the slot "
                    "mask, Q, accumulator in and out; exp-throughput-bound rather than HBM-bound when many bullets are live",
        }
        del kv_b, b_mask, merged

    # ---- fp32 attention at an evaluation shape (crossover runs without autocast), kernel beside the library ----
    if not args.no_fp32_attention:
        Be, NMe = 1024, 160
        qkv_e = torch.randn(Be, NMe, 3 * D, device=dev, generator=gen)
        alive_e = torch.rand(Be, NMe, device=dev, generator=gen) < 0.7
        alive_e[:, 0] = True
        n_e = max(4, min(steps, 16))
        t_e = timed_loop(lambda t: ops.sdpa_masked(qkv_e, alive_e, H), n_e, 3) / n_e
        t_e_valu = timed_loop(lambda t: ops.sdpa_masked(qkv_e, alive_e, H, path="valu"), n_e, 3) / n_e

        def attention_library(t):
            q, k, v = (a.reshape(Be, NMe, H, D // H).transpose(1, 2) for a in qkv_e.split(D, dim=-1))
            bias = (1.0 - alive_e.reshape(Be, 1, 1, NMe).float()) * (torch.finfo(torch.float32).min / 2)
            return F.scaled_dot_product_attention(q, k, v, attn_mask=bias).transpose(1, 2).reshape(Be, NMe, D)

        t_e_lib = None if args.no_torch_baseline else timed_loop(attention_library, n_e, 3) / n_e
        flops_e = 4.0 * Be * NMe * NMe * D
        result["fp32_attention_kernel"] = {
            "environments": Be, "tokens": NMe, "avg_launch_us": t_e * 1e6, "tflops": flops_e / t_e / 1e12,
            "frac_of_fp32_mfma_peak": flops_e / t_e / 157.3e12, "vector_kernel_us": t_e_valu * 1e6,
            "eager_torch_us": None if t_e_lib is None else t_e_lib * 1e6,
            "what": "masked attention in float32 on v_mfma_f32_32x32x2_f32 (flops counted over all keys, 70 % of them "
                    "alive); vector_kernel = the float32 vector-ALU kernel on the same input; eager = torch SDPA with the "
                    "additive key bias and the head-merge copy",
        }
        del qkv_e

    # ---- team pooling over the ships (the value head's input), kernel beside the library composition ----
    if not args.no_team_pool:
        pma = bnb.TeamPMA(D, H).to(dev).eval()
        with torch.no_grad():
            pma.seeds.normal_(0.0, 0.02)
        xs_t = torch.randn(w.B, w.NM, D, device=dev, generator=gen)
        team_t = torch.randint(0, 2, (w.B, w.NM), device=dev, generator=gen, dtype=torch.int32)
        alive_t = alive_steps[0]
        ship_x, ship_team, ship_alive = xs_t[:, :w.N], team_t[:, :w.N], alive_t[:, :w.N]
        n_p = max(4, min(steps, 16))
        with torch.no_grad():
            t_pool = timed_loop(lambda t: pma(ship_x, ship_team, ship_alive), n_p, 3) / n_p

        def pool_library(t):
            # the same function through the library: two attention calls with the seed as query
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=bf16):
                team_pool = ship_x.new_zeros(w.B, 2, D)
                for team in range(2):
                    keys = (ship_team == team) & ship_alive
                    o, _ = pma.attn(pma.seeds[team].view(1, 1, D).expand(w.B, 1, D), ship_x, ship_x,
                                    key_padding_mask=~keys, need_weights=False)
                    o = o.squeeze(1).nan_to_num(0.0) * keys.any(dim=1).unsqueeze(1).to(o.dtype)
                    team_pool[:, team] = pma.norm(o)
                return team_pool.gather(1, ship_team.clamp(0, 1).long().unsqueeze(-1).expand(w.B, w.N, D))

        t_pool_lib = None if args.no_torch_baseline else timed_loop(pool_library, n_p, 3) / n_p
        pool_bytes = w.B * w.N * (D * 4 + 4 + 1 + D * 4)
        result["team_pool_kernel"] = {
            "environments": w.B, "ships": w.N, "avg_launch_us": t_pool * 1e6, "algorithmic_bytes_per_launch": pool_bytes,
            "achieved_GBps": pool_bytes / t_pool / 1e9, "frac_of_hbm_peak": pool_bytes / t_pool / peak,
            "eager_torch_us": None if t_pool_lib is None else t_pool_lib * 1e6,
            "attend_algorithmic_bytes": w.B * w.N * (D * 4 + 4 + 1) + w.B * 2 * H * D * 4,
            "handout_algorithmic_bytes": w.B * 2 * D * 4 + w.B * w.N * (4 + D * 4),
            "what": "per-team attention pooling with a learned seed as the only query, out projection, RMSNorm and the "
                    "broadcast back to the ships, fp32: a kernel that reads the ship rows once, one library GEMM on the pooled rows, a "
                    "kernel that writes (B, N, D) once; eager = "
                    "two nn.MultiheadAttention calls, norm and gather in torch ops (bf16 autocast on bf16 workloads)",
        }
        del xs_t

    # ---- update path: the recurrence over a stored rollout (T = 128), forward and backward ----
    if not args.no_sequence:
        Rs, Ts = 8192, 128  # 1024 environments x 8 ships, the rollout length of the reference's training run
        g_dt = torch.bfloat16 if bf16 else torch.float32
        xs = torch.randn(Ts, Rs, D, device=dev, generator=gen)
        gs = torch.randn(Ts, Rs, 2 * D, device=dev, generator=gen).to(g_dt)
        hs = torch.randn(Rs, D, device=dev, generator=gen)
        dn = torch.rand(Rs, Ts, device=dev, generator=gen) < 0.02
        lam_s = lam
        t_scan = timed_loop(lambda t: ops.rglru_scan(xs, gs, lam_s, 8.0, hs, dn, y_dtype=g_dt, time_major=True), 8, 2) / 8
        es = 2 if bf16 else 4
        scan_bytes = Rs * Ts * D * (4 + 2 * es + es) + Rs * Ts
        leaves = [t.clone().requires_grad_(True) for t in (xs, gs, lam_s, hs)]

        def scan_train(t):
            for leaf in leaves:
                leaf.grad = None
            with torch.enable_grad():
                y, _ = ops.rglru_scan(leaves[0], leaves[1], leaves[2], 8.0, leaves[3], dn, time_major=True)
                y.backward(xs)

        t_train = timed_loop(scan_train, 4, 2) / 4
        bwd_bytes = Rs * Ts * D * (4 + 2 * es + 4 + 4 + 4 + 2 * es)  # x, gates, y, dy in; dx, dgates out
        t_ref = t_ref_train = None
        if not args.no_torch_baseline:
            xr, gr = xs.transpose(0, 1).contiguous(), gs.transpose(0, 1).contiguous()
            t_ref = timed_loop(lambda t: torch_scan_region(xr, gr, lam_s, 8.0, hs, dn), 2, 1) / 2
            rl = [t.clone().requires_grad_(True) for t in (xr, gr, lam_s, hs)]

            def ref_train(t):
                for leaf in rl:
                    leaf.grad = None
                with torch.enable_grad():
                    torch_scan_region(rl[0], rl[1], rl[2], 8.0, rl[3], dn)[0].backward(xr)

            t_ref_train = timed_loop(ref_train, 2, 1) / 2
            del xr, gr, rl
        result["sequence"] = {
            "rows": Rs, "T": Ts, "scan_fwd_us": t_scan * 1e6, "scan_fwd_algorithmic_bytes": scan_bytes,
            "scan_fwd_GBps": scan_bytes / t_scan / 1e9, "scan_fwd_frac_of_hbm_peak": scan_bytes / t_scan / peak,
            "scan_fwd_bwd_us": t_train * 1e6, "scan_bwd_algorithmic_bytes": bwd_bytes,
            "eager_torch_fwd_us": None if t_ref is None else t_ref * 1e6,
            "eager_torch_fwd_bwd_us": None if t_ref_train is None else t_ref_train * 1e6,
            "what": "bnb_rglru_scan_fwd / _bwd over (T, rows, D): x fp32, gate pre-activations and states in the "
                    "projection dtype; eager = the reference's coefficient chain + Hillis-Steele scan in torch ops "
                    "(and autograd through it)",
        }
        del xs, gs, hs, dn, leaves

        # weight gradients of the trunk's Linear layers over a stored rollout: rows = T x environments x tokens
        if bf16:
            Rw = 128 * 256 * 12  # T = 128, 256 environments of 4v4 (8 ships + 4 fields)
            wg = {}
            for name, (Nw, Kw) in (("qkv", (3 * D, D)), ("square", (D, D)), ("gate_or_up", (4 * D, D)), ("down", (D, 4 * D))):
                dy_w = torch.randn(Rw, Nw, device=dev, generator=gen).to(torch.bfloat16)
                x_w = torch.randn(Rw, Kw, device=dev, generator=gen).to(torch.bfloat16)
                dw = torch.empty(Nw, Kw, device=dev)
                t_w = timed_loop(lambda t: ops.linear_wgrad(dy_w, x_w, out=dw), 8, 3) / 8
                t_w_lib = None if args.no_torch_baseline else timed_loop(lambda t: torch.mm(dy_w.t(), x_w), 4, 2) / 4
                by = Rw * (Nw + Kw) * 2 + Nw * Kw * 4
                wg[name] = {"N": Nw, "K": Kw, "us": t_w * 1e6, "algorithmic_bytes": by, "GBps": by / t_w / 1e9,
                            "frac_of_hbm_peak": by / t_w / peak, "tflops": 2.0 * Rw * Nw * Kw / t_w / 1e12,
                            "library_us": None if t_w_lib is None else t_w_lib * 1e6}
                del dy_w, x_w, dw
            cfg_u = bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=1, n_spatial_per_block=2, n_temporal_per_block=1)
            torch.manual_seed(w.seed)
            blk = bnb.YemongBlock(cfg_u).to(dev)
            Tu, Bu, Nu, Mu = 128, 256, 8, 4
            xu = torch.randn(Tu, Bu, Nu + Mu, D, device=dev, generator=gen)
            au = torch.rand(Tu, Bu, Nu + Mu, device=dev, generator=gen) < 0.9
            hu = torch.zeros(1, Bu * Nu, D, device=dev)
            cu = torch.zeros(1, Bu * Nu, 3, D, device=dev)
            du = torch.rand(Tu, Bu, device=dev, generator=gen) < 0.02

            def update_step(t):
                blk.zero_grad(set_to_none=True)
                with torch.enable_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                    out_u = blk.sequence(xu, au, hu, cu, du, num_recurrent=Nu)[0]
                out_u.float().square().mean().backward()

            go_blk = torch.randn(Tu, Bu, Nu + Mu, D, device=dev, generator=gen)

            def update_step_given_grad(t):  # the block alone: the gradient of its output is handed in, no loss kernels
                blk.zero_grad(set_to_none=True)
                with torch.enable_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                    out_u = blk.sequence(xu, au, hu, cu, du, num_recurrent=Nu)[0]
                out_u.backward(go_blk)

            from boost_and_broadside_amd import trunk as trunk_module
            t_up = timed_loop(update_step, 3, 2) / 3
            t_up_g = timed_loop(update_step_given_grad, 3, 2) / 3
            t_up_lib = None
            if not args.no_torch_baseline:
                with trunk_module.library_update_path():
                    t_up_lib = timed_loop(update_step, 3, 2) / 3
            # the same block reading the bullets in flight (the reference's shipped default: one bullet-reading
            # attention sublayer per block, 10 slots per ship, a quarter of them live)
            cfg_b = bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=1, n_spatial_per_block=2, n_temporal_per_block=1,
                                    n_bullet_cross_per_block=1)
            torch.manual_seed(w.seed)
            blk_b = bnb.YemongBlock(cfg_b).to(dev)
            bul_u = torch.randn(Tu * Bu, Nu * 10, D, device=dev, generator=gen, requires_grad=True)
            bm_u = torch.rand(Tu * Bu, Nu * 10, device=dev, generator=gen) < 0.25

            def update_step_bullets(t):
                blk_b.zero_grad(set_to_none=True)
                bul_u.grad = None
                with torch.enable_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                    out_b = blk_b.sequence(xu, au, hu, cu, du, Nu, bul_u, bm_u)[0]
                out_b.float().square().mean().backward()

            t_upb = timed_loop(update_step_bullets, 3, 2) / 3
            t_upb_lib = None
            if not args.no_torch_baseline:
                with trunk_module.library_update_path():
                    t_upb_lib = timed_loop(update_step_bullets, 2, 1) / 2
            del blk_b, bul_u, bm_u

            # the other update-path kernels at the same size, each against its algorithmic bytes
            def stream_leg(fn, nbytes, reps=8):
                t = timed_loop(fn, reps, 3) / reps
                return {"us": t * 1e6, "algorithmic_bytes": nbytes, "GBps": nbytes / t / 1e9, "frac_of_hbm_peak": nbytes / t / peak}

            kern = {}
            xn = torch.randn(Rw, D, device=dev, generator=gen)
            dyn = torch.randn(Rw, D, device=dev, generator=gen).to(torch.bfloat16)
            gsn = torch.randn(Rw, D, device=dev, generator=gen)
            wn = torch.ones(D, device=dev)
            kern["rmsnorm_bwd"] = stream_leg(lambda t: ops.rmsnorm_bwd(xn, dyn, wn, grad_sum=gsn), Rw * D * (4 + 2 + 4 + 4))
            del xn, dyn, gsn
            ag = torch.randn(Rw, 4 * D, device=dev, generator=gen).to(torch.bfloat16)
            bg = torch.randn(Rw, 4 * D, device=dev, generator=gen).to(torch.bfloat16)
            dg = torch.randn(Rw, 4 * D, device=dev, generator=gen).to(torch.bfloat16)
            kern["gelu_mul_bwd"] = stream_leg(lambda t: ops.gelu_mul_bwd(ag, bg, dg), Rw * 4 * D * 2 * 5)
            del ag, bg, dg
            # the gated MLP of the update: fused tail forward that keeps s and n, and the recompute-backward
            # (n 256 B + dy 512 B in, dn 256 B + dy bf16 256 B + [dg | du] 2 KB + h 1 KB out per row; 2 * 2560 * 128 flops
            # per row: gate/up again, dh, dn)
            mlp_u = bnb.GatedMLP(D).to(dev)
            ws_u = (mlp_u.gate_proj.weight, mlp_u.up_proj.weight, mlp_u.down_proj.weight)
            pf_u, pb_u = ops.pack_ffn_weights(*ws_u), ops.pack_ffn_bwd_weights(*ws_u)
            nn_u = torch.randn(Rw, D, device=dev, generator=gen).to(torch.bfloat16)
            dy_u = torch.randn(Rw, D, device=dev, generator=gen)
            kern["ffn_bwd"] = stream_leg(lambda t: ops.ffn_bwd(nn_u, dy_u, pb_u), Rw * (256 + 512 + 256 + 256 + 2048 + 1024))
            kern["ffn_bwd"]["tflops"] = 2.0 * Rw * 2560 * D / (kern["ffn_bwd"]["us"] * 1e-6) / 1e12
            xt_u = torch.randn(Rw, D, device=dev, generator=gen, requires_grad=True)
            dl_u = torch.randn(Rw, D, device=dev, generator=gen).to(torch.bfloat16).requires_grad_()
            nw_u = torch.ones(D, device=dev, requires_grad=True)

            def tail_fwd(t):
                with torch.enable_grad():
                    ops.ffn_tail_train(xt_u, dl_u, nw_u, *ws_u, eps=None, packed_fwd=pf_u, packed_bwd=pb_u)

            kern["ffn_tail_train_fwd"] = stream_leg(tail_fwd, Rw * (512 + 256 + 512 + 256 + 512))
            del mlp_u, nn_u, dy_u, xt_u, dl_u
            Ba = Tu * Bu
            qa = torch.randn(Ba, Nu + Mu, 3 * D, device=dev, generator=gen).to(torch.bfloat16)
            aa = torch.rand(Ba, Nu + Mu, device=dev, generator=gen) < 0.9
            oa = ops.sdpa_masked(qa, aa, H)
            da = torch.randn(Ba, Nu + Mu, D, device=dev, generator=gen).to(torch.bfloat16)
            kern["sdpa_masked_bwd"] = stream_leg(lambda t: ops.sdpa_masked_bwd(qa, aa, H, oa, da), Ba * (Nu + Mu) * D * 2 * (3 + 1 + 1 + 3))
            kern["sdpa_masked_fwd"] = stream_leg(lambda t: ops.sdpa_masked(qa, aa, H, out=oa), Ba * (Nu + Mu) * D * 2 * 4)
            del qa, aa, oa, da
            Rc = Bu * Nu
            bc = torch.randn(Tu, Rc, D, device=dev, generator=gen).to(torch.bfloat16)
            cc = torch.randn(Rc, 3, D, device=dev, generator=gen)
            wc = torch.randn(D, 1, 4, device=dev, generator=gen)
            dc = torch.rand(Rc, Tu, device=dev, generator=gen) < 0.02
            dvc = torch.randn(Tu, Rc, D, device=dev, generator=gen)
            kern["conv_seq_bwd"] = stream_leg(lambda t: ops.conv_seq_bwd(bc, cc, wc, dc, dvc, time_major=True), Tu * Rc * D * (2 + 4 + 2))
            del bc, cc, dvc
            # the value head's team pooling over the same rollout, forward + backward
            pma_u = bnb.TeamPMA(D, H).to(dev)
            with torch.no_grad():
                pma_u.seeds.normal_(0.0, 0.02)
            xs_u = torch.randn(Tu * Bu, Nu, D, device=dev, generator=gen, requires_grad=True)
            tm_u = torch.randint(0, 2, (Tu * Bu, Nu), device=dev, generator=gen, dtype=torch.int32)
            al_u = torch.rand(Tu * Bu, Nu, device=dev, generator=gen) < 0.9
            go_u = torch.randn(Tu * Bu, Nu, D, device=dev, generator=gen)

            def pool_step(t):
                pma_u.zero_grad(set_to_none=True)
                xs_u.grad = None
                with torch.enable_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
                    pma_u(xs_u, tm_u, al_u).backward(go_u)

            t_pool_up = timed_loop(pool_step, 4, 2) / 4
            t_pool_up_lib = None
            if not args.no_torch_baseline:
                with trunk_module.library_update_path():
                    t_pool_up_lib = timed_loop(pool_step, 3, 2) / 3
            del pma_u, xs_u, tm_u, al_u, go_u
            result["update_path"] = {
                "rows": Rw, "linear_wgrad": wg, "kernels": kern, "block_fwd_bwd_ms": t_up * 1e3,
                "block_fwd_bwd_given_grad_ms": t_up_g * 1e3,
                "block_with_bullets_fwd_bwd_ms": t_upb * 1e3,
                "block_with_bullets_fwd_bwd_library_ms": None if t_upb_lib is None else t_upb_lib * 1e3,
                "team_pool_fwd_bwd_ms": t_pool_up * 1e3,
                "team_pool_fwd_bwd_library_ms": None if t_pool_up_lib is None else t_pool_up_lib * 1e3,
                "block_fwd_bwd_library_ms": None if t_up_lib is None else t_up_lib * 1e3,
                "what": "bnb_linear_wgrad_fwd (dW = dy^T x, bf16 in, fp32 out, rows split over the chip) beside the library "
                        "GEMM on the same operands; kernels = the norm, gelu-gate, gated-MLP, attention and conv backward kernels at the "
                        "sizes of the block below; block = one YemongBlock (2 attention + 1 temporal sublayer), T = 128 x 256 "
                        "environments of 4v4, forward + backward of mean(out^2) under bf16 autocast (given_grad: backward from a "
                        "given gradient of the output instead, i.e. without the loss's own kernels), on the update-path kernels and with "
                        "torch's own differentiable ops in their place (the recurrence keeps its kernels in both); block_with_bullets = "
                        "the same with one attention sublayer reading 80 bullet slots per environment, 25 % live; team_pool = TeamPMA "
                        "forward + backward over the ships of the same rollout (32,768 environments x 8 ships), kernels and library",
            }
            del blk, xu, au, hu, cu, du

    # ---- whole trunk (reference default: 2 blocks x (2 spatial + 1 temporal)), state carried ----
    if not args.no_trunk:
        cfg = bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=2, n_spatial_per_block=2, n_temporal_per_block=1)
        torch.manual_seed(w.seed)
        trunk = bnb.YemongTrunk(cfg).to(dev).eval()
        x32 = [t.float() for t in tokens_pool[:2]]
        n_tr = max(4, min(steps, 16))
        hid = [trunk.initial_hidden(w.B, w.N, dev), None]
        hid[1] = torch.empty_like(hid[0])

        def trunk_step(t):
            with torch.autocast("cuda", dtype=torch.bfloat16, enabled=bf16):
                trunk(x32[t & 1], alive_steps[t % n_alive], hid[t & 1], out_state=hid[(t + 1) & 1])

        wall_tr = timed_loop(trunk_step, n_tr, 10)  # first calls pay GEMM heuristics and code loading
        ref_h = [trunk.initial_hidden(w.B, w.N, dev)]

        def trunk_step_eager(t):
            with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16, enabled=bf16):
                _, ref_h[0] = reference_style_trunk_step(trunk, x32[t & 1], alive_steps[t % n_alive], ref_h[0], w.N)

        with eager_kernels():
            wall_te = timed_loop(trunk_step_eager, n_tr, 10)
        graphed = bnb.GraphedTrunk(trunk, w.B, w.NM, w.N, autocast_dtype=torch.bfloat16 if bf16 else None)
        wall_g = timed_loop(lambda t: graphed.step(x32[t & 1], alive_steps[t % n_alive]), n_tr, 4)
        # a producer that writes tokens and mask straight into the capture's input buffers: no staging copies
        wall_gi = timed_loop(lambda t: graphed.step(graphed.tokens, graphed.alive, graphed.reset), n_tr, 4)
        del graphed
        # the shipped default (config/defaults.py:21-31) also reads the bullets in flight in the first attention sublayer
        # of each block: 10 slots per ship, a quarter of them live here
        wall_tb = None
        if not args.no_bullets and bf16:
            cfg_tb = bnb.ModelConfig(d_model=D, n_heads=H, n_yemong_blocks=2, n_spatial_per_block=2, n_temporal_per_block=1,
                                     n_bullet_cross_per_block=1)
            torch.manual_seed(w.seed)
            trunk_b = bnb.YemongTrunk(cfg_tb).to(dev).eval()
            bul_t = torch.randn(w.B, w.N * 10, D, device=dev, generator=gen)
            bm_t = torch.rand(w.B, w.N * 10, device=dev, generator=gen) < 0.25

            def trunk_step_bullets(t):
                with torch.autocast("cuda", dtype=torch.bfloat16):
                    trunk_b(x32[t & 1], alive_steps[t % n_alive], hid[t & 1], bul_t, bm_t, out_state=hid[(t + 1) & 1])

            wall_tb = timed_loop(trunk_step_bullets, n_tr, 6)
            del trunk_b, bul_t, bm_t
        result["trunk"] = {
            "value": tokens * n_tr / wall_tr, "unit": "entity-tokens/s", "ms_per_step": wall_tr / n_tr * 1e3,
            "hip_graph_ms_per_step": wall_g / n_tr * 1e3,
            "hip_graph_inputs_in_place_ms_per_step": wall_gi / n_tr * 1e3,
            "with_bullet_read_ms_per_step": None if wall_tb is None else wall_tb / n_tr * 1e3,
            "steps": n_tr, "eager_torch_ms_per_step": wall_te / n_tr * 1e3, "speedup_over_eager_torch": wall_te / wall_tr,
            "what": "YemongTrunk.forward, 2 blocks x (2 attention + 1 temporal sublayer), d_model 128, packed fp32 state "
                    "carried, " + ("bf16 autocast" if bf16 else "fp32") + "; with_bullet_read = the shipped default, whose first "
                    "attention sublayer of each block also reads the bullets in flight (10 slots per ship, 25 % live); eager = same modules with the kernels "
                    "replaced by the reference's torch ops and its unpack/cat/re-pack of the state",
        }
        del trunk, hid, ref_h

    # free the device before the host leg
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(w, p, args.cpu_seconds)
    else:
        result["cpu_baseline"] = None

    # the figures a reader of the last few hundred characters of the line needs
    trunk_leg = result.get("trunk") or {}
    result["summary"] = {
        "value": result["value"], "ms_per_step": result["ms_per_step"], "roofline_frac": result["roofline"]["frac"],
        "roofline_step_frac": result["roofline_step"]["frac"], "vs_torch_gpu_baseline": result.get("vs_torch_gpu_baseline"),
        "trunk_ms_per_step": trunk_leg.get("ms_per_step"),
        "trunk_with_bullet_read_ms_per_step": trunk_leg.get("with_bullet_read_ms_per_step"),
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
