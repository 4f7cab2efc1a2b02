"""Benchmark of the CVMM hot path: one analog SigmaMoE layer, forward + backward, on one MI355X.

A step = one pass of the hot path over one batch of synthetic input already resident in HBM:
expert sort -> up-projection (DAC, K-tile split, noise, ADC, ReLU) -> down-projection ->
gate-weighted reduction, then the full backward (both weight gradients, both input gradients
with clip masks, input-range gradients, gate gradient).  Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3|c3_f16|c2|c2_f32|c4|c1|c5]

The default workload is BASELINE.json's 64-expert tile-split layer (configs[2]), the one its
metric's MFMA-peak target is quoted on.  Only one GPU is used; --gpus N > 1 exits.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

CONFIGS = {
    # T tokens, D d_model, E experts, F expert_size, k heads
    "c1": dict(T=256, D=128, E=8, F=64, k=2, dtype="f32", routing="router", mis=-1, noise=0.0,
               name="config1: d_model=128 E=8 F=64 k=2 256 tokens fp32"),
    "c2": dict(T=8192, D=412, E=16, F=128, k=4, dtype="bf16", routing="router", mis=-1, noise=0.04,
               name="config2: d_model=412 E=16 F=128 k=4 8192 tokens bf16"),
    "c2_f32": dict(T=8192, D=412, E=16, F=128, k=4, dtype="f32", routing="router", mis=-1, noise=0.04,
                   name="config2: d_model=412 E=16 F=128 k=4 8192 tokens fp32"),
    "c3": dict(T=16384, D=1024, E=64, F=256, k=8, dtype="bf16", routing="uniform", mis=512, noise=0.04,
               name="config3: d_model=1024 (2x512 tiles) E=64 F=256 k=8 16384 tokens bf16 uniform routing"),
    # the same layer when the experts' loads differ by a few percent (k consecutive experts from a random start per
    # token: 2048 +- 5 % rows per expert), as a router produces them: a check on the work split, not a headline
    "c3_near": dict(T=16384, D=1024, E=64, F=256, k=8, dtype="bf16", routing="near_uniform", mis=512, noise=0.04,
                    name="config3 with near-uniform routing (2048 +- 5 % rows per expert): d_model=1024 (2x512 tiles) "
                         "E=64 F=256 k=8 16384 tokens bf16"),
    "c3_f16": dict(T=16384, D=1024, E=64, F=256, k=8, dtype="f16", routing="uniform", mis=512, noise=0.04,
                   name="config3 in fp16 (the reference's reduced-precision type): d_model=1024 (2x512 tiles) E=64 "
                        "F=256 k=8 16384 tokens uniform routing"),
    "c4": dict(T=32768, D=2048, E=128, F=512, k=4, dtype="bf16", routing="zipf", mis=-1, noise=0.04,
               name="config4: d_model=2048 E=128 F=512 k=4 32768 tokens bf16 Zipf(1.2) routing"),
    # the layer inside its caller: a 16-layer decoder training step (attention and norms are stock PyTorch)
    "c5": dict(T=16384, D=1024, E=64, F=256, k=8, dtype="bf16", routing="router", mis=-1, noise=0.04,
               layers=16, heads=16, context=1024, batch=16, vocab=8000,
               name="config5: 16-layer SigmaMoE decoder training step, d_model=1024, 16 heads, 64 experts x 256, "
                    "k=8, context 1024, batch 16, vocab 8000, bf16"),
}
PEAK = {"bf16": 2.5e15, "f16": 2.5e15, "f32": 157.3e12}       # dense MFMA, MI355X
# roofline.traffic (HBM bytes of the dominant launch) comes from profiles/bench_<config>_hbm_traffic.json, written by
# bench_traffic.py from two rocprofv3 counter runs of this file; it is null when no such run is recorded or the
# kernel sources changed after it.


def cpu_baseline(cfg, pr, budget_tokens):
    """Per-expert eager-PyTorch layer (oracle/layer_cpu.py) on the host cores, fp32, on the first
    `budget_tokens` tokens of the same inputs; noise tensors are drawn inside the timed region."""
    import torch
    from oracle.layer_cpu import moe_layer_per_expert
    from oracle.cvmm_oracle import tile_bounds
    n = min(budget_tokens, cfg["T"])
    E, k, D, F = cfg["E"], cfg["k"], cfg["D"], cfg["F"]
    x = pr["x"][:n].float().cpu().requires_grad_()
    keys = pr["keys"].float().cpu().requires_grad_()
    values = pr["values"].float().cpu().requires_grad_()
    gate = pr["gate"][:n].float().cpu().requires_grad_()
    idx = pr["idx"][:n].cpu()
    dy = pr["dy"][:n].float().cpu()
    bu, bd = tile_bounds(D, cfg["mis"]), tile_bounds(F, cfg["mis"])
    ir = torch.full((2, E, max(len(bu), len(bd)) - 1), 3.0, requires_grad=True)

    def step():
        wu = keys.detach().abs().amax((1, 2)).reshape(E, 1)
        wd = values.detach().abs().amax((1, 2)).reshape(E, 1)
        nu = nd = None
        if cfg["noise"] > 0:
            flat = idx.reshape(-1)
            nu = torch.randn(len(bu) - 1, n * k, F) * cfg["noise"] * wu[flat]
            nd = torch.randn(len(bd) - 1, n * k, D) * cfg["noise"] * wd[flat]
        y = moe_layer_per_expert(x, keys, values, idx, gate, ir, inp_res=1 / 127, noise_up=nu, noise_down=nd,
                                 wmax_up=wu, wmax_down=wd, out_bound=12.0, out_res=254.0, bounds_up=bu,
                                 bounds_down=bd)
        y.backward(dy)
        for t in (x, keys, values, gate, ir):
            t.grad = None

    step()
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or (time.perf_counter() - t0 < 8.0 and reps < 20):
        step()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": n / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"first {n} of {cfg['T']} tokens, all {E} experts, fp32, {reps} iterations, "
                      f"{dt * 1e3:.1f} ms each"}


def bench_decoder(args, cfg):
    """Configuration 5: forward, loss, backward and optimizer step of a 16-layer SigmaMoE decoder whose
    feed-forward blocks are the analog layer.  Reports whole-step tokens/s and, from a second timing with the
    feed-forward blocks switched off, the share and the TFLOP/s of the MoE part."""
    import torch
    from torch import nn
    from analog_moe_amd import config as cfgmod, ops
    from analog_moe_amd.decoder import SigmaMoEDecoder
    from analog_moe_amd.moe_layer import AnalogSigmaMoELayer

    ops.get_lib()
    dev = torch.device("cuda:0")
    D, E, F, k = (cfg[n] for n in "DEFk")
    B, S, V, L = cfg["batch"], cfg["context"], cfg["vocab"], cfg["layers"]

    def rpu():
        r = cfgmod.TorchInferenceRPUConfig()
        r.forward.inp_res = r.forward.out_res = 2 ** 8 - 2
        r.forward.out_bound = 12.0
        r.forward.out_noise = cfg["noise"]
        r.pre_post.input_range.enable = True
        r.pre_post.input_range.learn_input_range = True
        r.pre_post.input_range.init_value = 3.0
        r.pre_post.input_range.decay = 0.01
        return r

    class NoFFN(nn.Module):
        def forward(self, x):
            return torch.zeros_like(x), x.new_zeros(())

    def build(with_moe):
        torch.manual_seed(0)
        make = (lambda i: AnalogSigmaMoELayer(rpu(), d_model=D, n_experts=E, expert_size=F, k=k)) if with_moe \
            else (lambda i: NoFFN())
        model = SigmaMoEDecoder(V, D, L, cfg["heads"], S, make).to(dev).to(torch.bfloat16)
        model.train()
        for blk in model.blocks:
            if with_moe:
                blk.ffn.use_device_noise_counter()
        return model

    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, V, (B, S), generator=g).to(dev)          # uniform random token ids
    labels = torch.roll(ids, -1, dims=1)

    def timed(model, graph):
        # capturable: the step count and the bias corrections live on the device, for eager launches as well
        opt = torch.optim.AdamW(model.parameters(), lr=1e-4, capturable=True, fused=True)

        def step():
            loss, _ = model(ids, labels, reg_weight=0.01)
            loss.backward()
            opt.step()
            model.post_update_step()
            return loss.detach()

        def eager_step():
            opt.zero_grad(set_to_none=True)
            return step()
        if not graph:
            run = eager_step
        else:
            # the whole step (forward, loss, backward, AdamW, weight clipping) captured once and replayed; the
            # gradients live in the graph's own memory pool, the noise seeds advance in device memory
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    eager_step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            opt.zero_grad(set_to_none=True)
            with torch.cuda.graph(g):
                captured_loss = step()

            def run():
                g.replay()
                return captured_loss
        for _ in range(args.warmup):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            last = run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3, float(last)

    ms_eager, loss_eager = timed(build(True), False)
    ms_rest, _ = timed(build(False), not args.no_graph)
    if args.no_graph:
        ms, loss = ms_eager, loss_eager
    else:
        ms, loss = timed(build(True), True)
    T = B * S
    moe_ms = ms - ms_rest
    moe_flops = L * 12.0 * T * k * D * F
    out = {
        "metric": "SigmaMoE decoder HWA training step tokens/sec on 1 GPU", "value": T / (ms * 1e-3),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "ms_per_step_eager": ms_eager, "launch": "eager" if args.no_graph else "hip graph replay",
        "config": {"workload": cfg["name"], "optimizer": "AdamW (fused, capturable)",
                   "analog": "learned input range 3.0, 8-bit DAC, 8-bit ADC (out_bound 12), output noise 0.04 x "
                             "max|W| drawn in-kernel; analog router"},
        "loss_after_last_step": loss, "loss_after_last_step_eager": loss_eager,
        "ms_per_step_without_ffn": ms_rest, "moe_part_ms": moe_ms, "moe_part_share": moe_ms / ms,
        "moe_part_tflops": moe_flops / (moe_ms * 1e-3) / 1e12,
        "moe_part_pct_of_mfma_peak": 100.0 * moe_flops / (moe_ms * 1e-3) / PEAK["bf16"],
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="c3", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=1024)
    ap.add_argument("--modifier", default="none",
                    help="weight modifier type of the training forward (e.g. add_normal_per_channel, "
                         "discretize_add_normal_per_channel); not part of the headline workload")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches instead of HIP-graph replays")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run one 256 MiB device copy first (reference reading for HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the single-GPU hot path only; run it with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from analog_moe_amd import config as cfgmod, ops
    from analog_moe_amd.moe_layer import AnalogSigmaMoELayer
    from analog_moe_amd.synthetic import make_problem

    cfg = CONFIGS[args.config]
    if "layers" in cfg:
        return bench_decoder(args, cfg)
    ops.get_lib()
    dev = torch.device("cuda:0")
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[cfg["dtype"]]
    T, D, E, F, k = (cfg[n] for n in "TDEFk")

    rpu = cfgmod.TorchInferenceRPUConfig()
    rpu.forward.inp_res = 2 ** 8 - 2
    rpu.forward.out_res = 2 ** 8 - 2
    rpu.forward.out_bound = 12.0
    rpu.forward.out_noise = cfg["noise"]
    rpu.mapping.max_input_size = cfg["mis"]
    rpu.pre_post.input_range.enable = True
    rpu.pre_post.input_range.learn_input_range = True
    rpu.pre_post.input_range.init_value = 3.0
    rpu.pre_post.input_range.decay = 0.01
    if args.modifier.lower() != "none":
        rpu.modifier.type = cfgmod.WeightModifierType[args.modifier.upper()]
        rpu.modifier.std_dev, rpu.modifier.res = 0.02, 2 ** 8 - 2
    torch.manual_seed(0)
    layer = AnalogSigmaMoELayer(rpu, d_model=D, n_experts=E, expert_size=F, k=k).to(dev).to(tdt)
    layer.train()
    pr = make_problem(0, T, D, E, F, k, dtype=tdt, routing=cfg["routing"])
    with torch.no_grad():
        layer.keys.copy_(pr["keys"])
        layer.values.copy_(pr["values"])
    x = pr["x"].to(dev).requires_grad_()
    gate = pr["gate"].to(dev).requires_grad_()
    idx = pr["idx"].to(dev)
    dy = pr["dy"].to(dev)
    params = [layer.keys, layer.values, layer.input_range, x, gate]

    layer.use_device_noise_counter()        # per-step noise seed in device memory: graph replays draw new noise

    def step():
        y = layer.forward_selected(x, gate, idx)
        y.backward(dy)
        for p in params:
            p.grad = None

    # HIP events around every launch, on the stream the kernels are launched on; a launch is named
    # by its op and its position among that op's calls within one step
    ROLES = {"cvmm_fwd": ["fwd_up (up-projection forward)", "fwd_down (down-projection forward)"],
             "cvmm_bwd_w": ["wgrad_down (weight gradient of the down-projection)",
                            "wgrad_up (weight gradient of the up-projection)"],
             "cvmm_bwd_x": ["xgrad_down (input gradient of the down-projection)",
                            "xgrad_up (input gradient of the up-projection)"]}
    events = {}
    counter = {}

    def timed(name):
        fn = getattr(ops, name)

        def wrapper(*a, **kw):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            r = fn(*a, **kw)
            e.record()
            i = counter.get(name, 0)
            counter[name] = i + 1
            roles = ROLES.get(name)
            key = roles[i % len(roles)] if roles else name
            events.setdefault(key, []).append((s, e))
            return r
        return fn, wrapper

    if args.copy_calibration:
        # a plain device copy of known size: the scale for FETCH_SIZE / WRITE_SIZE readings of this run
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # pass 1 (eager): HIP events around every launch give the per-launch durations.  Every step starts behind a
    # spin kernel of about 2 ms, so that the host has issued the whole step before the GPU begins it: an event
    # pair then brackets the launch's time on the GPU and not the host's time between two launches.
    spin = getattr(torch.cuda, "_sleep", None)
    spin_cycles = 0
    if spin is not None:
        spin(1000)                             # (loads the kernel: not part of the calibration)
        torch.cuda.synchronize()
        s0, e0 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s0.record()
        spin(1_000_000)
        e0.record()
        torch.cuda.synchronize()
        spin_cycles = int(2.0 / max(s0.elapsed_time(e0), 1e-3) * 1_000_000)
    saved = {}
    for name in ("cvmm_fwd", "cvmm_bwd_w", "cvmm_bwd_x", "prepare_sel", "gate_reduce", "gate_grad", "ksum",
                 "ksum_clip", "weight_abs_max", "weight_abs_max_pair", "segment_sum", "gate_reduce_codes",
                 "gate_grad_codes"):
        saved[name], w = timed(name)
        setattr(ops, name, w)
    torch.cuda.synchronize()
    for _ in range(args.steps):
        if spin_cycles:
            spin(spin_cycles)
        step()
    torch.cuda.synchronize()
    for name, fn in saved.items():
        setattr(ops, name, fn)
    # the same steps without events and spin kernels: the eager step time
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) / args.steps * 1e3

    # pass 2 (the headline): the same step captured once in a HIP graph and replayed; the launches
    # are then back to back on the GPU instead of waiting for the Python that issues them
    if args.no_graph:
        elapsed = eager_ms * 1e-3 * args.steps
    else:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0

    ms = elapsed / args.steps * 1e3
    M = T * k
    flops_step = 12.0 * M * D * F                 # six GEMM launches of 2*M*D*F
    kern = {n: sum(s.elapsed_time(e) for s, e in ev) / len(ev) for n, ev in events.items()}
    calls = {n: len(ev) // args.steps for n, ev in events.items()}
    per_step = {n: kern[n] * calls[n] for n in kern}
    gemms = [r for rs in ROLES.values() for r in rs if r in kern]
    # The dominant kernel is the GEMM kernel with the most time per step.  The two weight-gradient launches run one
    # kernel (a kernel trace lists them as one line with one average), so they count together and the figure is the
    # average over both; the forward and input-gradient launches may be different kernels and count alone.
    groups = {r: [r] for r in gemms if r not in ROLES["cvmm_bwd_w"]}
    wg = [r for r in ROLES["cvmm_bwd_w"] if r in kern]
    if wg:
        groups["wgrad (both weight-gradient launches, one kernel)"] = wg
    dom = max(groups, key=lambda g: sum(kern[r] for r in groups[g]))
    dom_ms = sum(kern[r] for r in groups[dom]) / len(groups[dom])       # average launch duration of that kernel
    gemm_flops = 2.0 * M * D * F                  # algorithmic flops of one launch of any of them
    achieved = gemm_flops / (dom_ms * 1e-3)
    peak = PEAK[cfg["dtype"]]
    from bench_traffic import load_traffic
    recorded, traffic_note = load_traffic(args.config)
    traffic = None
    if recorded is not None and all(r.split(" ")[0] in recorded for r in groups[dom]):
        traffic = sum(recorded[r.split(" ")[0]] for r in groups[dom]) / len(groups[dom])
    out = {
        "metric": "analog MoE layer fwd+bwd tokens/sec on 1 GPU; % of MFMA peak TFLOP/s",
        "value": T / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "ms_per_step_eager": eager_ms, "launch": "eager" if args.no_graph else "hip graph replay",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg["dtype"], "data": "synthetic",
        "config": {"workload": cfg["name"], "tokens": T, "d_model": D, "n_experts": E, "expert_size": F,
                   "top_k": k, "analog": "learned input range 3.0, 8-bit DAC, 8-bit ADC (out_bound 12), "
                   f"output noise {cfg['noise']} x max|W| drawn in-kernel, max_input_size {cfg['mis']}"
                   + ("" if args.modifier.lower() == "none" else f", weight modifier {args.modifier.lower()} "
                      "(std_dev 0.02, 254 states)")},
        "tflops": flops_step / (ms * 1e-3) / 1e12,
        "pct_of_mfma_peak": 100.0 * flops_step / (ms * 1e-3) / peak,
        "roofline": {"bound": "mfma", "kernel": dom,
                     "achieved": achieved / 1e12, "peak": peak / 1e12, "unit": "TFLOP/s",
                     "frac": achieved / peak, "traffic": traffic,
                     "flops_per_launch": gemm_flops, "avg_launch_ms": dom_ms, "launches_per_step": len(groups[dom]),
                     **({} if traffic_note is None else {"traffic_note": traffic_note})},
        # every launch of the step together, against the memory system: recorded HBM bytes per step over the step time
        **({} if recorded is None or not recorded.get("step_total") else
           {"step_hbm": {"bytes_per_step": recorded["step_total"], "achieved_GBps": recorded["step_total"] / ms / 1e6,
                         "peak_GBps": 8000.0, "frac": recorded["step_total"] / ms / 1e6 / 8000.0}}),
        "launch_ms": {n: round(v, 4) for n, v in sorted(kern.items(), key=lambda kv: -kv[1])},
        "gemm_frac_of_peak": {n.split(" ")[0]: round(gemm_flops / (kern[n] * 1e-3) / peak, 4) for n in gemms},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, pr, args.cpu_tokens)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
