#!/usr/bin/env python3
"""Benchmark of the MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c5|c4|c3|c1] [--no-cpu] [--no-secondary]

A step is one infmoe_enqueue over one batch of synthetic input that is already resident in
HBM.  The default workload is the configuration the headline metric is quoted on: cpm_2,
E=32, d=4096, h=10240, FP32, 4096 tokens, all experts resident.  One JSON line is printed:
whole-layer tokens/s, the roofline of the dominant kernel (measured with HIP events on the
stream the kernels run on) and the C/OpenMP restatement of the same math timed on the host
cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense FP32 matrix
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
PCIE_PEAK_GBS = 64.0           # host link, PCIe Gen5 x16, one direction
# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this
# benchmark scaled by what the same counters read for the row-copy kernels of known size
# (profiles/c2_expert_gemm_grouped_kernel_stats.txt, profiles/c5_expert_skinny_kernel_stats.txt,
# profiles/c4_expert_gemm_grouped_kernel_stats.txt;
# counters cannot be read from inside a run).  Kept as the ratio counter bytes / algorithmic bytes of the
# profiled launches (c2: 5.77 GB on average over the two launches against 5.60 GB of weights and
# activations; c5: 4.03 GB against 4.03 GB of weights of 24 active experts; c4: 7.90 GB against 4.97 GB, the
# weights of an expert with more than 256 rows being fetched once per row tile) and applied to the
# algorithmic bytes of the run at hand, whose number of active experts may differ.
MEASURED_TRAFFIC_RATIO = {"c2": 5.77 / 5.60, "c5": 4.03 / 4.03, "c4": 7.90 / 4.97}

CONFIGS = {
    # name: variant, E, d, h, mc, (B, S), zipf
    "c1": dict(variant="default", E=4, d=64, h=256, mc=2, shape=(2, 16), zipf=False),
    "c2": dict(variant="cpm_2", E=32, d=4096, h=10240, mc=32, shape=(8, 512), zipf=False),
    "c3": dict(variant="cpm_2", E=32, d=4096, h=10240, mc=2, shape=(8, 512), zipf=False),
    "c4": dict(variant="base_layer", E=64, d=2048, h=8192, mc=64, shape=(16, 1024), zipf=True),
    "c5": dict(variant="cpm_2", E=32, d=4096, h=10240, mc=32, shape=(64, 1), zipf=False),
    # the reference's own example (python/examples/stacked_moe.py:23-27): three stacked layers that share one
    # sub-layer, 80 x 512 tokens, experts streamed through four slots
    "ex": dict(variant="cpm_2", E=20, d=4096, h=16384, mc=4, shape=(80, 512), zipf=False, layers=3),
}


def zipf_score_bias(x, centroids, s=1.2, iters=30):
    """Input synthesis for the skewed workload: a per-expert additive score bias such that the
    top-1 counts follow p_e ~ (e+1)^-s (fixed-point iteration on the host; not a reference attribute)."""
    aff = np.asarray(x, np.float64) @ np.asarray(centroids, np.float64).T
    T, E = aff.shape
    target = np.arange(1, E + 1) ** (-float(s))
    target = target / target.sum()
    bias = np.zeros(E)
    for _ in range(iters):
        p = np.bincount(np.argmax(aff + bias, axis=1), minlength=E) / T
        bias += 0.5 * (np.log(target) - np.log(np.maximum(p, 0.5 / T)))
    return bias.astype(np.float32)


def build_layer(torch, cfg, seed=0, keep_host=True, replicate=False):
    """Synthetic tensors drawn on the GPU (fixed seed), expert weights handed to the library by
    host pointer, as a caller holding an npz in memory would."""
    from infmoe_amd import MoELayerConfig, MoELayerPlugin
    E, d, h = cfg["E"], cfg["d"], cfg["h"]
    B, S = cfg["shape"]
    T = B * S
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    x = torch.randn(T, d, generator=gen, device="cuda")
    cent = (torch.randn(d, E, generator=gen, device="cuda") / d ** 0.5).t().contiguous()  # logical [d,E] -> [E][d]
    gamma = 1 + 0.1 * torch.randn(d, generator=gen, device="cuda")
    gated = cfg.get("ffn", "relu") == "gated_gelu"
    mcfg = MoELayerConfig(seq_len=S, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=cfg["mc"],
                          moe_variant=cfg["variant"], sublayer_type="T5_FF", max_batch_size=B,
                          ffn_kind=cfg.get("ffn", "relu"),
                          expert_centroids=cent.cpu().numpy(),
                          layernorm_weight=gamma.cpu().numpy() if cfg["variant"] == "cpm_2" else None)
    plugin = MoELayerPlugin(mcfg).create_plugin()
    slots = []
    # [gamma | wi [h][d] | wo [d][h]], or [gamma | wi_0 | wi_1 | wo] for the gated form
    inner = ("wi_0_weight", "wi_1_weight") if gated else ("wi_weight",)
    slot_floats = d + (len(inner) + 1) * d * h

    def hand_over(e, base):
        plugin.set_expert_weights_ptr(e, "layer_norm_weight", base, d)
        for i, name in enumerate(inner):
            plugin.set_expert_weights_ptr(e, name, base + 4 * (d + i * d * h), d * h)
        plugin.set_expert_weights_ptr(e, "wo_weight", base + 4 * (d + len(inner) * d * h), d * h)

    for e in range(E):
        if replicate and e > 0:  # profiling runs: every expert gets expert 0's values (same work, short set-up)
            hand_over(e, slots[0].ctypes.data if keep_host else slot.ctypes.data)
            if keep_host:
                slots.append(slots[0])
            continue
        slot = np.empty(slot_floats, np.float32)
        slot[:d] = (1 + 0.1 * torch.randn(d, generator=gen, device="cuda")).cpu().numpy()
        for i in range(len(inner)):
            slot[d + i * d * h:d + (i + 1) * d * h] = (torch.randn(h, d, generator=gen, device="cuda") / d ** 0.5).cpu().numpy().ravel()
        slot[d + len(inner) * d * h:] = (torch.randn(d, h, generator=gen, device="cuda") / h ** 0.5).cpu().numpy().ravel()
        hand_over(e, slot.ctypes.data)
        if keep_host:
            slots.append(slot)
    bias = None
    if cfg["zipf"]:
        bias = zipf_score_bias(x.cpu().numpy(), cent.cpu().numpy(), s=1.2)
        plugin.set_score_bias(bias)
    plugin.configure([B, S, d])
    plugin.initialize()
    return plugin, x.view(B, S, d), cent, gamma, slots, bias


def cpu_baseline(cfg, x, cent, gamma, slots, bias, sample_tokens):
    """C/OpenMP restatement (oracle/moe_cpu.c) on the first `sample_tokens` tokens of the batch."""
    from oracle import moe_cpu
    xs = x.reshape(-1, cfg["d"])[:sample_tokens].cpu().numpy()
    c = cent.cpu().numpy()
    g = gamma.cpu().numpy() if cfg["variant"] == "cpm_2" else None
    cores = moe_cpu.load().moe_cpu_threads()
    moe_cpu.layer(xs[:64], c, cfg["variant"], slots, gamma=g, bias=bias, h=cfg["h"])  # warm the pages
    # repeat the pass until about ten seconds of CPU work are on the clock (at most 50 passes)
    passes, t0 = 0, time.perf_counter()
    while True:
        moe_cpu.layer(xs, c, cfg["variant"], slots, gamma=g, bias=bias, h=cfg["h"])
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= 10.0 or passes >= 50:
            break
    return {"value": round(passes * xs.shape[0] / dt, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"first {xs.shape[0]} tokens of the batch through all {cfg['E']} experts, {passes} passes, "
                      f"oracle/moe_cpu.c (FP32, OpenMP, AVX2), {dt:.2f} s"}


def measure(torch, plugin, cfg, name, x, steps, warmup, gated=False, stack=None):
    """W untimed steps, then K timed ones between two events on the layer's stream, with the library's phase
    marks (HIP events on the same stream) kept for exactly those K steps."""
    n_mat = 3 if gated else 2  # weight matrices of an expert
    E, d, h = cfg["E"], cfg["d"], cfg["h"]
    B, S = x.shape[0], x.shape[1]
    T = B * S
    dims = [B, S, d]
    ws = torch.empty(plugin.workspace_size(dims), dtype=torch.uint8, device="cuda")
    y = torch.empty_like(x)
    stream = torch.cuda.current_stream().cuda_stream

    if stack:  # layers that share the sub-layer, each fed with its predecessor's output; one workspace for all
        bufs = [x, y, torch.empty_like(x)]

        def step():
            for i, layer in enumerate(stack):
                layer.enqueue(dims, bufs[i % 3].data_ptr(), bufs[(i + 1) % 3].data_ptr(), ws.data_ptr(), stream)
    else:
        def step():
            plugin.enqueue(dims, x.data_ptr(), y.data_ptr(), ws.data_ptr(), stream)

    plugin.set_timing(steps)  # HIP events at the phase boundaries, kept for every step of the timed region
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t_wall = time.perf_counter()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        step()
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t_wall) * 1e3 / steps
    ms_per_step = start.elapsed_time(end) / steps
    # per-phase averages over exactly the steps of the timed region (events recorded on the layer's stream)
    phase_runs = plugin.timing_history(steps)
    assert len(phase_runs) == steps
    last = phase_runs[-1]
    phases = {k: float(np.mean([p[k] for p in phase_runs])) for k in phase_runs[0]}
    count, stats = plugin.last_routing()
    active = int((count > 0).sum())

    resident = cfg["mc"] >= E
    few_rows = T <= 16 * E  # same rule the sub-layer uses to pick the few-row kernels
    # average launch of the two expert kernels; the gated form's first launch takes two matrices, so its
    # figures are per matrix: (time of both launches) / 3
    gemm_ms = (phases["expert_gemm1"] + phases["expert_gemm2"]) / n_mat
    launches = ("two launches per step: wi_0 and wi_1 with gelu*mul, wo with residual; figures per weight matrix"
                if gated else "two launches per step: wi with ReLU, wo with residual")
    copies = plugin.last_streaming()[0] if not resident else 0
    if not resident and copies > 0:
        # streamed experts: the host link bounds the call, not HBM and not the matrix core (experts still in a
        # slot from the call before are not copied again)
        bytes_per_call = copies * 4.0 * (d + n_mat * d * h)
        roofline = {"bound": "pcie", "achieved": round(bytes_per_call / (phases["expert_gemm1"] * 1e-3) / 1e9, 2),
                    "peak": PCIE_PEAK_GBS, "unit": "GB/s", "traffic": None,
                    "kernel": f"host-to-device copies of {copies} of {active} active experts overlapped with expert kernels",
                    "note": "bounded by the host link (PCIe Gen5 x16, 64 GB/s per direction): achieved = streamed weight "
                            "bytes / expert-loop time"}
    elif few_rows:
        bytes_per_launch = active * 4.0 * d * h  # one weight matrix per launch; activations are negligible
        roofline = {"bound": "hbm", "achieved": round(bytes_per_launch / (gemm_ms * 1e-3) / 1e9, 2),
                    "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "traffic": None if gated or name not in MEASURED_TRAFFIC_RATIO
                    else round(MEASURED_TRAFFIC_RATIO[name] * bytes_per_launch),
                    "kernel": f"expert_skinny_kernel ({launches})",
                    "algorithmic_bytes_per_launch": bytes_per_launch, "avg_launch_ms": round(gemm_ms, 4)}
    else:
        flops_per_launch = 2.0 * T * d * h
        roofline = {"bound": "mfma", "achieved": round(flops_per_launch / (gemm_ms * 1e-3) / 1e12, 3),
                    "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "traffic": None if gated or name not in MEASURED_TRAFFIC_RATIO
                    else round(MEASURED_TRAFFIC_RATIO[name] * 4.0 * (E * d * h + T * d + T * h)),
                    "kernel": f"expert_gemm_grouped_kernel ({launches})",
                    "algorithmic_flops_per_launch": flops_per_launch, "avg_launch_ms": round(gemm_ms, 4)}
    roofline["frac"] = round(roofline["achieved"] / roofline["peak"], 4)

    # (with the rms norm of every workload here the expert norm is no phase of its own: it rides on the first
    # expert product)
    # the bandwidth-bound phases: algorithmic bytes / phase time (the phase times include the launch
    # gaps and the event marks, a few microseconds each), against the HBM peak
    cpm2 = cfg["variant"] == "cpm_2"
    mix = cfg["variant"] == "base_layer"
    phase_bytes = {
        "gating": 4.0 * (T * d + E * d + (d if cpm2 else 0) + 2 * T),
        "scatter": 4.0 * (2 * T * d + T + 2 * T + (2 * T if mix else 0)),  # rows, pos, row statistics, coefficients
        "gather": 4.0 * ((3 * T * d + 2 * T) if mix else (2 * T * d + T)),
    }
    phase_rates = {k: {"bytes": v, "GB/s": round(v / (phases[k] * 1e-3) / 1e9, 1),
                       "frac_of_hbm_peak": round(v / (phases[k] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
                   for k, v in phase_bytes.items() if phases.get(k, 0) > 0}
    return dict(ms_per_step=ms_per_step, wall_ms=wall_ms, phases=phases, last=last, count=count, stats=stats,
                active=active, resident=resident, roofline=roofline, phase_rates=phase_rates, tokens=T)


def secondary_line(m, cfg, name):
    """What the headline line says of the primary workload, shortened, for a further workload of the same run."""
    return {"workload": f"{name}: {cfg['variant']} E={cfg['E']} d={cfg['d']} h={cfg['h']} tokens={m['tokens']}",
            "value": round(m["tokens"] / (m["ms_per_step"] * 1e-3), 1), "unit": "tokens/s",
            "ms_per_step": round(m["ms_per_step"], 4), "active_experts": m["active"],
            "tokens_per_expert_min_max": [int(m["count"].min()), int(m["count"].max())],
            "roofline": m["roofline"], "phases_ms": {k: round(v, 4) for k, v in m["phases"].items()},
            "phase_rates": m["phase_rates"]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-sample", type=int, default=4096)
    ap.add_argument("--ffn", default="relu", choices=["relu", "gated_gelu"],
                    help="relu: the two-matrix form the headline metric is quoted on; gated_gelu: the three-matrix "
                         "form (an extra measurement, without the CPU leg)")
    ap.add_argument("--sweep-tokens", default="",
                    help="comma-separated token counts: after the workload proper, the same layer is timed on that many "
                         "tokens of the batch each (e.g. 256,512,1024,2048 with c2: 8 to 64 rows per expert)")
    ap.add_argument("--mc", type=int, default=0, help="override the workload's max_concurrency")
    ap.add_argument("--no-secondary", action="store_true",
                    help="with the default workload: do not also measure the decode shape (c5) and the skewed one (c4)")
    ap.add_argument("--replicate-weights", action="store_true",
                    help="profiling aid: give every expert the values of expert 0 (short set-up, same work)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this layer runs on one GPU; --gpus above 1 is not supported "
                 "(no collectives are part of this build)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from infmoe_amd import capi
    capi.load()  # fails loudly when the HIP library has not been built

    cfg = dict(CONFIGS[args.config], ffn=args.ffn)
    if args.mc > 0:
        cfg["mc"] = args.mc
    gated = args.ffn == "gated_gelu"
    if gated:
        args.no_cpu = True
    n_mat = 3 if gated else 2  # weight matrices of an expert
    E, d, h = cfg["E"], cfg["d"], cfg["h"]
    B, S = cfg["shape"]
    T = B * S
    torch.cuda.set_device(0)
    plugin, x, cent, gamma, slots, bias = build_layer(torch, cfg, keep_host=not args.no_cpu,
                                                      replicate=args.replicate_weights)
    stack = None
    if cfg.get("layers", 1) > 1:  # clones share the sub-layer and so the host copy of the weights
        stack = [plugin]
        for _ in range(cfg["layers"] - 1):
            twin = plugin.clone()
            twin.configure([B, S, d])
            twin.initialize()
            stack.append(twin)
    m = measure(torch, plugin, cfg, args.config, x, args.steps, args.warmup, gated, stack=stack)
    count, stats, active, resident = m["count"], m["stats"], m["active"], m["resident"]
    ms_per_step, wall_ms, phases, last = m["ms_per_step"], m["wall_ms"], m["phases"], m["last"]
    roofline, phase_rates = m["roofline"], m["phase_rates"]

    out = {
        "metric": f"MoE-layer tokens/s (E={E},d={d},h={h},fp32)",
        "value": round(T / (ms_per_step * 1e-3), 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic" + (" (expert 0 replicated)" if args.replicate_weights else ""),
        "config": {"workload": f"{args.config}: {cfg['variant']} E={E} d={d} h={h} tokens={T} ({B}x{S}) "
                               f"max_concurrency={cfg['mc']} ({'resident' if resident else 'streamed'} experts), "
                               f"T5_FF rms norm + {'gated gelu (three matrices)' if gated else 'relu'}", "tokens": T, "active_experts": active,
                   "tokens_per_expert_min_max": [int(count.min()), int(count.max())]},
        "roofline": roofline,
        "phases_ms": {k: round(v, 4) for k, v in phases.items()},
        "phases_ms_last_timed_step": {k: round(v, 4) for k, v in last.items()},
        "phase_rates": phase_rates,
        "host_ms_per_step": round(wall_ms, 4),
        "routing": stats,
    }
    if stack:
        out["config"]["stacked_layers"] = len(stack)
        out["value"] = round(T / (ms_per_step * 1e-3), 1)  # tokens through the whole stack per second
    if not resident:
        copies, hits = plugin.last_streaming()
        out["streaming_last_call"] = {"experts_copied": copies, "experts_found_in_slots": hits}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, x, cent, gamma, slots, bias, min(args.cpu_sample, T))
    # Further workloads of the same run (the headline `value` above is untouched by them):
    #   c5, the decode shape: same layer (E, d, h as c2), 64 tokens of the same batch
    #   c4, the skewed base_layer workload: a layer of its own, built after the first is released
    secondary = {}
    if args.config == "c2" and not args.no_secondary and not gated:
        c5 = dict(CONFIGS["c5"], ffn=args.ffn)
        x5 = x.reshape(T, d)[:64].reshape(64, 1, d).contiguous()
        secondary["c5"] = secondary_line(measure(torch, plugin, c5, "c5", x5, max(args.steps, 50), args.warmup), c5, "c5")
    # Few to many rows per expert on the same layer: the expert kernels' achieved weight-byte rate (they are
    # bound by streaming the weights until an expert has some tens of rows) next to their flop rate
    if args.sweep_tokens:
        sweep = {}
        for n in [int(v) for v in args.sweep_tokens.split(",") if v]:
            xn = x.reshape(T, d)[:n].reshape(n, 1, d).contiguous()
            mm = measure(torch, plugin, cfg, None, xn, args.steps, args.warmup, gated)
            g_ms = (mm["phases"]["expert_gemm1"] + mm["phases"]["expert_gemm2"]) / n_mat
            sweep[str(n)] = {"ms_per_step": round(mm["ms_per_step"], 4), "tokens_per_s": round(n / (mm["ms_per_step"] * 1e-3), 1),
                             "active_experts": mm["active"], "rows_per_expert_min_max": [int(mm["count"].min()), int(mm["count"].max())],
                             "expert_launch_ms": round(g_ms, 4),
                             "weight_GBs": round(mm["active"] * 4.0 * d * h / (g_ms * 1e-3) / 1e9, 1),
                             "frac_of_hbm_peak": round(mm["active"] * 4.0 * d * h / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                             "TFLOPs": round(2.0 * n * d * h / (g_ms * 1e-3) / 1e12, 2),
                             "phases_ms": {k: round(v, 4) for k, v in mm["phases"].items()}}
        out["sweep_tokens"] = sweep
    plugin.terminate()
    plugin.destroy()
    del slots
    if args.config == "c2" and not args.no_secondary and not gated:
        try:
            c4 = dict(CONFIGS["c4"], ffn=args.ffn)
            p4, x4, *_ = build_layer(torch, c4, keep_host=False)
            secondary["c4"] = secondary_line(measure(torch, p4, c4, "c4", x4.contiguous(), args.steps, args.warmup), c4, "c4")
            p4.terminate()
        except Exception as exc:  # the headline line must not depend on the extras
            secondary["c4"] = {"error": repr(exc)}
    if secondary:
        out["secondary"] = secondary
    print(json.dumps(out))


if __name__ == "__main__":
    main()
