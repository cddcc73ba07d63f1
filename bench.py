#!/usr/bin/env python3
"""Benchmark of the MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2|c5|c4|c3|c1|ex] [--no-cpu] [--no-secondary]

A step is one infmoe_enqueue over one batch of synthetic input that is already resident in
HBM.  The default workload is the configuration the headline metric is quoted on: cpm_2,
E=32, d=4096, h=10240, FP32, 4096 tokens, all experts resident.  One JSON line is printed:
whole-layer tokens/s (median of the K per-step times, taken with the library's phase marks switched
off), the roofline of the dominant kernel (from a second pass of K steps with the phase marks on: HIP
events on the stream the kernels run on) and the C/OpenMP restatement of the same math timed on the
host cores on a bounded sample of the same workload.  Under "secondary" the same line carries the
other regimes of the same run: the decode shape, the streamed configuration with its overlap
efficiency, the skewed workload with the expert kernels' rate against rows per expert, a token sweep
between decode and prefill, and the vendor's batched FP32 GEMM on the uniform version of the same
problem next to the library's expert launches on a uniformly routed batch.
"""
from __future__ import annotations

import argparse
import concurrent.futures
import hashlib
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
# HBM bytes per launch of the dominant kernel cannot be counted from inside a run: they come from rocprofv3
# FETCH_SIZE / WRITE_SIZE runs of this benchmark, scaled by what the same counters read for the row-copy
# kernels of known size, and are kept as the ratio (counter bytes) / (algorithmic bytes) of the profiled
# launches, applied to the algorithmic bytes of the run at hand (whose number of active experts may differ).
# Each entry names the summary it was taken from and the digest of the kernel source that summary was
# collected with; the JSON line repeats both next to the digest of the source as it is now, so that a
# figure that has outlived its kernel shows as stale.
KERNEL_SOURCES = {
    "gemm": ("infmoe_amd/csrc/kernels/expert_gemm_tile.h", "infmoe_amd/csrc/kernels/expert_gemm.hip",
             "infmoe_amd/csrc/kernels/dispatch.hip"),
    "skinny": ("infmoe_amd/csrc/kernels/expert_skinny.hip",),
}
MEASURED_TRAFFIC = {
    # c2: 5.73 GB (mean of the two launches, fetched + written) against 5.60 GB of weights, rows and hidden rows
    "c2": dict(ratio=5.726 / 5.604, kernel="gemm", source="profiles/c2_expert_gemm_grouped_kernel_stats.txt",
               source_digest="b1d327d74c73"),
    # c5: 4.70 GB against 4.70 GB of weights of the 28 active experts
    "c5": dict(ratio=4.698 / 4.698, kernel="skinny", source="profiles/c5_expert_skinny_kernel_stats.txt",
               source_digest="977acad6e33c"),
    # c4: 6.82 GB against 4.97 GB: the weights of an expert with several row tiles are fetched more than once
    "c4": dict(ratio=6.820 / 4.966, kernel="gemm", source="profiles/c4_expert_gemm_grouped_kernel_stats.txt",
               source_digest="b1d327d74c73"),
}

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


def source_digest(kind):
    hsh = hashlib.sha256()
    for rel in KERNEL_SOURCES[kind]:
        with open(os.path.join(ROOT, rel), "rb") as f:
            hsh.update(f.read())
    return hsh.hexdigest()[:12]


def traffic_of(name, algorithmic_bytes):
    """(bytes, provenance) of the dominant kernel's HBM traffic per launch, or (None, None)."""
    t = MEASURED_TRAFFIC.get(name)
    if t is None:
        return None, None
    now = source_digest(t["kernel"])
    return round(t["ratio"] * algorithmic_bytes), {
        "ratio_counter_over_algorithmic": round(t["ratio"], 4), "from": t["source"],
        "kernel_source_digest_when_profiled": t["source_digest"], "kernel_source_digest_now": now,
        "stale": t["source_digest"] != now}


# ---------------------------------------------------------------- synthetic tensors
# numpy default_rng on a SeedSequence(0) child per tensor: tensors do not depend on the order they are drawn in
# and the experts can be generated side by side.  Matrices are drawn in their logical shape (centroids [d,E],
# wi [d,h], wo [h,d]) and handed over in the layout the layer takes them in ([E][d], [h][d], [d][h]).
def _rng(*key):
    return np.random.default_rng(np.random.SeedSequence(entropy=0, spawn_key=tuple(key)))


def _normal(key, shape, scale=1.0):
    a = _rng(*key).standard_normal(shape, dtype=np.float32)
    if scale != 1.0:
        a *= np.float32(scale)
    return a


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


def draw_slot(e, d, h, n_inner):
    """Packed weights of expert e: [gamma | wi [h][d] | wo [d][h]], or [gamma | wi_0 | wi_1 | wo]."""
    import torch  # (its blocked CPU transpose is ten times faster than numpy's strided copy)
    slot = np.empty(d + (n_inner + 1) * d * h, np.float32)
    slot[:d] = 1.0 + 0.1 * _normal((100 + e, 0), d)

    def put(dst, logical):
        torch.from_numpy(dst).copy_(torch.from_numpy(logical).t())

    for i in range(n_inner):
        put(slot[d + i * d * h:d + (i + 1) * d * h].reshape(h, d), _normal((100 + e, 1 + i), (d, h), d ** -0.5))
    put(slot[d + n_inner * d * h:].reshape(d, h), _normal((100 + e, 3), (h, d), h ** -0.5))
    return slot


def build_layer(torch, cfg, keep_host=True, replicate=False, slots=None):
    """Synthetic tensors (see above), uploaded once; expert weights handed to the library by host pointer, as a
    caller holding an npz in memory would.  `slots`: packed experts drawn earlier (a second layer over the same
    weights)."""
    from infmoe_amd import MoELayerConfig, MoELayerPlugin
    E, d, h = cfg["E"], cfg["d"], cfg["h"]
    B, S = cfg["shape"]
    T = B * S
    x = torch.from_numpy(_normal((0,), (T, d))).cuda()
    cent_host = np.ascontiguousarray(_normal((1,), (d, E), d ** -0.5).T)  # logical [d,E] -> [E][d]
    gamma_host = 1.0 + 0.1 * _normal((2,), d)
    gated = cfg.get("ffn", "relu") == "gated_gelu"
    mcfg = MoELayerConfig(seq_len=S, expert_count=E, embedding_size=d, hidden_size=h, max_concurrency=cfg["mc"],
                          moe_variant=cfg["variant"], sublayer_type="T5_FF", max_batch_size=B,
                          ffn_kind=cfg.get("ffn", "relu"), expert_centroids=cent_host,
                          layernorm_weight=gamma_host if cfg["variant"] == "cpm_2" else None)
    plugin = MoELayerPlugin(mcfg).create_plugin()
    inner = ("wi_0_weight", "wi_1_weight") if gated else ("wi_weight",)

    def hand_over(e, slot):
        base = slot.ctypes.data
        plugin.set_expert_weights_ptr(e, "layer_norm_weight", base, d)
        for i, name in enumerate(inner):
            plugin.set_expert_weights_ptr(e, name, base + 4 * (d + i * d * h), d * h)
        plugin.set_expert_weights_ptr(e, "wo_weight", base + 4 * (d + len(inner) * d * h), d * h)

    if slots is None:
        # profiling runs: every expert gets expert 0's values (same work, short set-up)
        todo = [0] if replicate else list(range(E))
        workers = min(len(todo), max(1, min(16, os.cpu_count() or 1)))
        kept = []
        with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
            # a few experts at a time, so that at most `workers` slots beyond the kept ones are alive
            for lo in range(0, len(todo), workers):
                drawn = list(pool.map(lambda e: draw_slot(e, d, h, len(inner)), todo[lo:lo + workers]))
                for e, slot in zip(todo[lo:lo + workers], drawn):
                    if replicate:
                        for ee in range(E):
                            hand_over(ee, slot)
                    else:
                        hand_over(e, slot)
                    if keep_host:
                        kept.append(slot)
        slots = kept * E if (replicate and keep_host) else kept
    else:
        for e in range(E):
            hand_over(e, slots[e])
    bias = None
    cent = torch.from_numpy(cent_host).cuda()
    gamma = torch.from_numpy(gamma_host).cuda()
    if cfg["zipf"]:
        bias = zipf_score_bias(x.cpu().numpy(), cent_host, s=1.2)
        plugin.set_score_bias(bias)
    plugin.configure([B, S, d])
    plugin.initialize()
    return plugin, x.view(B, S, d), cent, gamma, slots, bias


def uniform_batch(torch, cent, rows_per_expert, like_std=1.0, key=7):
    """A batch that the gating routes to exactly `rows_per_expert` tokens per expert (token t leans towards the
    centroid of expert t mod E), with the scale of the ordinary batch.  The caller checks the realised counts."""
    E, d = cent.shape
    T = E * rows_per_expert
    noise = torch.from_numpy(_normal((key,), (T, d))).cuda()
    xu = 50.0 * cent[torch.arange(T, device="cuda") % E] + 0.5 * noise
    return (xu * (like_std / xu.std())).contiguous()


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


def spin_up(torch, step, seconds=1.0):
    """Untimed steps until `seconds` of wall time have passed: a part that comes out of idle takes a second or two of
    load to settle its clocks (the reference's example stack ran 246, 239, 237 ms per step in three consecutive passes
    of six steps), and a short run would otherwise report the settling.  Returns the number of steps."""
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        step()
        torch.cuda.synchronize()
        n += 1
    return n


def time_steps(torch, step, steps, warmup):
    """W untimed steps, then K timed ones with an event between every two of them (on torch's current stream,
    which is the stream `step` queues on).  Returns (per-step ms [K], ms from first to last event / K, host ms / K)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t_wall = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        step()
        marks[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t_wall) * 1e3 / steps
    per_step = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
    return per_step, marks[0].elapsed_time(marks[steps]) / steps, wall_ms


def measure(torch, plugin, cfg, name, x, steps, warmup, gated=False, stack=None):
    """Two passes of W untimed + K timed steps.  The first runs with the library's phase marks off and gives the
    per-step times (`value` comes from their median); the second, of the same length, runs with the marks on (HIP
    events on the layer's stream at the phase boundaries, kept for exactly its K steps) and gives the phase times
    the roofline figures are computed from."""
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

    plugin.set_timing(0)
    settled = spin_up(torch, step)
    per_step, mean_ms, wall_ms = time_steps(torch, step, steps, warmup)
    plugin.set_timing(steps)
    marked_steps, marked_mean_ms, _ = time_steps(torch, step, steps, warmup)
    # per-phase averages over exactly the steps of the second pass
    phase_runs = plugin.timing_history(steps)
    plugin.set_timing(0)
    assert len(phase_runs) == steps
    last = phase_runs[-1]
    phases = {k: float(np.mean([p[k] for p in phase_runs])) for k in phase_runs[0]}
    count, stats = plugin.last_routing()
    active = int((count > 0).sum())

    resident = cfg["mc"] >= E
    # which roofline bounds the expert launches: streaming the active experts' weights at the HBM peak, or the
    # flops at the matrix peak, whichever takes longer; the kernel is named by the sub-layer's own rules
    hbm_bound = active * 4.0 * d * h / (HBM_PEAK_GBS * 1e9) > 2.0 * T * d * h / (MFMA_FP32_PEAK_TFLOPS * 1e12)
    tile_kernel = "expert_gemm_grouped_small_kernel" if (T <= 64 * E and not gated) else "expert_gemm_grouped_kernel"
    kernel_name = "expert_skinny_kernel" if T <= 2 * E else tile_kernel
    # average launch of the two expert kernels; the gated form's first launch takes two matrices, so its
    # figures are per matrix: (time of both launches) / 3
    gemm_ms = (phases["expert_gemm1"] + phases["expert_gemm2"]) / n_mat
    launches = ("two launches per step: wi_0 and wi_1 with gelu*mul, wo with residual; figures per weight matrix"
                if gated else "two launches per step: wi with ReLU, wo with residual")
    copies = plugin.last_streaming()[0] if not resident else 0
    provenance = None
    if not resident and copies > 0:
        # streamed experts: the host link bounds the call, not HBM and not the matrix core (experts still in a
        # slot from the call before are not copied again)
        bytes_per_call = copies * 4.0 * (d + n_mat * d * h)
        roofline = {"bound": "pcie", "achieved": round(bytes_per_call / (phases["expert_gemm1"] * 1e-3) / 1e9, 2),
                    "peak": PCIE_PEAK_GBS, "unit": "GB/s", "traffic": None,
                    "kernel": f"host-to-device copies of {copies} of {active} active experts overlapped with expert kernels",
                    "note": "bounded by the host link (PCIe Gen5 x16, 64 GB/s per direction): achieved = streamed weight "
                            "bytes / expert-loop time"}
    elif hbm_bound:
        bytes_per_launch = active * 4.0 * d * h  # one weight matrix per launch; activations are negligible
        traffic, provenance = (None, None) if gated else traffic_of(name, bytes_per_launch)
        roofline = {"bound": "hbm", "achieved": round(bytes_per_launch / (gemm_ms * 1e-3) / 1e9, 2),
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "traffic": traffic,
                    "kernel": f"{kernel_name} ({launches})",
                    "algorithmic_bytes_per_launch": bytes_per_launch, "avg_launch_ms": round(gemm_ms, 4)}
    else:
        flops_per_launch = 2.0 * T * d * h
        traffic, provenance = (None, None) if gated else traffic_of(name, 4.0 * (E * d * h + T * d + T * h))
        roofline = {"bound": "mfma", "achieved": round(flops_per_launch / (gemm_ms * 1e-3) / 1e12, 3),
                    "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "traffic": traffic,
                    "kernel": f"{kernel_name} ({launches})",
                    "algorithmic_flops_per_launch": flops_per_launch, "avg_launch_ms": round(gemm_ms, 4)}
    roofline["frac"] = round(roofline["achieved"] / roofline["peak"], 4)
    if provenance:
        roofline["traffic_provenance"] = provenance

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
    return dict(ms_per_step=float(np.median(per_step)), mean_ms=mean_ms, min_ms=float(np.min(per_step)),
                marked_ms=float(np.median(marked_steps)), settled=settled, wall_ms=wall_ms, phases=phases, last=last, count=count,
                stats=stats, active=active, resident=resident, roofline=roofline, phase_rates=phase_rates, tokens=T)


def secondary_line(m, cfg, name):
    """What the headline line says of the primary workload, shortened, for a further workload of the same run."""
    return {"workload": f"{name}: {cfg['variant']} E={cfg['E']} d={cfg['d']} h={cfg['h']} tokens={m['tokens']}",
            "value": round(m["tokens"] / (m["ms_per_step"] * 1e-3), 1), "unit": "tokens/s",
            "ms_per_step": round(m["ms_per_step"], 4), "ms_per_step_with_phase_marks": round(m["marked_ms"], 4),
            "active_experts": m["active"],
            "tokens_per_expert_min_max": [int(m["count"].min()), int(m["count"].max())],
            "roofline": m["roofline"], "phases_ms": {k: round(v, 4) for k, v in m["phases"].items()},
            "phase_rates": m["phase_rates"]}


def sweep_point(mm, n, d, h, n_mat):
    """One point of a sweep over rows per expert: the expert launches against both of their rooflines.  `attainable_ms`
    is what a launch cannot beat: the active experts' weight bytes at the HBM peak or its flops at the matrix peak,
    whichever takes longer."""
    g_ms = (mm["phases"]["expert_gemm1"] + mm["phases"]["expert_gemm2"]) / n_mat
    weight_bytes = mm["active"] * 4.0 * d * h
    flops = 2.0 * n * d * h
    attainable_ms = max(weight_bytes / (HBM_PEAK_GBS * 1e9), flops / (MFMA_FP32_PEAK_TFLOPS * 1e12)) * 1e3
    return {"ms_per_step": round(mm["ms_per_step"], 4), "tokens_per_s": round(n / (mm["ms_per_step"] * 1e-3), 1),
            "active_experts": mm["active"], "rows_per_expert_min_max": [int(mm["count"].min()), int(mm["count"].max())],
            "expert_launch_ms": round(g_ms, 4), "attainable_launch_ms": round(attainable_ms, 4),
            "frac_of_attainable": round(attainable_ms / g_ms, 4),
            "weight_GBs": round(weight_bytes / (g_ms * 1e-3) / 1e9, 1),
            "frac_of_hbm_peak": round(weight_bytes / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "TFLOPs": round(flops / (g_ms * 1e-3) / 1e12, 2),
            "frac_of_mfma_peak": round(flops / (g_ms * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4)}


def vendor_bmm(torch, E, rows, d, h, steps, warmup):
    """The vendor library's batched FP32 GEMM (torch.bmm) on the uniform version of the expert problem: E x
    [rows x d] . [h x d]^T and E x [rows x h] . [d x h]^T with Gaussian operands, weights K-contiguous as the
    layer stores them.  A comparator on the same box in the same run, not part of the product."""
    torch.backends.cuda.matmul.allow_tf32 = False
    out = {}
    for label, (N, K) in (("wi", (h, d)), ("wo", (d, h))):
        a = torch.from_numpy(_normal((50, N), (E, rows, K))).cuda()
        b = torch.from_numpy(_normal((51, N), (E, N, K), K ** -0.5)).cuda()
        bt = b.transpose(1, 2)
        c = torch.empty(E, rows, N, device="cuda")
        per_step, mean_ms, _ = time_steps(torch, lambda: torch.bmm(a, bt, out=c), steps, warmup)
        ms = float(np.median(per_step))
        out[label] = {"ms": round(ms, 4), "TFLOPs": round(2.0 * E * rows * N * K / (ms * 1e-3) / 1e12, 2)}
        del a, b, bt, c
    total_ms = out["wi"]["ms"] + out["wo"]["ms"]
    out["both"] = {"ms": round(total_ms, 4), "TFLOPs": round(4.0 * E * rows * d * h / (total_ms * 1e-3) / 1e12, 2)}
    out["what"] = f"torch.bmm fp32, {E} x [{rows} x K] . [N x K]^T for (N, K) = ({h}, {d}) and ({d}, {h}), Gaussian operands"
    return out


def h2d_rate(torch, nbytes, reps=5):
    """Bare rate of asynchronous host-to-device copies of `nbytes` from page-locked memory (GB/s)."""
    src = torch.empty(nbytes, dtype=torch.uint8, pin_memory=True)
    src.fill_(1)
    dst = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    per_step, _, _ = time_steps(torch, lambda: dst.copy_(src, non_blocking=True), reps, 2)
    return nbytes / (float(np.median(per_step)) * 1e-3) / 1e9


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
    ap.add_argument("--sweep-tokens", default=None,
                    help="comma-separated token counts: after the workload proper, the same layer is timed on that many "
                         "tokens of the batch each (default with c2: 256,512,1024,2048, i.e. 8 to 64 rows per expert; "
                         "'' for none)")
    ap.add_argument("--mc", type=int, default=0, help="override the workload's max_concurrency")
    ap.add_argument("--tokens", type=int, default=0,
                    help="run the workload on the first N tokens of its batch only (as one sequence per token), e.g. to "
                         "profile a point of the token sweep by itself")
    ap.add_argument("--no-secondary", action="store_true",
                    help="with the default workload: only the headline workload (no decode shape, streamed configuration, "
                         "skewed workload, sweeps or vendor comparator)")
    ap.add_argument("--legs", default="all",
                    help="with the default workload: which of the further workloads to run, comma-separated, of "
                         "c5,c2_uniform,vendor_bmm,sweep,c3,c4 (default all; e.g. c2_uniform,vendor_bmm to profile the two "
                         "side by side)")
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
    extras = args.config == "c2" and not args.no_secondary and not gated
    if args.sweep_tokens is None:
        args.sweep_tokens = "256,512,1024,2048" if extras else ""
    torch.cuda.set_device(0)
    # the host copies of the experts are kept for the CPU leg and for the streamed layer over the same weights
    keep_host = (not args.no_cpu) or (extras and not args.replicate_weights)
    plugin, x, cent, gamma, slots, bias = build_layer(torch, cfg, keep_host=keep_host, replicate=args.replicate_weights)
    stack = None
    if cfg.get("layers", 1) > 1:  # clones share the sub-layer and so the host copy of the weights
        stack = [plugin]
        for _ in range(cfg["layers"] - 1):
            twin = plugin.clone()
            twin.configure([B, S, d])
            twin.initialize()
            stack.append(twin)
    if 0 < args.tokens < T:
        x = x.reshape(T, d)[:args.tokens].reshape(args.tokens, 1, d).contiguous()
        B, S, T = args.tokens, 1, args.tokens
        extras = False
    m = measure(torch, plugin, cfg, args.config if not args.tokens else None, x, args.steps, args.warmup, gated, stack=stack)
    count, stats, active, resident = m["count"], m["stats"], m["active"], m["resident"]
    ms_per_step, phases, last = m["ms_per_step"], m["phases"], m["last"]
    roofline, phase_rates = m["roofline"], m["phase_rates"]

    out = {
        "metric": f"MoE-layer tokens/s (E={E},d={d},h={h},fp32)",
        "value": round(T / (ms_per_step * 1e-3), 1),  # tokens through the layer (the whole stack, if stacked) per second
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic: numpy default_rng on SeedSequence(0) children, one per tensor, uploaded once"
                + (" (expert 0's weights replicated to every expert)" if args.replicate_weights else ""),
        "config": {"workload": f"{args.config}: {cfg['variant']} E={E} d={d} h={h} tokens={T} ({B}x{S}) "
                               f"max_concurrency={cfg['mc']} ({'resident' if resident else 'streamed'} experts), "
                               f"T5_FF rms norm + {'gated gelu (three matrices)' if gated else 'relu'}", "tokens": T, "active_experts": active,
                   "tokens_per_expert_min_max": [int(count.min()), int(count.max())]},
        "timing": {"value_from": "median of the per-step times of a pass with the library's phase marks off",
                   "ms_per_step_mean": round(m["mean_ms"], 4), "ms_per_step_min": round(m["min_ms"], 4),
                   "ms_per_step_with_phase_marks": round(m["marked_ms"], 4),
                   "phases_from": "a second pass of the same length with the phase marks on",
                   "untimed_steps_before_the_warmup": m["settled"],
                   "why": "a second of load first, so that the part's clocks have settled when the W warm-up steps begin"},
        "roofline": roofline,
        "phases_ms": {k: round(v, 4) for k, v in phases.items()},
        "phases_ms_last_timed_step": {k: round(v, 4) for k, v in last.items()},
        "phase_rates": phase_rates,
        "host_ms_per_step": round(m["wall_ms"], 4),
        "routing": stats,
    }
    if stack:
        out["config"]["stacked_layers"] = len(stack)
    if not resident:
        copies, hits = plugin.last_streaming()
        out["streaming_last_call"] = {"experts_copied": copies, "experts_found_in_slots": hits}
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, x, cent, gamma, slots, bias, min(args.cpu_sample, T))

    # Further workloads of the same run (the headline `value` above is untouched by them).
    secondary = {}

    legs = None if args.legs == "all" else set(args.legs.split(","))

    def extra(key, fn):  # the headline line must not depend on the extras
        if legs is not None and key not in legs:
            return
        try:
            secondary[key] = fn()
        except Exception as exc:
            secondary[key] = {"error": repr(exc)}

    if extras:
        # c5, the decode shape: same layer (E, d, h as c2), 64 tokens of the same batch
        def leg_c5():
            c5 = dict(CONFIGS["c5"], ffn=args.ffn)
            x5 = x.reshape(T, d)[:64].reshape(64, 1, d).contiguous()
            return secondary_line(measure(torch, plugin, c5, "c5", x5, max(args.steps, 50), args.warmup), c5, "c5")
        extra("c5", leg_c5)

        # the same layer on a batch routed to exactly T/E rows per expert, and the vendor's batched GEMM on that
        # uniform problem: what separates the expert kernel from the best known code for the shape
        def leg_uniform():
            xu = uniform_batch(torch, cent, T // E, like_std=float(x.std())).view(B, S, d)
            mu = measure(torch, plugin, cfg, None, xu, args.steps, args.warmup)
            g1, g2 = mu["phases"]["expert_gemm1"], mu["phases"]["expert_gemm2"]
            fl = 2.0 * T * d * h
            return {"rows_per_expert_min_max": [int(mu["count"].min()), int(mu["count"].max())],
                    "ms_per_step": round(mu["ms_per_step"], 4),
                    "wi": {"ms": round(g1, 4), "TFLOPs": round(fl / (g1 * 1e-3) / 1e12, 2)},
                    "wo": {"ms": round(g2, 4), "TFLOPs": round(fl / (g2 * 1e-3) / 1e12, 2)},
                    "both": {"ms": round(g1 + g2, 4), "TFLOPs": round(2 * fl / ((g1 + g2) * 1e-3) / 1e12, 2)},
                    "what": "the library's two expert launches (norm + ReLU, residual epilogues included) on a batch the "
                            "gating routes uniformly"}
        extra("c2_uniform", leg_uniform)
        extra("vendor_bmm", lambda: vendor_bmm(torch, E, T // E, d, h, args.steps, args.warmup))

    # Few to many rows per expert on the same layer: the expert launches against what neither roofline lets
    # them beat (they are bound by streaming the weights until an expert has some tens of rows)
    if args.sweep_tokens:
        def leg_sweep():
            sweep = {}
            for n in [int(v) for v in args.sweep_tokens.split(",") if v]:
                xn = x.reshape(T, d)[:n].reshape(n, 1, d).contiguous()
                sweep[str(n)] = sweep_point(measure(torch, plugin, cfg, None, xn, args.steps, args.warmup, gated), n, d, h, n_mat)
            return sweep
        extra("sweep", leg_sweep)

    if extras:
        # c3: the same weights streamed through two slots (a second layer over the same host arrays), with the
        # overlap efficiency max(t_copy, t_compute) / t_total: t_compute is the resident layer's expert time of
        # this run, t_copy the streamed bytes at the bare rate of asynchronous copies of one slot
        def leg_c3():
            c3 = dict(CONFIGS["c3"], ffn=args.ffn)
            if not slots:
                raise RuntimeError("the streamed layer needs the host copies of the experts (not with --replicate-weights)")
            p3, x3, *_ = build_layer(torch, c3, keep_host=True, slots=slots)
            try:
                steps3 = min(args.steps, 10)
                m3 = measure(torch, p3, c3, "c3", x3, steps3, 2)
                copies, hits = p3.last_streaming()
                slot_bytes = 4 * (d + n_mat * d * h)
                bare = h2d_rate(torch, slot_bytes)
                t_copy = copies * slot_bytes / (bare * 1e9) * 1e3
                t_compute = phases["expert_gemm1"] + phases["expert_gemm2"]
                t_total = m3["ms_per_step"]
                line = secondary_line(m3, c3, "c3")
                line.update({"steps": steps3, "copies": copies, "hits": hits,
                             "h2d_GBs": round(copies * slot_bytes / (t_total * 1e-3) / 1e9, 2),
                             "bare_h2d_GBs_one_slot": round(bare, 2), "t_copy_ms": round(t_copy, 3),
                             "t_compute_ms": round(t_compute, 3), "t_total_ms": round(t_total, 3),
                             "overlap_efficiency": round(max(t_copy, t_compute) / t_total, 4)})
                return line
            finally:
                p3.terminate()
                p3.destroy()
        extra("c3", leg_c3)

    plugin.terminate()
    plugin.destroy()
    del slots
    if extras:
        # c4, the skewed base_layer workload: a layer of its own, built after the first is released; then the
        # same layer without the score bias on uniformly routed batches: the expert kernels' rate against rows
        # per expert (what an expert of each size of the skewed histogram gets)
        def leg_c4():
            c4 = dict(CONFIGS["c4"], ffn=args.ffn)
            p4, x4, cent4, *_ = build_layer(torch, c4, keep_host=False)
            try:
                m4 = measure(torch, p4, c4, "c4", x4.contiguous(), args.steps, args.warmup)
                line = secondary_line(m4, c4, "c4")
                line["tokens_per_expert"] = [int(v) for v in m4["count"]]
                p4.set_score_bias(None)
                table = {}
                for rows in (16, 32, 64, 128, 256, 512, 1024, 2048):
                    n = rows * c4["E"]
                    xu = uniform_batch(torch, cent4, rows, like_std=float(x4.std())).view(n, 1, c4["d"])
                    mu = measure(torch, p4, c4, None, xu, max(5, args.steps // 2), 2)
                    pt = sweep_point(mu, n, c4["d"], c4["h"], 2)
                    table[str(rows)] = {k: pt[k] for k in ("rows_per_expert_min_max", "expert_launch_ms", "TFLOPs",
                                                           "frac_of_mfma_peak", "frac_of_attainable")}
                line["expert_rate_vs_rows_per_expert"] = table
                return line
            finally:
                p4.terminate()
        extra("c4", leg_c4)
    if secondary:
        out["secondary"] = secondary
    print(json.dumps(out))


if __name__ == "__main__":
    main()
