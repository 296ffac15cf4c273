#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: a full MoE layer forward + backward at the Swin-MoE-S
stage-3 shape (T=18432 tokens, d=384, h=1536, 32 experts, top-2, bf16 with fp32 accumulation).

One step = hexa_moe.moe.MoE_Cascaded.forward on a MoE depth (gate projection, softmax, top-2, auxiliary
loss, the routing segment pass, fc1 ESMM with the fused GELU, fc2 ESMM) and the whole backward (2x ESS,
2x ESTMM, 2x backward ESMM, GELU', the gate's backward), with every input already resident in HBM.
Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
"""
import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "hexa-moe_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E peak

T, D, H, E, K_TOP = 18432, 384, 1536, 32, 2
SEED = 1235

# The six matmul launches of a step, in the order the library's event pairs number them: (direction, pair index).
# (In the backward the slot sum, the ESTMM fix-ups and the fold of the column sums run in batch launches of
# small tasks behind the matmul kernels, outside the event pairs.)
MAJOR = [("fc1_esmm+gelu", "fwd", 0), ("fc2_esmm+slot_sum", "fwd", 1), ("dy1_esmm+gelu'+colsum", "bwd", 0),
         ("dx_esmm", "bwd", 1), ("dW2_estmm", "bwd", 2), ("dW1_estmm", "bwd", 3)]
ROOFLINE_KERNEL = "fc1_esmm+gelu"   # fixed: the launch with the largest share of the step among equal-FLOP matmuls


def measured_traffic(label):
    """HBM bytes per launch (fetch + write) of a matmul launch, read from the `@traffic <label> <fetch_bytes>
    <write_bytes>` lines of profiles/*.hbm_traffic.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE passes scaled by a
    copy kernel of known size; the commands are in that file).  None when no profile covers the label."""
    import glob
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.hbm_traffic.txt"))):
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 4 and parts[0] == "@traffic" and parts[1] == label:
                    return float(parts[2]) + float(parts[3])
    return None


def make_module_and_inputs(dev, T=None, D=None, H=None, E=None, K_TOP=None, seed=None):
    """MoE_Cascaded with one MoE depth at the benchmark shape (or the shape given).  Expert parameters are bf16, the gate is
    fp32 (fp32_gate).  The uneven expert load of the recipe -- logits ~ N(0,1) plus a per-expert bias
    ~ N(0,0.5) -- is produced through the ordinary bias-free gate: feature 0 of every token is the
    constant 1 and column 0 of the gate weight holds the per-expert bias."""
    import torch
    import torch.nn.functional as F
    from hexa_moe import moe as hmoe
    gl = globals()
    T, D, H, E, K_TOP = (gl[n] if v is None else v for n, v in (("T", T), ("D", D), ("H", H), ("E", E), ("K_TOP", K_TOP)))
    g = torch.Generator().manual_seed(SEED if seed is None else seed)
    bf = torch.bfloat16
    u = lambda shape, bound: (torch.rand(shape, generator=g) * 2 - 1) * bound  # noqa: E731
    m = hmoe.MoE_Cascaded(gate_type={'type': 'top', 'k': K_TOP, 'gate_noise': 0.0, 'fp32_gate': True},
                          model_dim_list=[D], moe_idx_list=[0], mlp_ratio=H / D, num_global_experts=E, total_depth=1,
                          data_centric=True, mlp_fc1_bias=True, mlp_fc2_bias=True, activation_fn=F.gelu)
    with torch.no_grad():
        m.batched_fc1_w[0].copy_(u((E, H, D), 1 / math.sqrt(D)))
        m.batched_fc2_w[0].copy_(u((E, H, D), 1 / math.sqrt(H)))
        m.batched_fc1_bias[0].copy_(u((E, H), 1 / math.sqrt(D)))
        m.batched_fc2_bias[0].copy_(u((E, D), 1 / math.sqrt(H)))
        wg = torch.randn(E, D, generator=g) / math.sqrt(D - 1)
        wg[:, 0] = 0.5 * torch.randn(E, generator=g)
        m.gates[0].wg.weight.copy_(wg)
    m = m.to(dev)
    for plist in (m.batched_fc1_w, m.batched_fc2_w, m.batched_fc1_bias, m.batched_fc2_bias):
        for prm in plist:
            prm.data = prm.data.to(bf)
    x = torch.randn(T, D, generator=g)
    x[:, 0] = 1.0
    dy = torch.randn(T, D, generator=g)
    return m.train(), x.to(bf).to(dev).requires_grad_(True), dy.to(bf).to(dev)


def layer_bytes(T, D, H, E, K):
    """Algorithmic HBM bytes of one layer forward + backward (2-byte elements): every operand of the six matmul
    launches read once and every result written once -- fc1+GELU (x, W1, b1 -> y1, y2), fc2 (y2, W2, b2 -> y),
    dW2 (y2, dy -> dW2), dy1 (dy, W2, y1 -> dy1), dW1 (dy1, x -> dW1), dx (dy1, W1 -> dx)."""
    x, hid, w = T * D, T * K * H, E * H * D
    return 2.0 * ((x + w + E * H + 2 * hid) + (hid + w + E * D + x) + (hid + x + w) + (x + w + 2 * hid) + (hid + x + w) + (hid + w + x))


def time_loop(fn, steps, warmup):
    """(ms per call, host microseconds per call to enqueue it) of fn() over `steps` calls after `warmup`."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    host = time.perf_counter() - t0
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps, host * 1e6 / steps


def layer_config(dev, T, D, H, E, K, seed, steps, warmup):
    """A full MoE layer forward + backward at another shape, as the headline's step."""
    import torch
    m, x, dy = make_module_and_inputs(dev, T, D, H, E, K, seed)
    params = list(m.parameters())
    one = torch.ones((), device=dev)

    def step():
        x.grad = None
        for prm in params:
            prm.grad = None
        y, l_aux = m(0, x)
        torch.autograd.backward([y, l_aux], [dy, one])

    ms, host_us = time_loop(step, steps, warmup)
    # the same step as ONE graph launch (the library neither allocates nor synchronises, so the step captures): what the
    # GPU needs when the host's enqueue time (one Python call per operator of the surrounding autograd graph) is out
    # of the way -- at small shapes the eager loop above is bound by the host
    graph_ms = None
    try:
        x.grad = None
        for prm in params:
            prm.grad = None
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        x.grad = None
        for prm in params:
            prm.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y, l_aux = m(0, x)
            torch.autograd.backward([y, l_aux], [dy, one])
        graph_ms, _ = time_loop(graph.replay, steps, warmup)
    except Exception as e:   # noqa: BLE001  (a capture failure is reported, not fatal for the benchmark line)
        graph_ms = f"capture failed: {type(e).__name__}"
    counts = torch.bincount(m.dispatch_params.routing_.reshape(-1).long(), minlength=E)
    flop, nbytes = 12.0 * T * K * D * H, layer_bytes(T, D, H, E, K)
    return {"workload": f"MoE layer fwd+bwd T={T} d={D} h={H} E={E} top-{K} bf16", "ms": round(ms, 4),
            "tokens_per_s": round(T / (ms * 1e-3), 1), "tflops": round(flop / ms / 1e9, 1),
            "mfma_frac": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "algorithmic_bytes": nbytes,
            "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "host_enqueue_us": round(host_us, 1),
            "graph_replay_ms": round(graph_ms, 4) if isinstance(graph_ms, float) else graph_ms,
            "rows_per_expert": {"mean": round(T * K / E, 1), "min": int(counts.min()), "max": int(counts.max())},
            "steps": steps}


def operator_config(dev, name, steps, warmup):
    """The operator-level configurations: ESMM alone at the headline shape, and the skewed stress case
    (ESMM forward, ESTMM and ESS of the same routing)."""
    import torch
    from hexa_moe import _lib, ops
    bf = torch.bfloat16
    if name == "c2":
        T_, d, h, E_, k, seed = T, D, H, E, K_TOP, SEED
        g = torch.Generator().manual_seed(seed)
        logits = torch.randn(T_, E_, generator=g) + 0.5 * torch.randn(E_, generator=g)
        routing = torch.topk(torch.softmax(logits, 1), k, dim=1).indices
    else:   # c5: Zipf(1.2) ranks over a seeded expert permutation, four experts without tokens
        T_, d, h, E_, k, seed = 32768, 1024, 4096, 64, 2, 1238
        g = torch.Generator().manual_seed(seed)
        live = E_ - 4
        w = 1.0 / torch.arange(1, live + 1, dtype=torch.float64) ** 1.2
        perm = torch.randperm(E_, generator=g)[:live]
        first = torch.multinomial(w, T_, replacement=True, generator=g)
        second = torch.multinomial(w, T_, replacement=True, generator=g)
        second[second == first] = (second[second == first] + 1) % live
        routing = torch.stack([perm[first], perm[second]], 1)
    x = torch.randn(T_, d, generator=g).to(bf).to(dev)
    W = ((torch.rand(E_, d, h, generator=g) * 2 - 1) / math.sqrt(d)).to(bf).to(dev)
    b = ((torch.rand(E_, h, generator=g) * 2 - 1) / math.sqrt(d)).to(bf).to(dev)
    route = ops.route_build(routing.to(dev), E_)
    gemm = 2.0 * T_ * k * d * h
    out = {"workload": f"{'ESMM forward alone' if name == 'c2' else 'skewed stress: ESMM forward, ESTMM, ESS'} "
                       f"T={T_} d={d} h={h} E={E_} top-{k} bf16", "steps": steps}

    def entry(ms, host_us, flop, nbytes):
        e = {"ms": round(ms, 4), "host_enqueue_us": round(host_us, 1), "algorithmic_bytes": nbytes,
             "hbm_frac": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
        if flop:
            e.update(tflops=round(flop / ms / 1e9, 1), mfma_frac=round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4))
        return e

    y = torch.empty(k, T_, h, dtype=bf, device=dev)
    ms, host_us = time_loop(lambda: ops.esmm(x, W, b, route, False, _lib.HEXA_W_IN_OUT, out=y), steps, warmup)
    out["esmm"] = entry(ms, host_us, gemm, 2.0 * (T_ * d + E_ * d * h + E_ * h + T_ * k * h))
    if name == "c5":
        dy = torch.randn(k, T_, h, generator=g).to(bf).to(dev)
        ms, host_us = time_loop(lambda: ops.estmm(dy, x, route, True, False), steps, warmup)
        out["estmm"] = entry(ms, host_us, gemm, 2.0 * (T_ * k * h + T_ * d + E_ * d * h))
        ms, host_us = time_loop(lambda: ops.ess(dy, route, True), steps, warmup)
        out["ess"] = entry(ms, host_us, 0.0, 2.0 * T_ * k * h + 4.0 * E_ * h)
        counts = route.counts.sum(0)
        out["rows_per_expert"] = {"mean": round(T_ * k / E_, 1), "min": int(counts.min()), "max": int(counts.max())}
    return out


def swin_config(dev, steps, warmup):
    """Swin-MoE-S-shaped model, batch 64 of 192x192 images, bf16 autocast, forward + backward: images/s.  Attention,
    normalisation and the dense depths are stock PyTorch; the MoE depths (every other block of stages 3 and 4) run
    this library."""
    import torch
    import swin_moe_harness as S
    torch.manual_seed(1237)
    m = S.SwinMoE(num_experts=32, top_value=1, init_std=0.02).to(dev).train()
    images = torch.randn(64, 3, 192, 192, generator=torch.Generator().manual_seed(1237)).to(dev)

    def step():
        m.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            logits, l_aux = m(images)
            loss = logits.float().square().mean() + l_aux
        loss.backward()

    ms, host_us = time_loop(step, steps, warmup)
    return {"workload": "Swin-MoE-S-shaped fwd+bwd, 64 images 192x192, 32 experts top-1, bf16 autocast", "ms": round(ms, 3),
            "images_per_s": round(64 / (ms * 1e-3), 1), "host_enqueue_us": round(host_us, 1), "steps": steps}


OTHER = {
    "c2": lambda dev, n, w: operator_config(dev, "c2", n, w),
    "c3": lambda dev, n, w: layer_config(dev, 4608, 768, 3072, 32, 1, 1236, n, w),
    "stage4": lambda dev, n, w: layer_config(dev, 2304, 768, 3072, 32, 1, 1240, n, w),
    "short384": lambda dev, n, w: layer_config(dev, 2304, 384, 1536, 32, 1, 1241, n, w),   # 72 rows per expert at d = 384
    "c4": lambda dev, n, w: swin_config(dev, max(3, n // 4), 2),
    "c5": lambda dev, n, w: operator_config(dev, "c5", n, w),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-events", action="store_true")
    ap.add_argument("--other-configs", default="c2,c3,stage4,c5,c4",
                    help="comma-separated subset of c2,c3,stage4,c4,c5 measured after the headline (outside `value`); '' = none")
    ap.add_argument("--only", default=None, choices=sorted(OTHER),
                    help="run ONLY that configuration's loop (--steps/--warmup apply) and print its figures: for profiling")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run a plain elementwise kernel over 256 MiB in / 256 MiB out (for scaling HBM counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (data-centric mode, no expert or model sharding, no "
                 "collectives); --gpus must be 1")

    import torch
    import torch.nn.functional as F

    from hexa_moe import _lib

    _lib.load()  # no fallback: a missing library is an error
    dev = torch.device("cuda:0")
    if args.only:
        print(json.dumps({"config": args.only, **OTHER[args.only](dev, args.steps, args.warmup)}))
        return
    m, x, dy = make_module_and_inputs(dev)
    params = [prm for prm in m.parameters()]
    one = torch.ones((), device=dev)

    def step():
        x.grad = None
        for prm in params:
            prm.grad = None
        y, l_aux = m(0, x)
        torch.autograd.backward([y, l_aux], [dy, one])
        return y, m.dispatch_params.routing_

    if args.calibrate_copy:   # known traffic: 2^27 bf16 read + 2^27 bf16 written per launch
        src = torch.ones(1 << 27, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    from hexa_moe.impls.layers import FusedMoEDepth

    for _ in range(args.warmup):
        step()
    # Event pairs around the six matmul launches are recorded by the library itself on the launch stream
    # (hexa_moe_depth_forward / _backward take caller-owned events).  One pair per timed step, in rotation: a
    # record costs a few microseconds of stream time, and one per step keeps `value` honest.
    pairs = []
    if not args.no_kernel_events:
        for _ in range(args.steps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); b.record()           # creates the handles
            pairs.append((a, b))
    torch.cuda.synchronize()
    host = 0.0
    t0 = time.perf_counter()
    for i in range(args.steps):
        if pairs:
            _, direction, j = MAJOR[i % len(MAJOR)]
            arr = [None] * 8
            arr[2 * j], arr[2 * j + 1] = pairs[i]
            FusedMoEDepth.events = {"fwd": arr if direction == "fwd" else None, "bwd": arr if direction == "bwd" else None}
        y, idx = step()
    host = time.perf_counter() - t0            # the host has enqueued every step; the device is still running
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    FusedMoEDepth.events = None
    ms = (t1 - t0) * 1e3 / args.steps
    host_us = host * 1e6 / args.steps
    flops_step = 12.0 * T * K_TOP * D * H
    tokens_per_s = T / (ms * 1e-3)

    # ---- the six matmul launches, timed inside the timed steps ----
    kernels = {}
    roofline = None
    if pairs:
        gemm = 2.0 * T * K_TOP * D * H
        # algorithmic bytes of each launch (2-byte elements; every operand once, every result once)
        xb, hid, wb = T * D, T * K_TOP * H, E * H * D
        alg = {"fc1_esmm+gelu": 2.0 * (xb + wb + E * H + 2 * hid), "fc2_esmm+slot_sum": 2.0 * (hid + wb + E * D + xb),
               "dy1_esmm+gelu'+colsum": 2.0 * (xb + wb + 2 * hid), "dx_esmm": 2.0 * (hid + wb + xb),
               "dW2_estmm": 2.0 * (hid + xb + wb), "dW1_estmm": 2.0 * (hid + xb + wb)}
        ridge = PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)
        samples = {}
        for i, (a, b) in enumerate(pairs):
            samples.setdefault(MAJOR[i % len(MAJOR)][0], []).append(a.elapsed_time(b))   # ms
        for label, vals in samples.items():
            avg_ms = statistics.mean(vals)
            tf = gemm / (avg_ms * 1e-3) / 1e12
            gbs = alg[label] / (avg_ms * 1e-3) / 1e9
            # the roof that bounds a launch follows from its own arithmetic intensity against the machine's ridge
            kernels[label] = {"avg_us": round(avg_ms * 1e3, 2), "samples": len(vals),
                              "bound": "hbm" if gemm / alg[label] < ridge else "mfma",
                              "tflops": round(tf, 1), "frac": round(tf / PEAK_BF16_TFLOPS, 4),
                              "algorithmic_gbs": round(gbs, 1), "hbm_frac": round(gbs / PEAK_HBM_GBS, 4)}
        if ROOFLINE_KERNEL in kernels:
            # fc1 + GELU per launch: 2*T*k*d*h FLOP; algorithmic bytes = x rows once (T*d), W1 and b1 once, y1 and y2
            # written once (2 * T*k*h), 2-byte elements.  Its arithmetic intensity (156 FLOP/B) is below the machine's
            # ridge (2.5 PFLOP/s / 8 TB/s = 312 FLOP/B): the roof that bounds it is HBM, at 0.5 of the MFMA peak.
            d = kernels[ROOFLINE_KERNEL]
            alg_bytes = alg[ROOFLINE_KERNEL]
            secs = d["avg_us"] * 1e-6
            gbs = alg_bytes / secs / 1e9
            intensity = gemm / alg_bytes
            hbm_bound = intensity < ridge
            roofline = {"kernel": ROOFLINE_KERNEL, "bound": "hbm" if hbm_bound else "mfma",
                        "achieved": round(gbs, 1) if hbm_bound else d["tflops"],
                        "peak": PEAK_HBM_GBS if hbm_bound else PEAK_BF16_TFLOPS,
                        "unit": "GB/s" if hbm_bound else "TFLOP/s",
                        "frac": round(gbs / PEAK_HBM_GBS, 4) if hbm_bound else d["frac"],
                        "traffic": measured_traffic(ROOFLINE_KERNEL),
                        "algorithmic_bytes": alg_bytes, "algorithmic_flop": gemm, "avg_us": d["avg_us"],
                        "arithmetic_intensity_flop_per_byte": round(intensity, 1), "ridge_flop_per_byte": round(ridge, 1),
                        "hbm_frac": round(gbs / PEAK_HBM_GBS, 4), "mfma_tflops": d["tflops"], "mfma_frac": d["frac"]}

    # ---- CPU baseline: the oracle's plain-PyTorch fp32 evaluation of the same layer on the host ----
    cpu = None
    parity = None
    if not args.no_cpu_baseline:
        from oracle import hexa_oracle as O
        # as many threads as the box grants this process: its CPU share (OMP_NUM_THREADS, 16 per GPU on the
        # benchmark boxes) or, where none is set, every logical CPU
        logical = os.cpu_count() or 1
        threads = max(1, min(logical, int(os.environ.get("OMP_NUM_THREADS", logical))))
        torch.set_num_threads(threads)
        c = {"x": x, "W1": m.batched_fc1_w[0], "W2": m.batched_fc2_w[0], "b1": m.batched_fc1_bias[0],
             "b2": m.batched_fc2_bias[0], "dy": dy}
        c = {k: v.detach().float().cpu() for k, v in c.items()}
        routing = idx.cpu().long()
        run = lambda: O.moe_layer_fwd_bwd_cpu(c["x"], c["W1"], c["W2"], c["b1"], c["b2"], routing, c["dy"], F.gelu)  # noqa: E731
        run()
        times = []
        for _ in range(3):
            a = time.perf_counter()
            ref = run()
            times.append(time.perf_counter() - a)
        sec = statistics.median(times)
        cpu = {"value": round(T / sec, 1), "unit": "tokens/s", "cores": threads, "threads": threads,   # cores = threads in use
               "host_logical_cpus": logical, "kind": "port",
               "gflops": round(flops_step / sec / 1e9, 1),
               "sample": f"the full workload (T={T}, one layer fwd+bwd, fp32, per-expert index_select/mm/index_add), "
                         f"1 warm-up + median of 3 on {threads} threads of {logical} logical CPUs"}
        names = ["y", "dx", "dW1", "dW2", "db1", "db2"]
        got = [y, x.grad, m.batched_fc1_w[0].grad, m.batched_fc2_w[0].grad, m.batched_fc1_bias[0].grad,
               m.batched_fc2_bias[0].grad]
        # (dx also carries the auxiliary loss's gradient through the gate, 1e-4 of its norm at weight 1: inside the tolerance)
        parity = {n: float((g_.detach().float().cpu() - r).norm() / r.norm()) for n, g_, r in zip(names, got, ref)}
        parity = {k: float(f"{v:.3e}") for k, v in parity.items()}

    out = {
        "metric": "moe_layer_fwd_bwd_tokens_per_s", "value": round(tokens_per_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "full MoE layer fwd+bwd (gate, top-2 routing, fc1 ESMM+GELU, fc2 ESMM, ESS, ESTMM, "
                               "backward ESMM), Swin-MoE-S stage-3 shape",
                   "tokens": T, "d": D, "h": H, "experts": E, "top_k": K_TOP, "seed": SEED,
                   "routing": "top-2 of softmax(x.wg), logits ~ N(0,1) + N(0,0.5) per-expert bias"},
        "tflops": round(flops_step / (ms * 1e-3) / 1e12, 1),
        "frac_bf16_mfma_peak": round(flops_step / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
        "host_enqueue_us_per_step": round(host_us, 1),
        "roofline": roofline, "cpu_baseline": cpu, "parity_rel_err_vs_cpu": parity, "kernels": kernels,
        "kernels_note": "the six matmul launches, each timed by a HIP event pair the library records on the launch stream, "
                        "one launch per timed step in rotation; every other kernel of the step is in profiles/*.kernel_stats.txt",
    }
    # ---- the other named configurations, after the headline's timed region and outside `value` ----
    others = {}
    for name in [n for n in args.other_configs.split(",") if n]:
        if name not in OTHER:
            sys.exit(f"bench.py: unknown configuration '{name}'")
        torch.cuda.empty_cache()
        others[name] = OTHER[name](dev, 20, 5)
    out["other_configs"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
