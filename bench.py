#!/usr/bin/env python3
"""Benchmark of the W4 MoE-block hot path on one MI355X.

A step is one whole MoE block (router -> dispatch -> W4 gate_up+SiLU*mul -> W4 down ->
combine) over one batch of synthetic tokens, through odsd_moe_forward.  The headline
workload is the Mixtral-8x7B-shaped verify layer with T=160 tokens; `--workload NAME`
selects another one and `--all` adds the remaining configurations under "workloads".

The printed JSON line carries, next to the throughput, the roofline of the dominant kernel
(the gate_up W4 stream for verify shapes: algorithmic bytes / measured kernel time against
8 TB/s; for the prefill shape algorithmic flops against 2.5 PFLOP/s) and a CPU baseline (the
oracle's per-expert loop on the host cores over the same inputs).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
HEADLINE = "mixtral_t160"

# HBM bytes per launch of the gate_up kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# runs of this command (summaries and calibration in profiles/w4_gemm_gate_up_hbm_traffic.md):
# FETCH_SIZE reads half of the bytes a plain 1 GiB device copy moves (factor 2.0), WRITE_SIZE
# reads them in KiB (factor 1.0).
MEASURED_TRAFFIC_BYTES = {
    "mixtral_t160": 260564.9 * 2.0 * 1024 + 8964.6 * 1024,
}


def _build_layer(wl, dev, layer=0):
    import torch
    import on_device_sd_amd as odsd
    from on_device_sd_amd.workloads import LayerInputs
    inp = LayerInputs(wl, dev, layer)
    gate = inp.gate_weight()
    bank = odsd.W4ExpertBank(wl.E, wl.H, wl.I, dev)
    for e, gw, uw, dw in inp.experts():
        bank.load_expert(e, gw, uw, dw)
    x = inp.x()
    return gate, bank, x


def _clone_bank(bank):
    return bank.clone()


def _event_ms(fn, n):
    """Average duration of fn() over n launches, each bracketed by its own pair of events on
    the current stream (the stream the kernels are launched on)."""
    import torch
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for i, (a, b) in enumerate(evs):
        a.record()
        fn(i)
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in evs)
    return sum(ts) / len(ts), ts[len(ts) // 2], ts[0]


def _event_ms_sequence(stages, n):
    """Average / median / minimum duration of every stage of a sequence that is launched n times
    back to back, with an event between consecutive stages (on the launch stream)."""
    import torch
    ns = len(stages)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(ns + 1)] for _ in range(n)]
    for i in range(n):
        evs[i][0].record()
        for k, fn in enumerate(stages):
            fn(i)
            evs[i][k + 1].record()
    torch.cuda.synchronize()
    out = []
    for k in range(ns):
        ts = sorted(evs[i][k].elapsed_time(evs[i][k + 1]) for i in range(n))
        out.append((sum(ts) / len(ts), ts[len(ts) // 2], ts[0]))
    return out


def bench_layer(wl, dev, steps, warmup, with_cpu):
    import torch
    from on_device_sd_amd import ops
    gate, bank, x = _build_layer(wl, dev)
    # rotate over weight replicas so that the 256 MB memory-side cache cannot hold the stream
    layer_bytes = wl.E * wl.expert_w4_bytes
    n_rep = max(2, min(4, -(-(1 << 30) // layer_bytes)))
    banks = [bank] + [_clone_bank(bank) for _ in range(n_rep - 1)]
    tables = [b.table() for b in banks]
    plan = ops.MoeForwardPlan(wl.T, wl.H, wl.E, wl.K, wl.I, wl.renorm, wl.act_dtype, dev)

    def step(i):
        plan.run(x, gate, tables[i % n_rep])

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    counts = plan.counts.cpu()
    active = int((counts > 0).sum())

    # per-kernel durations through the stage entry points
    idx, w, _, x16 = ops.router_topk(x, gate, wl.K, wl.renorm, want_f16=True)
    disp = ops.dispatch(idx, wl.E)
    st = ops.ExpertStages(wl.T, wl.H, wl.E, wl.K, wl.I, wl.act_dtype, dev)
    out32 = torch.empty(wl.T, wl.H, dtype=torch.float32, device=dev)
    n = max(steps, 10)
    for i in range(3):
        st.gate_up(x16, tables[i % n_rep], disp); st.down(tables[i % n_rep], disp)
    # every stage bracketed by its own events INSIDE the sequence of a whole step (router ->
    # dispatch -> gate_up -> down -> combine), so that each kernel is timed under the clocks and
    # cache state it sees in the timed region, not in a loop of its own
    stages = [
        lambda i: ops.router_topk(x, gate, wl.K, wl.renorm, want_f16=True),
        lambda i: ops.dispatch(idx, wl.E),
        lambda i: st.gate_up(x16, tables[i % n_rep], disp),
        lambda i: st.down(tables[i % n_rep], disp),
        lambda i: st.combine(idx, w, disp, tables[0], out_f32=out32),
    ]
    k_rt, k_dp, k_gu, k_dn, k_cb = _event_ms_sequence(stages, n)
    # the two-call path of the reference engine loops: route_experts, the host reads the
    # activated set, forward_moe (reported beside the whole-block call, never as `value`)
    import on_device_sd_amd as odsd
    cfg = odsd.MoEConfig(hidden_size=wl.H, num_hidden_layers=n_rep, num_experts=wl.E,
                         num_experts_per_token=wl.K, moe_intermediate_size=wl.I, norm_topk_prob=wl.renorm,
                         torch_dtype="float32" if wl.act_dtype == torch.float32 else "bfloat16")
    runner = odsd.W4MoERunner(cfg, [gate] * n_rep, banks)
    placements = [odsd.ExpertPlacement(gpu_expert_params=b.all_expert_params(), cpu_expert_params={})
                  for b in banks]

    def engine_step(i):
        l = i % n_rep
        placements[l].routing_result = runner.route_experts(l, x)
        runner.forward_moe(l, odsd.AttentionOutput(hidden_states=x, post_attn_normed=x, residual=x),
                           placements[l])

    for i in range(max(3, warmup)):
        engine_step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(n):
        engine_step(i)
    torch.cuda.synchronize()
    engine_ms = (time.perf_counter() - t0) * 1e3 / n

    gu_bytes = active * (wl.expert_w4_bytes * 2 // 3)
    gu_flops = 4 * wl.pairs * wl.H * wl.I
    if wl.regime == "prefill":
        ach = gu_flops / (k_gu[0] * 1e-3) / 1e12
        roof = {"bound": "mfma", "kernel": "w4_gemm_kernel<gate_up>", "achieved": round(ach, 2),
                "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / MFMA_F16_PEAK_TFLOPS, 4),
                "traffic": None}
    else:
        ach = gu_bytes / (k_gu[0] * 1e-3) / 1e9
        roof = {"bound": "hbm", "kernel": "w4_gemm_kernel<gate_up>", "achieved": round(ach, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get(wl.name)}
        roof["algorithmic_bytes"] = gu_bytes
    roof["kernel_ms"] = round(k_gu[0], 4)
    layer_bytes_alg = wl.algorithmic_bytes(active)
    res = {
        "workload": wl.name, "T": wl.T, "H": wl.H, "E": wl.E, "K": wl.K, "I": wl.I,
        "tokens_per_s": wl.T / (ms * 1e-3), "ms_per_step": ms, "engine_path_ms": engine_ms,
        "active_experts": active,
        "max_rows_per_expert": int(counts.max()), "weight_replicas": n_rep,
        "layer_hbm_frac": layer_bytes_alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "layer_mfma_frac": wl.algorithmic_flops() / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
        "kernel_ms": {"router": k_rt[0], "dispatch": k_dp[0], "gate_up": k_gu[0], "down": k_dn[0],
                      "combine": k_cb[0]},
        "roofline": roof,
    }
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline(wl, gate, bank, x)
    return res


def bench_stack(wl, dev, steps, warmup):
    """48-layer RMSNorm -> MoE -> residual stack, all experts resident."""
    import torch
    import on_device_sd_amd as odsd
    from on_device_sd_amd.workloads import LayerInputs
    cfg = odsd.MoEConfig(hidden_size=wl.H, num_hidden_layers=wl.layers, num_experts=wl.E,
                         num_experts_per_token=wl.K, moe_intermediate_size=wl.I,
                         norm_topk_prob=wl.renorm)
    gates, banks, x = [], [], None
    for l in range(wl.layers):
        g, b, xl = _build_layer(wl, dev, l)
        gates.append(g); banks.append(b)
        if l == 0:
            x = xl
    norms = [torch.ones(wl.H, dtype=wl.act_dtype, device=dev) for _ in range(wl.layers)]
    stack = odsd.MoEOnlyStack(cfg, gates, norms, banks, wl.T)
    out = {}
    for mode in ("eager", "graph"):
        if mode == "graph":
            stack.capture()
        for _ in range(warmup):
            stack.forward(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            stack.forward(x)
        torch.cuda.synchronize()
        out[mode] = (time.perf_counter() - t0) * 1e3 / steps
    ms = min(out.values())
    total_bytes = wl.layers * wl.algorithmic_bytes(wl.E, out_bytes=2)
    return {"workload": wl.name, "T": wl.T, "layers": wl.layers, "ms_per_step": ms,
            "ms_eager": out["eager"], "ms_graph": out["graph"], "tokens_per_s": wl.T / (ms * 1e-3),
            "resident_weight_gb": wl.layers * wl.E * wl.expert_w4_bytes / 1e9,
            "layer_hbm_frac": total_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}


def cpu_baseline(wl, gate, bank, x):
    """The reference's CPU MoE path restated by the oracle (router F.linear -> top-k ->
    per-expert expert_forward loop -> weighted accumulate) on the host cores, fp32, with the
    W4 weights dequantised once beforehand.  Bounded: only as many experts are dequantised
    and timed as fit a ~20 s budget; the rate is scaled by pairs processed."""
    import numpy as np
    import torch
    from oracle import moe_oracle as orc
    from tests.helpers import unpack_bank_expert
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    xc, gc = x.cpu(), gate.cpu()
    idx, w = orc.route(orc.router_logits(xc, gc), wl.K, wl.renorm)
    counts = np.bincount(idx.reshape(-1), minlength=wl.E)
    order = [int(e) for e in np.argsort(-counts) if counts[e] > 0]
    budget_weights = 4.0e8          # dequantised fp32 weights held at once (1.6 GB)
    per_expert = 3 * wl.H * wl.I
    n_exp = max(1, min(len(order), int(budget_weights // per_expert)))
    chosen = order[:n_exp]
    experts = {e: unpack_bank_expert(bank, e).dequant() for e in chosen}
    pairs = int(sum(counts[e] for e in chosen))

    def run():
        return orc.moe_forward(xc, idx, w, experts)
    for _ in range(2):
        run()
    ts = []
    t_end = time.perf_counter() + 15.0
    while len(ts) < 5 or (len(ts) < 20 and time.perf_counter() < t_end and sum(ts) < 5.0):
        t0 = time.perf_counter(); run(); ts.append(time.perf_counter() - t0)
        if time.perf_counter() > t_end:
            break
    med = sorted(ts)[len(ts) // 2]
    # time for the whole layer = time for the sampled pairs scaled to all pairs
    layer_s = med * (wl.pairs / max(pairs, 1))
    return {"value": wl.T / layer_s, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{n_exp} of {len(order)} active experts ({pairs} of {wl.pairs} token-expert pairs), "
                      f"fp32 dequantised weights, median of {len(ts)} runs, scaled by pairs"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=HEADLINE)
    ap.add_argument("--all", action="store_true", help="also run the other configurations")
    ap.add_argument("--no-cpu", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (use --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    from on_device_sd_amd.workloads import CONFIGS
    from on_device_sd_amd import _lib
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    wl = CONFIGS[args.workload]
    if wl.layers > 1:
        main_res = bench_stack(wl, dev, max(3, args.steps // 10), max(1, args.warmup // 5))
    else:
        main_res = bench_layer(wl, dev, args.steps, args.warmup, not args.no_cpu)
    line = {
        "metric": "int4 MoE-layer tokens/s", "value": round(main_res["tokens_per_s"], 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(main_res["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 MFMA / fp32 accumulate on int4 weights (bf16 activations in and out)",
        "data": "synthetic",
        "config": {"workload": wl.name, "T": wl.T, "hidden": wl.H, "experts": wl.E, "top_k": wl.K,
                   "intermediate": wl.I, "renorm": wl.renorm, "weights": "W4 group-128 asymmetric fp16 scale/zero"},
        "roofline": main_res.get("roofline"),
        "cpu_baseline": main_res.get("cpu_baseline"),
        "detail": {k: v for k, v in main_res.items() if k not in ("roofline", "cpu_baseline")},
    }
    if args.all:
        others = []
        for name, w2 in CONFIGS.items():
            if name == wl.name or name == "tiny":
                continue
            torch.cuda.empty_cache()
            if w2.layers > 1:
                others.append(bench_stack(w2, dev, 5, 2))
            else:
                others.append(bench_layer(w2, dev, max(10, args.steps // 2), args.warmup, False))
        line["workloads"] = others
    print(json.dumps(line))


if __name__ == "__main__":
    main()
