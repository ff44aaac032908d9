#!/usr/bin/env python3
"""Benchmark of the W4 MoE-block hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic tokens.  The headline workload is
the largest single-GPU configuration, the Qwen3-30B-A3B-shaped 48-layer MoE-only stack at T=256
(15.4 GB of W4 experts resident in HBM; one step = RMSNorm -> router -> dispatch -> W4 gate_up +
SiLU*mul -> W4 down -> combine -> residual, 48 times); the other four configurations are measured
the same way and reported under "workloads".  `--workload NAME` measures one configuration only.

Every result carries
  * the whole-step time (host clock around K back-to-back steps, inputs resident in HBM),
  * per-kernel GPU times from HIP events: in the timed steps every kernel launch of the library
    carries its own start / stop events on the launch stream (odsd_moe_forward_events), which the
    runtime stamps with the kernel's begin and end; nothing is inserted between the kernels, so
    the kernel times add up to at most the step time,
  * the roofline of the dominant kernel (verify shapes: the gate_up W4 stream, algorithmic bytes
    over its event time against 8 TB/s; prefill shape: algorithmic flops against 2.5 PFLOP/s),
  * a CPU baseline: the oracle's restatement of the reference's per-expert loop on the host cores
    over the same inputs, with fp32 weights dequantised beforehand.
"""
import argparse
import dataclasses
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
HEADLINE = "qwen3_30b_stack48_t256"
OTHERS = ("mixtral_t160", "mixtral_t5", "qwen3_30b_t64_zipf", "qwen3_235b_t4096")
# beside the five configurations: the 48-layer stack under a Zipf-skewed router (no CPU baseline: the
# arithmetic per token is that of the headline)
SKEWED = ("qwen3_30b_stack48_t256_zipf",)
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def _log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def _host_threads():
    n = os.cpu_count() or 1
    for var in ("OMP_NUM_THREADS",):
        try:
            n = min(n, int(os.environ[var]))
        except (KeyError, ValueError):
            pass
    return max(1, n)


SETTLE_S = 0.4


def _settle(step, seconds=SETTLE_S):
    """Run `step(i)` untimed for `seconds` before a workload's W warm-up steps.  After the host-side
    set-up of a workload the GPU sits idle for a while, and its first milliseconds of work run at
    reduced clocks: five warm-up steps of a 0.1 - 0.2 ms layer end before the clocks have come up,
    and the timed steps then read 6 - 15 % slow against the steady state of a serving loop (the same
    loop timed a second time in one process: 0.235 -> 0.198 ms for the Mixtral T = 160 layer)."""
    import torch
    torch.cuda.synchronize()
    t_end = time.perf_counter() + seconds
    i = 0
    while time.perf_counter() < t_end:
        for _ in range(8):
            step(i)
            i += 1
        torch.cuda.synchronize()


def _build_layer(wl, dev, layer=0, keep_canonical=False):
    import on_device_sd_amd as odsd
    from on_device_sd_amd.workloads import LayerInputs
    inp = LayerInputs(wl, dev, layer)
    gate = inp.gate_weight()
    bank = odsd.W4ExpertBank(wl.E, wl.H, wl.I, dev)
    canon = {}
    for e, gw, uw, dw in inp.experts():
        c = bank.load_expert(e, gw, uw, dw, keep_canonical=keep_canonical)
        if keep_canonical:
            canon[e] = c
    x = inp.x()
    return gate, bank, x, canon


def _dequant_to_host(canon_expert):
    """fp32 (gate, up, down) weights of one expert on the host.  The arithmetic is the oracle's
    dequantize_w4, (code - zero) * scale in fp32, done with torch on the device because numpy
    needs tens of seconds for the larger layers; this is preparation, not part of any timing."""
    import torch
    out = []
    for q, s, z in canon_expert:
        n, kb = q.shape
        codes = torch.stack((q & 15, q >> 4), dim=-1).view(n, kb * 2).to(torch.float32)
        g = kb * 2 // 128
        d = codes.view(n, g, 128) - z.to(torch.float32)[:, :, None]
        out.append((d * s.to(torch.float32)[:, :, None]).view(n, kb * 2).cpu())
    return tuple(out)


def _stage_stats(per_step):
    """per_step: list (steps) of lists (stages) of ms -> per-stage average over the steps."""
    n = len(per_step)
    return [sum(s[k] for s in per_step) / n for k in range(len(per_step[0]))]


def _traffic(wl_name, kernel=None):
    """HBM bytes per launch of the dominant kernel as measured offline with rocprofv3 --pmc
    (FETCH_SIZE, WRITE_SIZE) and recorded, with the commit it was measured on, in
    profiles/hbm_traffic.json; None when there is no record for the workload."""
    try:
        rec = json.load(open(TRAFFIC_FILE))[wl_name]
        if kernel and not rec.get("kernel", "").startswith(kernel):
            return None, None          # measured on another kernel than the one in use
        return rec["bytes_per_launch"], rec.get("commit")
    except (OSError, KeyError, ValueError):
        return None, None


def _dominant(wl, k, active_experts, launches=1):
    """The dominant kernel of a workload, its time per launch and the algorithmic bytes of one launch:
    the one-launch expert kernel (gate_up + down weights of the active experts) where the library
    uses it, the gate_up stream (two thirds of an expert's bytes) otherwise."""
    if k.get("experts", 0.0) > 0.0:
        return "w4_expert_fused_kernel", k["experts"] / launches, active_experts * wl.expert_w4_bytes / launches
    return None, k["gate_up"] / launches, active_experts * (wl.expert_w4_bytes * 2 // 3) / launches


def _roofline(wl, kernel_ms, algorithmic_bytes, kernel=None):
    gu_flops = 4 * wl.pairs * wl.H * wl.I
    traffic, commit = _traffic(wl.name, kernel)
    if wl.regime == "prefill":
        ach = gu_flops / (kernel_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "kernel": "w4_gemm_prefill_kernel<gate_up>", "achieved": round(ach, 2),
                "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(ach / MFMA_F16_PEAK_TFLOPS, 4),
                "traffic": traffic, "algorithmic_flops": gu_flops}
    else:
        ach = algorithmic_bytes / (kernel_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "kernel": kernel or "w4_gemm_kernel<gate_up>", "achieved": round(ach, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                "traffic": traffic, "algorithmic_bytes": int(algorithmic_bytes)}
    if commit:
        roof["traffic_measured_at_commit"] = commit
    roof["kernel_ms"] = round(kernel_ms, 5)
    return roof


def bench_layer(wl, dev, steps, warmup, with_cpu):
    """One MoE layer; weight replicas are rotated from step to step so that the 256 MB memory-side
    cache cannot hold the weight stream."""
    import torch
    from on_device_sd_amd import _hip, _lib, ops
    _log(f"{wl.name}: building the layer")
    gate, bank, x, canon = _build_layer(wl, dev, keep_canonical=with_cpu)
    layer_bytes = wl.E * wl.expert_w4_bytes
    n_rep = max(2, min(4, -(-(1 << 30) // layer_bytes)))
    banks = [bank] + [bank.clone() for _ in range(n_rep - 1)]
    tables = [b.table() for b in banks]
    plan = ops.MoeForwardPlan(wl.T, wl.H, wl.E, wl.K, wl.I, wl.renorm, wl.act_dtype, dev)
    # timed region: K whole-block calls back to back
    _settle(lambda i: plan.run(x, gate, tables[i % n_rep]))
    for i in range(warmup):
        plan.run(x, gate, tables[i % n_rep])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        plan.run(x, gate, tables[i % n_rep])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps

    # the same K steps once more with every kernel launch carrying its start / stop events (the
    # runtime's handling of those events makes the step itself slower, the kernels are not)
    events = [_hip.EventList(2 * _lib.N_KERNELS) for _ in range(steps)]
    masks = [0] * steps
    plan.run_events(events[0], x, gate, tables[0])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        masks[i] = plan.run_events(events[i], x, gate, tables[i % n_rep])
    torch.cuda.synchronize()
    ms_events = (time.perf_counter() - t0) * 1e3 / steps
    stage_ms = _stage_stats([ev.kernel_ms(m) for ev, m in zip(events, masks)])
    counts = plan.counts.cpu()
    active = int((counts > 0).sum())

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

    _settle(engine_step, 0.2)
    for i in range(max(3, warmup)):
        engine_step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        engine_step(i)
    torch.cuda.synchronize()
    engine_ms = (time.perf_counter() - t0) * 1e3 / steps

    k = dict(zip(_lib.KERNEL_NAMES, stage_ms))
    dom_kernel, dom_ms, dom_bytes = _dominant(wl, k, active)
    res = {
        "workload": wl.name, "T": wl.T, "H": wl.H, "E": wl.E, "K": wl.K, "I": wl.I,
        "tokens_per_s": round(wl.T / (ms * 1e-3), 1), "ms_per_step": round(ms, 5),
        "ms_per_step_with_kernel_events": round(ms_events, 5), "engine_path_ms": round(engine_ms, 5),
        "active_experts": active, "max_rows_per_expert": int(counts.max()), "weight_replicas": n_rep,
        "layer_hbm_frac": round(wl.algorithmic_bytes(active) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "layer_mfma_frac": round(wl.algorithmic_flops() / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4),
        "kernel_ms": {n: round(v, 5) for n, v in k.items()},
        "kernel_ms_sum": round(sum(stage_ms), 5),
        "roofline": _roofline(wl, dom_ms, dom_bytes, dom_kernel),
    }
    if k.get("down", 0.0) > 0.0:
        # the down projection's own stream (a third of an expert's packed bytes) against HBM, or its
        # flops against the matrix cores at the prefill shape
        down_bytes = active * (wl.expert_w4_bytes // 3)
        if wl.regime == "prefill":
            ach = 2 * wl.pairs * wl.H * wl.I / (k["down"] * 1e-3) / 1e12
            res["down_roofline"] = {"bound": "mfma", "kernel": "w4_gemm_prefill_kernel<down>", "achieved": round(ach, 2),
                                    "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                    "frac": round(ach / MFMA_F16_PEAK_TFLOPS, 4), "kernel_ms": round(k["down"], 5)}
        else:
            ach = down_bytes / (k["down"] * 1e-3) / 1e9
            res["down_roofline"] = {"bound": "hbm", "kernel": "w4_gemm_kernel<down>", "achieved": round(ach, 1),
                                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4),
                                    "algorithmic_bytes": int(down_bytes), "kernel_ms": round(k["down"], 5)}
    del runner, placements, plan, banks, tables
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline_layer(wl, gate, x, canon)
    return res


def bench_stack(wl, dev, steps, warmup, with_cpu, cpu_layers=4):
    """48-layer RMSNorm -> MoE -> residual stack, all experts resident."""
    import torch
    import on_device_sd_amd as odsd
    from on_device_sd_amd import _hip, _lib
    cfg = odsd.MoEConfig(hidden_size=wl.H, num_hidden_layers=wl.layers, num_experts=wl.E,
                         num_experts_per_token=wl.K, moe_intermediate_size=wl.I,
                         norm_topk_prob=wl.renorm)
    _log(f"{wl.name}: building {wl.layers} layers")
    gates, banks, x, canon_layers = [], [], None, []
    for l in range(wl.layers):
        keep = with_cpu and l < cpu_layers
        g, b, xl, canon = _build_layer(wl, dev, l, keep_canonical=keep)
        gates.append(g); banks.append(b)
        if keep:
            canon_layers.append(canon)
        if l == 0:
            x = xl
    norms = [torch.ones(wl.H, dtype=wl.act_dtype, device=dev) for _ in range(wl.layers)]
    stack = odsd.MoEOnlyStack(cfg, gates, norms, banks, wl.T)
    # timed region: K passes through the stack, as eager launches and as one HIP graph
    out = {}
    for mode in ("eager", "graph"):
        if mode == "graph":
            stack.capture()
        _settle(lambda i: stack.forward(x))
        for _ in range(warmup):
            stack.forward(x)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            stack.forward(x)
        torch.cuda.synchronize()
        out[mode] = (time.perf_counter() - t0) * 1e3 / steps
    ms = min(out.values())
    stack.graph = None

    # the same K steps once more (eager) with every kernel launch carrying its start / stop events
    events = [_hip.EventList(wl.layers * 2 * _lib.N_KERNELS) for _ in range(steps)]
    masks = [None] * steps
    stack.forward_events(x, events[0])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        masks[i] = stack.forward_events(x, events[i])
    torch.cuda.synchronize()
    ms_events = (time.perf_counter() - t0) * 1e3 / steps
    # per layer: the kernel times; per step: their sums over the layers
    per_step = []
    for i in range(steps):
        tot = [0.0] * _lib.N_KERNELS
        for l in range(wl.layers):
            for s, v in enumerate(events[i].kernel_ms_at(l * 2 * _lib.N_KERNELS, masks[i][l], _lib.N_KERNELS)):
                tot[s] += v
        per_step.append(tot)
    stage_ms = _stage_stats(per_step)

    k = dict(zip(_lib.KERNEL_NAMES, stage_ms))
    # active experts per layer: re-run the layers' routing through the whole-block outputs
    active, max_rows = _stack_active_experts(stack, x, wl)
    dom_kernel, dom_ms, dom_bytes = _dominant(wl, k, sum(active), wl.layers)
    alg_bytes = sum(wl.algorithmic_bytes(a, out_bytes=2) for a in active)
    res = {
        "workload": wl.name, "T": wl.T, "H": wl.H, "E": wl.E, "K": wl.K, "I": wl.I, "layers": wl.layers,
        "tokens_per_s": round(wl.T / (ms * 1e-3), 1), "ms_per_step": round(ms, 5),
        "ms_per_step_eager": round(out["eager"], 5), "ms_per_step_graph": round(out["graph"], 5),
        "ms_per_step_with_kernel_events": round(ms_events, 5),
        "resident_weight_gb": round(wl.layers * wl.E * wl.expert_w4_bytes / 1e9, 3),
        "active_experts_per_layer_mean": round(sum(active) / len(active), 2),
        "max_rows_per_expert": {"mean_over_layers": round(sum(max_rows) / len(max_rows), 1), "max": max(max_rows)},
        "layer_hbm_frac": round(alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "kernel_ms": {n: round(v, 5) for n, v in k.items()},
        "kernel_ms_sum": round(sum(stage_ms), 5),
        "kernel_ms_note": f"sums over the {wl.layers} layers of one step",
        # the dominant kernel runs once per layer: average launch = sum over layers / layers
        "roofline": _roofline(wl, dom_ms, dom_bytes, dom_kernel),
    }
    del stack, events
    if with_cpu:
        res["cpu_baseline"] = cpu_baseline_stack(wl, gates, norms, x, canon_layers)
    return res


def bench_attention(dev, steps, warmup, with_cpu):
    """The step on the other side of the MoE block in a verify pass: the draft tokens' K / V rows are
    scattered into the paged cache and every query attends its sequence's cached keys (Qwen3-30B-A3B
    heads: 32 query / 4 KV heads of 128; 32 sequences x 8 draft tokens, 2048 cached tokens each,
    256-token cache blocks in random order).  Timed as replays of a HIP graph holding one store +
    one attention call, so that the Python wrapper's host time is not in the figure."""
    import torch
    import on_device_sd_amd as odsd
    name = "qwen3_30b_verify_attention_s32_q8_ctx2048"
    H, KVH, HD, bs, n_seqs, ql, L = 32, 4, 128, 256, 32, 8, 2048
    _log(f"{name}: building the cache")
    nb = L // bs
    g = torch.Generator().manual_seed(0)
    tables = torch.randperm(n_seqs * nb, generator=g).view(n_seqs, nb).to(torch.int32)
    k_cache = torch.randn(n_seqs * nb * bs, KVH * HD, generator=g).to(torch.bfloat16).to(dev)
    v_cache = torch.randn(n_seqs * nb * bs, KVH * HD, generator=g).to(torch.bfloat16).to(dev)
    q = torch.randn(n_seqs * ql, H, HD, generator=g).to(torch.bfloat16).to(dev)
    k_new = torch.randn(n_seqs * ql, KVH, HD, generator=g).to(torch.bfloat16).to(dev)
    v_new = torch.randn(n_seqs * ql, KVH, HD, generator=g).to(torch.bfloat16).to(dev)
    pos = torch.arange(L - ql, L)
    slots = (tables[:, (pos // bs)].to(torch.int64) * bs + (pos % bs)).reshape(-1).to(torch.int32).to(dev)
    ctx = {"block_tables": tables.to(dev), "context_lens": torch.full((n_seqs,), L, dtype=torch.int32, device=dev),
           "verify_query_lens": torch.full((n_seqs,), ql, dtype=torch.int32, device=dev), "slot_mapping": slots}

    def step():
        odsd.store_kvcache(k_new, v_new, k_cache, v_cache, slots)
        return odsd.paged_attention(q, k_cache, v_cache, ctx, KVH, bs, max_q_len=ql)

    def timed(fn):
        _settle(lambda i: fn(), 0.2)
        for _ in range(max(3, warmup)):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    eager_ms = timed(step)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step()
    graph_ms = timed(graph.replay)
    g_attn = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g_attn):
        odsd.paged_attention(q, k_cache, v_cache, ctx, KVH, bs, max_q_len=ql)
    attn_ms = timed(g_attn.replay)
    kv_bytes = 2 * n_seqs * L * KVH * HD * 2 + 2 * q.numel() * 2
    ach = kv_bytes / (attn_ms * 1e-3) / 1e9
    traffic, traffic_commit = _traffic(name)
    n_tok = n_seqs * ql
    res = {
        "workload": name, "kind": "kv-cache store + paged causal attention (one layer of a verify step)",
        "sequences": n_seqs, "query_tokens_per_sequence": ql, "context_len": L, "heads": H, "kv_heads": KVH,
        "head_dim": HD, "block_size": bs, "tokens_per_s": round(n_tok / (graph_ms * 1e-3), 1),
        "ms_per_step": round(graph_ms, 5), "ms_per_step_eager_python": round(eager_ms, 5),
        "roofline": {"bound": "hbm", "kernel": "paged_attn_kernel + paged_attn_merge_kernel", "achieved": round(ach, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "algorithmic_bytes": kv_bytes, "kernel_ms": round(attn_ms, 5)},
    }
    if traffic_commit:
        res["roofline"]["traffic_measured_at_commit"] = traffic_commit
    if with_cpu:
        # the oracle's restatement of the reference's fallback attention on a sample of the sequences
        from oracle import moe_oracle as oracle
        n_s = 4
        qs = q[:n_s * ql].float().cpu()
        kc, vc = k_cache.float().cpu(), v_cache.float().cpu()
        cl = [L] * n_s
        torch.set_num_threads(_host_threads())

        def run():
            oracle.paged_attention(qs, kc, vc, tables[:n_s], cl, [ql] * n_s, KVH, bs, HD ** -0.5)
        sec, _ = _time_cpu(run, 10.0)
        res["cpu_baseline"] = {"value": round(n_s * ql / sec, 1), "unit": "tokens/s", "cores": _host_threads(),
                               "kind": "port", "sample": f"{n_s} of the {n_seqs} sequences (fp32 gather + matmul "
                               "attention per sequence, the reference's fallback path), tokens/s of the sample"}
    return res


def _stack_active_experts(stack, x, wl):
    """Experts with at least one token and the largest per-expert row count, per layer, from the
    counts the whole-block call returns."""
    import torch
    from on_device_sd_amd import ops
    plan = ops.MoeForwardPlan(wl.T, wl.H, wl.E, wl.K, wl.I, wl.renorm, wl.act_dtype, x.device,
                              want_f32=False, want_act=True)
    h = x.clone()
    active, max_rows = [], []
    for l in range(stack.L):
        o = plan.run(h, stack.gate[l], stack.tables[l], stack.norm[l], stack.config.rms_norm_eps,
                     add_residual=True)
        active.append(int((o.counts > 0).sum()))
        max_rows.append(int(o.counts.max()))
        h = o.out_act.clone()
    torch.cuda.synchronize()
    return active, max_rows


def _time_cpu(run, budget_s, min_runs=2, max_runs=10):
    run()                                         # warm-up (thread pool, page faults)
    ts = []
    t_end = time.perf_counter() + budget_s
    while len(ts) < min_runs or (len(ts) < max_runs and time.perf_counter() < t_end):
        t0 = time.perf_counter(); run(); ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2], len(ts)


def cpu_baseline_layer(wl, gate, x, canon):
    """The reference's CPU MoE path restated by the oracle (router F.linear -> top-k -> per-expert
    expert_forward loop -> weighted accumulate) on the host cores, fp32, over the whole layer:
    every active expert, weights dequantised once beforehand."""
    import numpy as np
    import torch
    from oracle import moe_oracle as orc
    cores = _host_threads()
    torch.set_num_threads(cores)
    xc, gc = x.cpu(), gate.cpu()
    idx, w = orc.route(orc.router_logits(xc, gc), wl.K, wl.renorm)
    active = [int(e) for e in np.unique(idx)]
    _log(f"{wl.name}: CPU baseline, dequantising {len(active)} experts")
    experts = {e: _dequant_to_host(canon[e]) for e in active}
    canon.clear()

    def run():
        i2, w2 = orc.route(orc.router_logits(xc, gc), wl.K, wl.renorm)
        return orc.moe_forward(xc, i2, w2, experts)
    med, n = _time_cpu(run, budget_s=12.0)
    return {"value": round(wl.T / med, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"the whole layer: all {len(active)} active experts, {wl.pairs} token-expert pairs, "
                      f"fp32 dequantised weights in host memory, median of {n} runs"}


def cpu_baseline_stack(wl, gates, norms, x, canon_layers):
    """The first n layers of the stack on the host cores (RMSNorm -> router -> per-expert loop ->
    combine -> residual per layer), scaled by layers/n."""
    import torch
    from oracle import moe_oracle as orc
    cores = _host_threads()
    torch.set_num_threads(cores)
    n = len(canon_layers)
    _log(f"{wl.name}: CPU baseline, dequantising {n} layers")
    layers = []
    for l in range(n):
        experts = {e: _dequant_to_host(c) for e, c in canon_layers[l].items()}
        canon_layers[l].clear()
        layers.append((norms[l].cpu(), gates[l].cpu(), experts))
    xc = x.cpu()

    def run():
        h = xc
        for nw, gw, experts in layers:
            h = orc.moe_only_layer(h, nw, gw, experts, wl.K, wl.renorm)[0]
        return h
    med, runs = _time_cpu(run, budget_s=12.0)
    stack_s = med * wl.layers / n
    return {"value": round(wl.T / stack_s, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"layers 0..{n - 1} of {wl.layers} (all 128 experts each, fp32 dequantised weights in "
                      f"host memory), median of {runs} runs, time scaled by {wl.layers}/{n}"}


def run_workload(wl, dev, steps, warmup, with_cpu):
    import torch
    res = bench_stack(wl, dev, steps, warmup, with_cpu) if wl.layers > 1 else \
        bench_layer(wl, dev, steps, warmup, with_cpu)
    torch.cuda.empty_cache()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=None, help="measure this configuration only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--layers", type=int, default=None,
                    help="stack workloads: run this many layers instead of the configuration's (hardware-counter "
                         "runs, where every dispatch is costly; a kernel's per-launch figures do not depend on it)")
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

    if args.workload == "attention":
        print(json.dumps(bench_attention(dev, args.steps, args.warmup, not args.no_cpu)))
        return
    head = CONFIGS[args.workload or HEADLINE]
    if args.layers is not None:
        if head.layers <= 1 or args.layers < 1:
            print("--layers applies to a stack workload and must be positive", file=sys.stderr)
            sys.exit(2)
        head = dataclasses.replace(head, layers=args.layers)
    main_res = run_workload(head, dev, args.steps, args.warmup, not args.no_cpu)
    line = {
        "metric": "int4 MoE-layer tokens/s", "value": main_res["tokens_per_s"], "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16 MFMA / fp32 accumulate on int4 weights (bf16 activations in and out)",
        "data": "synthetic",
        "config": {"workload": head.name, "T": head.T, "hidden": head.H, "experts": head.E, "top_k": head.K,
                   "intermediate": head.I, "layers": head.layers, "renorm": head.renorm,
                   "weights": "W4 group-128 asymmetric fp16 scale/zero"},
        "roofline": main_res.get("roofline"),
        "cpu_baseline": main_res.get("cpu_baseline"),
        "detail": {k: v for k, v in main_res.items() if k not in ("roofline", "cpu_baseline")},
    }
    if args.workload is None:
        line["workloads"] = [run_workload(CONFIGS[name], dev, args.steps, args.warmup, not args.no_cpu)
                             for name in OTHERS]
        line["workloads"] += [run_workload(CONFIGS[name], dev, args.steps, args.warmup, False) for name in SKEWED]
        line["workloads"].append(bench_attention(dev, args.steps, args.warmup, not args.no_cpu))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
