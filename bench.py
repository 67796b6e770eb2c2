#!/usr/bin/env python3
"""Benchmark of the routed-expert MoE FFN path on one MI355X.

A step is one pass of a workload's batch through every MoE layer of the workload: one execute of a graph with
one Op::MoeFfn per layer (plus the shared-expert ops where the shape has one), each layer with its own
HBM-resident weights and its own N(0,1) activation rows.  Headline workload: the Qwen3-30B-A3B-shaped stack
(48 layers, hidden 2048, 128 experts, top-8, intermediate 768, Q4_K gate/up + Q6_K down), decode batch 1,
synthetic seeded weights.

The LAST line of stdout is the headline as one compact JSON object (under 2,000 bytes): whole-job decode tok/s of
the headline workload, the roofline of its dominant kernel measured live with HIP events attached to each dispatch
on the backend's stream, the time a chain of dependent plain reads of the same sizes takes on this device (what a
kernel chain of this shape cannot go below), and a CPU baseline (the oracle, a scalar C restatement of the
reference's CPU path, timed on this host's cores on a bounded sample).  With no --config every other benchmark
configuration (single Q8_0 layer, multi-stream decode, prefill chunks, the large shape with a shared expert) is
measured the same way and printed as a compact JSON line of its own BEFORE the headline; the per-kernel tables and
floors of every workload go to the file named by --detail (see its default below).
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

import moe4all_amd as M  # noqa: E402
from moe4all_amd import DType, TensorDesc, synth  # noqa: E402

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0   # dense fp16/bf16 matrix-core peak of one MI355X
SEED0 = 20260101
N_TOKENS = 16  # distinct activation sets rotated through the steps
TRAFFIC_FILE = os.path.join("profiles", "hbm_traffic.json")


def shape_of(config, tokens):
    return {"c1": synth.CONFIG_1, "c2": synth.CONFIG_2, "c5": synth.CONFIG_5, "mxfp4": synth.CONFIG_MXFP4,
            "c4": synth.MoeShape(f"c4-prefill-{tokens}-zipf1.1-q8_0", 1, 2048, 128, 8, 768, DType.Q8_0, DType.Q8_0),
            "c4k": synth.MoeShape(f"c4-prefill-{tokens}-zipf1.1-q4k-q6k", 1, 2048, 128, 8, 768, DType.Q4K, DType.Q6K)}[config]


class Stack:
    """The resident weights of a workload's layers, generated in HBM, shared by every batch size measured on them."""

    def __init__(self, be, shape, n_layer, prefill):
        self.be, self.shape, self.n_layer, self.prefill = be, shape, n_layer, prefill
        t0 = time.time()
        self.layers = [synth.LayerWeights(be, shape, SEED0, l, on_device=True) for l in range(n_layer)]
        if prefill:
            # skewed expert popularity through the op's own inputs: x[:, 0] = 1, router[e, 0] = ln Zipf(1.1)
            for lw in self.layers:
                router = be.download(lw.router, dtype=np.float32).reshape(shape.n_expert, shape.ne).copy()
                router[:, 0] = synth.zipf_bias(shape.n_expert, 1.1, SEED0)
                be.upload(lw.router, router)
        be.sync()
        self.setup_s = time.time() - t0

    def free(self):
        for lw in self.layers:
            lw.free()
        self.layers = []


def build_graph(stack, batch, sublayer=False):
    """One graph with n_layer MoeFfn ops (+ shared-expert ops).  With `sublayer` every layer is the model's whole FFN
    sublayer: y = x + ffn(rmsnorm(x) * w)."""
    shape = stack.shape
    g = M.Graph()
    ids = []
    for _ in range(stack.n_layer):
        x = x_raw = g.input(TensorDesc([batch, shape.ne], DType.F32))
        out = g.output(TensorDesc([batch, shape.ne], DType.F32))
        norm_w = None
        if sublayer:
            norm_w = g.weight(TensorDesc([shape.ne], DType.F32))
            x = g.internal(TensorDesc([batch, shape.ne], DType.F32))
            g.rms_norm(x=x_raw, weight=norm_w, dst=x, rows=batch, dim=shape.ne, eps=1e-6)
        router = g.weight(TensorDesc([shape.n_expert, shape.ne], DType.F32))
        gate = g.weight(TensorDesc([shape.n_expert, shape.n_ff, shape.ne], shape.gate_dtype))
        up = g.weight(TensorDesc([shape.n_expert, shape.n_ff, shape.ne], shape.gate_dtype))
        down = g.weight(TensorDesc([shape.n_expert, shape.ne, shape.n_ff], shape.down_dtype))
        dst = g.internal(TensorDesc([batch, shape.ne], DType.F32)) if sublayer else out
        d = dict(x=x_raw, router=router, gate=gate, up=up, down=down, dst=out, norm_w=norm_w)
        if shape.shared_ff:
            moe = g.internal(TensorDesc([batch, shape.ne], DType.F32))
            g.moe_ffn(x=x, router=router, gate_exps=gate, up_exps=up, down_exps=down, dst=moe, ne=shape.ne,
                      n_expert=shape.n_expert, n_used=shape.n_used, n_ff_exp=shape.n_ff)
            sg = g.weight(TensorDesc([shape.shared_ff, shape.ne], shape.gate_dtype))
            su = g.weight(TensorDesc([shape.shared_ff, shape.ne], shape.gate_dtype))
            sd = g.weight(TensorDesc([shape.ne, shape.shared_ff], shape.down_dtype))
            tg, tu = (g.internal(TensorDesc([batch, shape.shared_ff], DType.F32)) for _ in range(2))
            ta = g.internal(TensorDesc([batch, shape.shared_ff], DType.F32))
            ts = g.internal(TensorDesc([batch, shape.ne], DType.F32))
            g.linear(x=x, weight=sg, dst=tg, m=batch, in_f=shape.ne, out_f=shape.shared_ff)
            g.linear(x=x, weight=su, dst=tu, m=batch, in_f=shape.ne, out_f=shape.shared_ff)
            g.gated_act(gate=tg, up=tu, dst=ta, rows=batch, nff=shape.shared_ff)
            g.linear(x=ta, weight=sd, dst=ts, m=batch, in_f=shape.shared_ff, out_f=shape.ne)
            g.add(a=moe, b=ts, dst=dst, n=batch * shape.ne)
            d.update(sg=sg, su=su, sd=sd)
        else:
            g.moe_ffn(x=x, router=router, gate_exps=gate, up_exps=up, down_exps=down, dst=dst, ne=shape.ne,
                      n_expert=shape.n_expert, n_used=shape.n_used, n_ff_exp=shape.n_ff)
        if sublayer:
            g.add(a=x_raw, b=dst, dst=out, n=batch * shape.ne)
        ids.append(d)
    return g, ids


def algorithmic_tables(shape, batch, distinct, prefill):
    """Algorithmic HBM bytes and FLOPs per launch of each kernel name the backend's profiler reports."""
    gate_b = M.backend.bytes_for(shape.gate_dtype, shape.n_ff * shape.ne)
    down_b = M.backend.bytes_for(shape.down_dtype, shape.ne * shape.n_ff)
    n_sel = distinct if batch > 1 else shape.n_used
    pairs = batch * shape.n_used
    alg = {
        "router_logits": shape.router_bytes() + batch * shape.ne * 4 + batch * shape.n_expert * 4,
        "moe_gate_up": n_sel * 2 * gate_b + batch * shape.ne * 4 + pairs * shape.n_ff * 4,
        "moe_down_combine": n_sel * down_b + pairs * shape.n_ff * 4 + batch * shape.ne * 4,
    }
    # the decode kernel that routes its own token row also reads that row's logits
    alg["moe_route_gate_up"] = alg["moe_gate_up"] + batch * shape.n_expert * 4
    # banks on the 32-element-unit kernels: per-pair down results, then the rank-ordered sum as its own launch
    alg["moe_gate_up_units"], alg["moe_route_gate_up_units"] = alg["moe_gate_up"], alg["moe_route_gate_up"]
    alg["moe_down_units"] = n_sel * down_b + pairs * shape.n_ff * 4 + pairs * shape.ne * 4
    alg["moe_down_combine_units"] = alg["moe_down_combine"]
    alg["moe_gate_up_bucketed"] = alg["moe_gate_up"]
    if not prefill and batch < 32:
        alg["moe_unbucket_combine"] = pairs * shape.ne * 4 + batch * shape.ne * 4
    alg["rms_norm_router_logits"] = alg["router_logits"] + shape.ne * 4 + batch * shape.ne * 4
    # the whole single-token op as one launch: the three stages' bytes, each counted once (h and the logits stay on chip
    # or in L2: the hand-over records are not algorithmic traffic)
    alg["moe_layer"] = (shape.router_bytes() + shape.ne * 4 + shape.n_used * (2 * gate_b + down_b) + shape.ne * 4)
    alg["moe_layer_inorder"] = alg["moe_layer"]
    if shape.shared_ff:
        sh_gate_b = M.backend.bytes_for(shape.gate_dtype, shape.shared_ff * shape.ne)
        sh_down_b = M.backend.bytes_for(shape.down_dtype, shape.ne * shape.shared_ff)
        # the always-on expert as one more slot of the routed kernels
        alg["moe_layer_shared"] = alg["moe_layer"] + 2 * sh_gate_b + sh_down_b
        alg["moe_route_gate_up_shared"] = alg["moe_route_gate_up"] + 2 * sh_gate_b + batch * shape.shared_ff * 4
        alg["moe_down_combine_shared"] = alg["moe_down_combine"] + sh_down_b + batch * shape.shared_ff * 4
        alg["linear_gate_up_act"] = 2 * sh_gate_b + batch * shape.ne * 4 + batch * shape.shared_ff * 4
        alg["linear_add"] = sh_down_b + batch * shape.shared_ff * 4 + 2 * batch * shape.ne * 4
    flops = {  # 2 per multiply-add
        "moe_grouped_gate_up": 2.0 * pairs * 2 * shape.n_ff * shape.ne,
        "moe_grouped_down": 2.0 * pairs * shape.ne * shape.n_ff,
    }
    flops["moe_grouped_units_gate_up"], flops["moe_grouped_units_down"] = flops["moe_grouped_gate_up"], flops["moe_grouped_down"]
    return alg, flops


def measure(be, stack, config, batch, steps, warmup, *, sublayer=False, kernel_timing=True, cpu_budget_s=12.0, floor=True,
            no_fusion=False):
    """One workload on resident weights: the timed steps, per-kernel durations, the dependent-read floor, the CPU baseline."""
    shape, n_layer, prefill = stack.shape, stack.n_layer, stack.prefill
    g, ids = build_graph(stack, batch, sublayer)
    norm_w = be.buffer_from(np.ones(shape.ne, np.float32)) if sublayer else None
    plan = be.compile(g)
    # activations: N_TOKENS independent sets of per-layer N(0,1) rows, resident in HBM
    xbufs = []
    for t in range(N_TOKENS):
        row = []
        for l in range(n_layer):
            n_x = -(-batch * shape.ne // 256) * 256   # the generator writes whole 256-element groups
            xb = be.alloc(n_x * 4)
            synth.weights_device(be, xb, DType.F32, synth.stream_seed(SEED0 + 1 + t, l, synth.ROLE_X), n_x, sigma=1.0)
            if prefill:
                xh = be.download(xb, dtype=np.float32).reshape(batch, shape.ne).copy()
                xh[:, 0] = 1.0
                be.upload(xb, xh)
            row.append(xb)
        xbufs.append(row)
    ybufs = [be.alloc(batch * shape.ne * 4) for _ in range(n_layer)]
    binds = []
    for t in range(N_TOKENS):
        b = M.Bindings()
        for l in range(n_layer):
            d, lw = ids[l], stack.layers[l]
            b.bind(d["x"], xbufs[t][l]).bind(d["router"], lw.router).bind(d["gate"], lw.gate)
            b.bind(d["up"], lw.up).bind(d["down"], lw.down).bind(d["dst"], ybufs[l])
            if shape.shared_ff:
                b.bind(d["sg"], lw.shared[0]).bind(d["su"], lw.shared[1]).bind(d["sd"], lw.shared[2])
            if norm_w is not None:
                b.bind(d["norm_w"], norm_w)
        binds.append(b)
    be.sync()

    for i in range(warmup):
        be.execute(plan, binds[i % N_TOKENS])
    be.sync()
    t0 = time.perf_counter()
    for i in range(steps):
        be.execute(plan, binds[i % N_TOKENS])
    be.sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / steps
    tok_s = batch * steps / elapsed
    # spread: the same steps again in ten groups, each bracketed by a sync
    groups = max(1, min(10, steps))
    per_group = max(10, steps // groups)   # long enough that a group's sync and first dispatch do not show in its mean
    group_ms = []
    for gi in range(groups):
        t1 = time.perf_counter()
        for i in range(per_group):
            be.execute(plan, binds[(gi * per_group + i) % N_TOKENS])
        be.sync()
        group_ms.append((time.perf_counter() - t1) * 1e3 / per_group)

    # distinct experts actually selected per layer (batch > 1 shares experts between tokens)
    r = be.moe_routing(plan, 1 if sublayer else 0)
    distinct = len(set(r["idx"].ravel().tolist()))
    layer_bytes = shape.algorithmic_bytes(batch, distinct if batch > 1 else None)
    layer_gbps = layer_bytes * n_layer / (ms_per_step * 1e-3) / 1e9

    # ---- per-kernel durations: HIP events attached to each kernel's own dispatch on the backend's stream, separate pass
    roofline, kernels = None, {}
    alg, flops = algorithmic_tables(shape, batch, distinct, prefill)
    if kernel_timing:
        be.prof_enable(True)
        for i in range(max(1, min(steps, 50))):
            be.execute(plan, binds[i % N_TOKENS])
        be.sync()
        prof = be.prof_read()
        be.prof_enable(False)
        for name, p in prof.items():
            avg_us = p["total_ms"] * 1e3 / max(p["launches"], 1)
            kernels[name] = {"launches": int(p["launches"]), "avg_us": round(avg_us, 3), "min_us": round(p["min_ms"] * 1e3, 3)}
            if name in alg:
                kernels[name]["alg_bytes"] = alg[name]
                kernels[name]["GBps"] = round(alg[name] / (avg_us * 1e-6) / 1e9, 1)
            if name in flops:
                kernels[name]["alg_flops"] = flops[name]
                kernels[name]["TFLOPs"] = round(flops[name] / (avg_us * 1e-6) / 1e12, 1)
        total_us = lambda k: kernels[k]["avg_us"] * kernels[k]["launches"]
        cand = [k for k in kernels if k in flops] or [k for k in kernels if "alg_bytes" in kernels[k]]
        dom = max(cand, key=total_us, default=None)
        # HBM bytes per launch from hardware counters: taken in separate profiler runs of this same command and kept in
        # profiles/ (the counters cannot be read from inside this process); reported only for the workload they cover
        traffic, traffic_source = None, None
        if dom:
            try:
                with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
                    if n_layer == shape.n_layer and not sublayer and not no_fusion:
                        key = f"{config}/tokens{batch}" if prefill else f"{config}/batch{batch}"
                        traffic = json.load(f).get(key, {}).get(dom)
                        traffic_source = TRAFFIC_FILE if traffic is not None else None
            except OSError:
                pass
        if dom and dom in flops:
            ach = flops[dom] / (kernels[dom]["avg_us"] * 1e-6) / 1e12
            roofline = {"bound": "mfma", "kernel": dom, "achieved": round(ach, 1), "peak": MFMA_F16_PEAK_TFLOPS,
                        "unit": "TFLOP/s", "frac": round(ach / MFMA_F16_PEAK_TFLOPS, 4), "traffic": traffic,
                        "traffic_source": traffic_source,
                        "alg_flops_per_launch": flops[dom], "avg_launch_us": kernels[dom]["avg_us"]}
        elif dom:
            ach = alg[dom] / (kernels[dom]["avg_us"] * 1e-6) / 1e9
            roofline = {"bound": "hbm", "kernel": dom, "achieved": round(ach, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                        "frac": round(ach / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_source": traffic_source,
                        "alg_bytes_per_launch": alg[dom], "avg_launch_us": kernels[dom]["avg_us"]}

    # ---- what a chain of dependent kernels of these sizes cannot go below: plain reads, no arithmetic, the window of
    # each stage chosen by a word the stage before wrote (decode workloads; stage sizes = the kernels' algorithmic bytes)
    floor_out = None
    if floor and kernels and not prefill and roofline and roofline["bound"] == "hbm":
        chain = [k for k in kernels if "alg_bytes" in kernels[k]]
        order = {"router_logits": 0, "rms_norm_router_logits": 0, "route_topk": 1}
        chain.sort(key=lambda k: (order.get(k, 2 if "gate_up" in k else 3), k))
        sizes = [max(1024, int(kernels[k]["alg_bytes"])) for k in chain]
        pool = be.alloc_uninit(2 << 30)
        try:
            pr = be.probe_dependent_reads(pool, sizes, 200)
        finally:
            pool.free()
        floor_out = {"kernels": chain, "stage_bytes": sizes, "stage_us": [round(v, 3) for v in pr["stage_us"]],
                     "chain_us": round(pr["chain_us"], 3),
                     "achievable_frac_of_hbm_peak": round(sum(sizes) / (pr["chain_us"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                     "note": "dependent kernels that only read these byte counts (all loads of a block in flight at once)"}
        dom = roofline["kernel"]
        if dom in chain:
            st = pr["stage_us"][chain.index(dom)]
            roofline["floor_launch_us"] = round(st, 3)
            roofline["achievable_frac"] = round(kernels[dom]["alg_bytes"] / (st * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)

    # ---- prefill: what the dominant GEMM's data movement alone takes.  The same launches with the kernels' measurement
    # variant (loads, LDS reads and barriers as built; no unpacking, no matrix instructions; output meaningless)
    if floor and kernels and prefill and roofline and roofline["bound"] == "mfma":
        be.probe_grouped_loads_only(True)
        try:
            be.prof_enable(True)
            for i in range(max(1, min(steps, 30))):
                be.execute(plan, binds[i % N_TOKENS])
            be.sync()
            prof = be.prof_read()
            be.prof_enable(False)
        finally:
            be.probe_grouped_loads_only(False)
        lo = {k: p["total_ms"] * 1e3 / max(p["launches"], 1) for k, p in prof.items() if k in flops}
        if lo:
            dom = roofline["kernel"]
            floor_out = {"kernels": sorted(lo), "launch_us": [round(lo[k], 3) for k in sorted(lo)],
                         "note": "the same grouped GEMM launches moving their data (global -> LDS loads, LDS reads, barriers) "
                                 "without unpacking weights or issuing matrix instructions"}
            if dom in lo:
                roofline["floor_launch_us"] = round(lo[dom], 3)
                roofline["frac_of_data_movement_floor"] = round(lo[dom] / kernels[dom]["avg_us"], 4)
        be.execute(plan, binds[0])   # leave real results behind
        be.sync()

    # ---- CPU baseline: the oracle on this host's cores, layer 0's weights, a bounded sample
    cpu = None
    if cpu_budget_s > 0:
        import oracle as O
        lw = stack.layers[0]
        router = be.download(lw.router, dtype=np.float32)
        gate, up, down = be.download(lw.gate), be.download(lw.up), be.download(lw.down)
        threads = O.hw_threads()
        n_sample, spent = 0, 0.0
        cpu_rows = min(batch, 256)   # a prefill chunk is sampled by its first 256 tokens
        # the int8 batch numerics exist for the formats with an integer dot on the CPU (Q8_0, Q4_K, Q6_K)
        production = cpu_rows >= 2 and {shape.gate_dtype, shape.down_dtype} <= {DType.Q8_0, DType.Q4K, DType.Q6K}
        while spent < cpu_budget_s and n_sample < 4 * max(n_layer, 12):
            x = synth.normal(synth.stream_seed(SEED0 + 1, n_sample, synth.ROLE_X), batch * shape.ne, 1.0)
            x = x.reshape(batch, shape.ne)[:cpu_rows].copy()
            if prefill:
                x[:, 0] = 1.0
            t1 = time.perf_counter()
            # from two rows on the CPU backend's own numerics are int8 activations against the quantised rows
            # (crates/infr-cpu/src/lib.rs:3679); a single row runs the f32 dequantise-and-dot path either way
            O.moe_ffn(x, router, gate, up, down, ne=shape.ne, n_expert=shape.n_expert, n_used=shape.n_used,
                      n_ff_exp=shape.n_ff, gate_dtype=int(shape.gate_dtype), down_dtype=int(shape.down_dtype),
                      n_threads=threads, production=production)
            spent += time.perf_counter() - t1
            n_sample += 1
        per_layer_s = spent / n_sample
        cpu = {"value": round(cpu_rows / (per_layer_s * n_layer), 3), "unit": "tok/s", "cores": threads, "kind": "port",
               "sample": f"scalar auto-vectorised C restatement of the reference's CPU path, not its AVX2/AVX-512/VNNI tiers; "
                         f"{n_sample} passes of layer 0 (routed experts, {cpu_rows} token rows), {per_layer_s * 1e3:.2f} ms each, "
                         f"{'int8-activation production numerics' if production else 'f32 dequantise-and-dot numerics'}, "
                         f"scaled to {n_layer} layers",
               "ms_per_layer": round(per_layer_s * 1e3, 3)}

    out = {
        "metric": "MoE prefill tok/s" if prefill else "MoE decode tok/s", "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_min": round(min(group_ms), 4), "ms_per_step_max": round(max(group_ms), 4),
        "spread": f"min / max over {groups} groups of {per_group} steps run after the timed region, a sync after each group",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        # decode: exact integer dots (v_dot4 on byte planes) on 23-bit fixed-point activations, scales and sums in f32;
        # batched path: f16 operands on the matrix cores with f32 accumulation
        "dtype": "f16-mfma/f32-acc" if batch >= 32 else "i8dot-23bit-act/f32-acc", "data": "synthetic",
        "config": {"workload": (shape.name if n_layer == shape.n_layer else f"{shape.name}[{n_layer} layers]") +
                               ("+rmsnorm+residual" if sublayer else "") + ("/unfused" if no_fusion else ""),
                   "layers": n_layer, "hidden": shape.ne, "experts": shape.n_expert, "top_k": shape.n_used,
                   "intermediate": shape.n_ff, "gate_up": shape.gate_dtype.name, "down": shape.down_dtype.name,
                   "shared_intermediate": shape.shared_ff, "batch": batch, "parallelism": "single-gpu",
                   "resident_weight_bytes": shape.layer_resident_bytes() * n_layer},
        "layer": {"us_per_layer": round(ms_per_step * 1e3 / n_layer, 3), "alg_bytes_per_layer": layer_bytes,
                  "achieved_GBps": round(layer_gbps, 1), "frac_of_hbm_peak": round(layer_gbps / HBM_PEAK_GBPS, 4),
                  "distinct_experts_layer0": distinct},
        "roofline": roofline, "floor": floor_out, "kernels": kernels, "cpu_baseline": cpu,
    }
    plan.free()
    for row in xbufs:
        for xb in row:
            xb.free()
    for yb in ybufs:
        yb.free()
    if norm_w is not None:
        norm_w.free()
    return out


# the other benchmark configurations, measured after the headline when no --config is given:
# (config, layers (0 = the shape's), batches or chunk sizes)
OTHER_WORKLOADS = (("c1", 0, (1, 4, 16)), ("c4", 0, (512, 2048)), ("c4k", 0, (512, 2048)), ("c5", 0, (1, 8)))
LINE_LIMIT = 1900   # bytes; the harness that records this run keeps only the tail of stdout


def compact(res, headline):
    """The one-line form of a result: the contract's keys, the roofline and the CPU baseline, no per-kernel tables."""
    keep = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "ms_per_step_min", "ms_per_step_max",
            "higher_is_better", "scaling", "vs_baseline", "dtype", "data")
    out = {k: res[k] for k in keep if k in res}
    c = res["config"]
    out["config"] = {k: c[k] for k in ("workload", "layers", "hidden", "experts", "top_k", "intermediate", "gate_up", "down",
                                       "shared_intermediate", "batch", "parallelism")}
    out["layer"] = {k: res["layer"][k] for k in ("us_per_layer", "alg_bytes_per_layer", "frac_of_hbm_peak")}
    out["roofline"] = res["roofline"]
    cpu = res.get("cpu_baseline")
    if cpu:
        cpu = dict(cpu)
        if not headline:
            cpu["sample"] = cpu["sample"].split(";")[1].strip() if ";" in cpu["sample"] else cpu["sample"]
        out["cpu_baseline"] = cpu
    if headline:
        for k in ("device", "compute_units", "detail"):
            if k in res:
                out[k] = res[k]
    line = json.dumps(out, separators=(",", ":"))
    if len(line) > LINE_LIMIT and cpu:      # never let prose push the line past what the recorder keeps
        cpu["sample"] = cpu["sample"][:max(40, len(cpu["sample"]) - (len(line) - LINE_LIMIT))]
        line = json.dumps(out, separators=(",", ":"))
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default=None, choices=["c1", "c2", "c4", "c4k", "c5", "mxfp4"],
                    help="one workload only.  c1/c2/c5: decode stacks (use --batch for multi-stream decode); c4: one config-1 layer "
                         "(Q8_0), prefill chunk of --tokens with Zipf(1.1) expert popularity; c4k: same with "
                         "Q4_K gate/up + Q6_K down; mxfp4: a decode stack of the gpt-oss-120b expert shape with MXFP4 banks "
                         "(the 32-element-unit kernels; use --batch >= 32 for the unit-decoder grouped GEMM).  Default: c2 as the "
                         "headline (last line) after one line per other benchmark configuration")
    ap.add_argument("--headline-only", action="store_true", help="with no --config: measure the headline workload only")
    ap.add_argument("--detail", default=os.path.join(ROOT, "gpurun_out", "bench_configs.json"),
                    help="file that receives the full results (per-kernel tables, floors) of every workload; '' = none")
    ap.add_argument("--tokens", type=int, default=2048, help="prefill chunk size for c4/c4k")
    ap.add_argument("--layers", type=int, default=0, help="override the layer count (0 = the config's)")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--sublayer", action="store_true",
                    help="time the model's whole FFN sublayer per layer (RmsNorm -> MoeFfn [+ shared expert] -> "
                         "residual Add) instead of the MoeFfn op alone; not the headline metric")
    ap.add_argument("--no-fusion", action="store_true", help="one launch per op (infr_hip_config.disable_op_fusion)")
    ap.add_argument("--three-launch", action="store_true",
                    help="single-token MoeFfn as three launches (infr_hip_config.disable_single_launch_moe), for comparison")
    ap.add_argument("--in-order", action="store_true",
                    help="single-token MoeFfn on the single-launch kernel that runs its stages in order "
                         "(infr_hip_config.disable_single_launch_guess), for comparison")
    ap.add_argument("--logits", type=int, default=0, choices=[0, 1, 2],
                    help="single-launch kernel: 1 = every router logit once for the grid, 2 = once per group of workgroups "
                         "(infr_hip_config.single_launch_logits), 0 = the built-in choice")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--no-floor", action="store_true", help="skip the dependent-read probe")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run one plain device-to-device copy of this many MiB (a known-size kernel that "
                         "calibrates hardware byte counters in a profiler run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists in this tree)",
              file=sys.stderr)
        sys.exit(2)

    headline_cfg = args.config or "c2"
    prefill = headline_cfg in ("c4", "c4k")
    shape = shape_of(headline_cfg, args.tokens)
    n_layer = args.layers or shape.n_layer
    batch = args.tokens if prefill else args.batch
    be = M.Backend(0, disable_op_fusion=args.no_fusion, disable_single_launch_moe=args.three_launch,
                   disable_single_launch_guess=args.in_order, single_launch_logits=args.logits)
    caps = be.capabilities()
    stack = Stack(be, shape, n_layer, prefill)
    if args.copy_probe_mib:
        n = args.copy_probe_mib << 20
        src, dst = be.alloc(n), be.alloc(n)
        be.copy_buffer(src, dst, n)
        be.sync()
        src.free()
        dst.free()
    out = measure(be, stack, headline_cfg, batch, args.steps, args.warmup, sublayer=args.sublayer,
                  kernel_timing=not args.no_kernel_timing,
                  cpu_budget_s=0.0 if (args.no_cpu_baseline or args.sublayer) else 12.0,   # the CPU sample times Op::MoeFfn alone
                  floor=not args.no_floor, no_fusion=args.no_fusion)
    out["device"], out["compute_units"], out["setup_s"] = caps["name"], caps["compute_units"], round(stack.setup_s, 1)
    stack.free()

    detail = {"headline": out, "configs": []}
    if args.config is None and not args.headline_only:
        for cfg, layers, sizes in OTHER_WORKLOADS:
            pf = cfg in ("c4", "c4k")
            stacks = {}
            for size in sizes:
                sh = shape_of(cfg, size)
                key = 0 if not pf else size    # a prefill shape's name carries its chunk size; the weights are the same
                if key not in stacks:
                    if pf and stacks:
                        st = next(iter(stacks.values()))
                        st.shape = sh
                        stacks[key] = st
                    else:
                        stacks[key] = Stack(be, sh, layers or sh.n_layer, pf)
                st = stacks[key]
                # a one-layer workload of well under a millisecond needs many steps for a stable mean
                steps = max(5, min(args.steps, 40)) if st.n_layer > 1 else max(args.steps, 200)
                res = measure(be, st, cfg, size, steps, max(min(args.warmup, 5), 5 if st.n_layer == 1 else 0),
                              cpu_budget_s=0.0 if args.no_cpu_baseline else 2.5,
                              kernel_timing=not args.no_kernel_timing, floor=not args.no_floor)
                res["setup_s"] = round(st.setup_s, 1)
                detail["configs"].append(res)
                print(compact(res, headline=False), flush=True)
            for st in {id(v): v for v in stacks.values()}.values():
                st.free()
    be.close()
    # per-kernel tables, floors and spreads of every workload: to a file, not to stdout
    if args.detail:
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.detail)), exist_ok=True)
            with open(args.detail, "w") as f:
                json.dump(detail, f, indent=1)
            out["detail"] = os.path.relpath(args.detail, ROOT) if os.path.abspath(args.detail).startswith(ROOT) else args.detail
        except OSError as e:
            print(f"bench.py: could not write {args.detail}: {e}", file=sys.stderr)
    print(compact(out, headline=True), flush=True)


if __name__ == "__main__":
    main()
