#!/usr/bin/env python3
"""Benchmark of the mixed-bit MoE routed-expert path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2-t64] [--no-extras] [--no-cpu]

A "step" is one pass of the hot path over one batch that is already resident in HBM:
routing/permute -> gate & up -> SiLU*mul -> down -> top-k weighted combine
(operator scope: from the router's top-k ids to rank_accum [T, rank_out]; one call of
bitsmoe_moe_forward_routed, which runs small batches without a routing kernel -- the forward's kernels find
their assignments themselves -- and builds routing tables first otherwise; `config.routing` says which).  The layer is
synthetic (random-init factors of the named shape, quantised and packed on the GPU).

Cold weights.  A model streams a different layer's weights on every step, so a benchmark that
replays ONE layer (active set 179 MB at 64 tokens) may be served from the 256 MB memory-side
cache instead of HBM.  The decode workloads therefore build `--layers` distinct copies of the
layer (different seeds: different weights and bit draws) and cycle through them inside the timed
loop; with 4 copies 555 MB of other weights pass between two visits of a layer.  The headline
`value`, `ms_per_step` and `roofline` are the COLD figures; the one-layer replay is reported
beside them as `warm`.  `c5-stack-*` runs the stack configuration of the benchmark set: the 26-layer DeepSeek-V2-Lite-
shaped stack, one step = one pass over all 26 layers (per-layer figures reported).

The LAST stdout line is one compact JSON record (< 4 KB); the full record with every field of every workload
is written to bench_out/bench_full.json (--full-json PATH; --print-full also prints it as an earlier line).
`value` is tokens/s of the primary workload (default: the
Qwen3-30B-A3B-shaped layer at decode, 64 tokens); `extras` holds the other decode batch
sizes, the 4096-token prefill, the other layer shapes of the benchmark set (c1, c4), checkpoint-shaped experts and the
stack; `roofline` is the dominant kernel of the primary workload
(algorithmic bytes / HIP-event duration against 8 TB/s, or algorithmic FLOP/s against the
2.5 PFLOP/s dense bf16 MFMA peak); `cpu_baseline` is the CPU restatement of the reference
algorithm (oracle/oracle.c, OpenMP) timed on this host's cores on the same workload — the
reference publishes no CPU path and no numbers, so this is a reported baseline only.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E peak, GB/s
GRAPH_LAYER_STEPS = 32         # layer-steps one HIP graph of a decode-size workload holds (rounds over the distinct layers)
GRAPH_ROUNDS_MAX_TOKENS = 256  # ... larger batches: one round (every captured call keeps a workspace of its own)
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA peak, TFLOP/s

WORKLOADS = {
    # name: (spec key, tokens, roofline bound)
    "c2-t1": ("c2", 1, "hbm"),
    "c2-t8": ("c2", 8, "hbm"),
    "c2-t32": ("c2", 32, "hbm"),
    "c2-t64": ("c2", 64, "hbm"),
    "c3-t4096": ("c3", 4096, "mfma"),
    "c2-ckpt-t64": ("c2", 64, "hbm"),
    "c3-ckpt-t4096": ("c3", 4096, "mfma"),
    # two of the 128 experts dense ("super" experts: 16-bit rows, run by the operator's side kernels)
    "c2-super2-t64": ("c2", 64, "hbm"),
    # intermediate size 1440: the last column tile holds 32 columns
    "c2-i1440-t64": ("c2i", 64, "hbm"),
    "c1-t16": ("c1", 16, "hbm"),
    "c4-t256": ("c4", 256, "hbm"),
    "c5-stack-t32": ("c5", 32, "hbm"),
    "c5-stack-t2048": ("c5", 2048, "mfma"),
}
WORKLOAD_DESC = {
    "c2": "Qwen3-30B-A3B-shaped MoE layer (128 experts, top-8, hidden 2048, intermediate 768, mixed 2/3/4-bit, group 128)",
    "c3": "Qwen3-30B-A3B-shaped MoE layer (128 experts, top-8, hidden 2048, intermediate 768, mixed 2/3/4-bit, group 128)",
    "c2i": "Qwen3-30B-A3B-shaped MoE layer with intermediate 1440 (128 experts, top-8, hidden 2048, mixed 2/3/4-bit, group 128)",
    "c1": "DeepSeek-V2-Lite-shaped MoE layer (64 experts, top-6, hidden 2048, intermediate 1408, mixed 2/3/4-bit, group 128)",
    "c4": "Qwen3-Next-80B-A3B-shaped MoE layer (512 experts, top-10, one shared expert outside the operator, hidden 2048, "
          "intermediate 512, mixed 2/3/4-bit, group 128)",
    "c5": "DeepSeek-V2-Lite-shaped stack of 26 MoE layers (64 routed + 2 shared experts, top-6, hidden 2048, "
          "intermediate 1408, mixed 2/3/4-bit, group 128, Zipf(1.2)-skewed routing)",
}
PROFILES_DIR = os.path.join(ROOT, "profiles")


def matrix_bytes(lists, e):
    payload, rank_idx, tile_meta, slab_meta, scale, s = lists
    return (payload[e].numel() * 4 + scale[e].numel() * 2 + s[e].numel() * 2 + rank_idx[e].numel() * 4
            + slab_meta[e].numel() * 4 + tile_meta[e].numel() * 4)


def algorithmic_work(block, counts, tokens, n_assign, super_counts=()):
    """Algorithmic bytes (per kernel) and FLOPs of one forward for the ACTUAL active experts; `super_counts`:
    assignments of the block's dense experts (f16 weights, hidden-sized activations)."""
    gate, up, down = (block._static_lists(p) for p in ("gate", "up", "down"))
    rank_g = int(block.shared_vh_gate_proj.shape[0])
    rank_u = int(block.shared_vh_up_proj.shape[0])
    rank_out = int(block.shared_u_down.shape[1])
    isz = int(block._packed_intermediate_size)
    active = [e for e, c in enumerate(counts) if c > 0]
    b_gateup = sum(matrix_bytes(gate, e) + matrix_bytes(up, e) for e in active)
    b_down = sum(matrix_bytes(down, e) for e in active)
    b_gateup += 2 * tokens * (rank_g + rank_u) + 4 * n_assign
    b_down += 4 * tokens * rank_out + 8 * n_assign
    flops = sum(2 * counts[e] * isz * (gate[1][e].numel() + up[1][e].numel() + down[1][e].numel()) for e in active)
    fl_gateup = sum(2 * counts[e] * isz * (gate[1][e].numel() + up[1][e].numel()) for e in active)
    for (_, layer), c in zip(block._super_expert_items, super_counts):
        if c <= 0:
            continue
        wg, wd = layer.gate_proj.weight, layer.down_proj.weight
        b_gateup += 2 * 2 * wg.numel() + 2 * tokens * int(wg.shape[1])
        b_down += 2 * wd.numel() + 4 * tokens * int(wd.shape[0])
        flops += 2 * c * 3 * wg.numel()
        fl_gateup += 2 * c * 2 * wg.numel()
    return {"bytes_gateup": b_gateup, "bytes_down": b_down, "bytes_total": b_gateup + b_down,
            "flops": flops, "flops_gateup": fl_gateup, "flops_down": flops - fl_gateup, "active_experts": len(active)}


class _LayerState:
    """Everything one layer-step needs, resident on the device."""

    def __init__(self, block, spec, tokens, seed):
        import torch

        from bitsmoe_amd.synth import draw_selected

        dev = block._runtime_device()
        block._ensure_runtime_cache(dev)
        self.block = block
        self.sets = block._ensure_matsets()
        g = torch.Generator().manual_seed(seed + tokens)
        self.x = torch.randn((tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(dev)
        vh_gate, vh_up, _ = block._shared_basis(torch.bfloat16)
        self.h_gate = (self.x @ vh_gate.T).contiguous()
        self.h_up = (self.x @ vh_up.T).contiguous()
        self.selected, self.weights = draw_selected(spec, tokens, seed + 1000 + tokens, dev)
        self.rank_out = int(block.shared_u_down.shape[1])
        self.isz = int(block._packed_intermediate_size)
        self.g2l = block._packed_global_to_local
        self.l2g = block._packed_local_to_global
        self.n_packed = block._packed_expert_count
        # dense ("super") experts among the routed ones: a second operator call on their own matrix sets
        self.has_super = bool(block._super_expert_items)


def run_workload(blocks, spec, tokens, steps, warmup, seed=42, use_graph=True, layers_per_step=1, block_scope=True):
    """Times `steps` steps; a step is `layers_per_step` consecutive layer-steps (routing + operator, from the
    router's top-k output to rank_accum: one call, bitsmoe_moe_forward_routed) of the rotation blocks[0],
    blocks[1], ... (one block: the same layer replayed, warm caches)."""
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip

    n_layers = len(blocks)
    layers = [_LayerState(b, spec, tokens, seed + 17 * i) for i, b in enumerate(blocks)]
    dev = layers[0].block._runtime_device()

    def layer_step(i, profile=None):
        st = layers[i % n_layers]
        gate, up, down = st.sets
        side = None
        if st.has_super:
            # the dense experts' matrix sets: a second call of the operator (output in hidden space), on a side stream
            # beside the packed experts' call, as the block runs it
            from bitsmoe_amd.models.base_block import _side_stream

            cur = torch.cuda.current_stream(dev)
            side = _side_stream(dev)
            side.wait_stream(cur)
            with torch.cuda.stream(side):
                sup = st.block._super_operator_output(st.x, st.selected, st.weights)
        out = hip.moe_forward_routed(st.h_gate, st.h_up, st.selected, st.weights, st.g2l, st.l2g, gate, up, down,
                                     st.rank_out, st.isz, 0, profile=profile)
        if side is not None:
            cur.wait_stream(side)
            sup.record_stream(cur)
        return out

    def layer_tables(i):      # (the routing tables, for the accounting and the CPU check only)
        st = layers[i % n_layers]
        return hip.route(st.selected, st.weights, st.g2l, st.n_packed)

    n_layer_steps = steps * layers_per_step
    for i in range(max(warmup * layers_per_step, n_layers)):
        layer_step(i)
    torch.cuda.synchronize(dev)
    # (1) eager launches, no instrumentation: what a caller of the operator sees per call
    t0 = time.perf_counter()
    for i in range(n_layer_steps):
        layer_step(i)
    torch.cuda.synchronize(dev)
    eager = time.perf_counter() - t0
    # (2) the same layer-steps with HIP events between the kernels (per-kernel durations for the roofline)
    n_prof = min(n_layer_steps, 2000)
    profiles = [hip.Profile() for _ in range(n_prof)]
    for i in range(n_prof):
        layer_step(i, profiles[i])
    torch.cuda.synchronize(dev)
    # (3) one round over the layers captured into a HIP graph and replayed: the operator never allocates
    # or synchronises, so a serving loop can drop the per-launch host cost this way
    elapsed, launch, graph_ms = eager, "eager", None
    if use_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                for i in range(n_layers):
                    layer_step(i)
            torch.cuda.current_stream(dev).wait_stream(side)
            torch.cuda.synchronize(dev)
            # (a decode-size batch: several rounds over the layers in ONE graph -- a serving step replays the MoE layers
            # of a whole model as one graph, and a graph of eight kernels would charge its launch to four layer-steps)
            rounds = max(1, GRAPH_LAYER_STEPS // n_layers) if tokens <= GRAPH_ROUNDS_MAX_TOKENS else 1
            with torch.cuda.graph(graph):
                g_outs = [layer_step(i) for i in range(n_layers * rounds)]
            # every replay must reproduce the eager result (fp32 atomics: summation order may differ)
            for _ in range(3):
                graph.replay()
                torch.cuda.synchronize(dev)
                for i in (0, n_layers - 1):
                    ref_out = layer_step(i)
                    torch.cuda.synchronize(dev)
                    if not torch.allclose(g_outs[i], ref_out, rtol=1e-4, atol=1e-5 * float(ref_out.abs().max())):
                        raise RuntimeError("graph replay differs from the eager result")
            per_replay = n_layers * rounds
            replays = max(1, (n_layer_steps + per_replay - 1) // per_replay)
            for _ in range(max(1, (warmup * layers_per_step) // per_replay)):
                graph.replay()
            torch.cuda.synchronize(dev)
            t0 = time.perf_counter()
            for _ in range(replays):
                graph.replay()
            torch.cuda.synchronize(dev)
            replay = (time.perf_counter() - t0) * n_layer_steps / (replays * per_replay)     # for the same number of layer-steps
            if replay < eager:       # large steps hide the launch cost anyway and replay has its own
                elapsed, launch = replay, "hipgraph"
            graph_ms = replay / steps * 1e3
        except Exception as exc:   # noqa: BLE001 - the eager figure stands
            print(f"bench.py: graph replay unavailable ({exc}); reporting eager launches", file=sys.stderr)
    phases = [p.read() for p in profiles]
    # What two consecutive HIP events read with NOTHING between them, on this stream, through the same entry
    # point: a forward without assignments records the six events back to back.  Every phase carries this much
    # on top of its kernels (the event packet itself); the per-kernel durations below have it taken off, the
    # raw readings are kept beside them.
    st0 = layers[0]
    no_tok = torch.zeros((0,), dtype=torch.int32, device=dev)
    no_off = torch.zeros((st0.n_packed + 1,), dtype=torch.int32, device=dev)
    no_rw = torch.zeros((0,), dtype=torch.float32, device=dev)
    gaps = []
    for _ in range(50):
        pr = hip.Profile()
        hip.moe_forward_sets(st0.h_gate, st0.h_up, no_tok, no_off, no_rw, *st0.sets, st0.rank_out, st0.isz, 0, profile=pr)
        torch.cuda.synchronize(dev)
        gaps.extend(pr.read()[:4])
    gaps.sort()
    event_gap = gaps[len(gaps) // 2]
    # phases of the operator: preparation (with the routing launch before it), gate/up kernel,
    # SiLU pass, down kernel, combine (third and fifth: launches of their own at prefill only);
    # averages per LAYER-step
    raw = [sum(p[i] for p in phases) / n_prof for i in range(5)]
    ms_fill, ms_gateup, ms_silu, ms_down, ms_combine = (max(v - event_gap, 0.0) for v in raw)
    ms_all = ms_fill + ms_gateup + ms_silu + ms_down + ms_combine
    # algorithmic work of one layer-step: the mean over the layers of the rotation
    works, last = [], None
    for i in range(n_layers):
        out = layer_step(i)
        tok, off, rw = layer_tables(i)
        torch.cuda.synchronize(dev)
        counts = (off[1:] - off[:-1]).cpu().tolist()
        sel_flat = layers[i].selected.reshape(-1)
        super_counts = [int((sel_flat == idx).sum()) for idx, _ in layers[i].block._super_expert_items]
        works.append(algorithmic_work(layers[i].block, counts, tokens, int(tok.numel()), super_counts))
        if i == 0:
            last = (tok, off, rw, out)
    work = {k: sum(w[k] for w in works) / n_layers for k in works[0]}
    ms_layer = elapsed / n_layer_steps * 1e3
    res = {
        "tokens": tokens, "layers_in_rotation": n_layers, "layers_per_step": layers_per_step,
        "ms_per_step": elapsed / steps * 1e3, "ms_per_layer": ms_layer, "tokens_per_s": tokens * steps / elapsed,
        "launch": launch, "eager_ms_per_step": eager / steps * 1e3, "hipgraph_ms_per_step": graph_ms,
        "routing": "inside the forward's kernels" if hip.routed_is_inline(
            layers[0].h_gate, layers[0].h_up, int(layers[0].selected.shape[1]), *layers[0].sets) else "routing kernel(s) first",
        # one kernel per (expert, tile) from the activations to the atomic combine (its time is the `gate_up` phase)
        "fused": hip.decode_is_fused(layers[0].h_gate, layers[0].h_up, int(layers[0].selected.numel()), *layers[0].sets),
        "kernel_ms": {"prepare": ms_fill, "gate_up": ms_gateup, "silu_mul": ms_silu, "down": ms_down,
                      "combine": ms_combine},
        "kernel_ms_events_raw": dict(zip(("prepare", "gate_up", "silu_mul", "down", "combine"), raw)),
        "event_gap_ms": event_gap,
        "active_experts": work["active_experts"], "algorithmic_bytes": work["bytes_total"] * layers_per_step,
        "algorithmic_flops": work["flops"] * layers_per_step,
        "gateup_GBps": work["bytes_gateup"] / (ms_gateup * 1e-3) / 1e9 if ms_gateup > 0 else None,
        "down_GBps": work["bytes_down"] / (ms_down * 1e-3) / 1e9 if ms_down > 0 else None,
        "kernels_GBps": work["bytes_total"] / (ms_all * 1e-3) / 1e9,
        "kernels_TFLOPs": work["flops"] / (ms_all * 1e-3) / 1e12,
        "gateup_TFLOPs": work["flops_gateup"] / (ms_gateup * 1e-3) / 1e12 if ms_gateup > 0 else None,
        "down_TFLOPs": work["flops_down"] / (ms_down * 1e-3) / 1e12 if ms_down > 0 else None,
        # the whole operator against the wall clock of the timed loop (launch gaps, routing kernel and all)
        "operator_GBps": work["bytes_total"] / (ms_layer * 1e-3) / 1e9,
        "operator_TFLOPs": work["flops"] / (ms_layer * 1e-3) / 1e12,
    }
    if block_scope:
        res["block_scope"] = run_block_scope(layers, tokens, steps, layers_per_step, use_graph)
    tok, off, rw, out = last
    st0 = layers[0]
    inputs = {"h_gate": st0.h_gate, "h_up": st0.h_up, "tok": tok, "off": off, "rw": rw, "out": out, "work": work,
              "selected": st0.selected, "weights": st0.weights}
    return res, inputs


def run_block_scope(layers, tokens, steps, layers_per_step, use_graph):
    """Block scope: router + the two shared-basis GEMMs + the operator + the output projection + shared
    experts (torch / hipBLASLt for everything around the operator), over the same rotation of layers."""
    import torch

    dev = layers[0].block._runtime_device()
    n_layers = len(layers)
    xs = [st.x.reshape(1, tokens, -1) for st in layers]
    n_layer_steps = steps * layers_per_step
    with torch.no_grad():
        for i in range(max(3, n_layers)):
            layers[i % n_layers].block(xs[i % n_layers])
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for i in range(n_layer_steps):
            layers[i % n_layers].block(xs[i % n_layers])
        torch.cuda.synchronize(dev)
    block_s = (time.perf_counter() - t0) / steps
    out = {"ms_per_step": block_s * 1e3, "tokens_per_s": tokens / block_s, "launch": "eager",
           "eager_ms_per_step": block_s * 1e3, "note": "whole MoE block forward on its own router"}
    if use_graph:
        try:       # the block forward has no host synchronisation either: capture and replay it
            bgraph = torch.cuda.CUDAGraph()
            first = lambda y: y[0] if isinstance(y, tuple) else y
            rounds = max(1, GRAPH_LAYER_STEPS // n_layers) if tokens <= GRAPH_ROUNDS_MAX_TOKENS else 1
            with torch.no_grad():
                with torch.cuda.graph(bgraph):
                    ybs = [first(layers[i % n_layers].block(xs[i % n_layers])) for i in range(n_layers * rounds)]
                for _ in range(3):
                    bgraph.replay()
                    torch.cuda.synchronize(dev)
                    ye = first(layers[n_layers - 1].block(xs[n_layers - 1]))
                    torch.cuda.synchronize(dev)
                    if not torch.allclose(ybs[-1].float(), ye.float(), rtol=2e-2, atol=2e-2 * float(ye.float().abs().max())):
                        raise RuntimeError("block graph replay differs from the eager result")
                per_replay = n_layers * rounds
                replays = max(1, (n_layer_steps + per_replay - 1) // per_replay)
                t0 = time.perf_counter()
                for _ in range(replays):
                    bgraph.replay()
                torch.cuda.synchronize(dev)
            replay_s = (time.perf_counter() - t0) * layers_per_step / (replays * per_replay)
            out["hipgraph_ms_per_step"] = replay_s * 1e3
            if replay_s < block_s:
                out.update(ms_per_step=replay_s * 1e3, tokens_per_s=tokens / replay_s, launch="hipgraph")
        except Exception as exc:   # noqa: BLE001
            print(f"bench.py: block graph replay unavailable ({exc})", file=sys.stderr)
    return out


def counter_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` from hardware counters (FETCH_SIZE + WRITE_SIZE, each scaled by
    what it reads for a plain copy of known size), as summarised in profiles/<workload>_hbm_traffic_counters.txt
    by a line `traffic_bytes_per_launch <kernel> <bytes>`; None when no such summary exists."""
    path = os.path.join(PROFILES_DIR, f"{workload}_hbm_traffic_counters.txt")
    try:
        with open(path) as f:
            for line in f:
                parts = line.split()
                if len(parts) == 3 and parts[0] == "traffic_bytes_per_launch" and parts[1] == kernel:
                    return int(float(parts[2]))
    except OSError:
        pass
    return None


def roofline_of(res, inputs, bound, workload=None):
    """The dominant kernel (the fused gate+up launch: two thirds of the weight bytes / flops) against its
    roofline, HIP-event duration; `operator_*`: ALL algorithmic bytes / flops of a layer-step against the
    wall clock per layer-step of the timed loop (the figure the 70 % / 40 % layer targets are about)."""
    work = inputs["work"]
    if bound == "hbm" and res.get("fused"):
        # the one-kernel forward: ALL the algorithmic bytes of a layer-step move in that kernel
        ms = res["kernel_ms"]["gate_up"]
        achieved = work["bytes_total"] / (ms * 1e-3) / 1e9
        return {"bound": "hbm", "kernel": "fused", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": counter_traffic(workload, "fused"),
                "algorithmic_bytes_per_launch": work["bytes_total"], "launch_ms": ms,
                "launch_ms_events_raw": res["kernel_ms_events_raw"]["gate_up"], "event_gap_ms": res["event_gap_ms"],
                "weights": "cold" if res["layers_in_rotation"] > 1 else "warm", "down_kernel_frac": None,
                "all_kernels_GBps": res["kernels_GBps"], "all_kernels_frac": res["kernels_GBps"] / HBM_PEAK_GBS,
                "operator_GBps": res["operator_GBps"], "operator_frac": res["operator_GBps"] / HBM_PEAK_GBS}
    if bound == "hbm":
        achieved = res["gateup_GBps"]
        return {"bound": "hbm", "kernel": "gate_up", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": counter_traffic(workload, "gate_up"),
                "algorithmic_bytes_per_launch": work["bytes_gateup"], "launch_ms": res["kernel_ms"]["gate_up"],
                "launch_ms_events_raw": res["kernel_ms_events_raw"]["gate_up"], "event_gap_ms": res["event_gap_ms"],
                "weights": "cold" if res["layers_in_rotation"] > 1 else "warm",
                "down_kernel_frac": (res["down_GBps"] or 0.0) / HBM_PEAK_GBS,
                "all_kernels_GBps": res["kernels_GBps"], "all_kernels_frac": res["kernels_GBps"] / HBM_PEAK_GBS,
                "operator_GBps": res["operator_GBps"], "operator_frac": res["operator_GBps"] / HBM_PEAK_GBS}
    achieved = res["gateup_TFLOPs"]
    return {"bound": "mfma", "kernel": "gate_up", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": counter_traffic(workload, "gate_up"),
            "algorithmic_flops_per_launch": work["flops_gateup"], "launch_ms": res["kernel_ms"]["gate_up"],
            "launch_ms_events_raw": res["kernel_ms_events_raw"]["gate_up"], "event_gap_ms": res["event_gap_ms"],
            "weights": "cold" if res["layers_in_rotation"] > 1 else "warm",
            "down_kernel_frac": (res["down_TFLOPs"] or 0.0) / MFMA_BF16_PEAK_TFLOPS,
            "all_kernels_TFLOPs": res["kernels_TFLOPs"], "all_kernels_frac": res["kernels_TFLOPs"] / MFMA_BF16_PEAK_TFLOPS,
            "operator_TFLOPs": res["operator_TFLOPs"], "operator_frac": res["operator_TFLOPs"] / MFMA_BF16_PEAK_TFLOPS}


def cpu_baseline(block, inputs, tokens, budget_s=12.0):
    """CPU restatement of the reference algorithm on the same workload, timed on this host's
    cores (OpenMP); also the parity gate of the GPU output."""
    import numpy as np

    from oracle import c_oracle

    isz = int(block._packed_intermediate_size)
    rank_out = int(block.shared_u_down.shape[1])
    arrays = [c_oracle.MatrixArray(c_oracle.matrices_from_torch(*block._static_lists(p), dim=isz))
              for p in ("gate", "up", "down")]
    h_gate = inputs["h_gate"].float().cpu().numpy()
    h_up = inputs["h_up"].float().cpu().numpy()
    tok, off, rw = (inputs[k].cpu().numpy() for k in ("tok", "off", "rw"))
    # routing parity (bit-exact) against the C restatement
    g2l = block._packed_global_to_local.cpu().numpy()
    tok_c, off_c, rw_c = c_oracle.route(inputs["selected"].cpu().numpy(), inputs["weights"].cpu().numpy(), g2l,
                                        block._packed_expert_count)
    a = int(off_c[-1])
    routing_ok = bool(np.array_equal(off, off_c) and np.array_equal(tok[:a], tok_c) and np.array_equal(rw[:a], rw_c))
    n_threads = c_oracle.num_threads()
    times = []
    ref = None
    t_begin = time.perf_counter()
    while not times or (time.perf_counter() - t_begin < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        ref = c_oracle.moe_forward(h_gate, h_up, tok[:a], off, rw[:a], arrays[0], arrays[1], arrays[2], rank_out, isz)
        times.append(time.perf_counter() - t0)
    best = min(times)
    got = inputs["out"].cpu().numpy()
    denom = float(np.abs(ref).max()) or 1.0
    err = float(np.abs(got - ref).max()) / denom
    return {"value": tokens / best, "unit": "tokens/s", "cores": n_threads, "kind": "port",
            "sample": f"{len(times)} full forwards of the same workload ({tokens} tokens), best of {len(times)}, "
                      f"{best * 1e3:.1f} ms each; host has {os.cpu_count()} logical CPUs",
            "note": "CPU restatement of the reference algorithm (the reference publishes no CPU path)"}, \
        {"routing_bit_exact": routing_ok, "output_max_norm_err": err, "output_tolerance": 1e-2,
         "output_ok": bool(err <= 1e-2)}


COMPACT_LIMIT = 4096     # bytes: the last stdout line must stay below this


def _r(v, digits=4):
    return round(v, digits) if isinstance(v, float) else v


def compact_line(full):
    """The last stdout line: the contract's fields, the roofline and CPU baseline of the primary workload, and
    per extra workload only {ms_per_step, launch, operator_frac, gateup_frac, down_frac, block_ms}."""
    roof = full.get("roofline") or {}
    keep_roof = ("bound", "kernel", "achieved", "peak", "unit", "frac", "traffic", "launch_ms", "weights",
                 "down_kernel_frac", "operator_frac")
    cpu = full.get("cpu_baseline")
    if cpu:
        cpu = {k: _r(cpu[k], 2) for k in ("value", "unit", "cores", "kind", "sample") if k in cpu}
    extras = {}
    for name, r in (full.get("extras") or {}).items():
        rf = r.get("roofline") or {}
        extras[name] = {"ms_per_step": _r(r.get("ms_per_step"), 5), "launch": r.get("launch"),
                        "operator_frac": _r(rf.get("operator_frac")), "gateup_frac": _r(rf.get("frac")),
                        "down_frac": _r(rf.get("down_kernel_frac")),
                        "block_ms": _r((r.get("block_scope") or {}).get("ms_per_step"), 5)}
    cfg = dict(full.get("config") or {})
    out = {k: full.get(k) for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                    "higher_is_better", "scaling", "vs_baseline", "dtype", "data")}
    out["value"] = _r(out["value"], 1)
    out["ms_per_step"] = _r(out["ms_per_step"], 6)
    out["config"] = cfg
    out["roofline"] = {k: _r(roof[k], 5) for k in keep_roof if k in roof}
    out["cpu_baseline"] = cpu
    out["parity"] = full.get("parity")
    out["block_ms"] = _r((full.get("block_scope") or {}).get("ms_per_step"), 5)
    out["warm_ms_per_step"] = _r((full.get("warm") or {}).get("ms_per_step"), 6)
    out["extras"] = extras
    text = json.dumps(out)
    if len(text) >= COMPACT_LIMIT:       # never let the tail grow past what is kept: drop the least needed first
        for victim in ("extras", "parity", "warm_ms_per_step", "block_ms"):
            out.pop(victim, None)
            if len(json.dumps(out)) < COMPACT_LIMIT:
                break
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)      # (the closing synchronize costs as much as several steps)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2-t64", choices=sorted(WORKLOADS))
    ap.add_argument("--layers", type=int, default=4,
                    help="distinct copies of the layer the decode / prefill workloads cycle through (cold weights); "
                         "1 = replay one layer (warm).  The c5 stack always has its 26 layers")
    ap.add_argument("--no-extras", action="store_true", help="measure the primary workload only")
    ap.add_argument("--no-stack", action="store_true", help="leave the 26-layer c5 stack out of the extras")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay)")
    ap.add_argument("--full-json", default=None,
                    help="where the full record is written (default bench_out/bench_full.json)")
    ap.add_argument("--print-full", action="store_true", help="also print the full record as an earlier stdout line")
    ap.add_argument("--no-warm", action="store_true", help="skip the one-layer (warm) replay of the same workload")
    ap.add_argument("--no-block", action="store_true", help="skip the block-scope timing")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="a library experiment switch for this run, e.g. decode_fused=0 (bitsmoe_set_option)")
    ap.add_argument("--only", default=None, help="comma-separated extras to measure (default: all)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run 5 plain fp32 copies (torch.mul(src, 1, out=dst)) of this many MiB: the known-size "
                         "kernel that hardware byte counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (one process, no collectives); run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    from bitsmoe_amd.algorithms import _HAS_MLP_FORWARD_CUDA, _MLP_FORWARD_IMPORT_ERROR, get_cuda_device_name
    from bitsmoe_amd.synth import SPECS, make_layer

    if not _HAS_MLP_FORWARD_CUDA:
        raise RuntimeError(f"libbitsmoe_hip.so not loadable: {_MLP_FORWARD_IMPORT_ERROR}")
    if not torch.cuda.is_available():
        raise RuntimeError("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    from bitsmoe_amd.algorithms import mlp_forward_cuda as _hip
    for opt in args.option:
        name, _, value = opt.partition("=")
        _hip.set_option(name, int(value))
    use_graph = not args.no_graph
    built = {}       # spec key of the layer shape -> its distinct copies (c2 and c3 are one layer shape and seed)
    build_seconds = {}

    def blocks_of(spec_key, layout="uniform"):
        shape_key = "c2" if spec_key == "c3" else spec_key
        if layout != "uniform":
            shape_key += "/" + layout
        if shape_key not in built:
            spec = SPECS[spec_key]
            n = spec.n_layers if spec.n_layers > 1 else max(1, args.layers)
            t0 = time.perf_counter()
            # (the stack shares its three orthonormal bases between the layers: they are outside the operator
            # and factorising 78 matrices of 2048 x 2048 on the host would take longer than the benchmark)
            built[shape_key] = [make_layer(SPECS[shape_key.split("/")[0]], device=dev, dtype=torch.bfloat16, seed=42, layer_idx=i,
                                           basis_seed=(42 if spec.n_layers > 1 or layout != "uniform" else None),
                                           layout="uniform" if layout == "super2" else layout,
                                           super_experts=(5, 77) if layout == "super2" else ()) for i in range(n)]
            torch.cuda.synchronize()
            build_seconds[id(built[shape_key])] = time.perf_counter() - t0
        return built[shape_key]

    def measure(name, steps, warmup):
        skey, toks, bnd = WORKLOADS[name]
        # "-ckpt-": the same shape with checkpoint-shaped matrices (three widths per matrix, ragged slabs,
        # dropped ranks) instead of one width per expert
        blocks = blocks_of(skey, "checkpoint" if "-ckpt-" in name else "super2" if "-super2-" in name else "uniform")
        stack = SPECS[skey].n_layers > 1
        if stack:       # one step = one pass over the whole stack
            r, inp = run_workload(blocks, SPECS[skey], toks, max(2, steps // len(blocks)), max(1, warmup // len(blocks)),
                                  use_graph=use_graph, layers_per_step=len(blocks), block_scope=not args.no_block)
        else:
            r, inp = run_workload(blocks, SPECS[skey], toks, steps, warmup, use_graph=use_graph,
                                  block_scope=not args.no_block)
        r["roofline"] = roofline_of(r, inp, bnd, name)
        if len(blocks) > 1 and not stack and not args.no_warm:
            # the same workload replaying ONE layer: weights may stay in the memory-side cache
            w, winp = run_workload(blocks[:1], SPECS[skey], toks, steps, warmup, use_graph=use_graph, block_scope=False)
            r["warm"] = {k: w[k] for k in ("ms_per_step", "tokens_per_s", "launch", "kernel_ms", "gateup_GBps", "down_GBps",
                                           "gateup_TFLOPs", "down_TFLOPs", "operator_GBps", "operator_TFLOPs")}
            r["warm"]["roofline_frac"] = roofline_of(w, winp, bnd, name)["frac"]
        return r, inp, blocks

    spec_key, tokens, bound = WORKLOADS[args.workload]
    res, inputs, blocks = measure(args.workload, args.steps, args.warmup)
    roof = res.pop("roofline")
    block = blocks[0]
    if args.copy_probe_mib > 0:
        n = args.copy_probe_mib * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    cpu, parity = (None, None)
    if not args.no_cpu:
        cpu, parity = cpu_baseline(block, inputs, tokens)
    extras = {}
    if not args.no_extras:
        for name, (skey, toks, bnd) in WORKLOADS.items():
            if name == args.workload or (args.no_stack and SPECS[skey].n_layers > 1):
                continue
            if args.only is not None and name not in args.only.split(","):
                continue
            r, _, _ = measure(name, max(5, args.steps // 2), max(2, args.warmup // 2))
            extras[name] = r
    bits = block.expert_bits
    shape_key = "c2" if spec_key == "c3" else spec_key
    line = {
        "metric": "MoE-layer tokens/s", "value": res["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": res["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {WORKLOAD_DESC[spec_key]}, {tokens} tokens, operator scope "
                               "(routing + gate/up + SiLU*mul + down + combine), inputs resident in HBM, "
                               f"{res['layers_in_rotation']} distinct layers in rotation "
                               f"({'cold' if res['layers_in_rotation'] > 1 else 'warm'} weights)",
                   "tokens": tokens, "mean_bits": sum(bits) / len(bits), "active_experts": res["active_experts"],
                   "device": get_cuda_device_name(), "layer_build_s": round(build_seconds[id(blocks)], 2),
                   "launch": res["launch"], "routing": res["routing"], "fused_kernel": bool(res.get("fused")),
                   "activation_dtype": "bf16",
                   "arithmetic": "bf16 activations in, f16 MFMA operands, fp32 accumulation"},
        "eager_ms_per_step": res["eager_ms_per_step"], "hipgraph_ms_per_step": res["hipgraph_ms_per_step"],
        "block_scope": res.get("block_scope"), "warm": res.get("warm"),
        "kernel_ms": res["kernel_ms"], "algorithmic_bytes": res["algorithmic_bytes"],
        "algorithmic_flops": res["algorithmic_flops"],
        "roofline": roof, "cpu_baseline": cpu, "parity": parity, "extras": extras,
    }
    # The full record (every workload with all its fields) goes to a file and to an EARLIER stdout line; the
    # LAST line is the compact one, small enough for any harness that keeps only the tail of stdout.
    full_path = args.full_json or os.path.join(ROOT, "bench_out", "bench_full.json")
    try:
        os.makedirs(os.path.dirname(full_path), exist_ok=True)
        with open(full_path, "w") as f:
            json.dump(line, f, indent=1)
    except OSError as exc:
        print(f"bench.py: full record not written ({exc})", file=sys.stderr)
    if args.print_full:
        print(json.dumps(line))
    print(json.dumps(compact_line(line)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
