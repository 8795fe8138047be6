#!/usr/bin/env python3
"""Benchmark of the mixed-bit MoE routed-expert path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2-t64] [--no-extras] [--no-cpu]

A "step" is one pass of the hot path over one batch that is already resident in HBM:
routing/permute kernel -> gate & up -> SiLU*mul -> down -> top-k weighted combine
(operator scope: from the router's top-k ids to rank_accum [T, rank_out]).  The layer is
synthetic (random-init factors of the named shape, quantised and packed on the GPU).

Prints ONE JSON line.  `value` is tokens/s of the primary workload (default: the
Qwen3-30B-A3B-shaped layer at decode, 64 tokens); `extras` holds the other decode batch
sizes and the 4096-token prefill; `roofline` is the dominant kernel of the primary workload
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
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16 MFMA peak, TFLOP/s

WORKLOADS = {
    # name: (spec key, tokens, roofline bound)
    "c2-t1": ("c2", 1, "hbm"),
    "c2-t8": ("c2", 8, "hbm"),
    "c2-t32": ("c2", 32, "hbm"),
    "c2-t64": ("c2", 64, "hbm"),
    "c3-t4096": ("c3", 4096, "mfma"),
}
WORKLOAD_DESC = {
    "c2": "Qwen3-30B-A3B-shaped MoE layer (128 experts, top-8, hidden 2048, intermediate 768, mixed 2/3/4-bit, group 128)",
    "c3": "Qwen3-30B-A3B-shaped MoE layer (128 experts, top-8, hidden 2048, intermediate 768, mixed 2/3/4-bit, group 128)",
}


def matrix_bytes(lists, e):
    payload, rank_idx, tile_meta, slab_meta, scale, s = lists
    return (payload[e].numel() * 4 + scale[e].numel() * 2 + s[e].numel() * 2 + rank_idx[e].numel() * 4
            + slab_meta[e].numel() * 4 + tile_meta[e].numel() * 4)


def algorithmic_work(block, counts, tokens, n_assign):
    """Algorithmic bytes (per kernel) and FLOPs of one forward for the ACTUAL active experts."""
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
    return {"bytes_gateup": b_gateup, "bytes_down": b_down, "bytes_total": b_gateup + b_down,
            "flops": flops, "flops_gateup": fl_gateup, "flops_down": flops - fl_gateup, "active_experts": len(active)}


def run_workload(block, spec, tokens, steps, warmup, seed=42, use_graph=True):
    import torch

    from bitsmoe_amd.algorithms import mlp_forward_cuda as hip
    from bitsmoe_amd.synth import draw_selected

    dev = block._runtime_device()
    block._ensure_runtime_cache(dev)
    gate, up, down = block._ensure_matsets()
    g = torch.Generator().manual_seed(seed + tokens)
    x = torch.randn((tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(dev)
    vh_gate, vh_up, _ = block._shared_basis(torch.bfloat16)
    h_gate = (x @ vh_gate.T).contiguous()
    h_up = (x @ vh_up.T).contiguous()
    selected, weights = draw_selected(spec, tokens, seed + 1000 + tokens, dev)
    rank_out = int(block.shared_u_down.shape[1])
    isz = int(block._packed_intermediate_size)
    g2l = block._packed_global_to_local
    n_packed = block._packed_expert_count

    def step(profile=None):
        tok, off, rw = hip.route(selected, weights, g2l, n_packed)
        out = hip.moe_forward_sets(h_gate, h_up, tok, off, rw, gate, up, down, rank_out, isz, 0, profile=profile)
        return tok, off, rw, out

    for _ in range(max(warmup, 1)):
        tok, off, rw, out = step()
    torch.cuda.synchronize(dev)
    # (1) eager launches, no instrumentation: what a caller of the operator sees per call
    t0 = time.perf_counter()
    for i in range(steps):
        step()
    torch.cuda.synchronize(dev)
    eager = time.perf_counter() - t0
    # (2) the same steps with HIP events between the kernels (per-kernel durations for the roofline)
    profiles = [hip.Profile() for _ in range(steps)]
    for i in range(steps):
        step(profiles[i])
    torch.cuda.synchronize(dev)
    # (3) the step captured once into a HIP graph and replayed: the operator never allocates or
    # synchronises, so a serving loop can drop the per-launch host cost this way
    elapsed, launch, graph_ms = eager, "eager", None
    if use_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            with torch.cuda.stream(side):
                step()
            torch.cuda.current_stream(dev).wait_stream(side)
            torch.cuda.synchronize(dev)
            with torch.cuda.graph(graph):
                g_tok, g_off, g_rw, g_out = step()
            # every replay must reproduce the eager result (fp32 atomics: summation order may differ)
            for _ in range(3):
                graph.replay()
                torch.cuda.synchronize(dev)
                ref_out = step()[3]
                torch.cuda.synchronize(dev)
                if not torch.allclose(g_out, ref_out, rtol=1e-4, atol=1e-5 * float(ref_out.abs().max())):
                    raise RuntimeError("graph replay differs from the eager result")
            for _ in range(max(warmup, 1)):
                graph.replay()
            torch.cuda.synchronize(dev)
            t0 = time.perf_counter()
            for i in range(steps):
                graph.replay()
            torch.cuda.synchronize(dev)
            replay = time.perf_counter() - t0
            if replay < eager:       # large steps hide the launch cost anyway and replay has its own
                elapsed, launch = replay, "hipgraph"
            graph_ms = replay / steps * 1e3
        except Exception as exc:   # noqa: BLE001 - the eager figure stands
            print(f"bench.py: graph replay unavailable ({exc}); reporting eager launches", file=sys.stderr)
    phases = [p.read() for p in profiles]
    # phases of the operator: preparation (with the routing launch before it), gate/up kernel,
    # SiLU pass, down kernel, combine (third and fifth: launches of their own at prefill only)
    ms_fill, ms_gateup, ms_silu, ms_down, ms_combine = (sum(p[i] for p in phases) / steps for i in range(5))
    ms_all = ms_fill + ms_gateup + ms_silu + ms_down + ms_combine
    counts = (off[1:] - off[:-1]).cpu().tolist()
    work = algorithmic_work(block, counts, tokens, int(tok.numel()))
    res = {
        "tokens": tokens, "ms_per_step": elapsed / steps * 1e3, "tokens_per_s": tokens * steps / elapsed,
        "launch": launch, "eager_ms_per_step": eager / steps * 1e3, "hipgraph_ms_per_step": graph_ms,
        "kernel_ms": {"prepare": ms_fill, "gate_up": ms_gateup, "silu_mul": ms_silu, "down": ms_down,
                      "combine": ms_combine},
        "active_experts": work["active_experts"], "algorithmic_bytes": work["bytes_total"],
        "algorithmic_flops": work["flops"],
        "gateup_GBps": work["bytes_gateup"] / (ms_gateup * 1e-3) / 1e9 if ms_gateup > 0 else None,
        "down_GBps": work["bytes_down"] / (ms_down * 1e-3) / 1e9 if ms_down > 0 else None,
        "kernels_GBps": work["bytes_total"] / (ms_all * 1e-3) / 1e9,
        "kernels_TFLOPs": work["flops"] / (ms_all * 1e-3) / 1e12,
        "gateup_TFLOPs": work["flops_gateup"] / (ms_gateup * 1e-3) / 1e12 if ms_gateup > 0 else None,
        "down_TFLOPs": work["flops_down"] / (ms_down * 1e-3) / 1e12 if ms_down > 0 else None,
    }
    # block scope: router + the two shared-basis GEMMs + the operator + the output projection
    # (torch / hipBLASLt for everything around the operator), reported beside the operator figure
    xb = x.reshape(1, tokens, -1)
    with torch.no_grad():
        for _ in range(3):
            block(xb)
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        for _ in range(steps):
            block(xb)
        torch.cuda.synchronize(dev)
    block_s = (time.perf_counter() - t0) / steps
    res["block_scope"] = {"ms_per_step": block_s * 1e3, "tokens_per_s": tokens / block_s, "launch": "eager",
                          "eager_ms_per_step": block_s * 1e3,
                          "note": "whole MoE block forward on its own router"}
    if use_graph:
        try:       # the block forward has no host synchronisation either: capture and replay it
            bgraph = torch.cuda.CUDAGraph()
            with torch.no_grad():
                with torch.cuda.graph(bgraph):
                    yb = block(xb)
                yb = yb[0] if isinstance(yb, tuple) else yb
                for _ in range(3):
                    bgraph.replay()
                    torch.cuda.synchronize(dev)
                    ye = block(xb)
                    ye = ye[0] if isinstance(ye, tuple) else ye
                    torch.cuda.synchronize(dev)
                    if not torch.allclose(yb.float(), ye.float(), rtol=2e-2, atol=2e-2 * float(ye.float().abs().max())):
                        raise RuntimeError("block graph replay differs from the eager result")
                t0 = time.perf_counter()
                for _ in range(steps):
                    bgraph.replay()
                torch.cuda.synchronize(dev)
            replay_s = (time.perf_counter() - t0) / steps
            res["block_scope"]["hipgraph_ms_per_step"] = replay_s * 1e3
            if replay_s < block_s:
                res["block_scope"].update(ms_per_step=replay_s * 1e3, tokens_per_s=tokens / replay_s, launch="hipgraph")
        except Exception as exc:   # noqa: BLE001
            print(f"bench.py: block graph replay unavailable ({exc})", file=sys.stderr)
    inputs = {"h_gate": h_gate, "h_up": h_up, "tok": tok, "off": off, "rw": rw, "out": out, "work": work,
              "selected": selected, "weights": weights}
    return res, inputs


# HBM bytes per launch of the dominant kernel from hardware counters (FETCH_SIZE + WRITE_SIZE,
# each scaled by what it reads for a 256 MiB copy); collected offline with rocprofv3 --pmc on
# this same script (profiles/*_hbm_traffic_counters.txt), None where not collected.
HBM_TRAFFIC_BYTES = {"c2-t64": int((59366.5 * 2.0 + 3584.0) * 1024),         # k_gateup_walk
                     "c3-t4096": int((268522.9 * 2.0 + 98304.0) * 1024)}     # k_gateup_mfma


def roofline_of(res, inputs, bound, workload=None):
    work = inputs["work"]
    traffic = HBM_TRAFFIC_BYTES.get(workload)
    if bound == "hbm":
        # dominant kernel at decode: the fused gate+up launch (two thirds of the weight bytes)
        achieved = res["gateup_GBps"]
        return {"bound": "hbm", "kernel": "gate_up", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                "algorithmic_bytes_per_launch": work["bytes_gateup"], "launch_ms": res["kernel_ms"]["gate_up"],
                "all_kernels_GBps": res["kernels_GBps"], "all_kernels_frac": res["kernels_GBps"] / HBM_PEAK_GBS}
    achieved = res["gateup_TFLOPs"]
    return {"bound": "mfma", "kernel": "gate_up", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": traffic,
            "algorithmic_flops_per_launch": work["flops_gateup"], "launch_ms": res["kernel_ms"]["gate_up"],
            "all_kernels_TFLOPs": res["kernels_TFLOPs"], "all_kernels_frac": res["kernels_TFLOPs"] / MFMA_BF16_PEAK_TFLOPS}


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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)      # (the closing synchronize costs as much as several steps)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2-t64", choices=sorted(WORKLOADS))
    ap.add_argument("--no-extras", action="store_true", help="measure the primary workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity leg")
    ap.add_argument("--no-graph", action="store_true", help="time eager launches only (no HIP graph replay)")
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
    spec_key, tokens, bound = WORKLOADS[args.workload]
    t0 = time.perf_counter()
    block = make_layer(SPECS[spec_key], device=dev, dtype=torch.bfloat16, seed=42)
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0

    res, inputs = run_workload(block, SPECS[spec_key], tokens, args.steps, args.warmup, use_graph=not args.no_graph)
    roof = roofline_of(res, inputs, bound, args.workload)
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
            if name == args.workload:
                continue
            # c2 and c3 are the same layer (same seed, shape and bit draw); only routing differs
            r, inp = run_workload(block, SPECS[skey], toks, max(5, args.steps // 2), max(2, args.warmup // 2),
                                  use_graph=not args.no_graph)
            r["roofline"] = roofline_of(r, inp, bnd, name)
            extras[name] = r
    bits = block.expert_bits
    line = {
        "metric": "MoE-layer tokens/s", "value": res["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": res["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {WORKLOAD_DESC[spec_key]}, {tokens} tokens, operator scope "
                               "(routing kernel + gate/up + SiLU*mul + down + combine), inputs resident in HBM",
                   "tokens": tokens, "mean_bits": sum(bits) / len(bits), "active_experts": res["active_experts"],
                   "device": get_cuda_device_name(), "layer_build_s": round(build_s, 2),
                   "launch": res["launch"]},
        "eager_ms_per_step": res["eager_ms_per_step"], "hipgraph_ms_per_step": res["hipgraph_ms_per_step"],
        "block_scope": res["block_scope"],
        "kernel_ms": res["kernel_ms"], "algorithmic_bytes": res["algorithmic_bytes"],
        "algorithmic_flops": res["algorithmic_flops"],
        "roofline": roof, "cpu_baseline": cpu, "parity": parity, "extras": extras,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
