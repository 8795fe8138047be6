"""In-kernel timelines of the decode kernels (a diagnostic, not part of the operator).

    python -m bitsmoe_amd.build --timeline
    BITSMOE_LIB_VARIANT=timeline python -m bitsmoe_amd.timeline --workload c2 --tokens 64 [--kernels two|fused]

The timeline build of the library stamps the 100 MHz wall clock at the phase boundaries of every workgroup's first
assignment chunk.  This script builds the synthetic layer of the named benchmark shape, runs the forward over a
rotation of distinct layers (cold weights), reads the stamps of ONE forward and prints, in microseconds, when
workgroups start and end relative to the kernel's first start and how long each phase lasts.
  --kernels two    (default) the gate/up kernel and the down kernel of the two-kernel decode forward
  --kernels prefill  the grouped-GEMM kernels k_gateup_mfma / k_down_mfma (use with a prefill-sized --tokens)
  --kernels fused  the one-kernel forward (option decode_fused = 1): tables + routing scan | gate + up walk (per slab
                   group: operand staged | barrier | multiplied) | z + barrier | down + atomics
"""
from __future__ import annotations

import argparse
import ctypes
import statistics
import sys

STAMPS = 64
PHASES = ("tables+route", "gate walk", "up walk", "z+barrier", "down+atomics")


def _pct(values, q):
    values = sorted(values)
    return values[min(len(values) - 1, int(q * len(values)))]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="c2", help="layer shape of the benchmark set (c1, c2, c4, c5)")
    ap.add_argument("--tokens", type=int, default=64)
    ap.add_argument("--layers", type=int, default=4)
    ap.add_argument("--kernels", default="two", choices=("two", "fused", "prefill"))
    args = ap.parse_args()

    import torch

    from bitsmoe_amd.algorithms import _capi, mlp_forward_cuda as hip
    from bitsmoe_amd.synth import SPECS, draw_selected, make_layer

    lib = _capi.load()
    if not hasattr(lib, "bitsmoe_timeline_read"):
        print("this library has no time stamps: build with `python -m bitsmoe_amd.build --timeline` and run with "
              "BITSMOE_LIB_VARIANT=timeline", file=sys.stderr)
        return 2
    lib.bitsmoe_timeline_read.restype = ctypes.c_int32
    lib.bitsmoe_timeline_read.argtypes = [ctypes.c_void_p, ctypes.c_int32]
    lib.bitsmoe_timeline_clear.restype = ctypes.c_int32
    lib.bitsmoe_timeline_read_decode.restype = ctypes.c_int32
    lib.bitsmoe_timeline_read_decode.argtypes = [ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32]
    lib.bitsmoe_timeline_clear_decode.restype = ctypes.c_int32
    hip.set_option("decode_fused", 1 if args.kernels == "fused" else 0)
    dev = torch.device("cuda:0")
    spec = SPECS[args.workload]
    n_layers = spec.n_layers if spec.n_layers > 1 else args.layers
    blocks = [make_layer(spec, device=dev, dtype=torch.bfloat16, seed=42, layer_idx=i,
                         basis_seed=42 if spec.n_layers > 1 else None) for i in range(min(n_layers, 6))]
    states = []
    for i, block in enumerate(blocks):
        block._ensure_runtime_cache(dev)
        sets = block._ensure_matsets()
        g = torch.Generator().manual_seed(42 + 17 * i + args.tokens)
        x = torch.randn((args.tokens, spec.hidden_size), generator=g).to(torch.bfloat16).to(dev)
        vh_gate, vh_up, _ = block._shared_basis(torch.bfloat16)
        sel, w = draw_selected(spec, args.tokens, 42 + 17 * i + 1000 + args.tokens, dev)
        states.append((block, sets, (x @ vh_gate.T).contiguous(), (x @ vh_up.T).contiguous(), sel, w))

    def step(i):
        block, sets, hg, hu, sel, w = states[i % len(states)]
        return hip.moe_forward_routed(hg, hu, sel, w, block._packed_global_to_local, block._packed_local_to_global, *sets,
                                      int(block.shared_u_down.shape[1]), int(block._packed_intermediate_size), 0)

    for i in range(3 * len(states)):
        step(i)
    torch.cuda.synchronize()
    block, sets, hg, hu, sel, w = states[0]
    us = lambda ticks: ticks / 100.0
    if args.kernels == "prefill":
        lib.bitsmoe_timeline_read_prefill.restype = ctypes.c_int32
        lib.bitsmoe_timeline_read_prefill.argtypes = [ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32]
        lib.bitsmoe_timeline_clear_prefill.restype = ctypes.c_int32
        _capi.check(lib.bitsmoe_timeline_clear_prefill())
        step(0)
        torch.cuda.synchronize()
        print(f"workload {args.workload} T={args.tokens}, grouped-GEMM kernels (the first 8192 workgroups of each launch)")
        first_start = None
        for which, kname in ((0, "k_gateup_mfma"), (1, "k_down_mfma")):
            n = 8192
            raw = (ctypes.c_uint64 * (8 * n))()
            _capi.check(lib.bitsmoe_timeline_read_prefill(which, raw, n))
            rows = [raw[8 * i:8 * i + 8] for i in range(n)]
            started = [r for r in rows if r[0]]
            worked = [r for r in started if r[6] and r[3] and r[2] and r[1]]
            if not worked:
                print(f"  {kname}: did not run")
                continue
            t0 = min(r[0] for r in started)
            first_start = t0 if first_start is None else first_start
            print(f"  {kname}: {len(started)} workgroups started, {len(worked)} had a tile; first start {us(t0 - first_start):.2f} us "
                  f"after the first kernel's; span {us(max(r[6] or r[0] for r in started) - t0):.2f} us")
            for label, vals in (("start", [us(r[0] - t0) for r in worked]), ("end", [us(r[6] - t0) for r in worked])):
                print(f"    {label:>14}: p10 {_pct(vals, 0.1):7.2f}  p50 {_pct(vals, 0.5):7.2f}  p90 {_pct(vals, 0.9):7.2f}  max {max(vals):7.2f}")
            for label, lo, hi in (("tables", 0, 1), ("first loads", 1, 2), ("steps", 2, 3), ("epilogue", 3, 6), ("lifetime", 0, 6)):
                vals = [us(r[hi] - r[lo]) for r in worked]
                print(f"    {label:>14}: mean {statistics.mean(vals):7.2f}  p10 {_pct(vals, 0.1):7.2f}  p50 {_pct(vals, 0.5):7.2f}  "
                      f"p90 {_pct(vals, 0.9):7.2f}  max {max(vals):7.2f}")
        return 0
    if args.kernels == "two":
        _capi.check(lib.bitsmoe_timeline_clear_decode())
        step(0)
        torch.cuda.synchronize()
        print(f"workload {args.workload} T={args.tokens}, two-kernel decode forward "
              f"(routing {'inside the kernels' if hip.routed_is_inline(hg, hu, int(sel.shape[1]), *sets) else 'by a kernel first'})")
        names = {0: ("k_gateup_walk", [("tables+route", 0, 1), ("walk+store", 1, 2)]),
                 1: ("k_down_decode", [("tables+route", 0, 1), ("z+barrier", 1, 2), ("tiles", 2, 3), ("atomics", 3, 4)])}
        first_start = None
        for which in (0, 1):
            n = 8192
            raw = (ctypes.c_uint64 * (8 * n))()
            _capi.check(lib.bitsmoe_timeline_read_decode(which, raw, n))
            rows = [raw[8 * i:8 * i + 8] for i in range(n)]
            started = [r for r in rows if r[0]]
            worked = [r for r in started if r[6] and r[1]]
            if not started:
                print(f"  {names[which][0]}: did not run (the launcher chose another kernel)")
                continue
            t0 = min(r[0] for r in started)
            first_start = t0 if first_start is None else first_start
            print(f"  {names[which][0]}: {len(started)} workgroups started, {len(worked)} had assignments; first start "
                  f"{us(t0 - first_start):.2f} us after the forward's first; span {us(max(r[6] or r[0] for r in started) - t0):.2f} us")
            for label, vals in (("start", [us(r[0] - t0) for r in worked]), ("end", [us(r[6] - t0) for r in worked])):
                print(f"    {label:>14}: p10 {_pct(vals, 0.1):6.2f}  p50 {_pct(vals, 0.5):6.2f}  p90 {_pct(vals, 0.9):6.2f}  max {max(vals):6.2f}")
            for label, lo, hi in names[which][1]:
                vals = [us(r[hi] - r[lo]) for r in worked if r[hi] and r[lo]]
                if vals:
                    print(f"    {label:>14}: mean {statistics.mean(vals):6.2f}  p10 {_pct(vals, 0.1):6.2f}  p50 {_pct(vals, 0.5):6.2f}  "
                          f"p90 {_pct(vals, 0.9):6.2f}  max {max(vals):6.2f}")
            life = [us(r[6] - r[0]) for r in worked]
            print(f"    {'lifetime':>14}: mean {statistics.mean(life):6.2f}  p10 {_pct(life, 0.1):6.2f}  p50 {_pct(life, 0.5):6.2f}  "
                  f"p90 {_pct(life, 0.9):6.2f}  max {max(life):6.2f}")
        return 0
    if not hip.decode_is_fused(hg, hu, int(sel.numel()), *sets):
        print("this workload does not run the one-kernel forward", file=sys.stderr)
        return 2
    _capi.check(lib.bitsmoe_timeline_clear())
    step(0)          # layer 0 again after the others have passed through the caches
    torch.cuda.synchronize()
    n_wg = min(4096, int(block._packed_expert_count) * ((int(block._packed_intermediate_size) + 127) // 128) * 2)
    raw = (ctypes.c_uint64 * (STAMPS * n_wg))()
    _capi.check(lib.bitsmoe_timeline_read(raw, n_wg))
    rows = [raw[STAMPS * i:STAMPS * (i + 1)] for i in range(n_wg)]
    started = [r for r in rows if r[0]]
    worked = [r for r in started if r[6] and r[5] and r[4] and r[3] and r[1]]
    t0 = min(r[0] for r in started)
    print(f"workload {args.workload} T={args.tokens}, one-kernel forward: {len(started)} workgroups started, {len(worked)} had assignments")
    print(f"kernel span (first start to last end): {us(max(r[6] or r[0] for r in started) - t0):.2f} us")
    for name, vals in (("start", [us(r[0] - t0) for r in worked]), ("end", [us(r[6] - t0) for r in worked])):
        print(f"  {name:>14}: p10 {_pct(vals, 0.1):6.2f}  p50 {_pct(vals, 0.5):6.2f}  p90 {_pct(vals, 0.9):6.2f}  max {max(vals):6.2f}")
    # (experts whose three matrices share one width walk gate and up as one sequence: no stamp between them)
    single = [r for r in worked if not r[2]]
    spans = [("tables+route", 0, 1, worked), ("gate+up walk", 1, 3, single), ("gate walk", 1, 2, [r for r in worked if r[2]]),
             ("up walk", 2, 3, [r for r in worked if r[2]]), ("z+barrier", 3, 4, worked), ("down+atomics", 4, 5, worked)]
    for name, lo, hi, group in spans:
        if not group:
            continue
        vals = [us(r[hi] - r[lo]) for r in group]
        print(f"  {name:>14}: mean {statistics.mean(vals):6.2f}  p10 {_pct(vals, 0.1):6.2f}  p50 {_pct(vals, 0.5):6.2f}  "
              f"p90 {_pct(vals, 0.9):6.2f}  max {max(vals):6.2f}")
    # inside the one walk: per slab group, from its start to the staged operand, the barrier, the end of its MFMAs
    for vg in range(12):
        grp = [r for r in single if r[8 + 4 * vg] and r[8 + 4 * vg + 3]]
        if not grp:
            continue
        b = 8 + 4 * vg
        parts = [statistics.mean(us(r[b + k + 1] - r[b + k]) for r in grp) for k in range(3)]
        nxt = [us(r[b + 4] - r[b + 3]) for r in grp if vg < 11 and r[b + 4]]
        print(f"  group {vg:2d}: stage {parts[0]:5.2f}  barrier {parts[1]:5.2f}  multiply {parts[2]:5.2f}"
              + (f"  (to next start {statistics.mean(nxt):5.2f})" if nxt else ""))
    life = [us(r[6] - r[0]) for r in worked]
    print(f"  {'lifetime':>14}: mean {statistics.mean(life):6.2f}  p10 {_pct(life, 0.1):6.2f}  p50 {_pct(life, 0.5):6.2f}  "
          f"p90 {_pct(life, 0.9):6.2f}  max {max(life):6.2f}")
    per_xcd = {}
    for r in worked:
        per_xcd[r[7] >> 32] = per_xcd.get(r[7] >> 32, 0) + 1
    print("  workgroups with work per XCD:", " ".join(f"{k}:{v}" for k, v in sorted(per_xcd.items())))
    return 0


if __name__ == "__main__":
    sys.exit(main())
