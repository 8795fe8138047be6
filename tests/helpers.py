"""Shared test helpers: small packed layers built with the oracle packer, conversions
between the oracle's numpy dicts and device tensors, error metrics."""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np

from oracle import ref_oracle as o

BUF_KEYS = ("payload", "rank_idx", "tile_meta", "slab_meta", "scale", "s")


def random_segments(rng: np.random.Generator, rank: int, choices=(2, 3, 4), n_cuts: int = 3, drop: bool = False,
                    multiple: int = 1):
    if multiple > 1:       # cut only at multiples so that every slab is full
        units = rank // multiple
        cuts = sorted(set(int(c) * multiple for c in rng.integers(1, max(units, 2), size=n_cuts))) if units > 1 else []
        cuts = [c for c in cuts if 0 < c < rank]
    else:
        cuts = sorted(set(int(c) for c in rng.integers(1, rank, size=n_cuts))) if rank > 1 else []
    edges = [0] + cuts + [rank]
    segs = []
    for a, b in zip(edges[:-1], edges[1:]):
        bits = int(rng.choice(choices))
        segs.append((bits, (a, b)))
    if drop and len(segs) > 1:
        segs[0] = (0, segs[0][1])          # rows of a 0-bit segment are dropped by the packer
    return segs


def make_matrix(rng, rank: int, dim: int, segments, s_mode="rand", std=0.02) -> Dict[str, np.ndarray]:
    w = rng.normal(0.0, std, size=(rank, dim)).astype(np.float32)
    s = rng.uniform(0.5, 1.5, size=rank).astype(np.float32) if s_mode == "rand" else np.ones(rank, np.float32)
    m = o.pack_matrix(w, s, segments)
    m["source"] = w
    return m


def make_experts(seed: int, n_experts: int, rank_in: int, rank_out: int, dim: int, choices=(2, 3, 4),
                 uniform_bits: bool = False, s_mode="rand", permute_rank: bool = False, slab_multiple=None):
    """gate/up/down lists of oracle matrices.  gate/up rows index h columns [0, rank_in);
    down rows index output ranks [0, rank_out)."""
    rng = np.random.default_rng(seed)
    gate, up, down = [], [], []
    for _ in range(n_experts):
        for lst, rank in ((gate, rank_in), (up, rank_in), (down, rank_out)):
            if uniform_bits:
                segs = [(int(rng.choice(choices)), (0, rank))]
            else:
                segs = random_segments(rng, rank, choices, multiple=slab_multiple or 1)
            lst.append(make_matrix(rng, rank, dim, segs, s_mode=s_mode))
    return gate, up, down


def to_device_lists(mats: Sequence[Dict[str, np.ndarray]], device):
    import torch

    out = {k: [] for k in BUF_KEYS}
    for m in mats:
        out["payload"].append(torch.from_numpy(m["payload"].view(np.int32).copy()).view(torch.uint32).to(device))
        out["rank_idx"].append(torch.from_numpy(m["rank_idx"].astype(np.int32)).to(device))
        out["tile_meta"].append(torch.from_numpy(m["tile_meta"].astype(np.int32).reshape(-1, 3)).to(device))
        out["slab_meta"].append(torch.from_numpy(m["slab_meta"].astype(np.int32).reshape(-1, 4)).to(device))
        out["scale"].append(torch.from_numpy(m["scale"].astype(np.float16)).to(device))
        out["s"].append(torch.from_numpy(m["s"].astype(np.float16)).to(device))
    return tuple(tuple(out[k]) for k in BUF_KEYS)


def from_torch_matrix(payload, rank_idx, tile_meta, slab_meta, scale, s, dim: int) -> Dict[str, np.ndarray]:
    """Device buffers of one packed matrix -> the oracle's dict."""
    import torch

    return {
        "payload": payload.detach().cpu().view(torch.int32).numpy().view(np.uint32),
        "rank_idx": rank_idx.detach().cpu().numpy().astype(np.int32),
        "tile_meta": tile_meta.detach().cpu().numpy().astype(np.int32).reshape(-1, 3),
        "slab_meta": slab_meta.detach().cpu().numpy().astype(np.int32).reshape(-1, 4),
        "scale": scale.detach().cpu().numpy().astype(np.float16),
        "s": s.detach().cpu().numpy().astype(np.float16),
        "dim": int(dim),
    }


def norm_err(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| / max |ref| — the layer-output parity metric."""
    denom = float(np.max(np.abs(ref)))
    return float(np.max(np.abs(np.asarray(got, dtype=np.float64) - ref))) / (denom if denom > 0 else 1.0)


def bf16_round(x: np.ndarray) -> np.ndarray:
    return o._round_to(np.asarray(x, dtype=np.float64), "bf16").astype(np.float32)
