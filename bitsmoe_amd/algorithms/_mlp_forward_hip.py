"""Packed routed-expert forward on gfx950: the operator module.

Mirrors the reference's pybind module `bitsmoe.algorithms._mlp_forward_cuda`
(bitsmoe/algorithms/cpp/mlp_forward_binding.cpp:157-189): `moe_packed_forward` takes the
same 26 arguments in the same order, applies the same checks with the same messages
(mlp_forward_binding.cpp:80-126) and returns fp32 `[tokens, rank_out]`.  The work is done
by libbitsmoe_hip.so through its C ABI; torch only supplies device memory and the stream.

Additions the reference does not have: bf16 activations, an explicit `MatrixSet` handle
(the reference caches the equivalent tables keyed on raw pointers,
bitsmoe/algorithms/cpp/mlp_forward.cu:2464-2503), `route`, `dequant_matrix`.
"""
from __future__ import annotations

import ctypes
import operator
import os
from collections import OrderedDict
from typing import List, Optional, Sequence, Tuple

import torch

from . import _capi

_lib = _capi.load()
# BITSMOE_NO_PREPARE=1 keeps every matrix set on the generic kernels (no wave-native copy)
_AUTO_PREPARE = os.environ.get("BITSMOE_NO_PREPARE", "0") != "1"


def set_option(name: str, value: int = -1) -> None:
    """One of the launchers' experiment switches for the whole process ("route_inline", "route_jobs",
    "decode_fused_z", "decode_split_z", "decode_fused", "prefill_split", "router_wide"): 0 / 1, or -1 for the library's own choice.  The
    library reads the BITSMOE_* environment forms of these once, when it is loaded."""
    _capi.check(_lib.bitsmoe_set_option(name.encode(), int(value)))


def _stream_ptr(device: torch.device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


class MatrixSet:
    """The packed matrices of every expert for one projection (gate, up or down).

    Owns a `bitsmoe_matset` handle; keeps the tensors alive for the handle's lifetime.
    """

    def __init__(self, payload: Sequence[torch.Tensor], rank_idx: Sequence[torch.Tensor],
                 tile_meta: Sequence[torch.Tensor], slab_meta: Sequence[torch.Tensor],
                 scale: Sequence[torch.Tensor], s: Sequence[torch.Tensor],
                 intermediate_size: int, name: str = "payload"):
        n = len(payload)
        for lst, what in ((rank_idx, "rank_idx"), (tile_meta, "tile_meta"), (slab_meta, "slab_meta"),
                          (scale, "scale"), (s, "s")):
            _check(len(lst) == n, f"{name}: {what} list length {len(lst)} != {n}")
        self._keep = (tuple(payload), tuple(rank_idx), tuple(tile_meta), tuple(slab_meta), tuple(scale), tuple(s))
        self._keep_lists = self._keep
        self._name = name
        self._fingerprint = fingerprint(self._keep)
        self.n_experts = n
        self.intermediate_size = int(intermediate_size)
        self.device = payload[0].device if n else torch.device("cuda", torch.cuda.current_device())
        descs = (_capi.MatrixDesc * max(n, 1))()
        for i in range(n):
            p, rk, tm, sm, sc, sv = payload[i], rank_idx[i], tile_meta[i], slab_meta[i], scale[i], s[i]
            for t, what, dt in ((p, "payload", torch.uint32), (rk, "rank_idx", torch.int32),
                                (tm, "tile_meta", torch.int32), (sm, "slab_meta", torch.int32),
                                (sc, "scale", torch.float16), (sv, "s_buffer", torch.float16)):
                _check(t.is_cuda, f"{what} must be CUDA")
                _check(t.is_contiguous(), f"{what} must be contiguous")
                _check(t.dtype == dt, f"{what} must be {str(dt).replace('torch.', '')}")
            _check(rk.dim() == 1, "rank_idx must be 1D")
            _check(sc.dim() == 1, "scale must be 1D")
            _check(sv.dim() == 1, "s_buffer must be 1D")
            _check(tm.dim() == 2 and tm.shape[1] == 3, "tile_meta must be [N,3]")
            _check(sm.dim() == 2 and sm.shape[1] == 4, "slab_meta must be [N,4]")
            _check(sv.numel() == rk.numel(), "s_buffer and rank_idx lengths differ")
            d = descs[i]
            d.payload, d.rank_idx, d.tile_meta = p.data_ptr(), rk.data_ptr(), tm.data_ptr()
            d.slab_meta, d.scale, d.s = sm.data_ptr(), sc.data_ptr(), sv.data_ptr()
            d.payload_words, d.scale_len = p.numel(), sc.numel()
            d.rank_len, d.num_tiles, d.num_slabs = rk.numel(), tm.shape[0], sm.shape[0]
        handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            _capi.check(_lib.bitsmoe_matset_create(descs, n, self.intermediate_size,
                                                   _stream_ptr(self.device), ctypes.byref(handle)))
        self._handle = handle
        info = (ctypes.c_int64 * 8)()
        _capi.check(_lib.bitsmoe_matset_info(handle, info))
        self.total_slabs = int(info[2])
        self.max_rank_plus1 = int(info[3])
        self.regular = bool(info[4])
        self.fast_capable = bool(int(info[7]) & 1)   # the wave-native fast kernels can take this set
        self.role = -1                               # -1 until prepare() has re-laid the payload out
        self.wide_slabs = 0                          # 64-row slabs of 6/8/16-bit rows in the prepared set's side table

    @property
    def handle(self) -> ctypes.c_void_p:
        return self._handle

    def prepare(self, role: int) -> bool:
        """One-time re-layout of the payload for the fast kernels (role 0: gate/up, 1: down).
        Returns False (and leaves the set on the generic kernels) when the layout is not regular."""
        if self.role == role:
            return True
        if not self.fast_capable or self.role >= 0:
            return False
        with torch.cuda.device(self.device):
            _capi.check(_lib.bitsmoe_matset_prepare(self._handle, int(role), _stream_ptr(self.device)))
        self.role = int(role)
        info = (ctypes.c_int64 * 8)()
        _capi.check(_lib.bitsmoe_matset_info(self._handle, info))
        self.wide_slabs = int(info[7]) >> 8
        return True

    def is_current(self) -> bool:
        """False once any buffer the set was built from has been written in place since (the set
        is a snapshot: validated metadata, prepared payload copy, folded scales)."""
        return self._fingerprint == fingerprint(self._keep)

    def payload_current(self) -> bool:
        """The cheap form of is_current(): only the payload tensors' version counters are compared."""
        return self._fingerprint[:self.n_experts] == fingerprint(self._keep[:1])

    def refresh(self) -> None:
        """Rebuild the snapshot from the buffers' current contents (same tensors, same role)."""
        role = self.role
        self.close()
        self.__init__(*self._keep, intermediate_size=self.intermediate_size, name=self._name)
        if role >= 0:
            self.prepare(role)

    def dequant_prepared(self, expert: int) -> torch.Tensor:
        """Dense fp32 matrix decoded from the prepared (wave-native) copy."""
        out = torch.zeros((self.rank_len(expert), self.intermediate_size), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            _capi.check(_lib.bitsmoe_dequant_matrix_prepared(self._handle, int(expert), out.data_ptr(),
                                                             _stream_ptr(self.device)))
        return out

    def rank_len(self, expert: int) -> int:
        return int(self._keep[1][expert].numel())

    def dequant(self, expert: int) -> torch.Tensor:
        """Dense fp32 [rank_len, intermediate_size] of one expert matrix (local row order)."""
        out = torch.empty((self.rank_len(expert), self.intermediate_size), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            _capi.check(_lib.bitsmoe_dequant_matrix(self._handle, int(expert), out.data_ptr(), _stream_ptr(self.device)))
        return out

    def close(self) -> None:
        if getattr(self, "_handle", None):
            _lib.bitsmoe_matset_destroy(self._handle)
            self._handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Profile:
    """Per-phase HIP-event timing of one forward, in ms: preparation, gate/up kernel, SiLU pass,
    down kernel, combine (the third and fifth are launches of their own only on the grouped-GEMM path)."""

    def __init__(self):
        h = ctypes.c_void_p()
        _capi.check(_lib.bitsmoe_profile_create(ctypes.byref(h)))
        self._handle = h

    def read(self) -> Tuple[float, ...]:
        ms = (ctypes.c_float * _capi.PROFILE_PHASES)()
        _capi.check(_lib.bitsmoe_profile_read(self._handle, ms))
        return tuple(float(v) for v in ms)

    def __del__(self):
        try:
            if self._handle:
                _lib.bitsmoe_profile_destroy(self._handle)
                self._handle = None
        except Exception:
            pass


# ----------------------------------------------------------------------------------------
# matrix-set cache for the list-based reference signature
# ----------------------------------------------------------------------------------------
# A MatrixSet is a SNAPSHOT of the caller's buffers: creation validates and caches the metadata,
# prepare() makes a re-laid-out copy of the payload and a folded scale table.  The reference keeps
# only meta tables per raw pointer and reads the payload live
# (bitsmoe/algorithms/cpp/mlp_forward.cu:2464-2503, 2608-2619), so a caller of the list signature
# may overwrite or swap buffers between calls.  Two levels:
#   1. the six container objects of a projection are looked up by identity (the block's runtime cache holds
#      stable tuples, bitsmoe/models/base_block.py:195-214); a hit is confirmed by a cheap staleness token --
#      mutable containers: every element still the same tensor object; all containers: the version counters
#      of the PAYLOAD tensors (any reload or re-quantisation writes them) -- about 35 us per call for 3 x 128
#      experts instead of milliseconds for
#   2. the full fingerprint: address, size and version counter of EVERY tensor of EVERY expert, taken on a
#      level-1 miss (new containers, a swapped expert, a payload written in place) and on every call with
#      BITSMOE_LIST_CACHE_CHECK=full; a fingerprint miss builds a fresh set.
# BITSMOE_LIST_CACHE_CHECK=identity trusts the containers alone.  Inference tensors carry no version
# counter: they are keyed by address and size only, and an in-place write to them needs
# clear_matset_cache() (or MatrixSet.refresh()).
_SET_CACHE: "OrderedDict[tuple, MatrixSet]" = OrderedDict()
_SET_CACHE_LIMIT = int(os.environ.get("BITSMOE_SET_CACHE_LIMIT", "384"))     # sets kept (each pins its GPU copy)
_LIST_CACHE_CHECK = os.environ.get("BITSMOE_LIST_CACHE_CHECK", "payload")
if _LIST_CACHE_CHECK not in ("payload", "full", "identity"):
    raise RuntimeError(f"BITSMOE_LIST_CACHE_CHECK={_LIST_CACHE_CHECK!r}: expected payload, full or identity")
_IDENT_CACHE: "dict[tuple, tuple]" = {}     # ids of the six containers -> (containers, element snapshots, token, set)
_is = operator.is_


def clear_matset_cache() -> None:
    for ms in _SET_CACHE.values():
        ms.close()
    _SET_CACHE.clear()
    _IDENT_CACHE.clear()


def _version(t: torch.Tensor) -> int:
    """Version counter of a tensor; inference tensors have none (reading it raises)."""
    return -1 if t.is_inference() else t._version


def fingerprint(lists: Sequence[Sequence[torch.Tensor]]) -> tuple:
    """(address, element count, version counter) of every tensor of the six buffer lists."""
    return tuple((t.data_ptr(), t.numel(), _version(t)) for seq in lists for t in seq)


def _payload_token(payload: Sequence[torch.Tensor]) -> tuple:
    try:
        return tuple(map(_get_version, payload))
    except RuntimeError:       # an inference tensor among them
        return tuple(map(_version, payload))


_get_version = operator.attrgetter("_version")


def _lookup_set(lists: tuple, intermediate_size: int, name: str) -> MatrixSet:
    ident = (int(intermediate_size),) + tuple(map(id, lists))
    hit = _IDENT_CACHE.get(ident) if _LIST_CACHE_CHECK != "full" else None
    if hit is not None:
        containers, snaps, token, ms = hit
        if ms._handle and all(map(_is, containers, lists)) and all(
                isinstance(cur, tuple) or (len(cur) == len(snap) and all(map(_is, snap, cur)))
                for snap, cur in zip(snaps, lists)) and (
                _LIST_CACHE_CHECK == "identity" or token == _payload_token(lists[0])):
            return ms
        del _IDENT_CACHE[ident]
    key = (len(lists[0]), int(intermediate_size), fingerprint(lists))
    ms = _SET_CACHE.get(key)
    if ms is not None:
        _SET_CACHE.move_to_end(key)
    else:
        # a set built from the same list objects or the same first payload address whose key no longer
        # matches is stale (its buffers were overwritten or swapped): release its GPU copy now
        for old_key, old in list(_SET_CACHE.items()):
            if all(a is b for a, b in zip(old._keep_lists, lists)) or (
                    len(lists[0]) and old.n_experts and old._keep[0][0].data_ptr() == lists[0][0].data_ptr()):
                old.close()
                del _SET_CACHE[old_key]
        ms = MatrixSet(*lists, intermediate_size=intermediate_size, name=name)
        ms._keep_lists = lists
        while len(_SET_CACHE) >= max(_SET_CACHE_LIMIT, 1):
            _SET_CACHE.popitem(last=False)[1].close()
        # the set holds the tensors themselves, so no address of the key can be recycled while it lives
        _SET_CACHE[key] = ms
    if len(_IDENT_CACHE) >= 4 * max(_SET_CACHE_LIMIT, 1):
        _IDENT_CACHE.clear()
    # (the entry holds the containers, so their ids cannot be recycled while it lives)
    _IDENT_CACHE[ident] = (lists, tuple(tuple(seq) for seq in lists), _payload_token(lists[0]), ms)
    return ms


_WORKSPACES = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """A per-(device, stream) scratch buffer that only grows; reused across calls."""
    key = (device.index, _stream_ptr(device))
    buf = _WORKSPACES.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty((max(nbytes, 1 << 20),), dtype=torch.uint8, device=device)
        _WORKSPACES[key] = buf
    return buf


def moe_forward_sets(h_gate: torch.Tensor, h_up: torch.Tensor, token_indices: torch.Tensor,
                     expert_offsets: torch.Tensor, route_weights: torch.Tensor, gate: MatrixSet,
                     up: MatrixSet, down: MatrixSet, rank_out: int, intermediate_size: int,
                     act_type: int = 0, path: int = _capi.PATH_AUTO,
                     profile: Optional[Profile] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The forward over explicit matrix sets.  Returns rank_accum fp32 [tokens, rank_out].
    h_gate / h_up may be column ranges of a wider row-major tensor (unit column stride)."""
    _check(h_gate.dim() == 2 and h_up.dim() == 2 and h_gate.stride(1) == 1 and h_up.stride(1) == 1,
           "h_gate/h_up must be 2D with unit column stride")
    dev = h_gate.device
    n_tokens = int(h_gate.shape[0])
    n_assign = int(token_indices.numel())
    dt = _capi.DT_F16 if h_gate.dtype == torch.float16 else _capi.DT_BF16
    if path != _capi.PATH_GENERIC and _AUTO_PREPARE and gate.role < 0 and up.role < 0 and down.role < 0:
        # first use: lay the payloads out for the fast kernels (one-time, allocates the copy)
        if gate.fast_capable and up.fast_capable and down.fast_capable:
            gate.prepare(0)
            up.prepare(0)
            down.prepare(1)
    if out is None:
        out = torch.empty((n_tokens, int(rank_out)), dtype=torch.float32, device=dev)
    nbytes = int(_lib.bitsmoe_forward_workspace_bytes_sets(gate.handle, up.handle, down.handle, n_tokens,
                                                           n_assign, int(path)))
    ws = _workspace(dev, nbytes)
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_moe_forward_strided(
            gate.handle, up.handle, down.handle, h_gate.data_ptr(), h_up.data_ptr(), dt, n_tokens,
            int(h_gate.shape[1]), int(h_up.shape[1]), int(h_gate.stride(0)) if n_tokens > 1 else int(h_gate.shape[1]),
            int(h_up.stride(0)) if n_tokens > 1 else int(h_up.shape[1]),
            token_indices.data_ptr(), expert_offsets.data_ptr(),
            route_weights.data_ptr(), n_assign, int(rank_out), int(intermediate_size), int(act_type),
            int(path), out.data_ptr(), ws.data_ptr(), ws.numel(),
            profile._handle if profile is not None else None, _stream_ptr(dev)))
    return out


def routed_is_inline(h_gate: torch.Tensor, h_up: torch.Tensor, top_k: int, gate: MatrixSet, up: MatrixSet, down: MatrixSet,
                     path: int = _capi.PATH_AUTO) -> bool:
    """Would moe_forward_routed run these activations without a routing kernel?"""
    n_tokens = int(h_gate.shape[0])
    return bool(_lib.bitsmoe_forward_routed_is_inline(
        gate.handle, up.handle, down.handle, h_gate.data_ptr(), h_up.data_ptr(), int(h_gate.shape[1]), int(h_up.shape[1]),
        int(h_gate.stride(0)) if n_tokens > 1 else int(h_gate.shape[1]),
        int(h_up.stride(0)) if n_tokens > 1 else int(h_up.shape[1]), n_tokens, int(top_k), int(path)))


def decode_is_fused(h_gate: torch.Tensor, h_up: torch.Tensor, n_assign: int, gate: MatrixSet, up: MatrixSet, down: MatrixSet,
                    path: int = _capi.PATH_AUTO) -> bool:
    """Would a forward over n_assign assignments run as one kernel per (expert, tile) (no gate/up and down launches)?"""
    n_tokens = int(h_gate.shape[0])
    return bool(_lib.bitsmoe_forward_decode_is_fused(
        gate.handle, up.handle, down.handle, h_gate.data_ptr(), h_up.data_ptr(), int(h_gate.shape[1]), int(h_up.shape[1]),
        int(h_gate.stride(0)) if n_tokens > 1 else int(h_gate.shape[1]),
        int(h_up.stride(0)) if n_tokens > 1 else int(h_up.shape[1]), int(n_assign), int(path)))


def moe_forward_routed(h_gate: torch.Tensor, h_up: torch.Tensor, selected: torch.Tensor, weights: torch.Tensor,
                       global_to_local: torch.Tensor, local_to_global: torch.Tensor, gate: MatrixSet, up: MatrixSet,
                       down: MatrixSet, rank_out: int, intermediate_size: int, act_type: int = 0,
                       path: int = _capi.PATH_AUTO, profile: Optional[Profile] = None,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Routing and forward in one call, from the router's output: selected [T, k] expert ids (int32 / int64) and
    weights fp32 [T, k]; global_to_local int32 [n_global] (-1: not a packed expert) and its inverse
    local_to_global int32 [n_experts].  Small batches run without any routing kernel (the forward's kernels find
    their assignments themselves); otherwise the routing tables are built first.  Returns rank_accum fp32
    [tokens, rank_out], equal to moe_forward_sets(*route(...)) up to the order of fp32 atomics."""
    _check(h_gate.dim() == 2 and h_up.dim() == 2 and h_gate.stride(1) == 1 and h_up.stride(1) == 1,
           "h_gate/h_up must be 2D with unit column stride")
    _check(selected.dim() == 2 and selected.shape == weights.shape and selected.shape[0] == h_gate.shape[0],
           "selected and weights must be [tokens, top_k]")
    _check(selected.dtype in (torch.int32, torch.int64), "selected must be int32 or int64")
    _check(weights.dtype == torch.float32 and global_to_local.dtype == torch.int32 and local_to_global.dtype == torch.int32,
           "weights must be float32, the id maps int32")
    dev = h_gate.device
    selected = selected.contiguous()
    weights = weights.contiguous()
    n_tokens, top_k = int(selected.shape[0]), int(selected.shape[1])
    dt = _capi.DT_F16 if h_gate.dtype == torch.float16 else _capi.DT_BF16
    if path != _capi.PATH_GENERIC and _AUTO_PREPARE and gate.role < 0 and up.role < 0 and down.role < 0:
        if gate.fast_capable and up.fast_capable and down.fast_capable:
            gate.prepare(0)
            up.prepare(0)
            down.prepare(1)
    if out is None:
        out = torch.empty((n_tokens, int(rank_out)), dtype=torch.float32, device=dev)
    nbytes = int(_lib.bitsmoe_forward_routed_workspace_bytes(gate.handle, up.handle, down.handle, n_tokens, top_k, int(path)))
    ws = _workspace(dev, nbytes)
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_moe_forward_routed(
            gate.handle, up.handle, down.handle, h_gate.data_ptr(), h_up.data_ptr(), dt, n_tokens,
            int(h_gate.shape[1]), int(h_up.shape[1]), int(h_gate.stride(0)) if n_tokens > 1 else int(h_gate.shape[1]),
            int(h_up.stride(0)) if n_tokens > 1 else int(h_up.shape[1]),
            selected.data_ptr(), 1 if selected.dtype == torch.int64 else 0, weights.data_ptr(), top_k,
            global_to_local.data_ptr(), int(global_to_local.numel()), local_to_global.data_ptr(),
            int(rank_out), int(intermediate_size), int(act_type), int(path), out.data_ptr(), ws.data_ptr(), ws.numel(),
            profile._handle if profile is not None else None, _stream_ptr(dev)))
    return out


def _check_cuda_contig(t: torch.Tensor, name: str) -> None:
    _check(t.is_cuda, f"{name} must be CUDA tensor")
    _check(t.is_contiguous(), f"{name} must be contiguous")


def moe_packed_forward(h_gate, h_up, token_indices, expert_offsets, route_weights,
                       gate_payload, gate_rank_idx, gate_tile_meta, gate_slab_meta, gate_scale, gate_s,
                       up_payload, up_rank_idx, up_tile_meta, up_slab_meta, up_scale, up_s,
                       down_payload, down_rank_idx, down_tile_meta, down_slab_meta, down_scale, down_s,
                       rank_out, intermediate_size, act_type):
    """Packed routed-expert forward (same signature as the reference operator)."""
    _check(h_gate.dim() == 2, "h_gate must be 2D [tokens, rank]")
    _check(h_up.dim() == 2, "h_up must be 2D [tokens, rank]")
    _check(h_gate.shape[0] == h_up.shape[0], "h_gate/h_up token dim mismatch")
    _check(token_indices.dim() == 1, "token_indices must be 1D")
    _check(expert_offsets.dim() == 1, "expert_offsets must be 1D")
    _check(route_weights.dim() == 1, "route_weights must be 1D")
    _check_cuda_contig(h_gate, "h_gate")
    _check_cuda_contig(h_up, "h_up")
    _check_cuda_contig(token_indices, "token_indices")
    _check_cuda_contig(expert_offsets, "expert_offsets")
    _check_cuda_contig(route_weights, "route_weights")
    _check(h_gate.dtype in (torch.float16, torch.bfloat16), "h_gate must be float16 or bfloat16")
    _check(h_up.dtype == h_gate.dtype, "h_up must have the dtype of h_gate")
    _check(token_indices.dtype == torch.int32, "token_indices must be int32")
    _check(expert_offsets.dtype == torch.int32, "expert_offsets must be int32")
    _check(route_weights.dtype == torch.float32, "route_weights must be float32")
    num_experts = expert_offsets.numel() - 1
    _check(num_experts >= 0, "expert_offsets must have length >= 1")
    _check(token_indices.numel() == route_weights.numel(), "token_indices/route_weights size mismatch")
    for lst, name in (
        (gate_payload, "gate_payload"), (gate_rank_idx, "gate_rank_idx"), (gate_tile_meta, "gate_tile_meta"),
        (gate_slab_meta, "gate_slab_meta"), (gate_scale, "gate_scale"), (gate_s, "gate_s"),
        (up_payload, "up_payload"), (up_rank_idx, "up_rank_idx"), (up_tile_meta, "up_tile_meta"),
        (up_slab_meta, "up_slab_meta"), (up_scale, "up_scale"), (up_s, "up_s"),
        (down_payload, "down_payload"), (down_rank_idx, "down_rank_idx"), (down_tile_meta, "down_tile_meta"),
        (down_slab_meta, "down_slab_meta"), (down_scale, "down_scale"), (down_s, "down_s"),
    ):
        _check(len(lst) == num_experts, f"{name} size mismatch, expected {num_experts}, got {len(lst)}")
    _check(intermediate_size > 0, "intermediate_size must be > 0")
    _check(rank_out > 0, "rank_out must be > 0")
    _check(act_type == 0, "only SiLU act_type=0 is currently supported")

    n_tokens = int(h_gate.shape[0])
    if token_indices.numel() == 0 or num_experts == 0:
        return torch.zeros((n_tokens, int(rank_out)), dtype=torch.float32, device=h_gate.device)

    gate = _lookup_set((gate_payload, gate_rank_idx, gate_tile_meta, gate_slab_meta, gate_scale, gate_s),
                       int(intermediate_size), "gate_payload")
    up = _lookup_set((up_payload, up_rank_idx, up_tile_meta, up_slab_meta, up_scale, up_s),
                     int(intermediate_size), "up_payload")
    down = _lookup_set((down_payload, down_rank_idx, down_tile_meta, down_slab_meta, down_scale, down_s),
                       int(intermediate_size), "down_payload")
    return moe_forward_sets(h_gate, h_up, token_indices, expert_offsets, route_weights, gate, up, down,
                            int(rank_out), int(intermediate_size), int(act_type))


def route(selected_experts: torch.Tensor, route_weights: torch.Tensor, global_to_local: torch.Tensor,
          n_packed: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Device-side routing tables from top-k ids [T,k] and fp32 weights [T,k]:
    (token_indices int32 [T*k], expert_offsets int32 [n_packed+1], route_flat fp32 [T*k]).
    Entries mapped to a negative local id are dropped; the kept count is
    expert_offsets[-1] (stays on the device) and only that prefix of the outputs is defined."""
    _check(selected_experts.dim() == 2 and route_weights.shape == selected_experts.shape,
           "selected_experts / route_weights must be [tokens, top_k]")
    _check(selected_experts.dtype in (torch.int32, torch.int64), "selected_experts must be int32 or int64")
    _check(route_weights.dtype == torch.float32, "route_weights must be float32")
    _check(global_to_local.dtype == torch.int32, "global_to_local must be int32")
    dev = selected_experts.device
    sel = selected_experts.contiguous()
    w = route_weights.contiguous()
    t, k = int(sel.shape[0]), int(sel.shape[1])
    n_flat = t * k
    token_indices = torch.empty((n_flat,), dtype=torch.int32, device=dev)
    route_flat = torch.empty((n_flat,), dtype=torch.float32, device=dev)
    expert_offsets = torch.empty((int(n_packed) + 1,), dtype=torch.int32, device=dev)
    nbytes = int(_lib.bitsmoe_route_workspace_bytes(n_flat, int(n_packed)))
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_route(
            sel.data_ptr(), 1 if sel.dtype == torch.int64 else 0, w.data_ptr(), global_to_local.data_ptr(),
            int(global_to_local.numel()), t, k, int(n_packed), token_indices.data_ptr(),
            expert_offsets.data_ptr(), route_flat.data_ptr(), ws.data_ptr(), ws.numel(), _stream_ptr(dev)))
    return token_indices, expert_offsets, route_flat


def pack_bitplanes(levels: torch.Tensor, bits: int) -> torch.Tensor:
    """int8 [rows, cols] -> uint32 [rows, ceil(cols/32)*bits] on the device."""
    rows, cols = int(levels.shape[0]), int(levels.shape[1])
    groups = (cols + 31) // 32
    out = torch.empty((rows, groups * bits), dtype=torch.uint32, device=levels.device)
    with torch.cuda.device(levels.device):
        _capi.check(_lib.bitsmoe_pack_bitplanes(levels.data_ptr(), rows, cols, int(bits), out.data_ptr(),
                                                _stream_ptr(levels.device)))
    return out


def unpack_bitplanes(words: torch.Tensor, bits: int) -> torch.Tensor:
    """uint32 [rows, groups*bits] -> int8 [rows, groups*32] on the device."""
    rows = int(words.shape[0])
    groups = int(words.shape[1]) // int(bits)
    out = torch.empty((rows, groups * 32), dtype=torch.int8, device=words.device)
    with torch.cuda.device(words.device):
        _capi.check(_lib.bitsmoe_unpack_bitplanes(words.data_ptr(), rows, groups, int(bits), out.data_ptr(),
                                                  _stream_ptr(words.device)))
    return out


def quantize_tiles(rows: torch.Tensor, bits: int, iters: int = 50) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp32 [k, dim] -> (levels int8 [k, ceil(dim/128)*128], scale fp32 [k, ceil(dim/128)]): the symmetric
    quantiser per (row, 128-column tile), one wavefront each."""
    _check(rows.dim() == 2 and rows.is_cuda and rows.dtype == torch.float32 and rows.stride(1) == 1,
           "rows must be a CUDA fp32 matrix with unit column stride")
    k, dim = int(rows.shape[0]), int(rows.shape[1])
    n_tiles = (dim + 127) // 128
    levels = torch.empty((k, n_tiles * 128), dtype=torch.int8, device=rows.device)
    scale = torch.empty((k, n_tiles), dtype=torch.float32, device=rows.device)
    with torch.cuda.device(rows.device):
        _capi.check(_lib.bitsmoe_quantize_tiles(rows.data_ptr(), k, dim, int(rows.stride(0)) if k > 1 else dim, int(bits),
                                                int(iters), levels.data_ptr(), scale.data_ptr(), _stream_ptr(rows.device)))
    return levels, scale


def pack_slabs(levels: torch.Tensor, scale: torch.Tensor, dim: int, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Levels / scales of one bit bucket (quantize_tiles) -> (payload uint32 words in runtime order for the
    bucket's slabs of <= 64 rows, fp16 scales [slab][tile][row])."""
    k = int(levels.shape[0])
    n_tiles = (int(dim) + 127) // 128
    _check(levels.is_cuda and levels.dtype == torch.int8 and levels.is_contiguous() and levels.shape[1] == n_tiles * 128,
           "levels must be a contiguous CUDA int8 [k, ceil(dim/128)*128] tensor")
    _check(scale.dtype == torch.float32 and scale.is_contiguous() and tuple(scale.shape) == (k, n_tiles),
           "scale must be contiguous fp32 [k, ceil(dim/128)]")
    payload = torch.empty((k * n_tiles * 4 * int(bits),), dtype=torch.uint32, device=levels.device)
    scale16 = torch.empty((k * n_tiles,), dtype=torch.float16, device=levels.device)
    with torch.cuda.device(levels.device):
        _capi.check(_lib.bitsmoe_pack_slabs(levels.data_ptr(), scale.data_ptr(), k, int(dim), int(bits), payload.data_ptr(),
                                            scale16.data_ptr(), _stream_ptr(levels.device)))
    return payload, scale16


def router_softmax_topk(router_logits: torch.Tensor, top_k: int, renormalize: bool = True,
                        round_dtype: Optional[torch.dtype] = None, weight_scale: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """softmax (fp32) -> top-k -> optional renormalisation -> * weight_scale -> optional round trip through
    `round_dtype`, in one kernel.  The logits may be a column range of a wider row-major tensor (unit column
    stride).  Returns (selected int64 [T, k], weights fp32 [T, k])."""
    _check(router_logits.dim() == 2, "router_logits must be [tokens, experts]")
    _check(router_logits.is_cuda, "router_logits must be CUDA tensor")
    _check(router_logits.dtype in (torch.float16, torch.bfloat16, torch.float32), "router_logits must be a float tensor")
    _check(round_dtype in (None, torch.float16, torch.bfloat16), "round_dtype must be None, float16 or bfloat16")
    dev = router_logits.device
    logits = router_logits if router_logits.stride(1) == 1 else router_logits.contiguous()
    t, e = int(logits.shape[0]), int(logits.shape[1])
    ld = int(logits.stride(0)) if t > 1 else e
    selected = torch.empty((t, int(top_k)), dtype=torch.int64, device=dev)
    weights = torch.empty((t, int(top_k)), dtype=torch.float32, device=dev)
    codes = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_router_softmax_topk_strided(
            logits.data_ptr(), codes[logits.dtype], ld, t, e, int(top_k), 1 if renormalize else 0, float(weight_scale),
            -1 if round_dtype is None else codes[round_dtype], selected.data_ptr(), 1, weights.data_ptr(),
            _stream_ptr(dev)))
    return selected, weights


def router_linear_topk_possible(hidden: torch.Tensor, weight, top_k: int) -> bool:
    """Can router_linear_topk take these tensors?  (16-bit hidden states [T, K] with unit column stride and 16-byte
    aligned rows, a contiguous weight [E, K] of the same dtype -- or a PreparedLinearWeight of it --, K a multiple of
    128, at most 256 experts.)"""
    if isinstance(weight, PreparedLinearWeight):
        w_dtype, e, k = weight.dtype, weight.out_features, weight.in_features
    else:
        if not (weight.dim() == 2 and weight.is_contiguous() and weight.data_ptr() % 16 == 0):
            return False
        w_dtype, e, k = weight.dtype, int(weight.shape[0]), int(weight.shape[1])
    return (hidden.is_cuda and hidden.dim() == 2 and hidden.dtype in (torch.float16, torch.bfloat16) and w_dtype == hidden.dtype
            and hidden.stride(1) == 1 and int(hidden.shape[1]) == k and k % 128 == 0
            and (int(hidden.shape[0]) <= 1 or int(hidden.stride(0)) % 8 == 0) and hidden.data_ptr() % 16 == 0
            and 1 <= int(top_k) <= min(64, e) and e <= 256)


def router_linear_topk(hidden: torch.Tensor, weight, top_k: int, renormalize: bool = True,
                       round_dtype: Optional[torch.dtype] = None, weight_scale: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """The router's linear layer with fp32 logits (hidden.float() @ weight.float().T: exact products of 16-bit values,
    fp32 sums), softmax, top-k, optional renormalisation, * weight_scale, optional round trip through `round_dtype`:
    ONE kernel, no logits in memory.  `weight`: a tensor [E, K] or a PreparedLinearWeight of it (the same sums in the same
    order from consecutive memory).  Returns (selected int64 [T, k], weights fp32 [T, k])."""
    _check(router_linear_topk_possible(hidden, weight, top_k), "router_linear_topk: unsupported shapes, dtypes or alignment")
    _check(round_dtype in (None, torch.float16, torch.bfloat16), "round_dtype must be None, float16 or bfloat16")
    dev = hidden.device
    prepared = isinstance(weight, PreparedLinearWeight)
    t, k_dim = int(hidden.shape[0]), int(hidden.shape[1])
    e = weight.out_features if prepared else int(weight.shape[0])
    selected = torch.empty((t, int(top_k)), dtype=torch.int64, device=dev)
    weights = torch.empty((t, int(top_k)), dtype=torch.float32, device=dev)
    codes = {torch.float16: 0, torch.bfloat16: 1}
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_router_linear_topk(
            hidden.data_ptr(), codes[hidden.dtype], int(hidden.stride(0)) if t > 1 else k_dim,
            weight.data.data_ptr() if prepared else weight.data_ptr(), 1 if prepared else 0, t, k_dim, e,
            int(top_k), 1 if renormalize else 0, float(weight_scale), -1 if round_dtype is None else codes[round_dtype],
            selected.data_ptr(), 1, weights.data_ptr(), _stream_ptr(dev)))
    return selected, weights


def prepared_linear_weight_of(owner, weight: torch.Tensor) -> "PreparedLinearWeight":
    """The PreparedLinearWeight of `weight`, cached on `owner` (any object) and remade when the tensor is rebound or
    written in place (address and version counter)."""
    stamp = (weight.data_ptr(), -1 if weight.is_inference() else weight._version, tuple(weight.shape), weight.dtype)
    cached = getattr(owner, "_bitsmoe_prepared_weight", None)
    if cached is None or cached[0] != stamp:
        cached = (stamp, PreparedLinearWeight(weight.detach()))
        try:
            object.__setattr__(owner, "_bitsmoe_prepared_weight", cached)
        except (AttributeError, TypeError):
            pass
    return cached[1]


SKINNY_LINEAR_MAX_ROWS = 64


class PreparedLinearWeight:
    """A weight [N, K] re-laid out once into the order the few-rows kernel's MFMAs take it (every load of a wavefront
    is then 1 KB of consecutive memory).  A snapshot of the weight's values."""

    def __init__(self, weight: torch.Tensor):
        _check(weight.is_cuda and weight.dim() == 2 and weight.dtype in (torch.float16, torch.bfloat16) and weight.is_contiguous()
               and int(weight.shape[1]) % 128 == 0 and int(weight.shape[0]) >= 1 and weight.data_ptr() % 16 == 0,
               "PreparedLinearWeight: a contiguous 16-bit CUDA weight [N, K] with K a multiple of 128")
        self.out_features, self.in_features = int(weight.shape[0]), int(weight.shape[1])
        self.dtype, self.device = weight.dtype, weight.device
        n = int(_lib.bitsmoe_prepared_linear_weight_elements(self.in_features, self.out_features))
        self.data = torch.empty((n,), dtype=weight.dtype, device=weight.device)
        with torch.cuda.device(weight.device):
            _capi.check(_lib.bitsmoe_prepare_linear_weight(weight.data_ptr(), self.in_features, self.out_features,
                                                           self.data.data_ptr(), _stream_ptr(weight.device)))


def skinny_linear_possible(x: torch.Tensor, weight) -> bool:
    """Can skinny_linear take these tensors?  (at most 64 rows of x [T, K] in the weight's 16-bit dtype -- or at most 16
    rows of fp32, rounded to that dtype inside the kernel -- with unit column stride and 16-byte aligned rows, a
    contiguous weight [N, K], K a multiple of 128, N even; a PreparedLinearWeight: at most 16 rows.)"""
    prepared = isinstance(weight, PreparedLinearWeight)
    if prepared:
        w_dtype, n, k = weight.dtype, weight.out_features, weight.in_features
        if n % 2 != 0:
            return False
    else:
        if not (weight.dim() == 2 and weight.dtype in (torch.float16, torch.bfloat16) and weight.is_contiguous()
                and weight.data_ptr() % 16 == 0 and int(weight.shape[0]) % 2 == 0):
            return False
        w_dtype, n, k = weight.dtype, int(weight.shape[0]), int(weight.shape[1])
    if not (x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and int(x.shape[1]) == k and k % 128 == 0 and x.data_ptr() % 16 == 0):
        return False
    rows = int(x.shape[0])
    if x.dtype == torch.float32:
        return 1 <= rows <= 16 and (rows <= 1 or int(x.stride(0)) % 4 == 0)
    return x.dtype == w_dtype and 1 <= rows <= SKINNY_LINEAR_MAX_ROWS and (rows <= 1 or int(x.stride(0)) % 8 == 0)


def skinny_linear(x: torch.Tensor, weight, addend: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x @ weight.T for a few rows (a bias-free linear layer at decode sizes): the weight is streamed once at HBM speed,
    fp32 sums in a fixed order, result in the weight's dtype.  fp32 x (at most 16 rows) is rounded to that dtype first,
    inside the kernel: x.to(weight.dtype) @ weight.T without the cast's own pass.  `weight`: a tensor [N, K] or a
    PreparedLinearWeight.  `addend`: fp32 [T, N] added to the sums before the result is rounded."""
    _check(skinny_linear_possible(x, weight), "skinny_linear: unsupported shapes, dtypes or alignment")
    dev = x.device
    prepared = isinstance(weight, PreparedLinearWeight)
    w_dtype = weight.dtype
    t, k = int(x.shape[0]), int(x.shape[1])
    n = weight.out_features if prepared else int(weight.shape[0])
    out = torch.empty((t, n), dtype=w_dtype, device=dev)
    w_ptr = weight.data.data_ptr() if prepared else weight.data_ptr()
    if addend is not None:
        _check(addend.dtype == torch.float32 and tuple(addend.shape) == (t, n) and addend.stride(1) == 1 and addend.device == dev,
               "skinny_linear: addend must be float32 [T, N] with unit column stride on x's device")
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_skinny_linear(x.data_ptr(), _capi.DT_F16 if w_dtype == torch.float16 else _capi.DT_BF16,
                                               1 if x.dtype == torch.float32 else 0, int(x.stride(0)) if t > 1 else k, w_ptr,
                                               1 if prepared else 0, t, k, n, out.data_ptr(), n,
                                               None if addend is None else addend.data_ptr(),
                                               0 if addend is None else (int(addend.stride(0)) if t > 1 else n), _stream_ptr(dev)))
    return out


def block_finish(rank_accum: torch.Tensor, dtype: torch.dtype, shared_gate_out: Optional[torch.Tensor] = None,
                 shared_up_out: Optional[torch.Tensor] = None, shared_gate_logit: Optional[torch.Tensor] = None) -> torch.Tensor:
    """[T, rank_out + I_sh] in `dtype`: rank_accum cast, beside it silu(gate_out) * up_out (* sigmoid(gate_logit)) of an
    always-on shared expert -- the operand of the block's single output GEMM.  gate_out / up_out [T, I_sh] may be
    column ranges of one wider tensor (same row stride), gate_logit [T, 1] likewise."""
    _check(rank_accum.dtype == torch.float32 and rank_accum.is_contiguous(), "rank_accum must be contiguous float32")
    _check(dtype in (torch.float16, torch.bfloat16), "dtype must be float16 or bfloat16")
    t, r = int(rank_accum.shape[0]), int(rank_accum.shape[1])
    i_sh = 0 if shared_gate_out is None else int(shared_gate_out.shape[1])
    dev = rank_accum.device
    out = torch.empty((t, r + i_sh), dtype=dtype, device=dev)
    ld_sh = ld_g = 0
    if i_sh:
        _check(shared_up_out is not None and shared_up_out.shape == shared_gate_out.shape and shared_gate_out.dtype == dtype
               and shared_up_out.dtype == dtype and shared_gate_out.stride(1) == 1 and shared_up_out.stride(1) == 1,
               "shared_gate_out / shared_up_out must be [T, I_sh] of the activation dtype with unit column stride")
        ld_sh = int(shared_gate_out.stride(0)) if t > 1 else i_sh
        _check(t <= 1 or int(shared_up_out.stride(0)) == ld_sh, "shared_gate_out / shared_up_out must share their row stride")
        if shared_gate_logit is not None:
            _check(shared_gate_logit.dtype == dtype and shared_gate_logit.shape[0] == t, "shared_gate_logit must be [T, 1]")
            ld_g = int(shared_gate_logit.stride(0)) if t > 1 else 1
    with torch.cuda.device(dev):
        _capi.check(_lib.bitsmoe_block_finish(
            rank_accum.data_ptr(), t, r, shared_gate_out.data_ptr() if i_sh else None,
            shared_up_out.data_ptr() if i_sh else None, ld_sh, i_sh,
            shared_gate_logit.data_ptr() if (i_sh and shared_gate_logit is not None) else None, ld_g,
            _capi.DT_F16 if dtype == torch.float16 else _capi.DT_BF16, out.data_ptr(), r + i_sh, _stream_ptr(dev)))
    return out


# ----------------------------------------------------------------------------------------
# PyTorch operator registration: torch.ops.bitsmoe.moe_packed_forward / torch.ops.bitsmoe.route
# ----------------------------------------------------------------------------------------
_MATRIX_ARGS = ", ".join(f"Tensor[] {m}_{b}" for m in ("gate", "up", "down")
                         for b in ("payload", "rank_idx", "tile_meta", "slab_meta", "scale", "s"))
_OPS = torch.library.Library("bitsmoe", "DEF")
_OPS.define("moe_packed_forward(Tensor h_gate, Tensor h_up, Tensor token_indices, Tensor expert_offsets, "
            f"Tensor route_weights, {_MATRIX_ARGS}, int rank_out, int intermediate_size, int act_type) -> Tensor")
_OPS.define("route(Tensor selected_experts, Tensor route_weights, Tensor global_to_local, int n_packed) "
            "-> (Tensor, Tensor, Tensor)")
_OPS.define("router_softmax_topk(Tensor router_logits, int top_k, bool renormalize=True, ScalarType? round_dtype=None, "
            "float weight_scale=1.0) -> (Tensor, Tensor)")
# only an accelerator implementation exists: on other devices the dispatcher raises
_OPS.impl("moe_packed_forward", moe_packed_forward, "CUDA")
_OPS.impl("route", route, "CUDA")
_OPS.impl("router_softmax_topk", router_softmax_topk, "CUDA")


@torch.library.register_fake("bitsmoe::moe_packed_forward")
def _moe_packed_forward_fake(h_gate, h_up, token_indices, expert_offsets, route_weights, *rest):
    return h_gate.new_empty((h_gate.shape[0], int(rest[-3])), dtype=torch.float32)


@torch.library.register_fake("bitsmoe::route")
def _route_fake(selected_experts, route_weights, global_to_local, n_packed):
    n_flat = selected_experts.numel()
    return (selected_experts.new_empty((n_flat,), dtype=torch.int32),
            selected_experts.new_empty((int(n_packed) + 1,), dtype=torch.int32),
            route_weights.new_empty((n_flat,), dtype=torch.float32))


@torch.library.register_fake("bitsmoe::router_softmax_topk")
def _router_fake(router_logits, top_k, renormalize=True, round_dtype=None, weight_scale=1.0):
    t = router_logits.shape[0]
    return (router_logits.new_empty((t, int(top_k)), dtype=torch.int64),
            router_logits.new_empty((t, int(top_k)), dtype=torch.float32))
