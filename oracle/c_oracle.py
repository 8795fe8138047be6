"""ctypes wrapper of liboracle.so (oracle.c).  TEST INFRASTRUCTURE ONLY — see oracle/__init__.py."""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, Sequence

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "liboracle.so")
_lib = None


class _Matrix(ctypes.Structure):
    _fields_ = [
        ("payload", ctypes.c_void_p), ("rank_idx", ctypes.c_void_p), ("tile_meta", ctypes.c_void_p),
        ("slab_meta", ctypes.c_void_p), ("scale", ctypes.c_void_p), ("s", ctypes.c_void_p),
        ("num_slabs", ctypes.c_int32), ("num_tiles", ctypes.c_int32), ("rank_len", ctypes.c_int32),
        ("pad", ctypes.c_int32),
    ]


def load(build_if_missing: bool = True):
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        if not build_if_missing:
            raise RuntimeError("oracle/liboracle.so is missing: run `make -C oracle`")
        subprocess.run(["make", "-C", _DIR], check=True, capture_output=True)
    lib = ctypes.CDLL(_LIB_PATH)
    lib.oracle_dequant_matrix.restype = None
    lib.oracle_dequant_matrix.argtypes = [ctypes.POINTER(_Matrix), ctypes.c_int32, ctypes.c_void_p]
    lib.oracle_moe_forward.restype = ctypes.c_int
    lib.oracle_moe_forward.argtypes = [
        ctypes.POINTER(_Matrix), ctypes.POINTER(_Matrix), ctypes.POINTER(_Matrix), ctypes.c_int32,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32,
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
        ctypes.c_void_p, ctypes.c_int32,
    ]
    lib.oracle_route.restype = None
    lib.oracle_route.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64,
                                 ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_num_threads.restype = ctypes.c_int
    _lib = lib
    return lib


class MatrixArray:
    """A C array of oracle_matrix built from the numpy dicts of ref_oracle.pack_matrix."""

    def __init__(self, mats: Sequence[Dict[str, np.ndarray]]):
        self.keep = []
        self.arr = (_Matrix * max(len(mats), 1))()
        for i, m in enumerate(mats):
            bufs = {
                "payload": np.ascontiguousarray(m["payload"], dtype=np.uint32),
                "rank_idx": np.ascontiguousarray(m["rank_idx"], dtype=np.int32),
                "tile_meta": np.ascontiguousarray(m["tile_meta"], dtype=np.int32),
                "slab_meta": np.ascontiguousarray(m["slab_meta"], dtype=np.int32),
                "scale": np.ascontiguousarray(m["scale"], dtype=np.float16),
                "s": np.ascontiguousarray(m["s"], dtype=np.float16),
            }
            self.keep.append(bufs)
            c = self.arr[i]
            for k, v in bufs.items():
                setattr(c, k, v.ctypes.data)
            c.num_slabs = int(bufs["slab_meta"].reshape(-1, 4).shape[0])
            c.num_tiles = int(bufs["tile_meta"].reshape(-1, 3).shape[0])
            c.rank_len = int(bufs["rank_idx"].size)
        self.n = len(mats)


def dequant_matrix(m: Dict[str, np.ndarray], dim: int) -> np.ndarray:
    lib = load()
    arr = MatrixArray([m])
    out = np.empty((int(m["rank_idx"].size), dim), dtype=np.float32)
    lib.oracle_dequant_matrix(arr.arr, dim, out.ctypes.data)
    return out


def moe_forward(h_gate: np.ndarray, h_up: np.ndarray, tok: np.ndarray, off: np.ndarray, rw: np.ndarray,
                gate: MatrixArray, up: MatrixArray, down: MatrixArray, rank_out: int, dim: int,
                n_threads: int = 0) -> np.ndarray:
    lib = load()
    hg = np.ascontiguousarray(h_gate, dtype=np.float32)
    hu = np.ascontiguousarray(h_up, dtype=np.float32)
    tok = np.ascontiguousarray(tok, dtype=np.int32)
    off = np.ascontiguousarray(off, dtype=np.int32)
    rw = np.ascontiguousarray(rw, dtype=np.float32)
    out = np.empty((hg.shape[0], rank_out), dtype=np.float32)
    rc = lib.oracle_moe_forward(gate.arr, up.arr, down.arr, gate.n, hg.ctypes.data, hu.ctypes.data, hg.shape[0],
                                hg.shape[1], hu.shape[1], tok.ctypes.data, off.ctypes.data, rw.ctypes.data,
                                rank_out, dim, out.ctypes.data, n_threads)
    if rc != 0:
        raise MemoryError("oracle_moe_forward could not allocate its scratch buffers")
    return out


def route(selected: np.ndarray, weights: np.ndarray, g2l: np.ndarray, n_packed: int):
    lib = load()
    sel = np.ascontiguousarray(selected, dtype=np.int64)
    t, k = sel.shape
    w = np.ascontiguousarray(weights, dtype=np.float32)
    g2l = np.ascontiguousarray(g2l, dtype=np.int32)
    tok = np.zeros(t * k, dtype=np.int32)
    rf = np.zeros(t * k, dtype=np.float32)
    off = np.zeros(n_packed + 1, dtype=np.int32)
    lib.oracle_route(sel.ctypes.data, w.ctypes.data, g2l.ctypes.data, g2l.size, t, k, n_packed, tok.ctypes.data,
                     off.ctypes.data, rf.ctypes.data)
    a = int(off[-1])
    return tok[:a], off, rf[:a]


def num_threads() -> int:
    return int(load().oracle_num_threads())


def matrices_from_torch(payload, rank_idx, tile_meta, slab_meta, scale, s, dim: int):
    """Per-expert device tensor lists (the operator's argument lists) -> list of numpy dicts."""
    import torch

    mats = []
    cache = {}

    def host(t, view=None):
        key = (t.data_ptr(), t.numel())
        if key not in cache:
            c = t.detach().cpu()
            cache[key] = (c.view(view) if view is not None else c).numpy()
        return cache[key]

    for i in range(len(payload)):
        mats.append({
            "payload": host(payload[i], torch.int32).view(np.uint32),
            "rank_idx": host(rank_idx[i]),
            "tile_meta": host(tile_meta[i]).reshape(-1, 3),
            "slab_meta": host(slab_meta[i]).reshape(-1, 4),
            "scale": host(scale[i]),
            "s": host(s[i]),
            "dim": int(dim),
        })
    return mats
