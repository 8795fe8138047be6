"""ctypes binding of libbitsmoe_hip.so (the C ABI declared in include/bitsmoe_hip.h).

The library is loaded from the package tree (bitsmoe_amd/csrc/libbitsmoe_hip.so); there is
no fallback: if it is missing, `load()` raises and the operator is reported as absent.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

import os

# BITSMOE_LIB_VARIANT=timeline loads the build with in-kernel time stamps (python -m bitsmoe_amd.build --timeline)
_VARIANT = os.environ.get("BITSMOE_LIB_VARIANT", "")
LIB_PATH = Path(__file__).resolve().parent.parent / "csrc" / (
    f"libbitsmoe_hip_{_VARIANT}.so" if _VARIANT else "libbitsmoe_hip.so")

DT_F16 = 0
DT_BF16 = 1
PATH_AUTO = 0
PATH_GENERIC = 1
PATH_DECODE = 2
PATH_MFMA = 3
PROFILE_PHASES = 5

# every extern "C" symbol include/bitsmoe_hip.h declares
EXPORTED_SYMBOLS = (
    "bitsmoe_last_error",
    "bitsmoe_version",
    "bitsmoe_set_option",
    "bitsmoe_matset_create",
    "bitsmoe_matset_destroy",
    "bitsmoe_matset_info",
    "bitsmoe_dequant_matrix",
    "bitsmoe_matset_prepare",
    "bitsmoe_dequant_matrix_prepared",
    "bitsmoe_route_workspace_bytes",
    "bitsmoe_route",
    "bitsmoe_router_softmax_topk",
    "bitsmoe_router_softmax_topk_strided",
    "bitsmoe_router_linear_topk",
    "bitsmoe_block_finish",
    "bitsmoe_skinny_linear",
    "bitsmoe_prepared_linear_weight_elements",
    "bitsmoe_prepare_linear_weight",
    "bitsmoe_forward_workspace_bytes",
    "bitsmoe_forward_workspace_bytes_sets",
    "bitsmoe_moe_forward",
    "bitsmoe_moe_forward_strided",
    "bitsmoe_static_scratch_bytes",
    "bitsmoe_moe_forward_static",
    "bitsmoe_forward_routed_workspace_bytes",
    "bitsmoe_moe_forward_routed",
    "bitsmoe_forward_routed_is_inline",
    "bitsmoe_forward_decode_is_fused",
    "bitsmoe_profile_create",
    "bitsmoe_profile_destroy",
    "bitsmoe_profile_read",
    "bitsmoe_pack_bitplanes",
    "bitsmoe_unpack_bitplanes",
    "bitsmoe_quantize_tiles",
    "bitsmoe_pack_slabs",
)


class MatrixDesc(Structure):
    _fields_ = [
        ("payload", c_void_p),
        ("rank_idx", c_void_p),
        ("tile_meta", c_void_p),
        ("slab_meta", c_void_p),
        ("scale", c_void_p),
        ("s", c_void_p),
        ("payload_words", c_int64),
        ("scale_len", c_int64),
        ("rank_len", c_int32),
        ("num_tiles", c_int32),
        ("num_slabs", c_int32),
        ("reserved", c_int32),
    ]


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m bitsmoe_amd.build` "
            "(the packed routed-expert forward has no fallback path)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    lib.bitsmoe_last_error.restype = c_char_p
    lib.bitsmoe_last_error.argtypes = []
    lib.bitsmoe_version.restype = c_char_p
    lib.bitsmoe_version.argtypes = []
    lib.bitsmoe_set_option.restype = c_int32
    lib.bitsmoe_set_option.argtypes = [c_char_p, c_int32]
    lib.bitsmoe_matset_create.restype = c_int32
    lib.bitsmoe_matset_create.argtypes = [POINTER(MatrixDesc), c_int32, c_int32, c_void_p, POINTER(c_void_p)]
    lib.bitsmoe_matset_destroy.restype = None
    lib.bitsmoe_matset_destroy.argtypes = [c_void_p]
    lib.bitsmoe_matset_info.restype = c_int32
    lib.bitsmoe_matset_info.argtypes = [c_void_p, POINTER(c_int64)]
    lib.bitsmoe_dequant_matrix.restype = c_int32
    lib.bitsmoe_dequant_matrix.argtypes = [c_void_p, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_matset_prepare.restype = c_int32
    lib.bitsmoe_matset_prepare.argtypes = [c_void_p, c_int32, c_void_p]
    lib.bitsmoe_dequant_matrix_prepared.restype = c_int32
    lib.bitsmoe_dequant_matrix_prepared.argtypes = [c_void_p, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_route_workspace_bytes.restype = c_size_t
    lib.bitsmoe_route_workspace_bytes.argtypes = [c_int64, c_int32]
    lib.bitsmoe_route.restype = c_int32
    lib.bitsmoe_route.argtypes = [
        c_void_p, c_int32, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32,
        c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p,
    ]
    lib.bitsmoe_router_softmax_topk.restype = c_int32
    lib.bitsmoe_router_softmax_topk.argtypes = [c_void_p, c_int32, c_int64, c_int32, c_int32, c_int32, c_int32,
                                                c_void_p, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_router_softmax_topk_strided.restype = c_int32
    lib.bitsmoe_router_softmax_topk_strided.argtypes = [c_void_p, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_float,
                                                        c_int32, c_void_p, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_router_linear_topk.restype = c_int32
    lib.bitsmoe_router_linear_topk.argtypes = [c_void_p, c_int32, c_int64, c_void_p, c_int32, c_int64, c_int32, c_int32, c_int32,
                                               c_int32, c_float, c_int32, c_void_p, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_skinny_linear.restype = c_int32
    lib.bitsmoe_skinny_linear.argtypes = [c_void_p, c_int32, c_int32, c_int64, c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p,
                                          c_int64, c_void_p, c_int64, c_void_p]
    lib.bitsmoe_prepared_linear_weight_elements.restype = c_int64
    lib.bitsmoe_prepared_linear_weight_elements.argtypes = [c_int32, c_int32]
    lib.bitsmoe_prepare_linear_weight.restype = c_int32
    lib.bitsmoe_prepare_linear_weight.argtypes = [c_void_p, c_int32, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_block_finish.restype = c_int32
    lib.bitsmoe_block_finish.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_int64,
                                         c_int32, c_void_p, c_int64, c_void_p]
    lib.bitsmoe_forward_workspace_bytes.restype = c_size_t
    lib.bitsmoe_forward_workspace_bytes.argtypes = [c_int64, c_int64, c_int32, c_int32, c_int32]
    lib.bitsmoe_forward_workspace_bytes_sets.restype = c_size_t
    lib.bitsmoe_forward_workspace_bytes_sets.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32]
    lib.bitsmoe_moe_forward.restype = c_int32
    lib.bitsmoe_moe_forward.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32,
        c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32, c_int32,
        c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
    ]
    lib.bitsmoe_moe_forward_strided.restype = c_int32
    lib.bitsmoe_moe_forward_strided.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_int64, c_int64,
        c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32, c_int32,
        c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
    ]
    lib.bitsmoe_static_scratch_bytes.restype = c_size_t
    lib.bitsmoe_static_scratch_bytes.argtypes = []
    lib.bitsmoe_moe_forward_static.restype = c_int32
    lib.bitsmoe_moe_forward_static.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_int64, c_int64,
        c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p,
    ]
    lib.bitsmoe_forward_routed_workspace_bytes.restype = c_size_t
    lib.bitsmoe_forward_routed_workspace_bytes.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32]
    lib.bitsmoe_forward_routed_is_inline.restype = c_int32
    lib.bitsmoe_forward_routed_is_inline.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                                     c_int64, c_int64, c_int64, c_int32, c_int32]
    lib.bitsmoe_forward_decode_is_fused.restype = c_int32
    lib.bitsmoe_forward_decode_is_fused.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                                    c_int64, c_int64, c_int64, c_int32]
    lib.bitsmoe_moe_forward_routed.restype = c_int32
    lib.bitsmoe_moe_forward_routed.argtypes = [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int32, c_int64, c_int64,
        c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, c_int32,
        c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
    ]
    lib.bitsmoe_profile_create.restype = c_int32
    lib.bitsmoe_profile_create.argtypes = [POINTER(c_void_p)]
    lib.bitsmoe_profile_destroy.restype = None
    lib.bitsmoe_profile_destroy.argtypes = [c_void_p]
    lib.bitsmoe_profile_read.restype = c_int32
    lib.bitsmoe_profile_read.argtypes = [c_void_p, POINTER(c_float)]
    lib.bitsmoe_pack_bitplanes.restype = c_int32
    lib.bitsmoe_pack_bitplanes.argtypes = [c_void_p, c_int64, c_int64, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_unpack_bitplanes.restype = c_int32
    lib.bitsmoe_unpack_bitplanes.argtypes = [c_void_p, c_int64, c_int64, c_int32, c_void_p, c_void_p]
    lib.bitsmoe_quantize_tiles.restype = c_int32
    lib.bitsmoe_quantize_tiles.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p]
    lib.bitsmoe_pack_slabs.restype = c_int32
    lib.bitsmoe_pack_slabs.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_int32, c_void_p, c_void_p, c_void_p]
    _lib = lib
    return lib


def check(rc: int) -> None:
    """Turn a negative status into the RuntimeError the reference's TORCH_CHECKs raise."""
    if rc != 0:
        msg = load().bitsmoe_last_error()
        raise RuntimeError(msg.decode("utf-8", "replace") if msg else f"bitsmoe_hip error {rc}")
