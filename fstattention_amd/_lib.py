"""ctypes binding of ``libfsta.so`` (declarations mirror ``include/fsta.h``)."""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint32, c_void_p

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libfsta.so")

F32, F16, BF16, F64 = 0, 1, 2, 3
OK, EINVAL, EUNSUPPORTED, EHIP = 0, -1, -2, -3
FLAG_FAST_PV, FLAG_GENERIC, FLAG_WIDE_WAVES, FLAG_SHARE_TILES, FLAG_STREAM = 1, 2, 4, 8, 16


DFS_ORDER_MAX_NODES = 131072
DFS_ORDER_STATIC_MAX_NODES = 16384


def dfs_order_workspace_ints(n: int) -> int:
    """FSTA_DFS_ORDER_WORKSPACE_INTS(n): int32 entries of scratch fsta_dfs_order wants for n nodes."""
    return 6 * int(n) + 8


def flag_key_splits(n: int) -> int:
    """FSTA_FLAG_KEY_SPLITS(n): force n runs of prefix keys (1 = never split, 0 = library decides)."""
    return (int(n) & 0xFF) << 8


PRE_TOO_MANY_ANCESTORS, PRE_BAD_NODE_ID, PRE_BAD_LEVEL = 1, 2, 4
TREE_NOT_PREFIX_CLOSED = 8
ABI_VERSION = 2

# name -> (restype, argtypes); every symbol include/fsta.h declares
SIGNATURES = {
    "fsta_abi_version": (c_int, []),
    "fsta_last_error": (c_char_p, []),
    "fsta_last_attention_kernel": (c_char_p, []),
    "fsta_mask_words": (c_int32, [c_int32]),
    "fsta_block_plan_bytes": (c_size_t, [c_int32, c_int32, c_int32]),
    "fsta_precompute": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32,
                                c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "fsta_precompute_from_parents": (c_int, [c_void_p, c_int64, c_int64, c_int32, c_int32, c_int32, c_void_p, c_void_p,
                                             c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "fsta_pack_mask": (c_int, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int64, c_void_p, c_void_p,
                               c_void_p, c_void_p]),
    "fsta_attention_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
                                   c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                                   c_int32, c_int32, c_int32, c_float, c_uint32, c_void_p]),
    "fsta_attention_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                                                  c_int32, c_float, c_uint32]),
    "fsta_attention_fwd_ws": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
                                      c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                                      c_int32, c_int32, c_int32, c_float, c_uint32, c_void_p, c_size_t, c_void_p]),
    "fsta_attention_fwd_kv8": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                                       c_int32, c_int32, c_float, c_void_p]),
    "fsta_lineage_from_parents": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                          c_void_p]),
    "fsta_dfs_order": (c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p]),
    "fsta_dfs_order_static": (c_int, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "fsta_renumber_parents": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "fsta_medusa_tree": (c_int, [c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p]),
    "fsta_medusa_workspace_bytes": (c_size_t, [c_int32, c_int32]),
    "fsta_medusa_tree_ws": (c_int, [c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_size_t,
                                    c_void_p]),
    "fsta_probe_empty_launch": (c_int, [c_int32, c_int32, c_void_p]),
    "fsta_probe_hbm_read": (c_int, [c_void_p, c_size_t, c_int32, c_int32, c_void_p, c_void_p]),
    "fsta_merge_states": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                  c_int32, c_int32, c_void_p]),
}

_lib = None


class FstaError(RuntimeError):
    """A libfsta entry point returned an error code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libfsta error {code}: {message}")
        self.code = code


def load():
    """Loads the library once; raises if it has not been built.

    There is no CPU fallback: without the HIP library the package cannot compute.
    """
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m fstattention_amd.build` "
            "(needs hipcc; the package has no CPU fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.fsta_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.fsta_abi_version()}, expected {ABI_VERSION}")
    _lib = lib
    return lib


TORCH_OPS_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_fsta_torch.so")
_ops = None


def load_torch_ops():
    """``torch.ops.fsta`` (the operator registration of ``csrc/fsta_torch_binding.cpp``), loaded once."""
    global _ops
    if _ops is not None:
        return _ops
    load()
    if not os.path.exists(TORCH_OPS_PATH):
        raise ImportError(f"{TORCH_OPS_PATH} is missing: build it with `python -m fstattention_amd.build`")
    import torch
    torch.ops.load_library(TORCH_OPS_PATH)
    _ops = torch.ops.fsta
    return _ops


def check(code: int):
    if code != OK:
        raise FstaError(code, load().fsta_last_error().decode("utf-8", "replace"))
