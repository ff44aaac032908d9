"""ctypes binding of libodsd_moe.so (the C ABI declared in include/odsd_moe.h).

There is no fallback: if the shared library is missing or a call returns a non-zero status,
an exception is raised.  Build it with ``python -c "import __graft_entry__ as g; g.build()"``
or ``make -C on_device_sd_amd/csrc``.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

LIB_NAME = "libodsd_moe.so"
LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), LIB_NAME)

DT_F32 = 0
DT_BF16 = 1
DT_F16 = 2
TABLE_COLS = 4


class MoeShape(C.Structure):
    """Mirror of ``odsd_moe_shape``."""
    _fields_ = [("T", C.c_int32), ("H", C.c_int32), ("E", C.c_int32), ("K", C.c_int32),
                ("I", C.c_int32), ("renorm", C.c_int32), ("act_dtype", C.c_int32),
                ("max_rows", C.c_int32)]


_P = C.c_void_p
_SP = C.POINTER(MoeShape)

# name -> (restype, argtypes); must list every function include/odsd_moe.h declares
SIGNATURES = {
    "odsd_version": (C.c_int, []),
    "odsd_status_string": (C.c_char_p, [C.c_int]),
    "odsd_w4_quantize": (C.c_int, [_P, C.c_int32, C.c_int64, C.c_int64, _P, _P, _P, _P]),
    "odsd_w4_packed_q_bytes": (C.c_size_t, [C.c_int64, C.c_int64]),
    "odsd_w4_packed_sz_bytes": (C.c_size_t, [C.c_int64, C.c_int64]),
    "odsd_w4_pack": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int64, C.c_int32, C.c_int32, _P, _P, _P]),
    "odsd_rmsnorm": (C.c_int, [_P, _P, C.c_int32, C.c_int32, C.c_int32, C.c_float, _P, _P]),
    "odsd_add_rmsnorm": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, C.c_int32, C.c_float, _P, _P, _P]),
    "odsd_router_workspace_bytes": (C.c_size_t, [_SP]),
    "odsd_router_topk": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "odsd_router_topk_logits": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "odsd_route_dispatch": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "odsd_route_dispatch_host_counts": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, C.c_uint32,
                                                  _P, C.c_size_t, _P]),
    "odsd_convert_act_f16": (C.c_int, [_P, C.c_int32, C.c_int64, _P, _P]),
    "odsd_dispatch": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P]),
    "odsd_experts_workspace_bytes": (C.c_size_t, [_SP]),
    "odsd_experts_w4": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "odsd_w4_gate_up_silu": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P]),
    "odsd_w4_down_splits": (C.c_int32, [_SP]),
    "odsd_experts_one_launch": (C.c_int32, [_SP]),
    "odsd_w4_down": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P]),
    "odsd_combine": (C.c_int, [_SP, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "odsd_moe_workspace_bytes": (C.c_size_t, [_SP]),
    "odsd_moe_forward": (C.c_int, [_SP, _P, _P, C.c_float, _P, _P, C.c_int32, _P, _P, _P, _P, _P, _P,
                                   _P, _P, _P, _P, C.c_size_t, _P]),
    "odsd_kv_store": (C.c_int, [_P, _P, C.c_int64, C.c_int64, _P, _P, _P, _P, C.c_int32, C.c_int32, C.c_int32,
                                C.c_int32, C.c_int64, _P]),
    "odsd_paged_attention": (C.c_int, [_P, _P, _P, _P, _P, _P, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                       C.c_int32, C.c_int32, C.c_int64, C.c_float, C.c_int32, _P, _P, C.c_size_t, _P]),
    "odsd_paged_attention_workspace_bytes": (C.c_size_t, [C.c_int32] * 7),
    "odsd_varlen_attention": (C.c_int, [_P, _P, _P, _P, _P] + [C.c_int32] * 6 + [C.c_float, C.c_int32, _P, _P,
                                                                                C.c_size_t, _P]),
    "odsd_varlen_attention_workspace_bytes": (C.c_size_t, [C.c_int32] * 6),
    "odsd_moe_forward_events": (C.c_int, [_SP, _P, _P, C.c_float, _P, _P, C.c_int32, _P, _P, _P, _P, _P,
                                          C.c_size_t, _P, _P, _P]),
    "odsd_moe_stack_workspace_bytes": (C.c_size_t, [_SP]),
    "odsd_moe_stack_forward": (C.c_int, [_SP, C.c_int32, _P, _P, _P, _P, C.c_float, _P, _P, C.c_size_t, _P]),
    "odsd_moe_stack_forward_events": (C.c_int, [_SP, C.c_int32, _P, _P, _P, _P, C.c_float, _P, _P, C.c_size_t, _P,
                                                _P, _P]),
    "odsd_moe_static_init": (C.c_int, []),
    "odsd_moe_forward_static": (C.c_int, [_SP, _P, _P, C.c_float, _P, _P, C.c_int32, _P, _P, _P, _P, _P,
                                          _P, _P, _P, _P, _P]),
}

N_KERNELS = 8                          # ODSD_N_KERNELS
KERNEL_NAMES = ("norm", "router_logits", "router_topk", "dispatch", "gate_up", "down", "combine", "experts")
STATIC_SCRATCH_BYTES = 64 << 20        # ODSD_STATIC_SCRATCH_BYTES

_lib: Optional[C.CDLL] = None


class OdsdError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


def load() -> C.CDLL:
    """Load the shared library (once) and declare every signature."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP extension has not been built. There is no "
            "CPU or PyTorch fallback for the MoE path; run __graft_entry__.build().")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().odsd_status_string(status).decode()
        raise OdsdError(f"{what}: odsd status {status} ({msg})")
