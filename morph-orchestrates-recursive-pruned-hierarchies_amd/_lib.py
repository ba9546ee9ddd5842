"""ctypes binding of libmortar_hip.so (the C-ABI declared in include/mortar_hip.h).

There is no fallback: if the library is missing or a call fails, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmortar_hip.so")

c_i32, c_i64, c_vp, c_f32 = C.c_int32, C.c_int64, C.c_void_p, C.c_float


class BcsrStruct(C.Structure):
    """mortar_bcsr_t"""
    _fields_ = [("codes", c_vp), ("sdup", c_vp), ("col", c_vp), ("row_ptr", c_vp), ("row_desc", c_vp),
                ("codes_o", c_vp), ("sd_o", c_vp), ("col_o", c_vp), ("codes4_o", c_vp),
                ("Rb", c_i32), ("Cb", c_i32), ("nnz", c_i32),
                ("seg_cb", c_i32), ("uniform_scale", c_f32), ("reserved_", c_i32)]


_SIGS = {
    "mortar_last_error": (C.c_char_p, []),
    "mortar_abi_version": (C.c_int, []),
    "mortar_encode_blocks_host": (C.c_int, [c_vp, c_i64, c_vp, c_i64, c_vp, c_vp]),
    "mortar_uniform_scale_host": (C.c_int, [c_vp, c_i64, c_vp]),
    "mortar_decode_blocks_host": (C.c_int, [c_vp, c_i64, c_vp]),
    "mortar_octet_layout_host": (c_i64, [c_vp, c_i32, c_i32, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "mortar_fp4_stream_host": (C.c_int, [c_vp, c_i64, c_vp]),
    "mortar_octet_positions_host": (C.c_int, [c_vp, c_i32, c_i32, c_i32, c_vp, c_vp]),
    "mortar_transpose_topology_host": (C.c_int, [c_vp, c_vp, c_i32, c_i32, c_vp, c_vp, c_vp]),
    "mortar_requantize_workspace_bytes": (c_i64, []),
    "mortar_requantize": (C.c_int, [c_vp, c_vp, c_i32, c_vp, c_vp, c_i32, c_i32, c_f32, c_vp, c_vp, c_vp, c_i32, c_f32,
                                  c_vp, c_vp]),
    "mortar_poison_on_status": (C.c_int, [c_vp, c_i64, c_vp, c_vp]),
    "mortar_swiglu_bf16": (C.c_int, [c_vp, c_i64, c_i64, c_i32, c_vp, c_i64, c_vp]),
    "mortar_swiglu_backward_bf16": (C.c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_i32, c_vp, c_i64, c_vp]),
    "mortar_sdd_blocks_per_wave_host": (c_i32, [c_vp, c_vp, c_i32, c_i32, c_i64]),
    "mortar_sdd_plan_host": (c_i64, [c_vp, c_vp, c_i32, c_i32, c_i32, c_vp, c_i64]),
    "mortar_sdd_workspace_bytes": (c_i64, [c_i32, c_i32, c_i32, c_i64]),
    "mortar_sdd_bf16": (C.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp, c_i64, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp]),
    "mortar_prefill_max_seg_cb": (C.c_int, []),
    "mortar_decode_max_seg_cb": (C.c_int, [c_i32]),
    "mortar_validate_bcsr_host": (C.c_int, [c_vp, c_vp, c_i32, c_i32]),
    "mortar_schedule_host": (C.c_int, [c_vp, c_i32, c_i32, c_i32, c_vp, c_vp]),
    "mortar_unit_order_host": (C.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "mortar_unit_order_segments_host": (C.c_int, [c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp]),
    "mortar_decode_worklist_host": (c_i64, [c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp, c_vp, c_vp]),
    "mortar_spmm_bf16": (C.c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_i64, c_vp]),
    "mortar_gateup_swiglu_bf16": (C.c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_i64, c_vp, c_i32,
                                            c_vp, c_vp, c_vp]),
    "mortar_norm_gateup_swiglu_bf16": (C.c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_f32, c_vp, c_i64, c_vp, c_i32,
                                                 c_vp, c_vp, c_vp]),
    "mortar_norm_fusable": (C.c_int, [c_i32]),
    "mortar_values_seg_cb": (c_i32, [c_i32]),
    "mortar_segment_ptr_host": (C.c_int, [c_vp, c_vp, c_i32, c_i32, c_i32, c_vp]),
    "mortar_dds_values_bf16": (C.c_int, [c_vp, c_vp, c_vp, c_vp, c_i32, c_i32, c_i64, c_vp, c_i64, c_i64, c_vp, c_i64, c_vp]),
    "mortar_mlp_hidden_bytes": (c_i64, [c_i64, c_i32]),
    "mortar_mlp_bf16": (C.c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i32, c_vp, c_f32, c_vp, c_i32, c_vp, c_vp, c_i64,
                                  c_i32, c_vp]),
    "mortar_spmm_bf16_masked": (C.c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_i64, c_vp, c_i32, c_vp]),
    "mortar_route_tile": (C.c_int, [c_i32, c_i64]),
    "mortar_remoe_gates": (C.c_int, [c_vp, c_i64, c_i32, c_i32, c_vp, c_vp, c_vp]),
    "mortar_remoe_route": (C.c_int, [c_vp, c_i64, c_i32, c_i32, c_vp, c_vp, c_vp]),
    "mortar_router_bf16": (C.c_int, [c_vp, c_i32, c_i64, c_i32, c_i64, c_vp, c_vp, c_vp, c_vp, c_f32, c_vp, c_vp, c_i32,
                                     c_vp, c_i32, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "mortar_router_tail_f32": (C.c_int, [c_vp, c_i64, c_i32, c_i64, c_vp, c_vp, c_vp, c_f32, c_vp, c_vp, c_i32, c_vp, c_i32,
                                         c_i32, c_vp, c_vp, c_vp, c_vp]),
    "mortar_route_flags": (C.c_int, [c_vp, c_i64, c_i32, c_i64, c_i32, c_vp, c_i64, c_vp, c_i64, c_vp]),
    "mortar_stack_table_bytes": (c_i64, [c_i32]),
    "mortar_stack_prepare": (C.c_int, [c_i32, c_i32, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_vp, c_vp]),
    "mortar_stack_run": (C.c_int, [c_i32, c_i32, c_vp, c_i64, c_vp, c_vp]),
    "mortar_gemv_bf16": (C.c_int, [c_vp, c_vp, c_i64, c_i32, c_vp, c_i32, c_i32, c_vp, c_i32, c_i64, c_vp, c_i64,
                                   c_vp, c_vp, c_i32, c_i64, c_vp, c_i64, c_vp, c_i64, c_vp]),
    "mortar_rmsnorm_bf16": (C.c_int, [c_vp, c_i64, c_i32, c_i64, c_vp, c_f32, c_vp, c_i64, c_vp]),
    "mortar_spmm_hc_post": (C.c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_i32, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp, c_i32, c_vp]),
    "mortar_gemv_f32_workspace_bytes": (c_i64, [c_vp, c_i32, c_i32]),
    "mortar_gemv_f32": (C.c_int, [c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_i32, c_vp, c_i32, c_i32, c_i32, c_vp, c_i32, c_i64, c_vp, c_i64,
                                  c_vp, c_i64, c_vp, c_i32, c_i64, c_vp, c_i64, c_vp, c_i64, c_vp]),
    "mortar_gemv_noalloc_max_floats": (c_i64, []),
    "mortar_gemv_bf16_noalloc": (C.c_int, [c_vp, c_vp, c_i64, c_i32, c_vp, c_i32, c_i32, c_vp, c_i32, c_i64, c_vp, c_i64,
                                           c_vp, c_i32, c_i64, c_vp, c_i64, c_vp, c_i64, c_vp]),
}

EXPORTS = tuple(_SIGS)
_lib = None


def lib():
    """The loaded library.  Raises if it has not been built (run `python build.py` in the package)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the MORTAR HIP extension has not been built "
                "(run __graft_entry__.build() or `python build.py` in the package directory)")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(l, name)
            fn.restype, fn.argtypes = res, args
        _lib = l
    return _lib


def check(rc: int, what: str) -> int:
    if rc < 0:
        msg = lib().mortar_last_error().decode("utf-8", "replace")
        err = ValueError if rc in (-1, -2, -4) else RuntimeError
        raise err(f"{what} failed ({rc}): {msg}")
    return rc
