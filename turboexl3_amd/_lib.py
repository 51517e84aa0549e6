"""Loads libturboexl3_hip.so (built in-tree by turboexl3_amd.build) and declares the C ABI of
include/turboexl3_hip.h to ctypes. There is no fallback: a missing library is an error."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libturboexl3_hip.so")

T3_MAX_DIMS = 8
STATIC_SCRATCH_BYTES = 16 << 20

# t3_dtype
F32, F16, BF16, U16, I16, U32, I32 = range(7)

STATUS_NAMES = [
    "ok", "BadExl3Shape", "BadExl3Dtype", "Exl3EngineNotImplemented", "Exl3EngineCacheFull",
    "Exl3GateUpRateMismatch", "InvalidExl3Clamp", "Exl3TopKExceedsReduceBank", "Exl3WindowUnsupported",
    "ExpertLayoutUnsupported", "InvalidTurboexl3Config", "WorkspaceTooSmall", "HipFailed", "BadArgs",
]


class Array(C.Structure):
    _fields_ = [("data", C.c_void_p), ("ndim", C.c_int32), ("dtype", C.c_int32), ("shape", C.c_int64 * T3_MAX_DIMS)]


class Decode(C.Structure):
    _fields_ = [("codebook", C.c_int32), ("window_bits", C.c_int32)]


class Proj(C.Structure):
    _fields_ = [("trellis", Array), ("suh", Array), ("svh", Array)]


class Bank(C.Structure):
    _fields_ = [("gate", Proj), ("up", Proj), ("down", Proj)]


class Config(C.Structure):
    _fields_ = [("decode_form", C.c_int32), ("dec_one", C.c_int32), ("prefill", C.c_int32),
                ("mcg_pair", C.c_int32), ("mul1_defer", C.c_int32), ("dense_gemm_rows", C.c_int32),
                ("dense_rows_alone", C.c_int32)]


class Block(C.Structure):
    _fields_ = [("kind", C.c_int32), ("codebook", C.c_int32), ("window_bits", C.c_int32), ("n", C.c_int32)]


class Weight(C.Structure):
    _fields_ = [("w", Array), ("scales", Array), ("biases", Array), ("layout", C.c_int32), ("flags", C.c_int32),
                ("block", C.c_int32)]


CLAIM_NO, CLAIM_BY_TYPE, CLAIM_BY_MARKER = 0, 1, 2
VERDICT_OK, VERDICT_UNSUPPORTED, VERDICT_FAILED, VERDICT_TOO_LARGE = 0, 1, 2, 3
BLOCK_TRUNK, BLOCK_BANK = 0, 1

# every symbol include/turboexl3_hip.h declares: name -> (restype, argtypes)
_AP, _BP = C.POINTER(Array), C.POINTER(Bank)
_KP, _WP, _SZP = C.POINTER(Block), C.POINTER(Weight), C.POINTER(C.c_size_t)
class LinearPlan(C.Structure):
    _fields_ = [("path", C.c_int32), ("launches", C.c_int32), ("rows", C.c_uint32), ("in_f", C.c_uint32),
                ("out_f", C.c_uint32), ("n", C.c_uint32), ("tiles_a_load", C.c_uint32), ("k_slices", C.c_uint32),
                ("tiles_a_wave", C.c_uint32), ("workgroups", C.c_uint32), ("code_bytes", C.c_uint64),
                ("workspace_bytes", C.c_size_t)]


class MoePlan(C.Structure):
    _fields_ = [("path", C.c_int32), ("launches", C.c_int32), ("rows", C.c_uint32), ("row_slots", C.c_uint32),
                ("hidden", C.c_uint32), ("inter", C.c_uint32), ("topk", C.c_uint32), ("shared_slots", C.c_uint32),
                ("tiles_a_wave_gu", C.c_uint32), ("k_slices_gu", C.c_uint32), ("tiles_a_load_gu", C.c_uint32),
                ("tiles_a_wave_dn", C.c_uint32), ("k_slices_dn", C.c_uint32), ("tiles_a_load_dn", C.c_uint32),
                ("k_slices_a_workgroup_dn", C.c_uint32),
                ("item_rows", C.c_uint32), ("max_items", C.c_uint32), ("expert_code_bytes", C.c_uint64),
                ("workspace_bytes", C.c_size_t), ("route_order_at", C.c_size_t), ("route_inv_at", C.c_size_t),
                ("route_items_at", C.c_size_t), ("route_counts_at", C.c_size_t)]


_u16p = C.POINTER(C.c_uint16)
SYMBOLS = {
    "t3_error_name": (C.c_char_p, [C.c_int32]),
    "t3_config_default": (None, [C.POINTER(Config)]),
    "t3_configure": (C.c_int32, [C.POINTER(Config)]),
    "t3_release_engines": (None, []),
    "t3_linear": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, _AP, Decode, _AP, C.c_void_p, C.c_size_t]),
    "t3_linear_static": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, _AP, Decode, _AP]),
    "t3_linear_static_reset": (C.c_int32, [C.c_void_p]),
    "t3_linear_workspace_bytes": (C.c_int32, [_AP, _AP, Decode, C.POINTER(C.c_size_t)]),
    "t3_linear_plan_of": (C.c_int32, [_AP, _AP, Decode, C.POINTER(LinearPlan)]),
    "t3_moe_plan_of": (C.c_int32, [_AP, _BP, _AP, _BP, C.POINTER(MoePlan)]),
    "t3_linear_chain": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, _AP, Decode, _AP, C.c_void_p, C.c_size_t]),
    "t3_linear_stages": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, _AP, Decode, _AP, C.c_void_p, C.c_size_t, C.c_uint32]),
    "t3_linear_bias": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, _AP, _AP, Decode, _AP, C.c_void_p, C.c_size_t]),
    "t3_dequant": (C.c_int32, [C.c_void_p, _AP, Decode, _AP]),
    "t3_linear_resident_workspace_bytes": (C.c_int32, [_AP, _AP, C.POINTER(C.c_size_t)]),
    "t3_linear_resident": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, _AP, _AP, C.c_void_p, C.c_size_t]),
    "t3_unrot_workspace_bytes": (C.c_int32, [_AP, C.POINTER(C.c_size_t)]),
    "t3_unrot_weight": (C.c_int32, [C.c_void_p, _AP, _AP, _AP, Decode, _AP, C.c_int64, C.c_void_p, C.c_void_p,
                                    C.c_size_t]),
    "t3_linear_unrot": (C.c_int32, [C.c_void_p, _AP, _AP, C.c_int64, C.c_int64, _AP]),
    "t3_linear_unrot_workspace_bytes": (C.c_int32, [_AP, _AP, C.c_int64, C.c_int64, C.POINTER(C.c_size_t)]),
    "t3_linear_unrot_parts": (C.c_int32, [C.c_void_p, _AP, _AP, C.c_int64, C.c_int64, _AP, C.c_void_p, C.c_size_t]),
    "t3_moe": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, C.c_int32, _AP, C.c_void_p, C.c_size_t]),
    "t3_moe_clamped": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, C.c_int32, _AP, C.c_void_p, C.c_size_t]),
    "t3_moe_swiglu": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, C.c_int32, C.c_int32, _AP, C.c_void_p,
                                   C.c_size_t]),
    "t3_moe_with_shared": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, C.c_int32, _AP, _AP, C.c_void_p,
                                        C.c_size_t]),
    "t3_moe_shared_expert": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, C.c_int32, _BP, _AP, C.c_void_p,
                                          C.c_size_t]),
    "t3_moe_stages": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, C.c_int32, _BP, _AP, C.c_void_p, C.c_size_t,
                                  C.c_uint32]),
    "t3_moe_fused_shared": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, _AP, Decode, _BP, _AP, _AP, _AP, C.c_void_p,
                                        C.c_size_t]),
    "t3_moe_fused_shared_routed_workspace_bytes": (C.c_int32, [_AP, _BP, _AP, C.c_int64, _BP, C.POINTER(C.c_size_t)]),
    "t3_moe_fused_shared_routed": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, C.c_int64, Decode, _BP, _AP, _AP, _AP, _AP,
                                               C.c_void_p, C.c_size_t]),
    "t3_moe_glm": (C.c_int32, [C.c_void_p, _AP, _BP, _AP, Decode, C.c_int32, _AP, C.c_void_p, C.c_size_t]),
    "t3_moe_workspace_bytes": (C.c_int32, [_AP, _BP, _AP, _BP, C.POINTER(C.c_size_t)]),
    "t3_rate_admitted": (C.c_int32, [C.c_int64]),
    "t3_admit_topk": (C.c_int32, [C.c_int64]),
    "t3_trellis_admitted": (C.c_int32, [C.POINTER(C.c_int64), C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int64]),
    "t3_table_parse_block": (C.c_int32, [C.c_char_p, _KP]),
    "t3_table_claims": (C.c_int32, [C.c_char_p, C.c_char_p, C.c_int32]),
    "t3_table_validate": (C.c_int32, [C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t]),
    "t3_table_bill": (C.c_uint64, [C.c_char_p, C.c_char_p, C.c_uint64]),
    "t3_table_load_tensor": (C.c_int32, [_KP, _AP, _AP, _AP, C.c_uint32, _WP, C.c_char_p, C.c_size_t]),
    "t3_table_load_bank": (C.c_int32, [_KP, _AP, _AP, _AP, C.c_uint32, _WP, C.c_char_p, C.c_size_t]),
    "t3_table_matmul": (C.c_int32, [C.c_void_p, _WP, _AP, _AP, C.c_void_p, C.c_size_t, C.c_char_p, C.c_size_t]),
    "t3_table_matmul_workspace_bytes": (C.c_int32, [_WP, _AP, _SZP]),
    "t3_table_moe": (C.c_int32, [C.c_char_p, C.c_size_t]),
    "t3_table_swiglu": (C.c_int32, [C.c_void_p, _WP, _WP, _WP, _AP, _AP, _AP, C.c_int32, C.c_int32, _AP, C.c_void_p,
                                    C.c_size_t, C.c_char_p, C.c_size_t]),
    "t3_table_swiglu_workspace_bytes": (C.c_int32, [_WP, _WP, _WP, _AP, _AP, _SZP]),
    "t3_test_codebooks": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "t3_test_lane": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p,
                                 C.c_void_p]),
    "t3_test_convert": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64]),
    "t3_test_mfma": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "t3_test_hbm_read": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_void_p, C.c_int32]),
}

_lib = None


def lib() -> C.CDLL:
    """The loaded library with every entry point typed. Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m turboexl3_amd.build` "
                "(there is no CPU or PyTorch fallback for the HIP kernels)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def error_name(status: int) -> str:
    return lib().t3_error_name(status).decode()
