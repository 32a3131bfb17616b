"""ctypes binding of libmfq_amd.so (the C ABI declared in include/mfq_amd.h).

The library is the product: there is no CPU fallback.  Loading fails with an explicit
error when the shared object has not been built (``python -m mfq_amd.build``).
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path

ROOT = Path(__file__).resolve().parent
LIB_PATH = ROOT / "libmfq_amd.so"

OK, ERR_INVALID, ERR_RUNTIME, ERR_UNSUPPORTED = 0, -1, -2, -3
FAMILY_NINT, FAMILY_NVQ, FAMILY_MXFP4 = 1, 2, 3
F32, F16, BF16 = 0, 1, 2

c_void_pp = C.POINTER(C.c_void_p)


class Projection(C.Structure):
    """``mfq_amd_projection``."""
    _fields_ = [
        ("fields", C.c_void_p * 9),
        ("sizes", C.c_int64 * 3),
        ("expert_local", C.c_void_p),
        ("family", C.c_int32),
        ("local_experts", C.c_int32), ("output_rows", C.c_int32), ("input_width", C.c_int32),
        ("groups", C.c_int32), ("group_size", C.c_int32),
        ("format", C.c_int32), ("sub_bits", C.c_int32), ("sign_mode", C.c_int32),
        ("nvec", C.c_int32), ("nsign", C.c_int32),
        ("uniform_bits", C.c_int32),
        ("q_expert_stride", C.c_int64),
        ("reserved", C.c_int64 * 2),
    ]


class MoeTensor(C.Structure):
    """``mfq_amd_moe_tensor``."""
    _fields_ = [("pools", C.POINTER(Projection)), ("pool_count", C.c_int32),
                ("experts", C.c_int32), ("out_per_expert", C.c_int32), ("neuron_len", C.c_int32)]


class MoeFfnConfig(C.Structure):
    """``mfq_amd_moe_ffn_config``."""
    _fields_ = [("gate", MoeTensor), ("up", MoeTensor), ("down", MoeTensor),
                ("top_k", C.c_int32), ("max_tokens", C.c_int32), ("x_dtype", C.c_int32),
                ("out_dtype", C.c_int32), ("swiglu_limit", C.c_float), ("decode_token_limit", C.c_int32),
                ("launch_mode", C.c_int32), ("mx_scaled_mfma", C.c_int32), ("expert_activation", C.c_int32),
                ("group_pairs", C.c_int32)]


EXPORTS = {
    # name: (restype, argtypes)
    "mfq_amd_last_error": (C.c_char_p, []),
    "mfq_amd_abi_version": (C.c_int, []),
    "mfq_amd_init": (C.c_int, []),
    "mfq_amd_moe_ffn_decode_limit": (C.c_int32, [C.c_int32, C.c_int32]),
    "mfq_amd_tensor_load": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int64, C.c_int32, c_void_pp]),
    "mfq_amd_tensor_host_view": (C.c_int, [C.c_void_p, C.POINTER(Projection)]),
    "mfq_amd_tensor_upload": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.POINTER(Projection)]),
    "mfq_amd_tensor_free": (None, [C.c_void_p]),
    "mfq_amd_mfe_load": (C.c_int, [C.c_void_p, C.c_int64, c_void_pp]),
    "mfq_amd_mfe_info": (C.c_int, [C.c_void_p] + [C.POINTER(C.c_int32)] * 4),
    "mfq_amd_mfe_pool": (C.c_int, [C.c_void_p, C.c_int32, c_void_pp, c_void_pp, C.POINTER(C.c_int32)]),
    "mfq_amd_mfe_upload": (C.c_int, [C.c_void_p, C.POINTER(Projection), C.c_int32]),
    "mfq_amd_mfe_free": (None, [C.c_void_p]),
    "mfq_amd_nvq_grid": (C.c_int, [C.c_char_p, C.c_void_p, C.c_int64, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "mfq_amd_dequant": (C.c_int, [C.POINTER(Projection), C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_gemv": (C.c_int, [C.POINTER(Projection), C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.c_int64,
                               C.c_void_p, C.c_int64, C.c_void_p]),
    "mfq_amd_router_logits": (C.c_int, [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                        C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_topk": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_float,
                               C.c_float, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mfq_amd_route_plan": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                     C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "mfq_amd_moe_ffn_create": (C.c_int, [C.POINTER(MoeFfnConfig), c_void_pp]),
    "mfq_amd_moe_ffn_run_logits": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_float, C.c_float,
                                            C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_moe_ffn_run_router": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_float, C.c_float,
                                            C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_moe_ffn_set_shared": (C.c_int, [C.c_void_p, C.POINTER(Projection), C.POINTER(Projection), C.POINTER(Projection),
                                            C.c_int32]),
    "mfq_amd_moe_ffn_run_shared": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                            C.c_void_p, C.c_void_p]),
    "mfq_amd_moe_ffn_routes": (C.c_int, [C.c_void_p, c_void_pp, c_void_pp]),
    "mfq_amd_moe_ffn_mx_scaled_slots": (C.c_int, [C.c_void_p, C.POINTER(C.c_int32)]),
    "mfq_amd_moe_ffn_run": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_void_p,
                                      C.c_void_p]),
    "mfq_amd_moe_ffn_buffers": (C.c_int, [C.c_void_p, c_void_pp, c_void_pp]),
    "mfq_amd_moe_ffn_touched_bytes": (C.c_int, [C.c_void_p, C.POINTER(C.c_int64), C.POINTER(C.c_int32)]),
    "mfq_amd_moe_ffn_enable_timing": (C.c_int, [C.c_void_p, C.c_int32]),
    "mfq_amd_moe_ffn_stage_times": (C.c_int, [C.c_void_p, C.POINTER(C.c_float)]),
    "mfq_amd_moe_ffn_empty_bracket_ms": (C.c_int, [C.c_void_p, C.POINTER(C.c_float)]),
    "mfq_amd_moe_ffn_destroy": (None, [C.c_void_p]),
    "mfq_amd_grouped_matmul_workspace": (C.c_int64, [C.c_int32, C.c_int32, C.c_int32]),
    "mfq_amd_grouped_matmul": (C.c_int, [C.POINTER(MoeTensor), C.c_void_p, C.c_int32, C.c_int32, C.c_void_p,
                                         C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]),
    "mfq_amd_grouped_matmul_static_capacity": (C.c_int64, []),
    "mfq_amd_grouped_matmul_static": (C.c_int, [C.POINTER(MoeTensor), C.c_void_p, C.c_int32, C.c_int32, C.c_void_p,
                                                C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_swiglu": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_float, C.c_void_p, C.c_void_p]),
    "mfq_amd_weighted_reduce_shared_gate": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                                     C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_add_shared_gate": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]),
    "mfq_amd_weighted_reduce": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_void_p,
                                          C.c_int32, C.c_void_p]),
}

_lib = None


class MfqAmdError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"mfq_amd status {status}: {message}")
        self.status = status


class InvalidArgument(MfqAmdError, ValueError):
    """MFQ_AMD_ERR_INVALID -- the reference raises std::invalid_argument here."""


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension has not been built. "
                "Run `python -m mfq_amd.build` (or __graft_entry__.build()); there is no CPU fallback.")
        handle = C.CDLL(str(LIB_PATH))
        for name, (restype, argtypes) in EXPORTS.items():
            fn = getattr(handle, name)      # AttributeError if the export is missing
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status == OK:
        return
    message = lib().mfq_amd_last_error().decode("utf-8", "replace")
    if status == ERR_INVALID:
        raise InvalidArgument(status, message)
    raise MfqAmdError(status, message)
