"""ctypes declarations of the C ABI in include/mfmoe.h.

Loads the in-tree libmfmoe.so and fails loudly when it is missing: there is no
CPU fallback for any operator.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmfmoe.so")

GROUP_SIZE = 64
MAX_TOKENS = 8
MAX_TOPK = 8
MAX_EXPERTS = 512
STATIC_ACT_ELEMS = MAX_TOKENS * 32768  # MF_STATIC_ACT_ELEMS

BITS_TERNARY, BITS_2, BITS_4, BITS_8 = 1, 2, 4, 8
ROUTER_TOPK_SOFTMAX, ROUTER_FULL_SOFTMAX = 0, 1

STATUS_NAMES = {
    0: "MF_OK", -1: "MF_ERR_INVALID_ARGUMENT", -2: "MF_ERR_DIMENSION_MISMATCH",
    -3: "MF_ERR_UNSUPPORTED_BITS", -4: "MF_ERR_SCRATCH_TOO_SMALL", -5: "MF_ERR_NO_DEVICE",
    -6: "MF_ERR_OUT_OF_MEMORY", -7: "MF_ERR_LAUNCH", -10: "MF_ERR_QUERY_COUNT",
    -11: "MF_ERR_TOPK", -12: "MF_ERR_NUM_EXPERTS", -13: "MF_ERR_TILE_EXPERT_COUNT",
    -14: "MF_ERR_PAIR_COUNT", -15: "MF_ERR_TOKEN_RANGE", -16: "MF_ERR_RANK_RANGE",
    -17: "MF_ERR_EXPERT_RANGE", -18: "MF_ERR_DUPLICATE_TOKEN_RANK", -19: "MF_ERR_SORT_KEY_COUNT",
}


class ExpertOffsets(C.Structure):
    """mf_expert_offsets (MoEExpertOffsets, Kernels/MoE/MoE.swift:4-29)."""
    _fields_ = [(n, C.c_uint32) for n in (
        "gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b")]


class QTensor(C.Structure):
    """mf_qtensor: device pointers of one quantized projection."""
    _fields_ = [("weights", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p)]


class MoEConfig(C.Structure):
    _fields_ = [
        ("d", C.c_uint32), ("f", C.c_uint32), ("num_experts", C.c_uint32), ("top_k", C.c_uint32),
        ("bits", C.c_int), ("router_mode", C.c_int), ("swiglu_limit", C.c_float),
        ("shared_f", C.c_uint32), ("shared_bits", C.c_int), ("maple_rounding", C.c_uint32),
        ("gate_group_size", C.c_uint32),
    ]


class LayerWeights(C.Structure):
    _fields_ = [
        ("router_w", C.c_void_p), ("expert_base", C.c_void_p), ("expert_stride", C.c_size_t),
        ("offsets", ExpertOffsets),
        ("shared_gate", QTensor), ("shared_up", QTensor), ("shared_down", QTensor),
        ("w_sg", C.c_void_p),
        ("w_sg_q8", QTensor),
        ("expert_tiled", C.c_void_p),
    ]


class Pair(C.Structure):
    _fields_ = [("token", C.c_uint32), ("expert", C.c_uint32), ("rank", C.c_uint32),
                ("weight_bits", C.c_uint32)]


# every entry point include/mfmoe.h declares: name -> (restype, argtypes)
_P, _SZ, _U32, _I = C.c_void_p, C.c_size_t, C.c_uint32, C.c_int
SIGNATURES = {
    "mf_abi_version": (_I, []),
    "mf_status_string": (C.c_char_p, [_I]),
    "mf_ctx_create": (_I, [_I, C.POINTER(_P)]),
    "mf_ctx_destroy": (None, [_P]),
    "mf_last_hip_error": (C.c_char_p, [_P]),
    "mf_quantize_affine": (_I, [_P, _P, _P, _SZ, _SZ, _I, _P, _P, _P]),
    "mf_dequantize": (_I, [_P, _P, QTensor, _SZ, _SZ, _I, _P]),
    "mf_gemv": (_I, [_P, _P, QTensor, _I, _P, _P, _U32, _U32, _U32, _I]),
    "mf_silu_mul": (_I, [_P, _P, _P, _P, _P, _U32]),
    "mf_sigmoid_scalar_mul": (_I, [_P, _P, _P, _P, _U32, _U32]),
    "mf_residual_add": (_I, [_P, _P, _P, _P, _U32]),
    "mf_residual_rmsnorm": (_I, [_P, _P, _P, _P, _P, _P, _U32, _U32, C.c_float]),
    "mf_shared_expert": (_I, [_P, _P, _P, QTensor, QTensor, QTensor, _I, _U32, _U32, _U32, _P, _P,
                              _SZ]),
    "mf_shared_expert_scratch_bytes": (_SZ, [_U32, _U32, _U32]),
    "mf_shared_expert_int8": (_I, [_P, _P, _P, QTensor, QTensor, QTensor, _U32, _U32, _U32, _I, _P, _P, _SZ]),
    "mf_qmm_workspace_bytes": (_SZ, [_U32, _U32, _U32]),
    "mf_qmm": (_I, [_P, _P, QTensor, _I, _P, _P, _U32, _U32, _U32, _I, _P, _SZ]),
    "mf_qmm_path": (_I, [QTensor, _I, _P, _P, _U32, _U32, _U32, _P, _SZ]),
    "mf_shared_expert_static": (_I, [_P, _P, _P, QTensor, QTensor, QTensor, _I, _U32, _U32, _U32, _P]),
    "mf_expert_blob_layout": (_I, [_U32, _U32, _I, _U32, C.POINTER(ExpertOffsets), C.POINTER(_SZ), C.POINTER(_SZ)]),
    "mf_expert_blob_layout_repacked": (_I, [_U32, _U32, _I, _U32, C.POINTER(ExpertOffsets), C.POINTER(_SZ), C.POINTER(_SZ)]),
    "mf_moe_config_check": (_I, [C.POINTER(MoEConfig)]),
    "mf_moe_create": (_I, [_P, C.POINTER(MoEConfig), C.POINTER(_P)]),
    "mf_moe_destroy": (None, [_P]),
    "mf_moe_router": (_I, [_P, _P, _P, _P, _U32, _U32, _P, _P, _P]),
    "mf_router_sqrtsoftplus": (_I, [_P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _P, C.c_float, _P, _P, _P]),
    "mf_router_hash_weights": (_I, [_P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _P, C.c_float, _P, _P]),
    "mf_router_inkling": (_I, [_P, _P, _P, _P, _U32, _U32, _U32, _U32, _U32, _U32, _P, _P, C.c_float, _P,
                               _P, _P, _P]),
    "mf_router_gemma4": (_I, [_P, _P, _P, _P, _P, _P, _U32, _U32, _P, _P, _U32, _U32, _U32, _P, _P, _P]),
    "mf_moe_phase1": (_I, [_P, _P, _P, _SZ, C.POINTER(ExpertOffsets), _P, _P, _U32, _U32, _P]),
    "mf_moe_phase1_subset": (_I, [_P, _P, _P, _SZ, C.POINTER(ExpertOffsets), _P, _P, _U32, _U32, _P, _P, _U32]),
    "mf_moe_phase2": (_I, [_P, _P, _P, _SZ, C.POINTER(ExpertOffsets), _P, _P, _P, _P, _U32, _P]),
    "mf_moe_decode_layer": (_I, [_P, _P, C.POINTER(LayerWeights), _P, _U32, _P, _P, _P, _P]),
    "mf_moe_decode_layer_normed": (_I, [_P, _P, C.POINTER(LayerWeights), _P, _P, _P, C.c_float, _U32, _P, _P, _P]),
    "mf_moe_set_fused": (_I, [_P, _I]),
    "mf_moe_set_prefill_route_rounding": (_I, [_P, _I]),
    "mf_moe_tile_experts": (_I, [_P, _P, _P, _SZ, C.POINTER(ExpertOffsets), _P]),
    "mf_moe_status": (_I, [_P, _P]),
    "mf_moe_set_phase_trace": (_I, [_P, _P, _SZ]),
    "mf_ctx_num_cu": (_I, [_P]),
    "mf_moe_group": (_I, [_P, _P, _P, _P, _U32, _P, _P, _P]),
    "mf_moe_group_status": (_I, [_P, _P]),
    "mf_moe_prefill_workspace_bytes": (_SZ, [_P, _U32]),
    "mf_moe_prefill_layer": (_I, [_P, _P, C.POINTER(LayerWeights), _P, _U32, _P, _P, _SZ, _P, _P]),
    "mf_moe_slot_lookup": (_I, [_P, _P, _P, _U32, _P, C.c_uint64, _P, _P]),
    "mf_moe_phase1_slots": (_I, [_P, _P, _P, _P, _P, C.POINTER(ExpertOffsets), _P, _U32, _U32, _P]),
    "mf_moe_phase2_slots": (_I, [_P, _P, _P, _P, _P, C.POINTER(ExpertOffsets), _P, _P, _P, _U32, _P]),
    "mf_moe_ragged_qmm": (_I, [_P, _P, _P, _SZ, C.POINTER(ExpertOffsets), _P, _P, _P, _U32, _P, _P, _SZ]),
    "mf_moe_unpermute": (_I, [_P, _P, _P, _P, _P, _P, _U32, _P]),
    "mf_group_pairs_host": (_I, [_P, _SZ, _I, _I, _I, _I, _P, _SZ, _P, _P, _P, _P,
                                 C.POINTER(_SZ), _P, C.POINTER(_SZ), _P]),
}

_lib = None


class LibraryMissing(RuntimeError):
    pass


def lib() -> C.CDLL:
    """The loaded libmfmoe.so.  Raises LibraryMissing if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                f"{LIB_PATH} is missing: build it with `python -m mference_amd.build` "
                "(there is no CPU fallback)")
        # torch carries its own HIP runtime; it has to be the one already loaded
        # when libmfmoe resolves libamdhip64, or device pointers and streams
        # would belong to a different runtime instance than the kernels.
        import torch  # noqa: F401
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class MfError(RuntimeError):
    """A negative mf_status (the reference's `throws` / precondition failures)."""

    def __init__(self, status: int, detail: str = ""):
        self.status = status
        self.name = STATUS_NAMES.get(status, str(status))
        text = lib().mf_status_string(status).decode()
        super().__init__(f"{self.name}: {text}" + (f" ({detail})" if detail else ""))


def check(status: int, ctx=None) -> None:
    if status != 0:
        detail = ""
        if status == -7 and ctx:
            detail = lib().mf_last_hip_error(ctx).decode()
        raise MfError(status, detail)
