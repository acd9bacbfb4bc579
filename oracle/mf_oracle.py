"""ctypes binding of the CPU oracle (libmf_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmf_oracle.so")

BITS_TERNARY, BITS_2, BITS_4, BITS_8 = 1, 2, 4, 8
GROUP = 64

ERR = {
    -1: "invalidQueryCount", -2: "invalidTopK", -3: "invalidNumExperts",
    -4: "invalidTileExpertCount", -5: "pairCountMismatch", -6: "tokenOutOfRange",
    -7: "rankOutOfRange", -8: "expertOutOfRange", -9: "duplicateTokenRank",
    -10: "expertSortKeyCountMismatch", -20: "badArgument",
}


def build() -> str:
    """Compile the oracle with its Makefile (always recompiles)."""
    subprocess.run(["make", "-B", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


class ExpertOffsets(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b", "down_w", "down_s", "down_b")]


class _Rng(C.Structure):
    _fields_ = [("state", C.c_uint64)]


class _Layer(C.Structure):
    _fields_ = [
        ("d", C.c_size_t), ("f", C.c_size_t), ("e", C.c_size_t), ("k", C.c_size_t),
        ("fs", C.c_size_t), ("bits", C.c_int), ("shared_bits", C.c_int),
        ("router_mode", C.c_int), ("swiglu_limit", C.c_float),
        ("router_w", C.c_void_p), ("experts", C.c_void_p), ("expert_stride", C.c_size_t),
        ("off", ExpertOffsets),
        ("sgw", C.c_void_p), ("sgs", C.c_void_p), ("sgb", C.c_void_p),
        ("suw", C.c_void_p), ("sus", C.c_void_p), ("sub", C.c_void_p),
        ("sdw", C.c_void_p), ("sds", C.c_void_p), ("sdb", C.c_void_p),
        ("w_sg", C.c_void_p), ("maple_rounding", C.c_int), ("gate_group", C.c_int),
        ("gqw", C.c_void_p), ("gqs", C.c_void_p), ("gqb", C.c_void_p),
        ("narrow_routes", C.c_int),
    ]


PAIR_DTYPE = np.dtype([("token", "<u4"), ("expert", "<u4"), ("rank", "<u4"),
                       ("weight_bits", "<u4")])
GROUP_DTYPE = np.dtype([("expert", "<u4"), ("pair_start", "<u4"), ("pair_count", "<u4")])
TILE_DTYPE = np.dtype([("group_start", "<u4"), ("group_count", "<u4"),
                       ("pair_start", "<u4"), ("pair_count", "<u4")])

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.mfo_bf16_bits.restype = C.c_uint16
        L.mfo_bf16_bits.argtypes = [C.c_float]
        L.mfo_bf16_to_float.restype = C.c_float
        L.mfo_bf16_to_float.argtypes = [C.c_uint16]
        L.mfo_rng_seed.restype = _Rng
        L.mfo_rng_seed.argtypes = [C.c_uint64]
        L.mfo_seed_tree_key.restype = _Rng
        L.mfo_seed_tree_key.argtypes = [C.c_uint64, C.c_char_p]
        L.mfo_rng_next.restype = C.c_uint64
        L.mfo_rng_next.argtypes = [C.POINTER(_Rng)]
        L.mfo_rng_uniform.restype = C.c_float
        L.mfo_rng_uniform.argtypes = [C.POINTER(_Rng), C.c_float, C.c_float]
        L.mfo_rng_normal.restype = None
        L.mfo_rng_normal.argtypes = [C.POINTER(_Rng), C.c_float, C.c_float, C.c_void_p, C.c_size_t]
        L.mfo_rng_uniform_fill.restype = None
        L.mfo_rng_uniform_fill.argtypes = [C.POINTER(_Rng), C.c_float, C.c_float, C.c_void_p,
                                           C.c_size_t]
        L.mfo_exp.restype = C.c_float
        L.mfo_exp.argtypes = [C.c_float]
        for fn in (L.mfo_log_1to2, L.mfo_sqrtsoftplus):
            fn.restype = C.c_float
            fn.argtypes = [C.c_float]
        L.mfo_dot_int8_laneorder.restype = C.c_float
        L.mfo_dot_int8_laneorder.argtypes = [C.c_void_p] * 5 + [C.c_size_t]
        L.mfo_silu.restype = C.c_float
        L.mfo_silu.argtypes = [C.c_float]
        L.mfo_dot_bf16_laneorder.restype = C.c_float
        L.mfo_dot_bf16_laneorder.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.mfo_packed_row_bytes.restype = C.c_size_t
        L.mfo_packed_row_bytes.argtypes = [C.c_int, C.c_size_t]
        _lib = L
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------- bf16

def bf16_bits(x) -> np.ndarray:
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().mfo_bf16_encode(_p(x), C.c_size_t(x.size), _p(out))
    return out


def bf16_to_float(b) -> np.ndarray:
    b = _c(b, np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().mfo_bf16_decode(_p(b), C.c_size_t(b.size), _p(out))
    return out


# ---------------------------------------------------------------- PRNG

class Rng:
    """SplitMix64 stream (MferenceValidation/Support/PRNG/SplitMix64.swift)."""

    def __init__(self, seed: int):
        self._r = lib().mfo_rng_seed(C.c_uint64(seed & 0xFFFFFFFFFFFFFFFF))

    @classmethod
    def key(cls, root: int, label: str) -> "Rng":
        r = cls.__new__(cls)
        r._r = lib().mfo_seed_tree_key(C.c_uint64(root & 0xFFFFFFFFFFFFFFFF), label.encode())
        return r

    def next(self) -> int:
        return int(lib().mfo_rng_next(C.byref(self._r)))

    def uniform(self, lo: float, hi: float) -> float:
        return float(lib().mfo_rng_uniform(C.byref(self._r), lo, hi))

    def uniform_fill(self, lo: float, hi: float, n: int) -> np.ndarray:
        out = np.empty(n, np.float32)
        lib().mfo_rng_uniform_fill(C.byref(self._r), lo, hi, _p(out), C.c_size_t(n))
        return out

    def normal(self, mean: float, sigma: float, n: int) -> np.ndarray:
        out = np.empty(n, np.float32)
        lib().mfo_rng_normal(C.byref(self._r), mean, sigma, _p(out), C.c_size_t(n))
        return out


# ---------------------------------------------------------------- quantization

@dataclass
class QTensor:
    """rows x n affine-quantized tensor: packed codes + bf16 scale/bias per 64."""
    packed: np.ndarray   # uint8 [rows, row_bytes]
    scales: np.ndarray   # uint16 [rows, n/64]
    biases: Optional[np.ndarray]  # uint16 [rows, n/64] (None for ternary)
    bits: int
    rows: int
    n: int


def packed_row_bytes(bits: int, n: int) -> int:
    return int(lib().mfo_packed_row_bytes(bits, n))


def quantize(w, bits: int = BITS_4) -> QTensor:
    w = _c(w, np.float32)
    rows, n = w.shape
    packed = np.empty((rows, packed_row_bytes(bits, n)), np.uint8)
    scales = np.empty((rows, n // GROUP), np.uint16)
    biases = np.empty((rows, n // GROUP), np.uint16)
    rc = lib().mfo_quantize_affine(_p(w), C.c_size_t(rows), C.c_size_t(n), bits, _p(packed),
                                   _p(scales), _p(biases))
    if rc:
        raise ValueError(f"mfo_quantize_affine: {ERR.get(rc, rc)}")
    return QTensor(packed, scales, biases, bits, rows, n)


def pack_codes(codes, bits: int) -> np.ndarray:
    codes = _c(codes, np.uint8)
    rows, n = codes.shape
    packed = np.empty((rows, packed_row_bytes(bits, n)), np.uint8)
    rc = lib().mfo_pack_codes(_p(codes), C.c_size_t(rows), C.c_size_t(n), bits, _p(packed))
    if rc:
        raise ValueError("mfo_pack_codes")
    return packed


def dequantize(q: QTensor) -> np.ndarray:
    out = np.empty((q.rows, q.n), np.float32)
    rc = lib().mfo_dequantize(_p(q.packed), _p(q.scales), _p(q.biases), C.c_size_t(q.rows),
                              C.c_size_t(q.n), q.bits, _p(out))
    if rc:
        raise ValueError("mfo_dequantize")
    return out


# ---------------------------------------------------------------- router

def exp(x: float) -> float:
    return float(lib().mfo_exp(C.c_float(x)))


def silu(x: float) -> float:
    return float(lib().mfo_silu(C.c_float(x)))


def dot_bf16_laneorder(w, x) -> float:
    w = _c(w, np.uint16)
    x = _c(x, np.uint16)
    return float(lib().mfo_dot_bf16_laneorder(_p(w), _p(x), C.c_size_t(x.size)))


def router_logits(w, x) -> np.ndarray:
    w = _c(w, np.uint16)
    x = _c(x, np.uint16)
    e, d = w.shape
    out = np.empty(e, np.float32)
    lib().mfo_router_logits_bf16(_p(w), _p(x), C.c_size_t(e), C.c_size_t(d), _p(out))
    return out


def topk_softmax(logits, k: int, full_softmax: bool = False):
    logits = _c(logits, np.float32)
    idx = np.empty(k, np.uint32)
    w = np.empty(k, np.float32)
    fn = lib().mfo_topk_full_softmax if full_softmax else lib().mfo_topk_softmax
    fn(_p(logits), C.c_size_t(logits.size), C.c_size_t(k), _p(idx), _p(w))
    return idx, w


def log_1to2(t: float) -> float:
    return float(lib().mfo_log_1to2(C.c_float(t)))


def sqrtsoftplus(x: float) -> float:
    return float(lib().mfo_sqrtsoftplus(C.c_float(x)))


def router_sqrtsoftplus(logits, correction_bias, k: int, route_scale: float):
    """DeepSeek-V4 learned routing: (indices, weights)."""
    logits = _c(logits, np.float32)
    bias = _c(correction_bias, np.float32)
    idx = np.empty(k, np.uint32)
    w = np.empty(k, np.float32)
    lib().mfo_router_sqrtsoftplus(_p(logits), _p(bias), C.c_size_t(logits.size), C.c_size_t(k),
                                  C.c_float(route_scale), _p(idx), _p(w))
    return idx, w


def router_hash_weights(logits, indices, route_scale: float) -> np.ndarray:
    """DeepSeek-V4 hash routing: weights of the given experts."""
    logits = _c(logits, np.float32)
    idx = _c(indices, np.uint32)
    w = np.empty(idx.size, np.float32)
    lib().mfo_router_hash_weights(_p(logits), _p(idx), C.c_size_t(idx.size), C.c_float(route_scale), _p(w))
    return w


def router_inkling(logits, bias, global_scale: float, n_routed: int, n_shared: int, k: int,
                   route_scale: float):
    """Inkling sigmoid router with shared sinks: (indices, weights, gammas)."""
    logits = _c(logits, np.float32)
    bias = _c(bias, np.float32)
    assert logits.size == n_routed + n_shared and k <= 8 and n_shared <= 8
    idx = np.empty(k, np.uint32)
    w = np.empty(k, np.float32)
    gam = np.empty(max(n_shared, 1), np.float32)
    lib().mfo_router_inkling(_p(logits), _p(bias), C.c_float(global_scale), C.c_size_t(n_routed),
                             C.c_size_t(n_shared), C.c_size_t(k), C.c_float(route_scale), _p(idx), _p(w),
                             _p(gam))
    return idx, w, gam[:n_shared]


def router_logits_int8(codes, scales, biases, x, effective_scale) -> np.ndarray:
    """Gemma's 8-bit affine router rows in the build's lane order."""
    codes = _c(codes, np.uint8)
    scales = _c(scales, np.uint16)
    biases = _c(biases, np.uint16)
    x = _c(x, np.uint16)
    es = _c(effective_scale, np.uint16)
    e, d = codes.shape
    out = np.empty(e, np.float32)
    lib().mfo_router_logits_int8(_p(codes), _p(scales), _p(biases), _p(x), _p(es), C.c_size_t(e),
                                 C.c_size_t(d), _p(out))
    return out


def topk_softmax_scaled(logits, per_expert_scale, k: int):
    logits = _c(logits, np.float32)
    sc = _c(per_expert_scale, np.uint16)
    idx = np.empty(k, np.uint32)
    w = np.empty(k, np.float32)
    lib().mfo_topk_softmax_scaled(_p(logits), _p(sc), C.c_size_t(logits.size), C.c_size_t(k), _p(idx), _p(w))
    return idx, w


# ---------------------------------------------------------------- GEMV / FFN

def gemv(q: QTensor, x) -> np.ndarray:
    x = _c(x, np.float32)
    y = np.empty(q.rows, np.float32)
    rc = lib().mfo_gemv(_p(q.packed), _p(q.scales), _p(q.biases), q.bits, C.c_size_t(q.rows),
                        C.c_size_t(q.n), _p(x), _p(y))
    if rc:
        raise ValueError("mfo_gemv")
    return y


def gemv_multix(q: QTensor, x_bits) -> np.ndarray:
    x_bits = _c(x_bits, np.uint16)
    t = x_bits.shape[0]
    y = np.empty((t, q.rows), np.float32)
    rc = lib().mfo_gemv_multix(_p(q.packed), _p(q.scales), _p(q.biases), q.bits,
                               C.c_size_t(q.rows), C.c_size_t(q.n), C.c_size_t(t), _p(x_bits),
                               _p(y))
    if rc:
        raise ValueError("mfo_gemv_multix")
    return y


def expert_phase1(blob, off: ExpertOffsets, bits: int, d: int, f: int, x_bits,
                  swiglu_limit: float = 0.0, maple: bool = False, gate_group: int = GROUP) -> np.ndarray:
    blob = _c(blob, np.uint8)
    x_bits = _c(x_bits, np.uint16)
    acts = np.empty(f, np.uint16)
    rc = lib().mfo_expert_phase1_gate(_p(blob), C.byref(off), bits, C.c_size_t(d), C.c_size_t(f),
                                      C.c_size_t(gate_group), C.c_float(swiglu_limit),
                                      C.c_int(1 if maple else 0), _p(x_bits), _p(acts))
    if rc:
        raise ValueError("mfo_expert_phase1")
    return acts


def expert_down(blob, off: ExpertOffsets, bits: int, d: int, f: int, acts_bits) -> np.ndarray:
    blob = _c(blob, np.uint8)
    acts_bits = _c(acts_bits, np.uint16)
    v = np.empty(d, np.float32)
    rc = lib().mfo_expert_down(_p(blob), C.byref(off), bits, C.c_size_t(d), C.c_size_t(f),
                               _p(acts_bits), _p(v))
    if rc:
        raise ValueError("mfo_expert_down")
    return v


def shared_expert(gate: QTensor, up: QTensor, down: QTensor, x_bits) -> np.ndarray:
    x_bits = _c(x_bits, np.uint16)
    d, f = gate.n, gate.rows
    y = np.empty(d, np.uint16)
    rc = lib().mfo_shared_expert(_p(gate.packed), _p(gate.scales), _p(gate.biases),
                                 _p(up.packed), _p(up.scales), _p(up.biases),
                                 _p(down.packed), _p(down.scales), _p(down.biases),
                                 gate.bits, C.c_size_t(d), C.c_size_t(f), _p(x_bits), _p(y))
    if rc:
        raise ValueError("mfo_shared_expert")
    return y


def gelu_tanh(x: float) -> float:
    """the tanh form of GELU on the build's exp (dequant_int8.metal:44-49)"""
    fn = lib().mfo_gelu_tanh
    fn.restype = C.c_float
    fn.argtypes = [C.c_float]
    return float(fn(C.c_float(x)))


def shared_expert_int8(gate: QTensor, up: QTensor, down: QTensor, x_bits, silu: bool = False) -> np.ndarray:
    """SharedExpertInt8.encode (SharedExpertInt8.swift:78-181) for one token row; 8-bit affine tensors"""
    x_bits = _c(x_bits, np.uint16)
    d, f = gate.n, gate.rows
    y = np.empty(d, np.uint16)
    rc = lib().mfo_shared_expert_int8(_p(gate.packed), _p(gate.scales), _p(gate.biases),
                                      _p(up.packed), _p(up.scales), _p(up.biases),
                                      _p(down.packed), _p(down.scales), _p(down.biases),
                                      C.c_size_t(d), C.c_size_t(f), C.c_int(1 if silu else 0), _p(x_bits), _p(y))
    if rc:
        raise ValueError("mfo_shared_expert_int8")
    return y


def maple_swiglu(gate: float, up: float) -> float:
    """MapleMoE's activation, every intermediate a bf16 number (maple_moe.metal:153-164)"""
    fn = lib().mfo_maple_swiglu
    fn.restype = C.c_float
    fn.argtypes = [C.c_float, C.c_float]
    return float(fn(gate, up))


def residual_rmsnorm(hidden_bits, weight_bits, eps: float, delta_bits=None):
    """rows of hidden [t, d] (or [d]): (hidden after the add, normalised rows), both uint16"""
    h = _c(hidden_bits, np.uint16).copy()
    w = _c(weight_bits, np.uint16)
    h2 = h.reshape(-1, w.size)
    dl = None if delta_bits is None else _c(delta_bits, np.uint16).reshape(h2.shape)
    out = np.empty_like(h2)
    for i in range(h2.shape[0]):
        lib().mfo_residual_rmsnorm(_p(h2[i]), None if dl is None else _p(dl[i]), _p(w), _p(out[i]),
                                   C.c_size_t(w.size), C.c_float(eps))
    return h2.reshape(h.shape), out.reshape(h.shape)


def sigmoid_scalar_mul(y_bits, gate_bits: int) -> np.ndarray:
    y = _c(y_bits, np.uint16).copy()
    lib().mfo_sigmoid_scalar_mul(_p(y), C.c_size_t(y.size), C.c_uint16(gate_bits))
    return y


@dataclass
class Layer:
    """Host copy of one MoE layer's tensors, laid out as the kernels read them."""
    d: int
    f: int
    e: int
    k: int
    bits: int
    router_w: np.ndarray            # uint16 [e, d]
    experts: np.ndarray             # uint8 [e, stride]
    off: ExpertOffsets
    fs: int = 0
    shared_bits: int = BITS_4
    shared: Optional[tuple] = None  # (gate, up, down) QTensors
    w_sg: Optional[np.ndarray] = None  # uint16 [d]
    router_mode: int = 0
    swiglu_limit: float = 0.0
    maple_rounding: bool = False    # MapleMoE's activation and bf16 down outputs
    gate_group: int = GROUP         # group of the routed gate tables (32: the DeepSeek-V4 conversion)
    w_sg_q8: Optional["QTensor"] = None  # the scalar gate as an 8-bit affine row [1, d] (replaces w_sg)
    narrow_routes: bool = False     # a route's down output narrowed to bf16 before its weight (prefill.metal:817-819)

    def _struct(self) -> _Layer:
        L = _Layer()
        L.d, L.f, L.e, L.k, L.fs = self.d, self.f, self.e, self.k, self.fs
        L.bits, L.shared_bits = self.bits, self.shared_bits
        L.router_mode, L.swiglu_limit = self.router_mode, self.swiglu_limit
        L.maple_rounding = 1 if self.maple_rounding else 0
        L.narrow_routes = 1 if self.narrow_routes else 0
        L.gate_group = self.gate_group
        L.router_w = self.router_w.ctypes.data
        L.experts = self.experts.ctypes.data
        L.expert_stride = self.experts.strides[0]
        L.off = self.off
        if self.shared is not None:
            g, u, dn = self.shared
            L.sgw, L.sgs, L.sgb = g.packed.ctypes.data, g.scales.ctypes.data, g.biases.ctypes.data
            L.suw, L.sus, L.sub = u.packed.ctypes.data, u.scales.ctypes.data, u.biases.ctypes.data
            L.sdw, L.sds, L.sdb = dn.packed.ctypes.data, dn.scales.ctypes.data, dn.biases.ctypes.data
        if self.w_sg is not None:
            L.w_sg = self.w_sg.ctypes.data
        if self.w_sg_q8 is not None:
            q = self.w_sg_q8
            L.gqw, L.gqs, L.gqb = q.packed.ctypes.data, q.scales.ctypes.data, q.biases.ctypes.data
        return L


def moe_layer(layer: Layer, x_bits):
    """x_bits uint16 [t, d] (or [d]) -> (y uint16 [t,d], idx uint32 [t,k], w f32 [t,k])."""
    x_bits = _c(x_bits, np.uint16)
    single = x_bits.ndim == 1
    x2 = x_bits.reshape(-1, layer.d)
    t = x2.shape[0]
    y = np.empty((t, layer.d), np.uint16)
    idx = np.empty((t, layer.k), np.uint32)
    w = np.empty((t, layer.k), np.float32)
    S = layer._struct()
    rc = lib().mfo_moe_layer_tokens(C.byref(S), _p(x2), C.c_size_t(t), _p(y), _p(idx), _p(w), 1)
    if rc:
        raise ValueError(f"mfo_moe_layer_tokens rc={rc}")
    if single:
        return y[0], idx[0], w[0]
    return y, idx, w


def moe_layer_logits(layer: Layer, x_bits) -> np.ndarray:
    return router_logits(layer.router_w, x_bits)


# ---------------------------------------------------------------- grouping

class GroupingError(ValueError):
    def __init__(self, code: int):
        super().__init__(ERR.get(code, str(code)))
        self.code = code
        self.kind = ERR.get(code, str(code))


def make_pairs(idx, weight_bits) -> np.ndarray:
    idx = _c(idx, np.uint32)
    weight_bits = _c(weight_bits, np.uint32)
    t, k = idx.shape
    out = np.empty(t * k, PAIR_DTYPE)
    lib().mfo_make_pairs(_p(idx), _p(weight_bits), C.c_size_t(t), C.c_size_t(k), _p(out))
    return out


def group_pairs(pairs, query_count: int, top_k: int, num_experts: int,
                tile_expert_count: int = 16, sort_keys=None):
    pairs = _c(pairs, PAIR_DTYPE)
    n = pairs.size
    sorted_ = np.empty(n, PAIR_DTYPE)
    ne = max(num_experts, 1)
    offsets = np.empty(ne, np.uint32)
    counts = np.empty(ne, np.uint32)
    groups = np.empty(max(min(ne, n), 1), GROUP_DTYPE)
    tiles = np.empty(max(min(ne, n), 1), TILE_DTYPE)
    ng, nt = C.c_size_t(0), C.c_size_t(0)
    keys = None if sort_keys is None else _c(sort_keys, np.uint64)
    rc = lib().mfo_group_pairs(_p(pairs), C.c_size_t(n), query_count, top_k, num_experts,
                               tile_expert_count, _p(keys),
                               C.c_size_t(0 if keys is None else keys.size), _p(sorted_),
                               _p(offsets), _p(counts), _p(groups), C.byref(ng), _p(tiles),
                               C.byref(nt))
    if rc:
        raise GroupingError(rc)
    return dict(sorted=sorted_, offsets=offsets, counts=counts, groups=groups[:ng.value],
                tiles=tiles[:nt.value])


def reduce_token_major(partials, w) -> np.ndarray:
    partials = _c(partials, np.float32)
    w = _c(w, np.float32)
    t, k, d = partials.shape
    out = np.empty((t, d), np.float32)
    lib().mfo_reduce_token_major(_p(partials), _p(w), C.c_size_t(t), C.c_size_t(k),
                                 C.c_size_t(d), _p(out))
    return out


# ---------------------------------------------------------------- layer builder

def blob_layout(d: int, f: int, bits: int, align: int = 256, gate_group: int = GROUP):
    """Sub-tensor byte offsets inside one expert blob, in the reference's order
    gate{W,s,b}, up{W,s,b}, down{W,s,b} (RepackPlanner.swift:544-712), and the
    blob stride rounded up to `align`.  Ternary stores no biases.  `gate_group` 32: the gate
    tables hold an entry per 32 weights (ModelExpertIO.swift:118-135)."""
    gu_w = f * packed_row_bytes(bits, d)
    gu_s = f * (d // GROUP) * 2
    dn_w = d * packed_row_bytes(bits, f)
    dn_s = d * (f // GROUP) * 2
    has_b = bits != BITS_TERNARY
    off = ExpertOffsets()
    pos = 0
    for name, wsz, ssz in (("gate", gu_w, f * (d // gate_group) * 2), ("up", gu_w, gu_s), ("down", dn_w, dn_s)):
        setattr(off, f"{name}_w", pos)
        pos += wsz
        setattr(off, f"{name}_s", pos)
        pos += ssz
        setattr(off, f"{name}_b", pos if has_b else 0)
        if has_b:
            pos += ssz
    stride = (pos + align - 1) // align * align
    return off, pos, stride


def pack_expert_blob(gate: QTensor, up: QTensor, down: QTensor, off: ExpertOffsets,
                     out: np.ndarray) -> None:
    for name, q in (("gate", gate), ("up", up), ("down", down)):
        wo, so, bo = (getattr(off, f"{name}_{s}") for s in "wsb")
        out[wo:wo + q.packed.size] = q.packed.reshape(-1)
        out[so:so + q.scales.size * 2] = q.scales.reshape(-1).view(np.uint8)
        if q.bits != BITS_TERNARY:
            out[bo:bo + q.biases.size * 2] = q.biases.reshape(-1).view(np.uint8)


def quantize_group32_q2(w) -> QTensor:
    """2-bit affine quantization with a scale / bias entry per 32 weights, out of the group-64
    quantizer: every run of 32 is laid out twice in a row of twice the length, so each group of 64
    there has the run's own minimum and maximum; its table entry is the run's, its first 32 codes
    are the run's codes."""
    w = _c(w, np.float32)
    rows, n = w.shape
    runs = w.reshape(rows, n // 32, 32)
    q = quantize(np.concatenate([runs, runs], axis=2).reshape(rows, 2 * n), BITS_2)
    codes = ((q.packed[:, :, None] >> (2 * np.arange(4, dtype=np.uint8))) & 3).reshape(rows, n // 32, 64)
    packed = pack_codes(np.ascontiguousarray(codes[:, :, :32]).reshape(rows, n), BITS_2)
    return QTensor(packed, q.scales, q.biases, BITS_2, rows, n)


def synth_layer(root: int, d: int, f: int, e: int, k: int, bits: int = BITS_4, fs: int = 0,
                shared_bits: int = BITS_4, sigma: float = 0.02, router_mode: int = 0,
                swiglu_limit: float = 0.0, with_w_sg: bool = True, maple_rounding: bool = False,
                gate_group: int = GROUP) -> Layer:
    """Seeded synthetic layer: one SeedTree stream per tensor (labels "router",
    "shared.gate|up|down", "w_sg", "expert<i>.gate|up|down"), N(0, sigma)
    weights by Box-Muller, quantized per group of 64."""
    def nrm(label, rows, cols):
        return Rng.key(root, label).normal(0.0, sigma, rows * cols).reshape(rows, cols)

    router_w = bf16_bits(nrm("router", e, d))
    off, _, stride = blob_layout(d, f, bits, gate_group=gate_group)
    experts = np.zeros((e, stride), np.uint8)
    for i in range(e):
        if bits == BITS_TERNARY:
            qs = []
            for name, rows, cols in (("gate", f, d), ("up", f, d), ("down", d, f)):
                r = Rng.key(root, f"expert{i}.{name}")
                u = r.uniform_fill(0.0, 1.0, rows * cols).reshape(rows, cols)
                codes = np.where(u < 0.25, 0, np.where(u < 0.75, 1, 2)).astype(np.uint8)
                alpha = np.abs(r.normal(0.0, sigma, rows * (cols // GROUP))) + 1e-3
                qs.append(QTensor(pack_codes(codes, BITS_TERNARY),
                                  bf16_bits(alpha.reshape(rows, cols // GROUP)), None,
                                  BITS_TERNARY, rows, cols))
            pack_expert_blob(qs[0], qs[1], qs[2], off, experts[i])
        else:
            gate_w = nrm(f"expert{i}.gate", f, d)
            g = quantize_group32_q2(gate_w) if gate_group == 32 else quantize(gate_w, bits)
            u = quantize(nrm(f"expert{i}.up", f, d), bits)
            dn = quantize(nrm(f"expert{i}.down", d, f), bits)
            pack_expert_blob(g, u, dn, off, experts[i])
    shared = None
    w_sg = None
    if fs:
        shared = (quantize(nrm("shared.gate", fs, d), shared_bits),
                  quantize(nrm("shared.up", fs, d), shared_bits),
                  quantize(nrm("shared.down", d, fs), shared_bits))
        if with_w_sg:
            w_sg = bf16_bits(nrm("w_sg", 1, d).reshape(d))
    return Layer(d=d, f=f, e=e, k=k, bits=bits, router_w=router_w, experts=experts, off=off,
                 fs=fs, shared_bits=shared_bits, shared=shared, w_sg=w_sg,
                 router_mode=router_mode, swiglu_limit=swiglu_limit, maple_rounding=maple_rounding,
                 gate_group=gate_group)


def synth_x(root: int, t: int, d: int, label: str = "x") -> np.ndarray:
    return bf16_bits(Rng.key(root, label).normal(0.0, 1.0, t * d).reshape(t, d))
