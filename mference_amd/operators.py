"""Host-side mirror of Mference's Swift operator surface over the C ABI.

Class and method names follow Sources/Mference/Kernels/** (Swift camelCase
turned into snake_case); a command buffer becomes a HIP stream, an
(MTLBuffer, offset) pair becomes a torch tensor (device memory only: torch is
the allocator and stream provider, every computation is libmfmoe's).
Argument errors raise MfError carrying the mf_status the C ABI returned.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

from . import _capi
from ._capi import (BITS_2, BITS_4, BITS_8, BITS_TERNARY, GROUP_SIZE, MAX_TOKENS, ROUTER_FULL_SOFTMAX,
                    ROUTER_TOPK_SOFTMAX, ExpertOffsets, MfError, check)

__all__ = [
    "MetalContext", "QuantizedTensor", "Quantization", "DequantInt4GEMV", "DequantInt4GEMVMultiX",
    "Elementwise", "FamilyRouters", "SharedExpertInt4", "MPPPrefillInt4QMM", "MoEExpertOffsets", "MoE", "MoELayerWeights",
    "PrefillMoEGrouping", "PrefillTokenExpertPair", "MfError", "BITS_2", "BITS_4", "BITS_TERNARY",
    "ROUTER_TOPK_SOFTMAX", "ROUTER_FULL_SOFTMAX", "bf16_tensor", "bf16_bits",
]

MoEExpertOffsets = ExpertOffsets


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("libmfmoe operates on device memory; got a CPU tensor")
    return t.data_ptr()


def _stream(stream) -> int:
    if stream is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def bf16_tensor(bits: np.ndarray, device="cuda") -> torch.Tensor:
    """uint16 bf16 bit patterns (host) -> torch.bfloat16 tensor on `device`."""
    a = np.ascontiguousarray(bits, dtype=np.uint16)
    return torch.from_numpy(a.view(np.int16)).to(device).view(torch.bfloat16)


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    """torch.bfloat16 tensor -> uint16 bit patterns on the host."""
    return t.detach().contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


class MetalContext:
    """Device + kernel state every operator is built from
    (Infrastructure/Metal/MetalContext.swift:45-65)."""

    def __init__(self, device: int = 0):
        self._h = C.c_void_p()
        check(_capi.lib().mf_ctx_create(device, C.byref(self._h)))
        self.device = torch.device("cuda", device)

    @property
    def handle(self):
        return self._h

    def close(self):
        if self._h:
            _capi.lib().mf_ctx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


@dataclass
class QuantizedTensor:
    """rows x n group-quantized tensor in device memory
    (Quantization.Int4AffineRow for every row, Quantization.swift:34-46)."""
    packed: torch.Tensor            # uint8 [rows, n*bits/8]
    scales: torch.Tensor            # bf16 [rows, n/64]
    biases: Optional[torch.Tensor]  # bf16 [rows, n/64]; None for ternary
    bits: int
    rows: int
    n: int

    def c(self) -> _capi.QTensor:
        return _capi.QTensor(_ptr(self.packed), _ptr(self.scales), _ptr(self.biases))

    @classmethod
    def from_host(cls, packed: np.ndarray, scales: np.ndarray, biases: Optional[np.ndarray],
                  bits: int, rows: int, n: int, device="cuda") -> "QuantizedTensor":
        return cls(torch.from_numpy(np.ascontiguousarray(packed)).to(device),
                   bf16_tensor(scales, device),
                   None if biases is None else bf16_tensor(biases, device), bits, rows, n)


class Quantization:
    """Infrastructure/ModelIO/Quantization.swift:3 on device."""
    group_size = GROUP_SIZE

    def __init__(self, context: MetalContext):
        self.context = context

    def quantize_affine(self, w: torch.Tensor, bits: int = BITS_4, stream=None) -> QuantizedTensor:
        """quantizeInt4Affine (Quantization.swift:50-102) for every row of w (fp32)."""
        if w.dtype != torch.float32 or w.dim() != 2:
            raise ValueError("w must be a 2-D float32 tensor")
        w = w.contiguous()
        rows, n = w.shape
        store = {BITS_8: 8, BITS_4: 4}.get(bits, 2)   # 8-bit: quantizeInt8Affine (Quantization.swift:135-176)
        packed = torch.empty((rows, n * store // 8), dtype=torch.uint8, device=w.device)
        scales = torch.empty((rows, n // GROUP_SIZE), dtype=torch.bfloat16, device=w.device)
        biases = torch.empty_like(scales)
        check(_capi.lib().mf_quantize_affine(self.context.handle, _stream(stream), _ptr(w), rows, n,
                                             bits, _ptr(packed), _ptr(scales), _ptr(biases)),
              self.context.handle)
        return QuantizedTensor(packed, scales, biases, bits, rows, n)

    def dequantize(self, q: QuantizedTensor, stream=None) -> torch.Tensor:
        """dequantizeInt4Affine (Quantization.swift:104-119): fp32 [rows, n]."""
        out = torch.empty((q.rows, q.n), dtype=torch.float32, device=q.packed.device)
        check(_capi.lib().mf_dequantize(self.context.handle, _stream(stream), q.c(), q.rows, q.n,
                                        q.bits, _ptr(out)), self.context.handle)
        return out


class DequantInt4GEMV:
    """Kernels/Quant/DequantInt4GEMV.swift:57-103 (any supported bit width)."""

    def __init__(self, context: MetalContext):
        self.context = context

    def encode(self, weights: QuantizedTensor, x: torch.Tensor, y: torch.Tensor, m: int, n: int,
               output_float32: bool = False, stream=None, t: int = 1) -> None:
        check(_capi.lib().mf_gemv(self.context.handle, _stream(stream), weights.c(), weights.bits,
                                  _ptr(x), _ptr(y), m, n, t, 1 if output_float32 else 0),
              self.context.handle)


class DequantInt4GEMVMultiX(DequantInt4GEMV):
    """Kernels/Quant/DequantInt4GEMVMultiX.swift:48-82: x [t, n], y [t, m], t <= 8."""
    max_tokens = MAX_TOKENS

    def encode(self, weights: QuantizedTensor, x: torch.Tensor, y: torch.Tensor, m: int, n: int,
               t: int, output_float32: bool = False, stream=None) -> None:
        super().encode(weights, x, y, m, n, output_float32, stream, t)


class MPPPrefillInt4QMM:
    """Kernels/TensorCore/MPPPrefillInt4QMM.swift:34-78: y[m, n] = x[m, k] . deq(W[n, k])^T for many
    rows.  `encode` returns the path taken, like the reference's `Path`."""
    tile_m, tile_n, tile_k = 64, 32, GROUP_SIZE

    def __init__(self, context: MetalContext):
        self.context = context
        self._ws = None

    def workspace_bytes(self, m: int, n: int, k: int) -> int:
        return int(_capi.lib().mf_qmm_workspace_bytes(m, n, k))

    def encode(self, weights: QuantizedTensor, x: torch.Tensor, y: torch.Tensor, m: int, n: int, k: int,
               workspace: Optional[torch.Tensor] = None, stream=None) -> str:
        if workspace is None:
            need = self.workspace_bytes(m, n, k)
            if self._ws is None or self._ws.numel() < need:
                self._ws = torch.empty(max(need, 256), dtype=torch.uint8, device=x.device)
            workspace = self._ws
        ws_bytes = workspace.numel() * workspace.element_size()
        # the reference's guard conditions (MPPPrefillInt4QMM.swift:43-55) give "unavailable"; a path that
        # ran is named for the kernel that ran it
        path = _capi.lib().mf_qmm_path(weights.c(), weights.bits, _ptr(x), _ptr(y), m, n, k, _ptr(workspace), ws_bytes)
        if path < 0:
            return "unavailable"
        check(_capi.lib().mf_qmm(self.context.handle, _stream(stream), weights.c(), weights.bits, _ptr(x), _ptr(y),
                                 m, n, k, 1 if y.dtype == torch.float32 else 0, _ptr(workspace), ws_bytes),
              self.context.handle)
        return self.PATHS[path]

    PATHS = {1: "affine-matrix-core-bf16", 2: "affine-rows-gemv"}


class Elementwise:
    """Kernels/Primitives/Elementwise.swift:60-87."""

    def __init__(self, context: MetalContext):
        self.context = context

    def encode_silu_mul(self, gate, up, out, count: int, stream=None):
        check(_capi.lib().mf_silu_mul(self.context.handle, _stream(stream), _ptr(gate), _ptr(up),
                                      _ptr(out), count), self.context.handle)

    def encode_sigmoid_scalar_mul(self, y, gate, count: int, rows: int = 1, stream=None):
        check(_capi.lib().mf_sigmoid_scalar_mul(self.context.handle, _stream(stream), _ptr(y),
                                                _ptr(gate), count, rows), self.context.handle)

    def encode_residual_add(self, hidden, delta, count: int, stream=None):
        check(_capi.lib().mf_residual_add(self.context.handle, _stream(stream), _ptr(hidden),
                                          _ptr(delta), count), self.context.handle)


class RMSNorm:
    """Kernels/Primitives/RMSNorm.swift:52-64 (`encodeBF16W`), with the residual add that
    precedes it in the runner folded into the same launch when `delta` is given."""

    def __init__(self, context: MetalContext):
        self.context = context

    def encode_bf16w(self, x, weight, out, d: int, eps: float, t: int = 1, delta=None, stream=None):
        """x [t, d] bf16 is the hidden state: updated in place by `delta` when given"""
        check(_capi.lib().mf_residual_rmsnorm(self.context.handle, _stream(stream), _ptr(x), _ptr(delta),
                                              _ptr(weight), _ptr(out), d, t, C.c_float(eps)),
              self.context.handle)


class SharedExpertInt4:
    """Kernels/MoE/SharedExpertInt4.swift:70-165 (also the dense SwiGLU MLP)."""

    def __init__(self, context: MetalContext):
        self.context = context

    def encode(self, x: torch.Tensor, gate: QuantizedTensor, up: QuantizedTensor,
               down: QuantizedTensor, y: torch.Tensor, scratch_act: torch.Tensor, t: int = 1,
               stream=None) -> None:
        if not (gate.rows == up.rows and gate.n == up.n and down.rows == gate.n
                and down.n == gate.rows):
            raise MfError(-2, f"gate=({gate.rows},{gate.n}) up=({up.rows},{up.n}) "
                              f"down=({down.rows},{down.n})")
        check(_capi.lib().mf_shared_expert(
            self.context.handle, _stream(stream), _ptr(x), gate.c(), up.c(), down.c(), gate.bits,
            gate.n, gate.rows, t, _ptr(y), _ptr(scratch_act),
            scratch_act.numel() * scratch_act.element_size()), self.context.handle)


    @staticmethod
    def scratch_bytes(d: int, f: int, t: int) -> int:
        """bytes of scratch the call can use for t rows (the matrix-core path from 32 rows on)"""
        return int(_capi.lib().mf_shared_expert_scratch_bytes(d, f, t))

    def encode_static(self, x: torch.Tensor, gate: QuantizedTensor, up: QuantizedTensor,
                      down: QuantizedTensor, y: torch.Tensor, t: int = 1, stream=None) -> None:
        """The same operator for callers that cannot allocate and bring no scratch: the
        activations go through the library's built-in device array (mf_shared_expert_static;
        t * f <= STATIC_ACT_ELEMS, calls on one GPU must not overlap)."""
        if not (gate.rows == up.rows and gate.n == up.n and down.rows == gate.n
                and down.n == gate.rows):
            raise MfError(-2, f"gate=({gate.rows},{gate.n}) up=({up.rows},{up.n}) "
                              f"down=({down.rows},{down.n})")
        check(_capi.lib().mf_shared_expert_static(
            self.context.handle, _stream(stream), _ptr(x), gate.c(), up.c(), down.c(), gate.bits,
            gate.n, gate.rows, t, _ptr(y)), self.context.handle)


class SharedExpertInt8:
    """Kernels/MoE/SharedExpertInt8.swift:78-181: the dense MLP on 8-bit affine tensors, GELU (tanh form) by
    default, SiLU with silu_activation (the reference's siluActivation)."""

    def __init__(self, context: MetalContext, silu_activation: bool = False):
        self.context = context
        self.silu_activation = silu_activation

    def encode(self, x: torch.Tensor, gate: QuantizedTensor, up: QuantizedTensor, down: QuantizedTensor,
               y: torch.Tensor, scratch_act: torch.Tensor, t: int = 1, stream=None) -> None:
        if not (gate.rows == up.rows and gate.n == up.n and down.rows == gate.n and down.n == gate.rows):
            raise MfError(-2, f"gate=({gate.rows},{gate.n}) up=({up.rows},{up.n}) down=({down.rows},{down.n})")
        check(_capi.lib().mf_shared_expert_int8(
            self.context.handle, _stream(stream), _ptr(x), gate.c(), up.c(), down.c(), gate.n, gate.rows, t,
            1 if self.silu_activation else 0, _ptr(y), _ptr(scratch_act),
            scratch_act.numel() * scratch_act.element_size()), self.context.handle)


class FamilyRouters:
    """The family-specific routers of the reference's operator classes, stand-alone: every call
    runs the router GEMV into the caller's fp32 `logits` buffer [t, rows] and then the selection.
    Routing weights are fp32 (the reference narrows them to fp16)."""

    def __init__(self, context: MetalContext):
        self.context = context

    def encode_router_top_k(self, weights, hidden, correction_bias, out_indices, out_weights,
                            num_experts: int, d: int, route_scale: float, logits, top_k: int = 6,
                            t: int = 1, x_stride: Optional[int] = None, stream=None):
        """MoEDeepseekV4.encodeRouterTopK (MoEDeepseekV4.swift:92-124): sqrtsoftplus selection."""
        check(_capi.lib().mf_router_sqrtsoftplus(
            self.context.handle, _stream(stream), _ptr(weights), _ptr(hidden), t,
            d if x_stride is None else x_stride, num_experts, d, top_k, _ptr(correction_bias),
            route_scale, _ptr(logits), _ptr(out_indices), _ptr(out_weights)), self.context.handle)

    def encode_router_hash_weights(self, weights, hidden, indices, out_weights, num_experts: int,
                                   d: int, route_scale: float, logits, top_k: int = 6, t: int = 1,
                                   x_stride: Optional[int] = None, stream=None):
        """MoEDeepseekV4.encodeRouterHashWeights (MoEDeepseekV4.swift:126-151)."""
        check(_capi.lib().mf_router_hash_weights(
            self.context.handle, _stream(stream), _ptr(weights), _ptr(hidden), t,
            d if x_stride is None else x_stride, num_experts, d, top_k, _ptr(indices), route_scale,
            _ptr(logits), _ptr(out_weights)), self.context.handle)

    def encode_router_inkling(self, weights, hidden, gate_bias, global_scale, out_indices,
                              out_weights, gammas_out, num_routed: int, num_shared: int, top_k: int,
                              route_scale: float, d: int, logits, t: int = 1,
                              x_stride: Optional[int] = None, stream=None):
        """InklingKernels.encodeRouter / encodeRouterPrefill (InklingKernels.swift:377-476)."""
        check(_capi.lib().mf_router_inkling(
            self.context.handle, _stream(stream), _ptr(weights), _ptr(hidden), t,
            d if x_stride is None else x_stride, num_routed, num_shared, d, top_k, _ptr(gate_bias),
            _ptr(global_scale), route_scale, _ptr(logits), _ptr(out_indices), _ptr(out_weights),
            _ptr(gammas_out)), self.context.handle)

    def encode_router_gemma4(self, weights, scales, biases, hidden, effective_scale,
                             per_expert_scale, out_indices, out_weights, num_experts: int, d: int,
                             top_k: int, logits, t: int = 1, x_stride: Optional[int] = None,
                             stream=None):
        """MoE.encodeRouterGemma4 (MoE.swift:153-202): 8-bit affine router rows."""
        check(_capi.lib().mf_router_gemma4(
            self.context.handle, _stream(stream), _ptr(weights), _ptr(scales), _ptr(biases),
            _ptr(hidden), t, d if x_stride is None else x_stride, _ptr(effective_scale),
            _ptr(per_expert_scale), num_experts, d, top_k, _ptr(logits), _ptr(out_indices),
            _ptr(out_weights)), self.context.handle)


def expert_blob_layout(d: int, f: int, bits: int = BITS_4, align: int = 256, repacked: bool = False):
    """(offsets, blob_bytes, stride) of one routed expert in the reference's blob order
    (RepackPlanner.swift:544-712, ModelExpertIO.swift:20-35): mf_expert_blob_layout, or with
    `repacked` mf_expert_blob_layout_repacked -- the byte layout of a packed_experts file, which for
    ternary experts also carries the negated-scale bias tables (RepackPlanner.swift:619-640)."""
    off = ExpertOffsets()
    blob, stride = C.c_size_t(0), C.c_size_t(0)
    fn = _capi.lib().mf_expert_blob_layout_repacked if repacked else _capi.lib().mf_expert_blob_layout
    check(fn(d, f, bits, align, C.byref(off), C.byref(blob), C.byref(stride)))
    return off, blob.value, stride.value


@dataclass
class MoELayerWeights:
    """Everything one MoE layer reads, resident in device memory."""
    router_w: torch.Tensor                 # bf16 [e, d]
    experts: torch.Tensor                  # uint8 [e, stride]
    offsets: ExpertOffsets
    shared: Optional[Sequence[QuantizedTensor]] = None  # gate, up, down
    w_sg: Optional[torch.Tensor] = None    # bf16 [d]
    w_sg_q8: Optional[QuantizedTensor] = None  # the scalar gate as an 8-bit affine row [1, d] (replaces w_sg)
    experts_tiled: Optional[torch.Tensor] = None  # uint8 [e, stride]: the pool in the prefill matmul's order (MoE.tile_experts)

    def c(self) -> _capi.LayerWeights:
        if self.experts.ndim != 2 or self.experts.stride(1) != 1:
            # a 1-D pool would make stride(0) one byte: every expert would read expert 0's bytes
            raise MfError(-1, "experts must be a [num_experts, stride] byte tensor")
        L = _capi.LayerWeights()
        L.router_w = _ptr(self.router_w)
        L.expert_base = _ptr(self.experts)
        L.expert_stride = self.experts.stride(0)
        L.offsets = self.offsets
        if self.shared is not None:
            L.shared_gate, L.shared_up, L.shared_down = (q.c() for q in self.shared)
        L.w_sg = _ptr(self.w_sg)
        if self.w_sg_q8 is not None:
            L.w_sg_q8 = self.w_sg_q8.c()
        if self.experts_tiled is not None:
            if self.experts_tiled.shape != self.experts.shape or self.experts_tiled.stride(0) != self.experts.stride(0):
                raise MfError(-1, "experts_tiled must have the pool's shape and stride")
            L.expert_tiled = _ptr(self.experts_tiled)
        return L


class MoE:
    """Router + routed experts operator: MoE (Kernels/MoE/MoE.swift),
    MoEDeepseekV4 (2-bit, top-6) and MapleMoE (ternary) in one class, selected
    by `bits`, `top_k` and `router_mode`."""

    def __init__(self, context: MetalContext, d: int, f: int, num_experts: int, top_k: int,
                 bits: int = BITS_4, router_mode: int = ROUTER_TOPK_SOFTMAX,
                 swiglu_limit: float = 0.0, shared_f: int = 0, shared_bits: int = BITS_4,
                 maple_rounding: bool = False, gate_group_size: int = 0):
        """gate_group_size 32: MoEDeepseekV4.encodeRoutedPhase1(gateGroupSize:) -- the routed gate
        projection's tables hold an entry per 32 weights (2-bit experts only)."""
        self.context = context
        self.cfg = _capi.MoEConfig(d, f, num_experts, top_k, bits, router_mode, swiglu_limit,
                                   shared_f, shared_bits, 1 if maple_rounding else 0, gate_group_size)
        self._h = C.c_void_p()
        check(_capi.lib().mf_moe_create(context.handle, C.byref(self.cfg), C.byref(self._h)),
              context.handle)

    def close(self):
        if self._h:
            _capi.lib().mf_moe_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def encode_decode_layer_normed(self, weights: MoELayerWeights, hidden, norm_weight, y, t: int = 1, delta=None,
                                   eps: float = 1e-6, out_indices=None, out_weights=None, stream=None):
        """hidden += delta, x = RMSNorm(hidden) * norm_weight, y = layer(x), hidden += y: one launch where the
        fused launch takes the layer (RealForwardRunner.swift:2799-2808 and the layer behind it)."""
        lw = weights.c()
        check(_capi.lib().mf_moe_decode_layer_normed(self._h, _stream(stream), C.byref(lw), _ptr(hidden), _ptr(delta),
                                                     _ptr(norm_weight), eps, t, _ptr(y), _ptr(out_indices),
                                                     _ptr(out_weights)), self.context.handle)

    def set_fused(self, enabled) -> None:
        """single fused launch (True / 1, default) or the chain of separate launches (False / 0); 2: the fused
        launch through the instance that reads every dimension from its arguments"""
        check(_capi.lib().mf_moe_set_fused(self._h, int(enabled)), self.context.handle)

    def tile_experts(self, experts: torch.Tensor, offsets: ExpertOffsets, stream=None) -> torch.Tensor:
        """a copy of the expert pool [e, stride] in the prefill matmul's own order (mf_moe_tile_experts): pass it
        as MoELayerWeights.experts_tiled"""
        out = torch.empty_like(experts)
        check(_capi.lib().mf_moe_tile_experts(self._h, _stream(stream), _ptr(experts), experts.stride(0),
                                              C.byref(offsets), _ptr(out)), self.context.handle)
        return out

    def set_prefill_route_rounding(self, narrow: bool) -> None:
        """per-route down results of the prefill layer narrowed to bf16 before their routing weights (True: the
        reference's prefill rule, prefill.metal:817-819) or kept in fp32 as the decode step keeps them (False)"""
        check(_capi.lib().mf_moe_set_prefill_route_rounding(self._h, 1 if narrow else 0), self.context.handle)

    def set_phase_trace(self, buffer: Optional[torch.Tensor]) -> None:
        """int64 device tensor of num_cu*8 entries receiving per-workgroup stage
        timestamps of the fused launch (100 MHz clock); None switches it off"""
        check(_capi.lib().mf_moe_set_phase_trace(
            self._h, _ptr(buffer), 0 if buffer is None else buffer.numel() * 8),
            self.context.handle)

    def status(self, stream=None) -> None:
        """synchronises and raises if a fused launch gave up on a grid barrier"""
        check(_capi.lib().mf_moe_status(self._h, _stream(stream)), self.context.handle)

    def encode_router(self, router_w, x, out_indices, out_weights, t: int = 1,
                      x_stride: Optional[int] = None, out_logits=None, stream=None):
        """encodeRouterGemma4 (MoE.swift:153-203) / encodeRouterTopK / encodeRouterTop8."""
        check(_capi.lib().mf_moe_router(self._h, _stream(stream), _ptr(router_w), _ptr(x), t,
                                        self.cfg.d if x_stride is None else x_stride,
                                        _ptr(out_indices), _ptr(out_weights), _ptr(out_logits)),
              self.context.handle)

    def encode_routed_phase1(self, experts: torch.Tensor, offsets: ExpertOffsets, indices, x, acts,
                             t: int = 1, x_stride: Optional[int] = None, stream=None):
        """encodeRoutedPersistentPhase1U16Load (MoE.swift:220-253)."""
        check(_capi.lib().mf_moe_phase1(self._h, _stream(stream), _ptr(experts), experts.stride(0),
                                        C.byref(offsets), _ptr(indices), _ptr(x), t,
                                        self.cfg.d if x_stride is None else x_stride, _ptr(acts)),
              self.context.handle)

    def encode_routed_phase1_subset(self, experts: torch.Tensor, offsets: ExpertOffsets, indices, x, acts,
                                    active_slots, active_count: int, t: int = 1,
                                    x_stride: Optional[int] = None, stream=None):
        """encodeRoutedPersistentPhase1SubsetU16Load (MoE.swift:255-298): only the listed slots."""
        check(_capi.lib().mf_moe_phase1_subset(self._h, _stream(stream), _ptr(experts), experts.stride(0),
                                               C.byref(offsets), _ptr(indices), _ptr(x), t,
                                               self.cfg.d if x_stride is None else x_stride, _ptr(acts),
                                               _ptr(active_slots), active_count),
              self.context.handle)

    def encode_routed_phase2_reduce(self, experts: torch.Tensor, offsets: ExpertOffsets, indices,
                                    routing_weights, acts, residual, y, t: int = 1, stream=None):
        """encodeRoutedPersistentPhase2Reduce (MoE.swift:400-440)."""
        check(_capi.lib().mf_moe_phase2(self._h, _stream(stream), _ptr(experts), experts.stride(0),
                                        C.byref(offsets), _ptr(indices), _ptr(routing_weights),
                                        _ptr(acts), _ptr(residual), t, _ptr(y)),
              self.context.handle)

    def encode_slot_lookup(self, indices, slot_of, slot_stride: int, out_slot_offsets, out_all_hit,
                           t: int = 1, stream=None):
        """router_slot_lookup_k8 (moe.metal:594-617): slot byte offsets of the routed experts from the
        caller's expert -> slot table (int16, negative = not resident), and the all-hit word."""
        check(_capi.lib().mf_moe_slot_lookup(self._h, _stream(stream), _ptr(indices), t, _ptr(slot_of),
                                             slot_stride, _ptr(out_slot_offsets), _ptr(out_all_hit)),
              self.context.handle)

    def encode_routed_phase1_slots(self, slab, slot_offsets, offsets: ExpertOffsets, x, acts, t: int = 1,
                                   all_hit=None, stream=None):
        """Phase 1 over slots named directly (MoE.swift:205-253 with `slab=None` and a table of device
        addresses; MoE.swift:333-407 with a slab and byte offsets, guarded by `all_hit`)."""
        check(_capi.lib().mf_moe_phase1_slots(self._h, _stream(stream), _ptr(slab), _ptr(slot_offsets),
                                              _ptr(all_hit), C.byref(offsets), _ptr(x), t, x.stride(0) if x.dim() > 1 else self.cfg.d,
                                              _ptr(acts)), self.context.handle)

    def encode_routed_phase2_reduce_slots(self, slab, slot_offsets, offsets: ExpertOffsets, routing_weights,
                                          acts, residual, y, t: int = 1, all_hit=None, stream=None):
        """Phase 2 + rank-ordered reduce over slots named directly (MoE.swift:409-440, 333-407)."""
        check(_capi.lib().mf_moe_phase2_slots(self._h, _stream(stream), _ptr(slab), _ptr(slot_offsets),
                                              _ptr(all_hit), C.byref(offsets), _ptr(routing_weights),
                                              _ptr(acts), _ptr(residual), t, _ptr(y)), self.context.handle)

    def encode_decode_layer(self, weights: MoELayerWeights, x, y, t: int = 1, hidden=None,
                            out_indices=None, out_weights=None, stream=None):
        """The fused decode layer (router -> experts -> shared add), one call."""
        lw = weights.c()
        check(_capi.lib().mf_moe_decode_layer(self._h, _stream(stream), C.byref(lw), _ptr(x), t,
                                              _ptr(y), _ptr(hidden), _ptr(out_indices),
                                              _ptr(out_weights)), self.context.handle)

    def encode_group(self, indices, routing_weights, t: int, sorted_pairs, expert_offsets,
                     expert_counts, stream=None):
        """PrefillRouter.makeTokenExpertPairs + PrefillMoEGrouping.groupTokenExpertPairs
        (PrefillRouter.swift:91-111, PrefillMoEGrouping.swift:91-192) on device.
        sorted_pairs: int32/uint8 device tensor of t*top_k 16-byte records."""
        check(_capi.lib().mf_moe_group(self._h, _stream(stream), _ptr(indices),
                                       _ptr(routing_weights), t, _ptr(sorted_pairs),
                                       _ptr(expert_offsets), _ptr(expert_counts)),
              self.context.handle)

    def group_status(self, stream=None) -> None:
        """synchronises; raises MfError(expert out of range) if the last
        encode_group saw an index >= num_experts"""
        check(_capi.lib().mf_moe_group_status(self._h, _stream(stream)), self.context.handle)

    def prefill_workspace_bytes(self, t: int) -> int:
        return int(_capi.lib().mf_moe_prefill_workspace_bytes(self._h, t))

    def encode_prefill_layer(self, weights: MoELayerWeights, x, y, t: int, workspace=None,
                             out_indices=None, out_weights=None, stream=None):
        """Ragged prefill layer over t tokens (PrefillGroupedRoutedMoE.encodeStreamedBatched,
        PrefillGroupedRoutedMoE.swift:392-466, + reduce + shared expert).  `workspace`: uint8
        device tensor of at least prefill_workspace_bytes(t); allocated when None."""
        need = self.prefill_workspace_bytes(t)  # 0 for formats that take the decode launch
        if workspace is None:
            workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=x.device)
        lw = weights.c()
        check(_capi.lib().mf_moe_prefill_layer(self._h, _stream(stream), C.byref(lw), _ptr(x), t,
                                               _ptr(y), _ptr(workspace), workspace.numel(),
                                               _ptr(out_indices), _ptr(out_weights)),
              self.context.handle)
        return workspace


    def encode_streamed_batched(self, experts: torch.Tensor, offsets: ExpertOffsets, hidden, sorted_pairs,
                                expert_counts, route_partials, t: int, workspace=None, stream=None):
        """PrefillGroupedRoutedMoE.encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:392-466): the
        routed experts over a grouping the caller holds (encode_group's sorted pairs and counts).
        route_partials: float32 [t * top_k, d], row token * top_k + rank.  A grouping that fails the
        device check computes nothing and group_status() raises."""
        if experts.dim() != 2:
            raise ValueError("experts must be a 2-D uint8 pool [num_experts, blob_stride]")
        if workspace is None:
            workspace = torch.empty(max(self.prefill_workspace_bytes(t), 16), dtype=torch.uint8,
                                    device=hidden.device)
        check(_capi.lib().mf_moe_ragged_qmm(self._h, _stream(stream), _ptr(experts), experts.stride(0),
                                            C.byref(offsets), _ptr(hidden), _ptr(sorted_pairs),
                                            _ptr(expert_counts), t, _ptr(route_partials),
                                            _ptr(workspace), workspace.numel()), self.context.handle)
        return workspace

    def encode_reduce_token_major(self, route_partials, route_weights, h2, t: int, indices=None,
                                  residual=None, stream=None):
        """PrefillMoE.encodeReduceTokenMajor (PrefillMoE.swift:11-38): h2[token] = sum over ranks of
        route_weights[token, rank] * route_partials[token * top_k + rank] (+ residual), bf16."""
        check(_capi.lib().mf_moe_unpermute(self._h, _stream(stream), _ptr(route_partials),
                                           _ptr(route_weights), _ptr(indices), _ptr(residual), t,
                                           _ptr(h2)), self.context.handle)


PAIR_DTYPE = np.dtype([("token", "<u4"), ("expert", "<u4"), ("rank", "<u4"),
                       ("weight_bits", "<u4")])
GROUP_DTYPE = np.dtype([("expert", "<u4"), ("pair_start", "<u4"), ("pair_count", "<u4")])
TILE_DTYPE = np.dtype([("group_start", "<u4"), ("group_count", "<u4"), ("pair_start", "<u4"),
                       ("pair_count", "<u4")])


def PrefillTokenExpertPair(token: int, expert: int, rank: int, weight_bits: int):
    """One route record (Kernels/Prefill/MoE/PrefillRouter.swift:4-28)."""
    return (token, expert, rank, weight_bits)


@dataclass
class PrefillMoEGroupedRoutes:
    """Kernels/Prefill/MoE/PrefillMoEGrouping.swift:32-50."""
    sorted_pairs: np.ndarray
    per_expert_offsets: np.ndarray
    per_expert_counts: np.ndarray
    groups: np.ndarray
    tiles: np.ndarray
    query_count: int

    @property
    def max_pairs_per_expert(self) -> int:
        return int(self.groups["pair_count"].max()) if self.groups.size else 0

    @property
    def max_pairs_per_tile(self) -> int:
        return int(self.tiles["pair_count"].max()) if self.tiles.size else 0

    @property
    def max_live_experts_per_tile(self) -> int:
        return int(self.tiles["group_count"].max()) if self.tiles.size else 0


class PrefillMoEGrouping:
    """Kernels/Prefill/MoE/PrefillMoEGrouping.swift:90-192 (host, integer)."""

    @staticmethod
    def make_token_expert_pairs(indices: np.ndarray, weight_bits: np.ndarray, query_count: int,
                                top_k: int) -> np.ndarray:
        """PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:91-111)."""
        indices = np.asarray(indices, np.uint32).reshape(-1)
        weight_bits = np.asarray(weight_bits, np.uint32).reshape(-1)
        if indices.size != query_count * top_k or weight_bits.size != query_count * top_k:
            raise ValueError("indices / weights count mismatch")
        out = np.empty(query_count * top_k, PAIR_DTYPE)
        out["token"] = np.repeat(np.arange(query_count, dtype=np.uint32), top_k)
        out["rank"] = np.tile(np.arange(top_k, dtype=np.uint32), query_count)
        out["expert"] = indices
        out["weight_bits"] = weight_bits
        return out

    @staticmethod
    def group_token_expert_pairs(pairs, query_count: int, top_k: int, num_experts: int,
                                 tile_expert_count: int = 16,
                                 expert_sort_keys=None) -> PrefillMoEGroupedRoutes:
        if isinstance(pairs, np.ndarray) and pairs.dtype == PAIR_DTYPE:
            p = np.ascontiguousarray(pairs)
        else:
            p = np.array([tuple(x) for x in pairs], dtype=PAIR_DTYPE)
        n = p.size
        sorted_ = np.empty(n, PAIR_DTYPE)
        ne = max(num_experts, 1)
        offsets = np.empty(ne, np.uint32)
        counts = np.empty(ne, np.uint32)
        cap = max(min(ne, n), 1)
        groups = np.empty(cap, GROUP_DTYPE)
        tiles = np.empty(cap, TILE_DTYPE)
        ng, nt = C.c_size_t(0), C.c_size_t(0)
        keys = None if expert_sort_keys is None else np.ascontiguousarray(expert_sort_keys, np.uint64)
        detail = (C.c_uint32 * 2)()
        vp = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
        rc = _capi.lib().mf_group_pairs_host(
            vp(p), n, query_count, top_k, num_experts, tile_expert_count, vp(keys),
            0 if keys is None else keys.size, vp(sorted_), vp(offsets), vp(counts), vp(groups),
            C.byref(ng), vp(tiles), C.byref(nt), C.cast(detail, C.c_void_p))
        if rc != 0:
            err = MfError(rc, f"detail={detail[0]},{detail[1]}")
            err.detail = (int(detail[0]), int(detail[1]))
            raise err
        return PrefillMoEGroupedRoutes(sorted_, offsets[:num_experts], counts[:num_experts],
                                       groups[:ng.value], tiles[:nt.value], query_count)
