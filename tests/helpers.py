"""Shared helpers of the parity tests: move oracle-side layers to the device and
compare outputs under the layer tolerance."""
from __future__ import annotations

import numpy as np
import torch

from mference_amd import operators as ops

ROOT_SEED = 0x4D464D4F00000000  # seeds: ROOT_SEED + 0x100 * config + layer

# layer-output tolerance of the parity contract: fp32 accumulation, bf16 outputs
MAX_ABS = 2e-2
REL_L2 = 1e-3


def to_device_q(q, device="cuda") -> ops.QuantizedTensor:
    """oracle QTensor (host numpy) -> device QuantizedTensor"""
    return ops.QuantizedTensor.from_host(q.packed, q.scales, q.biases, q.bits, q.rows, q.n, device)


def to_device_layer(layer, device="cuda") -> ops.MoELayerWeights:
    off = ops.MoEExpertOffsets()
    for name, _ in off._fields_:
        setattr(off, name, getattr(layer.off, name))
    shared = None if layer.shared is None else [to_device_q(q, device) for q in layer.shared]
    return ops.MoELayerWeights(
        router_w=ops.bf16_tensor(layer.router_w, device),
        experts=torch.from_numpy(layer.experts).to(device),
        offsets=off, shared=shared,
        w_sg=None if layer.w_sg is None else ops.bf16_tensor(layer.w_sg, device))


def make_moe(ctx, layer) -> ops.MoE:
    return ops.MoE(ctx, layer.d, layer.f, layer.e, layer.k, bits=layer.bits,
                   router_mode=layer.router_mode, swiglu_limit=layer.swiglu_limit,
                   shared_f=layer.fs, shared_bits=layer.shared_bits)


def errors(actual: np.ndarray, ref: np.ndarray):
    a = actual.astype(np.float64).reshape(-1)
    r = ref.astype(np.float64).reshape(-1)
    max_abs = float(np.max(np.abs(a - r))) if a.size else 0.0
    rel_l2 = float(np.linalg.norm(a - r) / max(np.linalg.norm(r), 1e-30))
    return max_abs, rel_l2


def assert_layer_close(actual: np.ndarray, ref: np.ndarray, what: str = ""):
    max_abs, rel_l2 = errors(actual, ref)
    assert max_abs <= MAX_ABS and rel_l2 <= REL_L2, (
        f"{what}: max_abs={max_abs:.3e} (<= {MAX_ABS}), rel_l2={rel_l2:.3e} (<= {REL_L2})")
