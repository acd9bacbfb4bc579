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
        w_sg=None if layer.w_sg is None else ops.bf16_tensor(layer.w_sg, device),
        w_sg_q8=None if getattr(layer, "w_sg_q8", None) is None else to_device_q(layer.w_sg_q8, device))


def make_moe(ctx, layer) -> ops.MoE:
    return ops.MoE(ctx, layer.d, layer.f, layer.e, layer.k, bits=layer.bits,
                   router_mode=layer.router_mode, swiglu_limit=layer.swiglu_limit,
                   shared_f=layer.fs, shared_bits=layer.shared_bits,
                   maple_rounding=getattr(layer, "maple_rounding", False),
                   gate_group_size=getattr(layer, "gate_group", 64))


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


def write_packed_experts(directory, layer, physical_order=None, page=16384):
    """Write `layer` (an oracle Layer) as the reference's packed_experts/ directory: layout.json
    and layer_00.bin, every expert one blob at a stride rounded up to `page`
    (RepackPlanner.swift:544-712); `physical_order[rank]` = logical expert stored at that rank."""
    import json
    import os
    import numpy as np
    d, f, e, bits = layer.d, layer.f, layer.e, layer.bits
    blob = layer.experts.shape[1]
    stride = (blob + page - 1) // page * page
    order = list(range(e)) if physical_order is None else list(physical_order)
    rank_of = {ex: r for r, ex in enumerate(order)}
    pack_bits = 2 if bits == 1 else bits
    gu_w, gu_s = f * d * pack_bits // 8, f * (d // 64) * 2
    dn_w, dn_s = d * f * pack_bits // 8, d * (f // 64) * 2
    gg = getattr(layer, "gate_group", 64)
    g_s = f * (d // gg) * 2
    off = layer.off
    tensors = {
        "gate": dict(offset=off.gate_w, size=gu_w, dtype="U32", shape=[f, d * pack_bits // 32], bits=pack_bits),
        "gate_scales": dict(offset=off.gate_s, size=g_s, dtype="BF16", shape=[f, d // gg]),
        "up": dict(offset=off.up_w, size=gu_w, dtype="U32", shape=[f, d * pack_bits // 32], bits=pack_bits),
        "up_scales": dict(offset=off.up_s, size=gu_s, dtype="BF16", shape=[f, d // 64]),
        "down": dict(offset=off.down_w, size=dn_w, dtype="U32", shape=[d, f * pack_bits // 32], bits=pack_bits),
        "down_scales": dict(offset=off.down_s, size=dn_s, dtype="BF16", shape=[d, f // 64]),
    }
    if bits != 1:
        tensors["gate_biases"] = dict(offset=off.gate_b, size=g_s, dtype="BF16", shape=[f, d // gg])
        tensors["up_biases"] = dict(offset=off.up_b, size=gu_s, dtype="BF16", shape=[f, d // 64])
        tensors["down_biases"] = dict(offset=off.down_b, size=dn_s, dtype="BF16", shape=[d, f // 64])
    experts = [dict(expert=ex, physicalRank=rank_of[ex], offset=rank_of[ex] * stride, size=stride,
                    tensors=tensors) for ex in range(e)]
    root = dict(expertStride=stride, numLayers=1, expertsPerLayer=e,
                layers=[dict(layer=0, file="layer_00.bin", experts=experts)])
    pe = os.path.join(directory, "packed_experts")
    os.makedirs(pe, exist_ok=True)
    with open(os.path.join(pe, "layout.json"), "w") as fh:
        json.dump(root, fh, sort_keys=True)
    data = np.zeros((e, stride), np.uint8)
    for r, ex in enumerate(order):
        data[r, :blob] = layer.experts[ex]
    data.tofile(os.path.join(pe, "layer_00.bin"))
    return stride
