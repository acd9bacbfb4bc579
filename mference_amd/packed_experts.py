"""Reader of the reference's `packed_experts/` directory: `layout.json` plus one
`layer_XX.bin` per MoE layer, every routed expert one contiguous blob
(gate, gate_scales, gate_biases, up, ..., down_biases) at a fixed stride.

Mirrors `PackedExpertsLayoutReader.load`
(Sources/Mference/Infrastructure/ModelIO/PackedExpertsLayout.swift:46-157: same keys, same
checks, same error cases), `Model.routedExpertOffsets` / `routedExpertPhysicalOffsets`
(Sources/Mference/Runtime/Inference/ModelExpertIO.swift:20-39) and `routedGateGroupSize`
(ModelExpertIO.swift:118-135), and loads a layer file straight into the resident HBM expert
pool the operators address as `expert_base + expert * stride`.

The group-32 gate projection of the DeepSeek conversion is detected (`routed_gate_group_size`) and,
for 2-bit codes, accepted (`require_supported_gate_group` returns the group to hand to
`MoE(gate_group_size=...)`); other groupings are refused.  Maple's per-row alpha tables: see
`expand_row_alpha`.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Dict, List, Optional

DEFAULT_MAX_BYTES = 64 * 1024 * 1024   # PackedExpertsLayout.swift:49
GROUP_SIZE = 64                        # Quantization.groupSize


class ModelError(Exception):
    """ModelTypes.swift:795-800: `missingFile(name)` and `indexCorrupt(detail)`."""

    def __init__(self, kind: str, text: str):
        super().__init__(f"{kind}: {text}")
        self.kind = kind
        self.text = text

    @classmethod
    def missing_file(cls, name: str) -> "ModelError":
        return cls("missingFile", name)

    @classmethod
    def index_corrupt(cls, detail: str) -> "ModelError":
        return cls("indexCorrupt", detail)


@dataclass(frozen=True)
class SubTensorEntry:          # PackedExpertsLayout.swift:3-6
    offset: int                # relative to the expert blob's start
    size: int                  # bytes; scale slices encode the group count


@dataclass(frozen=True)
class ExpertEntry:             # PackedExpertsLayout.swift:8-28
    expert: int                # logical routed-expert id
    offset: int                # absolute byte offset of the blob inside its layer file
    size: int                  # bytes of the blob (== expert_stride)
    sub_tensors: Dict[str, SubTensorEntry]


@dataclass(frozen=True)
class LayerLayout:             # PackedExpertsLayout.swift:30-34
    layer: int
    file: str                  # basename, e.g. "layer_00.bin"
    experts: List[ExpertEntry]


@dataclass(frozen=True)
class PackedExpertsLayout:     # PackedExpertsLayout.swift:36-46
    expert_stride: int
    num_layers: int
    experts_per_layer: int
    layers: List[LayerLayout]

    def expert(self, layer: int, expert: int) -> ExpertEntry:
        return self.layers[layer].experts[expert]


# ---- layout.json as a schema: a kind per field, one checker for every level of the document.
# The reference walks the document with a guard per level (PackedExpertsLayout.swift:75-141); the
# error a level reports when any of its fields has the wrong kind is that level's `what`.

def _is_int(v) -> bool:
    return isinstance(v, int) and not isinstance(v, bool)


def _as_uint(v) -> Optional[int]:
    """NSNumber.uint64Value of a JSON number: integers, and floats holding one"""
    if _is_int(v) and v >= 0:
        return v
    if isinstance(v, float) and v >= 0 and v == int(v):
        return int(v)
    return None


_KINDS = {
    "uint": _as_uint,
    "int": lambda v: v if _is_int(v) else None,
    "str": lambda v: v if isinstance(v, str) else None,
    "objects": lambda v: v if isinstance(v, list) and all(isinstance(x, dict) for x in v) else None,
    "object_map": lambda v: v if isinstance(v, dict) and all(isinstance(x, dict) for x in v.values()) else None,
    "ints": lambda v: v if isinstance(v, list) and all(_is_int(x) for x in v) else None,
}
_TOP = (("expertStride", "uint"), ("numLayers", "int"), ("expertsPerLayer", "int"), ("layers", "objects"))
_LAYER = (("layer", "int"), ("file", "str"), ("experts", "objects"))
_EXPERT = (("offset", "uint"), ("size", "uint"), ("tensors", "object_map"))
_TENSOR = (("offset", "uint"), ("size", "uint"), ("dtype", "str"), ("shape", "ints"))


def _take(obj, schema, what: str) -> list:
    """The schema's fields of `obj`, each converted by its kind; `what` names the level in the error."""
    out = []
    for key, kind in schema:
        v = _KINDS[kind](obj.get(key)) if isinstance(obj, dict) else None
        if v is None:
            raise ModelError.index_corrupt(f"layout.json: {what}")
        out.append(v)
    return out


def _optional_int(obj, key) -> Optional[int]:
    v = obj.get(key)
    return v if _is_int(v) else None


def _sub_tensors(tensors: dict) -> Dict[str, SubTensorEntry]:
    subs: Dict[str, SubTensorEntry] = {}
    for role, t in tensors.items():
        off, size, _, _ = _take(t, _TENSOR, f"malformed tensor {role}")
        if "bits" in t and not _is_int(t["bits"]):
            raise ModelError.index_corrupt(f"layout.json: malformed tensor bits {role}")
        subs[role] = SubTensorEntry(off, size)
    return subs


def _layer_experts(entries: list, per_layer: int) -> List[ExpertEntry]:
    """The experts of one layer by LOGICAL id; an entry without an id takes the next free position in
    file order; every id of the layer has to be there."""
    by_id: Dict[int, ExpertEntry] = {}
    for obj in entries:
        off, size, tensors = _take(obj, _EXPERT, "malformed expert entry")
        subs = _sub_tensors(tensors)
        expert_id = _optional_int(obj, "expert")
        if expert_id is None:
            expert_id = len(by_id)
        if not 0 <= expert_id < per_layer:
            raise ModelError.index_corrupt("layout.json: expert id out of range")
        rank = _optional_int(obj, "physicalRank")
        if rank is not None and not 0 <= rank < per_layer:
            raise ModelError.index_corrupt("layout.json: physicalRank out of range")
        by_id[expert_id] = ExpertEntry(expert_id, off, size, subs)
    if len(by_id) != per_layer:
        raise ModelError.index_corrupt("layout.json: missing expert entries")
    return [by_id[i] for i in range(per_layer)]


class PackedExpertsLayoutReader:
    """`PackedExpertsLayoutReader.load(directoryURL:maxBytes:)`"""

    default_max_bytes = DEFAULT_MAX_BYTES

    @staticmethod
    def load(directory: str, max_bytes: int = DEFAULT_MAX_BYTES) -> PackedExpertsLayout:
        path = os.path.join(directory, "packed_experts", "layout.json")
        if not os.path.isfile(path):
            raise ModelError.missing_file("packed_experts/layout.json")
        size = os.path.getsize(path)
        if size > max_bytes:   # checked before anything is decoded
            raise ModelError.index_corrupt(f"layout.json size {size} exceeds metadata cap {max_bytes}")
        try:
            with open(path, "rb") as fh:
                root = json.loads(fh.read().decode("utf-8"))
        except (ValueError, UnicodeDecodeError) as exc:
            raise ModelError.index_corrupt(f"layout.json: {exc}") from None
        stride, n_layers, per_layer, layer_objs = _take(root, _TOP, "missing top-level keys")
        layers: List[LayerLayout] = []
        for obj in layer_objs:
            index, file, entries = _take(obj, _LAYER, "malformed layer entry")
            # a leading dense-FFN layer is an entry without experts and without a blob file
            layers.append(LayerLayout(index, file, _layer_experts(entries, per_layer) if entries else []))
        return PackedExpertsLayout(stride, n_layers, per_layer, layers)


_ROLES = ("gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases",
          "down", "down_scales", "down_biases")


def routed_expert_offsets(layout: PackedExpertsLayout, layer: int):
    """`Model.routedExpertOffsets(layer:)`: the nine sub-tensor offsets of expert 0 of the layer
    (a missing role reads as 0), as the operators' MoEExpertOffsets."""
    from .operators import MoEExpertOffsets
    subs = layout.expert(layer, 0).sub_tensors
    vals = [subs[r].offset if r in subs else 0 for r in _ROLES]
    off = MoEExpertOffsets()
    for (name, _), v in zip(off._fields_, vals):
        setattr(off, name, v)
    return off


def routed_expert_physical_offsets(layout: PackedExpertsLayout, layer: int) -> List[int]:
    """`Model.routedExpertPhysicalOffsets(layer:)`"""
    return [e.offset for e in layout.layers[layer].experts]


def routed_gate_group_size(layout: PackedExpertsLayout, layer: int, moe_intermediate: int, hidden: int) -> int:
    """`Model.routedGateGroupSize(layer:)`: the gate projection's quantization group, from the
    byte size of its scale slice (bf16 entries, one per row and group)."""
    scales = layout.expert(layer, 0).sub_tensors.get("gate_scales")
    if scales is None or moe_intermediate <= 0:
        return GROUP_SIZE
    groups = scales.size // (2 * moe_intermediate)
    if groups <= 0 or hidden % groups:
        return GROUP_SIZE
    return hidden // groups


def gate_code_bits(layout: PackedExpertsLayout, layer: int, moe_intermediate: int, hidden: int) -> int:
    """Bits per weight of the gate projection's packed codes, from the byte size of its slice
    (0 when the slice or the shape is unknown)."""
    gate = layout.expert(layer, 0).sub_tensors.get("gate")
    if gate is None or moe_intermediate <= 0 or hidden <= 0:
        return 0
    return gate.size * 8 // (moe_intermediate * hidden)


def require_supported_gate_group(layout: PackedExpertsLayout, layer: int, moe_intermediate: int, hidden: int) -> int:
    """The layer's gate quantization group, for `MoE(gate_group_size=...)`: 64, or 32 with 2-bit codes
    (the DeepSeek conversion's gate_proj, ModelExpertIO.swift:122-135, which the operators run on their
    chain of launches).  Any other combination raises: the operators would compute wrong activations
    from such a blob without noticing."""
    g = routed_gate_group_size(layout, layer, moe_intermediate, hidden)
    if g == GROUP_SIZE:
        return g
    bits = gate_code_bits(layout, layer, moe_intermediate, hidden)
    if g == 32 and bits == 2:
        return g
    raise ModelError.index_corrupt(
        f"layer {layer}: gate projection uses quantization group {g} with {bits}-bit codes; "
        f"the resident operators take group {GROUP_SIZE}, or group 32 with 2-bit codes")


def load_layer_experts(directory: str, layout: PackedExpertsLayout, layer: int, device="cuda",
                       moe_intermediate: Optional[int] = None, hidden: Optional[int] = None):
    """Read `packed_experts/<layer file>` into one resident uint8 tensor of
    experts_per_layer * expert_stride bytes in LOGICAL expert order (the operators address
    expert e at e * stride; the file may hold the blobs in any physical order).  Returns
    (tensor, stride).  The read goes through a pinned staging buffer in chunks, so a 453 MB
    layer never needs a second full copy in host memory.  With `moe_intermediate` and `hidden`
    given, a layer whose gate projection's quantization group the operators do not take is refused
    (`require_supported_gate_group`) before anything is read."""
    import numpy as np
    import torch

    entry = layout.layers[layer]
    if not entry.experts:
        raise ModelError.index_corrupt(f"layer {layer} has no routed experts")
    if moe_intermediate is not None and hidden is not None:
        require_supported_gate_group(layout, layer, moe_intermediate, hidden)
    path = os.path.join(directory, "packed_experts", entry.file)
    if not os.path.isfile(path):
        raise ModelError.missing_file(entry.file)
    stride, n = layout.expert_stride, layout.experts_per_layer
    file_size = os.path.getsize(path)
    for e in entry.experts:
        if e.size > stride or e.offset + e.size > file_size:
            raise ModelError.index_corrupt(f"{entry.file}: expert {e.expert} lies outside the file")
    pool = torch.empty((n * stride,), dtype=torch.uint8, device=device)
    src = np.memmap(path, dtype=np.uint8, mode="r")
    in_order = all(e.offset == i * stride and e.size == stride for i, e in enumerate(entry.experts))
    chunk = max(stride, 64 << 20) // stride * stride
    use_pin = torch.device(device).type == "cuda"
    stage = torch.empty((chunk,), dtype=torch.uint8, pin_memory=use_pin)
    stage_np = stage.numpy()
    if in_order:
        for pos in range(0, n * stride, chunk):
            m = min(chunk, n * stride - pos)
            stage_np[:m] = src[pos:pos + m]
            pool[pos:pos + m].copy_(stage[:m], non_blocking=False)
    else:
        per = chunk // stride
        for e0 in range(0, n, per):
            cnt = min(per, n - e0)
            stage_np[:cnt * stride] = 0
            for j in range(cnt):
                e = entry.experts[e0 + j]
                stage_np[j * stride:j * stride + e.size] = src[e.offset:e.offset + e.size]
            pool[e0 * stride:(e0 + cnt) * stride].copy_(stage[:cnt * stride], non_blocking=False)
    del src
    return pool, stride


# ---- Maple's routed tensors: per-row alpha instead of per-group tables

def expand_row_alpha(row_alpha, input_width: int):
    """A Maple routed tensor ships 2-bit codes {0, 1, 2} and ONE bf16 `row_alpha` per output row;
    the expert blob the kernels read holds a scale and a bias entry per row and group of 64 inputs.
    The reference's repacker makes them by repeating every alpha input_width / 64 times, the bias
    copy with the sign bit flipped (RepackPlanner.swift:596-640, the `.repeatBF16(count:negated:)`
    transform of SourceByteProvider.swift:369-393): weight = (q - 1) * alpha.
    row_alpha: uint16 bf16 bit patterns, shape [rows] (or [experts, rows]).  Returns
    (scales, biases), uint16 arrays of shape [..., rows, input_width // 64]."""
    import numpy as np
    a = np.asarray(row_alpha)
    if a.dtype != np.uint16:
        raise ModelError.index_corrupt(f"row_alpha must be bf16 bit patterns (uint16), got {a.dtype}")
    if input_width <= 0 or input_width % GROUP_SIZE:
        raise ModelError.index_corrupt(f"row_alpha: input width {input_width} is no positive multiple of {GROUP_SIZE}")
    reps = input_width // GROUP_SIZE
    scales = np.repeat(a[..., None], reps, axis=-1)
    return scales, scales ^ np.uint16(0x8000)


def maple_expert_blob(gate, up, down, align: int = 16384):
    """One routed expert's blob from Maple source tensors, in the repacker's order
    gate {codes, scales, biases}, up {...}, down {...} (RepackPlanner.swift:544-651).
    Each of gate / up / down is (packed 2-bit codes uint8 [rows, input / 4], row_alpha uint16 [rows]).
    Returns (blob uint8 [stride], MoEExpertOffsets, stride); the ternary operators read the codes and
    the scale tables (their bias is -scale by construction; the bias tables are carried for
    byte-compatibility with the reference's layout)."""
    import numpy as np
    from .operators import MoEExpertOffsets
    off = MoEExpertOffsets()
    chunks = []
    pos = 0
    for role, (codes, alpha) in (("gate", gate), ("up", up), ("down", down)):
        codes = np.ascontiguousarray(codes, dtype=np.uint8)
        rows, row_bytes = codes.shape
        width = row_bytes * 4
        alpha = np.asarray(alpha)
        if alpha.shape != (rows,):
            raise ModelError.index_corrupt(
                f"{role}: row_alpha shape {alpha.shape} does not match the {rows} output rows")
        scales, biases = expand_row_alpha(alpha, width)
        for suffix, arr in (("w", codes), ("s", scales), ("b", biases)):
            setattr(off, f"{role}_{suffix}", pos)
            raw = np.ascontiguousarray(arr).reshape(-1).view(np.uint8)
            chunks.append(raw)
            pos += raw.size
    stride = (pos + align - 1) // align * align
    blob = np.zeros(stride, np.uint8)
    blob[:pos] = np.concatenate(chunks)
    return blob, off, stride
