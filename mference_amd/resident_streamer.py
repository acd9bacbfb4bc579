"""All-resident routed-expert backend on HBM: the counterpart of the reference's
`ResidentExpertStreamer` (Sources/Mference/Infrastructure/Streaming/ResidentExpertStreamer.swift:10-116),
which maps a layer file and wraps every expert blob in a buffer of its own so that the existing
runners address experts as (buffer, offset, size).  Here the streamed region of the layer file is
read once into one device tensor and every expert is a view into it; the operators need no view
per expert at all -- they take `pool` as `expert_base` and `layout.expert_stride` as stride -- but
`expert_buffer` keeps the reference's call for code written against it.

Same layout type (`StreamLayout`, ExpertStreamer.swift:36-66) and the same error cases
(`StreamerError`, ExpertStreamer.swift:3-12) as far as they can occur without a slot cache.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import List, Optional, Tuple


class StreamerError(Exception):
    """ExpertStreamer.swift:3-31; `kind` is the case name"""

    def __init__(self, kind: str, text: str):
        super().__init__(text)
        self.kind = kind

    @classmethod
    def open_failed(cls, path: str, errno_: int) -> "StreamerError":
        return cls("openFailed", f"open({path}) failed: errno {errno_}")

    @classmethod
    def size_mismatch(cls, expected: int, actual: int) -> "StreamerError":
        return cls("sizeMismatch", f"file size mismatch: expected {expected}, got {actual}")

    @classmethod
    def offset_out_of_range(cls, offset: int) -> "StreamerError":
        return cls("offsetOutOfRange", f"offset {offset} is outside the streamed range")

    @classmethod
    def slot_out_of_range(cls, slot: int) -> "StreamerError":
        return cls("slotOutOfRange", f"expert cache slot {slot} is out of range")


@dataclass(frozen=True)
class StreamLayout:
    """ExpertStreamer.swift:36-66: where the routed experts of a layer file are."""
    path: str
    stream_offset: int
    stream_size: int
    experts_per_layer: int
    expert_stride: int
    expert_offsets: Optional[List[int]] = None   # physical offsets of layer 0's experts, logical order

    def expert_offset(self, layer: int, expert: int) -> int:
        if layer == 0 and self.expert_offsets is not None and 0 <= expert < len(self.expert_offsets):
            return self.expert_offsets[expert]
        return layer * self.experts_per_layer * self.expert_stride + expert * self.expert_stride


class ResidentExpertStreamer:
    """`ResidentExpertStreamer(layout:device:)`: the whole streamed region resident, one copy."""

    def __init__(self, layout: StreamLayout, device="cuda"):
        import numpy as np
        import torch

        self.layout = layout
        try:
            fd = os.open(layout.path, os.O_RDONLY)
        except OSError as exc:
            raise StreamerError.open_failed(layout.path, exc.errno or 0) from None
        try:
            required = layout.stream_offset + layout.stream_size
            actual = os.fstat(fd).st_size
            if actual < required:
                raise StreamerError.size_mismatch(required, actual)
            for expert in range(layout.experts_per_layer):
                region = layout.expert_offset(0, expert)
                if region + layout.expert_stride > layout.stream_size:
                    raise StreamerError.offset_out_of_range(region)
        finally:
            os.close(fd)
        stride, n = layout.expert_stride, layout.experts_per_layer
        # experts land in LOGICAL order at expert * stride, whatever order the file holds them in:
        # the kernels index the pool by expert id
        self.pool = torch.empty((n, stride), dtype=torch.uint8, device=device)
        src = np.memmap(layout.path, dtype=np.uint8, mode="r", offset=layout.stream_offset,
                        shape=(layout.stream_size,))
        per = max(1, (64 << 20) // max(stride, 1))
        use_pin = torch.device(device).type == "cuda"
        stage = torch.empty((per, stride), dtype=torch.uint8, pin_memory=use_pin)
        stage_np = stage.numpy()
        for e0 in range(0, n, per):
            cnt = min(per, n - e0)
            for j in range(cnt):
                at = layout.expert_offset(0, e0 + j)
                stage_np[j] = src[at:at + stride]
            self.pool[e0:e0 + cnt].copy_(stage[:cnt], non_blocking=False)
        del src

    def expert_buffer(self, layer: int, expert: int) -> Tuple["object", int, int]:
        """(buffer, offset, size) of one expert (`expertBuffer(layer:expert:)`): the buffer is the
        expert's row of the pool, the offset inside it 0."""
        if layer != 0:  # the pool holds the one layer of the file the layout names
            raise StreamerError.offset_out_of_range(layer)
        if not 0 <= expert < self.layout.experts_per_layer:
            raise StreamerError.slot_out_of_range(expert)
        return self.pool[expert], 0, self.layout.expert_stride

    def warm_up(self) -> None:
        """`warmUp()`: the reference touches its mapping page by page; the pool is already in HBM"""
        return None


def stream_layout_for_packed_layer(directory: str, layout, layer: int) -> StreamLayout:
    """StreamLayout of one layer of a packed_experts directory (the reference builds it from
    PackedExpertsLayout in Model.ensureLayerOpened; one file per layer, so the stream starts at 0
    and `layer` inside the streamer is always 0)."""
    entry = layout.layers[layer]
    path = os.path.join(directory, "packed_experts", entry.file)
    offsets = [e.offset for e in entry.experts]
    size = max((o + layout.expert_stride for o in offsets), default=0)
    return StreamLayout(path=path, stream_offset=0, stream_size=size,
                        experts_per_layer=layout.experts_per_layer, expert_stride=layout.expert_stride,
                        expert_offsets=offsets)
