"""Reader of the reference's packed_experts/ directory (layout.json + layer files)."""
import json
import os

import numpy as np
import pytest

from helpers import ROOT_SEED, write_packed_experts
from mference_amd import packed_experts as pe


def _toy_layout(directory):
    """the layout PackedExpertsLayoutTests.swift:10-72 writes: one layer, two experts, two
    sub-tensors each"""
    def expert(i, extra):
        e = dict(expert=i, offset=16384 * i, size=16384, tensors={
            "gate": dict(offset=0, size=4096, dtype="U32", shape=[64, 64], bits=4),
            "gate_scales": dict(offset=4096, size=256, dtype="BF16", shape=[64, 1])})
        e.update(extra)
        return e
    root = dict(expertStride=16384, numLayers=1, expertsPerLayer=2,
                layers=[dict(layer=0, file="layer_00.bin", experts=[expert(0, {}), expert(1, dict(physicalRank=1))])])
    os.makedirs(os.path.join(directory, "packed_experts"))
    with open(os.path.join(directory, "packed_experts", "layout.json"), "w") as fh:
        json.dump(root, fh, sort_keys=True)
    return root


def test_decodes_toy_layout(tmp_path):
    """PackedExpertsLayoutTests.swift:74-92 (decodesToyLayout), value for value"""
    _toy_layout(str(tmp_path))
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert layout.expert_stride == 16384 and layout.num_layers == 1 and layout.experts_per_layer == 2
    assert len(layout.layers) == 1
    e0 = layout.expert(0, 0)
    assert e0.offset == 0 and e0.size == 16384
    assert e0.sub_tensors["gate"].offset == 0 and e0.sub_tensors["gate_scales"].offset == 4096
    e1 = layout.expert(0, 1)
    assert e1.offset == 16384 and e1.expert == 1
    off = pe.routed_expert_offsets(layout, 0)       # ModelExpertIO.swift:20-35: missing roles read 0
    assert (off.gate_w, off.gate_s, off.gate_b, off.up_w, off.down_b) == (0, 4096, 0, 0, 0)
    assert pe.routed_expert_physical_offsets(layout, 0) == [0, 16384]


def test_missing_layout_json_is_missing_file(tmp_path):
    """PackedExpertsLayoutTests.swift:94-109"""
    os.makedirs(tmp_path / "packed_experts")
    with pytest.raises(pe.ModelError) as err:
        pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert err.value.kind == "missingFile"


def test_oversized_layout_rejected_before_decode(tmp_path):
    """PackedExpertsLayoutTests.swift:111-130: 64 bytes of blanks against a 16-byte cap"""
    _toy_layout(str(tmp_path))
    with open(tmp_path / "packed_experts" / "layout.json", "wb") as fh:
        fh.write(b" " * 64)
    with pytest.raises(pe.ModelError) as err:
        pe.PackedExpertsLayoutReader.load(str(tmp_path), max_bytes=16)
    assert err.value.kind == "indexCorrupt" and "metadata cap" in err.value.text


@pytest.mark.parametrize("mutate,needle", [
    (lambda r: r.pop("expertStride"), "missing top-level keys"),
    (lambda r: r["layers"][0].pop("file"), "malformed layer entry"),
    (lambda r: r["layers"][0]["experts"][0].pop("size"), "malformed expert entry"),
    (lambda r: r["layers"][0]["experts"][0]["tensors"]["gate"].pop("dtype"), "malformed tensor gate"),
    (lambda r: r["layers"][0]["experts"][0]["tensors"]["gate"].update(bits="4"), "malformed tensor bits gate"),
    (lambda r: r["layers"][0]["experts"][1].update(expert=2), "expert id out of range"),
    (lambda r: r["layers"][0]["experts"][1].update(physicalRank=5), "physicalRank out of range"),
    (lambda r: r["layers"][0]["experts"][1].update(expert=0), "missing expert entries"),
])
def test_malformed_layouts_are_index_corrupt(tmp_path, mutate, needle):
    """every guard of PackedExpertsLayoutReader.load (PackedExpertsLayout.swift:75-141)"""
    root = _toy_layout(str(tmp_path))
    mutate(root)
    with open(tmp_path / "packed_experts" / "layout.json", "w") as fh:
        json.dump(root, fh)
    with pytest.raises(pe.ModelError) as err:
        pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert err.value.kind == "indexCorrupt" and needle in err.value.text


def test_layer_without_experts_and_absent_ids(tmp_path):
    """a leading dense layer is an empty entry (PackedExpertsLayout.swift:87-91); experts without
    an id take the next free position (:123)"""
    root = _toy_layout(str(tmp_path))
    for e in root["layers"][0]["experts"]:
        e.pop("expert")
    root["layers"].insert(0, dict(layer=0, file="layer_00.bin", experts=[]))
    root["layers"][1]["layer"] = 1
    root["numLayers"] = 2
    with open(tmp_path / "packed_experts" / "layout.json", "w") as fh:
        json.dump(root, fh)
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert layout.layers[0].experts == [] and [e.expert for e in layout.layers[1].experts] == [0, 1]


@pytest.mark.parametrize("bits", [4, 2, 1])
def test_round_trip_of_a_synthetic_layer(tmp_path, oracle, bits):
    """a layer written in the reference's blob order comes back with the offsets the kernels use
    and, through the loader, byte for byte in logical expert order -- also when the file holds
    the blobs in another physical order"""
    d, f, e, k = 256, 128, 8, 4
    layer = oracle.synth_layer(ROOT_SEED + 0xB000 + bits, d, f, e, k, bits=bits)
    order = [3, 0, 7, 1, 6, 2, 5, 4]
    stride = write_packed_experts(str(tmp_path), layer, physical_order=order)
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert layout.expert_stride == stride and stride % 16384 == 0
    off = pe.routed_expert_offsets(layout, 0)
    for name, _ in layer.off._fields_:
        assert getattr(off, name) == getattr(layer.off, name), name
    assert pe.routed_expert_physical_offsets(layout, 0) == [order.index(i) * stride for i in range(e)]
    assert pe.routed_gate_group_size(layout, 0, f, d) == 64
    pool, got_stride = pe.load_layer_experts(str(tmp_path), layout, 0, device="cpu")
    assert got_stride == stride
    got = pool.numpy().reshape(e, stride)
    blob = layer.experts.shape[1]
    assert np.array_equal(got[:, :blob], layer.experts) and not got[:, blob:].any()


def test_gate_group_size_from_the_scale_slice(tmp_path, oracle):
    """ModelExpertIO.swift:118-135: a gate scale slice twice as large means group 32"""
    layer = oracle.synth_layer(ROOT_SEED + 0xB100, 256, 128, 4, 2, bits=4)
    write_packed_experts(str(tmp_path), layer)
    path = tmp_path / "packed_experts" / "layout.json"
    root = json.loads(path.read_text())
    for e in root["layers"][0]["experts"]:
        e["tensors"]["gate_scales"]["size"] *= 2
    path.write_text(json.dumps(root))
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert pe.routed_gate_group_size(layout, 0, 128, 256) == 32
    assert pe.routed_gate_group_size(layout, 0, 0, 256) == 64
    # a 4-bit gate at group 32 is refused before its file is read: group 32 goes with 2-bit codes only
    assert pe.gate_code_bits(layout, 0, 128, 256) == 4
    with pytest.raises(pe.ModelError, match="group 32") as err:
        pe.load_layer_experts(str(tmp_path), layout, 0, device="cpu", moe_intermediate=128, hidden=256)
    assert err.value.kind == "indexCorrupt"
    with pytest.raises(pe.ModelError):
        pe.require_supported_gate_group(layout, 0, 128, 256)
    assert pe.require_supported_gate_group(layout, 0, 0, 256) == 64   # unknown intermediate size: falls back to 64


def test_group32_gate_of_2bit_experts_is_accepted(tmp_path, oracle):
    """the DeepSeek conversion's layers: 2-bit codes, gate tables per 32 weights (ModelExpertIO.swift:118-135)"""
    d, f, e, k = 256, 128, 4, 2
    layer = oracle.synth_layer(ROOT_SEED + 0xB110, d, f, e, k, bits=2, gate_group=32)
    write_packed_experts(str(tmp_path), layer)
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    assert pe.routed_gate_group_size(layout, 0, f, d) == 32
    assert pe.gate_code_bits(layout, 0, f, d) == 2
    assert pe.require_supported_gate_group(layout, 0, f, d) == 32
    off = pe.routed_expert_offsets(layout, 0)
    for name, _ in layer.off._fields_:
        assert getattr(off, name) == getattr(layer.off, name), name
    pool, stride = pe.load_layer_experts(str(tmp_path), layout, 0, device="cpu", moe_intermediate=f, hidden=d)
    blob = layer.experts.shape[1]
    assert np.array_equal(pool.numpy().reshape(e, stride)[:, :blob], layer.experts)


def test_layer_file_checks(tmp_path, oracle):
    layer = oracle.synth_layer(ROOT_SEED + 0xB200, 256, 128, 4, 2, bits=4)
    write_packed_experts(str(tmp_path), layer)
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    path = tmp_path / "packed_experts" / "layer_00.bin"
    data = path.read_bytes()
    path.write_bytes(data[:-1])
    with pytest.raises(pe.ModelError) as err:
        pe.load_layer_experts(str(tmp_path), layout, 0, device="cpu")
    assert err.value.kind == "indexCorrupt"
    path.unlink()
    with pytest.raises(pe.ModelError) as err:
        pe.load_layer_experts(str(tmp_path), layout, 0, device="cpu")
    assert err.value.kind == "missingFile"


@pytest.mark.gpu
def test_loaded_layer_runs_like_the_directly_built_one(tmp_path, gpu, oracle):
    """packed_experts/ -> HBM pool -> decode layer: same bits as the layer uploaded directly"""
    import torch
    from mference_amd import operators as ops
    from helpers import assert_layer_close, make_moe, to_device_layer
    d, f, e, k, fs = 512, 256, 16, 4, 256
    layer = oracle.synth_layer(ROOT_SEED + 0xB300, d, f, e, k, bits=4, fs=fs)
    write_packed_experts(str(tmp_path), layer, physical_order=list(reversed(range(e))))
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    pool, stride = pe.load_layer_experts(str(tmp_path), layout, 0, device="cuda")
    direct = to_device_layer(layer)
    loaded = ops.MoELayerWeights(router_w=direct.router_w, experts=pool.view(e, stride),
                                 offsets=pe.routed_expert_offsets(layout, 0),
                                 shared=direct.shared, w_sg=direct.w_sg)
    moe = make_moe(gpu, layer)
    x_bits = oracle.synth_x(ROOT_SEED + 0xB300, 3, d)
    x = ops.bf16_tensor(x_bits)
    ref_y, ref_idx, _ = oracle.moe_layer(layer, x_bits)
    ys = []
    for wts in (direct, loaded):
        y = torch.zeros((3, d), dtype=torch.bfloat16, device="cuda")
        idx = torch.zeros((3, k), dtype=torch.int32, device="cuda")
        moe.encode_decode_layer(wts, x, y, t=3, out_indices=idx)
        moe.status()
        assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
        ys.append(ops.bf16_bits(y))
    assert np.array_equal(ys[0], ys[1])
    assert_layer_close(oracle.bf16_to_float(ys[1]), oracle.bf16_to_float(ref_y), "layer from packed_experts")


# ------------------------------------------------------- resident streamer (HBM pool behind the streamer calls)

def test_stream_layout_offsets():
    """StreamLayout.expertOffset (ExpertStreamer.swift:58-65): the explicit table for layer 0, else
    layer * experts * stride + expert * stride"""
    from mference_amd.resident_streamer import StreamLayout
    plain = StreamLayout("x", 0, 4 * 4096, 4, 4096)
    assert plain.expert_offset(0, 3) == 3 * 4096 and plain.expert_offset(2, 1) == 2 * 4 * 4096 + 4096
    table = StreamLayout("x", 0, 4 * 4096, 4, 4096, expert_offsets=[8192, 0, 12288, 4096])
    assert [table.expert_offset(0, e) for e in range(4)] == [8192, 0, 12288, 4096]
    assert table.expert_offset(1, 2) == 4 * 4096 + 2 * 4096   # the table covers layer 0 only
    assert table.expert_offset(0, 7) == 7 * 4096              # and only its own length


def test_resident_streamer_views_and_errors(tmp_path, oracle):
    from mference_amd import resident_streamer as rs
    layer = oracle.synth_layer(ROOT_SEED + 0xB400, 256, 128, 8, 4, bits=4)
    order = [5, 2, 7, 0, 1, 6, 3, 4]
    stride = write_packed_experts(str(tmp_path), layer, physical_order=order)
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    sl = rs.stream_layout_for_packed_layer(str(tmp_path), layout, 0)
    assert sl.stream_offset == 0 and sl.stream_size == 8 * stride and sl.expert_stride == stride
    st = rs.ResidentExpertStreamer(sl, device="cpu")
    st.warm_up()
    blob = layer.experts.shape[1]
    for e in range(8):
        buf, off, size = st.expert_buffer(0, e)
        assert off == 0 and size == stride
        assert np.array_equal(buf.numpy()[:blob], layer.experts[e])
    with pytest.raises(rs.StreamerError) as err:
        st.expert_buffer(0, 8)
    assert err.value.kind == "slotOutOfRange"
    with pytest.raises(rs.StreamerError) as err:
        rs.ResidentExpertStreamer(rs.StreamLayout(str(tmp_path / "nothing.bin"), 0, stride, 1, stride), device="cpu")
    assert err.value.kind == "openFailed"
    with pytest.raises(rs.StreamerError) as err:   # the file is shorter than offset + size
        rs.ResidentExpertStreamer(rs.StreamLayout(sl.path, stride, 8 * stride, 8, stride), device="cpu")
    assert err.value.kind == "sizeMismatch"
    with pytest.raises(rs.StreamerError) as err:   # an expert lies past the streamed range
        rs.ResidentExpertStreamer(rs.StreamLayout(sl.path, 0, 4 * stride, 8, stride), device="cpu")
    assert err.value.kind == "offsetOutOfRange"


@pytest.mark.gpu
def test_resident_streamer_pool_runs_a_layer(tmp_path, gpu, oracle):
    import torch
    from mference_amd import operators as ops
    from mference_amd import resident_streamer as rs
    from helpers import assert_layer_close, make_moe, to_device_layer
    d, f, e, k = 512, 256, 16, 4
    layer = oracle.synth_layer(ROOT_SEED + 0xB500, d, f, e, k, bits=2)
    write_packed_experts(str(tmp_path), layer, physical_order=[(3 * i) % e for i in range(e)])
    layout = pe.PackedExpertsLayoutReader.load(str(tmp_path))
    st = rs.ResidentExpertStreamer(rs.stream_layout_for_packed_layer(str(tmp_path), layout, 0), device="cuda")
    direct = to_device_layer(layer)
    wts = ops.MoELayerWeights(router_w=direct.router_w, experts=st.pool,
                              offsets=pe.routed_expert_offsets(layout, 0))
    x_bits = oracle.synth_x(ROOT_SEED + 0xB500, 2, d)
    ref_y, ref_idx, _ = oracle.moe_layer(layer, x_bits)
    y = torch.zeros((2, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((2, k), dtype=torch.int32, device="cuda")
    moe = make_moe(gpu, layer)
    moe.encode_decode_layer(wts, ops.bf16_tensor(x_bits), y, t=2, out_indices=idx)
    moe.status()
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), "layer from the streamer's pool")


def test_row_alpha_expansion(oracle):
    """RepackPlanner.swift:596-640 / SourceByteProvider.swift:369-393: every alpha repeated once per
    group of 64 inputs, the bias copy with the sign bit flipped"""
    alpha = oracle.bf16_bits(np.array([0.5, 0.0, 0.0123, 3.0], np.float32))
    scales, biases = pe.expand_row_alpha(alpha, 256)
    assert scales.shape == biases.shape == (4, 4) and scales.dtype == np.uint16
    assert np.array_equal(scales, np.tile(alpha[:, None], (1, 4)))
    assert np.array_equal(oracle.bf16_to_float(biases), -oracle.bf16_to_float(scales))
    assert biases[1, 0] == 0x8000  # -0.0: the sign bit is flipped, nothing is computed
    s3, _ = pe.expand_row_alpha(np.stack([alpha, alpha]), 128)
    assert s3.shape == (2, 4, 2)
    with pytest.raises(pe.ModelError):
        pe.expand_row_alpha(alpha, 96)
    with pytest.raises(pe.ModelError):
        pe.expand_row_alpha(alpha.astype(np.float32), 128)


@pytest.mark.gpu
def test_maple_layer_from_row_alpha(gpu, oracle):
    """A Maple layer whose experts come as codes + row_alpha: the blobs built by `maple_expert_blob`
    (scale and bias tables per group, the repacker's order) run to the result of the per-token oracle
    on the same weights written as scale-only ternary tables."""
    import torch
    from mference_amd import operators as ops
    from helpers import assert_layer_close
    d, f, e, k, t = 256, 128, 32, 8, 3
    rng = np.random.default_rng(ROOT_SEED + 0xB300)
    router_w = oracle.bf16_bits((rng.standard_normal((e, d)) * 0.02).astype(np.float32))
    off_o, _, stride_o = oracle.blob_layout(d, f, 1)
    experts_o = np.zeros((e, stride_o), np.uint8)
    blobs = []
    for ex in range(e):
        parts, q = [], []
        for rows, cols in ((f, d), (f, d), (d, f)):
            codes = rng.integers(0, 3, size=(rows, cols)).astype(np.uint8)
            alpha = oracle.bf16_bits((np.abs(rng.standard_normal(rows)) * 0.02 + 1e-3).astype(np.float32))
            packed = oracle.pack_codes(codes, 1)
            parts.append((packed, alpha))
            q.append(oracle.QTensor(packed, np.repeat(alpha[:, None], cols // 64, axis=1), None, 1, rows, cols))
        oracle.pack_expert_blob(q[0], q[1], q[2], off_o, experts_o[ex])
        blob, off, stride = pe.maple_expert_blob(*parts)
        blobs.append(blob)
    assert stride % 16384 == 0 and off.gate_b > off.gate_s > off.gate_w == 0
    layer = oracle.Layer(d=d, f=f, e=e, k=k, bits=1, router_w=router_w, experts=experts_o, off=off_o,
                         router_mode=1, maple_rounding=True)
    x = oracle.synth_x(ROOT_SEED + 0xB300, t, d)
    ref_y, ref_idx, _ = oracle.moe_layer(layer, x)
    moe = ops.MoE(gpu, d, f, e, k, bits=ops.BITS_TERNARY, router_mode=ops.ROUTER_FULL_SOFTMAX, maple_rounding=True)
    wts = ops.MoELayerWeights(ops.bf16_tensor(router_w), torch.from_numpy(np.stack(blobs)).cuda(), off)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    moe.encode_decode_layer(wts, ops.bf16_tensor(x), y, t=t, out_indices=idx)
    moe.status()
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), "maple from row_alpha")
