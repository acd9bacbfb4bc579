"""CPU-side checks of the C ABI: libmfmoe.so loads, exports every symbol that
include/mfmoe.h declares, rejects bad arguments without launching, and its host
grouping twin reproduces the reference's integer KATs.  No GPU, no compute."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from mference_amd import _capi
from mference_amd import operators as ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mfmoe.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mf_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(_capi.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in mfmoe.h but not exported"
    # and the ctypes table covers the same set
    assert sorted(_capi.SIGNATURES) == names


def test_every_entry_point_cites_the_reference():
    text = open(HEADER).read()
    for name in declared_symbols():
        pos = text.index(name + "(")
        comment = text[:pos].rsplit("/*", 1)[-1]
        assert ".swift" in comment or ".metal" in comment or "No counterpart" in comment \
            or "no counterpart" in comment or name in ("mf_ctx_destroy", "mf_status_string",
                                                       "mf_last_hip_error", "mf_abi_version",
                                                       "mf_moe_destroy", "mf_ctx_num_cu"), name


def test_status_strings_and_bad_arguments():
    lib = _capi.lib()
    assert lib.mf_abi_version() >= 1
    assert lib.mf_status_string(0) == b"ok"
    assert b"tileExpertCount" in lib.mf_status_string(-13)
    q = _capi.QTensor(None, None, None)
    # null context / null pointers: invalid argument, nothing launched
    assert lib.mf_gemv(None, None, q, 4, None, None, 8, 64, 1, 0) == -1
    assert lib.mf_dequantize(None, None, q, 1, 64, 4, None) == -1
    assert lib.mf_moe_router(None, None, None, None, 1, 64, None, None, None) == -1
    h = C.c_void_p()
    assert lib.mf_moe_create(None, None, C.byref(h)) == -1
    with pytest.raises(ops.MfError) as ei:
        _capi.check(-2)
    assert ei.value.name == "MF_ERR_DIMENSION_MISMATCH"


def test_operator_shapes_are_checked_without_a_device():
    """mf_moe_config_check: what mf_moe_create refuses, as a status (MoE.swift:165-167 traps instead).  The
    full-softmax router ranks 32 experts per lane step, so an expert count that is no multiple of 32 is refused
    in that mode -- the GPU tie tests skip exactly those parameters -- and accepted in the top-k softmax mode."""
    lib = _capi.lib()

    def status(**kw):
        base = dict(d=256, f=128, num_experts=64, top_k=8, bits=4, router_mode=0, swiglu_limit=0.0, shared_f=0,
                    shared_bits=4, maple_rounding=0, gate_group_size=0)
        base.update(kw)
        return lib.mf_moe_config_check(C.byref(_capi.MoEConfig(**base)))

    assert status() == 0
    assert lib.mf_moe_config_check(None) == -1
    for e in (8, 16, 24, 33, 100, 168, 255):          # RouterTopKParityTests.swift:34 expert counts
        assert status(num_experts=e, router_mode=0) == 0
        assert status(num_experts=e, router_mode=1) == (0 if e % 32 == 0 else -1), e
    for e in (32, 64, 128, 256):
        assert status(num_experts=e, router_mode=1) == 0
    assert status(d=100) == -2 and status(f=96) == -2 and status(shared_f=100) == -2
    assert status(bits=3) == -3 and status(shared_f=64, shared_bits=8) == -3
    assert status(num_experts=0) == -1 and status(num_experts=513) == -1
    assert status(top_k=0) == -1 and status(top_k=9) == -1
    assert status(router_mode=2) == -1 and status(maple_rounding=2) == -1
    assert status(gate_group_size=32, bits=4) == -1 and status(gate_group_size=32, bits=2) == 0
    assert status(gate_group_size=16, bits=2) == -1


KAT_PAIRS = [(0, 3, 0, 10), (0, 1, 1, 11), (0, 4, 2, 12), (1, 1, 0, 13), (1, 3, 1, 14), (1, 2, 2, 15),
             (2, 4, 0, 16), (2, 3, 1, 17), (2, 1, 2, 18), (3, 5, 0, 19), (3, 1, 1, 20), (3, 4, 2, 21)]
G = ops.PrefillMoEGrouping


def test_grouping_kat_through_the_library():
    # PrefillMoEGroupingTests.swift:5-53
    g = G.group_token_expert_pairs(KAT_PAIRS[::-1], 4, 3, 6, tile_expert_count=2)
    assert list(g.sorted_pairs["expert"]) == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert list(g.per_expert_offsets) == [0xFFFFFFFF, 0, 4, 5, 8, 11]
    assert list(g.per_expert_counts) == [0, 4, 1, 3, 3, 1]
    assert [tuple(x) for x in g.groups] == [(1, 0, 4), (2, 4, 1), (3, 5, 3), (4, 8, 3), (5, 11, 1)]
    assert [tuple(x) for x in g.tiles] == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]
    assert (g.max_pairs_per_expert, g.max_pairs_per_tile, g.max_live_experts_per_tile) == (4, 6, 2)


def test_grouping_errors_carry_the_reference_payloads():
    # PrefillMoEGroupingTests.swift:117-173
    cases = [
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=1, tile=17), "MF_ERR_TILE_EXPERT_COUNT", None),
        (dict(pairs=[(0, 2, 0, 1)], q=1, k=1, e=2, tile=1), "MF_ERR_EXPERT_RANGE", (2, 0)),
        (dict(pairs=[(0, 0, 0, 1), (0, 1, 0, 2)], q=1, k=2, e=2, tile=1),
         "MF_ERR_DUPLICATE_TOKEN_RANK", (0, 0)),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=2, tile=1, keys=[0]), "MF_ERR_SORT_KEY_COUNT", (2, 1)),
        (dict(pairs=[(0, 0, 0, 1)], q=2, k=1, e=2, tile=1), "MF_ERR_PAIR_COUNT", (2, 1)),
        (dict(pairs=[(5, 0, 0, 1)], q=1, k=1, e=2, tile=1), "MF_ERR_TOKEN_RANGE", (5, 0)),
        (dict(pairs=[(0, 0, 3, 1)], q=1, k=1, e=2, tile=1), "MF_ERR_RANK_RANGE", (3, 0)),
        (dict(pairs=[], q=-1, k=1, e=2, tile=1), "MF_ERR_QUERY_COUNT", None),
        (dict(pairs=[], q=0, k=0, e=2, tile=1), "MF_ERR_TOPK", None),
        (dict(pairs=[], q=0, k=1, e=0, tile=1), "MF_ERR_NUM_EXPERTS", None),
    ]
    for c, name, detail in cases:
        with pytest.raises(ops.MfError) as ei:
            G.group_token_expert_pairs(c["pairs"], c["q"], c["k"], c["e"], c["tile"], c.get("keys"))
        assert ei.value.name == name
        if detail is not None:
            assert ei.value.detail == detail


def test_grouping_matches_the_oracle_on_random_routes(oracle):
    rng = np.random.default_rng(5)
    for t, k, e, tile in [(1, 8, 256, 16), (32, 8, 128, 16), (128, 6, 64, 3), (0, 2, 4, 1)]:
        idx = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.uint32) if t else \
            np.zeros((0, k), np.uint32)
        wb = rng.integers(0, 2 ** 32, size=(t, k), dtype=np.uint32)
        pairs = G.make_token_expert_pairs(idx, wb, t, k)
        assert np.array_equal(pairs, oracle.make_pairs(idx, wb)) if t else pairs.size == 0
        shuffled = pairs[rng.permutation(pairs.size)]
        g = G.group_token_expert_pairs(shuffled, t, k, e, tile)
        ref = oracle.group_pairs(shuffled, t, k, e, tile)
        assert np.array_equal(g.sorted_pairs, ref["sorted"])
        assert np.array_equal(g.per_expert_offsets, ref["offsets"][:e])
        assert np.array_equal(g.per_expert_counts, ref["counts"][:e])
        assert np.array_equal(g.groups, ref["groups"]) and np.array_equal(g.tiles, ref["tiles"])


def _c_layout(tmp_path):
    """sizeof / offsetof of every struct in include/mfmoe.h, printed by a gcc-built probe."""
    import subprocess
    structs = {
        "mf_expert_offsets": ["gate_w", "gate_s", "gate_b", "up_w", "up_s", "up_b",
                              "down_w", "down_s", "down_b"],
        "mf_qtensor": ["weights", "scales", "biases"],
        "mf_pair": ["token", "expert", "rank", "weight_bits"],
        "mf_moe_config": ["d", "f", "num_experts", "top_k", "bits", "router_mode", "swiglu_limit",
                          "shared_f", "shared_bits", "maple_rounding", "gate_group_size"],
        "mf_moe_layer_weights": ["router_w", "expert_base", "expert_stride", "offsets",
                                 "shared_gate", "shared_up", "shared_down", "w_sg", "w_sg_q8", "expert_tiled"],
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "mfmoe.h"', 'int main(void){']
    for s, fields in structs.items():
        lines.append(f'printf("{s} size %zu\\n", sizeof({s}));')
        for f in fields:
            lines.append(f'printf("{s} {f} %zu\\n", offsetof({s}, {f}));')
    lines.append('return 0;}')
    src = tmp_path / "layout_probe.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout_probe"
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    table = {}
    for line in out.splitlines():
        s, f, v = line.split()
        table[(s, f)] = int(v)
    return structs, table


def test_struct_layouts_of_header_and_ctypes_mirror_agree(tmp_path):
    """The header compiles as plain C, and the ctypes structures the Python host side passes
    have the sizes and field offsets the C compiler gives the header's.  The route record keeps
    the reference's pinned layout: 16 bytes, stride 16, token / expert / rank / weight bits at
    0 / 4 / 8 / 12 (PrefillRouterTests.swift:12-19); the offset table is nine uint32
    (MoEExpertOffsets, Kernels/MoE/MoE.swift:4-29)."""
    structs, table = _c_layout(tmp_path)
    mirror = {"mf_expert_offsets": _capi.ExpertOffsets, "mf_qtensor": _capi.QTensor,
              "mf_pair": _capi.Pair, "mf_moe_config": _capi.MoEConfig,
              "mf_moe_layer_weights": _capi.LayerWeights}
    for s, fields in structs.items():
        cls = mirror[s]
        assert C.sizeof(cls) == table[(s, "size")], s
        assert [n for n, _ in cls._fields_] == fields, s
        for f in fields:
            assert getattr(cls, f).offset == table[(s, f)], (s, f)
    assert table[("mf_pair", "size")] == 16
    assert [table[("mf_pair", f)] for f in ("token", "expert", "rank", "weight_bits")] == [0, 4, 8, 12]
    assert table[("mf_expert_offsets", "size")] == 36
    assert [table[("mf_expert_offsets", f)] for f in structs["mf_expert_offsets"]] == list(range(0, 36, 4))
    pairs = (_capi.Pair * 3)()
    assert C.addressof(pairs[1]) - C.addressof(pairs[0]) == 16


@pytest.mark.parametrize("d,f,bits", [(2048, 512, 4), (4096, 2048, 2), (2048, 1024, 1), (128, 64, 4)])
def test_expert_blob_layout_matches_checker(d, f, bits):
    """mf_expert_blob_layout (the product's own helper) against the checker's restatement of the
    repacker's blob order; the Qwen expert is 1 769 472 bytes = 108 pages of 16 KiB exactly."""
    from mference_amd import operators as ops
    from oracle import mf_oracle as O
    off, blob, stride = ops.expert_blob_layout(d, f, bits, 16384)
    ref_off, ref_blob, ref_stride = O.blob_layout(d, f, bits, 16384)
    for name, _ in off._fields_:
        assert getattr(off, name) == getattr(ref_off, name), name
    assert (blob, stride) == (ref_blob, ref_stride)
    if (d, f, bits) == (2048, 512, 4):
        assert blob == 1769472 == 108 * 16384 == stride
    lib = _capi.lib()
    o = _capi.ExpertOffsets()
    assert lib.mf_expert_blob_layout(100, 64, 4, 256, C.byref(o), None, None) == -2
    assert lib.mf_expert_blob_layout(128, 64, 3, 256, C.byref(o), None, None) == -3
    assert lib.mf_expert_blob_layout(128, 64, 4, 0, C.byref(o), None, None) == -1
    assert lib.mf_expert_blob_layout(128, 64, 4, 256, None, None, None) == -1


@pytest.mark.parametrize("d,f", [(2048, 1024), (2048, 512), (256, 128)])
def test_repacked_ternary_layout_is_the_file_layout(d, f):
    """mf_expert_blob_layout_repacked against the blob a Maple packed_experts file holds (codes, scales and
    the negated-scale bias tables of all three projections, RepackPlanner.swift:544-651), as
    packed_experts.maple_expert_blob builds it from source tensors; 4-bit and 2-bit experts: both helpers agree."""
    from mference_amd import packed_experts as pe
    rng = np.random.default_rng(d + f)
    mk = lambda rows, width: (rng.integers(0, 256, size=(rows, width // 4), dtype=np.uint8),
                              rng.integers(0x3C00, 0x3E00, size=rows).astype(np.uint16))
    blob, off_file, stride_file = pe.maple_expert_blob(mk(f, d), mk(f, d), mk(d, f), align=16384)
    off, blob_bytes, stride = ops.expert_blob_layout(d, f, ops.BITS_TERNARY, 16384, repacked=True)
    for name, _ in off._fields_:
        assert getattr(off, name) == getattr(off_file, name), name
    assert stride == stride_file == blob.size
    assert blob_bytes == 3 * (d * f // 4) + 2 * 2 * (2 * f * (d // 64) + d * (f // 64))
    compact = ops.expert_blob_layout(d, f, ops.BITS_TERNARY, 16384)
    assert compact[1] < blob_bytes and compact[0].gate_b == 0
    for bits in (ops.BITS_4, ops.BITS_2):
        a, b = ops.expert_blob_layout(d, f, bits, 16384), ops.expert_blob_layout(d, f, bits, 16384, repacked=True)
        assert (a[1], a[2]) == (b[1], b[2])
        assert all(getattr(a[0], n) == getattr(b[0], n) for n, _ in a[0]._fields_)
