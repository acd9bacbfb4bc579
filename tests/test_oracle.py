"""Pins the CPU oracle (oracle/) against what the reference's own tests hold for
this path and against what the mathematics fixes.  No GPU.

Each block names the reference test it follows (paths relative to the Mference
repository root).  None of these checks re-types the oracle's formula: they are
published constants, literal integer KATs, invariants, or an independent fp64
numpy composition.
"""
import ctypes as C
import math

import numpy as np
import pytest
import torch

from oracle import mf_oracle as O


# ------------------------------------------------------------------ generators

def test_splitmix64_published_vectors():
    # first outputs of the public-domain splitmix64.c for seeds 0 and 1234567
    r = O.Rng(0)
    assert [r.next() for _ in range(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4,
                                            0x06C45D188009454F]
    r = O.Rng(1234567)
    assert [r.next() for _ in range(3)] == [6457827717110365317, 3203168211198807973,
                                            9817491932198370423]


def test_seed_tree_is_fnv1a64_of_label():
    # published FNV-1a 64 test vectors: "" , "a", "foobar"
    for label, h in (("", 0xCBF29CE484222325), ("a", 0xAF63DC4C8601EC8C),
                     ("foobar", 0x85944171F73967E8)):
        root = 0x1234_5678_9ABC_DEF0
        assert O.Rng.key(root, label).next() == O.Rng(root ^ h).next()


def test_uniform_is_24_bit_and_in_range():
    r, r2 = O.Rng(42), O.Rng(42)
    for _ in range(100):
        u = r.uniform(-1.0, 3.0)
        bits = r2.next() >> 40
        assert u == np.float32(-1.0) + np.float32(4.0) * (np.float32(bits) / np.float32(1 << 24))
        assert -1.0 <= u < 3.0


# ------------------------------------------------------------------------ bf16

def test_bf16_matches_torch_rne():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-30, 30, 20000),
                        np.array([0.0, -0.0, 1.0, -1.0, 0.5, 1 / 3, 12345.0, 1e-30, 3.25], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.bf16_bits(x), want)
    back = O.bf16_to_float(want)
    assert np.array_equal(back, torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy())
    # QuantizationAffineTests.swift:48-58: relative error <= 2^-7 on the listed values
    for v in [0.0, 1.0, -1.0, 0.5, -0.5, 1.0 / 3.0, 12345.0]:
        b = float(O.bf16_to_float(O.bf16_bits(np.array([v], np.float32)))[0])
        assert abs(b - v) / max(abs(v), 1e-6) < 8e-3


# ------------------------------------------------------------------- quantizer

def _np_unpack(q):
    """independent numpy unpack of packed codes -> [rows, n] integer codes"""
    p = q.packed.astype(np.uint32)
    if q.bits == 4:
        codes = np.empty((q.rows, q.n), np.uint32)
        codes[:, 0::2] = p & 0xF
        codes[:, 1::2] = p >> 4
    else:
        codes = np.empty((q.rows, q.n), np.uint32)
        for j in range(4):
            codes[:, j::4] = (p >> (2 * j)) & 3
    return codes


def _np_dequant64(q):
    s = O.bf16_to_float(q.scales).astype(np.float64)
    b = -s if q.biases is None else O.bf16_to_float(q.biases).astype(np.float64)
    codes = _np_unpack(q).astype(np.float64)
    return codes * np.repeat(s, 64, axis=1) + np.repeat(b, 64, axis=1)


def test_nibble_layout_low_even_high_odd():
    # QuantizationTests.swift:35-50
    row = (np.arange(64, dtype=np.float32) - 31.5).reshape(1, 64)
    q = O.quantize(row, 4)
    s = O.bf16_to_float(q.scales)[0, 0]
    b = O.bf16_to_float(q.biases)[0, 0]
    lo, hi = int(q.packed[0, 0] & 0xF), int(q.packed[0, 0] >> 4)
    assert abs(lo * s + b - row[0, 0]) <= s + 1e-3
    assert abs(hi * s + b - row[0, 1]) <= s + 1e-3
    assert lo == 0 and hi == 0 or hi >= lo  # monotone input -> monotone codes


def test_constant_group_reconstructs_bf16_value_exactly():
    # QuantizationAffineTests.swift:61-72
    q = O.quantize(np.full((1, 64), 0.42, np.float32), 4)
    r = O.dequantize(q)
    want = O.bf16_to_float(O.bf16_bits(np.array([0.42], np.float32)))[0]
    assert np.all(r == want)
    assert O.bf16_to_float(q.scales)[0, 0] == 1.0


def test_positive_only_range_uses_full_codebook():
    # QuantizationAffineTests.swift:76-88
    row = (np.arange(64, dtype=np.float32) / np.float32(63.0) + np.float32(1.0)).reshape(1, 64)
    codes = _np_unpack(O.quantize(row, 4))
    assert codes.min() == 0 and codes.max() == 15


def test_roundtrip_bounds():
    # QuantizationAffineTests.swift:10-30 and DequantInt4GEMVReferenceTests.swift:59-76
    row = np.concatenate([0.10 + np.arange(64) * 0.01, -0.50 - np.arange(64) * 0.005]).astype(np.float32)
    r = O.dequantize(O.quantize(row.reshape(1, -1), 4))[0]
    assert np.abs(r - row).max() < 0.025
    for n in (128, 256, 2816):
        raw = O.Rng.key(0xF5, f"int4-affine-roundtrip-n{n}").uniform_fill(-1.0, 1.0, n).reshape(1, n)
        q = O.quantize(raw, 4)
        rec = O.dequantize(q)
        bound = np.repeat(O.bf16_to_float(q.scales), 64, axis=1) + 1e-4
        assert np.all(np.abs(rec - raw) <= bound)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_codes_are_nearest_levels(bits):
    """brute force: every stored code is the nearest of the 2^bits levels q*s+b"""
    raw = O.Rng.key(0x51A71001, "int4-affine-round-trip").uniform_fill(-1.0, 1.0, 4 * 256).reshape(4, 256)
    q = O.quantize(raw, bits)
    s = np.repeat(O.bf16_to_float(q.scales), 64, axis=1).astype(np.float64)
    b = np.repeat(O.bf16_to_float(q.biases), 64, axis=1).astype(np.float64)
    codes = q.packed.astype(np.int64) if bits == 8 else _np_unpack(q).astype(np.int64)
    levels = np.arange(2 ** bits, dtype=np.float64)
    dist = np.abs(raw.astype(np.float64)[..., None] - (levels * s[..., None] + b[..., None]))
    best = dist.min(axis=-1)
    mine = np.take_along_axis(dist, codes[..., None], axis=-1)[..., 0]
    assert np.all(mine <= best + 1e-6 * np.abs(s))  # ties/rounding of (w-b)*inv allow 1 ulp slack


def test_quantizer_edge_cases():
    # Int4AffineEncoderParityTests.swift:41-51: the edge list quantizes to sane codes
    cases = [np.zeros(64), np.full(128, 3.25), np.arange(64) * 1e-30,
             np.where(np.arange(64) == 0, -1e4, 1e4), -np.arange(64) - 1.0,
             np.concatenate([np.full(64, -2.0), np.arange(64) / 7.0])]
    for c in cases:
        row = c.astype(np.float32).reshape(1, -1)
        q = O.quantize(row, 4)
        rec = O.dequantize(q)
        s = np.repeat(O.bf16_to_float(q.scales), 64, axis=1)
        tol = np.maximum(s, 1e-30) + np.abs(row) * 2.0 ** -7 + 1e-30
        assert np.all(np.abs(rec - row) <= tol), c[:4]
    # all-zero group: scale 1, bias 0, codes 0 (constant-group rule)
    q = O.quantize(np.zeros((1, 64), np.float32), 4)
    assert q.scales[0, 0] == 0x3F80 and q.biases[0, 0] == 0 and not q.packed.any()


def test_tensor_equals_row_by_row():
    # Int4AffineEncoderParityTests.swift:53-79 (LCG values)
    state = 0xC0FFEE
    vals = []
    for _ in range(6 * 192):
        state = (state * 6364136223846793005 + 1442695040888963407) & 0xFFFFFFFFFFFFFFFF
        vals.append((np.float32(state >> 40) / np.float32(1 << 24) - np.float32(0.5)) * np.float32(2))
    w = np.array(vals, np.float32).reshape(6, 192)
    full = O.quantize(w, 4)
    for r in range(6):
        one = O.quantize(w[r:r + 1], 4)
        assert np.array_equal(one.packed[0], full.packed[r])
        assert np.array_equal(one.scales[0], full.scales[r])
        assert np.array_equal(one.biases[0], full.biases[r])


# --------------------------------------------------------------------- dequant

def test_dequant_is_two_rounding_closed_form():
    raw = O.Rng(7).uniform_fill(-3.0, 3.0, 5 * 128).reshape(5, 128)
    for bits in (4, 2):
        q = O.quantize(raw, bits)
        s = np.repeat(O.bf16_to_float(q.scales), 64, axis=1)
        b = np.repeat(O.bf16_to_float(q.biases), 64, axis=1)
        want = (_np_unpack(q).astype(np.float32) * s).astype(np.float32) + b  # numpy fp32: 2 roundings
        assert np.array_equal(O.dequantize(q).view(np.uint32), want.astype(np.float32).view(np.uint32))


def test_two_bit_element_order_hand_built():
    # moe.metal:948-951: byte k holds elements 4k..4k+3, element j at bit 2*(j%4)
    codes = np.array([[(r * 5 + i * 3) & 3 for i in range(64)] for r in range(3)], np.uint8)
    packed = O.pack_codes(codes, 2)
    assert packed[0, 0] == (codes[0, 0] | codes[0, 1] << 2 | codes[0, 2] << 4 | codes[0, 3] << 6)
    q = O.QTensor(packed, O.bf16_bits(np.full((3, 1), 0.5, np.float32)),
                  O.bf16_bits(np.full((3, 1), -1.0, np.float32)), 2, 3, 64)
    assert np.array_equal(O.dequantize(q), codes.astype(np.float32) * 0.5 - 1.0)


def test_ternary_is_scale_times_minus_one_zero_one():
    # RepackPlanner.swift:629,640 / MapleMoETests.swift:327-332: bias = -scale
    codes = np.array([[i % 3 for i in range(128)]], np.uint8)
    q = O.QTensor(O.pack_codes(codes, 1), O.bf16_bits(np.array([[0.25, 0.5]], np.float32)), None, 1, 1, 128)
    want = (codes.astype(np.float32) - 1.0) * np.repeat(np.array([[0.25, 0.5]], np.float32), 64, axis=1)
    assert np.array_equal(O.dequantize(q), want)


# ------------------------------------------------------------------------- exp

def test_exp_close_to_libm_and_clamped():
    xs = np.concatenate([np.linspace(-85.9, 87.9, 4001), np.array([0.0, -0.0, 1e-8, -1e-8])])
    for x in xs:
        x = float(np.float32(x))
        got, want = O.exp(x), math.exp(x)
        assert abs(got - want) <= 3e-7 * want
    assert O.exp(-86.5) == 0.0 and O.exp(-1e30) == 0.0 and O.exp(float("-inf")) == 0.0
    assert O.exp(89.0) == float("inf") and math.isnan(O.exp(float("nan")))
    assert O.exp(0.0) == 1.0
    assert abs(O.silu(1.5) - 1.5 / (1 + math.exp(-1.5))) < 1e-6 and O.silu(-100.0) == -0.0


# ---------------------------------------------------------------------- router

def test_router_logits_against_fp64_and_unit_vectors():
    e, d = 16, 256
    rng = O.Rng(0xA5B61234)
    w = O.bf16_bits((rng.uniform_fill(-0.05, 0.05, e * d)).reshape(e, d))
    x = O.bf16_bits(rng.uniform_fill(-1.0, 1.0, d))
    ref = O.bf16_to_float(w).astype(np.float64) @ O.bf16_to_float(x).astype(np.float64)
    got = O.router_logits(w, x)
    assert np.abs(got - ref).max() <= 1e-6 * np.abs(ref).max() + 1e-7
    for i in (0, 7, 8, 63, 64, 255):  # x = e_i returns column i exactly
        unit = np.zeros(d, np.uint16)
        unit[i] = 0x3F80
        assert np.array_equal(O.router_logits(w, unit), O.bf16_to_float(w[:, i]))
    ones = np.full(d, 0x3F80, np.uint16)  # exactly representable weights: sum is exact
    wi = O.bf16_bits(np.tile(np.arange(-8, 8, dtype=np.float32), (e, d // 16)))
    assert np.array_equal(O.router_logits(wi, ones), np.full(e, -8.0 * (d // 16), np.float32))


def _tie_logits(count, trial, rng):
    # RouterTopKParityTests.swift:109-127
    kind = trial % 4
    if kind == 0:
        return np.array([rng.uniform(-4.0, 4.0) for _ in range(count)], np.float32)
    if kind == 1:
        return np.array([np.round(np.float32(rng.uniform(-3.0, 3.0)) * np.float32(4)) / np.float32(4)
                         for _ in range(count)], np.float32)
    if kind == 2:
        levels = [1.5, 0.5, -0.5]
        return np.array([levels[rng.next() % 3] for _ in range(count)], np.float32)
    return np.full(count, 0.75, np.float32)


@pytest.mark.parametrize("e", [8, 16, 24, 33, 100, 128, 168, 255, 256])
def test_topk_equals_sort_by_score_desc_index_asc(e):
    # RouterTopKParityTests.swift:34 seeds + RouterTopKTests.swift:86-96 reference
    rng = O.Rng(0x5EED0001 + e)
    k = 8
    for trial in range(12):
        logits = _tie_logits(e, trial, rng)
        for _ in range(e):
            rng.uniform(0.6, 1.4)
        idx, w = O.topk_softmax(logits, k)
        order = sorted(range(e), key=lambda i: (-float(logits[i]), i))[:k]
        assert list(idx) == order
        sel = logits[order].astype(np.float64)
        want = np.exp(sel - sel[0])
        want /= want.sum()
        assert np.abs(w - want).max() < 5e-7
        assert abs(float(w.sum()) - 1.0) < 2e-6


def test_full_softmax_router_on_the_tied_fixture():
    # MapleMoETests.swift:24-40: deliberate score ties {3,55},{7,63},{11,71},{19,95}
    logits = np.full(256, -4.0, np.float32)
    for i, s in {3: 8, 55: 8, 7: 7, 63: 7, 11: 6, 71: 6, 19: 5, 95: 5}.items():
        logits[i] = s
    idx, w = O.topk_softmax(logits, 8, full_softmax=True)
    assert list(idx) == [3, 55, 7, 63, 11, 71, 19, 95]
    p = np.exp(logits.astype(np.float64) - 8.0)
    p /= p.sum()
    want = p[idx] / p[idx].sum()
    assert np.abs(w - want).max() <= 2e-6 and abs(float(w.sum()) - 1) <= 2e-6
    for bad in (np.nan, np.inf, -np.inf):  # MapleMoETests.swift:141-185: sentinels
        l2 = logits.copy()
        l2[0] = bad
        idx, w = O.topk_softmax(l2, 8, full_softmax=True)
        assert list(idx) == [256] * 8 and not w.any()


def test_topk_fewer_experts_than_k_keeps_index_zero():
    idx, w = O.topk_softmax(np.array([1.0, 3.0, 2.0], np.float32), 8)
    assert list(idx[:3]) == [1, 2, 0] and list(idx[3:]) == [0] * 5 and not w[3:].any()


# -------------------------------------------------------------- family routers

def test_log_and_sqrtsoftplus_against_fp64():
    for t in np.linspace(1.0, 2.0, 4097):
        t = float(np.float32(t))
        assert abs(O.log_1to2(t) - math.log(t)) <= 1.2e-7 * max(math.log(t), 0.5)
    assert O.log_1to2(1.0) == 0.0
    # closed forms: sqrt(ln 2) at 0; the log term vanishes in fp32 beyond |x| = 20
    assert abs(O.sqrtsoftplus(0.0) - math.sqrt(math.log(2.0))) <= 1e-7
    for x in (20.0, 33.5, 1000.0):
        assert O.sqrtsoftplus(x) == float(np.sqrt(np.float32(x)))
        assert O.sqrtsoftplus(-x) == 0.0
    for x in np.linspace(-4.0, 12.0, 801):  # moe.metal:736-740 in fp64
        x = float(np.float32(x))
        want = math.sqrt(max(x, 0.0) + math.log1p(math.exp(-abs(x))))
        assert abs(O.sqrtsoftplus(x) - want) <= 1e-5 * want


@pytest.mark.parametrize("e", [8, 16, 24, 33, 100, 128, 168, 255, 256])
def test_sqrtsoftplus_router_selection_and_weights(e):
    # RouterTopKParityTests.swift:52-77: seeds, tie-heavy logits, duplicated correction biases
    rng = O.Rng(0x5EED0002 + e)
    k, route_scale = 6, 1.5
    for trial in range(12):
        logits = _tie_logits(e, trial, rng)
        bias = np.array([np.float32((i // 7) % 4) * np.float32(0.25) if trial % 3 == 0
                         else rng.uniform(-0.3, 0.3) for i in range(e)], np.float32)
        idx, w = O.router_sqrtsoftplus(logits, bias, k, route_scale)
        raw = np.array([O.sqrtsoftplus(float(v)) for v in logits], np.float32)
        sel = raw + bias
        assert list(idx) == sorted(range(e), key=lambda i: (-float(sel[i]), i))[:k]
        # the bias picks, the raw scores weigh (moe.metal:773-785)
        want = raw[idx].astype(np.float64)
        want = route_scale * want / want.sum()
        assert np.abs(w - want).max() <= 1e-6 and abs(float(w.sum()) - route_scale) <= 1e-6
        assert np.array_equal(O.router_hash_weights(logits, idx, route_scale), w)


def test_hash_router_weights_repeated_experts():
    # RouterTopKParityTests.swift:81-104: a frozen row may repeat experts
    rng = O.Rng(0x5EED0003)
    for trial in range(12):
        logits = _tie_logits(256, trial, rng)
        idx = [(slot % 2) * 17 if trial % 4 == 0 else rng.next() % 256 for slot in range(6)]
        w = O.router_hash_weights(logits, idx, 2.5)
        s = np.array([math.sqrt(max(float(logits[i]), 0) + math.log1p(math.exp(-abs(float(logits[i])))))
                      for i in idx])
        assert np.abs(w - 2.5 * s / s.sum()).max() <= 2e-5
        for a in range(6):
            for b in range(6):
                if idx[a] == idx[b]:
                    assert w[a] == w[b]


def test_inkling_router_is_sigmoid_share_with_sinks():
    # softmax over logsigmoid(x) is sigmoid(x_i) / sum sigmoid(x_j): an independent closed form of
    # inkling.metal:540-565 that a dropped sink, a wrong sign or a missing scale would break
    rng = O.Rng(0x1A2B3C)
    for trial in range(16):
        n_routed, n_shared, k = (256, 2, 8) if trial % 2 == 0 else (100, 1, 6)
        logits = _tie_logits(n_routed + n_shared, trial, rng)
        bias = np.array([rng.uniform(-0.2, 0.2) for _ in range(n_routed)], np.float32)
        if trial % 4 == 1:
            bias[:] = 0.125
        gs, rs = 0.75, 2.5
        idx, w, gam = O.router_inkling(logits, bias, gs, n_routed, n_shared, k, rs)
        sig = 1.0 / (1.0 + np.exp(-logits.astype(np.float64)))
        sel = np.array([np.float32(1.0) / (np.float32(1.0) + np.float32(O.exp(-float(v)))) for v in logits[:n_routed]],
                       np.float32) + bias
        assert list(idx) == sorted(range(n_routed), key=lambda i: (-float(sel[i]), i))[:k]
        members = list(idx) + list(range(n_routed, n_routed + n_shared))
        want = rs * gs * sig[members] / sig[members].sum()
        assert np.abs(np.concatenate([w, gam]) - want).max() <= 2e-6
        assert abs(float(w.sum() + gam.sum()) - rs * gs) <= 2e-6


def test_int8_router_rows_and_scaled_topk():
    e, d = 24, 256
    rng = O.Rng(0x6E44A)
    codes = np.array([rng.next() % 256 for _ in range(e * d)], np.uint8).reshape(e, d)
    scales = O.bf16_bits(rng.uniform_fill(0.001, 0.004, e * d // 64).reshape(e, d // 64))
    biases = O.bf16_bits(rng.uniform_fill(-0.3, -0.1, e * d // 64).reshape(e, d // 64))
    x = O.bf16_bits(rng.uniform_fill(-1.0, 1.0, d))
    eff = O.bf16_bits(rng.uniform_fill(0.5, 1.5, d))
    wf = (codes.astype(np.float64) * np.repeat(O.bf16_to_float(scales).astype(np.float64), 64, axis=1)
          + np.repeat(O.bf16_to_float(biases).astype(np.float64), 64, axis=1))
    ref = wf @ (O.bf16_to_float(x).astype(np.float64) * O.bf16_to_float(eff).astype(np.float64))
    got = O.router_logits_int8(codes, scales, biases, x, eff)
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(wf).sum(axis=1).max()
    one = np.full(d, 0x3F80, np.uint16)
    for i in (0, 1, 63, 64, 200, 255):  # x = e_i: the dequantized weight, two roundings (Quantization.swift:104-119)
        unit = np.zeros(d, np.uint16)
        unit[i] = 0x3F80
        s = O.bf16_to_float(scales[:, i // 64])
        b = O.bf16_to_float(biases[:, i // 64])
        assert np.array_equal(O.router_logits_int8(codes, scales, biases, unit, one),
                              (s * codes[:, i].astype(np.float32)).astype(np.float32) + b)
        twice = np.full(d, 0x4000, np.uint16)  # effective_scale = 2 doubles the row exactly
        assert np.array_equal(O.router_logits_int8(codes, scales, biases, unit, twice),
                              2 * O.router_logits_int8(codes, scales, biases, unit, one))
    # RouterTopKParityTests.swift:30-47: per-expert scales in [0.6, 1.4] as bf16
    r2 = O.Rng(0x5EED0001 + e)
    for trial in range(12):
        logits = _tie_logits(e, trial, r2)
        scale = O.bf16_bits(np.array([r2.uniform(0.6, 1.4) for _ in range(e)], np.float32))
        idx0, w0 = O.topk_softmax(logits, 8)
        idx, w = O.topk_softmax_scaled(logits, scale, 8)
        assert np.array_equal(idx, idx0)
        assert np.array_equal(w, w0 * O.bf16_to_float(scale[idx]))


# ------------------------------------------------------------------------ GEMV

@pytest.mark.parametrize("bits", [4, 2])
@pytest.mark.parametrize("m,n,seed", [(4, 128, 0xF1), (8, 256, 0xF2), (16, 512, 0xF3), (32, 2816, 0xF4)])
def test_gemv_matches_fp64_and_structure(bits, m, n, seed):
    # shapes / seeds of DequantInt4GEMVReferenceTests.swift:32-53
    rng = O.Rng.key(seed, f"int4-gemv-ref-m{m}-n{n}")
    q = O.quantize(rng.uniform_fill(-1.0, 1.0, m * n).reshape(m, n), bits)
    x = rng.uniform_fill(-1.0, 1.0, n)
    w64 = _np_dequant64(q)
    y = O.gemv(q, x)
    ref = w64 @ x.astype(np.float64)
    assert np.abs(y - ref).max() / max(np.abs(ref).max(), 1e-6) < 1e-5  # Tolerance.identity
    unit = np.zeros(n, np.float32)
    unit[n // 3] = 1.0
    assert np.array_equal(O.gemv(q, unit), O.dequantize(q)[:, n // 3])   # x = e_i -> column i
    ones = O.gemv(q, np.ones(n, np.float32))
    assert np.abs(ones - w64.sum(axis=1)).max() < 1e-3                   # x = 1 -> row sums
    y2 = O.gemv(q, (2.0 * x).astype(np.float32))                         # exact power-of-two scaling
    assert np.array_equal(y2, 2.0 * y)


def _np_layer64(layer, x_bits):
    """independent fp64 composition of the layer from unpacked tensors"""
    d, f, e, k = layer.d, layer.f, layer.e, layer.k
    x = O.bf16_to_float(x_bits).astype(np.float64)
    bf = lambda v: O.bf16_to_float(O.bf16_bits(np.asarray(v, np.float32))).astype(np.float64)
    silu = lambda v: v / (1.0 + np.exp(-v))
    logits = O.bf16_to_float(layer.router_w).astype(np.float64) @ x
    order = sorted(range(e), key=lambda i: (-logits[i], i))[:k]
    p = np.exp(logits[order] - logits[order[0]])
    w = p / p.sum()

    def sub(blob, name, rows, cols, bits):
        wo, so, bo = (getattr(layer.off, f"{name}_{s}") for s in "wsb")
        nb = rows * O.packed_row_bytes(bits, cols)
        ns = rows * (cols // 64)
        q = O.QTensor(blob[wo:wo + nb].reshape(rows, -1), blob[so:so + 2 * ns].view(np.uint16).reshape(rows, -1),
                      None if bits == 1 else blob[bo:bo + 2 * ns].view(np.uint16).reshape(rows, -1),
                      bits, rows, cols)
        return _np_dequant64(q)

    acc = np.zeros(d)
    if layer.fs:
        g, u, dn = (_np_dequant64(q) for q in layer.shared)
        a = bf(silu(bf(g @ x)) * bf(u @ x))
        hs = bf(dn @ a)
        if layer.w_sg is not None:
            gate = bf(O.bf16_to_float(layer.w_sg).astype(np.float64) @ x)
            hs = bf(hs / (1.0 + np.exp(-gate)))
        acc = hs.copy()
    for s, ex in enumerate(order):
        blob = layer.experts[ex]
        g = sub(blob, "gate", f, d, layer.bits) @ x
        u = sub(blob, "up", f, d, layer.bits) @ x
        a = bf(silu(g) * u)
        acc = acc + w[s] * (sub(blob, "down", d, f, layer.bits) @ a)
    return bf(acc), order, w


@pytest.mark.parametrize("bits,d,f,e,k,fs", [(4, 128, 64, 16, 8, 64), (4, 128, 64, 12, 6, 0),
                                             (2, 256, 128, 8, 6, 128), (1, 256, 128, 8, 4, 0)])
def test_layer_against_independent_fp64_composition(bits, d, f, e, k, fs):
    # MoEFusedFFNTests.swift:44-190 shape (D 128, F 64, K in {6, 8}), tolerance
    # fp16ChainedReduction = 1e-2 relative (Tolerances.swift:4-21)
    root = 0x2D3
    layer = O.synth_layer(root, d, f, e, k, bits=bits, fs=fs, sigma=0.1)
    x = O.synth_x(root, 1, d)[0]
    y, idx, w = O.moe_layer(layer, x)
    ref, order, wref = _np_layer64(layer, x)
    assert list(idx) == order
    assert np.abs(w - wref).max() < 1e-6
    yf = O.bf16_to_float(y).astype(np.float64)
    assert np.abs(yf - ref).max() / max(np.abs(ref).max(), 1e-6) < 1e-2
    assert np.linalg.norm(yf - ref) / np.linalg.norm(ref) < 1e-3


def test_maple_swiglu_known_answers():
    """maple_swiglu (maple_moe.metal:153-164) on values whose bf16 steps can be followed by hand
    (the test-side restatement in MapleMoETests.swift:411-418 is the same sequence):
    gate 0 -> exp 1, 1 + 1 = 2, 1/2, sigmoid 1 - 1/2, silu 0;
    gate 1, up 2 -> exp bf16(2.71828) = 2.71875, denominator 3.71875 (exact), reciprocal
      bf16(0.268908) = 0.26953125, sigmoid 1 - that = 0.73046875 (exact), silu the same, x 2;
    gate -1 takes the reciprocal itself as sigmoid;
    gate and up beyond the limit: gate clamps at 7 from above only, up at +-7; exp(7) = 1096.6 ->
      1096, + 1 -> 1096, reciprocal 9.1e-4, 1 - that rounds to 1, silu 7, 7 x 7 = 49;
    a very negative gate: exp overflows to inf, reciprocal 0, silu -0;
    gate 1 + 2^-8 is a bf16 tie and narrows to 1 (even), up 7.5 clamps to 7: bf16(0.73046875 x 7) = 5.125."""
    assert O.maple_swiglu(0.0, 3.0) == 0.0
    assert O.maple_swiglu(1.0, 2.0) == 1.4609375
    assert O.maple_swiglu(-1.0, 2.0) == -0.5390625
    assert O.maple_swiglu(100.0, 100.0) == 49.0
    assert O.maple_swiglu(100.0, -100.0) == -49.0
    assert O.maple_swiglu(-100.0, 5.0) == 0.0
    assert O.maple_swiglu(1.00390625, 7.5) == 5.125


def test_maple_layer_is_the_composition_of_its_pinned_parts():
    """with maple_rounding the layer is: activations through maple_swiglu, every expert's down
    output narrowed to bf16 before its routing weight, products added in rank order from the
    first (maple_moe_phase2, maple_moe.metal:243-264) -- rebuilt here from the phase-1 and down
    functions, and different from the layer without the flag"""
    d, f, e, k = 256, 128, 32, 8
    layer = O.synth_layer(0x3A91E, d, f, e, k, bits=O.BITS_TERNARY, router_mode=1, sigma=0.1, maple_rounding=True)
    x = O.synth_x(0x3A91E, 1, d)[0]
    y, idx, w = O.moe_layer(layer, x)
    bf = lambda v: O.bf16_to_float(O.bf16_bits(np.asarray(v, np.float32)))
    acc = np.zeros(d, np.float32)
    for s, ex in enumerate(idx):
        acts = O.expert_phase1(layer.experts[ex], layer.off, layer.bits, d, f, x, maple=True)
        g_u = O.expert_phase1(layer.experts[ex], layer.off, layer.bits, d, f, x, maple=False)
        assert not np.array_equal(acts, g_u)
        v = O.expert_down(layer.experts[ex], layer.off, layer.bits, d, f, acts)
        acc = (acc + np.float32(w[s]) * bf(v)).astype(np.float32)
    assert np.array_equal(y, O.bf16_bits(acc))
    layer.maple_rounding = False
    y0, idx0, _ = O.moe_layer(layer, x)
    assert np.array_equal(idx0, idx) and not np.array_equal(y0, y)
    # the two rules stay close: Maple's steps cost a few bf16 roundings
    a, b = O.bf16_to_float(y).astype(np.float64), O.bf16_to_float(y0).astype(np.float64)
    assert np.linalg.norm(a - b) / np.linalg.norm(b) < 2e-2


def test_residual_rmsnorm_hand_computed_rows():
    """rmsnorm_bf16w (rmsnorm.metal:30-92) after residual_add_fp16 (utility.metal:83-92):
    (3, 4, 0, ...) over 64 elements has mean square 25/64, so inv = 1.6 and the row becomes
    bf16(4.8) = 4.8125, bf16(6.4) = 6.40625; a weight of 0.5 halves them exactly; a unit vector over
    d = 64 becomes 8 e_i; the add is narrowed before the squares are summed: 1 + 2^-9 narrows to 1"""
    d = 64
    one = O.bf16_bits(np.ones(d, np.float32))
    x = np.zeros(d, np.float32); x[0], x[1] = 3.0, 4.0
    h, out = O.residual_rmsnorm(O.bf16_bits(x), one, 0.0)
    got = O.bf16_to_float(out)
    assert got[0] == 4.8125 and got[1] == 6.40625 and not got[2:].any()
    assert np.array_equal(h, O.bf16_bits(x))
    _, out = O.residual_rmsnorm(O.bf16_bits(x), O.bf16_bits(np.full(d, 0.5, np.float32)), 0.0)
    assert O.bf16_to_float(out)[0] == 2.40625 and O.bf16_to_float(out)[1] == 3.203125
    e5 = np.zeros(d, np.float32); e5[5] = -2.0
    _, out = O.residual_rmsnorm(O.bf16_bits(e5), one, 0.0)
    assert O.bf16_to_float(out)[5] == -8.0
    # zeros: only eps under the root; the row stays zero
    _, out = O.residual_rmsnorm(O.bf16_bits(np.zeros(d, np.float32)), one, 1e-6)
    assert not O.bf16_to_float(out).any()
    # hidden + delta is narrowed first: 1 + 2^-9 -> 1, every element 1, the norm returns 1
    h, out = O.residual_rmsnorm(one, one, 0.0, delta_bits=O.bf16_bits(np.full(d, 2.0 ** -9, np.float32)))
    assert np.array_equal(h, one) and np.array_equal(out, one)
    # against fp64 on a random row, to one bf16 step
    r = O.Rng.key(0x5151, "rms")
    xr = O.bf16_bits(r.normal(0.0, 1.5, 2048)); wr = O.bf16_bits(r.normal(1.0, 0.1, 2048))
    _, out = O.residual_rmsnorm(xr, wr, 1e-6)
    xf, wf = O.bf16_to_float(xr).astype(np.float64), O.bf16_to_float(wr).astype(np.float64)
    ref = xf / np.sqrt((xf * xf).mean() + 1e-6) * wf
    assert np.abs(O.bf16_to_float(out) - ref).max() <= np.abs(ref).max() * 2.0 ** -8


def test_shared_expert_rounding_points():
    # SharedExpertInt4Tests.swift:11-53 shape (D 128, F 64, seed 0x604)
    d, f = 128, 64
    t = O.Rng.key(0x604, "shared")
    g, u = (O.quantize(t.uniform_fill(-0.5, 0.5, f * d).reshape(f, d), 4) for _ in range(2))
    dn = O.quantize(t.uniform_fill(-0.5, 0.5, d * f).reshape(d, f), 4)
    x = O.bf16_bits(t.uniform_fill(-1.0, 1.0, d))
    y = O.bf16_to_float(O.shared_expert(g, u, dn, x)).astype(np.float64)
    xf = O.bf16_to_float(x).astype(np.float64)
    bf = lambda v: O.bf16_to_float(O.bf16_bits(np.asarray(v, np.float32))).astype(np.float64)
    a = bf(bf(_np_dequant64(g) @ xf) / (1 + np.exp(-bf(_np_dequant64(g) @ xf))) * bf(_np_dequant64(u) @ xf))
    ref = bf(_np_dequant64(dn) @ a)
    assert np.abs(y - ref).max() / np.abs(ref).max() < 6e-3


# -------------------------------------------------------------------- grouping

KAT_PAIRS = [(0, 3, 0, 10), (0, 1, 1, 11), (0, 4, 2, 12), (1, 1, 0, 13), (1, 3, 1, 14), (1, 2, 2, 15),
             (2, 4, 0, 16), (2, 3, 1, 17), (2, 1, 2, 18), (3, 5, 0, 19), (3, 1, 1, 20), (3, 4, 2, 21)]


def test_grouping_kat():
    # PrefillMoEGroupingTests.swift:5-53, literal expectations
    pairs = np.array(KAT_PAIRS[::-1], dtype=O.PAIR_DTYPE)
    g = O.group_pairs(pairs, 4, 3, 6, tile_expert_count=2)
    assert list(g["sorted"]["expert"]) == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert [[int(p["token"]), int(p["rank"])] for p in g["sorted"]] == [
        [0, 1], [1, 0], [2, 2], [3, 1], [1, 2], [0, 0], [1, 1], [2, 1], [0, 2], [2, 0], [3, 2], [3, 0]]
    assert list(g["offsets"]) == [0xFFFFFFFF, 0, 4, 5, 8, 11]
    assert list(g["counts"]) == [0, 4, 1, 3, 3, 1]
    assert [tuple(x) for x in g["groups"]] == [(1, 0, 4), (2, 4, 1), (3, 5, 3), (4, 8, 3), (5, 11, 1)]
    assert [tuple(x) for x in g["tiles"]] == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]


def test_grouping_order_independent_and_keeps_weight_bits():
    # PrefillMoEGroupingTests.swift:55-82
    tm = [(0, 2, 0, 101), (0, 1, 1, 102), (1, 2, 0, 103), (1, 0, 1, 104), (2, 1, 0, 105), (2, 2, 1, 106)]
    sh = [tm[5], tm[1], tm[3], tm[0], tm[4], tm[2]]
    a = O.group_pairs(np.array(tm, O.PAIR_DTYPE), 3, 2, 3, 2)
    b = O.group_pairs(np.array(sh, O.PAIR_DTYPE), 3, 2, 3, 2)
    for key in a:
        assert np.array_equal(a[key], b[key])
    assert list(a["sorted"]["weight_bits"]) == [104, 102, 105, 101, 103, 106]


def test_grouping_sort_keys_and_errors():
    # PrefillMoEGroupingTests.swift:84-173
    pairs = np.array([(0, 1, 0, 10), (0, 2, 1, 20), (1, 3, 0, 30), (1, 1, 1, 11), (2, 2, 0, 21),
                      (2, 3, 1, 31)], O.PAIR_DTYPE)
    g = O.group_pairs(pairs, 3, 2, 4, 2, sort_keys=[0, 30, 10, 20])
    assert list(g["groups"]["expert"]) == [2, 3, 1]
    assert list(g["sorted"]["expert"]) == [2, 2, 3, 3, 1, 1]
    assert list(g["offsets"]) == [0xFFFFFFFF, 4, 0, 2]
    assert [tuple(x) for x in g["tiles"]] == [(0, 2, 0, 4), (2, 1, 4, 2)]
    one = lambda *p: np.array([p], O.PAIR_DTYPE)
    with pytest.raises(O.GroupingError) as ei:
        O.group_pairs(one(0, 0, 0, 1), 1, 1, 1, 17)
    assert ei.value.kind == "invalidTileExpertCount"
    with pytest.raises(O.GroupingError) as ei:
        O.group_pairs(one(0, 2, 0, 1), 1, 1, 2, 1)
    assert ei.value.kind == "expertOutOfRange"
    with pytest.raises(O.GroupingError) as ei:
        O.group_pairs(np.array([(0, 0, 0, 1), (0, 1, 0, 2)], O.PAIR_DTYPE), 1, 2, 2, 1)
    assert ei.value.kind == "duplicateTokenRank"
    with pytest.raises(O.GroupingError) as ei:
        O.group_pairs(one(0, 0, 0, 1), 1, 1, 2, 1, sort_keys=[0])
    assert ei.value.kind == "expertSortKeyCountMismatch"


def test_grouping_pressure_case():
    # PrefillMoEGroupingTests.swift:175-203
    pairs = np.array([(t, (t + r * 7) % 74, r, t * 8 + r) for t in range(32) for r in range(8)], O.PAIR_DTYPE)
    g = O.group_pairs(pairs, 32, 8, 128, 16)
    assert g["sorted"].size == 256 and g["groups"].size <= 74
    assert g["tiles"]["group_count"].max() <= 16 and g["tiles"]["pair_count"].min() > 0
    assert int(g["counts"].sum()) == 256


def test_reduce_token_major_closed_form():
    # PrefillMoETests.swift:46-64 (cpuReduce)
    rng = np.random.default_rng(3)
    part = rng.standard_normal((5, 4, 16)).astype(np.float32)
    w = rng.random((5, 4)).astype(np.float32)
    got = O.reduce_token_major(part, w)
    ref = (part.astype(np.float64) * w.astype(np.float64)[..., None]).sum(axis=1)
    assert np.abs(got - ref).max() < 2e-6


def test_gate_projection_at_group_32_against_float64(oracle):
    """The group-32 form of the GEMV (the DeepSeek conversion's gate projection: a table entry per 32
    weights, entry = element / 32, moe.metal:996-1041) against float64 arithmetic on codes and tables
    taken apart by hand; group 64 through the same entry point is the ordinary GEMV bit for bit; and the
    helper that quantizes at group 32 gives, per run of 32, the levels nearest to the weights."""
    rng = np.random.default_rng(32)
    rows, n = 24, 256
    w = (rng.standard_normal((rows, n)) * 0.05).astype(np.float32)
    q = oracle.quantize_group32_q2(w)
    assert q.scales.shape == (rows, n // 32) and q.packed.shape == (rows, n // 4)
    codes = ((q.packed[:, :, None] >> (2 * np.arange(4, dtype=np.uint8))) & 3).reshape(rows, n).astype(np.float64)
    s = np.repeat(oracle.bf16_to_float(q.scales).astype(np.float64), 32, axis=1)
    b = np.repeat(oracle.bf16_to_float(q.biases).astype(np.float64), 32, axis=1)
    deq = codes * s + b
    # nearest level of the run's own four levels, up to the rounding of the tables to bf16
    levels = (np.arange(4)[None, None, :] * s[:, :, None] + b[:, :, None])
    best = np.abs(levels - w[:, :, None].astype(np.float64)).min(axis=2)
    assert np.all(np.abs(deq - w) <= best + 1e-3 * np.abs(s))
    x = (rng.standard_normal(n)).astype(np.float32)
    y = np.empty(rows, np.float32)
    lib = oracle.lib()
    rc = lib.mfo_gemv_group(oracle._p(q.packed), oracle._p(q.scales), oracle._p(q.biases), 2,
                            C.c_size_t(rows), C.c_size_t(n), C.c_size_t(32), oracle._p(x), oracle._p(y))
    assert rc == 0
    want = deq @ x.astype(np.float64)
    assert np.allclose(y, want, rtol=0, atol=2e-5 * np.abs(deq).sum(axis=1).max())
    # a wrong table index (entry = element / 64, or the second half reading the first entry) moves the result
    wrong = (codes * np.repeat(oracle.bf16_to_float(q.scales)[:, ::2].astype(np.float64), 64, axis=1)
             + np.repeat(oracle.bf16_to_float(q.biases)[:, ::2].astype(np.float64), 64, axis=1)) @ x.astype(np.float64)
    assert np.abs(wrong - want).max() > 100 * np.abs(y - want).max()
    q64 = oracle.quantize(w, 2)
    y64 = np.empty(rows, np.float32)
    rc = lib.mfo_gemv_group(oracle._p(q64.packed), oracle._p(q64.scales), oracle._p(q64.biases), 2,
                            C.c_size_t(rows), C.c_size_t(n), C.c_size_t(64), oracle._p(x), oracle._p(y64))
    assert rc == 0 and np.array_equal(y64.view(np.uint32), oracle.gemv(q64, x).view(np.uint32))
    assert lib.mfo_gemv_group(oracle._p(q.packed), oracle._p(q.scales), oracle._p(q.biases), 2,
                              C.c_size_t(rows), C.c_size_t(n), C.c_size_t(16), oracle._p(x), oracle._p(y)) != 0


def test_layer_with_int8_scalar_gate_matches_its_bf16_twin():
    """The layer with its scalar shared gate as an 8-bit affine row (RealForwardRunner.swift:2925-2941;
    dequant_int8.metal:66-107) against the same layer with the gate as bf16 numbers, for a row whose dequantized
    weights q / 128 - 1 are bf16 numbers themselves: the two gate logits differ by fp32 summation order only, so
    the layers agree to a bf16 step of the gated shared output -- and the gate is not a no-op."""
    import numpy as np
    from oracle import mf_oracle as O
    d, f, e, k, fs, t = 256, 128, 16, 4, 128, 6
    root = 0x4D464D4F00000000 + 0x1808
    layer = O.synth_layer(root, d, f, e, k, bits=4, fs=fs)
    codes = (np.array([O.Rng.key(root, "gate.codes").next() % 256 for _ in range(d)], np.uint8)).reshape(1, d)
    scales = np.full((1, d // 64), O.bf16_bits(np.array([1.0 / 128], np.float32))[0], np.uint16)
    biases = np.full((1, d // 64), O.bf16_bits(np.array([-1.0], np.float32))[0], np.uint16)
    q8 = O.QTensor(codes, scales, biases, 8, 1, d)
    twin = O.bf16_bits(O.dequantize(q8).reshape(d))
    assert np.array_equal(O.bf16_to_float(twin), O.dequantize(q8).reshape(d))   # exactly representable
    x = O.synth_x(root, t, d)
    layer.w_sg, layer.w_sg_q8 = twin, None
    y_bf16, idx_a, _ = O.moe_layer(layer, x)
    layer.w_sg, layer.w_sg_q8 = None, q8
    y_q8, idx_b, _ = O.moe_layer(layer, x)
    layer.w_sg_q8 = None
    y_none, _, _ = O.moe_layer(layer, x)
    assert np.array_equal(idx_a, idx_b)
    a, b = O.bf16_to_float(y_bf16).astype(np.float64), O.bf16_to_float(y_q8).astype(np.float64)
    assert np.abs(a - b).max() <= 2.0 ** -7 * max(np.abs(a).max(), 1e-3)
    assert (y_bf16 == y_q8).mean() > 0.9
    assert not np.array_equal(y_none, y_q8)
    # the gate logit itself: lane-order value against fp64 on the dequantized row
    ones = np.full(d, 0x3F80, np.uint16)
    w64 = O.dequantize(q8).reshape(d).astype(np.float64)
    for i in range(t):
        got = O.router_logits_int8(codes, scales, biases, x[i], ones)[0]
        ref = float(w64 @ O.bf16_to_float(x[i]).astype(np.float64))
        assert abs(got - ref) <= 1e-5 * max(1.0, abs(ref))


def test_layer_with_narrow_routes_rounds_each_route(oracle):
    """narrow_routes: a route's down output is a bf16 number before it meets its weight -- rebuilt here from
    the per-route functions (prefill.metal:817-819, 644-651)"""
    d, f, e, k = 128, 64, 8, 4
    layer = oracle.synth_layer(0x5EED0000 + 0x7A0, d, f, e, k, bits=4, fs=0)
    x = oracle.synth_x(0x5EED0000 + 0x7A0, 3, d)
    layer.narrow_routes = True
    y, idx, w = oracle.moe_layer(layer, x)
    for t in range(3):
        acc = np.zeros(d, dtype=np.float32)
        for r in range(k):
            ex = int(idx[t, r])
            acts = oracle.expert_phase1(layer.experts[ex], layer.off, 4, d, f, x[t])
            v = oracle.expert_down(layer.experts[ex], layer.off, 4, d, f, acts)
            v = oracle.bf16_to_float(oracle.bf16_bits(v)).astype(np.float32)
            acc = acc + (np.float32(w[t, r]) * v).astype(np.float32)
        assert np.array_equal(oracle.bf16_bits(acc), y[t])
    layer.narrow_routes = False
    y0, _, _ = oracle.moe_layer(layer, x)
    assert not np.array_equal(y0, y)


def test_gelu_tanh_and_the_int8_shared_expert(oracle):
    """mfo_gelu_tanh against the fp64 formula of dequant_int8.metal:44-49 and its limits; mfo_shared_expert_int8
    against an fp64 composition of the dequantized 8-bit tensors (SharedExpertInt8.swift:78-181)."""
    for x in (-30.0, -6.0, -1.5, -0.25, 0.0, 0.3, 1.0, 2.5, 7.0, 40.0):
        want = 0.5 * x * (1.0 + math.tanh(max(-20.0, min(20.0, 0.7978845608028654 * (x + 0.044715 * x ** 3)))))
        assert abs(oracle.gelu_tanh(x) - want) <= 1e-6 * max(1.0, abs(want)), x
    assert oracle.gelu_tanh(0.0) == 0.0 and oracle.gelu_tanh(40.0) == 40.0 and oracle.gelu_tanh(-40.0) == 0.0
    d, f = 128, 192
    rng = oracle.Rng.key(0x5EED0000 + 0x1E8, "int8-mlp")
    gq = oracle.quantize(rng.normal(0.0, 0.05, f * d).reshape(f, d), 8)
    uq = oracle.quantize(rng.normal(0.0, 0.05, f * d).reshape(f, d), 8)
    dq = oracle.quantize(rng.normal(0.0, 0.05, d * f).reshape(d, f), 8)
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, d))
    xf = oracle.bf16_to_float(x).astype(np.float64)
    wg, wu, wd = (oracle.dequantize(q).astype(np.float64) for q in (gq, uq, dq))
    for silu in (False, True):
        y = oracle.bf16_to_float(oracle.shared_expert_int8(gq, uq, dq, x, silu=silu)).astype(np.float64)
        g = oracle.bf16_to_float(oracle.bf16_bits((wg @ xf).astype(np.float32))).astype(np.float64)
        u = oracle.bf16_to_float(oracle.bf16_bits((wu @ xf).astype(np.float32))).astype(np.float64)
        a = g / (1.0 + np.exp(-g)) if silu else 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
        act = oracle.bf16_to_float(oracle.bf16_bits((a * u).astype(np.float32))).astype(np.float64)
        want = wd @ act
        # (the dequantized weights carry two roundings the kernel's s * (q . x) + b * sum(x) form does not:
        # a bf16 ulp on outputs of this size)
        assert np.abs(y - want).max() <= 2e-2 * max(1.0, np.abs(want).max()), (silu, np.abs(y - want).max())
    assert not np.array_equal(oracle.shared_expert_int8(gq, uq, dq, x), oracle.shared_expert_int8(gq, uq, dq, x, silu=True))
