"""The dense projection of many rows (mf_qmm = MPPPrefillInt4QMM.encode) and the block form of the
shared expert / dense MLP (mf_shared_expert beyond 8 rows), against the CPU checker and against the
closed-form inputs and tolerances of the reference's own test (MPPPrefillInt4QMMTests.swift)."""
import numpy as np
import pytest
import torch

from mference_amd import _capi
from mference_amd import operators as ops
from helpers import assert_layer_close, to_device_q

pytestmark = pytest.mark.gpu


def _reference_inputs(oracle, m, n, k, adversarial):
    """makeInputs of MPPPrefillInt4QMMTests.swift:20-62, with bf16 x where the reference has fp16"""
    groups = k // 64
    packed = ((np.arange(n * k // 2, dtype=np.int64) * 37 + 0x29) & 0xFF).astype(np.uint8).reshape(n, k // 2)
    row, grp = np.meshgrid(np.arange(n), np.arange(groups), indexing="ij")
    if adversarial:  # tiny, negative and denormal bf16 scales and biases
        one = lambda v: int(oracle.bf16_bits(np.array([v], np.float32))[0])
        adv_s = np.array([one(0.001), one(-0.0015), 0x0001, 0x8001], np.uint16)
        adv_b = np.array([one(-0.01), one(0.006), 0x0001, 0x8001], np.uint16)
        scales, biases = adv_s[(row + grp) % 4], adv_b[(row * 3 + grp) % 4]
    else:
        scales = oracle.bf16_bits((0.001 + ((row + grp) % 5) * 0.00025).astype(np.float32))
        biases = oracle.bf16_bits((-0.01 + ((row * 3 + grp) % 7) * 0.002).astype(np.float32))
    x = (((np.arange(m * k, dtype=np.int64) * 11) % 29 - 14) / 64.0).astype(np.float32).reshape(m, k)
    q = oracle.QTensor(np.ascontiguousarray(packed), np.ascontiguousarray(scales.astype(np.uint16)),
                       np.ascontiguousarray(biases.astype(np.uint16)), 4, n, k)
    return q, oracle.bf16_bits(x)


def _closed_form(oracle, q, x_bits):
    """cpuReference of the reference's test (:84-111) in fp64: sum of (q * scale + bias) * x"""
    w = oracle.dequantize(q).astype(np.float64)  # float(q) * scale + bias, the test's fma-free weight
    return oracle.bf16_to_float(x_bits).astype(np.float64) @ w.T


def _expected_path(n, k, weight_offset):
    return "affine-matrix-core-bf16" if n % 128 == 0 and k % 128 == 0 and weight_offset % 16 == 0 else "affine-rows-gemv"


def _offset_tensor(arr, offset_bytes):
    """device copy of `arr` that starts offset_bytes into its allocation"""
    raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
    buf = torch.zeros(raw.size + offset_bytes + 16, dtype=torch.uint8, device="cuda")
    buf[offset_bytes:offset_bytes + raw.size] = torch.from_numpy(raw.copy()).cuda()
    return buf, buf[offset_bytes:]


@pytest.mark.parametrize("m,n,k,adversarial,offsets", [
    (64, 32, 64, False, (0, 0, 0)), (64, 32, 128, True, (0, 0, 0)), (17, 35, 64, False, (0, 0, 0)),
    (17, 35, 128, True, (13, 2, 6)),                    # the reference's four cases (:191-205)
    (64, 128, 128, True, (0, 0, 0)), (96, 256, 2048, False, (0, 0, 0)), (33, 384, 4352, False, (0, 0, 0)),
    (130, 128, 8320, True, (0, 0, 0)),                  # matrix-core path: one window, two, three
])
def test_qmm_matches_reference_test_inputs(gpu, oracle, m, n, k, adversarial, offsets):
    q, xb = _reference_inputs(oracle, m, n, k, adversarial)
    keep_w, wdev = _offset_tensor(q.packed, offsets[0])
    keep_s, sdev = _offset_tensor(q.scales, offsets[1])
    keep_b, bdev = _offset_tensor(q.biases, offsets[2])
    qd = ops.QuantizedTensor(wdev, sdev.view(torch.bfloat16), bdev.view(torch.bfloat16), 4, n, k)
    op = ops.MPPPrefillInt4QMM(gpu)
    y = torch.full((m, n), 9.0, dtype=torch.bfloat16, device="cuda")
    path = op.encode(qd, ops.bf16_tensor(xb), y, m, n, k)
    torch.cuda.synchronize()
    # the path that ran (MPPPrefillInt4QMM.swift:5-8): the matrix-core kernel needs n and k multiples of 128 and
    # a 16-byte aligned weight buffer; everything else goes row by row through the GEMV kernels
    assert path == _expected_path(n, k, offsets[0])
    got = oracle.bf16_to_float(ops.bf16_bits(y)).astype(np.float64)
    ref = _closed_form(oracle, q, xb)
    max_abs = np.abs(got - ref).max()
    rel = max_abs / max(np.abs(ref).max(), 1e-6)   # RelError.compute: max|a - r| / max(max|r|, 1e-6)
    assert max_abs <= 0.03 and rel <= 5e-3, (m, n, k, max_abs, rel)  # bf16 outputs: 2^-8 relative per value
    # byte-stable across dispatches (the reference's fullProductionShapeIsByteStableAcross32Dispatches)
    for _ in range(3):
        y2 = torch.zeros_like(y)
        op.encode(qd, ops.bf16_tensor(xb), y2, m, n, k)
        torch.cuda.synchronize()
        assert torch.equal(y, y2)


@pytest.mark.parametrize("bits,m,n,k", [(4, 70, 256, 512), (2, 64, 128, 1024), (1, 40, 256, 256), (4, 9, 64, 192)])
def test_qmm_matches_gemv_oracle(gpu, oracle, bits, m, n, k):
    """random weights, every format; fp32 and bf16 outputs against the checker's GEMV row by row"""
    rng = oracle.Rng.key(0x0A11, f"qmm-{bits}-{m}-{n}-{k}")
    if bits == 1:
        codes = (rng.uniform_fill(0.0, 4.0, n * k).astype(np.int64) // 1).clip(0, 3)
        codes = np.where(codes == 3, 1, codes).astype(np.uint8).reshape(n, k)
        scales = oracle.bf16_bits(np.abs(rng.normal(0.0, 0.02, n * (k // 64))).reshape(n, k // 64) + 1e-3)
        q = oracle.QTensor(oracle.pack_codes(codes, 1), scales, None, 1, n, k)
    else:
        q = oracle.quantize(rng.normal(0.0, 0.02, n * k).reshape(n, k), bits)
    xb = oracle.bf16_bits(rng.normal(0.0, 1.0, m * k).reshape(m, k))
    ref = oracle.gemv_multix(q, xb)
    qd = to_device_q(q)
    op = ops.MPPPrefillInt4QMM(gpu)
    yf = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    yb = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    assert op.encode(qd, ops.bf16_tensor(xb), yf, m, n, k) == _expected_path(n, k, 0)
    op.encode(qd, ops.bf16_tensor(xb), yb, m, n, k)
    torch.cuda.synchronize()
    assert_layer_close(yf.cpu().numpy(), ref, f"qmm fp32 bits={bits}")
    # the narrowed output against the narrowed reference: narrowing alone is 2^-9 relative per value
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(yb)), oracle.bf16_to_float(oracle.bf16_bits(ref)),
                       f"qmm bf16 bits={bits}")


def test_qmm_unavailable_for_bad_arguments(gpu, oracle):
    """MPPPrefillInt4QMM.swift:43-55: a K that is no multiple of the group, empty sizes, odd table offsets"""
    q, xb = _reference_inputs(oracle, 8, 32, 64, False)
    qd = to_device_q(q)
    op = ops.MPPPrefillInt4QMM(gpu)
    y = torch.zeros((8, 32), dtype=torch.bfloat16, device="cuda")
    x = ops.bf16_tensor(xb)
    assert op.encode(qd, x, y, 8, 32, 96) == "unavailable"
    assert op.encode(qd, x, y, 0, 32, 64) == "unavailable"
    assert op.encode(qd, x, y, 8, 0, 64) == "unavailable"
    keep, odd = _offset_tensor(q.scales, 1)
    bad = ops.QuantizedTensor(qd.packed, odd, qd.biases, 4, 32, 64)
    assert op.encode(bad, x, y, 8, 32, 64) == "unavailable"
    torch.cuda.synchronize()


def _close_or_one_step(oracle, got_bits, ref_bits, what):
    """rel-L2 1e-3 and max-abs 2e-2 -- except where the outputs are so large that one bf16 step exceeds
    2e-2 (|y| >= 4: steps of 1/32 and more): there the max-abs bar is one step of the largest output"""
    got = oracle.bf16_to_float(got_bits).astype(np.float64)
    ref = oracle.bf16_to_float(ref_bits).astype(np.float64)
    rel_l2 = np.linalg.norm(got - ref) / np.linalg.norm(ref)
    step = 2.0 ** (np.floor(np.log2(np.abs(ref).max())) - 7)
    max_abs = np.abs(got - ref).max()
    assert rel_l2 <= 1e-3 and max_abs <= max(2e-2, step + 1e-9), (what, rel_l2, max_abs, step)


# (d = 7680: 120 K groups, more than one gate/up launch holds tables for -- the contraction goes in two windows
# that meet in the SwiGLU combine pass)
@pytest.mark.parametrize("d,f,t", [(2048, 512, 40), (1024, 1536, 128), (5120, 1536, 33), (7680, 256, 70)])
def test_shared_expert_block_form(gpu, oracle, d, f, t):
    """PrefillSharedExpert.encodeBlock: t >= 32 rows through the matrix cores == the checker's shared
    expert row by row within the layer tolerance; with only t*f of scratch the call goes row by row and
    gives the bits of t calls with one row each."""
    rng = oracle.Rng.key(0xB10C, f"block-{d}-{f}-{t}")
    gq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    uq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    dq = oracle.quantize(rng.normal(0.0, 0.02, d * f).reshape(d, f), 4)
    xb = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    ref = np.stack([oracle.shared_expert(gq, uq, dq, xb[i]) for i in range(t)])
    g, u, dn, x = to_device_q(gq), to_device_q(uq), to_device_q(dq), ops.bf16_tensor(xb)
    op = ops.SharedExpertInt4(gpu)
    need = op.scratch_bytes(d, f, t)
    assert need > t * f * 2
    big = torch.zeros(need, dtype=torch.uint8, device="cuda")
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    op.encode(x, g, u, dn, y, big, t=t)
    torch.cuda.synchronize()
    _close_or_one_step(oracle, ops.bf16_bits(y), ref, f"block mlp d={d} f={f} t={t}")
    small = torch.zeros((t, f), dtype=torch.bfloat16, device="cuda")
    y_rows = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    op.encode(x, g, u, dn, y_rows, small, t=t)
    y_one = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    for i in range(0, t, 7):
        op.encode(x[i:i + 1], g, u, dn, y_one[i:i + 1], small, t=1)
    torch.cuda.synchronize()
    _close_or_one_step(oracle, ops.bf16_bits(y_rows), ref, "row by row")
    for i in range(0, t, 7):
        assert torch.equal(y_rows[i], y_one[i])
