"""mf_shared_expert_static -- the entry point that allocates nothing -- against mf_shared_expert,
through the C ABI, bit for bit: two calls in a row, the second with a smaller input (the built-in
scratch array still holds the first call's activations)."""
from __future__ import annotations

import numpy as np
import pytest
import torch

from mference_amd import _capi, operators as ops
from helpers import to_device_q

pytestmark = pytest.mark.gpu


def _ternary(oracle, rng, rows, cols):
    u = rng.uniform_fill(0.0, 1.0, rows * cols).reshape(rows, cols)
    codes = np.where(u < 0.25, 0, np.where(u < 0.75, 1, 2)).astype(np.uint8)
    scales = oracle.bf16_bits(np.abs(rng.normal(0.0, 0.02, rows * (cols // 64))).reshape(rows, cols // 64) + 1e-3)
    return oracle.QTensor(oracle.pack_codes(codes, 1), scales, None, 1, rows, cols)


def _case(oracle, label, d, f, t, bits=4):
    rng = oracle.Rng.key(0xA110C, label)
    if bits == 1:
        gq, uq, dq = _ternary(oracle, rng, f, d), _ternary(oracle, rng, f, d), _ternary(oracle, rng, d, f)
    else:
        gq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), bits)
        uq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), bits)
        dq = oracle.quantize(rng.normal(0.0, 0.02, d * f).reshape(d, f), bits)
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    return gq, uq, dq, x


def _run_both(gpu, oracle, label, d, f, t, bits=4):
    gq, uq, dq, x = _case(oracle, label, d, f, t, bits)
    g, u, dn, xd = to_device_q(gq), to_device_q(uq), to_device_q(dq), ops.bf16_tensor(x)
    op = ops.SharedExpertInt4(gpu)
    y_ref = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    scratch = torch.zeros((t, f), dtype=torch.bfloat16, device="cuda")
    op.encode(xd, g, u, dn, y_ref, scratch, t=t)
    y = torch.full((t, d), 7.0, dtype=torch.bfloat16, device="cuda")
    op.encode_static(xd, g, u, dn, y, t=t)
    torch.cuda.synchronize()
    got, want = ops.bf16_bits(y), ops.bf16_bits(y_ref)
    assert np.array_equal(got, want), f"{label}: {(got != want).sum()} of {got.size} outputs differ"
    # and the existing entry point agrees with the CPU checker on this case
    ref = np.stack([oracle.shared_expert(gq, uq, dq, x[i]) for i in range(t)])
    err = np.abs(oracle.bf16_to_float(want).astype(np.float64) - oracle.bf16_to_float(ref).astype(np.float64)).max()
    assert err <= 2e-2, (label, err)


def test_static_scratch_matches_shared_expert_twice(gpu, oracle):
    print("case: mf_shared_expert_static d=2048 f=1024 t=4, then d=512 f=256 t=1", flush=True)
    _run_both(gpu, oracle, "first-large", 2048, 1024, 4)
    _run_both(gpu, oracle, "second-small", 512, 256, 1)
    _run_both(gpu, oracle, "third-2bit", 1024, 512, 2, bits=2)
    _run_both(gpu, oracle, "fourth-ternary", 512, 1024, 3, bits=1)


def test_static_scratch_allocates_nothing(gpu, oracle):
    """a run of calls leaves the device's free memory where it was: no hipMalloc / hipFree behind the entry point
    (operands and outputs are allocated before the first reading)"""
    gq, uq, dq, x = _case(oracle, "no-alloc", 1024, 512, 4)
    g, u, dn, xd = to_device_q(gq), to_device_q(uq), to_device_q(dq), ops.bf16_tensor(x)
    op = ops.SharedExpertInt4(gpu)
    y = torch.zeros((4, 1024), dtype=torch.bfloat16, device="cuda")
    op.encode_static(xd, g, u, dn, y, t=4)   # (first call on the device: whatever the runtime sets up lazily)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for n in range(20):
        op.encode_static(xd[:1 + n % 4], g, u, dn, y[:1 + n % 4], t=1 + n % 4)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)


def test_static_scratch_rejects_what_does_not_fit(gpu, oracle):
    lib = _capi.lib()
    gq, uq, dq, x = _case(oracle, "reject", 64, 64, 1)
    g, u, dn, xd = to_device_q(gq), to_device_q(uq), to_device_q(dq), ops.bf16_tensor(x)
    y = torch.zeros((8, 64), dtype=torch.bfloat16, device="cuda")
    f_big = _capi.STATIC_ACT_ELEMS // 8 + 64  # 8 rows of it exceed the array
    st = lib.mf_shared_expert_static(gpu.handle, None, xd.data_ptr(), g.c(), u.c(), dn.c(), 4, 64, f_big, 8,
                                     y.data_ptr())
    assert st == -4  # MF_ERR_SCRATCH_TOO_SMALL, nothing launched
    assert b"built-in scratch" in lib.mf_last_hip_error(gpu.handle)
    assert lib.mf_shared_expert_static(gpu.handle, None, xd.data_ptr(), g.c(), u.c(), dn.c(), 4, 64, 64, 9,
                                       y.data_ptr()) == -1
    assert lib.mf_shared_expert_static(gpu.handle, None, None, g.c(), u.c(), dn.c(), 4, 64, 64, 1,
                                       y.data_ptr()) == -1
    assert lib.mf_shared_expert_static(gpu.handle, None, xd.data_ptr(), g.c(), u.c(), dn.c(), 3, 64, 64, 1,
                                       y.data_ptr()) == -3
    torch.cuda.synchronize()
