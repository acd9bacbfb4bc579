"""Seeded sweeps over shapes nobody picked by hand: the decode call (fused launch and chain of
launches) and the prefill call against the per-token CPU oracle, and the stand-alone dense projection and
shared-expert MLP against the checker's rows.  Shapes are drawn from what
mf_moe_create accepts (widths in multiples of the group size, up to 8 routes per token), so the sweep
crosses the boundaries between the specialised kernels and their fall-backs: widths that are and are not
multiples of 128 or 512, expert counts that are no multiple of 32, tiles that are empty, partial and full."""
import numpy as np
import pytest
import torch

from mference_amd import operators as ops
from helpers import ROOT_SEED, assert_layer_close, make_moe, to_device_layer

pytestmark = pytest.mark.gpu


def _draw(seed, prefill):
    rng = np.random.default_rng(seed)
    bits = int(rng.choice([4, 4, 2, 1]))
    d = int(rng.choice([64, 128, 192, 256, 384, 512, 1024]))
    f = int(rng.choice([64, 128, 192, 256, 512]))
    e = int(rng.choice([8, 12, 16, 24, 32, 64, 100]))
    k = int(rng.choice([1, 2, 4, 6, 8]))
    k = min(k, e)
    fs = int(rng.choice([0, 0, 64, 128, f]))
    if bits != 4 and rng.integers(2):
        fs = 0
    mode = int(rng.integers(2)) if e % 32 == 0 else 0
    limit = float(rng.choice([0.0, 0.0, 7.0]))
    t = int(rng.integers(9, 420)) if prefill else int(rng.integers(1, 9))
    return bits, d, f, e, k, fs, t, mode, limit


@pytest.mark.parametrize("seed", range(40))
def test_decode_sweep(gpu, oracle, seed):
    bits, d, f, e, k, fs, t, mode, limit = _draw(0xD0C0 + seed, prefill=False)
    root = ROOT_SEED + 0xB000 + seed
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=mode, swiglu_limit=limit)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    what = f"seed {seed}: bits={bits} d={d} f={f} e={e} k={k} fs={fs} t={t} mode={mode} limit={limit}"
    results = {}
    for fused in (True, False):
        moe.set_fused(fused)
        y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
        idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
        for _ in range(2):
            y.zero_()
            moe.encode_decode_layer(wts, xd, y, t=t, out_indices=idx, out_weights=w)
            moe.status()
        assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx), what
        assert np.array_equal(w.cpu().numpy().view(np.uint32), ref_w.view(np.uint32)), what
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), what)
        results[fused] = ops.bf16_bits(y)
    assert np.array_equal(results[True], results[False]), what


@pytest.mark.parametrize("seed", range(28))
def test_prefill_sweep(gpu, oracle, seed):
    bits, d, f, e, k, fs, t, mode, limit = _draw(0xF111 + seed, prefill=True)
    root = ROOT_SEED + 0xB800 + seed
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=mode, swiglu_limit=limit)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    moe.encode_prefill_layer(wts, ops.bf16_tensor(x), y, t, out_indices=idx, out_weights=w)
    torch.cuda.synchronize()
    what = f"seed {seed}: bits={bits} d={d} f={f} e={e} k={k} fs={fs} t={t} mode={mode} limit={limit}"
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx), what
    assert np.array_equal(w.cpu().numpy().view(np.uint32), ref_w.view(np.uint32)), what
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), what)


@pytest.mark.parametrize("seed", range(8))
def test_prefill_long_sweep(gpu, oracle, seed):
    """the same draw with 2200 to 4400 tokens (beyond 8192 routes the layer call selects and groups its
    routes chunk by chunk): routing bit-exact on every row, 48 sampled rows against the per-token checker"""
    bits, d, f, e, k, fs, _, mode, limit = _draw(0xF1A0 + seed, prefill=True)
    d, f = min(d, 512), min(f, 256)   # the checker walks every sampled row's experts in numpy
    t = int(np.random.default_rng(0xF1A1 + seed).integers(2200, 4400))
    root = ROOT_SEED + 0xBC00 + seed
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=min(fs, f), router_mode=mode, swiglu_limit=limit)
    x = oracle.synth_x(root, t, d)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    moe.encode_prefill_layer(wts, ops.bf16_tensor(x), y, t, out_indices=idx, out_weights=w)
    torch.cuda.synchronize()
    what = f"seed {seed}: bits={bits} d={d} f={f} e={e} k={k} fs={min(fs, f)} t={t} mode={mode} limit={limit}"
    rows = np.sort(np.random.default_rng(seed).choice(t, size=48, replace=False))
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x[rows])
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32)[rows], ref_idx), what
    assert np.array_equal(w.cpu().numpy().view(np.uint32)[rows], ref_w.view(np.uint32)), what
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)[rows]), oracle.bf16_to_float(ref_y), what)


@pytest.mark.parametrize("seed", range(20))
def test_qmm_sweep(gpu, oracle, seed):
    """the dense projection of many rows (mf_qmm) over drawn (bits, m, n, k): one, two and three windows of
    the contraction, row counts on both sides of a tile, output widths in steps of the group"""
    from helpers import to_device_q
    rng0 = np.random.default_rng(0x0A50 + seed)
    bits = int(rng0.choice([4, 4, 2]))
    m = int(rng0.integers(1, 200))
    n = int(rng0.choice([64, 128, 192, 256, 384, 640]))
    k = int(rng0.choice([64, 128, 192, 512, 1024, 2048, 4352, 8320]))
    rng = oracle.Rng.key(0x0A51, f"qmm-sweep-{seed}")
    q = oracle.quantize(rng.normal(0.0, 0.02, n * k).reshape(n, k), bits)
    xb = oracle.bf16_bits(rng.normal(0.0, 1.0, m * k).reshape(m, k))
    ref = oracle.gemv_multix(q, xb)
    op = ops.MPPPrefillInt4QMM(gpu)
    y = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    path = op.encode(to_device_q(q), ops.bf16_tensor(xb), y, m, n, k)
    torch.cuda.synchronize()
    what = f"seed {seed}: bits={bits} m={m} n={n} k={k} path={path}"
    assert path != "unavailable", what
    assert_layer_close(y.cpu().numpy(), ref, what)


@pytest.mark.parametrize("seed", range(12))
def test_shared_expert_sweep(gpu, oracle, seed):
    """the shared expert / dense MLP over drawn (d, f, t): the GEMV kernels up to 8 rows, the matrix cores
    beyond, against the checker row by row"""
    from helpers import to_device_q
    rng0 = np.random.default_rng(0x5E50 + seed)
    d = int(rng0.choice([128, 256, 512, 1024, 2048]))
    f = int(rng0.choice([64, 128, 256, 512, 1536]))
    t = int(rng0.choice([1, 2, 3, 5, 8, 9, 31, 32, 33, 70, 129]))
    rng = oracle.Rng.key(0x5E51, f"mlp-sweep-{seed}")
    gq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    uq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    dq = oracle.quantize(rng.normal(0.0, 0.02, d * f).reshape(d, f), 4)
    xb = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    ref = np.stack([oracle.shared_expert(gq, uq, dq, xb[i]) for i in range(t)])
    op = ops.SharedExpertInt4(gpu)
    scratch = torch.zeros(max(op.scratch_bytes(d, f, t), t * f * 2), dtype=torch.uint8, device="cuda")
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    op.encode(ops.bf16_tensor(xb), to_device_q(gq), to_device_q(uq), to_device_q(dq), y, scratch, t=t)
    torch.cuda.synchronize()
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref),
                       f"seed {seed}: d={d} f={f} t={t}")
