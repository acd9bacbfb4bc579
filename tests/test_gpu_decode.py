"""GPU parity of the decode path against the CPU oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from mference_amd import _capi
from mference_amd import operators as ops
from helpers import ROOT_SEED, assert_layer_close, errors, make_moe, to_device_layer, to_device_q

pytestmark = pytest.mark.gpu


def _sync():
    torch.cuda.synchronize()


@pytest.mark.parametrize("bits", [4, 2, 8])
@pytest.mark.parametrize("rows,n", [(7, 64), (16, 256), (33, 2048), (5, 4096)])
def test_quantize_bit_exact(gpu, oracle, bits, rows, n):
    rng = oracle.Rng.key(0x51A71001, f"quant-{bits}-{rows}-{n}")
    w = rng.uniform_fill(-1.0, 1.0, rows * n).reshape(rows, n)
    w[0, :64] = 0.42                      # constant group
    if rows > 1:
        w[1, :64] = np.arange(64) * 1e-30  # denormal-scale group
    ref = oracle.quantize(w, bits)
    q = ops.Quantization(gpu).quantize_affine(torch.from_numpy(w).cuda(), bits)
    _sync()
    assert np.array_equal(q.packed.cpu().numpy(), ref.packed)
    assert np.array_equal(ops.bf16_bits(q.scales), ref.scales)
    assert np.array_equal(ops.bf16_bits(q.biases), ref.biases)


@pytest.mark.parametrize("bits", [4, 2, 1, 8])
def test_dequantize_bit_exact(gpu, oracle, bits):
    rows, n = 9, 512
    rng = oracle.Rng.key(0xF5, f"dequant-{bits}")
    if bits == 1:
        codes = (np.array([rng.next() % 3 for _ in range(rows * n)], np.uint8)).reshape(rows, n)
        q = oracle.QTensor(oracle.pack_codes(codes, 1),
                           oracle.bf16_bits(rng.uniform_fill(0.01, 0.2, rows * n // 64).reshape(rows, -1)),
                           None, 1, rows, n)
    else:
        q = oracle.quantize(rng.uniform_fill(-2.0, 2.0, rows * n).reshape(rows, n), bits)
        # adversarial scale/bias pairs: denormal bf16, negative scale, large bias
        q.scales[0, 0], q.biases[0, 0] = 0x0001, 0x8001
        q.scales[1, 1], q.biases[1, 1] = 0xBF80, 0x4700
    ref = oracle.dequantize(q)
    out = ops.Quantization(gpu).dequantize(to_device_q(q))
    _sync()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("bits", [4, 2, 1])
@pytest.mark.parametrize("m,n,t", [(64, 64, 1), (65, 128, 2), (129, 512, 1), (40, 2048, 4),
                                   (24, 4096, 7), (17, 192, 3), (8, 5120, 8)])
def test_gemv_matches_oracle(gpu, oracle, bits, m, n, t):
    rng = oracle.Rng.key(0xF1, f"gemv-{bits}-{m}-{n}-{t}")
    if bits == 1:
        u = rng.uniform_fill(0, 1, m * n).reshape(m, n)
        codes = np.where(u < 0.25, 0, np.where(u < 0.75, 1, 2)).astype(np.uint8)
        q = oracle.QTensor(oracle.pack_codes(codes, 1),
                           oracle.bf16_bits(rng.uniform_fill(0.01, 0.05, m * n // 64).reshape(m, -1)),
                           None, 1, m, n)
    else:
        q = oracle.quantize(rng.uniform_fill(-1.0, 1.0, m * n).reshape(m, n), bits)
    x = oracle.bf16_bits(rng.uniform_fill(-1.0, 1.0, t * n).reshape(t, n))
    ref = oracle.gemv_multix(q, x)
    xd = ops.bf16_tensor(x)
    y32 = torch.full((t, m), 7.0, dtype=torch.float32, device="cuda")
    y16 = torch.zeros((t, m), dtype=torch.bfloat16, device="cuda")
    g = ops.DequantInt4GEMVMultiX(gpu)
    dq = to_device_q(q)
    g.encode(dq, xd, y32, m, n, t, output_float32=True)
    g.encode(dq, xd, y16, m, n, t)
    _sync()
    got = y32.cpu().numpy()
    scale = max(np.abs(ref).max(), 1e-6)
    assert np.abs(got - ref).max() / scale < 2e-5
    assert np.array_equal(ops.bf16_bits(y16), oracle.bf16_bits(got))
    # multi-token rows are bit-identical to single-token calls
    # (MultiXKernelParityTests.swift:50-77)
    for i in range(t):
        yi = torch.zeros((1, m), dtype=torch.float32, device="cuda")
        g.encode(dq, xd[i:i + 1].contiguous(), yi, m, n, 1, output_float32=True)
        _sync()
        assert np.array_equal(yi.cpu().numpy()[0].view(np.uint32), got[i].view(np.uint32))


@pytest.mark.parametrize("bits,m,n,t", [
    (4, 1024, 2048, 1),    # one wave step per row: same partition as the per-row kernel
    (4, 1100, 5120, 1),    # 2.5 steps: the last step is half empty; rows not a multiple of the grid
    (4, 1024, 5120, 4),    # four token rows held in registers
    (4, 1024, 8192, 2),    # longer than one wave can hold at T=2: two waves per row, LDS combine
    (4, 1280, 17408, 1),   # nine steps, split over waves when there are few rows
    (2, 1024, 8192, 1),    # 2-bit: 64 elements per 16 bytes
    (2, 1024, 4096, 4),
    (4, 1056, 5120, 5),    # five to eight token rows of a 4-bit matrix the quad kernel takes: rows 0..3, then the rest
    (4, 1024, 17408, 8),
    (4, 1056, 5184, 5),    # K not a multiple of 512: the 32x32x16 matrix-core kernel (K split over waves)
    (4, 17408, 5120, 8),   # the dense MLP's projections at full size, the widest multi-token call
    (4, 5120, 17408, 8),
])
def test_gemv_streaming_rows_kernel(gpu, oracle, bits, m, n, t):
    """wide matrices take the streaming form (x slices resident in registers, rows walked by
    a wave); same contract as the per-row kernel"""
    rng = oracle.Rng.key(0xF3, f"stream-{bits}-{m}-{n}-{t}")
    q = oracle.quantize(rng.uniform_fill(-1.0, 1.0, m * n).reshape(m, n), bits)
    x = oracle.bf16_bits(rng.uniform_fill(-1.0, 1.0, t * n).reshape(t, n))
    ref = oracle.gemv_multix(q, x)
    xd = ops.bf16_tensor(x)
    y32 = torch.full((t, m), 7.0, dtype=torch.float32, device="cuda")
    g = ops.DequantInt4GEMVMultiX(gpu)
    dq = to_device_q(q)
    g.encode(dq, xd, y32, m, n, t, output_float32=True)
    _sync()
    got = y32.cpu().numpy()
    assert np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6) < 2e-5
    # Multi-token rows against single-token calls (MultiXKernelParityTests.swift:50-77).  4-bit matrices with
    # K a multiple of 512 run the quad kernel for every token count (five to eight rows as 4 + the rest), where
    # a token's instructions do not depend on the others: bit for bit, every row.  The other wide shapes
    # (2-bit, K not a multiple of 512) pick their split of a row over waves by the token count, so their
    # rows agree with single-token calls to fp32 summation order only.
    quad = bits == 4 and n % 512 == 0 and m % 4 == 0 and m >= 1024
    for i in (range(t) if quad else range(min(t, 2))):
        if t == 1:
            break
        yi = torch.zeros((1, m), dtype=torch.float32, device="cuda")
        g.encode(dq, xd[i:i + 1].contiguous(), yi, m, n, 1, output_float32=True)
        _sync()
        one = yi.cpu().numpy()[0]
        if quad:
            assert np.array_equal(one.view(np.uint32), got[i].view(np.uint32)), f"row {i} of {t}"
        else:
            assert np.abs(one - got[i]).max() / max(np.abs(ref).max(), 1e-6) < 2e-6


@pytest.mark.parametrize("m,n,t", [
    (1024, 2048, 3),    # one wave per row set, four slots
    (1100, 5120, 4),    # two waves per row set, five slots; 275 row sets
    (1280, 17408, 2),   # seven waves per row set, ragged last slot; workgroups walk several row sets
    (2048, 4096, 1),
])
def test_gemv_quad_rows_kernel(gpu, oracle, m, n, t):
    """4-bit matrices with K a multiple of 512 and up to 4 token rows take the quad matrix-core
    kernel: every token count runs the same instructions, so a token's row does not depend on how
    many tokens ride along (MultiXKernelParityTests.swift:50-77), bit for bit"""
    rng = oracle.Rng.key(0xF5, f"quad-{m}-{n}-{t}")
    q = oracle.quantize(rng.uniform_fill(-1.0, 1.0, m * n).reshape(m, n), 4)
    x = oracle.bf16_bits(rng.uniform_fill(-1.0, 1.0, t * n).reshape(t, n))
    ref = oracle.gemv_multix(q, x)
    xd = ops.bf16_tensor(x)
    g = ops.DequantInt4GEMVMultiX(gpu)
    dq = to_device_q(q)
    y32 = torch.full((t, m), 7.0, dtype=torch.float32, device="cuda")
    y16 = torch.zeros((t, m), dtype=torch.bfloat16, device="cuda")
    g.encode(dq, xd, y32, m, n, t, output_float32=True)
    g.encode(dq, xd, y16, m, n, t)
    _sync()
    got = y32.cpu().numpy()
    assert np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6) < 2e-5
    assert np.array_equal(ops.bf16_bits(y16), oracle.bf16_bits(got))
    for i in range(t):
        yi = torch.zeros((1, m), dtype=torch.float32, device="cuda")
        g.encode(dq, xd[i:i + 1].contiguous(), yi, m, n, 1, output_float32=True)
        _sync()
        assert np.array_equal(yi.cpu().numpy()[0].view(np.uint32), got[i].view(np.uint32))
    # twice the same launch: the partial sums meet in a fixed order
    y2 = torch.zeros((t, m), dtype=torch.float32, device="cuda")
    g.encode(dq, xd, y2, m, n, t, output_float32=True)
    _sync()
    assert np.array_equal(y2.cpu().numpy().view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("d,f,t", [(2048, 1024, 1), (5120, 1536, 4)])
def test_shared_expert_streaming_rows_kernel(gpu, oracle, d, f, t):
    """dense SwiGLU MLP wide enough for the streaming gate/up and down kernels"""
    rng = oracle.Rng.key(0xF4, f"mlp-{d}-{f}-{t}")
    gq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    uq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    dq = oracle.quantize(rng.normal(0.0, 0.02, d * f).reshape(d, f), 4)
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    ref = np.stack([oracle.shared_expert(gq, uq, dq, x[i]) for i in range(t)])
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    scratch = torch.zeros((t, f), dtype=torch.bfloat16, device="cuda")
    ops.SharedExpertInt4(gpu).encode(ops.bf16_tensor(x), to_device_q(gq), to_device_q(uq),
                                     to_device_q(dq), y, scratch, t=t)
    _sync()
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref), "streaming mlp")


def test_gemv_misaligned_pointers(gpu, oracle):
    m, n = 9, 256
    rng = oracle.Rng.key(0xF2, "gemv-misaligned")
    q = oracle.quantize(rng.uniform_fill(-1.0, 1.0, m * n).reshape(m, n), 4)
    x = oracle.bf16_bits(rng.uniform_fill(-1.0, 1.0, n))
    ref = oracle.gemv_multix(q, x.reshape(1, n))
    # weights at a 1-byte offset, x at a 2-byte offset, sentinel-padded output
    wbuf = torch.full((q.packed.size + 7,), 0xA5, dtype=torch.uint8, device="cuda")
    wbuf[1:1 + q.packed.size] = torch.from_numpy(q.packed.reshape(-1)).cuda()
    xbuf = torch.zeros(n + 8, dtype=torch.bfloat16, device="cuda")
    xbuf[1:1 + n] = ops.bf16_tensor(x)
    dq = to_device_q(q)
    dq.packed = wbuf[1:1 + q.packed.size]
    ybuf = torch.full((m + 8,), 123.0, dtype=torch.float32, device="cuda")
    ops.DequantInt4GEMV(gpu).encode(dq, xbuf[1:1 + n], ybuf[4:4 + m], m, n, output_float32=True)
    _sync()
    y = ybuf.cpu().numpy()
    assert np.all(y[:4] == 123.0) and np.all(y[4 + m:] == 123.0)
    assert np.abs(y[4:4 + m] - ref[0]).max() / np.abs(ref).max() < 2e-5


@pytest.mark.parametrize("e,d,k,t", [(256, 2048, 8, 1), (16, 128, 8, 3), (64, 2048, 8, 5),
                                     (256, 4096, 6, 2), (100, 192, 4, 9), (8, 64, 8, 1),
                                     # the block form (PrefillRouter.encodeGemma4Block): from 16 tokens on the
                                     # batched kernels take the logits -- register-tiled, then matrix-core
                                     (100, 192, 4, 33), (64, 512, 8, 40), (64, 1024, 8, 300)])
@pytest.mark.parametrize("mode", [0, 1])
def test_router_bit_exact(gpu, oracle, e, d, k, t, mode):
    if mode == 1 and e % 32:
        pytest.skip("full-softmax mode needs num_experts % 32 == 0")
    rng = oracle.Rng.key(0xA5B61234, f"router-{e}-{d}-{k}-{t}")
    wr = oracle.bf16_bits(rng.normal(0.0, 0.02, e * d).reshape(e, d))
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    moe = ops.MoE(gpu, d, 64, e, k, router_mode=mode)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, e), dtype=torch.float32, device="cuda")
    moe.encode_router(ops.bf16_tensor(wr), ops.bf16_tensor(x), idx, w, t=t, out_logits=lg)
    _sync()
    for i in range(t):
        ref_lg = oracle.router_logits(wr, x[i])
        assert np.array_equal(lg[i].cpu().numpy().view(np.uint32), ref_lg.view(np.uint32))
        ri, rw = oracle.topk_softmax(ref_lg, k, full_softmax=bool(mode))
        assert np.array_equal(idx[i].cpu().numpy().astype(np.uint32), ri)
        assert np.array_equal(w[i].cpu().numpy().view(np.uint32), rw.view(np.uint32))
    # without a logits buffer the call goes through the handle's own, 256 rows at a time: the same routes
    idx2, w2 = torch.zeros_like(idx), torch.zeros_like(w)
    moe.encode_router(ops.bf16_tensor(wr), ops.bf16_tensor(x), idx2, w2, t=t)
    _sync()
    assert torch.equal(idx2, idx) and torch.equal(w2, w)


def _tie_logits(oracle, count, trial, rng):
    """the four logit families of RouterTopKParityTests.swift:109-127"""
    kind = trial % 4
    if kind == 0:
        return np.array([rng.uniform(-4.0, 4.0) for _ in range(count)], np.float32)
    if kind == 1:
        return np.array([np.float32(np.round(np.float32(rng.uniform(-3.0, 3.0) * np.float32(4))) / 4)
                         for _ in range(count)], np.float32)
    if kind == 2:
        levels = [1.5, 0.5, -0.5]
        return np.array([levels[rng.next() % 3] for _ in range(count)], np.float32)
    return np.full(count, 0.75, np.float32)


@pytest.mark.parametrize("e", [8, 16, 24, 33, 100, 128, 168, 255, 256])
def test_topk_ties_match_serial(gpu, oracle, e):
    """tie-heavy logits straight into the selector through a one-hot x."""
    from mference_amd import _capi
    import ctypes as C
    rng = oracle.Rng(0x5EED0001 + e)
    k = 8
    for trial in range(12):
        logits = _tie_logits(oracle, e, trial, rng)
        for _ in range(e):
            rng.uniform(0.6, 1.4)  # the reference draws per-expert scales here
        # router weights = bf16(logit) column against x = e_0 reproduces bf16-rounded logits
        wr = np.zeros((e, 64), np.uint16)
        wr[:, 0] = oracle.bf16_bits(logits)
        x = np.zeros(64, np.uint16)
        x[0] = oracle.bf16_bits(np.array([1.0], np.float32))[0]
        lg_ref = oracle.bf16_to_float(wr[:, 0])
        for mode in ((0, 1) if e % 32 == 0 else (0,)):
            moe = ops.MoE(gpu, 64, 64, e, k, router_mode=mode)
            idx = torch.zeros((1, k), dtype=torch.int32, device="cuda")
            w = torch.zeros((1, k), dtype=torch.float32, device="cuda")
            moe.encode_router(ops.bf16_tensor(wr), ops.bf16_tensor(x), idx, w)
            _sync()
            ri, rw = oracle.topk_softmax(lg_ref, k, full_softmax=bool(mode))
            assert np.array_equal(idx[0].cpu().numpy().astype(np.uint32), ri), (e, trial, mode)
            assert np.array_equal(w[0].cpu().numpy().view(np.uint32), rw.view(np.uint32))


@pytest.mark.parametrize("bits,d,f,e,k,fs,t", [
    (4, 128, 64, 16, 8, 64, 1),
    (4, 256, 128, 32, 6, 0, 3),
    (4, 2048, 512, 32, 8, 512, 1),
    (2, 512, 256, 16, 6, 128, 4),
    (1, 512, 256, 16, 8, 0, 2),
    (4, 192, 320, 12, 4, 192, 2),
])
def test_decode_layer_matches_oracle(gpu, oracle, bits, d, f, e, k, fs, t):
    root = ROOT_SEED + 0x9000 + bits
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    results = {}
    for fused in (True, False):
        moe.set_fused(fused)
        y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
        idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
        for rep in range(3):  # the fused launch re-arms its own barrier counters
            y.zero_()
            moe.encode_decode_layer(wts, xd, y, t=t, out_indices=idx, out_weights=w)
            moe.status()
        assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
        assert np.array_equal(w.cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y),
                           f"decode layer fused={fused} bits={bits} d={d} f={f}")
        results[fused] = ops.bf16_bits(y)
    # one fused launch == the chain of separate launches, bit for bit
    # (the reference's fused == 3-dispatch gate, SharedExpertInt4Tests.swift:55-115)
    assert np.array_equal(results[True], results[False])


def test_decode_layer_residual_add_in_place(gpu, oracle):
    d, f, e, k, fs, t = 256, 128, 16, 4, 128, 2
    root = ROOT_SEED + 0x9100
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=fs)
    x = oracle.synth_x(root, t, d)
    ref_y, _, _ = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    for fused in (True, False):
        moe.set_fused(fused)
        hidden = ops.bf16_tensor(x)
        y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
        moe.encode_decode_layer(wts, hidden, y, t=t, hidden=hidden)
        moe.status()
        yb = ops.bf16_bits(y)
        want = oracle.bf16_bits(oracle.bf16_to_float(x) + oracle.bf16_to_float(yb))
        assert np.array_equal(ops.bf16_bits(hidden), want)
        assert_layer_close(oracle.bf16_to_float(yb), oracle.bf16_to_float(ref_y), "residual")


def test_two_phase_matches_oracle_and_fused(gpu, oracle):
    """phase 1 + phase 2 as separate calls (MoEFusedFFNTests.swift:44-190 shape D 128, F 64)."""
    d, f, e, k = 128, 64, 16, 8
    root = ROOT_SEED + 0x2D3
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=0)
    x = oracle.synth_x(root, 1, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    idx = torch.from_numpy(ref_idx.astype(np.int32)).cuda()
    w = torch.from_numpy(ref_w).cuda()
    acts = torch.zeros((1, k, f), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_routed_phase1(wts.experts, wts.offsets, idx, xd, acts)
    moe.encode_routed_phase2_reduce(wts.experts, wts.offsets, idx, w, acts, None, y)
    _sync()
    for s in range(k):
        ref_act = oracle.expert_phase1(layer.experts[ref_idx[0, s]], layer.off, 4, d, f, x[0])
        ma, rl = errors(oracle.bf16_to_float(ops.bf16_bits(acts[0, s])), oracle.bf16_to_float(ref_act))
        assert rl < 1e-3
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), "two-phase")


@pytest.mark.parametrize("d,f,e,k,fs,t", [(256, 128, 16, 6, 128, 3), (1024, 256, 32, 6, 0, 8), (4096, 128, 8, 2, 0, 1)])
def test_gate_projection_at_group_32(gpu, oracle, d, f, e, k, fs, t):
    """DeepSeek-V4's 2-bit experts with the gate tables per 32 weights
    (moe_int2_gate_up_rows_simd_dev_vec's gate_group_size, moe.metal:962-1060): phase 1 against the
    oracle row by row, the layer call (which runs the chain of launches for such a layer) against the
    per-token oracle, and the prefill call, which hands the rows to the decode launch.  A handle made
    for group 64 reads the same blob differently -- the tables are really used per 32."""
    root = ROOT_SEED + 0x2E0 + d
    layer = oracle.synth_layer(root, d, f, e, k, bits=2, fs=fs, gate_group=32, swiglu_limit=7.0)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    assert moe.cfg.gate_group_size == 32
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    idx = torch.from_numpy(ref_idx.astype(np.int32)).cuda()
    acts = torch.zeros((t, k, f), dtype=torch.bfloat16, device="cuda")
    moe.encode_routed_phase1(wts.experts, wts.offsets, idx, xd, acts, t=t)
    _sync()
    worst = 0.0
    for tok in range(t):
        for s in range(k):
            ref_act = oracle.expert_phase1(layer.experts[ref_idx[tok, s]], layer.off, 2, d, f, x[tok],
                                           swiglu_limit=7.0, gate_group=32)
            _, rl = errors(oracle.bf16_to_float(ops.bf16_bits(acts[tok, s])), oracle.bf16_to_float(ref_act))
            worst = max(worst, rl)
    assert worst < 2e-3, worst
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    out_idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    moe.encode_decode_layer(wts, xd, y, t=t, out_indices=out_idx)
    moe.status()
    assert np.array_equal(out_idx.cpu().numpy().astype(np.uint32), ref_idx)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), "group-32 gate layer")
    assert moe.prefill_workspace_bytes(t) == 0
    y2 = torch.zeros_like(y)
    moe.encode_prefill_layer(wts, xd, y2, t)
    _sync()
    assert np.array_equal(ops.bf16_bits(y2), ops.bf16_bits(y))
    # the same bytes through a group-64 handle: other activations
    other = ops.MoE(gpu, d, f, e, k, bits=2, swiglu_limit=7.0)
    acts64 = torch.zeros_like(acts)
    other.encode_routed_phase1(wts.experts, wts.offsets, idx, xd, acts64, t=t)
    _sync()
    assert not np.array_equal(ops.bf16_bits(acts64), ops.bf16_bits(acts))
    # group 32 goes with 2-bit codes only
    with pytest.raises(_capi.MfError):
        ops.MoE(gpu, d, f, e, k, bits=4, gate_group_size=32)


@pytest.mark.parametrize("bits,t", [(4, 1), (2, 2), (1, 1)])
def test_routed_phases_over_slots_named_directly(gpu, oracle, bits, t):
    """The slot-map form (MoE.encodeSlotMapGuardedFFN, MoE.swift:333-407; router_slot_lookup_k8,
    moe.metal:594-617) and the routed-argument-buffer form (K (buffer, offset) pairs, MoE.swift:205-253,
    409-440): experts copied into slots of a slab in another order -- or left in two separate buffers and
    named by address -- give the bits of the pool-indexed calls; with a routed expert missing from the
    slots the lookup clears the all-hit word and the guarded launches write nothing."""
    d, f, e, k = 256, 128, 32, 4
    root = ROOT_SEED + 0x2F0 + bits
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=0, router_mode=1 if bits == 1 else 0)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    idx = torch.from_numpy(ref_idx.astype(np.int32)).cuda()
    w = torch.from_numpy(ref_w).cuda()
    acts0 = torch.zeros((t, k, f), dtype=torch.bfloat16, device="cuda")
    y0 = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_routed_phase1(wts.experts, wts.offsets, idx, xd, acts0, t=t)
    moe.encode_routed_phase2_reduce(wts.experts, wts.offsets, idx, w, acts0, None, y0, t=t)
    # a slab of 24 slots, 16-byte aligned stride larger than the blob; the routed experts get slots in
    # descending order, the others none
    stride = (layer.experts.shape[1] + 255) // 256 * 256 + 16
    used = sorted(set(ref_idx.reshape(-1).tolist()))
    slot_of = np.full(e, -1, np.int16)
    slab_h = np.full((24, stride), 0xEE, np.uint8)
    for n, ex in enumerate(reversed(used)):
        slot_of[ex] = 23 - 2 * n if 23 - 2 * n >= 0 else n
        slab_h[slot_of[ex], :layer.experts.shape[1]] = layer.experts[ex]
    slab = torch.from_numpy(slab_h).cuda()
    so = torch.zeros(t * k, dtype=torch.int64, device="cuda")
    hit = torch.zeros(1, dtype=torch.int32, device="cuda")
    moe.encode_slot_lookup(idx, torch.from_numpy(slot_of).cuda(), stride, so, hit, t=t)
    _sync()
    assert hit.item() == 1
    assert np.array_equal(so.cpu().numpy(), slot_of[ref_idx.reshape(-1)].astype(np.int64) * stride)
    acts1 = torch.zeros_like(acts0)
    y1 = torch.zeros_like(y0)
    moe.encode_routed_phase1_slots(slab, so, wts.offsets, xd, acts1, t=t, all_hit=hit)
    moe.encode_routed_phase2_reduce_slots(slab, so, wts.offsets, w, acts1, None, y1, t=t, all_hit=hit)
    _sync()
    assert np.array_equal(ops.bf16_bits(acts1), ops.bf16_bits(acts0))
    assert np.array_equal(ops.bf16_bits(y1), ops.bf16_bits(y0))
    # ... and, directly, the checker's layer (no shared expert, no residual: y = sum of the weighted routes)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y1)), oracle.bf16_to_float(ref_y), f"slots bits={bits}")
    # a slab that starts 2 bytes into its allocation (all the reference promises) takes the byte-wise kernels
    raw = torch.zeros(slab.numel() + 32, dtype=torch.uint8, device="cuda")
    odd_slab = raw[2:2 + slab.numel()]
    odd_slab.copy_(slab.reshape(-1))
    acts_o = torch.zeros_like(acts0)
    y_o = torch.zeros_like(y0)
    moe.encode_routed_phase1_slots(odd_slab, so, wts.offsets, xd, acts_o, t=t, all_hit=hit)
    moe.encode_routed_phase2_reduce_slots(odd_slab, so, wts.offsets, w, acts_o, None, y_o, t=t, all_hit=hit)
    _sync()
    assert np.array_equal(ops.bf16_bits(y_o), ops.bf16_bits(y0))
    # refused without a launch: a slot stride that would break the 16-byte alignment of the blobs, and more
    # rows than one lookup (one guard word) covers
    with pytest.raises(_capi.MfError):
        moe.encode_slot_lookup(idx, torch.from_numpy(slot_of).cuda(), stride + 8, so, hit, t=t)
    with pytest.raises(_capi.MfError):
        moe.encode_routed_phase1_slots(slab, so, wts.offsets, xd, acts1, t=ops.MAX_TOKENS + 1, all_hit=hit)
    # one routed expert loses its slot: the word reads 0 and the guarded launches leave their outputs alone
    gone = slot_of.copy()
    gone[used[0]] = -1
    moe.encode_slot_lookup(idx, torch.from_numpy(gone).cuda(), stride, so, hit, t=t)
    acts2 = torch.full_like(acts0, 3.0)
    y2 = torch.full_like(y0, 5.0)
    moe.encode_routed_phase1_slots(slab, so, wts.offsets, xd, acts2, t=t, all_hit=hit)
    moe.encode_routed_phase2_reduce_slots(slab, so, wts.offsets, w, acts2, None, y2, t=t, all_hit=hit)
    _sync()
    assert hit.item() == 0 and torch.all(acts2 == 3.0).item() and torch.all(y2 == 5.0).item()
    # the argument-buffer form: no slab, the table holds the device address of every slot's blob; the
    # blobs sit in two separate allocations
    half = [ex for n, ex in enumerate(used) if n % 2 == 0]
    buf_a = torch.from_numpy(np.ascontiguousarray(layer.experts[half])).cuda()
    rest = [ex for ex in used if ex not in half]
    buf_b = torch.from_numpy(np.ascontiguousarray(layer.experts[rest])).cuda() if rest else buf_a
    addr = {ex: buf_a.data_ptr() + n * buf_a.stride(0) for n, ex in enumerate(half)}
    addr.update({ex: buf_b.data_ptr() + n * buf_b.stride(0) for n, ex in enumerate(rest)})
    table = torch.from_numpy(np.array([addr[int(ex)] for ex in ref_idx.reshape(-1)], np.int64)).cuda()
    acts3 = torch.zeros_like(acts0)
    y3 = torch.zeros_like(y0)
    moe.encode_routed_phase1_slots(None, table, wts.offsets, xd, acts3, t=t)
    moe.encode_routed_phase2_reduce_slots(None, table, wts.offsets, w, acts3, None, y3, t=t)
    _sync()
    assert np.array_equal(ops.bf16_bits(acts3), ops.bf16_bits(acts0))
    assert np.array_equal(ops.bf16_bits(y3), ops.bf16_bits(y0))


@pytest.mark.parametrize("bits,t", [(4, 1), (2, 3), (1, 2)])
def test_phase1_subsets_write_the_bits_of_the_full_call(gpu, oracle, bits, t):
    """MoEFusedFFNTests.swift:126-186: phase 1 split into slot subsets (the reference's cache hits and
    misses) followed by phase 2 gives the output of the full call bit for bit"""
    d, f, e, k = 256, 128, 16, 8
    root = ROOT_SEED + 0x2D4 + bits
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=0)
    x = oracle.synth_x(root, t, d)
    _, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    idx = torch.from_numpy(ref_idx.astype(np.int32)).cuda()
    w = torch.from_numpy(ref_w).cuda()
    full = torch.zeros((t, k, f), dtype=torch.bfloat16, device="cuda")
    split = torch.full((t, k, f), 7.0, dtype=torch.bfloat16, device="cuda")
    moe.encode_routed_phase1(wts.experts, wts.offsets, idx, xd, full, t=t)
    slots = np.arange(t * k, dtype=np.int32)
    parts = [slots[slots % 3 == 0], slots[slots % 3 == 1], np.concatenate([slots[slots % 3 == 2], [t * k + 5]])]
    for part in parts:  # the last list also names a slot past the table, which must do nothing
        moe.encode_routed_phase1_subset(wts.experts, wts.offsets, idx, xd, split,
                                        torch.from_numpy(part.astype(np.int32)).cuda(), len(part), t=t)
    moe.encode_routed_phase1_subset(wts.experts, wts.offsets, idx, xd, split, None, 0, t=t)  # no slots: no launch
    y_full = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    y_split = torch.zeros_like(y_full)
    moe.encode_routed_phase2_reduce(wts.experts, wts.offsets, idx, w, full, None, y_full, t=t)
    moe.encode_routed_phase2_reduce(wts.experts, wts.offsets, idx, w, split, None, y_split, t=t)
    _sync()
    assert torch.equal(full.view(torch.int16), split.view(torch.int16))
    assert torch.equal(y_full.view(torch.int16), y_split.view(torch.int16))
    # one subset alone leaves the other slots untouched
    lone = torch.full((t, k, f), 7.0, dtype=torch.bfloat16, device="cuda")
    moe.encode_routed_phase1_subset(wts.experts, wts.offsets, idx, xd, lone,
                                    torch.tensor([1], dtype=torch.int32, device="cuda"), 1, t=t)
    _sync()
    assert torch.equal(lone[0, 1].view(torch.int16), full[0, 1].view(torch.int16))
    assert bool((lone[0, 0] == 7.0).all()) and bool((lone[0, 2:] == 7.0).all())


@pytest.mark.parametrize("t", [1, 2, 5, 8])
def test_qwen_shape_specialised_launch(gpu, oracle, t):
    """the full Qwen3.6-shaped layer (D 2048, F 512, E 256, K 8, shared 512) takes the
    shape-specialised fused kernels (one for a single token row, one for any other count); weights drawn
    and quantized on the GPU as bench.py does"""
    import bench
    w = dict(bench.QWEN)
    stack = bench.build_stack(gpu, w, 1, torch.device("cuda", 0))
    host = bench.layer_to_host(stack[0], w)
    moe = ops.MoE(gpu, w["d"], w["f"], w["e"], w["k"], bits=4, shared_f=w["fs"])
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234)
    outs = {}
    for rep in range(3):
        x = torch.randn((t, w["d"]), generator=gen, device="cuda").to(torch.bfloat16)
        ref_y, ref_idx, ref_w = oracle.moe_layer(host, ops.bf16_bits(x))
        for fused in (True, False):
            moe.set_fused(fused)
            y = torch.zeros_like(x)
            idx = torch.zeros((t, w["k"]), dtype=torch.int32, device="cuda")
            rw = torch.zeros((t, w["k"]), dtype=torch.float32, device="cuda")
            moe.encode_decode_layer(stack[0], x, y, t=t, out_indices=idx, out_weights=rw)
            moe.status()
            assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
            assert np.array_equal(rw.cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
            assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y),
                               f"qwen shape fused={fused}")
            outs[fused] = ops.bf16_bits(y)
        assert np.array_equal(outs[True], outs[False])


@pytest.mark.parametrize("limit,maple", [(7.0, False), (0.0, True), (3.0, True)])
def test_qwen_shape_with_other_flags(gpu, oracle, limit, maple):
    """the Qwen-shaped layer with a SwiGLU clamp or Maple rounding: the one-token instance has "no clamp, no
    Maple rounding" as literals, so these calls take the instance that reads the flags from the arguments --
    one token row and three, against the checker and against the chain of launches"""
    import bench
    w = dict(bench.QWEN)
    stack = bench.build_stack(gpu, w, 1, torch.device("cuda", 0))
    host = bench.layer_to_host(stack[0], w)
    host.swiglu_limit, host.maple_rounding = limit, maple
    moe = ops.MoE(gpu, w["d"], w["f"], w["e"], w["k"], bits=4, shared_f=w["fs"], swiglu_limit=limit,
                  maple_rounding=maple)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(99)
    for t in (1, 3):
        x = torch.randn((t, w["d"]), generator=gen, device="cuda").to(torch.bfloat16)
        ref_y, ref_idx, ref_w = oracle.moe_layer(host, ops.bf16_bits(x))
        outs = {}
        for fused in (True, False):
            moe.set_fused(fused)
            y = torch.zeros_like(x)
            idx = torch.zeros((t, w["k"]), dtype=torch.int32, device="cuda")
            moe.encode_decode_layer(stack[0], x, y, t=t, out_indices=idx)
            moe.status()
            assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
            assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y),
                               f"qwen shape limit={limit} maple={maple} t={t} fused={fused}")
            outs[fused] = ops.bf16_bits(y)
        assert np.array_equal(outs[True], outs[False])


@pytest.mark.parametrize("workload,t", [("dsv4-2bit", 1), ("dsv4-2bit", 4), ("dsv4-2bit", 7), ("maple-ternary", 1),
                                        ("maple-ternary", 3), ("maple-ternary", 8), ("maple-preview", 1),
                                        ("maple-preview", 6)])
def test_other_shape_specialised_launches(gpu, oracle, workload, t):
    """the large 2-bit layer (D 4096, F 2048, E 256, K 6, 4-bit shared 2048) and the ternary layer
    (D 2048, F 1024, E 64, K 8, full-softmax router) at full size take their own shape-specialised fused
    kernels (one for a single token row, one for any other count); weights drawn and quantized on the GPU as bench.py does,
    checked against the CPU checker and against the chain of separate launches"""
    import bench
    w = dict(bench.WORKLOADS[workload])
    stack = bench.build_stack(gpu, w, 1, torch.device("cuda", 0))
    host = bench.layer_to_host(stack[0], w)
    mode = ops.ROUTER_FULL_SOFTMAX if w["bits"] == 1 else ops.ROUTER_TOPK_SOFTMAX
    host.router_mode = 1 if w["bits"] == 1 else 0
    moe = ops.MoE(gpu, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                  shared_bits=w["shared_bits"], router_mode=mode, maple_rounding=bool(w.get("maple")))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4321)
    x = torch.randn((t, w["d"]), generator=gen, device="cuda").to(torch.bfloat16)
    ref_y, ref_idx, ref_w = oracle.moe_layer(host, ops.bf16_bits(x))
    outs = {}
    for fused in (True, False):
        moe.set_fused(fused)
        y = torch.zeros_like(x)
        idx = torch.zeros((t, w["k"]), dtype=torch.int32, device="cuda")
        rw = torch.zeros((t, w["k"]), dtype=torch.float32, device="cuda")
        moe.encode_decode_layer(stack[0], x, y, t=t, out_indices=idx, out_weights=rw)
        moe.status()
        assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
        assert np.array_equal(rw.cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y),
                           f"{workload} T={t} fused={fused}")
        outs[fused] = ops.bf16_bits(y)
    assert np.array_equal(outs[True], outs[False])


def test_dense_mlp_full_size(gpu, oracle):
    """hidden 5120, intermediate 17408, 4 token rows (the dense-MLP configuration of bench.py):
    weights drawn and quantized on the GPU, every row against the CPU checker; rows of the
    4-token call equal the single-token calls bit for bit"""
    d, f, t = 5120, 17408, 4
    dev = torch.device("cuda", 0)
    gen = torch.Generator(device=dev)
    gen.manual_seed(2024)
    quant = ops.Quantization(gpu)
    qs = []
    for rows, cols in ((f, d), (f, d), (d, f)):
        raw = torch.randn((rows, cols), generator=gen, device=dev) * 0.02
        qs.append(quant.quantize_affine(raw, 4))
        del raw
    x = torch.randn((t, d), generator=gen, device=dev).to(torch.bfloat16)
    mlp = ops.SharedExpertInt4(gpu)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device=dev)
    scratch = torch.zeros((t, f), dtype=torch.bfloat16, device=dev)
    mlp.encode(x, qs[0], qs[1], qs[2], y, scratch, t=t)
    _sync()

    def hq(q):
        return oracle.QTensor(q.packed.cpu().numpy(), ops.bf16_bits(q.scales), ops.bf16_bits(q.biases), 4, q.rows, q.n)
    hg, hu, hd = hq(qs[0]), hq(qs[1]), hq(qs[2])
    ref = np.stack([oracle.shared_expert(hg, hu, hd, ops.bf16_bits(x[i])) for i in range(t)])
    got = oracle.bf16_to_float(ops.bf16_bits(y)).astype(np.float64)
    reff = oracle.bf16_to_float(ref).astype(np.float64)
    rel_l2 = np.linalg.norm(got - reff) / np.linalg.norm(reff)
    # |y| reaches 8..16 here, where one bf16 step is 0.0625: the max-abs bar is one step of the output
    assert rel_l2 <= 1e-3 and np.abs(got - reff).max() <= 0.0625 + 1e-6, (rel_l2, np.abs(got - reff).max())
    for i in range(t):
        yi = torch.zeros((1, d), dtype=torch.bfloat16, device=dev)
        si = torch.zeros((1, f), dtype=torch.bfloat16, device=dev)
        mlp.encode(x[i:i + 1].contiguous(), qs[0], qs[1], qs[2], yi, si, t=1)
        _sync()
        assert torch.equal(yi[0].view(torch.int16), y[i].view(torch.int16))


@pytest.mark.parametrize("bits,d,f,e,k,t", [(1, 256, 128, 32, 8, 1), (1, 512, 256, 64, 8, 3), (4, 256, 128, 32, 4, 2)])
def test_decode_layer_with_maple_rounding(gpu, oracle, bits, d, f, e, k, t):
    """MapleMoE's rounding points (bf16-stepped activation clamped at 7, bf16 down outputs before
    the routing weights; maple_moe.metal:153-164, 243-264) against the CPU checker, fused launch
    and launch chain bit for bit, and different from the same layer without the flag"""
    root = ROOT_SEED + 0x9A00 + bits + d
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, router_mode=1, sigma=0.1, maple_rounding=True)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, _ = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    results = {}
    for fused in (True, False):
        moe.set_fused(fused)
        y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
        idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
        moe.encode_decode_layer(wts, xd, y, t=t, out_indices=idx)
        moe.status()
        assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y),
                           f"maple rounding fused={fused} bits={bits}")
        results[fused] = ops.bf16_bits(y)
    assert np.array_equal(results[True], results[False])
    layer.maple_rounding = False
    plain = make_moe(gpu, layer)
    y0 = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    plain.encode_decode_layer(wts, xd, y0, t=t)
    plain.status()
    assert not np.array_equal(ops.bf16_bits(y0), results[True])


@pytest.mark.parametrize("d,t,with_delta", [(2048, 1, True), (2048, 5, False), (4096, 3, True), (320, 2, True)])
def test_residual_rmsnorm_matches_oracle(gpu, oracle, d, t, with_delta):
    """hidden += delta, then RMSNorm with a bf16 weight, one launch (rmsnorm.metal:30-92,
    utility.metal:83-92): the updated hidden bit for bit; the normalised rows within one bf16 step
    of the checker (it sums the squares in double, the kernel in fp32 in lane order) and equal on
    all but a few elements"""
    r = oracle.Rng.key(ROOT_SEED + 0x9B00 + d, "rms")
    hb = oracle.bf16_bits(r.normal(0.0, 1.5, t * d).reshape(t, d))
    db = oracle.bf16_bits(r.normal(0.0, 0.5, t * d).reshape(t, d)) if with_delta else None
    wb = oracle.bf16_bits(r.normal(1.0, 0.1, d))
    ref_h, ref_out = oracle.residual_rmsnorm(hb, wb, 1e-6, delta_bits=db)
    hidden = ops.bf16_tensor(hb)
    out = torch.zeros_like(hidden)
    ops.RMSNorm(gpu).encode_bf16w(hidden, ops.bf16_tensor(wb), out, d, 1e-6, t=t,
                                  delta=None if db is None else ops.bf16_tensor(db))
    torch.cuda.synchronize()
    assert np.array_equal(ops.bf16_bits(hidden), ref_h)
    got, ref = oracle.bf16_to_float(ops.bf16_bits(out)), oracle.bf16_to_float(ref_out)
    step = np.maximum(np.abs(ref), 2.0 ** -126) * 2.0 ** -7
    assert (np.abs(got - ref) <= step).all()
    assert (ops.bf16_bits(out) != ref_out).mean() < 0.01


@pytest.mark.parametrize("count", [1, 63, 512, 4099])
def test_silu_mul_matches_oracle(gpu, oracle, count):
    """silu_mul_fp16 (utility.metal:21-33): out = narrow(silu(gate) * up), one rounding, bit for bit
    against the checker's silu on every element (incl. large |gate|, zeros and negative zero)."""
    rng = oracle.Rng.key(0x51, f"silu-mul-{count}")
    g = rng.normal(0.0, 3.0, count).astype(np.float32)
    u = rng.normal(0.0, 2.0, count).astype(np.float32)
    g[: min(count, 6)] = np.array([0.0, -0.0, 40.0, -40.0, 88.5, -100.0], np.float32)[: min(count, 6)]
    gb, ub = oracle.bf16_bits(g), oracle.bf16_bits(u)
    gf, uf = oracle.bf16_to_float(gb), oracle.bf16_to_float(ub)
    ref = oracle.bf16_bits(np.array([np.float32(oracle.silu(float(a))) * np.float32(b) for a, b in zip(gf, uf)],
                                    np.float32))
    out = torch.full((count + 8,), 1.0, dtype=torch.bfloat16, device="cuda")  # 8 sentinels behind
    ops.Elementwise(gpu).encode_silu_mul(ops.bf16_tensor(gb), ops.bf16_tensor(ub), out, count)
    _sync()
    got = ops.bf16_bits(out)
    assert np.array_equal(got[:count], ref)
    assert np.all(got[count:] == 0x3F80)  # nothing written past count


@pytest.mark.parametrize("count", [1, 7, 64, 2048, 5001])
def test_residual_add_matches_oracle(gpu, oracle, count):
    """residual_add_fp16 (utility.metal:83-92): hidden = narrow(hidden + delta), one rounding, in place,
    nothing written past count"""
    rng = oracle.Rng.key(0x52, f"residual-add-{count}")
    hb = oracle.bf16_bits(rng.normal(0.0, 2.0, count).astype(np.float32))
    db = oracle.bf16_bits(rng.normal(0.0, 0.5, count).astype(np.float32))
    ref = oracle.bf16_bits(oracle.bf16_to_float(hb) + oracle.bf16_to_float(db))
    hidden = torch.full((count + 8,), 1.0, dtype=torch.bfloat16, device="cuda")
    hidden[:count] = ops.bf16_tensor(hb)
    ops.Elementwise(gpu).encode_residual_add(hidden, ops.bf16_tensor(db), count)
    _sync()
    got = ops.bf16_bits(hidden)
    assert np.array_equal(got[:count], ref)
    assert np.all(got[count:] == 0x3F80)


def test_nibble_widened_ternary_gemv_exact_bits(gpu, oracle):
    """MapleTernaryGEMV.encode on the resident projections' storage (maple_ternary.metal:12-81): ternary
    codes widened to nibbles with scale (alpha) and bias (-alpha) tables repeated over each source group
    of 128 -- a 4-bit affine tensor, so mf_gemv reads it as MF_BITS_4.  The reference's own vector
    (MapleTernaryGEMVTests.swift:61-134): codes (row*5 + index*3) & 3, alpha = (row+1)(source+1)/8,
    x = (index*7) % 13 - 6, nine rows (a tail of one past two blocks of four), every buffer entered at an
    offset; all values are small exact numbers, so the expected bf16 bits do not depend on summation order."""
    d, rows, groups = 2048, 9, 2048 // 64
    idx = np.arange(d)
    codes = ((np.arange(rows)[:, None] * 5 + idx[None, :] * 3) & 3).astype(np.uint8)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    alpha = ((np.arange(rows)[:, None] + 1) * (np.arange(groups // 2)[None, :] + 1) / 8.0).astype(np.float32)
    scales = np.repeat(oracle.bf16_bits(alpha), 2, axis=1)
    biases = np.repeat(oracle.bf16_bits(-alpha), 2, axis=1)
    x = ((idx * 7) % 13 - 6).astype(np.float32)
    xb = oracle.bf16_bits(x)
    # ternaryReference (:357-378) in exact arithmetic
    xs = oracle.bf16_to_float(xb).astype(np.float64)
    s = np.repeat(oracle.bf16_to_float(scales), 64, axis=1).astype(np.float64)
    b = np.repeat(oracle.bf16_to_float(biases), 64, axis=1).astype(np.float64)
    total = ((codes.astype(np.float64) * s + b) * xs[None, :]).sum(axis=1)
    assert np.all(total == total.astype(np.float32))  # exactly representable: any order gives these bits
    expected = oracle.bf16_bits(total.astype(np.float32))

    def at_offset(arr, prefix_bytes, fill):
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        buf = torch.full((prefix_bytes + raw.size + 6,), fill, dtype=torch.uint8, device="cuda")
        buf[prefix_bytes:prefix_bytes + raw.size] = torch.from_numpy(raw.copy()).cuda()
        return buf, buf[prefix_bytes:prefix_bytes + raw.size]

    kw, wd = at_offset(packed, 1, 0xA5)        # weightsOffset 1
    ks, sd = at_offset(scales, 6, 0xA5)        # 3 parameters in
    kb, bd = at_offset(biases, 6, 0xA5)
    kx, xd = at_offset(xb, 8, 0xA5)            # 4 activations in
    y = torch.full((5 + rows + 3,), 0, dtype=torch.int16, device="cuda")
    y[:] = 0x7BAD
    q = ops.QuantizedTensor(wd, sd.view(torch.bfloat16), bd.view(torch.bfloat16), ops.BITS_4, rows, d)
    ops.DequantInt4GEMV(gpu).encode(q, xd.view(torch.bfloat16), y[5:5 + rows].view(torch.bfloat16), rows, d)
    _sync()
    got = y.cpu().numpy().view(np.uint16)
    assert np.all(got[:5] == 0x7BAD) and np.all(got[5 + rows:] == 0x7BAD)
    assert np.array_equal(got[5:5 + rows], expected)


def test_single_expert_ffn_at_full_size(gpu, oracle):
    """One SwiGLU expert FFN at batch 1, hidden 2048 / intermediate 512, weights N(0, 0.02) quantized
    4-bit g64, x ~ N(0, 1) (the CPU-runnable configuration): as the shared-expert operator
    (gate and up narrowed before the activation, dequant_int4.metal:240-245) against the checker's
    shared expert, and as a routed expert through the two phases with K = 1, weight 1, no residual
    (gate and up kept fp32, moe.metal:526-528, 1262-1270) against the checker's phase functions."""
    d, f = 2048, 512
    rng = oracle.Rng.key(ROOT_SEED + 0x000, "single-expert")
    gq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    uq = oracle.quantize(rng.normal(0.0, 0.02, f * d).reshape(f, d), 4)
    dq = oracle.quantize(rng.normal(0.0, 0.02, d * f).reshape(d, f), 4)
    xb = oracle.bf16_bits(rng.normal(0.0, 1.0, d))
    x = ops.bf16_tensor(xb.reshape(1, d))
    # shared-expert form
    y = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    scratch = torch.zeros((1, f), dtype=torch.bfloat16, device="cuda")
    ops.SharedExpertInt4(gpu).encode(x, to_device_q(gq), to_device_q(uq), to_device_q(dq), y, scratch, t=1)
    _sync()
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)[0]), oracle.bf16_to_float(oracle.shared_expert(gq, uq, dq, xb)),
                       "single expert, shared form")
    # routed form: one blob in the reference's order, K = 1
    off, blob_bytes, stride = ops.expert_blob_layout(d, f, 4, 16384)
    assert blob_bytes == 1769472
    blob = np.zeros(stride, np.uint8)
    ooff = oracle.ExpertOffsets()
    for name, _ in off._fields_:
        setattr(ooff, name, getattr(off, name))
    oracle.pack_expert_blob(gq, uq, dq, ooff, blob)
    moe = ops.MoE(gpu, d, f, 1, 1, bits=4)
    experts = torch.from_numpy(blob.reshape(1, stride)).cuda()
    idx = torch.zeros((1, 1), dtype=torch.int32, device="cuda")
    w = torch.ones((1, 1), dtype=torch.float32, device="cuda")
    acts = torch.zeros((1, 1, f), dtype=torch.bfloat16, device="cuda")
    y2 = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_routed_phase1(experts, off, idx, x, acts)
    moe.encode_routed_phase2_reduce(experts, off, idx, w, acts, None, y2)
    _sync()
    ref_acts = oracle.expert_phase1(blob, ooff, 4, d, f, xb)
    assert np.array_equal(ops.bf16_bits(acts).reshape(-1), ref_acts) or \
        np.abs(oracle.bf16_to_float(ops.bf16_bits(acts).reshape(-1)) - oracle.bf16_to_float(ref_acts)).max() <= 2e-2
    ref_y = oracle.bf16_bits(oracle.expert_down(blob, ooff, 4, d, f, ref_acts))
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y2)[0]), oracle.bf16_to_float(ref_y), "single expert, routed form")


@pytest.mark.parametrize("e", [64, 256])
def test_fused_topk_on_non_finite_logits(gpu, oracle, e):
    """top-k softmax router (mode 0) on logits that are NaN, +inf, -inf, mostly -inf (fewer finite ones than
    routes) or all equal: NaN counts as -inf and is never picked, ranks nobody wins keep index 0 (the serial
    selector of moe.metal:190-240).  The fused launch -- threshold prefilter, its fallback to a rank count over
    all experts when more than 64 candidates tie, and the rank count itself -- gives the indices of the checker
    and the indices AND weight bits of the chain of launches, for the four rows in one call and one at a time."""
    d, f, k, t = 2 * e, 64, 8, 4
    root = ROOT_SEED + 0x9A0 + e
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=0)
    rng = oracle.Rng.key(root, "taps")
    a = oracle.bf16_bits(rng.normal(0.0, 1.0, e))
    b = np.full(e, 0xFF80, np.uint16)                      # -inf ...
    b[[1, e // 2, e - 2, 7, 11, 30, 40]] = oracle.bf16_bits(rng.normal(0.0, 1.0, 7))  # ... but k - 1 finite ones
    a[3], a[5], a[9], a[e - 1] = 0x7FC0, 0x7F80, 0xFF80, 0x7F80   # NaN, +inf, -inf, +inf
    rw = np.zeros((e, d), np.uint16)
    rw[np.arange(e), np.arange(e)] = a                     # logit[e] = a[e] x[e] + b[e] x[E + e]
    rw[np.arange(e), e + np.arange(e)] = b
    layer.router_w = rw
    one, zero = 0x3F80, 0
    x = np.zeros((t, d), np.uint16)
    x[0, :e] = one          # logits a: NaN and both infinities among ordinary scores
    x[1, e:] = one          # logits b (+ 0 * a: NaN where a is not finite): k - 1 finite scores
    x[2, :] = one           # a + b
    x[3, :] = zero          # all logits 0 (NaN where a tap is not finite): every expert ties
    ref_idx = np.stack([oracle.moe_layer(layer, x[i:i + 1])[1][0] for i in range(t)])
    ref_w = np.stack([oracle.moe_layer(layer, x[i:i + 1])[2][0] for i in range(t)])
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)

    def run(fused, rows):
        moe.set_fused(fused)
        n = len(rows)
        y = torch.zeros((n, d), dtype=torch.bfloat16, device="cuda")
        idx = torch.zeros((n, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((n, k), dtype=torch.float32, device="cuda")
        moe.encode_decode_layer(wts, xd[rows].contiguous(), y, t=n, out_indices=idx, out_weights=w)
        moe.status()
        return idx.cpu().numpy().astype(np.uint32), w.cpu().numpy().view(np.uint32), ops.bf16_bits(y)

    try:
        chain = run(False, list(range(t)))
        fused = run(True, list(range(t)))
        assert np.array_equal(chain[0], ref_idx) and np.array_equal(fused[0], ref_idx)
        finite = np.isfinite(ref_w)
        assert np.array_equal(chain[1][finite], ref_w.view(np.uint32)[finite])
        assert np.isnan(chain[1].view(np.float32)[~finite]).all()
        for part in range(3):
            assert np.array_equal(fused[part], chain[part]), ("indices", "weights", "outputs")[part]
        for i in range(t):
            one_row = run(True, [i])
            assert np.array_equal(one_row[0][0], ref_idx[i]) and np.array_equal(one_row[1][0], fused[1][i])
    finally:
        moe.set_fused(True)


@pytest.mark.parametrize("m,n,t", [(1, 2048, 1), (1, 2048, 8), (64, 64, 3), (65, 192, 2), (130, 2816, 1), (8, 5120, 8)])
def test_int8_gemv(gpu, oracle, m, n, t):
    """8-bit affine rows (DequantInt8GEMV.encode, Kernels/Quant/DequantInt8GEMV.swift:53; dequant_int8_gemv_simd,
    dequant_int8.metal:66-107): the value of every (token, row) has the bits of the checker's lane-order row dot
    (x unscaled), agrees with the reference's CPU path (bulk dequantize, scalar dot) to fp32 summation order, and
    does not depend on how many token rows ride along; weights two bytes into their allocation take the
    byte-wise loads."""
    rng = oracle.Rng.key(0x18, f"gemv8-{m}-{n}-{t}")
    q = oracle.quantize(rng.normal(0.0, 0.02, m * n).reshape(m, n), 8)
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, t * n).reshape(t, n))
    ones = np.full(n, 0x3F80, np.uint16)
    exact = np.stack([oracle.router_logits_int8(q.packed, q.scales, q.biases, x[i], ones) for i in range(t)])
    ref = oracle.gemv_multix(q, x)
    g = ops.DequantInt4GEMVMultiX(gpu)
    dq = to_device_q(q)
    xd = ops.bf16_tensor(x)
    y32 = torch.full((t, m), 7.0, dtype=torch.float32, device="cuda")
    y16 = torch.zeros((t, m), dtype=torch.bfloat16, device="cuda")
    g.encode(dq, xd, y32, m, n, t, output_float32=True)
    g.encode(dq, xd, y16, m, n, t)
    _sync()
    got = y32.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), exact.view(np.uint32))
    assert np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6) < 2e-5
    assert np.array_equal(ops.bf16_bits(y16), oracle.bf16_bits(got))
    for i in range(t):
        yi = torch.zeros((1, m), dtype=torch.float32, device="cuda")
        g.encode(dq, xd[i:i + 1].contiguous(), yi, m, n, 1, output_float32=True)
        _sync()
        assert np.array_equal(yi.cpu().numpy()[0].view(np.uint32), got[i].view(np.uint32))
    raw = torch.zeros(q.packed.size + 16, dtype=torch.uint8, device="cuda")
    raw[2:2 + q.packed.size] = torch.from_numpy(q.packed.reshape(-1)).cuda()
    odd = ops.QuantizedTensor(raw[2:2 + q.packed.size].view(m, n), dq.scales, dq.biases, 8, m, n)
    yo = torch.zeros((t, m), dtype=torch.float32, device="cuda")
    g.encode(odd, xd, yo, m, n, t, output_float32=True)
    _sync()
    assert np.array_equal(yo.cpu().numpy().view(np.uint32), exact.view(np.uint32))


@pytest.mark.parametrize("d,f,e,k,fs,t", [(2048, 512, 256, 8, 512, 1), (2048, 512, 256, 8, 512, 4), (512, 256, 32, 4, 256, 3)])
def test_layer_with_int8_scalar_gate(gpu, oracle, d, f, e, k, fs, t):
    """The scalar shared gate as the reference's model files store it -- an 8-bit affine row
    (RealForwardRunner.swift:2925-2941): the fused launch and the chain of launches give the same bits, the
    layer agrees with the checker, and so does the ragged prefill call on the same weights."""
    root = ROOT_SEED + 0x8A7E + d + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=fs)
    gate_row = oracle.Rng.key(root, "w_sg.q8").normal(0.0, 0.05, d).reshape(1, d)
    layer.w_sg_q8 = oracle.quantize(gate_row, 8)
    layer.w_sg = None
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    plain = oracle.synth_layer(root, d, f, e, k, bits=4, fs=fs, with_w_sg=False)
    assert not np.array_equal(oracle.moe_layer(plain, x)[0], ref_y), "the gate has to matter in this case"
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    outs = []
    try:
        for fused in (True, False):
            moe.set_fused(fused)
            y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
            idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
            moe.encode_decode_layer(wts, xd, y, t=t, out_indices=idx)
            moe.status()
            assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
            assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y),
                               f"int8 gate fused={fused}")
            outs.append(ops.bf16_bits(y))
    finally:
        moe.set_fused(True)
    assert np.array_equal(outs[0], outs[1])
    tp = 70
    xp = oracle.synth_x(root + 1, tp, d)
    ref_yp, ref_idxp, _ = oracle.moe_layer(layer, xp)
    yp = torch.zeros((tp, d), dtype=torch.bfloat16, device="cuda")
    idxp = torch.zeros((tp, k), dtype=torch.int32, device="cuda")
    moe.encode_prefill_layer(wts, ops.bf16_tensor(xp), yp, tp, out_indices=idxp)
    _sync()
    assert np.array_equal(idxp.cpu().numpy().astype(np.uint32), ref_idxp)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(yp)), oracle.bf16_to_float(ref_yp), "int8 gate prefill")


@pytest.mark.parametrize("t", [1, 4])
def test_listed_shape_instance_at_full_size(gpu, oracle, t):
    """A layer shape that is no benchmark shape -- Gemma 4's (hidden 2816, 128 experts of 704, top-8;
    ArchConfig.gemma4_26B_A4B, ModelTypes.swift:376-398) -- listed in fused_shapes.json: the build holds
    instances of the fused launch with its dimensions as literals.  At full size against the checker, and the
    same bits as the instance that reads every dimension from its arguments and as the chain of launches;
    with the routing given by the caller too (Gemma routes through its 8-bit router)."""
    d, f, e, k = 2816, 704, 128, 8
    root = ROOT_SEED + 0x6E44A + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=0)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    got = {}
    try:
        for mode in (1, 2, 0):
            moe.set_fused(mode)
            y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
            idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
            w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
            moe.encode_decode_layer(wts, xd, y, t=t, out_indices=idx, out_weights=w)
            moe.status()
            assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
            assert np.array_equal(w.cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
            got[mode] = ops.bf16_bits(y)
        moe.set_fused(1)
        given = ops.MoELayerWeights(None, wts.experts, wts.offsets, None, None)
        yg = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
        moe.encode_decode_layer(given, xd, yg, t=t, out_indices=idx, out_weights=w)
        moe.status()
    finally:
        moe.set_fused(1)
    assert_layer_close(oracle.bf16_to_float(got[1]), oracle.bf16_to_float(ref_y), f"gemma shape t={t}")
    assert np.array_equal(got[1], got[2]) and np.array_equal(got[1], got[0])
    assert np.array_equal(ops.bf16_bits(yg), got[1])


@pytest.mark.parametrize("d,f,t,silu", [(256, 128, 1, False), (2816, 2112, 3, False), (512, 1024, 9, True)])
def test_int8_shared_expert(gpu, oracle, d, f, t, silu):
    """SharedExpertInt8.encode (SharedExpertInt8.swift:78-181): 8-bit gate / up rows in one launch with the tanh
    GELU (or SiLU), 8-bit down rows -- the checker's bits (the lane order and the activation are defined)."""
    rng = oracle.Rng.key(ROOT_SEED + 0x1E8, f"int8-mlp-{d}-{f}")
    gq = oracle.quantize(rng.normal(0.0, 0.03, f * d).reshape(f, d), 8)
    uq = oracle.quantize(rng.normal(0.0, 0.03, f * d).reshape(f, d), 8)
    dq = oracle.quantize(rng.normal(0.0, 0.03, d * f).reshape(d, f), 8)
    xb = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    ref = np.stack([oracle.shared_expert_int8(gq, uq, dq, xb[i], silu=silu) for i in range(t)])
    g, u, dn, x = to_device_q(gq), to_device_q(uq), to_device_q(dq), ops.bf16_tensor(xb)
    op = ops.SharedExpertInt8(gpu, silu_activation=silu)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    scratch = torch.zeros((t, f), dtype=torch.bfloat16, device="cuda")
    op.encode(x, g, u, dn, y, scratch, t=t)
    torch.cuda.synchronize()
    assert np.array_equal(ops.bf16_bits(y), ref)
    lib = _capi.lib()
    assert lib.mf_shared_expert_int8(gpu.handle, None, x.data_ptr(), g.c(), u.c(), dn.c(), d, f, t, 0, y.data_ptr(),
                                     scratch.data_ptr(), t * f * 2 - 2) == -4
    assert lib.mf_shared_expert_int8(gpu.handle, None, x.data_ptr(), g.c(), u.c(), dn.c(), d + 8, f, t, 0, y.data_ptr(),
                                     scratch.data_ptr(), t * f * 2) == -2


@pytest.mark.parametrize("bits,d,f,e,k,fs,t,with_delta", [
    (4, 2048, 512, 256, 8, 512, 1, True),     # the headline shape's one-token instance
    (4, 2048, 512, 256, 8, 512, 5, False),    # ... its several-rows instance, no delta
    (4, 512, 256, 32, 4, 128, 8, True),       # the instance that reads every dimension; two rounds of four rows
    (2, 1024, 512, 16, 6, 0, 3, True),        # 2-bit, no shared expert
    (1, 512, 256, 32, 8, 0, 2, True),         # ternary, full-softmax router
    (4, 4608, 128, 16, 2, 0, 2, True),        # rows wider than 4096: two launches behind the same call
])
def test_decode_layer_with_the_norm_in_front(gpu, oracle, bits, d, f, e, k, fs, t, with_delta):
    """mf_moe_decode_layer_normed: hidden += delta, x = RMSNorm(hidden) * w, y = layer(x), hidden += y in one
    call -- the bits of mf_residual_rmsnorm followed by mf_moe_decode_layer (also with the fused launch off),
    and the checker's composition of the two."""
    root = ROOT_SEED + 0x4042 + d + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=1 if bits == 1 else 0,
                               maple_rounding=bits == 1)
    rng = oracle.Rng.key(root, "norm")
    hb = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    db = oracle.bf16_bits(rng.normal(0.0, 0.5, t * d).reshape(t, d)) if with_delta else None
    wb = oracle.bf16_bits(1.0 + rng.normal(0.0, 0.1, d))
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    # reference: the two calls
    h_ref = ops.bf16_tensor(hb).clone()
    xn = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    ops.RMSNorm(gpu).encode_bf16w(h_ref, ops.bf16_tensor(wb), xn, d, 1e-6, t=t,
                                  delta=None if db is None else ops.bf16_tensor(db))
    y_ref = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_decode_layer(wts, xn, y_ref, t, hidden=h_ref)
    for fused in (1, 0):
        moe.set_fused(fused)
        h = ops.bf16_tensor(hb).clone()
        y = torch.full((t, d), 3.0, dtype=torch.bfloat16, device="cuda")
        idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
        moe.encode_decode_layer_normed(wts, h, ops.bf16_tensor(wb), y, t, delta=None if db is None else ops.bf16_tensor(db),
                                       eps=1e-6, out_indices=idx, out_weights=w)
        torch.cuda.synchronize()
        moe.status()
        assert torch.equal(y, y_ref), f"y, fused={fused}"
        assert torch.equal(h, h_ref), f"hidden, fused={fused}"
    moe.set_fused(1)
    # the checker: norm, layer, residual add
    h1, x_ref = oracle.residual_rmsnorm(hb, wb, 1e-6, delta_bits=db)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x_ref)
    assert np.array_equal(ops.bf16_bits(xn), x_ref)
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(ref_y), "normed layer")
