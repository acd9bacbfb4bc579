"""GPU parity of the family-specific routers (DeepSeek-V4 sqrtsoftplus and hash routing, the
Inkling sigmoid router with shared sinks, Gemma's 8-bit router with per-expert scales) against the
CPU oracle, through the C ABI: logits, indices and routing weights bit for bit."""
import numpy as np
import pytest
import torch

from mference_amd import _capi
from mference_amd import operators as ops
from helpers import ROOT_SEED, assert_layer_close, make_moe, to_device_layer

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def _f32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def _tie_logits(count, trial, rng):
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


def _one_hot_router(oracle, logits_rows):
    """router rows whose bf16 column j against x = e_j reproduce (bf16-rounded) logits of row j"""
    t, e = logits_rows.shape
    d = 64
    wr = np.zeros((e, d), np.uint16)
    x = np.zeros((t, d), np.uint16)
    for j in range(t):
        wr[:, j] = oracle.bf16_bits(logits_rows[j])
        x[j, j] = 0x3F80
    return wr, x, oracle.bf16_to_float(wr[:, :t].T.copy())


def _draw(oracle, label, e, d, t, sigma_w=0.02):
    rng = oracle.Rng.key(ROOT_SEED + 0xFA31, label)
    wr = oracle.bf16_bits(rng.normal(0.0, sigma_w, e * d).reshape(e, d))
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    return rng, wr, x


@pytest.mark.parametrize("e,d,k,t", [(256, 4096, 6, 1), (256, 2048, 6, 4), (100, 512, 6, 3), (33, 256, 8, 2),
                                     (512, 1024, 8, 2), (256, 4096, 6, 300)])
def test_sqrtsoftplus_router_bit_exact(gpu, oracle, e, d, k, t):
    rng, wr, x = _draw(oracle, f"sqrtsoftplus-{e}-{d}-{k}-{t}", e, d, t, 0.05)
    bias = rng.uniform_fill(-0.3, 0.3, e)
    fam = ops.FamilyRouters(gpu)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, e), dtype=torch.float32, device="cuda")
    fam.encode_router_top_k(ops.bf16_tensor(wr), ops.bf16_tensor(x), _f32(bias), idx, w, e, d, 1.5, lg,
                            top_k=k, t=t)
    torch.cuda.synchronize()
    lg_h, idx_h, w_h = lg.cpu().numpy(), idx.cpu().numpy().astype(np.uint32), w.cpu().numpy()
    for i in list(range(min(t, 8))) + ([t - 1, t // 2] if t > 8 else []):
        ref_lg = oracle.router_logits(wr, x[i])
        assert np.array_equal(_bits(lg_h[i]), _bits(ref_lg))
        ri, rw = oracle.router_sqrtsoftplus(ref_lg, bias, k, 1.5)
        assert np.array_equal(idx_h[i], ri), (i, idx_h[i], ri)
        assert np.array_equal(_bits(w_h[i]), _bits(rw))
    # the hash form on the same experts gives the same weights
    w2 = torch.zeros_like(w)
    fam.encode_router_hash_weights(ops.bf16_tensor(wr), ops.bf16_tensor(x), idx, w2, e, d, 1.5, lg, top_k=k, t=t)
    torch.cuda.synchronize()
    assert torch.equal(w, w2)


@pytest.mark.parametrize("seed", range(14))
def test_router_logits_sweep(gpu, oracle, seed):
    """drawn (experts, width, tokens) across the batched router's kernels: the register-tiled one (up to 256
    tokens, widths that are no multiple of 512), the matrix-core walk as a loop (1536, 2560, 3072) and unrolled
    (1024, 2048, 4096), expert counts that leave rows over after the blocks of 32 (100, 258) -- logits bit for
    bit against the one-row order of the checker on sampled tokens, and the selection on top of them"""
    rng0 = np.random.default_rng(0x60A7 + seed)
    e = int(rng0.choice([32, 64, 100, 128, 256, 258, 512]))
    d = int(rng0.choice([512, 1024, 1536, 2048, 2560, 3072, 4096]))
    t = int(rng0.choice([17, 200, 257, 300, 700, 1500]))
    k = int(rng0.choice([2, 6, 8]))
    rng, wr, x = _draw(oracle, f"sweep-{seed}", e, d, t, 0.05)
    bias = rng.uniform_fill(-0.3, 0.3, e)
    fam = ops.FamilyRouters(gpu)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, e), dtype=torch.float32, device="cuda")
    fam.encode_router_top_k(ops.bf16_tensor(wr), ops.bf16_tensor(x), _f32(bias), idx, w, e, d, 1.5, lg,
                            top_k=k, t=t)
    torch.cuda.synchronize()
    lg_h, idx_h, w_h = lg.cpu().numpy(), idx.cpu().numpy().astype(np.uint32), w.cpu().numpy()
    what = f"seed {seed}: e={e} d={d} t={t} k={k}"
    for i in sorted(set([0, 1, 31, 32, t // 2, t - 2, t - 1]) & set(range(t))):
        ref_lg = oracle.router_logits(wr, x[i])
        assert np.array_equal(_bits(lg_h[i]), _bits(ref_lg)), (what, i)
        ri, rw = oracle.router_sqrtsoftplus(ref_lg, bias, k, 1.5)
        assert np.array_equal(idx_h[i], ri), (what, i)
        assert np.array_equal(_bits(w_h[i]), _bits(rw)), (what, i)


@pytest.mark.parametrize("e", [8, 16, 24, 33, 100, 128, 168, 255, 256])
def test_sqrtsoftplus_ties_match_serial(gpu, oracle, e):
    """RouterTopKParityTests.swift:52-77: tie-heavy logits and duplicated correction biases"""
    rng = oracle.Rng(0x5EED0002 + e)
    fam = ops.FamilyRouters(gpu)
    k = 6
    for trial in range(12):
        logits = _tie_logits(e, trial, rng)
        bias = np.array([np.float32((i // 7) % 4) * np.float32(0.25) if trial % 3 == 0
                         else rng.uniform(-0.3, 0.3) for i in range(e)], np.float32)
        wr, x, lg_ref = _one_hot_router(oracle, logits[None, :])
        idx = torch.zeros((1, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((1, k), dtype=torch.float32, device="cuda")
        lg = torch.zeros((1, e), dtype=torch.float32, device="cuda")
        fam.encode_router_top_k(ops.bf16_tensor(wr), ops.bf16_tensor(x), _f32(bias), idx, w, e, 64, 2.5, lg)
        torch.cuda.synchronize()
        ri, rw = oracle.router_sqrtsoftplus(lg_ref[0], bias, k, 2.5)
        assert np.array_equal(idx[0].cpu().numpy().astype(np.uint32), ri), (e, trial)
        assert np.array_equal(_bits(w[0].cpu().numpy()), _bits(rw)), (e, trial)


def test_sqrtsoftplus_and_log_device_functions_bit_exact(gpu, oracle):
    """a sweep of logit values through the hash form with one expert per token: weight = route_scale *
    s / (s + 1e-20) exposes nothing, so use two experts (the value and a fixed 0.0) and compare bits"""
    vals = np.concatenate([np.linspace(-30, 30, 1501), np.array([0.0, -0.0, 1e-6, -1e-6, 87.0, -87.0, 1e4])])
    vals = oracle.bf16_to_float(oracle.bf16_bits(vals.astype(np.float32)))
    t = vals.size
    fam = ops.FamilyRouters(gpu)
    wr = np.zeros((2, 64), np.uint16)
    wr[0, 0] = 0x3F80
    x = np.zeros((t, 64), np.uint16)
    x[:, 0] = oracle.bf16_bits(vals)
    given = torch.tensor([[0, 1]] * t, dtype=torch.int32, device="cuda")
    w = torch.zeros((t, 2), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, 2), dtype=torch.float32, device="cuda")
    fam.encode_router_hash_weights(ops.bf16_tensor(wr), ops.bf16_tensor(x), given, w, 2, 64, 1.0, lg, top_k=2, t=t)
    torch.cuda.synchronize()
    w_h = w.cpu().numpy()
    for i in range(t):
        rw = oracle.router_hash_weights(np.array([vals[i], 0.0], np.float32), [0, 1], 1.0)
        assert np.array_equal(_bits(w_h[i]), _bits(rw)), (vals[i], w_h[i], rw)


def test_hash_router_repeats_and_out_of_range(gpu, oracle):
    e, d, k, t = 256, 512, 6, 12
    rng, wr, x = _draw(oracle, "hash", e, d, t, 0.05)
    fam = ops.FamilyRouters(gpu)
    r2 = oracle.Rng(0x5EED0003)  # RouterTopKParityTests.swift:81-104
    given = np.array([[(s % 2) * 17 if trial % 4 == 0 else r2.next() % e for s in range(k)]
                      for trial in range(t)], np.uint32)
    given[5, 2] = e + 3  # past the table: weight 0, the others renormalise without it
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, e), dtype=torch.float32, device="cuda")
    fam.encode_router_hash_weights(ops.bf16_tensor(wr), ops.bf16_tensor(x),
                                   torch.from_numpy(given.astype(np.int32)).cuda(), w, e, d, 2.5, lg, t=t)
    torch.cuda.synchronize()
    w_h = w.cpu().numpy()
    for i in range(t):
        ref_lg = oracle.router_logits(wr, x[i])
        if i == 5:
            keep = [j for j in range(k) if j != 2]
            rw = oracle.router_hash_weights(ref_lg, given[i, keep], 2.5)
            assert w_h[i, 2] == 0.0
            assert np.abs(w_h[i, keep] - rw).max() <= 1e-6
        else:
            assert np.array_equal(_bits(w_h[i]), _bits(oracle.router_hash_weights(ref_lg, given[i], 2.5)))


@pytest.mark.parametrize("n_routed,n_shared,d,k,t", [(256, 2, 1024, 8, 1), (256, 2, 2048, 8, 5), (100, 1, 512, 6, 3),
                                                     (64, 0, 256, 4, 2), (256, 2, 1024, 8, 200), (256, 2, 2048, 8, 300),
                                                     (100, 1, 512, 6, 290)])
def test_inkling_router_bit_exact(gpu, oracle, n_routed, n_shared, d, k, t):
    rows = n_routed + n_shared
    rng, wr, x = _draw(oracle, f"inkling-{rows}-{d}-{k}-{t}", rows, d, t, 0.05)
    bias = rng.uniform_fill(-0.2, 0.2, n_routed)
    fam = ops.FamilyRouters(gpu)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    gam = torch.zeros((t, max(n_shared, 1)), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, rows), dtype=torch.float32, device="cuda")
    gs = _f32(np.array([0.75]))
    fam.encode_router_inkling(ops.bf16_tensor(wr), ops.bf16_tensor(x), _f32(bias), gs, idx, w,
                              gam if n_shared else None, n_routed, n_shared, k, 2.5, d, lg, t=t)
    torch.cuda.synchronize()
    idx_h, w_h, gam_h = idx.cpu().numpy().astype(np.uint32), w.cpu().numpy(), gam.cpu().numpy()
    lg_h = lg.cpu().numpy()
    for i in list(range(min(t, 8))) + ([t - 1, t // 2, 33] if t > 40 else []):
        ref_lg = oracle.router_logits(wr, x[i])
        assert np.array_equal(_bits(lg_h[i]), _bits(ref_lg))
        ri, rw, rg = oracle.router_inkling(ref_lg, bias, 0.75, n_routed, n_shared, k, 2.5)
        assert np.array_equal(idx_h[i], ri)
        assert np.array_equal(_bits(w_h[i]), _bits(rw))
        if n_shared:
            assert np.array_equal(_bits(gam_h[i].reshape(-1)[:n_shared]), _bits(rg))


def test_inkling_ties(gpu, oracle):
    rng = oracle.Rng(0x1A2B3C)
    fam = ops.FamilyRouters(gpu)
    n_routed, n_shared, k = 256, 2, 8
    for trial in range(12):
        logits = _tie_logits(n_routed + n_shared, trial, rng)
        bias = np.full(n_routed, 0.125, np.float32) if trial % 3 == 0 else \
            np.array([rng.uniform(-0.2, 0.2) for _ in range(n_routed)], np.float32)
        wr, x, lg_ref = _one_hot_router(oracle, logits[None, :])
        idx = torch.zeros((1, k), dtype=torch.int32, device="cuda")
        w = torch.zeros((1, k), dtype=torch.float32, device="cuda")
        gam = torch.zeros((1, n_shared), dtype=torch.float32, device="cuda")
        lg = torch.zeros((1, n_routed + n_shared), dtype=torch.float32, device="cuda")
        fam.encode_router_inkling(ops.bf16_tensor(wr), ops.bf16_tensor(x), _f32(bias), _f32(np.array([1.25])),
                                  idx, w, gam, n_routed, n_shared, k, 1.0, 64, lg)
        torch.cuda.synchronize()
        ri, rw, rg = oracle.router_inkling(lg_ref[0], bias, 1.25, n_routed, n_shared, k, 1.0)
        assert np.array_equal(idx[0].cpu().numpy().astype(np.uint32), ri), trial
        assert np.array_equal(_bits(w[0].cpu().numpy()), _bits(rw))
        assert np.array_equal(_bits(gam[0].cpu().numpy()), _bits(rg))


@pytest.mark.parametrize("e,d,k,t,shift", [(128, 2816, 8, 1, 0), (128, 2816, 8, 3, 0), (24, 256, 8, 2, 0),
                                           (128, 2816, 8, 2, 1), (256, 1024, 4, 150, 0), (128, 2816, 8, 40, 0),
                                           (66, 4096, 8, 33, 0), (24, 256, 8, 20, 0), (128, 2816, 8, 20, 1)])
def test_gemma4_router_bit_exact(gpu, oracle, e, d, k, t, shift):
    """8-bit affine router rows; shift = 1 hands over pointers that are only 1- / 2-byte aligned"""
    rng = oracle.Rng.key(ROOT_SEED + 0xFA32, f"gemma4-{e}-{d}-{k}-{t}")
    codes = np.array([rng.next() % 256 for _ in range(e * d)], np.uint8).reshape(e, d)
    scales = oracle.bf16_bits(rng.uniform_fill(0.0002, 0.0008, e * d // 64).reshape(e, d // 64))
    biases = oracle.bf16_bits(rng.uniform_fill(-0.08, -0.04, e * d // 64).reshape(e, d // 64))
    x = oracle.bf16_bits(rng.normal(0.0, 1.0, t * d).reshape(t, d))
    eff = oracle.bf16_bits(rng.uniform_fill(0.5, 1.5, d))
    pes = oracle.bf16_bits(rng.uniform_fill(0.6, 1.4, e))

    def dev_u8(a):
        buf = torch.zeros(a.size + 16, dtype=torch.uint8, device="cuda")
        buf[shift:shift + a.size] = torch.from_numpy(a.reshape(-1)).cuda()
        return buf[shift:shift + a.size]

    def dev_bf16(a):
        buf = torch.zeros(a.size + 16, dtype=torch.bfloat16, device="cuda")
        buf[shift:shift + a.size] = ops.bf16_tensor(a.reshape(-1))
        return buf[shift:shift + a.size]

    fam = ops.FamilyRouters(gpu)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, e), dtype=torch.float32, device="cuda")
    fam.encode_router_gemma4(dev_u8(codes), dev_bf16(scales), dev_bf16(biases), dev_bf16(x), dev_bf16(eff),
                             dev_bf16(pes), idx, w, e, d, k, lg, t=t)
    torch.cuda.synchronize()
    lg_h, idx_h, w_h = lg.cpu().numpy(), idx.cpu().numpy().astype(np.uint32), w.cpu().numpy()
    for i in list(range(min(t, 6))) + ([t - 1] if t > 6 else []):
        ref_lg = oracle.router_logits_int8(codes, scales, biases, x[i], eff)
        assert np.array_equal(_bits(lg_h[i]), _bits(ref_lg))
        ri, rw = oracle.topk_softmax_scaled(ref_lg, pes, k)
        assert np.array_equal(idx_h[i], ri)
        assert np.array_equal(_bits(w_h[i]), _bits(rw))


def test_family_router_argument_errors(gpu):
    fam = ops.FamilyRouters(gpu)
    z16 = torch.zeros(4096, dtype=torch.bfloat16, device="cuda")
    zf = torch.zeros(4096, dtype=torch.float32, device="cuda")
    zi = torch.zeros(64, dtype=torch.int32, device="cuda")
    with pytest.raises(ops.MfError) as e1:
        fam.encode_router_top_k(z16, z16, zf, zi, zf, 16, 64, 1.0, zf, top_k=9)
    assert e1.value.status == -11
    with pytest.raises(ops.MfError) as e2:
        fam.encode_router_top_k(z16, z16, zf, zi, zf, 513, 64, 1.0, zf)
    assert e2.value.status == -12
    with pytest.raises(ops.MfError) as e3:
        fam.encode_router_top_k(z16, z16, zf, zi, zf, 16, 12, 1.0, zf)
    assert e3.value.status == -1
    with pytest.raises(ops.MfError) as e4:
        fam.encode_router_inkling(z16, z16, zf, zf, zi, zf, zf, 16, 9, 4, 1.0, 64, zf)
    assert e4.value.status == -1
    with pytest.raises(ops.MfError) as e5:
        fam.encode_router_gemma4(torch.zeros(4096, dtype=torch.uint8, device="cuda"), z16, z16, z16, z16, z16,
                                 zi, zf, 16, 72, 8, zf)
    assert e5.value.status == -2
    with pytest.raises(ops.MfError) as e6:
        fam.encode_router_hash_weights(z16, z16, None, zf, 16, 64, 1.0, zf)
    assert e6.value.status == -1


def test_row_counts_beyond_the_limit_are_refused(gpu):
    """MF_MAX_ROWS (2^20) bounds t in every batched call: a larger count is an argument error and nothing
    is launched (the buffers here are far too small for such a call)."""
    too_many = (1 << 20) + 1
    fam = ops.FamilyRouters(gpu)
    z16 = torch.zeros(4096, dtype=torch.bfloat16, device="cuda")
    zf = torch.zeros(4096, dtype=torch.float32, device="cuda")
    zi = torch.zeros(64, dtype=torch.int32, device="cuda")
    with pytest.raises(ops.MfError) as err:
        fam.encode_router_top_k(z16, z16, zf, zi, zf, 16, 64, 1.0, zf, t=too_many)
    assert err.value.status == -1
    moe = ops.MoE(gpu, 64, 64, 16, 2, bits=4)
    offsets, blob_bytes, stride = ops.expert_blob_layout(64, 64, 4)
    experts = torch.zeros((16, stride), dtype=torch.uint8, device="cuda")
    calls = [
        lambda: moe.encode_router(z16, z16, zi, zf, t=too_many),
        lambda: moe.encode_routed_phase1(experts, offsets, zi, z16, z16, t=too_many),
        lambda: moe.encode_routed_phase2_reduce(experts, offsets, zi, zf, z16, None, z16, t=too_many),
    ]
    for call in calls:
        with pytest.raises(ops.MfError) as err:
            call()
        assert err.value.status == -1
    torch.cuda.synchronize()


def test_sqrtsoftplus_routing_feeds_the_two_phase_layer(gpu, oracle):
    """a 2-bit layer routed by the DeepSeek-V4 selector: router -> phase 1 -> phase 2 through the ABI
    against the checker's composition of the same parts"""
    d, f, e, k, t = 512, 256, 32, 6, 2
    root = ROOT_SEED + 0x4D5
    layer = oracle.synth_layer(root, d, f, e, k, bits=2, fs=0)
    x = oracle.synth_x(root, t, d)
    rng = oracle.Rng.key(root, "correction-bias")
    bias = rng.uniform_fill(-0.3, 0.3, e)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    fam = ops.FamilyRouters(gpu)
    xd = ops.bf16_tensor(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, e), dtype=torch.float32, device="cuda")
    acts = torch.zeros((t, k, f), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    fam.encode_router_top_k(wts.router_w, xd, _f32(bias), idx, w, e, d, 1.5, lg, top_k=k, t=t)
    moe.encode_routed_phase1(wts.experts, wts.offsets, idx, xd, acts, t=t)
    moe.encode_routed_phase2_reduce(wts.experts, wts.offsets, idx, w, acts, None, y, t=t)
    torch.cuda.synchronize()
    for i in range(t):
        ri, rw = oracle.router_sqrtsoftplus(oracle.router_logits(layer.router_w, x[i]), bias, k, 1.5)
        assert np.array_equal(idx[i].cpu().numpy().astype(np.uint32), ri)
        acc = np.zeros(d, np.float32)
        for s in range(k):
            a = oracle.expert_phase1(layer.experts[ri[s]], layer.off, 2, d, f, x[i])
            acc = acc + rw[s] * oracle.expert_down(layer.experts[ri[s]], layer.off, 2, d, f, a)
        ref = oracle.bf16_to_float(oracle.bf16_bits(acc))
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y[i])), ref, f"sqrtsoftplus layer row {i}")


def _layer_io(layer, t, oracle, root):
    x = oracle.synth_x(root, t, layer.d)
    return x, ops.bf16_tensor(x), torch.zeros((t, layer.d), dtype=torch.bfloat16, device="cuda")


def test_decode_layer_with_given_routing_equals_own_routing(gpu, oracle):
    """router_w = NULL: the layer reads the caller's routing; handing back the routing the layer's own
    router produced must give the same bits as the chain of launches"""
    root = ROOT_SEED + 0x4D6
    layer = oracle.synth_layer(root, 256, 128, 32, 8, bits=4, fs=128)
    t = 5
    x, xd, y0 = _layer_io(layer, t, oracle, root)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    idx = torch.zeros((t, layer.k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, layer.k), dtype=torch.float32, device="cuda")
    moe.set_fused(False)
    moe.encode_decode_layer(wts, xd, y0, t=t, out_indices=idx, out_weights=w)
    torch.cuda.synchronize()
    idx_before, w_before = idx.clone(), w.clone()
    given = ops.MoELayerWeights(router_w=None, experts=wts.experts, offsets=wts.offsets, shared=wts.shared,
                                w_sg=wts.w_sg)
    y1 = torch.zeros_like(y0)
    for fused in (True, False):  # the fused launch skips its router rows and top-k; the chain its two launches
        moe.set_fused(fused)
        y1.zero_()
        moe.encode_decode_layer(given, xd, y1, t=t, out_indices=idx, out_weights=w)
        moe.status()
        assert torch.equal(y0.view(torch.int16), y1.view(torch.int16)), fused
        assert torch.equal(idx, idx_before) and torch.equal(w, w_before)
    moe.set_fused(True)
    moe.encode_decode_layer(wts, xd, y1, t=t)  # and the handle still routes by itself afterwards
    moe.status()
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    ref_y, _, _ = oracle.moe_layer(layer, x)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y1)), oracle.bf16_to_float(ref_y), "given routing")
    with pytest.raises(ops.MfError) as err:  # no router and no routing
        moe.encode_decode_layer(given, xd, y1, t=t)
    assert err.value.status == -1


def test_prefill_layer_with_given_routing_equals_own_routing(gpu, oracle):
    root = ROOT_SEED + 0x4D7
    layer = oracle.synth_layer(root, 512, 256, 32, 8, bits=4, fs=256)
    t = 90
    x, xd, y0 = _layer_io(layer, t, oracle, root)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    idx = torch.zeros((t, layer.k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, layer.k), dtype=torch.float32, device="cuda")
    ws = moe.encode_prefill_layer(wts, xd, y0, t, out_indices=idx, out_weights=w)
    torch.cuda.synchronize()
    given = ops.MoELayerWeights(router_w=None, experts=wts.experts, offsets=wts.offsets, shared=wts.shared,
                                w_sg=wts.w_sg)
    y1 = torch.zeros_like(y0)
    moe.encode_prefill_layer(given, xd, y1, t, workspace=ws, out_indices=idx, out_weights=w)
    torch.cuda.synchronize()
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    with pytest.raises(ops.MfError) as err:
        moe.encode_prefill_layer(given, xd, y1, t, workspace=ws)
    assert err.value.status == -1


def test_two_bit_layer_routed_by_sqrtsoftplus_prefill_equals_decode(gpu, oracle):
    """the DeepSeek-V4 form end to end: learned sqrtsoftplus routing for 70 tokens, then the ragged
    prefill layer and the decode layer on that routing agree within the layer tolerance"""
    root = ROOT_SEED + 0x4D8
    layer = oracle.synth_layer(root, 512, 256, 32, 6, bits=2, fs=256)
    t = 70
    x, xd, y_pre = _layer_io(layer, t, oracle, root)
    bias = oracle.Rng.key(root, "correction-bias").uniform_fill(-0.3, 0.3, layer.e)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    fam = ops.FamilyRouters(gpu)
    idx = torch.zeros((t, layer.k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, layer.k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, layer.e), dtype=torch.float32, device="cuda")
    fam.encode_router_top_k(wts.router_w, xd, _f32(bias), idx, w, layer.e, layer.d, 1.5, lg, top_k=layer.k, t=t)
    given = ops.MoELayerWeights(router_w=None, experts=wts.experts, offsets=wts.offsets, shared=wts.shared,
                                w_sg=wts.w_sg)
    moe.encode_prefill_layer(given, xd, y_pre, t, out_indices=idx, out_weights=w)
    y_dec = torch.zeros_like(y_pre)
    for t0 in range(0, t, 8):
        n = min(8, t - t0)
        moe.encode_decode_layer(given, xd[t0:t0 + n], y_dec[t0:t0 + n], t=n, out_indices=idx[t0:t0 + n],
                                out_weights=w[t0:t0 + n])
    torch.cuda.synchronize()
    ri, _ = oracle.router_sqrtsoftplus(oracle.router_logits(layer.router_w, x[3]), bias, layer.k, 1.5)
    assert np.array_equal(idx[3].cpu().numpy().astype(np.uint32), ri)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y_pre)), oracle.bf16_to_float(ops.bf16_bits(y_dec)),
                       "prefill vs decode on sqrtsoftplus routing")
    assert float(y_pre.float().abs().max()) > 0
