"""GPU parity of the two halves of the ragged layer as calls of their own:
mf_moe_ragged_qmm (PrefillGroupedRoutedMoE.encodeStreamedBatched over a grouping the caller
holds) and mf_moe_unpermute (PrefillMoE.encodeReduceTokenMajor).  The routed matmuls are checked
against a float64 closed form over the reference test's synthetic expert pool
(PrefillGroupedRoutedMoETests.swift:207-303, its skewed 256-route fixture :7-30) and against the
per-route oracle; the reduction against the oracle's restatement of cpuReduce
(PrefillMoETests.swift:46-64)."""
import numpy as np
import pytest
import torch

from mference_amd import _capi
from mference_amd import operators as ops
from helpers import ROOT_SEED, assert_layer_close, make_moe, to_device_layer

pytestmark = pytest.mark.gpu


def _offsets(src) -> ops.MoEExpertOffsets:
    off = ops.MoEExpertOffsets()
    for name, _ in off._fields_:
        setattr(off, name, getattr(src, name))
    return off


def _group(moe, idx, w, t, k, e):
    sorted_pairs = torch.zeros((t * k, 4), dtype=torch.int32, device="cuda")
    offsets = torch.zeros(e, dtype=torch.int32, device="cuda")
    counts = torch.zeros(e, dtype=torch.int32, device="cuda")
    moe.encode_group(torch.from_numpy(idx.astype(np.int32)).cuda(), torch.from_numpy(w).cuda(), t,
                     sorted_pairs, offsets, counts)
    moe.group_status()
    return sorted_pairs, counts


def _synthetic_rows(rows, cols, expert, role):
    """The reference test's weight pattern (PrefillGroupedRoutedMoETests.swift:207-217)."""
    r = np.arange(rows, dtype=np.float32)[:, None]
    c = np.arange(cols, dtype=np.float32)[None, :]
    return (np.float32(expert + 1) * np.float32(0.001) + np.float32(role + 1) * np.float32(0.003)
            + (np.mod(r, 7) - 3) * np.float32(0.0004) + (np.mod(c, 11) - 5) * np.float32(0.0002)).astype(np.float32)


def test_ragged_qmm_synthetic_pool_closed_form(gpu, oracle):
    """The reference fixture's routing (32 tokens x 8 ranks: experts 0..15 with 15 or 14 routes,
    expert 16 with 27) over its synthetic pool.  Expected values: float64 arithmetic on the
    dequantised weights, SiLU(gate) * up rounded to bf16 between the two projections (the
    activation row is a bf16 buffer), in the row order token * top_k + rank.  Rows of routes that
    are not in the grouping keep their fill value (-99 in the reference's check)."""
    d, f, e, k, t = 256, 128, 128, 8, 32
    assign = np.concatenate([np.repeat(np.arange(16), [15] * 5 + [14] * 11), np.full(27, 16)]).astype(np.uint32)
    assert assign.size == 256
    idx = assign.reshape(t, k)
    w = np.tile((0.125 + np.arange(k) * 0.0625).astype(np.float32), (t, 1))
    off, blob, stride = oracle.blob_layout(d, f, 4)
    pool = np.zeros((e, stride), np.uint8)
    deq = {}
    for ex in range(17):  # only experts 0..16 are routed to; the rest of the pool stays zero
        q = [oracle.quantize(_synthetic_rows(f, d, ex, 0)), oracle.quantize(_synthetic_rows(f, d, ex, 1)),
             oracle.quantize(_synthetic_rows(d, f, ex, 2))]
        oracle.pack_expert_blob(q[0], q[1], q[2], off, pool[ex])
        deq[ex] = [oracle.dequantize(z).astype(np.float64) for z in q]
    rng = np.random.default_rng(ROOT_SEED + 77)
    x_bits = oracle.bf16_bits((rng.standard_normal((t, d)) * 0.5).astype(np.float32))
    x = oracle.bf16_to_float(x_bits).astype(np.float64)

    moe = ops.MoE(gpu, d, f, e, k)
    sorted_pairs, counts = _group(moe, idx, w, t, k, e)
    partials = torch.full((t * k, d), -99.0, dtype=torch.float32, device="cuda")
    experts = torch.from_numpy(pool).cuda()
    moe.encode_streamed_batched(experts, _offsets(off), ops.bf16_tensor(x_bits), sorted_pairs, counts, partials, t)
    moe.group_status()
    got = partials.cpu().numpy()

    want = np.empty((t * k, d), np.float64)
    for tok in range(t):
        for r in range(k):
            g, u, dn = deq[int(idx[tok, r])]
            gv, uv = g @ x[tok], u @ x[tok]
            act = gv / (1.0 + np.exp(-gv)) * uv
            act = oracle.bf16_to_float(oracle.bf16_bits(act.astype(np.float32))).astype(np.float64)
            want[tok * k + r] = dn @ act
    err = np.max(np.abs(got - want))
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    # fp32 accumulation over K <= 256 of bf16-exact products against float64: far inside the layer tolerance
    assert err <= 2e-3 and rel <= 1e-3, (err, rel)

    # a grouping of fewer routes leaves the other rows alone: drop expert 16's run (the last one)
    counts2 = counts.clone()
    counts2[16] = 0
    partials2 = torch.full((t * k, d), -99.0, dtype=torch.float32, device="cuda")
    moe.encode_streamed_batched(experts, _offsets(off), ops.bf16_tensor(x_bits), sorted_pairs, counts2, partials2, t)
    got2 = partials2.cpu().numpy()
    dropped = (idx.reshape(-1) == 16)
    assert np.all(got2[dropped] == -99.0)
    assert np.array_equal(got2[~dropped], got[~dropped])


@pytest.mark.parametrize("bits,d,f,e,k,t,mode", [(4, 512, 256, 32, 8, 200, 0), (2, 256, 128, 16, 4, 70, 0),
                                                 (1, 512, 256, 32, 4, 64, 1), (4, 2048, 512, 256, 8, 96, 0)])
def test_ragged_qmm_then_unpermute_is_the_layer_call(gpu, oracle, bits, d, f, e, k, t, mode):
    """group -> ragged matmuls -> un-permute, as three calls, gives the bits of the one layer call
    (no shared expert), and every route's row matches the per-route oracle."""
    root = ROOT_SEED + 0xB000 + d + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=0, router_mode=mode)
    x = oracle.synth_x(root, t, d)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    moe.encode_prefill_layer(wts, xd, y, t, out_indices=idx, out_weights=w)

    sorted_pairs = torch.zeros((t * k, 4), dtype=torch.int32, device="cuda")
    offsets = torch.zeros(e, dtype=torch.int32, device="cuda")
    counts = torch.zeros(e, dtype=torch.int32, device="cuda")
    moe.encode_group(idx, w, t, sorted_pairs, offsets, counts)
    moe.group_status()
    partials = torch.zeros((t * k, d), dtype=torch.float32, device="cuda")
    moe.encode_streamed_batched(wts.experts, wts.offsets, xd, sorted_pairs, counts, partials, t)
    moe.group_status()
    y2 = torch.zeros_like(y)
    moe.encode_reduce_token_major(partials, w, y2, t, indices=idx)
    torch.cuda.synchronize()
    assert np.array_equal(ops.bf16_bits(y), ops.bf16_bits(y2))

    got = partials.cpu().numpy()
    idx_h = idx.cpu().numpy()
    rng = np.random.default_rng(t)
    for tok in rng.choice(t, size=6, replace=False):
        for r in range(k):
            ex = int(idx_h[tok, r])
            acts = oracle.expert_phase1(layer.experts[ex], layer.off, bits, d, f, x[tok])
            ref = oracle.expert_down(layer.experts[ex], layer.off, bits, d, f, acts)
            assert_layer_close(got[tok * k + r], ref, f"route token={tok} rank={r} expert={ex}")


def test_unpermute_matches_cpu_reduce(gpu, oracle):
    """Random partials and weights against the oracle's restatement of the reference test's
    cpuReduce; then with a residual to start from and with routes that name no expert."""
    t, k, d, e = 37, 6, 384, 16
    rng = np.random.default_rng(ROOT_SEED + 5)
    partials = rng.standard_normal((t, k, d)).astype(np.float32)
    w = rng.random((t, k), dtype=np.float32)
    moe = ops.MoE(gpu, d, 128, e, k)
    pd = torch.from_numpy(partials.reshape(t * k, d)).cuda()
    wd = torch.from_numpy(w).cuda()
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_reduce_token_major(pd, wd, y, t)
    torch.cuda.synchronize()
    ref = oracle.reduce_token_major(partials, w)
    got = oracle.bf16_to_float(ops.bf16_bits(y))
    # the output is bf16: at most one bf16 step from the fp32 sum's rounding
    ref_b = oracle.bf16_to_float(oracle.bf16_bits(ref))
    step = np.maximum(np.abs(ref_b), 1e-30) * 2.0 ** -7
    assert np.all(np.abs(got - ref_b) <= step)
    assert np.mean(got == ref_b) > 0.99

    idx = rng.integers(0, e, size=(t, k)).astype(np.int32)
    idx[3, 2] = e
    idx[9, :] = e
    res = oracle.bf16_bits(rng.standard_normal((t, d)).astype(np.float32))
    y2 = torch.zeros_like(y)
    moe.encode_reduce_token_major(pd, wd, y2, t, indices=torch.from_numpy(idx).cuda(), residual=ops.bf16_tensor(res))
    torch.cuda.synchronize()
    w_live = np.where(idx >= e, np.float32(0), w)
    # fp32, rank order, starting from the residual
    acc = oracle.bf16_to_float(res).astype(np.float32)
    for r in range(k):
        acc = acc + (w_live[:, r:r + 1] * partials[:, r, :]).astype(np.float32)
    want = oracle.bf16_to_float(oracle.bf16_bits(acc))
    got2 = oracle.bf16_to_float(ops.bf16_bits(y2))
    assert np.array_equal(got2[9], oracle.bf16_to_float(res)[9])  # a token without routes keeps its residual
    assert np.all(np.abs(got2 - want) <= np.maximum(np.abs(want), 1e-30) * 2.0 ** -7)


def test_ragged_qmm_refuses_a_grouping_that_does_not_fit(gpu, oracle):
    """Counts that cover more routes than t * top_k, or a pair naming a token past t: nothing is
    computed and the grouping status reports it; a short workspace and an unsupported width are
    refused on the host."""
    d, f, e, k, t = 256, 128, 16, 4, 20
    layer = oracle.synth_layer(ROOT_SEED + 9, d, f, e, k, fs=0)
    x = oracle.synth_x(ROOT_SEED + 9, t, d)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    _, idx, w = oracle.moe_layer(layer, x)
    sorted_pairs, counts = _group(moe, idx, w, t, k, e)
    xd = ops.bf16_tensor(x)
    partials = torch.full((t * k, d), -7.0, dtype=torch.float32, device="cuda")

    big = counts.clone()
    big[0] += t * k
    moe.encode_streamed_batched(wts.experts, wts.offsets, xd, sorted_pairs, big, partials, t)
    with pytest.raises(_capi.MfError) as err:
        moe.group_status()
    assert err.value.status == -17
    assert torch.all(partials == -7.0).item()

    wrong = sorted_pairs.clone()
    wrong[5, 0] = t  # token out of range
    moe.encode_streamed_batched(wts.experts, wts.offsets, xd, wrong, counts, partials, t)
    with pytest.raises(_capi.MfError):
        moe.group_status()
    assert torch.all(partials == -7.0).item()

    moe.encode_streamed_batched(wts.experts, wts.offsets, xd, sorted_pairs, counts, partials, t)
    moe.group_status()  # re-armed by the next call
    assert not torch.any(partials == -7.0).item()

    short = torch.empty(64, dtype=torch.uint8, device="cuda")
    with pytest.raises(_capi.MfError) as err:
        moe.encode_streamed_batched(wts.experts, wts.offsets, xd, sorted_pairs, counts, partials, t, workspace=short)
    assert err.value.status == -4
    odd = ops.MoE(gpu, 192, 64, e, k)  # widths the matmul tiles do not divide
    with pytest.raises(_capi.MfError) as err:
        odd.encode_streamed_batched(wts.experts, wts.offsets, xd, sorted_pairs, counts, partials, t)
    assert err.value.status == -2
    torch.cuda.synchronize()


@pytest.mark.parametrize("bits,d,f,e,k,t", [(4, 512, 256, 32, 8, 200),     # down projection with K = 256 (x tile resident)
                                            (4, 256, 1024, 16, 4, 150),    # ... with K = 1024 (x tile ring)
                                            (2, 256, 128, 16, 4, 70)])
def test_prefill_route_rounding_narrows_every_route(gpu, oracle, bits, d, f, e, k, t):
    """mf_moe_set_prefill_route_rounding(h, 1): the layer call gives, bit for bit, what narrowing the fp32
    per-route results of the ragged call to bf16 and reducing them in rank order gives; it agrees with the
    checker under the same rule; and it differs from the default somewhere."""
    root = ROOT_SEED + 0xB700 + d + f
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=0)
    x = oracle.synth_x(root, t, d)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    xd = ops.bf16_tensor(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    y_wide = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_prefill_layer(wts, xd, y_wide, t, out_indices=idx, out_weights=w)
    moe.set_prefill_route_rounding(True)
    y = torch.zeros_like(y_wide)
    moe.encode_prefill_layer(wts, xd, y, t)
    moe.set_prefill_route_rounding(False)

    sorted_pairs = torch.zeros((t * k, 4), dtype=torch.int32, device="cuda")
    offsets = torch.zeros(e, dtype=torch.int32, device="cuda")
    counts = torch.zeros(e, dtype=torch.int32, device="cuda")
    moe.encode_group(idx, w, t, sorted_pairs, offsets, counts)
    partials = torch.zeros((t * k, d), dtype=torch.float32, device="cuda")
    moe.encode_streamed_batched(wts.experts, wts.offsets, xd, sorted_pairs, counts, partials, t)
    torch.cuda.synchronize()
    moe.group_status()
    q = oracle.bf16_to_float(oracle.bf16_bits(partials.cpu().numpy())).astype(np.float32).reshape(t, k, d)
    w_h = w.cpu().numpy()
    acc = np.zeros((t, d), dtype=np.float32)
    for r in range(k):
        acc = acc + (w_h[:, r:r + 1] * q[:, r, :]).astype(np.float32)
    assert np.array_equal(ops.bf16_bits(y), oracle.bf16_bits(acc))
    assert not np.array_equal(ops.bf16_bits(y), ops.bf16_bits(y_wide))

    layer.narrow_routes = True
    rows = np.random.default_rng(t).choice(t, size=24, replace=False)
    ref_y, ref_idx, _ = oracle.moe_layer(layer, x[rows])
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32)[rows], ref_idx)
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)[rows]), oracle.bf16_to_float(ref_y), "narrow routes")
