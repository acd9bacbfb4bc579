"""GPU parity of the ragged prefill path: device grouping against the oracle's
restatement of PrefillMoEGrouping, and the tokens-sorted-by-expert layer against
the per-token oracle (the reference's own gate for this path: grouped prefill ==
per-token decode, PrefillGroupedRoutedMoETests / PrefillMoETests)."""
import numpy as np
import pytest
import torch

from mference_amd import _capi
from mference_amd import operators as ops
from helpers import ROOT_SEED, assert_layer_close, make_moe, to_device_layer

pytestmark = pytest.mark.gpu


def _group_on_device(moe, idx, w, t, k, e):
    sorted_pairs = torch.zeros((t * k, 4), dtype=torch.int32, device="cuda")
    offsets = torch.zeros(e, dtype=torch.int32, device="cuda")
    counts = torch.zeros(e, dtype=torch.int32, device="cuda")
    moe.encode_group(torch.from_numpy(idx.astype(np.int32)).cuda(), torch.from_numpy(w).cuda(), t,
                     sorted_pairs, offsets, counts)
    return sorted_pairs, offsets, counts


@pytest.mark.parametrize("t,k,e,live", [(1, 8, 16, 16), (37, 4, 16, 16), (300, 8, 256, 256),
                                        (129, 8, 64, 9), (64, 2, 512, 40), (2048, 8, 256, 200),
                                        (1500, 8, 512, 512), (6000, 4, 128, 128)])
def test_device_grouping_matches_oracle(gpu, oracle, t, k, e, live):
    """`live` < e leaves experts without a token: their offset is 0xFFFFFFFF
    (PrefillMoEGrouping.swift:151-160)."""
    rng = np.random.default_rng(t * 1000 + e)
    idx = np.stack([rng.choice(live, size=k, replace=False) for _ in range(t)]).astype(np.uint32)
    w = rng.random((t, k), dtype=np.float32)
    moe = ops.MoE(gpu, 128, 64, e, k)
    sorted_pairs, offsets, counts = _group_on_device(moe, idx, w, t, k, e)
    moe.group_status()
    ref = oracle.group_pairs(oracle.make_pairs(idx, w.view(np.uint32)), t, k, e)
    got = sorted_pairs.cpu().numpy().view(np.uint32)
    assert np.array_equal(got[:, 0], ref["sorted"]["token"])
    assert np.array_equal(got[:, 1], ref["sorted"]["expert"])
    assert np.array_equal(got[:, 2], ref["sorted"]["rank"])
    assert np.array_equal(got[:, 3], ref["sorted"]["weight_bits"])
    assert np.array_equal(offsets.cpu().numpy().view(np.uint32), ref["offsets"])
    assert np.array_equal(counts.cpu().numpy().view(np.uint32), ref["counts"])


@pytest.mark.parametrize("t,k,e", [(40, 4, 16), (700, 8, 64), (2048, 8, 256), (5000, 6, 64)])
def test_device_grouping_with_an_expert_named_twice_in_a_token(gpu, oracle, t, k, e):
    """The reference's grouping takes any pair list; a token may name one expert under two ranks
    (PrefillMoEGrouping.swift:91-192 orders such routes by rank).  The device form -- one workgroup with a
    bit per (expert, token) up to a few thousand tokens, several launches beyond -- keeps that order."""
    rng = np.random.default_rng(t + e)
    idx = rng.integers(0, e, size=(t, k)).astype(np.uint32)   # with replacement: plenty of repeats
    idx[t // 2, :] = 3
    w = rng.random((t, k), dtype=np.float32)
    moe = ops.MoE(gpu, 128, 64, e, k)
    sorted_pairs, offsets, counts = _group_on_device(moe, idx, w, t, k, e)
    moe.group_status()
    ref = oracle.group_pairs(oracle.make_pairs(idx, w.view(np.uint32)), t, k, e)
    got = sorted_pairs.cpu().numpy().view(np.uint32)
    for col, name in enumerate(("token", "expert", "rank", "weight_bits")):
        assert np.array_equal(got[:, col], ref["sorted"][name]), name
    assert np.array_equal(offsets.cpu().numpy().view(np.uint32), ref["offsets"])
    assert np.array_equal(counts.cpu().numpy().view(np.uint32), ref["counts"])


def test_device_grouping_of_no_tokens(gpu):
    """queryCount == 0 is a valid call (PrefillMoEGrouping.swift:99-104): no pairs, every expert
    empty (count 0, offset 0xFFFFFFFF), status clean; an absurd token count is refused."""
    e, k = 24, 4
    moe = ops.MoE(gpu, 128, 64, e, k)
    offsets = torch.full((e,), 7, dtype=torch.int32, device="cuda")
    counts = torch.full((e,), 7, dtype=torch.int32, device="cuda")
    lib = _capi.lib()
    assert lib.mf_moe_group(moe._h, None, None, None, 0, None, offsets.data_ptr(), counts.data_ptr()) == 0
    moe.group_status()
    assert np.all(offsets.cpu().numpy().view(np.uint32) == 0xFFFFFFFF)
    assert np.all(counts.cpu().numpy() == 0)
    idx = torch.zeros((1, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((1, k), dtype=torch.float32, device="cuda")
    sp = torch.zeros((k, 4), dtype=torch.int32, device="cuda")
    assert lib.mf_moe_group(moe._h, None, idx.data_ptr(), w.data_ptr(), (1 << 20) + 1, sp.data_ptr(),
                            offsets.data_ptr(), counts.data_ptr()) == -10
    torch.cuda.synchronize()


def test_device_grouping_flags_expert_out_of_range(gpu):
    t, k, e = 9, 4, 16
    idx = np.tile(np.arange(k, dtype=np.uint32), (t, 1))
    idx[5, 2] = e + 3
    w = np.ones((t, k), np.float32)
    moe = ops.MoE(gpu, 128, 64, e, k)
    _group_on_device(moe, idx, w, t, k, e)
    with pytest.raises(_capi.MfError) as err:
        moe.group_status()
    assert err.value.status == -17
    idx[5, 2] = 1  # the status word is re-armed by the next call
    _group_on_device(moe, idx, w, t, k, e)
    moe.group_status()


def _run_prefill(moe, wts, x, t, d, k):
    xd = ops.bf16_tensor(x)
    y = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, k), dtype=torch.float32, device="cuda")
    moe.encode_prefill_layer(wts, xd, y, t, out_indices=idx, out_weights=w)
    torch.cuda.synchronize()
    return ops.bf16_bits(y), idx.cpu().numpy().astype(np.uint32), w.cpu().numpy()


@pytest.mark.parametrize("bits,d,f,e,k,fs,t,mode,limit", [
    (4, 256, 128, 16, 4, 0, 5, 0, 0.0),        # fewer tokens than a tile, no shared expert
    (4, 256, 128, 16, 4, 128, 70, 0, 0.0),     # one full tile + a ragged tail per busy expert
    (4, 512, 256, 32, 8, 256, 200, 0, 7.0),    # SwiGLU clamp (moe.metal:1080-1094)
    (4, 384, 128, 32, 2, 128, 131, 1, 0.0),    # full-softmax router, ng not a multiple of 8
    (4, 2048, 512, 256, 8, 512, 96, 0, 0.0),   # the headline layer shape
    (4, 512, 256, 16, 4, 128, 90, 0, 0.0),     # shared width != routed width: the two down projections differ in K
    (4, 256, 384, 16, 4, 384, 67, 0, 0.0),     # K of the down projection not 128, 256 or 512
    # 2-bit routed experts with a 4-bit shared expert (the shared matmuls are launches of their own)
    (2, 256, 128, 16, 4, 128, 70, 0, 0.0),
    (2, 512, 256, 32, 6, 256, 200, 0, 7.0),    # top-6 + SwiGLU clamp (moe.metal:902-1195)
    (2, 1024, 512, 16, 6, 0, 133, 0, 0.0),     # K a multiple of 512 (whole-table vector loads), no shared expert
    (2, 384, 384, 16, 2, 128, 45, 0, 0.0),     # neither down projection has K of 128, 256 or 512
    # ternary experts, scale-only tables, full-softmax router (maple_moe.metal:62-265)
    (1, 256, 128, 32, 8, 0, 131, 1, 0.0),
    (1, 512, 256, 32, 4, 0, 64, 1, 0.0),
    (1, 1024, 512, 64, 8, 0, 77, 1, 0.0),
])
def test_prefill_layer_matches_per_token_oracle(gpu, oracle, bits, d, f, e, k, fs, t, mode, limit):
    root = ROOT_SEED + 0xA000 + d + t + 0x10000 * (4 - bits)
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=mode, swiglu_limit=limit)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y, idx, w = _run_prefill(moe, wts, x, t, d, k)
    assert np.array_equal(idx, ref_idx)
    assert np.array_equal(w.view(np.uint32), ref_w.view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(y), oracle.bf16_to_float(ref_y),
                       f"prefill layer bits={bits} d={d} f={f} e={e} k={k} t={t}")
    # a second call into the same workspace-free handle gives the same bits (no stale state)
    y2, _, _ = _run_prefill(moe, wts, x, t, d, k)
    assert np.array_equal(y, y2)


_SKEWED = {}


def _skewed_qwen_layer(oracle):
    """the benchmark's layer: Qwen3.6-shaped, and a per-expert router bias ~ N(0, 1.5) carried by the last
    router column against a constant-one last feature of x, so that expert loads are uneven and many experts
    get no token"""
    if not _SKEWED:
        root = ROOT_SEED + 0xA000 + 0x5CE
        layer = oracle.synth_layer(root, 2048, 512, 256, 8, bits=4, fs=512)
        bias = oracle.Rng.key(root, "router.bias").normal(0.0, 1.5, 256)
        layer.router_w[:, -1] = oracle.bf16_bits(bias)
        _SKEWED["layer"] = layer
        _SKEWED["root"] = root
    return _SKEWED["layer"], _SKEWED["root"]


@pytest.mark.parametrize("t", [128, 512, 2048])
def test_skewed_qwen_prefill_against_the_checker(gpu, oracle, t):
    """The headline prefill configuration at its three token counts, directly against the per-token checker:
    routing indices and weights bit for bit on every row, the layer output within tolerance on 64 sampled rows
    (the busiest expert takes most tokens here, so full 64-route tiles, ragged tails and experts without
    tokens all occur in one call)."""
    layer, root = _skewed_qwen_layer(oracle)
    d, k = layer.d, layer.k
    x = oracle.synth_x(root + t, t, d)
    x[:, -1] = 0x3F80
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    # (the form the benchmark reports: the routed experts read from the tiled copy of the pool)
    wts.experts_tiled = moe.tile_experts(wts.experts, wts.offsets)
    y, idx, w = _run_prefill(moe, wts, x, t, d, k)
    rows = np.unique(np.concatenate([np.arange(8), np.arange(t - 8, t),
                                     np.random.default_rng(t).choice(t, size=48, replace=False)]))
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x[rows])
    assert np.array_equal(idx[rows], ref_idx)
    assert np.array_equal(w[rows].view(np.uint32), ref_w.view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(y[rows]), oracle.bf16_to_float(ref_y), f"skewed qwen prefill t={t}")
    counts = np.bincount(idx.reshape(-1), minlength=layer.e)
    assert (counts == 0).sum() > 0 and counts.max() > t // 2, "the routing of this case is meant to be skewed"


@pytest.mark.parametrize("bits,d,f,e,k,fs,t,mode", [
    (4, 512, 256, 32, 8, 256, 1100, 0),    # 8800 routes, the shared expert rides along
    (4, 1024, 128, 16, 8, 0, 1031, 0),     # few experts: long runs, an odd tile out at the end of every run
    (2, 512, 256, 16, 6, 128, 1500, 0),    # 2-bit codes; the 4-bit shared expert is a launch of its own
    (1, 512, 128, 32, 8, 0, 1030, 1),      # ternary rows, full-softmax router
    (4, 128, 128, 100, 3, 0, 3000, 0),     # 94 chunks of 32 tokens (two per wave of the selecting launch), 3 routes each
    (4, 128, 128, 24, 1, 128, 8500, 0),    # 133 chunks of 64 tokens, one route per token
    (4, 128, 128, 512, 2, 0, 16000, 0),    # 250 chunks of 64 tokens, the largest expert count
])
def test_prefill_long_batches_against_the_per_token_oracle(gpu, oracle, bits, d, f, e, k, fs, t, mode):
    """More than a thousand tokens on small layers (long runs per expert, many full tiles, an odd tile at
    the end of every run), checked directly against the per-token checker: routing bit-exact, sampled rows
    within the layer tolerance; and the rows do not depend on their neighbours (the first 300 tokens alone
    give the same bits).  Beyond 8192 routes the layer call selects and groups its routes in two launches
    of its own (chunks of up to 64 tokens, an expert's routes of a chunk as a 64-bit word); the 300-token
    call groups them in one workgroup: the same rows from both."""
    root = ROOT_SEED + 0xA400 + d + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=mode)
    x = oracle.synth_x(root, t, d)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y, idx, w = _run_prefill(moe, wts, x, t, d, k)
    rows = np.random.default_rng(t).choice(t, size=64, replace=False)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x[rows])
    assert np.array_equal(idx[rows], ref_idx)
    assert np.array_equal(w[rows].view(np.uint32), ref_w.view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(y[rows]), oracle.bf16_to_float(ref_y), f"long batch bits={bits} t={t}")
    y_short, _, _ = _run_prefill(moe, wts, x[:300], 300, d, k)
    assert np.array_equal(y_short, y[:300])


@pytest.mark.parametrize("bits,d,f,e,k,t", [(1, 512, 256, 32, 8, 150), (4, 256, 128, 32, 4, 70)])
def test_prefill_layer_with_maple_rounding(gpu, oracle, bits, d, f, e, k, t):
    """MapleMoE's rounding points in the prefill call: the SwiGLU epilogue takes maple_swiglu,
    the reduce narrows every down output to bf16 before its weight"""
    root = ROOT_SEED + 0xAA00 + bits + d
    # sigma keeps |y| below 2, where one bf16 step is still inside the max-abs bar
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, router_mode=1, sigma=0.03, maple_rounding=True)
    x = oracle.synth_x(root, t, d)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y, idx, w = _run_prefill(moe, wts, x, t, d, k)
    assert np.array_equal(idx, ref_idx)
    assert np.array_equal(w.view(np.uint32), ref_w.view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(y), oracle.bf16_to_float(ref_y), f"maple prefill bits={bits}")
    layer.maple_rounding = False
    y0, _, _ = _run_prefill(make_moe(gpu, layer), wts, x, t, d, k)
    assert not np.array_equal(y0, y)


def test_prefill_skewed_routing_and_decode_agreement(gpu, oracle):
    """All tokens identical -> every token takes the same k experts: k groups of
    t routes and e-k empty experts; and the prefill rows agree with the decode
    launch on the same token within the layer tolerance."""
    d, f, e, k, fs, t = 256, 128, 16, 4, 128, 150
    root = ROOT_SEED + 0xA100
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=fs)
    x1 = oracle.synth_x(root, 1, d)
    x = np.repeat(x1, t, axis=0)
    ref_y, ref_idx, _ = oracle.moe_layer(layer, x1)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y, idx, _ = _run_prefill(moe, wts, x, t, d, k)
    assert np.array_equal(idx, np.repeat(ref_idx, t, axis=0))
    assert np.array_equal(y, np.repeat(y[:1], t, axis=0))   # position in a tile does not matter
    assert_layer_close(oracle.bf16_to_float(y[0]), oracle.bf16_to_float(ref_y[0]), "skewed prefill")
    yd = torch.zeros((1, d), dtype=torch.bfloat16, device="cuda")
    moe.encode_decode_layer(wts, ops.bf16_tensor(x1), yd, t=1)
    moe.status()
    assert_layer_close(oracle.bf16_to_float(y[0]), oracle.bf16_to_float(ops.bf16_bits(yd)[0]),
                       "prefill vs decode launch")


def test_prefill_other_widths_take_the_decode_launch(gpu, oracle):
    """widths the matmul tiles do not divide (an intermediate size of 64) have no matrix-core
    path: the call runs the rows through the decode launch eight at a time and gives exactly
    the decode result, and asks for no workspace."""
    for bits, mode in ((4, 0), (2, 0), (1, 1)):
        d, f, e, k, fs, t = 256, 64, 32, 4, 64 if bits != 1 else 0, 19
        layer = oracle.synth_layer(ROOT_SEED + 0xA200 + bits, d, f, e, k, bits=bits, fs=fs, router_mode=mode)
        x = oracle.synth_x(ROOT_SEED + 0xA200 + bits, t, d)
        ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x)
        moe = make_moe(gpu, layer)
        assert moe.prefill_workspace_bytes(t) == 0
        wts = to_device_layer(layer)
        y, idx, w = _run_prefill(moe, wts, x, t, d, k)
        assert np.array_equal(idx, ref_idx)
        assert np.array_equal(w.view(np.uint32), ref_w.view(np.uint32))
        assert_layer_close(oracle.bf16_to_float(y), oracle.bf16_to_float(ref_y), f"prefill bits={bits}")
        yd = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
        xd = ops.bf16_tensor(x)
        for t0 in range(0, t, 8):
            n = min(8, t - t0)
            moe.encode_decode_layer(wts, xd[t0:t0 + n], yd[t0:t0 + n], t=n)
        moe.status()
        assert np.array_equal(y, ops.bf16_bits(yd))


@pytest.mark.parametrize("d,e,t", [(5120, 32, 40), (5120, 32, 300), (4224, 32, 40), (4224, 48, 290),
                                   (5120, 48, 290)])
def test_prefill_rows_wider_than_4096(gpu, oracle, d, e, t):
    """Hidden sizes past 4096: a multiple of 512 takes the matrix-core router for whole blocks of 32
    router rows (rows left over -- e = 48 -- and widths that are no multiple of 512 -- 4224 -- go one wave
    per (token, row)); the matmuls take any multiple of 128 up to 8192.  Routing bit-exact, layer within
    the tolerance."""
    f, k, fs = 128, 4, 128
    root = ROOT_SEED + 0xA300 + d + e + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=4, fs=fs)
    x = oracle.synth_x(root, t, d)
    moe = make_moe(gpu, layer)
    assert moe.prefill_workspace_bytes(t) > 0
    wts = to_device_layer(layer)
    y, idx, w = _run_prefill(moe, wts, x, t, d, k)
    rows = np.arange(t) if t <= 64 else np.random.default_rng(t).choice(t, size=48, replace=False)
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x[rows])
    assert np.array_equal(idx[rows], ref_idx)
    assert np.array_equal(w[rows].view(np.uint32), ref_w.view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(y[rows]), oracle.bf16_to_float(ref_y), f"prefill d={d} e={e} t={t}")


@pytest.mark.parametrize("workload,t", [("dsv4-2bit", 300), ("maple-ternary", 300)])
def test_prefill_other_formats_full_size(gpu, oracle, workload, t):
    """the large 2-bit layer (D 4096, F 2048, E 256, K 6, 4-bit shared 2048) and the ternary layer
    (D 2048, F 1024, E 64, K 8, full-softmax router) at full size through the matrix-core path:
    routing against the CPU checker for every token, sampled rows against the CPU checker and
    against the decode launch of the same token; a second call gives the same bits"""
    import bench
    w = dict(bench.WORKLOADS[workload])
    dev = torch.device("cuda", 0)
    lw = bench.build_stack(gpu, w, 1, dev)[0]
    host = bench.layer_to_host(lw, w)
    mode = ops.ROUTER_FULL_SOFTMAX if w["bits"] == 1 else ops.ROUTER_TOPK_SOFTMAX
    host.router_mode = 1 if w["bits"] == 1 else 0
    moe = ops.MoE(gpu, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                  shared_bits=w["shared_bits"], router_mode=mode, maple_rounding=bool(w.get("maple")))
    assert moe.prefill_workspace_bytes(t) > 0
    gen = torch.Generator(device=dev)
    gen.manual_seed(777)
    d, k = w["d"], w["k"]
    x = torch.randn((t, d), generator=gen, device=dev).to(torch.bfloat16)
    y = torch.zeros_like(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device=dev)
    rw = torch.zeros((t, k), dtype=torch.float32, device=dev)
    ws = moe.encode_prefill_layer(lw, x, y, t, out_indices=idx, out_weights=rw)
    torch.cuda.synchronize()
    sample = [0, 1, 63, 64, 150, t - 1]
    ref_y, ref_idx, ref_w = oracle.moe_layer(host, ops.bf16_bits(x[sample].contiguous()))
    assert np.array_equal(idx[sample].cpu().numpy().astype(np.uint32), ref_idx)
    assert np.array_equal(rw[sample].cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y[sample].contiguous())), oracle.bf16_to_float(ref_y),
                       f"{workload} prefill rows vs checker")
    for i in sample[:3]:
        yd = torch.zeros((1, d), dtype=torch.bfloat16, device=dev)
        idd = torch.zeros((1, k), dtype=torch.int32, device=dev)
        moe.encode_decode_layer(lw, x[i:i + 1].contiguous(), yd, t=1, out_indices=idd)
        moe.status()
        assert torch.equal(idd[0], idx[i])
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y[i:i + 1])),
                           oracle.bf16_to_float(ops.bf16_bits(yd)), f"{workload} prefill row {i} vs decode")
    y2 = torch.zeros_like(x)
    moe.encode_prefill_layer(lw, x, y2, t, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


def test_prefill_rejects_a_short_workspace(gpu, oracle):
    layer4 = oracle.synth_layer(ROOT_SEED + 0xA201, 256, 128, 16, 4, bits=4, fs=0)
    moe4 = make_moe(gpu, layer4)
    wts4 = to_device_layer(layer4)
    x = ops.bf16_tensor(oracle.synth_x(1, 4, 256))
    y = torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda")
    assert moe4.prefill_workspace_bytes(4) > 0
    with pytest.raises(_capi.MfError) as err:
        moe4.encode_prefill_layer(wts4, x, y, 4, workspace=torch.empty(256, dtype=torch.uint8, device="cuda"))
    assert err.value.status == -4


def test_prefill_full_size_rows_do_not_depend_on_their_neighbours(gpu, oracle):
    """Qwen-shaped layer, 2048 tokens, skewed routing (the bench.py configuration): a token's
    output row depends on that token alone, so permuting the tokens permutes the rows bit for
    bit (tiles, chunk boundaries and positions inside a tile all change); the routes of every
    expert add up; sampled rows agree with the decode launch of the same token."""
    import bench
    w = dict(bench.QWEN)
    dev = torch.device("cuda", 0)
    stack = bench.build_stack(gpu, w, 1, dev)
    lw = stack[0]
    gen = torch.Generator(device=dev)
    gen.manual_seed(99)
    router = lw.router_w.clone()
    router[:, -1] = (torch.randn((w["e"],), generator=gen, device=dev) * 1.5).to(torch.bfloat16)
    lw = ops.MoELayerWeights(router, lw.experts, lw.offsets, lw.shared, lw.w_sg)
    moe = ops.MoE(gpu, w["d"], w["f"], w["e"], w["k"], bits=4, shared_f=w["fs"], shared_bits=4)
    t, d, k = 2048, w["d"], w["k"]
    x = torch.randn((t, d), generator=gen, device=dev).to(torch.bfloat16)
    x[:, -1] = 1.0
    y = torch.zeros_like(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device=dev)
    ws = moe.encode_prefill_layer(lw, x, y, t, out_indices=idx)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y.float()).all())
    counts = torch.bincount(idx.flatten().long(), minlength=w["e"])
    assert int(counts.sum()) == t * k and int((counts == 0).sum()) > 0   # skew: some experts stay empty
    assert bool((idx.sort(dim=1).values.diff(dim=1) != 0).all())        # k distinct experts per token
    perm = torch.randperm(t, generator=gen, device=dev)
    xp = x[perm].contiguous()
    yp = torch.zeros_like(x)
    idxp = torch.zeros_like(idx)
    moe.encode_prefill_layer(lw, xp, yp, t, out_indices=idxp, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(idxp, idx[perm])
    assert torch.equal(yp.view(torch.int16), y[perm].view(torch.int16))
    for i in (0, 1, 777, 2047):   # the decode launch on single tokens
        yd = torch.zeros((1, d), dtype=torch.bfloat16, device=dev)
        idd = torch.zeros((1, k), dtype=torch.int32, device=dev)
        moe.encode_decode_layer(lw, x[i:i + 1].contiguous(), yd, t=1, out_indices=idd)
        moe.status()
        assert torch.equal(idd[0], idx[i])
        assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y[i:i + 1])),
                           oracle.bf16_to_float(ops.bf16_bits(yd)), f"prefill row {i} vs decode")


def test_prefill_16k_tokens_repeat_the_2048_token_rows(gpu):
    """16 384 tokens (131 072 routes, 2 000+ tiles, 1 GiB of per-route partial rows -- byte offsets
    of the down projection's stores reach 2^30): the batch is the 2048-token batch eight times
    over, so every block of 2048 output rows equals the rows of the 2048-token call bit for bit."""
    import bench
    w = dict(bench.QWEN)
    dev = torch.device("cuda", 0)
    lw = bench.build_stack(gpu, w, 1, dev)[0]
    gen = torch.Generator(device=dev)
    gen.manual_seed(4242)
    router = lw.router_w.clone()
    router[:, -1] = (torch.randn((w["e"],), generator=gen, device=dev) * 1.5).to(torch.bfloat16)
    lw = ops.MoELayerWeights(router, lw.experts, lw.offsets, lw.shared, lw.w_sg)
    moe = ops.MoE(gpu, w["d"], w["f"], w["e"], w["k"], bits=4, shared_f=w["fs"], shared_bits=4)
    t, d, k, reps = 2048, w["d"], w["k"], 8
    x = torch.randn((t, d), generator=gen, device=dev).to(torch.bfloat16)
    x[:, -1] = 1.0
    y = torch.zeros_like(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device=dev)
    moe.encode_prefill_layer(lw, x, y, t, out_indices=idx)
    torch.cuda.synchronize()
    xb = x.repeat(reps, 1).contiguous()
    yb = torch.zeros_like(xb)
    idxb = torch.zeros((t * reps, k), dtype=torch.int32, device=dev)
    moe.encode_prefill_layer(lw, xb, yb, t * reps, out_indices=idxb)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(yb.float()).all())
    assert torch.equal(idxb.view(reps, t, k), idx.expand(reps, t, k))
    assert torch.equal(yb.view(torch.int16).view(reps, t, d), y.view(torch.int16).expand(reps, t, d))


@pytest.mark.parametrize("d,f,t", [(512, 256, 100), (128, 128, 1100)])
def test_non_finite_token_takes_sentinel_routes(gpu, oracle, d, f, t):
    """full-softmax router: a token whose logits are not finite gets indices = num_experts and
    weights 0 (maple_moe.metal:73-79); its routes contribute nothing, in the decode launch and in
    the prefill call (short batch: grouped by one workgroup; long batch: selected and grouped chunk by
    chunk), and the other tokens of the batch are untouched"""
    e, k = 32, 8
    root = ROOT_SEED + 0xAB00 + t
    layer = oracle.synth_layer(root, d, f, e, k, bits=1, router_mode=1)
    x = oracle.synth_x(root, t, d)
    bad = [3, 64, t - 1]
    x[bad, 7] = 0x7FC0   # bf16 NaN
    rows = sorted(set(bad) | set(range(0, 8)) | set(range(60, 70)) | set(range(t - 10, t)))
    ref_y, ref_idx, ref_w = oracle.moe_layer(layer, x[rows])
    at = {r: i for i, r in enumerate(rows)}
    ref_bad = [at[r] for r in bad]
    assert (ref_idx[ref_bad] == e).all() and (ref_w[ref_bad] == 0).all() and (ref_y[ref_bad] == 0).all()
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y, idx, w = _run_prefill(moe, wts, x, t, d, k)
    assert np.array_equal(idx[rows], ref_idx)
    assert np.array_equal(w[rows].view(np.uint32), ref_w.view(np.uint32))
    assert (y[bad] == 0).all()
    good = [r for r in rows if r not in bad]
    assert_layer_close(oracle.bf16_to_float(y[good]), oracle.bf16_to_float(ref_y[[at[r] for r in good]]),
                       "tokens next to a NaN token")
    ref_idx = {r: ref_idx[at[r]] for r in (2, 3, 4)}
    yd = torch.zeros((3, d), dtype=torch.bfloat16, device="cuda")
    idd = torch.zeros((3, k), dtype=torch.int32, device="cuda")
    moe.encode_decode_layer(wts, ops.bf16_tensor(x[[2, 3, 4]]), yd, t=3, out_indices=idd)
    moe.status()
    assert np.array_equal(idd.cpu().numpy().astype(np.uint32), np.stack([ref_idx[r] for r in (2, 3, 4)]))
    assert (ops.bf16_bits(yd)[1] == 0).all()


@pytest.mark.parametrize("bits,d,f,e,k,fs,t,mode", [
    (4, 2048, 512, 256, 8, 512, 300, 0),   # the headline shape: K = 2048 through the ring, K = 512 resident
    (4, 256, 1024, 16, 4, 128, 150, 0),    # down projection through the ring kernel (K = 1024)
    (4, 384, 128, 32, 2, 128, 131, 1),     # K groups not a multiple of 8
    (2, 512, 256, 32, 6, 256, 200, 0),     # 2-bit codes: 8-byte pieces
    (1, 1024, 512, 64, 8, 0, 77, 1),       # ternary
])
def test_prefill_from_the_tiled_pool_gives_the_same_bits(gpu, oracle, bits, d, f, e, k, fs, t, mode):
    """mf_moe_tile_experts: the expert pool in the matmul's own order (a second copy; codes re-ordered inside
    each sub-tensor, tables in place) -- the prefill layer reads it and writes the bits it writes from the
    row-by-row pool; a decode call with the same weights struct ignores it."""
    root = ROOT_SEED + 0x711E + bits + d
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=mode)
    x = oracle.synth_x(root, t, d)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y0, idx0, w0 = _run_prefill(moe, wts, x, t, d, k)
    tiled = moe.tile_experts(wts.experts, wts.offsets)
    torch.cuda.synchronize()
    assert not torch.equal(tiled, wts.experts)
    # tables and everything outside the three code sub-tensors are copied as they are
    off = wts.offsets
    assert torch.equal(tiled[:, off.gate_s:off.gate_s + f * (d // 64) * 2], wts.experts[:, off.gate_s:off.gate_s + f * (d // 64) * 2])
    wts.experts_tiled = tiled
    y1, idx1, w1 = _run_prefill(moe, wts, x, t, d, k)
    assert np.array_equal(idx0, idx1) and np.array_equal(w0.view(np.uint32), w1.view(np.uint32))
    assert np.array_equal(y0, y1)
    # ... also with 16-bit per-route results
    moe.set_prefill_route_rounding(True)
    y2, _, _ = _run_prefill(moe, wts, x, t, d, k)
    wts.experts_tiled = None
    y3, _, _ = _run_prefill(moe, wts, x, t, d, k)
    moe.set_prefill_route_rounding(False)
    wts.experts_tiled = tiled
    assert np.array_equal(y2, y3)
    # decode ignores the tiled pool
    xd = ops.bf16_tensor(x[:3])
    ya = torch.zeros((3, d), dtype=torch.bfloat16, device="cuda")
    yb = torch.zeros_like(ya)
    moe.encode_decode_layer(wts, xd, ya, 3)
    wts.experts_tiled = None
    moe.encode_decode_layer(wts, xd, yb, 3)
    torch.cuda.synchronize()
    assert torch.equal(ya, yb)
    # in place is refused
    lib = _capi.lib()
    import ctypes as C
    assert lib.mf_moe_tile_experts(moe._h, None, wts.experts.data_ptr(), wts.experts.stride(0), C.byref(wts.offsets),
                                   wts.experts.data_ptr()) == -1
