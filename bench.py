#!/usr/bin/env python3
"""Benchmark of the MoE expert hot path on one MI355X.

Workload (default): the Qwen3.6-35B-A3B-shaped 4-bit MoE layer at T=1 decode,
run as a 40-layer stack with independent weights per layer (hidden 2048, 256
routed experts of intermediate 512, top-8, one shared expert of intermediate
512 gated by sigmoid(w_sg.x)).  A "step" is one token through the whole stack:
the 40 layers run back to back on one stream, each on its own input row and its
own weights, so every layer streams its expert bytes from HBM (40 x 453 MB of
resident experts, far beyond the 256 MB Infinity Cache).

Prints ONE JSON line: metric, value, unit, timing fields, `roofline` (dominant kernel against
the HBM or matrix-core peak) and `cpu_baseline` (the CPU checker timed on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix peak, published
ROOT_SEED = 0x4D464D4F00000000

QWEN = dict(name="qwen3.6-35b-a3b-moe-layer-decode-T1-4bit-g64", config=1, d=2048, f=512, e=256,
            k=8, fs=512, bits=4, shared_bits=4, t=1)
# the other decode configurations of the same path (selected with --workload; parity-test shapes,
# measured here so that every configuration has a number)
WORKLOADS = {
    "qwen-decode": QWEN,
    "dsv4-2bit": dict(name="large-2bit-moe-layer-decode-D4096-F2048-E256-K6", config=3, d=4096, f=2048,
                      e=256, k=6, fs=2048, bits=2, shared_bits=4, t=1, layers=4),
    "maple-ternary": dict(name="ternary-moe-layer-decode-D2048-F1024-E64-K8", config=4, d=2048, f=1024,
                          e=64, k=8, fs=0, bits=1, shared_bits=4, t=1, layers=40, maple=True),
    # the reference's MaplePreview architecture (ModelTypes.swift:515-560): 256 ternary experts of 512, top-8
    "maple-preview": dict(name="ternary-moe-layer-decode-D2048-F512-E256-K8", config=4, d=2048, f=512,
                          e=256, k=8, fs=0, bits=1, shared_bits=4, t=1, layers=40, maple=True),
}
DENSE_MLP = dict(name="dense-4bit-swiglu-mlp-D5120-F17408", d=5120, f=17408, bits=4, layers=8)


def algorithmic_bytes(w) -> dict:
    """Bytes one layer must read at T=1: the K selected experts + the shared
    expert ("expert bytes touched"), and the same plus router, w_sg, x and y."""
    def tensor(rows, cols, bits):
        if bits == 1:  # ternary: 2-bit codes, one bf16 scale per group, no bias table
            return rows * cols * 2 // 8 + rows * (cols // 64) * 2
        return rows * cols * bits // 8 + 2 * rows * (cols // 64) * 2
    expert = 2 * tensor(w["f"], w["d"], w["bits"]) + tensor(w["d"], w["f"], w["bits"])
    shared = (2 * tensor(w["fs"], w["d"], w["shared_bits"]) + tensor(w["d"], w["fs"], w["shared_bits"])
              if w["fs"] else 0)
    n_sel = w.get("experts_touched", w["k"])
    expert_bytes = n_sel * expert + shared
    total = expert_bytes + w["e"] * w["d"] * 2 + w["d"] * 2 + 2 * w["t"] * w["d"] * 2
    return dict(expert=expert, expert_bytes=expert_bytes, total=total)


def build_stack(ctx, w, layers, device):
    """Random-init weights of the named architecture, drawn on the GPU
    (N(0, 0.02), seeded per layer) and quantized by the library's own device
    quantizer into resident expert blobs."""
    import torch
    from mference_amd import operators as ops

    quant = ops.Quantization(ctx)
    off, _, stride = ops.expert_blob_layout(w["d"], w["f"], w["bits"])
    stack = []
    E, D, F = w["e"], w["d"], w["f"]
    for l in range(layers):
        gen = torch.Generator(device=device)
        gen.manual_seed((ROOT_SEED + 0x100 * w["config"] + l) & 0x7FFFFFFFFFFFFFFF)
        experts = torch.zeros((E, stride), dtype=torch.uint8, device=device)
        for name, rows, cols in (("gate", F, D), ("up", F, D), ("down", D, F)):
            if w["bits"] == 1:
                q = ternary_tensor(gen, E * rows, cols, device)
            else:
                raw = torch.randn((E * rows, cols), generator=gen, device=device,
                                  dtype=torch.float32) * 0.02
                q = quant.quantize_affine(raw, w["bits"])
                del raw
            wo, so, bo = (getattr(off, f"{name}_{s}") for s in "wsb")
            nb = q.packed.shape[1] * rows
            experts[:, wo:wo + nb] = q.packed.view(E, nb)
            ns = q.scales.shape[1] * rows * 2
            experts[:, so:so + ns] = q.scales.view(torch.uint8).view(E, ns)
            if w["bits"] != 1:
                experts[:, bo:bo + ns] = q.biases.view(torch.uint8).view(E, ns)
            del q
        router_w = (torch.randn((E, D), generator=gen, device=device) * 0.02).to(torch.bfloat16)
        shared = None
        w_sg = None
        if w["fs"]:
            shared = []
            for rows, cols in ((w["fs"], D), (w["fs"], D), (D, w["fs"])):
                raw = torch.randn((rows, cols), generator=gen, device=device) * 0.02
                shared.append(quant.quantize_affine(raw, w["shared_bits"]))
            w_sg = (torch.randn((D,), generator=gen, device=device) * 0.02).to(torch.bfloat16)
        stack.append(ops.MoELayerWeights(router_w, experts, off, shared, w_sg))
    torch.cuda.synchronize()
    return stack


def ternary_tensor(gen, rows, cols, device):
    """codes {0,1,2} with p = .25/.5/.25, four per byte; bf16 scale per group of 64 and bias = -scale
    (the stored form of the reference's row_alpha expansion)"""
    import torch
    from mference_amd import operators as ops
    u = torch.rand((rows, cols), generator=gen, device=device)
    codes = (u >= 0.25).to(torch.uint8) + (u >= 0.75).to(torch.uint8)
    c4 = codes.view(rows, cols // 4, 4)
    packed = (c4[..., 0] | (c4[..., 1] << 2) | (c4[..., 2] << 4) | (c4[..., 3] << 6)).contiguous()
    scales = (torch.randn((rows, cols // 64), generator=gen, device=device).abs() * 0.02 + 1e-3)
    scales = scales.to(torch.bfloat16)
    return ops.QuantizedTensor(packed, scales, -scales, 1, rows, cols)


def layer_to_host(wts, w):
    """device layer -> oracle Layer (for the parity check and the CPU baseline)"""
    from mference_amd import operators as ops
    from oracle import mf_oracle as O
    off = O.ExpertOffsets()
    for name, _ in off._fields_:
        setattr(off, name, getattr(wts.offsets, name))
    def q(t):
        return O.QTensor(t.packed.cpu().numpy(), ops.bf16_bits(t.scales),
                         None if t.biases is None else ops.bf16_bits(t.biases), t.bits, t.rows, t.n)
    shared = None if wts.shared is None else tuple(q(t) for t in wts.shared)
    return O.Layer(d=w["d"], f=w["f"], e=w["e"], k=w["k"], bits=w["bits"],
                   router_w=ops.bf16_bits(wts.router_w), experts=wts.experts.cpu().numpy(), off=off,
                   fs=w["fs"], shared_bits=w["shared_bits"], shared=shared,
                   w_sg=None if wts.w_sg is None else ops.bf16_bits(wts.w_sg),
                   router_mode=1 if w["bits"] == 1 else 0, maple_rounding=bool(w.get("maple")))


def profiled_traffic_bytes(name="fused_decode_qwen_t1.md", unit="launch"):
    """HBM bytes per launch of the fused kernel (per layer call of the prefill) from the committed
    rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size)."""
    import re
    path = os.path.join(ROOT, "profiles", name)
    try:
        m = re.search(r"Traffic per %s = \*\*([0-9,]+) B\*\*" % unit, open(path).read())
        return int(m.group(1).replace(",", "")) if m else None
    except OSError:
        return None


def pmc_calibration(device) -> str:
    """a kernel of known HBM traffic, so that FETCH_SIZE / WRITE_SIZE readings can be scaled"""
    import torch
    src = torch.zeros(256 << 20, dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    return "3 x 256 MiB device-to-device copy (reads 268435456 B, writes 268435456 B)"


def measure_prefill(ctx, w, layer, device, tokens=(128, 512, 2048), steps=100, warmup=100, use_graph=True,
                    side_runs=True):
    """Ragged prefill of one layer of the same shape: T tokens, top-k routing from skewed
    logits (router weights plus a per-expert bias ~ N(0, 1.5), carried by a constant-one last
    feature of x and the last column of the router, so expert loads are uneven and some
    experts get no token).  Parity at the smallest T against the per-token CPU checker."""
    import numpy as np
    import torch
    from mference_amd import operators as ops
    from oracle import mf_oracle as O

    gen = torch.Generator(device=device)
    gen.manual_seed((ROOT_SEED + 0x100 * 2 + 0x7F) & 0x7FFFFFFFFFFFFFFF)
    router = layer.router_w.clone()
    router[:, -1] = (torch.randn((w["e"],), generator=gen, device=device) * 1.5).to(torch.bfloat16)
    lw = ops.MoELayerWeights(router, layer.experts, layer.offsets, layer.shared, layer.w_sg)
    full_softmax = w["bits"] == 1
    moe = ops.MoE(ctx, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                  shared_bits=w["shared_bits"], maple_rounding=bool(w.get("maple")),
                  router_mode=ops.ROUTER_FULL_SOFTMAX if full_softmax else ops.ROUTER_TOPK_SOFTMAX)
    # the routed experts a second time, in the prefill matmul's own order (mf_moe_tile_experts): what the layer
    # call reads when it is given; same bits as from the row-by-row pool
    lw.experts_tiled = moe.tile_experts(layer.experts, layer.offsets)
    qwen = w["config"] == QWEN["config"]
    import re
    out = {"launch": "hip_graph" if use_graph else "eager",
           "expert_pool": "tiled copy of the layer's experts (mf_moe_tile_experts, +%d MB of HBM for this layer); "
                          "us_per_layer_row_by_row_pool is the same call without it" % (layer.experts.numel() >> 20),
           "workload": ("qwen3.6-35b-a3b-moe-layer-ragged-prefill-4bit-g64" if qwen
                        else re.sub(r"-T\d+$", "", w["name"]).replace("decode", "ragged-prefill")) + ", skewed routing",
           "dtype": "u%d codes (exact, as bf16) x bf16 activations on bf16 MFMA, fp32 accumulate"
                    % (4 if w["bits"] == 4 else 2),
           "runs": []}
    for t in tokens:
        x = torch.randn((t, w["d"]), generator=gen, device=device).to(torch.bfloat16)
        x[:, -1] = 1.0
        y = torch.zeros_like(x)
        idx = torch.zeros((t, w["k"]), dtype=torch.int32, device=device)
        ws = moe.encode_prefill_layer(lw, x, y, t, out_indices=idx)
        torch.cuda.synchronize()
        counts = torch.bincount(idx.flatten().long(), minlength=w["e"]).cpu().numpy()
        run = {"tokens": t}
        if t == min(tokens):
            host = layer_to_host(lw, w)
            n_par = t if qwen else min(t, 16)   # the large layers: the first 16 rows (the checker is a CPU loop)
            ref_y, ref_idx, _ = O.moe_layer(host, ops.bf16_bits(x[:n_par].contiguous()))
            got = O.bf16_to_float(ops.bf16_bits(y[:n_par].contiguous())).astype(np.float64)
            ref = O.bf16_to_float(ref_y).astype(np.float64)
            run["parity"] = dict(
                rows=n_par,
                routing_bit_exact=bool(np.array_equal(idx[:n_par].cpu().numpy().astype(np.uint32), ref_idx)),
                max_abs=float(np.abs(got - ref).max()),
                rel_l2=float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))
        # the layer call is several launches: replayed from a HIP graph (ten calls per graph) so that
        # short batches measure the kernels and not the host's launch rate
        per_graph = 10 if use_graph else 1

        def timed_us():
            def calls():
                for _ in range(per_graph):
                    moe.encode_prefill_layer(lw, x, y, t, workspace=ws)
            go = calls
            if use_graph:
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    calls()
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    calls()
                go = graph.replay
            reps = max(1, steps // per_graph)
            for _ in range(max(1, warmup // per_graph)):
                go()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                go()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / (reps * per_graph) * 1e3

        us = timed_us()
        if side_runs:
            tiled = lw.experts_tiled
            lw.experts_tiled = None
            run["us_per_layer_row_by_row_pool"] = round(timed_us(), 1)
            lw.experts_tiled = tiled
        if side_runs and not w.get("maple"):
            # the reference's prefill rule: a route's result is a 16-bit number before its weight (half the
            # bytes between the down projection and the reduce); the default keeps fp32 as the decode step does
            moe.set_prefill_route_rounding(True)
            run["us_per_layer_routes_bf16"] = round(timed_us(), 1)
            moe.set_prefill_route_rounding(False)
        flops = 2.0 * 3 * w["d"] * (t * w["k"] * w["f"] + t * w["fs"])
        tflops = flops / us / 1e6
        # algorithmic bytes of the call: the experts that got a token + the shared expert + router, once each,
        # the token rows in and out (the short batches are bound by these, not by the matrix cores)
        ab = algorithmic_bytes(dict(w, experts_touched=int((counts > 0).sum()), t=t))
        hbm_gbps = ab["total"] / us / 1e3
        run.update(us_per_layer=round(us, 1), tokens_per_s=round(t / us * 1e6, 1),
                   tflops=round(tflops, 1), mfma_frac=round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                   algorithmic_bytes=int(ab["total"]), hbm_gbps=round(hbm_gbps, 1),
                   hbm_frac=round(hbm_gbps / HBM_PEAK_GBPS, 4),
                   experts_without_tokens=int((counts == 0).sum()), max_expert_load=int(counts.max()),
                   output_finite=bool(torch.isfinite(y.float()).all().item()))
        out["runs"].append(run)
    last = out["runs"][-1]
    out["roofline"] = {"bound": "mfma", "achieved": last["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                       "unit": "TFLOP/s", "frac": last["mfma_frac"],
                       "traffic": profiled_traffic_bytes("prefill_qmm_qwen_t2048.md", "layer") if qwen and last["tokens"] == 2048 else None,
                       "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary committed as "
                                         "profiles/prefill_qmm_qwen_t2048.md (all launches of one layer call at T=2048; a "
                                         "constant of that profile run, not measured by this run)",
                       "kernel": "whole layer at T=%d (router, grouping, mf::qmm_kernel, mf::qmm_kres_kernel, reduce); "
                                 "algorithmic flops = 2*3*D*(T*K*F + T*Fs)" % last["tokens"]}
    return out


def _omp_threads(n):
    """thread count of the CPU checker's OpenMP loops (libgomp of this process); None = leave"""
    import ctypes
    try:
        gomp = ctypes.CDLL("libgomp.so.1")
        prev = gomp.omp_get_max_threads()
        if n:
            gomp.omp_set_num_threads(int(n))
        return prev
    except OSError:
        return None


def bench_single_expert(args, device) -> int:
    """One SwiGLU expert FFN at batch 1 (hidden 2048, intermediate 512, 4-bit g64): the shared-expert
    operator on one expert's projections, `layers` distinct experts in rotation; beside it the CPU checker
    (a restatement of the reference's CPU path) single-threaded and on all cores."""
    import numpy as np
    import torch
    from mference_amd import operators as ops
    from oracle import mf_oracle as O

    D, F = 2048, 512
    L = args.layers or 256  # 256 experts = 453 MB: more than the 256 MB last-level cache holds
    ctx = ops.MetalContext(0)
    quant = ops.Quantization(ctx)
    gen = torch.Generator(device=device)
    gen.manual_seed((ROOT_SEED + 0x000) & 0x7FFFFFFFFFFFFFFF)
    big = [quant.quantize_affine(torch.randn((L * r, c), generator=gen, device=device) * 0.02, 4)
           for r, c in ((F, D), (F, D), (D, F))]

    def view(q, i, rows):
        return ops.QuantizedTensor(q.packed[i * rows:(i + 1) * rows], q.scales[i * rows:(i + 1) * rows],
                                   q.biases[i * rows:(i + 1) * rows], 4, rows, q.n)
    sets = [[view(big[0], i, F), view(big[1], i, F), view(big[2], i, D)] for i in range(L)]
    mlp = ops.SharedExpertInt4(ctx)
    x = torch.randn((1, D), generator=gen, device=device).to(torch.bfloat16)
    y = torch.zeros((L, 1, D), dtype=torch.bfloat16, device=device)
    scratch = torch.zeros((1, F), dtype=torch.bfloat16, device=device)

    def step():
        for l in range(L):
            mlp.encode(x, sets[l][0], sets[l][1], sets[l][2], y[l], scratch, t=1)

    def hq(q):
        return O.QTensor(q.packed.cpu().numpy(), ops.bf16_bits(q.scales), ops.bf16_bits(q.biases), 4, q.rows, q.n)
    step()
    torch.cuda.synchronize()
    h0 = [hq(q) for q in sets[0]]
    xb = ops.bf16_bits(x[0])
    ref = O.bf16_to_float(O.shared_expert(h0[0], h0[1], h0[2], xb)).astype(np.float64)
    got = O.bf16_to_float(ops.bf16_bits(y[0][0])).astype(np.float64)
    parity = dict(max_abs=float(np.abs(got - ref).max()), rel_l2=float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / args.steps / L * 1e3
    nbytes = 3 * (D * F // 2 + 2 * 2 * (D * F // 64))  # 1 769 472
    achieved = nbytes / (us * 1e-6) / 1e9
    out = {
        "metric": "us_per_expert_ffn_T1", "value": round(us, 3), "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us * L / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "u4 codes x bf16 activations, fp32 accumulate", "data": "synthetic (N(0,0.02) weights, 4-bit g64; x ~ N(0,1))",
        "config": {"workload": "single-swiglu-expert-ffn-D2048-F512-T1", "weight_sets": L, "tokens": 1, "launch": "hip_graph"},
        "parity_set0": parity,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "mf::gate_up_act_kernel + mf::gemv_kernel (two launches per expert)",
                     "algorithmic_bytes": nbytes}}
    if not args.no_cpu_baseline:
        all_cores = int(os.environ.get("OMP_NUM_THREADS") or min(16, os.cpu_count() or 1))
        res = []
        for threads in (1, all_cores):
            prev = _omp_threads(threads)
            n, t0 = 0, time.perf_counter()
            while True:
                O.shared_expert(h0[0], h0[1], h0[2], xb)
                n += 1
                el = time.perf_counter() - t0
                if el >= args.cpu_seconds / 2 or n >= 20000:
                    break
            _omp_threads(prev)
            res.append({"value": round(el / n * 1e6, 1), "unit": "us", "cores": threads if prev else 1, "kind": "port",
                        "sample": f"{n} repetitions of the same expert FFN"})
        out["cpu_baseline"] = res[1]
        out["cpu_baseline_single_thread"] = res[0]
    print(json.dumps(out))
    return 0


def bench_dense_mlp(args, device) -> int:
    """Dense 4-bit SwiGLU MLP (hidden 5120, intermediate 17408) at T token rows: the shared-expert
    operator on a dense layer; `layers` distinct weight sets rotate so HBM is read every step."""
    import torch
    from mference_amd import operators as ops

    w = DENSE_MLP
    t = args.tokens or 1
    L = args.layers or w["layers"]
    ctx = ops.MetalContext(0)
    quant = ops.Quantization(ctx)
    gen = torch.Generator(device=device)
    gen.manual_seed((ROOT_SEED + 0x500) & 0x7FFFFFFFFFFFFFFF)
    D, F = w["d"], w["f"]
    sets = []
    for _ in range(L):
        qs = []
        for rows, cols in ((F, D), (F, D), (D, F)):
            raw = torch.randn((rows, cols), generator=gen, device=device) * 0.02
            qs.append(quant.quantize_affine(raw, 4))
            del raw
        sets.append(qs)
    mlp = ops.SharedExpertInt4(ctx)
    x = torch.randn((t, D), generator=gen, device=device).to(torch.bfloat16)
    y = torch.zeros((L, t, D), dtype=torch.bfloat16, device=device)
    # from 32 rows on the call takes the matrix-core matmul and wants its staging rows in the scratch
    scratch = torch.zeros(max(mlp.scratch_bytes(D, F, t), t * F * 2) // 2, dtype=torch.bfloat16, device=device)

    def step():
        for l in range(L):
            mlp.encode(x, sets[l][0], sets[l][1], sets[l][2], y[l], scratch, t=t)

    # parity of set 0 against the CPU checker
    import numpy as np
    from oracle import mf_oracle as O
    def hq(q):
        return O.QTensor(q.packed.cpu().numpy(), ops.bf16_bits(q.scales), ops.bf16_bits(q.biases), 4, q.rows, q.n)
    step()
    torch.cuda.synchronize()
    rows = list(range(t)) if t <= 8 else sorted({0, 1, t // 2, t - 1})  # the checker takes ~1 s per row
    h0 = [hq(q) for q in sets[0]]
    t_cpu = time.perf_counter()
    ref = np.stack([O.shared_expert(h0[0], h0[1], h0[2], ops.bf16_bits(x[i])) for i in rows])
    cpu_us_per_row = (time.perf_counter() - t_cpu) / len(rows) * 1e6
    cores = int(os.environ.get("OMP_NUM_THREADS") or min(16, os.cpu_count() or 1))
    cpu_baseline = {"value": round(cpu_us_per_row * t, 1), "unit": "us", "cores": cores, "kind": "port",
                    "sample": f"{len(rows)} token rows of weight set 0 through the CPU checker, scaled to {t} rows"}
    got = O.bf16_to_float(ops.bf16_bits(y[0][rows])).astype(np.float64)
    reff = O.bf16_to_float(ref).astype(np.float64)
    parity = dict(max_abs=float(np.abs(got - reff).max()),
                  rel_l2=float(np.linalg.norm(got - reff) / np.linalg.norm(reff)))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for _ in range(args.warmup):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / args.steps / L * 1e3
    nbytes = 3 * (D * F // 2 + 2 * 2 * (D * F // 64))
    achieved = nbytes / (us * 1e-6) / 1e9
    if t >= 32:  # the block form: a matmul, priced against the bf16 matrix-core peak
        flops = 6.0 * D * F * t
        tflops = flops / (us * 1e-6) / 1e12
        print(json.dumps({
            "metric": "us_per_dense_mlp_T%d" % t, "value": round(us, 3), "unit": "us", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us * L / 1e3, 5),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
            "dtype": "u4 codes x bf16 activations, fp32 accumulate", "data": "synthetic (N(0,0.02) weights, 4-bit g64)",
            "config": {"workload": w["name"] + "-T%d" % t, "weight_sets": L, "tokens": t, "launch": "hip_graph"},
            "tokens_per_s": round(t / (us * 1e-6), 1), "parity_set0_rows": rows, "parity_set0": parity,
            "cpu_baseline": cpu_baseline,
            "hbm_gbps_weight_bytes": round(achieved, 1),
            "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                         "kernel": "mf::qmm_kernel (gate/up + SwiGLU, then down in K windows)",
                         "algorithmic_flops": flops}}))
        return 0
    print(json.dumps({
        "metric": "us_per_dense_mlp_T%d" % t, "value": round(us, 3), "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us * L / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "u4 codes x bf16 activations, fp32 accumulate", "data": "synthetic (N(0,0.02) weights, 4-bit g64)",
        "config": {"workload": w["name"] + "-T%d" % t, "weight_sets": L, "tokens": t, "launch": "hip_graph"},
        "parity_set0": parity, "cpu_baseline": cpu_baseline,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "mf::rows_quad_kernel (gate/up + activation, then down)", "algorithmic_bytes": nbytes}}))
    return 0


def measure_given_routing(ctx, device, layers=16, replays=50):
    """Decode layers (T = 1) whose routing comes from a family router: the sqrtsoftplus router call followed
    by the layer call with router_w = NULL, against the layer routing by itself; µs per layer from HIP-graph
    replays over `layers` distinct weight sets."""
    import torch
    from mference_amd import operators as ops

    out = []
    fam = ops.FamilyRouters(ctx)
    for name in ("qwen-decode", "dsv4-2bit"):
        w = dict(WORKLOADS[name])
        stack = build_stack(ctx, w, layers, device)
        moes = [ops.MoE(ctx, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                        shared_bits=w["shared_bits"]) for _ in range(layers)]
        gen = torch.Generator(device=device)
        gen.manual_seed(7)
        xs = torch.randn((layers, 1, w["d"]), generator=gen, device=device).to(torch.bfloat16)
        ys = torch.zeros_like(xs)
        idx = torch.zeros((layers, 1, w["k"]), dtype=torch.int32, device=device)
        wt = torch.zeros((layers, 1, w["k"]), dtype=torch.float32, device=device)
        lg = torch.zeros((layers, 1, w["e"]), dtype=torch.float32, device=device)
        bias = torch.zeros((w["e"],), device=device)
        given = [ops.MoELayerWeights(router_w=None, experts=s.experts, offsets=s.offsets, shared=s.shared,
                                     w_sg=s.w_sg) for s in stack]

        def own():
            for l in range(layers):
                moes[l].encode_decode_layer(stack[l], xs[l], ys[l], t=1)

        def routed(with_router, fused):
            def f():
                for l in range(layers):
                    moes[l].set_fused(fused)
                    if with_router:
                        fam.encode_router_top_k(stack[l].router_w, xs[l], bias, idx[l], wt[l], w["e"], w["d"], 1.5,
                                                lg[l], top_k=w["k"])
                    moes[l].encode_decode_layer(given[l], xs[l], ys[l], t=1, out_indices=idx[l], out_weights=wt[l])
            return f

        run = {"layer": w["name"]}
        for label, fn in (("routes_itself_us", own), ("router_call_plus_layer_us", routed(True, True)),
                          ("layer_on_given_routing_us", routed(False, True)),
                          ("router_call_plus_chain_of_launches_us", routed(True, False))):
            fn()
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                fn()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                fn()
            for _ in range(10):
                graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(replays):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            run[label] = round(e0.elapsed_time(e1) / replays / layers * 1e3, 2)
        for m in moes:
            m.set_fused(True)
            m.status()
        out.append(run)
        del stack, moes, given
    return out


def bench_family_routers(args, device) -> int:
    """The four family routers at their reference shapes, T = 1 (decode) and T = 2048 (prefill): µs per
    call from HIP-graph replays, the decode call against the HBM roofline of its router bytes, and the
    routing of row 0 against the CPU checker bit for bit.  `sets` distinct weight sets rotate at T = 1."""
    import numpy as np
    import torch
    from mference_amd import operators as ops
    from oracle import mf_oracle as O

    ctx = ops.MetalContext(0)
    fam = ops.FamilyRouters(ctx)
    gen = torch.Generator(device=device)
    gen.manual_seed((ROOT_SEED + 0x600) & 0x7FFFFFFFFFFFFFFF)
    sets = 64
    shapes = {  # rows, shared sinks, D, K
        "sqrtsoftplus (DeepSeek-V4)": (256, 0, 4096, 6), "hash weights (DeepSeek-V4)": (256, 0, 4096, 6),
        "sigmoid + sinks (Inkling)": (256, 2, 2048, 8), "8-bit affine (Gemma)": (128, 0, 2816, 8)}
    results = []
    for name, (e, sh, d, k) in shapes.items():
        rows = e + sh
        int8 = name.startswith("8-bit")
        for t in (1, 2048):
            n_sets = sets if t == 1 else 1
            if int8:
                wr = torch.randint(0, 256, (n_sets, rows, d), generator=gen, device=device, dtype=torch.uint8)
                sc = (torch.rand((n_sets, rows, d // 64), generator=gen, device=device) * 6e-4 + 2e-4).to(torch.bfloat16)
                bi = (torch.rand((n_sets, rows, d // 64), generator=gen, device=device) * -0.04 - 0.04).to(torch.bfloat16)
                eff = (torch.rand((d,), generator=gen, device=device) + 0.5).to(torch.bfloat16)
                pes = (torch.rand((e,), generator=gen, device=device) * 0.8 + 0.6).to(torch.bfloat16)
                nbytes = rows * d + 2 * 2 * rows * (d // 64)
            else:
                wr = (torch.randn((n_sets, rows, d), generator=gen, device=device) * 0.05).to(torch.bfloat16)
                nbytes = rows * d * 2
            x = torch.randn((t, d), generator=gen, device=device).to(torch.bfloat16)
            bias = torch.rand((e,), generator=gen, device=device) * 0.6 - 0.3
            gs = torch.full((1,), 0.75, device=device)
            idx = torch.zeros((t, k), dtype=torch.int32, device=device)
            given = torch.randint(0, e, (t, k), generator=gen, device=device, dtype=torch.int32)
            wt = torch.zeros((t, k), dtype=torch.float32, device=device)
            gam = torch.zeros((t, max(sh, 1)), dtype=torch.float32, device=device)
            lg = torch.zeros((t, rows), dtype=torch.float32, device=device)

            def call(i):
                if int8:
                    fam.encode_router_gemma4(wr[i], sc[i], bi[i], x, eff, pes, idx, wt, e, d, k, lg, t=t)
                elif name.startswith("sqrt"):
                    fam.encode_router_top_k(wr[i], x, bias, idx, wt, e, d, 1.5, lg, top_k=k, t=t)
                elif name.startswith("hash"):
                    fam.encode_router_hash_weights(wr[i], x, given, wt, e, d, 1.5, lg, top_k=k, t=t)
                else:
                    fam.encode_router_inkling(wr[i], x, bias, gs, idx, wt, gam, e, sh, k, 2.5, d, lg, t=t)

            call(0)
            torch.cuda.synchronize()
            lg0 = lg[0].cpu().numpy()
            if int8:
                ref_lg = O.router_logits_int8(wr[0].cpu().numpy(), ops.bf16_bits(sc[0]), ops.bf16_bits(bi[0]),
                                              ops.bf16_bits(x[0]), ops.bf16_bits(eff))
                ri, rw = O.topk_softmax_scaled(ref_lg, ops.bf16_bits(pes), k)
            else:
                ref_lg = O.router_logits(ops.bf16_bits(wr[0]), ops.bf16_bits(x[0]))
                if name.startswith("sqrt"):
                    ri, rw = O.router_sqrtsoftplus(ref_lg, bias.cpu().numpy(), k, 1.5)
                elif name.startswith("hash"):
                    ri, rw = given[0].cpu().numpy().astype(np.uint32), O.router_hash_weights(
                        ref_lg, given[0].cpu().numpy().astype(np.uint32), 1.5)
                else:
                    ri, rw, _ = O.router_inkling(ref_lg, bias.cpu().numpy(), 0.75, e, sh, k, 2.5)
            exact = bool(np.array_equal(lg0.view(np.uint32), ref_lg.view(np.uint32))
                         and (name.startswith("hash") or np.array_equal(idx[0].cpu().numpy().astype(np.uint32), ri))
                         and np.array_equal(wt[0].cpu().numpy().view(np.uint32), rw.view(np.uint32)))
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for i in range(n_sets):
                    call(i)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            per_graph = n_sets if t == 1 else 10
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(per_graph):
                    call(i % n_sets)
            reps = max(1, args.steps // 10)
            for _ in range(max(1, args.warmup // 10)):
                graph.replay()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                graph.replay()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / (reps * per_graph) * 1e3
            run = {"router": name, "tokens": t, "rows": rows, "d": d, "top_k": k, "us_per_call": round(us, 2),
                   "row0_bit_exact_vs_cpu_checker": exact}
            if t == 1:
                run.update(router_bytes=nbytes, gbps=round(nbytes / us / 1e3, 1),
                           hbm_frac=round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4))
            else:
                run.update(tokens_per_s=round(t / us * 1e6))
            results.append(run)
    head = results[0]
    print(json.dumps({
        "metric": "us_per_router_call_T1", "value": head["us_per_call"], "unit": "us", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(head["us_per_call"] / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 / u8 router rows x bf16 activations, fp32 accumulate and selection",
        "data": "synthetic (N(0,0.05) router rows, N(0,1) activations)",
        "config": {"workload": "family-routers", "launch": "hip_graph", "weight_sets_T1": sets},
        "runs": results,
        "decode_layer_on_family_routing": measure_given_routing(ctx, device),
        "roofline": {"bound": "hbm", "achieved": head["gbps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": head["hbm_frac"], "traffic": None,
                     "kernel": "mf::router_logits_kernel + mf::family_select_kernel (two launches per call)",
                     "algorithmic_bytes": head["router_bytes"]}}))
    return 0


def prefill_phase_trace(ctx, w, layer, device, tokens) -> int:
    """Stage stamps of the work items (tile x row slice) of the routed gate/up matmul of the ragged prefill
    layer: 0 start, 1 loads issued, 2 tables and bias terms done, 3 main loop done, 4 end (100 MHz clock)."""
    import numpy as np
    import torch
    from mference_amd import operators as ops
    gen = torch.Generator(device=device)
    gen.manual_seed((ROOT_SEED + 0x100 * 2 + 0x7F) & 0x7FFFFFFFFFFFFFFF)
    router = layer.router_w.clone()
    router[:, -1] = (torch.randn((w["e"],), generator=gen, device=device) * 1.5).to(torch.bfloat16)
    lw = ops.MoELayerWeights(router, layer.experts, layer.offsets, layer.shared, layer.w_sg)
    moe = ops.MoE(ctx, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"], shared_bits=w["shared_bits"],
                  maple_rounding=bool(w.get("maple")),
                  router_mode=ops.ROUTER_FULL_SOFTMAX if w["bits"] == 1 else ops.ROUTER_TOPK_SOFTMAX)
    out = {"workload": w["name"], "unit": "us", "runs": []}
    for t in tokens:
        x = torch.randn((t, w["d"]), generator=gen, device=device).to(torch.bfloat16)
        x[:, -1] = 1.0
        y = torch.zeros_like(x)
        ws = moe.encode_prefill_layer(lw, x, y, t)
        stamps = torch.zeros((32768, 8), dtype=torch.int64, device=device)
        moe.set_phase_trace(stamps)
        for _ in range(3):
            stamps.zero_()
            moe.encode_prefill_layer(lw, x, y, t, workspace=ws)
        torch.cuda.synchronize()
        moe.set_phase_trace(None)
        s = stamps.cpu().numpy().astype(np.float64)
        s = s[s[:, 4] > 0]
        d = np.diff(s[:, :5], axis=1).mean(axis=0) / 100.0
        out["runs"].append({"tokens": t, "live_work_items": int(s.shape[0]),
                            "loads_issued": round(float(d[0]), 2), "tables_and_bias_terms": round(float(d[1]), 2),
                            "main_loop": round(float(d[2]), 2), "stores": round(float(d[3]), 2),
                            "per_item": round(float((s[:, 4] - s[:, 0]).mean() / 100.0), 2),
                            "span_first_start_to_last_end": round(float((s[:, 4].max() - s[:, 0].min()) / 100.0), 1)})
    print(json.dumps(out))
    return 0


def phase_trace(ctx, w, stack, moes, device, with_norm=False) -> int:
    """Stage stamps every workgroup of the fused decode launch writes (100 MHz wall clock): per stamp
    the median over the layers of the earliest / median / latest workgroup, in us from the start of the
    layer's first workgroup, and the time from the end of one launch to the start of the next."""
    import numpy as np
    import torch
    from mference_amd import _capi
    L = len(moes)
    ncu = _capi.lib().mf_ctx_num_cu(ctx.handle)
    xs = torch.randn((L, w["t"], w["d"]), device=device).to(torch.bfloat16)
    ys = torch.zeros_like(xs)
    stamps = torch.zeros((L, ncu * 8), dtype=torch.int64, device=device)
    for l in range(L):
        moes[l].set_phase_trace(stamps[l])
    nw = torch.ones((w["d"],), dtype=torch.bfloat16, device=device)
    dl = torch.zeros_like(xs)
    for _ in range(6):
        for l in range(L):
            if with_norm:  # the residual add and the norm inside the launch: xs is the hidden state
                moes[l].encode_decode_layer_normed(stack[l], xs[l], nw, ys[l], t=w["t"], delta=dl[l], eps=1e-6)
            else:
                moes[l].encode_decode_layer(stack[l], xs[l], ys[l], t=w["t"])
    torch.cuda.synchronize()
    for m in moes:
        m.status()
        m.set_phase_trace(None)
    t = stamps.cpu().numpy().reshape(L, ncu, 8).astype(np.float64)
    names = ["start", "stage_a_done", "logits_gathered", "topk_done", "stage_b_done", "activations_gathered", "end"]
    skip = min(8, L // 2)   # the first layers of a pass start behind an idle device
    rel = (t[:, :, :7] - t[:, :, 0].min(axis=1)[:, None, None]) / 100.0
    out = {"workload": w["name"], "layers": L, "workgroups": int(ncu), "unit": "us from the layer's first workgroup start",
           "stamps": {n: {"earliest": round(float(np.median(rel[skip:, :, i].min(axis=1))), 2),
                          "median": round(float(np.median(np.median(rel[skip:, :, i], axis=1))), 2),
                          "latest": round(float(np.median(rel[skip:, :, i].max(axis=1))), 2)}
                      for i, n in enumerate(names)},
           "norm_done_median": round(float(np.median(np.median((t[skip:, :, 7] - t[skip:, :, 0].min(axis=1)[:, None]) / 100.0, axis=1))), 2) if with_norm else None,
           "gap_end_to_next_start_us": round(float(np.median(
               [(t[l, :, 0].min() - t[l - 1, :, 6].max()) / 100.0 for l in range(skip + 1, L)])), 2)}
    print(json.dumps(out))
    return 0


OTHER_CONFIGS = [
    # (key, BASELINE.json configuration, extra arguments of this script)
    ("single_expert_ffn_T1", 0, ["--workload", "single-expert", "--steps", "20", "--warmup", "5"]),
    # the headline layer at the token count of an MTP verification step (not a BASELINE row of its own)
    ("qwen_layer_T4", 1, ["--tokens", "4", "--steps", "100", "--warmup", "10"]),
    ("large_2bit_layer_T1", 3, ["--workload", "dsv4-2bit", "--steps", "100", "--warmup", "10"]),
    ("large_2bit_layer_T4", 3, ["--workload", "dsv4-2bit", "--tokens", "4", "--steps", "100", "--warmup", "10"]),
    ("ternary_layer_T1", 4, ["--workload", "maple-ternary", "--steps", "100", "--warmup", "10"]),
    ("dense_mlp_T1", 4, ["--workload", "dense-mlp", "--steps", "50", "--warmup", "10"]),
    ("dense_mlp_T4", 4, ["--workload", "dense-mlp", "--tokens", "4", "--steps", "50", "--warmup", "10"]),
]


def measure_other_configs(cpu_seconds: float, budget_s: float = 400.0) -> dict:
    """The remaining BASELINE.json configurations, each measured by this script in a child process of its
    own (one GPU, one after the other, after the headline's timed region) and reduced to a few fields:
    time, algorithmic bytes, achieved rate and fraction of the HBM peak, parity against the CPU checker
    and the checker's own time."""
    import subprocess
    out, t_start = {}, time.perf_counter()
    for key, cfg, extra in OTHER_CONFIGS:
        if time.perf_counter() - t_start > budget_s:
            out[key] = {"skipped": "time budget of the default run"}
            continue
        cmd = [sys.executable, os.path.abspath(__file__), "--gpus", "1", "--no-prefill", "--no-other-configs",
               "--cpu-seconds", str(cpu_seconds)] + extra
        try:
            proc = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
            line = [l for l in proc.stdout.splitlines() if l.startswith("{")][-1]
            r = json.loads(line)
        except Exception as exc:  # a configuration that fails says so and does not take the headline down
            out[key] = {"error": repr(exc)[:200]}
            continue
        roof = r.get("roofline", {})
        entry = {"baseline_config": cfg, "workload": r["config"]["workload"], "us": r["value"],
                 "algorithmic_bytes": roof.get("algorithmic_bytes_per_layer", roof.get("algorithmic_bytes")),
                 "achieved_gbps": roof.get("achieved"), "hbm_frac": roof.get("frac"),
                 "parity": r.get("parity_layer0", r.get("parity_set0")), "kernel": roof.get("kernel")}
        for k in ("cpu_baseline", "cpu_baseline_single_thread"):
            if k in r:
                entry[k] = {f: r[k][f] for f in ("value", "unit", "cores")}
        out[key] = entry
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=None)
    ap.add_argument("--workload", default="qwen-decode",
                    choices=sorted(WORKLOADS) + ["dense-mlp", "family-routers", "single-expert"],
                    help="qwen-decode is the headline; the others measure the remaining "
                         "configurations of the same path")
    ap.add_argument("--tokens", type=int, default=None, help="token rows per step (decode: 1..8)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a kernel of known HBM "
                         "traffic) so that FETCH_SIZE / WRITE_SIZE counters can be scaled")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-prefill", action="store_true", help="skip the ragged prefill section")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of the other BASELINE configurations that the default run appends")
    ap.add_argument("--with-norm", action="store_true",
                    help="with --phase-trace: the launch that makes x itself (mf_moe_decode_layer_normed)")
    ap.add_argument("--no-side-runs", action="store_true",
                    help="with --prefill-only: time the layer call as it is reported (tiled expert pool, fp32 per-route "
                         "results) only, not the row-by-row pool and the 16-bit per-route results beside it (for profiling)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="one layer, the ragged prefill section only (for profiling)")
    ap.add_argument("--phase-trace", action="store_true",
                    help="stage stamps of the fused decode launch (eager launches, the layer stack six "
                         "times over, the last pass reported) instead of the timed run")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (--gpus 1); no multi-GPU path exists",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch
    from mference_amd import operators as ops

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    if args.workload == "dense-mlp":
        return bench_dense_mlp(args, device)
    if args.workload == "single-expert":
        return bench_single_expert(args, device)
    if args.workload == "family-routers":
        return bench_family_routers(args, device)
    w = dict(WORKLOADS[args.workload])
    if args.tokens:
        w["t"] = args.tokens
        w["name"] += f"-T{args.tokens}"
    if args.workload != "qwen-decode":
        args.no_prefill = True
    L, K, W = args.layers or w.get("layers", 40), args.steps, args.warmup
    if args.prefill_only:
        L = 1
    ctx = ops.MetalContext(0)
    stack = build_stack(ctx, w, L, device)
    if args.prefill_only and args.phase_trace:
        return prefill_phase_trace(ctx, w, stack[0], device, (args.tokens,) if args.tokens else (128, 512, 2048))
    if args.prefill_only:
        tokens = (args.tokens,) if args.tokens else (128, 512, 2048)
        res = {"prefill": measure_prefill(ctx, w, stack[0], device, tokens=tokens, steps=min(args.steps, 100),
                                          side_runs=not args.no_side_runs,
                                          warmup=min(args.warmup, 100), use_graph=not args.no_graph)}
        if args.pmc_calibration:
            res["pmc_calibration"] = pmc_calibration(device)
        print(json.dumps(res))
        return 0
    moes = [ops.MoE(ctx, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                    shared_bits=w["shared_bits"], maple_rounding=bool(w.get("maple")),
                    router_mode=ops.ROUTER_FULL_SOFTMAX if w["bits"] == 1 else ops.ROUTER_TOPK_SOFTMAX)
            for _ in range(L)]

    if args.phase_trace:
        return phase_trace(ctx, w, stack, moes, device, with_norm=args.with_norm)

    gen = torch.Generator(device=device)
    gen.manual_seed(ROOT_SEED + 0x100 * w["config"] + 0xFF)
    # one input row set per layer (the layer input in the engine is the post-attention
    # RMSNorm output, not the previous MoE output); layers run back to back on one stream
    xs = torch.randn((L, w["t"], w["d"]), generator=gen, device=device).to(torch.bfloat16)
    ys = torch.zeros_like(xs)
    x0 = xs[0]

    def step():
        for l in range(L):
            moes[l].encode_decode_layer(stack[l], xs[l], ys[l], t=w["t"])

    # ---- parity of layer 0 at full size against the CPU checker
    from oracle import mf_oracle as O
    host0 = layer_to_host(stack[0], w)
    host0.router_mode = 1 if w["bits"] == 1 else 0
    ref_y, ref_idx, ref_w = O.moe_layer(host0, ops.bf16_bits(x0))
    yy = torch.zeros_like(x0)
    idx = torch.zeros((w["t"], w["k"]), dtype=torch.int32, device=device)
    rw = torch.zeros((w["t"], w["k"]), dtype=torch.float32, device=device)
    moes[0].encode_decode_layer(stack[0], x0, yy, t=w["t"], out_indices=idx, out_weights=rw)
    torch.cuda.synchronize()
    got = O.bf16_to_float(ops.bf16_bits(yy)).astype(np.float64)
    ref = O.bf16_to_float(ref_y).astype(np.float64)
    parity = dict(
        routing_bit_exact=bool(np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)
                               and np.array_equal(rw.cpu().numpy().view(np.uint32),
                                                  ref_w.view(np.uint32))),
        max_abs=float(np.abs(got - ref).max()),
        rel_l2=float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))

    # ---- timed region
    use_graph = not args.no_graph
    graph = None
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        run = graph.replay
    else:
        run = step

    for _ in range(W):
        run()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(K):
        run()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = ev0.elapsed_time(ev1)
    ms_per_step = gpu_ms / K
    us_per_layer = ms_per_step * 1e3 / L
    # spread over single steps (their own event pairs, after the timed region): p10 / median / p90
    n_spread = min(K, 200)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_spread)]
    for a, b in evs:
        a.record()
        run()
        b.record()
    torch.cuda.synchronize()
    per_step = np.sort(np.array([a.elapsed_time(b) for a, b in evs])) * 1e3 / L
    spread = {"steps": n_spread, "p10": round(float(np.percentile(per_step, 10)), 3),
              "median": round(float(np.median(per_step)), 3), "p90": round(float(np.percentile(per_step, 90)), 3)}
    for m in moes:
        m.status()
    finite = bool(torch.isfinite(ys.float()).all().item())

    if w["t"] > 1:  # several tokens share experts: count the union layer 0 selected
        w["experts_touched"] = int(np.unique(ref_idx).size)
    ab = algorithmic_bytes(w)
    achieved = ab["expert_bytes"] / (us_per_layer * 1e-6) / 1e9
    out = {
        "metric": "us_per_moe_layer_decode_T%d" % w["t"],
        "value": round(us_per_layer, 4),
        "unit": "us",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5),
        "us_per_layer_single_steps": spread,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "%s codes x bf16 activations, fp32 accumulate" % {4: "u4", 2: "u2", 1: "ternary"}[w["bits"]],
        "data": "synthetic (random-init weights quantized g64 on device: N(0,0.02) affine, or ternary "
                "codes p=.25/.5/.25 with |N(0,0.02)| scales; x ~ N(0,1))",
        "config": {"workload": w["name"], "layers": L, "tokens": w["t"], "hidden": w["d"],
                   "experts": w["e"], "top_k": w["k"], "moe_intermediate": w["f"],
                   "shared_intermediate": w["fs"], "launch": "hip_graph" if use_graph else "eager"},
        "tokens_per_s": round(w["t"] / (ms_per_step * 1e-3), 2),
        "hbm_gbps_expert_bytes": round(achieved, 1),
        "hbm_gbps_all_bytes": round(ab["total"] / (us_per_layer * 1e-6) / 1e9, 1),
        "wall_ms_per_step": round(wall_ms / K, 5),
        "output_finite": finite,
        "parity_layer0": parity,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": profiled_traffic_bytes() if args.workload == "qwen-decode" else None,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary committed as "
                                       "profiles/fused_decode_qwen_t1.md (a constant of that profile run, not "
                                       "measured by this run)" if args.workload == "qwen-decode" else None,
                     "kernel": "mf::fused_decode_kernel (one launch per layer)",
                     "algorithmic_bytes_per_layer": ab["expert_bytes"]},
    }

    if use_graph and args.workload == "qwen-decode":
        # the layer with the step in front of it (hidden += delta, RMSNorm): one launch (mf_moe_decode_layer_normed)
        # against mf_residual_rmsnorm + mf_moe_decode_layer, the same 40 layers replayed from a graph
        hid = torch.randn((L, w["t"], w["d"]), generator=gen, device=device).to(torch.bfloat16)
        dlt = (torch.randn((L, w["t"], w["d"]), generator=gen, device=device) * 0.1).to(torch.bfloat16)
        nw = torch.ones((w["d"],), dtype=torch.bfloat16, device=device)
        xn = torch.zeros_like(hid)
        norm = ops.RMSNorm(ctx)

        def step_two():
            for l in range(L):
                norm.encode_bf16w(hid[l], nw, xn[l], w["d"], 1e-6, t=w["t"], delta=dlt[l])
                moes[l].encode_decode_layer(stack[l], xn[l], ys[l], t=w["t"], hidden=hid[l])

        def step_one():
            for l in range(L):
                moes[l].encode_decode_layer_normed(stack[l], hid[l], nw, ys[l], t=w["t"], delta=dlt[l], eps=1e-6)

        def graph_us(fn):
            s2 = torch.cuda.Stream()
            s2.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s2):
                fn()
            torch.cuda.current_stream().wait_stream(s2)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                fn()
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(max(1, K // 2)):
                g.replay()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / max(1, K // 2) * 1e3 / L

        out["layer_with_norm_in_front"] = {
            "us_per_layer_two_launches": round(graph_us(step_two), 3),
            "us_per_layer_one_launch": round(graph_us(step_one), 3),
            "what": "hidden += delta, x = RMSNorm(hidden) * w, y = layer(x), hidden += y per layer "
                    "(RealForwardRunner.swift:2799-2808 and the layer behind it); the two forms give the same bits"}
        for m in moes:
            m.status()
    if not args.no_prefill:
        out["prefill"] = measure_prefill(ctx, w, stack[0], device, use_graph=not args.no_graph)
    if not args.no_cpu_baseline:
        # the CPU checker (a restatement of the reference's CPU path: bulk
        # dequantize each row, scalar fp32 dot, experts in slot order) timed on
        # layer 0 for about cpu-seconds of work
        cores = int(os.environ.get("OMP_NUM_THREADS") or min(16, os.cpu_count() or 1))
        xb = ops.bf16_bits(x0)
        n = 0
        t_start = time.perf_counter()
        while True:
            O.moe_layer(host0, xb)
            n += 1
            el = time.perf_counter() - t_start
            if el >= args.cpu_seconds or n >= 2000:
                break
        out["cpu_baseline"] = {"value": round(el / n * 1e6, 1), "unit": "us", "cores": cores,
                               "kind": "port",
                               "sample": f"{n} repetitions of layer 0 of the same workload "
                                         f"(OpenMP over weight rows, {cores} threads)"}
        prev = _omp_threads(1)  # the same on one core
        if prev:
            n1, t1 = 0, time.perf_counter()
            while True:
                O.moe_layer(host0, xb)
                n1 += 1
                el1 = time.perf_counter() - t1
                if el1 >= args.cpu_seconds / 3 or n1 >= 2000:
                    break
            _omp_threads(prev)
            out["cpu_baseline_single_thread"] = {"value": round(el1 / n1 * 1e6, 1), "unit": "us", "cores": 1,
                                                 "kind": "port", "sample": f"{n1} repetitions of layer 0, one thread"}
    if args.pmc_calibration:
        out["pmc_calibration"] = pmc_calibration(device)
    if args.workload == "qwen-decode" and not args.tokens and not args.no_other_configs and not args.layers:
        # free the stack first: the children build their own weights on the same GPU
        del stack, moes, graph, run
        torch.cuda.empty_cache()
        out["other_configs"] = measure_other_configs(cpu_seconds=min(args.cpu_seconds, 2.0))
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
