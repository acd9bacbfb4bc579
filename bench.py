#!/usr/bin/env python3
"""Benchmark of the MoE expert hot path on one MI355X.

Workload (default): the Qwen3.6-35B-A3B-shaped 4-bit MoE layer at T=1 decode,
run as a 40-layer stack with independent weights per layer (hidden 2048, 256
routed experts of intermediate 512, top-8, one shared expert of intermediate
512 gated by sigmoid(w_sg.x)).  A "step" is one token through the whole stack:
the 40 layers run back to back on one stream, each on its own input row and its
own weights, so every layer streams its expert bytes from HBM (40 x 453 MB of
resident experts, far beyond the 256 MB Infinity Cache).

Prints ONE JSON line (see README / DESIGN.md for the field meanings).
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


def algorithmic_bytes(w) -> dict:
    """Bytes one layer must read at T=1: the K selected experts + the shared
    expert ("expert bytes touched"), and the same plus router, w_sg, x and y."""
    def tensor(rows, cols, bits):
        return rows * cols * bits // 8 + 2 * rows * (cols // 64) * 2
    expert = 2 * tensor(w["f"], w["d"], w["bits"]) + tensor(w["d"], w["f"], w["bits"])
    shared = (2 * tensor(w["fs"], w["d"], w["shared_bits"]) + tensor(w["d"], w["fs"], w["shared_bits"])
              if w["fs"] else 0)
    expert_bytes = w["k"] * expert + shared
    total = expert_bytes + w["e"] * w["d"] * 2 + w["d"] * 2 + 2 * w["d"] * 2
    return dict(expert=expert, expert_bytes=expert_bytes, total=total)


def build_stack(ctx, w, layers, device):
    """Random-init weights of the named architecture, drawn on the GPU
    (N(0, 0.02), seeded per layer) and quantized by the library's own device
    quantizer into resident expert blobs."""
    import torch
    from mference_amd import operators as ops
    from oracle import mf_oracle as O  # blob layout helper only (host arithmetic)

    quant = ops.Quantization(ctx)
    off_h, _, stride = O.blob_layout(w["d"], w["f"], w["bits"])
    off = ops.MoEExpertOffsets()
    for name, _ in off._fields_:
        setattr(off, name, getattr(off_h, name))
    stack = []
    E, D, F = w["e"], w["d"], w["f"]
    for l in range(layers):
        gen = torch.Generator(device=device)
        gen.manual_seed((ROOT_SEED + 0x100 * w["config"] + l) & 0x7FFFFFFFFFFFFFFF)
        experts = torch.zeros((E, stride), dtype=torch.uint8, device=device)
        for name, rows, cols in (("gate", F, D), ("up", F, D), ("down", D, F)):
            raw = torch.randn((E * rows, cols), generator=gen, device=device,
                              dtype=torch.float32) * 0.02
            q = quant.quantize_affine(raw, w["bits"])
            del raw
            wo, so, bo = (getattr(off, f"{name}_{s}") for s in "wsb")
            nb = q.packed.shape[1] * rows
            experts[:, wo:wo + nb] = q.packed.view(E, nb)
            ns = q.scales.shape[1] * rows * 2
            experts[:, so:so + ns] = q.scales.view(torch.uint8).view(E, ns)
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


def layer_to_host(wts, w):
    """device layer -> oracle Layer (for the parity check and the CPU baseline)"""
    from mference_amd import operators as ops
    from oracle import mf_oracle as O
    off = O.ExpertOffsets()
    for name, _ in off._fields_:
        setattr(off, name, getattr(wts.offsets, name))
    def q(t):
        return O.QTensor(t.packed.cpu().numpy(), ops.bf16_bits(t.scales), ops.bf16_bits(t.biases),
                         t.bits, t.rows, t.n)
    shared = None if wts.shared is None else tuple(q(t) for t in wts.shared)
    return O.Layer(d=w["d"], f=w["f"], e=w["e"], k=w["k"], bits=w["bits"],
                   router_w=ops.bf16_bits(wts.router_w), experts=wts.experts.cpu().numpy(), off=off,
                   fs=w["fs"], shared_bits=w["shared_bits"], shared=shared,
                   w_sg=None if wts.w_sg is None else ops.bf16_bits(wts.w_sg))


def profiled_traffic_bytes():
    """HBM bytes per launch of the fused kernel from the committed rocprofv3 --pmc
    summary (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size)."""
    import re
    path = os.path.join(ROOT, "profiles", "fused_decode_qwen_t1.md")
    try:
        m = re.search(r"Traffic per launch = \*\*([0-9,]+) B\*\*", open(path).read())
        return int(m.group(1).replace(",", "")) if m else None
    except OSError:
        return None


def measure_prefill(ctx, w, layer, device, tokens=(128, 512, 2048), steps=100, warmup=100):
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
    moe = ops.MoE(ctx, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                  shared_bits=w["shared_bits"])
    out = {"workload": "qwen3.6-35b-a3b-moe-layer-ragged-prefill-4bit-g64, skewed routing",
           "dtype": "u4 codes (exact, as bf16) x bf16 activations on bf16 MFMA, fp32 accumulate",
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
            ref_y, ref_idx, _ = O.moe_layer(host, ops.bf16_bits(x))
            got = O.bf16_to_float(ops.bf16_bits(y)).astype(np.float64)
            ref = O.bf16_to_float(ref_y).astype(np.float64)
            run["parity"] = dict(
                routing_bit_exact=bool(np.array_equal(idx.cpu().numpy().astype(np.uint32), ref_idx)),
                max_abs=float(np.abs(got - ref).max()),
                rel_l2=float(np.linalg.norm(got - ref) / np.linalg.norm(ref)))
        for _ in range(warmup):
            moe.encode_prefill_layer(lw, x, y, t, workspace=ws)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            moe.encode_prefill_layer(lw, x, y, t, workspace=ws)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / steps * 1e3
        flops = 2.0 * 3 * w["d"] * (t * w["k"] * w["f"] + t * w["fs"])
        tflops = flops / us / 1e6
        run.update(us_per_layer=round(us, 1), tokens_per_s=round(t / us * 1e6, 1),
                   tflops=round(tflops, 1), mfma_frac=round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
                   experts_without_tokens=int((counts == 0).sum()), max_expert_load=int(counts.max()),
                   output_finite=bool(torch.isfinite(y.float()).all().item()))
        out["runs"].append(run)
    last = out["runs"][-1]
    out["roofline"] = {"bound": "mfma", "achieved": last["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                       "unit": "TFLOP/s", "frac": last["mfma_frac"], "traffic": None,
                       "kernel": "whole layer at T=%d (router, grouping, mf::qmm_kernel x4, reduce); "
                                 "algorithmic flops = 2*3*D*(T*K*F + T*Fs)" % last["tokens"]}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=40)
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a kernel of known HBM "
                         "traffic) so that FETCH_SIZE / WRITE_SIZE counters can be scaled")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--no-prefill", action="store_true", help="skip the ragged prefill section")
    ap.add_argument("--prefill-only", action="store_true",
                    help="one layer, the ragged prefill section only (for profiling)")
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
    w = QWEN
    L, K, W = args.layers, args.steps, args.warmup
    if args.prefill_only:
        L = 1
    ctx = ops.MetalContext(0)
    stack = build_stack(ctx, w, L, device)
    if args.prefill_only:
        print(json.dumps({"prefill": measure_prefill(ctx, w, stack[0], device)}))
        return 0
    moes = [ops.MoE(ctx, w["d"], w["f"], w["e"], w["k"], bits=w["bits"], shared_f=w["fs"],
                    shared_bits=w["shared_bits"]) for _ in range(L)]

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
    for m in moes:
        m.status()
    finite = bool(torch.isfinite(ys.float()).all().item())

    ab = algorithmic_bytes(w)
    achieved = ab["expert_bytes"] / (us_per_layer * 1e-6) / 1e9
    out = {
        "metric": "us_per_moe_layer_decode_T1",
        "value": round(us_per_layer, 4),
        "unit": "us",
        "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u4 codes x bf16 activations, fp32 accumulate",
        "data": "synthetic (random-init N(0,0.02) weights quantized 4-bit g64 on device; x ~ N(0,1))",
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
                     "traffic": profiled_traffic_bytes(),
                     "kernel": "mf::fused_decode_kernel (one launch per layer)",
                     "algorithmic_bytes_per_layer": ab["expert_bytes"]},
    }

    if not args.no_prefill:
        out["prefill"] = measure_prefill(ctx, w, stack[0], device)
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
    if args.pmc_calibration:
        src = torch.zeros(256 << 20, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["pmc_calibration"] = "3 x 256 MiB device-to-device copy (reads 268435456 B, writes 268435456 B)"
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
