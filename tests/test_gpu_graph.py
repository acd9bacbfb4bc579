"""HIP-graph capture of the encode entry points: every replay against the eager call.

The entry points launch kernels only (no allocation, no memset, no synchronisation), so a caller may
record them into a graph.  Each test replays its graph several times, with eager work of the same
operator and synchronisations between the replays, on inputs that change from replay to replay, and
checks every replay bit for bit against the eager result."""
import numpy as np
import pytest
import torch

from helpers import ROOT_SEED, make_moe, to_device_layer
from mference_amd import operators as ops

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
    return graph


@pytest.mark.parametrize("bits,d,f,e,k,fs,t,fused", [
    (4, 2048, 512, 32, 8, 512, 1, True),     # the shape-specialised fused launch
    (4, 512, 256, 32, 8, 256, 4, True),
    (4, 512, 256, 32, 8, 256, 4, False),     # the chain of separate launches
    (2, 512, 256, 16, 6, 128, 2, True),
    (1, 256, 128, 32, 8, 0, 3, True),
])
def test_decode_layer_replays_equal_eager(gpu, oracle, bits, d, f, e, k, fs, t, fused):
    root = ROOT_SEED + 0xC000 + bits + d
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=1 if bits == 1 else 0)
    moe = make_moe(gpu, layer)
    moe.set_fused(fused)
    wts = to_device_layer(layer)
    x = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros_like(x)
    hidden = torch.zeros_like(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    graph = _capture(lambda: moe.encode_decode_layer(wts, x, y, t=t, hidden=hidden, out_indices=idx))
    for rep in range(4):
        xr = ops.bf16_tensor(oracle.synth_x(root + rep, t, d))
        hr = ops.bf16_tensor(oracle.synth_x(root + 100 + rep, t, d))
        # eager result on buffers of its own
        ye, he = torch.zeros_like(x), hr.clone()
        idxe = torch.zeros_like(idx)
        moe.encode_decode_layer(wts, xr, ye, t=t, hidden=he, out_indices=idxe)
        moe.status()
        x.copy_(xr)
        hidden.copy_(hr)
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        moe.status()
        assert torch.equal(idx, idxe), f"replay {rep}"
        assert torch.equal(y.view(torch.int16), ye.view(torch.int16)), f"replay {rep}"
        assert torch.equal(hidden.view(torch.int16), he.view(torch.int16)), f"replay {rep}"


@pytest.mark.parametrize("bits,d,f,e,k,fs,t", [(4, 512, 256, 32, 8, 256, 200), (2, 512, 256, 32, 6, 256, 150),
                                               (1, 512, 256, 32, 8, 0, 90)])
def test_prefill_layer_replays_equal_eager(gpu, oracle, bits, d, f, e, k, fs, t):
    """the routing (and with it the tile list, the grouping scratch and every launch's work) changes
    from replay to replay; grid sizes are fixed by t, so the recorded launches stay valid"""
    root = ROOT_SEED + 0xC100 + bits
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=1 if bits == 1 else 0)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    x = ops.bf16_tensor(oracle.synth_x(root, t, d))
    y = torch.zeros_like(x)
    idx = torch.zeros((t, k), dtype=torch.int32, device="cuda")
    ws = moe.encode_prefill_layer(wts, x, y, t, out_indices=idx)   # allocates the workspace
    torch.cuda.synchronize()
    graph = _capture(lambda: moe.encode_prefill_layer(wts, x, y, t, out_indices=idx, workspace=ws))
    seen = set()
    for rep in range(4):
        xr = ops.bf16_tensor(oracle.synth_x(root + 1 + rep, t, d))
        ye = torch.zeros_like(x)
        idxe = torch.zeros_like(idx)
        moe.encode_prefill_layer(wts, xr, ye, t, out_indices=idxe)   # eager, workspace of its own
        torch.cuda.synchronize()
        x.copy_(xr)
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(idx, idxe), f"replay {rep}"
        assert torch.equal(y.view(torch.int16), ye.view(torch.int16)), f"replay {rep}"
        seen.add(idx.cpu().numpy().tobytes())
    assert len(seen) == 4   # the replays did route differently


@pytest.mark.parametrize("bits,d,f,e,k,fs,t", [(4, 2048, 512, 256, 8, 512, 1), (4, 512, 256, 32, 8, 256, 6)])
def test_normed_decode_layer_replays_equal_eager(gpu, oracle, bits, d, f, e, k, fs, t):
    """the layer with the residual add and the norm in its own launch: hidden is read at the start of the launch and
    written at its end, replay after replay"""
    root = ROOT_SEED + 0xC200 + d
    layer = oracle.synth_layer(root, d, f, e, k, bits=bits, fs=fs)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    nw = ops.bf16_tensor(oracle.bf16_bits(1.0 + oracle.Rng.key(root, "nw").normal(0.0, 0.1, d)))
    hidden = torch.zeros((t, d), dtype=torch.bfloat16, device="cuda")
    delta = torch.zeros_like(hidden)
    y = torch.zeros_like(hidden)
    graph = _capture(lambda: moe.encode_decode_layer_normed(wts, hidden, nw, y, t, delta=delta, eps=1e-6))
    for rep in range(4):
        hr = ops.bf16_tensor(oracle.synth_x(root + rep, t, d))
        dr = ops.bf16_tensor(oracle.synth_x(root + 50 + rep, t, d))
        ye, he = torch.zeros_like(y), hr.clone()
        moe.encode_decode_layer_normed(wts, he, nw, ye, t, delta=dr, eps=1e-6)
        moe.status()
        hidden.copy_(hr)
        delta.copy_(dr)
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        moe.status()
        assert torch.equal(y.view(torch.int16), ye.view(torch.int16)), f"replay {rep}"
        assert torch.equal(hidden.view(torch.int16), he.view(torch.int16)), f"replay {rep}"
