"""Committed golden vectors (tests/golden/*.npz, written by make_golden.py):
the oracle must keep reproducing them (CPU), and the HIP path must match them
through the C ABI (GPU): routing bit-exact, outputs within the layer tolerance."""
import glob
import os

import numpy as np
import pytest

from helpers import assert_layer_close

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def _load(path, oracle):
    z = np.load(path, allow_pickle=False)
    d, f, e, k, bits, fs, t, mode = (int(v) for v in z["shape"])
    off = oracle.ExpertOffsets()
    for (name, _), v in zip(off._fields_, z["offsets"]):
        setattr(off, name, int(v))
    shared = None
    if fs:
        shared = tuple(oracle.QTensor(z[n + "_packed"], z[n + "_scales"], z[n + "_biases"], 4,
                                      *z[n + "_scales"].shape[:1], z[n + "_scales"].shape[1] * 64)
                       for n in ("sg", "su", "sd"))
    layer = oracle.Layer(d=d, f=f, e=e, k=k, bits=bits, router_w=z["router_w"], experts=z["experts"],
                         off=off, fs=fs, shared=shared, w_sg=z["w_sg"] if fs else None,
                         router_mode=mode)
    return z, layer, t


def test_fixtures_exist():
    assert len(FILES) >= 3


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p)[:-4] for p in FILES])
def test_oracle_reproduces_golden(path, oracle):
    z, layer, t = _load(path, oracle)
    y, idx, w = oracle.moe_layer(layer, z["x"])
    assert np.array_equal(idx, z["idx"])
    assert np.array_equal(w.view(np.uint32), z["w"].view(np.uint32))
    assert np.array_equal(y, z["y"])
    for i in range(t):
        assert np.array_equal(oracle.router_logits(layer.router_w, z["x"][i]).view(np.uint32),
                              z["logits"][i].view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(p)[:-4] for p in FILES])
def test_hip_matches_golden(path, oracle, gpu):
    import torch
    from mference_amd import operators as ops
    from helpers import make_moe, to_device_layer
    z, layer, t = _load(path, oracle)
    moe = make_moe(gpu, layer)
    wts = to_device_layer(layer)
    y = torch.zeros((t, layer.d), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((t, layer.k), dtype=torch.int32, device="cuda")
    w = torch.zeros((t, layer.k), dtype=torch.float32, device="cuda")
    lg = torch.zeros((t, layer.e), dtype=torch.float32, device="cuda")
    moe.encode_router(wts.router_w, ops.bf16_tensor(z["x"]), idx, w, t=t, out_logits=lg)
    torch.cuda.synchronize()
    assert np.array_equal(lg.cpu().numpy().view(np.uint32), z["logits"].view(np.uint32))
    moe.encode_decode_layer(wts, ops.bf16_tensor(z["x"]), y, t=t, out_indices=idx, out_weights=w)
    moe.status()
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), z["idx"])
    assert np.array_equal(w.cpu().numpy().view(np.uint32), z["w"].view(np.uint32))
    assert_layer_close(oracle.bf16_to_float(ops.bf16_bits(y)), oracle.bf16_to_float(z["y"]),
                       os.path.basename(path))
