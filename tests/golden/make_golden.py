"""Writes tests/golden/*.npz: small seeded input/output vectors of the hot path,
produced by the CPU oracle (oracle/).  Run from the repository root:

    python tests/golden/make_golden.py

The fixtures are data only (inputs, packed weights, expected outputs).  Header
of every file: the seed recipe.  Inputs are regenerated from
SeedTree(root).key(label) streams (SplitMix64, Box-Muller normals); root =
0x4D464D4F00000000 + 0x100 * config + layer.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import mf_oracle as O  # noqa: E402

ROOT_SEED = 0x4D464D4F00000000
RECIPE = ("SeedTree(root).key(label) -> SplitMix64; N(0,sigma) by Box-Muller in fp64; labels: x, router, "
          "shared.gate|up|down, w_sg, expert<i>.gate|up|down; weights MLX-affine g64")

CASES = {
    # name: (config id, d, f, e, k, bits, fs, t, router_mode)
    "layer_q4_d128_f64_e16_k8_shared": (0x10, 128, 64, 16, 8, 4, 64, 2, 0),
    "layer_q2_d256_f128_e8_k6_shared": (0x40, 256, 128, 8, 6, 2, 128, 1, 0),
    "layer_ternary_d256_f128_e32_k8_fullsoftmax": (0x50, 256, 128, 32, 8, 1, 0, 2, 1),
}


def main():
    for name, (cfg, d, f, e, k, bits, fs, t, mode) in CASES.items():
        root = ROOT_SEED + 0x100 * cfg
        layer = O.synth_layer(root, d, f, e, k, bits=bits, fs=fs, router_mode=mode)
        x = O.synth_x(root, t, d)
        y, idx, w = O.moe_layer(layer, x)
        logits = np.stack([O.router_logits(layer.router_w, x[i]) for i in range(t)])
        out = dict(recipe=np.array(RECIPE), root=np.array(root, np.uint64),
                   shape=np.array([d, f, e, k, bits, fs, t, mode], np.int64),
                   x=x, router_w=layer.router_w, experts=layer.experts,
                   offsets=np.array([getattr(layer.off, n) for n, _ in layer.off._fields_], np.uint32),
                   logits=logits, idx=idx, w=w, y=y)
        if fs:
            for nm, q in zip(("sg", "su", "sd"), layer.shared):
                out[nm + "_packed"], out[nm + "_scales"], out[nm + "_biases"] = q.packed, q.scales, q.biases
            out["w_sg"] = layer.w_sg
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
        print(name, "ok", os.path.getsize(os.path.join(HERE, name + ".npz")), "bytes")


if __name__ == "__main__":
    main()
