"""Writes tests/golden/tower_golden.npz: inputs and expected outputs of two
small seeded networks, computed by an independent float64 model that uses
direct 3x3 convolutions (torch conv2d) instead of Winograd transforms and
numpy for the heads.  The reference engine cannot be run in this image, so
these vectors come from the mathematics of the network definition; they let
both the CPU oracle and the HIP path be checked on a machine that has neither
torch-free tooling nor the reference tree.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import __graft_entry__ as entry  # noqa: E402
from helpers import heads_f64, tower_f64  # noqa: E402


def main():
    entry.load_package()
    import leela_zero_amd.netgen as netgen
    out = {}
    for tag, blocks, filters, seed, n in (("b1f8", 1, 8, 101, 3), ("b2f16", 2, 16, 102, 3)):
        net = netgen.make_network(blocks, filters, seed)
        x = netgen.synthetic_inputs(n, seed + 1000)
        t = tower_f64(net, x)
        hd = [heads_f64(net, t["pol"][i], t["val"][i]) for i in range(n)]
        out[tag + "_cfg"] = np.array([blocks, filters, seed], np.int64)
        out[tag + "_x"] = x
        out[tag + "_pol"] = t["pol"]
        out[tag + "_val"] = t["val"]
        out[tag + "_policy"] = np.stack([h["policy"] for h in hd])
        out[tag + "_logits"] = np.stack([h["logits"] for h in hd])
        out[tag + "_value"] = np.array([h["value"] for h in hd])
    np.savez_compressed(os.path.join(HERE, "tower_golden.npz"), **out)


if __name__ == "__main__":
    main()
