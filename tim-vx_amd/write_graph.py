#!/usr/bin/env python3
"""Writes a network's graph file pair for tvx_graph_runner.

  python tim-vx_amd/write_graph.py mobilenet_v2 --batch 64 --out DIR [--bench W K]
  python tim-vx_amd/write_graph.py lenet --weights tests/golden/lenet_asymu8.npz --out DIR
  tim-vx_amd/lib/tvx_graph_runner DIR/graphs.txt DIR/blob.bin DIR/out.bin
"""
import argparse
import importlib
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
GF = importlib.import_module("tim-vx_amd.graphfile")
G = importlib.import_module("tim-vx_amd.graphs")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("net", choices=["mobilenet_v2", "lenet"])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--res", type=int, default=224)
    ap.add_argument("--weights", help="npz with `weights` and `input` (lenet)")
    ap.add_argument("--out", required=True)
    ap.add_argument("--bench", type=int, nargs=2, metavar=("WARMUP", "ITERS"))
    a = ap.parse_args()
    if a.net == "lenet":
        z = np.load(a.weights)
        g = G.lenet_asymu8(z["weights"], z["input"], batch=a.batch)
    else:
        g = G.mobilenet_v2(batch=a.batch, res=a.res)
    os.makedirs(a.out, exist_ok=True)
    GF.write_graphs([g], os.path.join(a.out, "graphs.txt"), os.path.join(a.out, "blob.bin"),
                    tuple(a.bench) if a.bench else None)
    print("wrote", a.out, ":", len(g["ops"]), "operators,", G.mac_count(g), "MACs")


if __name__ == "__main__":
    main()
