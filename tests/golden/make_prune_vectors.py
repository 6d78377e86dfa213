#!/usr/bin/env python3
"""Writes tests/golden/prune_vectors.npz: inputs and outputs of the reference's TW mask
producers on small seeded inputs.

Run in the development container only (it needs /root/reference):

    python tests/golden/make_prune_vectors.py

It imports the NumPy-only module Pruning/VGG/prune_algo.py of the reference and calls
img2col_forward, tiled_wise_1d, tiled_wise_2d, tiled_wise_1d_mix and tiled_wise_2d_mix on
synthetic scores.  The fixture holds data
only: the seeds' score tensors (float32), the call parameters and the returned masks (packed
bits).  The NumPy version that executed the reference is recorded, because np.percentile's
arithmetic type depends on it.
"""
import importlib.util
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/Pruning/VGG/prune_algo.py"

CASES = [
    # name, shapes (2-D dense or 4-D HWIO conv), granularity, sparsities, seed, quantise
    ("mlp_small", [(40, 50), (64, 130), (17, 16)], 16, [50, 75.0, 90], 11, 0),
    ("conv_mix", [(3, 3, 8, 40), (96, 72), (1, 1, 32, 33)], 32, [25, 60.5], 12, 0),
    ("ties", [(48, 64), (32, 96)], 32, [50, 75], 13, 4),        # scores on a coarse grid: tied norms
    ("one_layer_g128", [(130, 300)], 128, [75], 14, 0),
    ("tiny", [(3, 5)], 2, [40, 0, 100], 15, 0),
]


def main():
    spec = importlib.util.spec_from_file_location("ref_prune_algo", REF)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    out = {}
    meta = {"numpy": np.__version__, "source": "Pruning/VGG/prune_algo.py", "cases": []}
    for name, shapes, g, sparsities, seed, quant in CASES:
        rng = np.random.default_rng(seed)
        weights = []
        for s in shapes:
            w = rng.standard_normal(s).astype(np.float32)
            if quant:
                w = (np.round(w * quant) / quant).astype(np.float32)
            weights.append(w)
        scores = ref.img2col_forward(weights)
        for i, w in enumerate(weights):
            out["%s/w%d" % (name, i)] = w
        for sp in sparsities:
            for fn in ("tiled_wise_1d", "tiled_wise_2d"):
                masks = getattr(ref, fn)(scores, sp, g)
                for i, m in enumerate(masks):
                    m = np.asarray(m)
                    out["%s/%s/%s/m%d" % (name, fn, repr(sp), i)] = np.packbits(m.astype(bool), axis=None)
        # the mixed producers (TW at sparsity + g1percent, then the element-wise remainder)
        mix = []
        for sp in sparsities:
            for fn, g1 in (("tiled_wise_1d_mix", 5), ("tiled_wise_2d_mix", 1),
                           ("tiled_wise_1d_mix", 2.5)):
                if sp + g1 > 100:
                    continue
                masks = getattr(ref, fn)(scores, sp, g, g1)
                for i, m in enumerate(masks):
                    m = np.asarray(m)
                    out["%s/%s/%s/%s/m%d" % (name, fn, repr(sp), repr(g1), i)] = \
                        np.packbits(m.astype(bool), axis=None)
                mix.append([fn, repr(sp), repr(g1)])
        meta.setdefault("mix", {})[name] = mix
        meta["cases"].append(dict(name=name, shapes=[list(s) for s in shapes], granularity=g,
                                  sparsities=[repr(s) for s in sparsities], seed=seed, quantise=quant))
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(HERE, "prune_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out) - 1, "arrays")


if __name__ == "__main__":
    sys.exit(main())
