"""Regenerate the golden fixtures of the SC convolution path.

The expected outputs come from the reference's own CPU kernel
(``torch_c/sc-extension/sc.cpp``, ``conv2d_add_partial_new``) compiled unmodified by
``oracle/build_oracle.py`` into ``oracle/_ref``; the reference's Python modules are not
imported.  Inputs follow the recipe in ``geo_amd/workloads.py``.  Two files are written
next to this script:

* ``fixtures_small.npz``  - inputs and int32 outputs of small cases (a few KB each)
* ``checksums.json``      - SHA-256 / sum / abs-sum / non-zero fraction of the int32
                            outputs of the full-size benchmark shapes (inputs are
                            regenerated from the seed wherever the check runs)

Run here (needs /root/reference for the build):  python tests/golden/make_fixtures.py [--big]
"""
from __future__ import annotations

import hashlib
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from geo_amd import workloads as wl  # noqa: E402
from oracle import sc_oracle as so  # noqa: E402

LENGTHS = (8, 16, 32, 64, 128, 256)


def ref_call(mod, x, w, L, pad):
    return mod.conv2d_add_partial_new(x, w, L, (pad, pad), (1, 1)).contiguous().numpy()


def small_cases():
    """name -> (x, w, L, pad)"""
    cases = {}
    for L in LENGTHS:
        x, w, pad, _ = wl.named("T1")
        cases[f"T1_L{L}"] = (x, w, L, pad)
    for name in ("T2", "T3", "T4"):
        x, w, pad, L = wl.named(name)
        cases[name] = (x, w, L, pad)
    # 1x1 kernel, odd channel counts
    x, w = wl.make_inputs((2, 7, 5, 6), (3, 7, 1, 1), "prescribed", seed=3)
    cases["K1x1_L32"] = (x, w, 32, 0)
    # 7-bit quantised inputs as the SC layer produces them, kaiming-scaled weights
    x, w = wl.make_inputs((2, 6, 7, 7), (5, 6, 3, 3), "q7", seed=5)
    cases["Q7_L128"] = (x, w, 128, 1)
    x, w = wl.make_inputs((1, 6, 7, 7), (5, 6, 3, 3), "q7", seed=6)
    cases["Q7_L256"] = (x, w, 256, 1)
    # sparse inputs, non-multiple-of-8/16 position counts (vector tails of the bit-matmul)
    x, w = wl.make_inputs((3, 9, 10, 7), (6, 9, 3, 2), "sparse", seed=7)
    cases["SPARSE_L64"] = (x, w, 64, 1)
    # values on and beyond the clamp edges: x<0, x=0, x=1, x>1, w=+-1, w=0, tiny w
    g = torch.Generator().manual_seed(11)
    x = torch.rand((2, 4, 6, 6), generator=g) * 1.6 - 0.3
    x.view(-1)[::7] = 1.0
    x.view(-1)[3::11] = 0.0
    w = torch.rand((5, 4, 3, 3), generator=g) * 2.6 - 1.3
    w.view(-1)[::5] = 0.0
    w.view(-1)[1::9] = 1.0
    w.view(-1)[2::9] = -1.0
    w.view(-1)[4::13] = 1.0 / 512
    w.view(-1)[6::13] = -1.0 / 512
    for L in (16, 64, 256):
        cases[f"EDGE_L{L}"] = (x.clone(), w.clone(), L, 1)
    # wide enough for several 16-position vector blocks plus a tail, 5 couts (4+1 tail)
    x, w = wl.make_inputs((2, 3, 9, 8), (5, 3, 3, 3), "prescribed", seed=13)
    cases["TAIL_L32"] = (x, w, 32, 1)
    return cases


def big_cases():
    """name -> (shape name, mode, L); the survey's checksum table"""
    out = {"C1_prescribed_L64": ("C1", "prescribed", 64)}
    for L in (32, 128, 256):
        out[f"C3_prescribed_L{L}"] = ("C3", "prescribed", L)
        out[f"C3_sparse_L{L}"] = ("C3", "sparse", L)
    for L in (128, 256):
        out[f"C3_kaiming_L{L}"] = ("C3", "kaiming", L)
        out[f"C3_q7_L{L}"] = ("C3", "q7", L)
    out["C5_prescribed_L256"] = ("C5", "prescribed", 256)
    out["C5_kaiming_L256"] = ("C5", "kaiming", 256)
    out["C5_sparse_L256"] = ("C5", "sparse", 256)
    out["C4_prescribed_L128"] = ("C4", "prescribed", 128)
    return out


def summary(y):
    return {
        "shape": list(y.shape),
        "sum": int(y.astype(np.int64).sum()),
        "abs_sum": int(np.abs(y.astype(np.int64)).sum()),
        "nonzero": float((y != 0).mean()),
        "sha256": hashlib.sha256(np.ascontiguousarray(y, dtype="<i4").tobytes()).hexdigest(),
    }


def main():
    variants = so.ref_variants_usable()
    if not variants:
        raise SystemExit("oracle/_ref is not built: run python oracle/build_oracle.py ref")
    mods = {v: so.load_ref(v) for v in variants}
    first = mods[variants[0]]

    arrays = {}
    for name, (x, w, L, pad) in small_cases().items():
        ys = {v: ref_call(m, x, w, L, pad) for v, m in mods.items()}
        y = ys[variants[0]]
        for v, yv in ys.items():
            assert np.array_equal(y, yv), f"{name}: reference ISA variants disagree ({v})"
        arrays[f"{name}/x"] = x.numpy()
        arrays[f"{name}/w"] = w.numpy()
        arrays[f"{name}/y"] = y.astype(np.int32)
        arrays[f"{name}/meta"] = np.array([L, pad], dtype=np.int32)
        print(name, tuple(y.shape), int(y.sum()), int(np.abs(y).sum()))
    np.savez_compressed(os.path.join(HERE, "fixtures_small.npz"), **arrays)

    path = os.path.join(HERE, "checksums.json")
    sums = {}
    if os.path.isfile(path):
        with open(path) as f:
            sums = json.load(f)
    if "--big" in sys.argv:
        for name, (shape, mode, L) in big_cases().items():
            x, w, pad, _ = wl.named(shape, mode)
            y = ref_call(first, x, w, L, pad)
            sums[name] = dict(summary(y), shape_name=shape, mode=mode, L=L, pad=pad)
            print(name, sums[name]["sha256"][:16], sums[name]["sum"], flush=True)
        with open(path, "w") as f:
            json.dump(sums, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
