#!/usr/bin/env python3
"""Writes tests/golden/blocks.npz: per block type, four known-answer blocks and one seeded 8 x 256 weight with
its packed bytes, its dequantised values and the float64 product with a seeded activation.

The vectors come from this repository's CPU oracle (the reference is Rust and cannot be run in this image);
they freeze the oracle's behaviour so that a later change to it, or a GPU path that drifts, shows up as a diff
against committed data.  Hand-computed known answers that pin the oracle itself live in
tests/test_oracle_codecs.py.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as o  # noqa: E402

TYPES = [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.F16, o.F32, o.Q4_K, o.Q6_K, o.Q5_K]


def kat_inputs(block):
    i = np.arange(block, dtype=np.float32)
    return np.stack([
        np.zeros(block, np.float32),                       # zero block: scale 1.0 rule
        i - block / 2,                                     # ramp
        np.where(i % 2 == 0, 0.5, -2.5).astype(np.float32) * (1 + (i % 7)),  # half-way quotients
        ((i * 37) % 11 - 5).astype(np.float32) / 8 + 1.0,  # offset data (min != 0)
    ])


def main():
    out = {}
    rng = np.random.default_rng(20240611)
    w = (rng.standard_normal((8, 256)) * 0.02).astype(np.float32)
    w[rng.random(w.shape) < 0.01] = 0.5
    x = rng.standard_normal((3, 256)).astype(np.float32)
    out["w"] = w
    out["x"] = x
    for t in TYPES:
        name = o.TYPE_NAMES[t]
        block = 256 if t in (o.Q4_K, o.Q6_K, o.Q5_K) else 32
        kin = kat_inputs(block)
        out[f"{name}.kat_in"] = kin
        out[f"{name}.kat_packed"] = np.stack([o.quantize(t, r) for r in kin])
        out[f"{name}.kat_deq"] = np.stack([o.dequantize(t, o.quantize(t, r), block) for r in kin])
        packed = o.quantize(t, w)
        deq = o.dequantize(t, packed, w.size).reshape(w.shape)
        out[f"{name}.packed"] = packed
        out[f"{name}.deq"] = deq
        out[f"{name}.y64"] = x.astype(np.float64) @ deq.astype(np.float64).T
    np.savez_compressed(os.path.join(HERE, "blocks.npz"), **out)
    print("wrote", os.path.join(HERE, "blocks.npz"), os.path.getsize(os.path.join(HERE, "blocks.npz")), "bytes")


if __name__ == "__main__":
    main()
