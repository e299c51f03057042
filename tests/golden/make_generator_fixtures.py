#!/usr/bin/env python3
"""Writes tests/golden/generator_fixtures.json: first and last eight values (as exact hexadecimal
floats) and a SHA-256 of the bytes of every seeded input generator of the oracle, at the sizes
of the BASELINE configurations' operands where that is cheap.  tests/test_oracle.py compares the
generators with this file, so a change to a generator - and with it to every seeded test input -
cannot pass unnoticed.  Run from the repository root:  python tests/golden/make_generator_fixtures.py"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402

CASES = [
    ("uniform", dict(n=1024 * 1024, seed=1, dtype="float32")),       # config 1 operands
    ("uniform", dict(n=4097 * 1034 + 5, seed=2, dtype="float32")),   # config 3, A of (4097,4095,1031) TN with ld = rows + 3
    ("uniform", dict(n=100000, seed=3, dtype="float64")),
    ("uniform", dict(n=50000, seed=4, dtype="complex64")),
    ("normal", dict(n=1024 * 1024, seed=22, dtype="float64")),       # configs 4 and 5 draw B like this
    ("normal", dict(n=100000, seed=5, dtype="float32")),
    ("integers", dict(n=100000, seed=6, limit=30, dtype="float32")),
    ("integers", dict(n=100000, seed=7, limit=1000, dtype="float64")),
    ("triangular", dict(n=512, ld=515, lower=True, seed=21, dtype="float64")),   # config 5's A, smaller order
    ("triangular", dict(n=300, ld=300, lower=False, seed=8, dtype="float32")),
]


def generate(kind, kw):
    kw = dict(kw)
    dtype = np.dtype(kw.pop("dtype"))
    if kind == "uniform":
        return oracle.uniform(kw["n"], kw["seed"], dtype.type)
    if kind == "normal":
        return oracle.normal(kw["n"], kw["seed"], dtype.type)
    if kind == "integers":
        return oracle.integers(kw["n"], kw["seed"], kw["limit"], dtype.type)
    return oracle.triangular(kw["n"], kw["ld"], kw["lower"], kw["seed"], dtype.type)


def describe(a):
    flat = a.view(np.float32 if a.dtype in (np.float32, np.complex64) else np.float64)
    return {"first8": [float(x).hex() for x in flat[:8]], "last8": [float(x).hex() for x in flat[-8:]],
            "sha256": hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest(), "count": int(flat.size)}


if __name__ == "__main__":
    out = []
    for kind, kw in CASES:
        out.append({"generator": kind, "args": kw, **describe(generate(kind, kw))})
    with open(os.path.join(HERE, "generator_fixtures.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote %d fixtures" % len(out))
