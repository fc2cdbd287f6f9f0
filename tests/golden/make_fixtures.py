#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/.

The reference (SSIGPRO/mamtorch) holds no golden vectors for this path: its tests are unseeded
and print-only.  The fixtures are therefore
  * kat.json          -- known answers derived by hand from the definition (products listed in
                         the comments), and
  * brute_small.npz   -- seeded small cases evaluated by oracle/brute.py, a pure-Python scalar
                         scan that shares no code with the C oracle or the PyTorch port.
Nothing of the reference is imported or run.  Usage: python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import brute  # noqa: E402

NEG0 = "-0.0"

KAT = [
    {   # products [2, -2, -3]: max 2 at k=0, min -3 at k=2, C = -1
        "name": "three_products",
        "a": [[1.0, -2.0, 3.0]], "b": [[2.0], [1.0], [-1.0]],
        "c": [[-1.0]], "argmax": [[0]], "argmin": [[2]],
        # a_grad = [b0*g, 0, b2*g] = [2g, 0, -g]; b_grad = [a0*g, 0, a2*g] = [g, 0, 3g]   (g = 1.5)
        "grad": [[1.5]], "a_grad": [[3.0, 0.0, -1.5]], "b_grad": [[1.5], [0.0], [4.5]],
    },
    {   # all products 5: first index wins both, the selected term counts twice in the backward
        "name": "all_equal",
        "a": [[1.0, 1.0, 1.0]], "b": [[5.0], [5.0], [5.0]],
        "c": [[10.0]], "argmax": [[0]], "argmin": [[0]],
        "grad": [[2.0]], "a_grad": [[20.0, 0.0, 0.0]], "b_grad": [[4.0], [0.0], [0.0]],
    },
    {   # column 0: products [-3, 6] -> C = 3, argmax 1, argmin 0
        # column 1: products [-0.0, +0.0]: equal under comparison, first index wins both,
        #           C = (-0.0) + (-0.0) = -0.0
        "name": "signed_zero_tie",
        "a": [[-1.0, 2.0]], "b": [[3.0, 0.0], [3.0, 0.0]],
        "c": [[3.0, NEG0]], "argmax": [[1, 0]], "argmin": [[0, 0]],
        "grad": [[1.0, 1.0]], "a_grad": [[3.0, 3.0]], "b_grad": [[-1.0, -2.0], [2.0, 0.0]],
    },
    {   # selection count: argmax picks (m=0,k=2) three times and (m=1,k=3) once
        "name": "selection_count",
        "sel_argmax": [[2, 3], [2, 3], [2, 1]], "sel_argmin": [[0, 0], [0, 0], [0, 0]],
        "M": 2, "K": 4,
        # reference mode: dedup per call, argmin also lands in max_count
        "ref_max_count": [[1, 0, 1, 0], [1, 1, 0, 1]],
        # hits mode
        "hits_max_count": [[0, 0, 3, 0], [0, 1, 0, 2]], "hits_min_count": [[3, 0, 0, 0], [3, 0, 0, 0]],
    },
]


def main():
    with open(os.path.join(HERE, "kat.json"), "w") as f:
        json.dump(KAT, f, indent=1)
    rng = np.random.default_rng(20240)
    out = {}
    shapes = [(3, 5, 4), (4, 9, 7), (2, 17, 3), (5, 8, 8), (1, 33, 2)]
    for i, (N, K, M) in enumerate(shapes):
        x = rng.standard_normal((N, K)).astype(np.float32)
        b = rng.standard_normal((K, M)).astype(np.float32)
        if i == 1:   # plant exact ties and zeros
            x[:, 3] = x[:, 1]
            b[3, :] = b[1, :]
            x[0, :] = 0.0
        if i == 3:   # quantised values: many equal products
            x = np.round(x * 2) / 2
            b = np.round(b * 2) / 2
        bias = rng.standard_normal(M).astype(np.float32)
        g = rng.standard_normal((N, M)).astype(np.float32)
        c, amax, amin = brute.forward(x, b, bias)
        xg, bg = brute.backward(x, b, g, amax, amin)
        for name, arr in (("x", x), ("b", b), ("bias", bias), ("grad", g), ("c", c), ("argmax", amax),
                          ("argmin", amin), ("x_grad", xg), ("b_grad", bg)):
            out["case%d_%s" % (i, name)] = arr
    np.savez(os.path.join(HERE, "brute_small.npz"), **out)
    print("wrote kat.json and brute_small.npz")


if __name__ == "__main__":
    main()
