"""Writes tests/golden/lookupffn_golden.json: small known-answer vectors for the
LookupFFN hot path, derived from closed forms only (numpy + python integers; no
oracle, no reference code is imported).

  hadamard   H_8 and H_16 from H[i,j] = (-1)^popcount(i & j), and x.H for an
             integer x (exact in any float format)
  codes      all 256 sign patterns of 8 values -> MSB-first code
             (PL/compute_code_score/kernel.py:32-34: mask 2^(k-1-d))
  score      sum|z| / prod(1 + exp(-2|z|)) at hand-checkable points, computed
             with python's math in double precision
  gather     4 tokens x 2 tables x 3 entries x 64 columns with small-integer rows
             and weights: exact in float32, summed with python integers

Run:  python tests/golden/make_golden.py
"""
import json
import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def popcount(v):
    return bin(v).count("1")


def hadamard(D):
    return [[(-1) ** popcount(i & j) for j in range(D)] for i in range(D)]


def main():
    g = {}
    rng = np.random.RandomState(1234)
    had = {}
    for D in (8, 16):
        H = hadamard(D)
        x = rng.randint(-9, 10, size=(3, D)).tolist()
        y = [[sum(xr[i] * H[i][j] for i in range(D)) for j in range(D)] for xr in x]
        had[str(D)] = {"H": H, "x": x, "xH": y}
    g["hadamard"] = had

    pats, codes = [], []
    for p in range(256):
        bits = [(p >> (7 - d)) & 1 for d in range(8)]  # d = 0 is the MSB
        # magnitudes vary so that the test does not depend on |z|
        z = [(1.0 + 0.25 * d) * (1 if b else -1) for d, b in enumerate(bits)]
        pats.append(z)
        codes.append(p)
    g["codes"] = {"z": pats, "code": codes}

    pts = [
        [0.0] * 8,                       # 0 / 2^8 = 0
        [50.0] * 8,                      # exp(-100) ~ 0 -> 400
        [-50.0] * 8,                     # same, signs do not matter
        [0.5, -0.25, 1.0, -2.0, 0.0, 3.0, -0.125, 0.75],
        [1.0],                           # k = 1: |z| * sigmoid(2|z|)
        [0.3, -0.7],                     # k = 2
    ]
    scores = []
    for z in pts:
        num = sum(abs(v) for v in z)
        den = 1.0
        for v in z:
            den *= 1.0 + math.exp(-2.0 * abs(v))
        scores.append(num / den)
    g["score"] = {"z": pts, "score": scores}

    B, T, S, Do = 4, 2, 3, 64
    tables = rng.randint(-8, 9, size=(T, S, Do))
    code = rng.randint(0, S, size=(B, T))
    w = rng.randint(-4, 5, size=(B, T))
    out = np.zeros((B, Do), dtype=np.int64)
    for b in range(B):
        for t in range(T):
            out[b] += int(w[b, t]) * tables[t, code[b, t]].astype(np.int64)
    gout = rng.randint(-5, 6, size=(B, Do))
    gw = np.zeros((B, T), dtype=np.int64)
    gt = np.zeros((T, S, Do), dtype=np.int64)
    for b in range(B):
        for t in range(T):
            gw[b, t] = int((gout[b].astype(np.int64) * tables[t, code[b, t]]).sum())
            gt[t, code[b, t]] += int(w[b, t]) * gout[b]
    g["gather"] = {
        "tables": tables.tolist(), "code": code.tolist(), "w": w.tolist(), "out": out.tolist(),
        "g_out": gout.tolist(), "g_w": gw.tolist(), "g_tables": gt.tolist(),
    }

    with open(os.path.join(HERE, "lookupffn_golden.json"), "w") as f:
        json.dump(g, f)
    print("wrote lookupffn_golden.json")


if __name__ == "__main__":
    main()
