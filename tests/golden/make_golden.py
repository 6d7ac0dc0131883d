"""Writes the committed golden fixtures of this directory.

* kat_forward.json — the reference's only known-answer test, testing/test.cpp:13-47 (values typed
  from that test: features, lookup, weights and the expected forward result).
* dense_*.npz — seeded inputs on three small shapes of the reference's grid (testing/test.cpp:50-59)
  with float64 results of the dense formulation out = X.D, gx = G.D^T, gw = (X^T G)[lookup, j]
  (the ground truth the reference's randomised tests compare against, reference.cpp:15-82),
  computed here with plain numpy loops that share no code with oracle/.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def dense_results(x, lookup, w, g):
    B, N = x.shape
    L, K = lookup.shape
    D = np.zeros((N, L), dtype=np.float64)
    for j in range(L):
        for k in range(K):
            D[lookup[j, k], j] += float(w[j, k])
    out = x.astype(np.float64) @ D
    gx = g.astype(np.float64) @ D.T
    xtg = x.astype(np.float64).T @ g.astype(np.float64)
    gw = np.zeros((L, K), dtype=np.float64)
    for j in range(L):
        for k in range(K):
            gw[j, k] = xtg[lookup[j, k], j]
    return out, gx, gw


def main():
    kat = {
        "source": "testing/test.cpp:13-47",
        "features": [[1.0, 2.0, 3.0], [4.0, 5.0, 6.0], [0.0, 1.0, 1.0]],
        "lookup": [[1, 2], [0, 2]],
        "weights": [[1.0, 2.0], [3.0, 4.0]],
        "expected": [[8.0, 15.0], [17.0, 36.0], [3.0, 4.0]],
    }
    with open(os.path.join(HERE, "kat_forward.json"), "w") as f:
        json.dump(kat, f, indent=1)

    for (B, N, L, K) in [(3, 5, 4, 2), (12, 8, 8, 4), (17, 12, 63, 44)]:
        rng = np.random.default_rng(1000 + B + L)
        x = rng.uniform(-1, 1, (B, N)).astype(np.float32)
        lookup = rng.integers(0, N, (L, K)).astype(np.int32)      # with replacement: duplicates occur
        w = rng.uniform(-1, 1, (L, K)).astype(np.float32)
        g = np.maximum(rng.uniform(-1, 1, (B, L)), 0).astype(np.float32)
        out, gx, gw = dense_results(x, lookup, w, g)
        np.savez(os.path.join(HERE, f"dense_{B}_{N}_{L}_{K}.npz"), features=x, lookup=lookup, weights=w,
                 out_grad=g, result=out, feature_grad=gx, weight_grad=gw)


if __name__ == "__main__":
    main()
