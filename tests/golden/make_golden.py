"""Writes tests/golden/kat_exact.json: known-answer vectors in exact rational arithmetic.

The reference repository holds no golden vectors for this path (its tests are
purely differential, reference tests/test_all_kernels.py:20-50), so these are
derived from the mathematical definition itself
(reference torch-ext/flex_sae/hierarchical_kernels.py:312-323 and
torch-ext/flex_sae/topk_kernels.py:226-237) with ``fractions.Fraction``: no
floating point is involved until the final conversion, and the gradients are
obtained by exact symbolic differentiation of the polynomial loss (each
parameter is perturbed through its exact linear/quadratic dependence), not by
the suffix-sum formulas the oracle and the kernels use.

Inputs are small dyadic rationals, exactly representable in bf16, fp16 and fp32.
Run:  python tests/golden/make_golden.py
"""
import json
import os
import random
from fractions import Fraction as Fr

HERE = os.path.dirname(os.path.abspath(__file__))


def dyadic(rng, lo=-8, hi=8, den=4):
    return Fr(rng.randint(lo * den, hi * den), den)


def loss_exact(mode, idx, W, v, bias, t):
    B, K, D = len(idx), len(idx[0]), len(bias)
    steps = range(K) if mode == "hier" else [K - 1]
    tot = Fr(0)
    for b in range(B):
        for k in steps:
            for d in range(D):
                r = bias[d] + sum(v[b][j] * W[idx[b][j]][d] for j in range(k + 1))
                tot += (r - t[b][d]) ** 2
    return tot / (B * len(steps) * D)


def grad_exact(f, x0):
    """d f / d x at x0 for f an (at most) quadratic polynomial in x: exact central difference."""
    return (f(x0 + 1) - f(x0 - 1)) / 2


def make_case(mode, B, K, F, D, seed, dup=False):
    rng = random.Random(seed)
    idx = [[rng.randrange(F) for _ in range(K)] for _ in range(B)]
    if dup and K >= 2:
        idx[0][1] = idx[0][0]
    W = [[dyadic(rng, -2, 2) for _ in range(D)] for _ in range(F)]
    v = [[abs(dyadic(rng, -2, 2)) for _ in range(K)] for _ in range(B)]
    bias = [dyadic(rng, -2, 2) for _ in range(D)]
    t = [[dyadic(rng, -2, 2) for _ in range(D)] for _ in range(B)]
    grad_out = dyadic(rng, -2, 2, 2) or Fr(1)

    L = loss_exact(mode, idx, W, v, bias, t)

    def with_W(f_, d_, x):
        W2 = [row[:] for row in W]
        W2[f_][d_] = x
        return loss_exact(mode, idx, W2, v, bias, t)

    def with_v(b_, k_, x):
        v2 = [row[:] for row in v]
        v2[b_][k_] = x
        return loss_exact(mode, idx, W, v2, bias, t)

    def with_bias(d_, x):
        b2 = bias[:]
        b2[d_] = x
        return loss_exact(mode, idx, W, v, b2, t)

    dW = [[grad_exact(lambda x: with_W(f_, d_, x), W[f_][d_]) * grad_out for d_ in range(D)]
          for f_ in range(F)]
    dv = [[grad_exact(lambda x: with_v(b_, k_, x), v[b_][k_]) * grad_out for k_ in range(K)]
          for b_ in range(B)]
    db = [grad_exact(lambda x: with_bias(d_, x), bias[d_]) * grad_out for d_ in range(D)]

    fl = lambda m: [[float(x) for x in row] for row in m]
    return {
        "mode": mode, "B": B, "K": K, "F": F, "D": D, "seed": seed,
        "indices": idx, "weight": fl(W), "vals": fl(v), "bias": [float(x) for x in bias],
        "target": fl(t), "grad_out": float(grad_out),
        "loss": float(L), "loss_exact": f"{L.numerator}/{L.denominator}",
        "dW": fl(dW), "dvals": fl(dv), "dbias": [float(x) for x in db],
    }


def main():
    shapes = [
        # B, K, F, D, dup
        (1, 1, 2, 1, False),
        (1, 2, 3, 2, True),
        (2, 3, 4, 3, False),   # K not a power of two
        (3, 4, 5, 2, True),
        (2, 8, 6, 4, False),   # K > F: duplicates guaranteed
        (4, 2, 16, 5, False),
    ]
    cases = []
    for mode in ("topk", "hier"):
        for i, (B, K, F, D, dup) in enumerate(shapes):
            cases.append(make_case(mode, B, K, F, D, seed=1234 + i, dup=dup))
    with open(os.path.join(HERE, "kat_exact.json"), "w") as fh:
        json.dump({"generator": "tests/golden/make_golden.py", "cases": cases}, fh, indent=1)
    print(f"wrote {len(cases)} cases")


if __name__ == "__main__":
    main()
