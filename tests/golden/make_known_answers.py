#!/usr/bin/env python3
"""Writes tests/golden/known_answers.json: small input/output vectors for the
LayerNorm and GELU nests, computed here in numpy fp32 one operation at a time
in the order the reference's builders emit them
(src/Frontend/Operators.cc:1184-1241 LayerNorm: sum, divide by N, subtract,
sum of squares, divide by N, add eps, sqrt, divide, multiply by gamma, add beta;
:986-994 GELU: 0.5*x, x^3, *0.044715, +x, *0.797884, tanh, +1, multiply).
Independent of the C oracle, which is checked against this file.

    python tests/golden/make_known_answers.py
"""
import json
import os

import numpy as np

f32 = np.float32


def layernorm_row(x, gamma, beta, eps):
    x = np.asarray(x, f32)
    n = f32(len(x))
    s = f32(0)
    for v in x:
        s = f32(s + v)
    mean = f32(s / n)
    d = (x - mean).astype(f32)
    q = f32(0)
    for v in d:
        q = f32(q + f32(v * v))
    var = f32(q / n)
    den = f32(np.sqrt(f32(var + f32(eps))))
    return [float(f32(f32(f32(g) * f32(v / den)) + f32(b))) for v, g, b in zip(d, gamma, beta)]


def gelu(x):
    x = f32(x)
    half = f32(f32(0.5) * x)
    cube = f32(f32(x * x) * x)
    inner = f32(f32(f32(0.044715) * cube) + x)
    t = f32(np.tanh(np.float64(f32(f32(0.797884) * inner))))
    return float(f32(half * f32(t + f32(1))))


def main():
    x = [1.0, 2.0, 3.0, 4.0]
    cases = []
    for gamma, beta in (([1.0] * 4, [0.0] * 4), ([0.5, 1.0, 1.5, 2.0], [0.1, -0.1, 0.0, 0.05])):
        cases.append({"x": x, "gamma": gamma, "beta": beta, "eps": 1e-5, "y": layernorm_row(x, gamma, beta, 1e-5)})
    xs = [-3.0, -1.0, -0.5, 0.0, 0.5, 1.0, 2.0, 3.0]
    out = {"layernorm": cases, "gelu": {"x": xs, "y": [gelu(v) for v in xs]}}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "known_answers.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")


if __name__ == "__main__":
    main()
