#!/usr/bin/env python3
"""Writes tests/golden/vectors.json: small seeded inputs and the outputs the pure-Python brute-force
restatements give for them (oracle.flare_oracle.mixer_bruteforce_py and the loops below, plain Python
floats, no tensor library arithmetic).  The reference is not involved: these are frozen known answers of
the DEFINITIONS (README.md:39-52, lra/models/backends.py:1285-1292, lra/models/triton/causal_linear.py:317-336
of the reference, and the causal restriction of the first), against which the torch oracle, the C oracle and
the HIP kernels are all checked, so that none of them can drift unnoticed.

    python tests/golden/make_vectors.py        # rewrites vectors.json (deterministic)
"""
import json
import math
import os
import random
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))


def rnd(rng, *shape, std=1.0):
    if len(shape) == 1:
        return [round(rng.gauss(0.0, std), 3) for _ in range(shape[0])]
    return [rnd(rng, *shape[1:], std=std) for _ in range(shape[0])]


def softmax(xs):
    m = max(xs)
    e = [math.exp(x - m) for x in xs]
    s = sum(e)
    return [x / s for x in e]


def mixer(q, k, v, scale):
    """q [H][M][D], k, v [H][N][D] (one batch element) -> y [H][N][D]."""
    out = []
    for h in range(len(q)):
        M, N, D = len(q[h]), len(k[h]), len(q[h][0])
        s = [[scale * sum(q[h][m][d] * k[h][n][d] for d in range(D)) for n in range(N)] for m in range(M)]
        z = []
        for m in range(M):
            a = softmax(s[m])
            z.append([sum(a[n] * v[h][n][d] for n in range(N)) for d in range(D)])
        y = []
        for n in range(N):
            b = softmax([s[m][n] for m in range(M)])
            y.append([sum(b[m] * z[m][d] for m in range(M)) for d in range(D)])
        out.append(y)
    return out


def causal(q, k, v, scale):
    """Row t of the mixer restricted to tokens 0..t."""
    out = []
    for h in range(len(q)):
        ys = []
        for t in range(len(k[h])):
            y = mixer([q[h]], [k[h][:t + 1]], [v[h][:t + 1]], scale)[0]
            ys.append(y[t])
        out.append(ys)
    return out


def triple(q1, q2, k1, k2, v):
    """state[i][j][k] = sum_n k1[n][i] v[n][j] k2[n][k] / N ; out[n][j] = sum_ik q1[n][i] state[i][j][k] q2[n][k]."""
    outs, states = [], []
    for h in range(len(v)):
        N, D, Dv = len(v[h]), len(k1[h][0]), len(v[h][0])
        st = [[[sum(k1[h][n][i] * v[h][n][j] * k2[h][n][kk] for n in range(N)) / N for kk in range(D)]
               for j in range(Dv)] for i in range(D)]
        o = [[sum(q1[h][n][i] * st[i][j][kk] * q2[h][n][kk] for i in range(D) for kk in range(D)) for j in range(Dv)]
             for n in range(N)]
        states.append(st)
        outs.append(o)
    return states, outs


def causal_linear(q, k, v):
    """y_t = (sum_{tau<=t} v_tau k_tau^T / N) q_t."""
    out = []
    for h in range(len(v)):
        N, Dk, Dv = len(v[h]), len(k[h][0]), len(v[h][0])
        S = [[0.0] * Dk for _ in range(Dv)]
        ys = []
        for t in range(N):
            for j in range(Dv):
                for i in range(Dk):
                    S[j][i] += v[h][t][j] * k[h][t][i] / N
            ys.append([sum(S[j][i] * q[h][t][i] for i in range(Dk)) for j in range(Dv)])
        out.append(ys)
    return out


def main():
    rng = random.Random(20240521)
    vec = {}
    q, k, v = rnd(rng, 2, 5, 4, std=0.7), rnd(rng, 2, 11, 4), rnd(rng, 2, 11, 4)
    vec["mixer"] = {"scale": 0.9, "q": q, "k": k, "v": v, "y": mixer(q, k, v, 0.9)}
    q, k, v = rnd(rng, 2, 4, 3, std=0.8), rnd(rng, 2, 9, 3), rnd(rng, 2, 9, 3)
    vec["causal"] = {"scale": 1.1, "q": q, "k": k, "v": v, "y": causal(q, k, v, 1.1)}
    q1, q2, k1, k2 = (rnd(rng, 2, 7, 3, std=0.6) for _ in range(4))
    v = rnd(rng, 2, 7, 2)
    st, o = triple(q1, q2, k1, k2, v)
    vec["triple"] = {"q1": q1, "q2": q2, "k1": k1, "k2": k2, "v": v, "state": st, "out": o}
    q, k, v = rnd(rng, 1, 10, 4), rnd(rng, 1, 10, 4), rnd(rng, 1, 10, 3)
    vec["causal_linear"] = {"q": q, "k": k, "v": v, "y": causal_linear(q, k, v)}
    with open(os.path.join(HERE, "vectors.json"), "w") as f:
        json.dump(vec, f, separators=(",", ":"))
    print("wrote", os.path.join(HERE, "vectors.json"))


if __name__ == "__main__":
    main()
