#!/usr/bin/env python3
"""Writes tests/golden/vectors.json: small seeded inputs and the outputs the pure-Python brute-force
restatements give for them (oracle.flare_oracle.mixer_bruteforce_py and the loops below, plain Python
floats, no tensor library arithmetic).  The reference is not involved: these are frozen known answers of
the DEFINITIONS (README.md:39-52, lra/models/backends.py:1285-1292, lra/models/triton/causal_linear.py:317-336,
pdebench/models/flare.py:45-59 and 204-215, lra/models/embeddings.py:136-147 of the reference, and the causal
restriction of the first), against which the torch oracle, the C oracle and
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


def mlp_stack(x, ws, bs, gamma, beta, eps, res):
    """res + ResidualMLP(LayerNorm(x)) for rows x [T][C] (pdebench/models/flare.py:45-59 inside :204-215), all widths
    equal so that both residual flags act: s = n + gelu(W0 n + b0); s += gelu(Wi s + bi) for the hidden layers;
    s += W_last s + b_last; tanh-GELU."""
    def gelu(t):
        return 0.5 * t * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (t + 0.044715 * t ** 3)))
    def lin(w, b, s):
        return [sum(w[o][i] * s[i] for i in range(len(s))) + b[o] for o in range(len(w))]
    out = []
    for t in range(len(x)):
        C = len(x[t])
        mu = sum(x[t]) / C
        var = sum((a - mu) ** 2 for a in x[t]) / C
        n = [(x[t][c] - mu) / math.sqrt(var + eps) * gamma[c] + beta[c] for c in range(C)]
        h = lin(ws[0], bs[0], n)
        s = [n[c] + gelu(h[c]) for c in range(C)]
        for l in range(1, len(ws) - 1):
            h = lin(ws[l], bs[l], s)
            s = [s[c] + gelu(h[c]) for c in range(C)]
        h = lin(ws[-1], bs[-1], s)
        out.append([res[t][c] + s[c] + h[c] for c in range(C)])
    return out


def rope(x, base):
    """lra/models/embeddings.py:136-147 for x [N][D]: rates base^-(j//2)/(D/2); partner = (-odd channels, even channels)."""
    out = []
    for p, row in enumerate(x):
        D = len(row)
        partner = [-row[2 * j + 1] for j in range(D // 2)] + [row[2 * j] for j in range(D // 2)]
        ang = [p * base ** (-(j // 2) / (D // 2)) for j in range(D)]
        out.append([row[j] * math.cos(ang[j]) + partner[j] * math.sin(ang[j]) for j in range(D)])
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
    # drawn after everything above, so that the earlier vectors keep their values
    C = 32
    ws = [rnd(rng, C, C, std=C ** -0.5) for _ in range(3)]
    bs = [rnd(rng, C, std=0.2) for _ in range(3)]
    gamma, beta = [1.0 + g_ for g_ in rnd(rng, C, std=0.2)], rnd(rng, C, std=0.2)
    x, res = rnd(rng, 3, C, std=1.5), rnd(rng, 3, C)
    vec["mlp_stack"] = {"x": x, "w": ws, "b": bs, "gamma": gamma, "beta": beta, "eps": 1e-5, "res": res,
                        "y": mlp_stack(x, ws, bs, gamma, beta, 1e-5, res)}
    x = rnd(rng, 6, 8)
    vec["rope"] = {"base": 50.0, "x": x, "y": rope(x, 50.0)}
    with open(os.path.join(HERE, "vectors.json"), "w") as f:
        json.dump(vec, f, separators=(",", ":"))
    print("wrote", os.path.join(HERE, "vectors.json"))


if __name__ == "__main__":
    main()
