#!/usr/bin/env python3
"""Writes tests/golden/golden_small.json: tiny inputs and expected outputs that
pin the CPU oracle (oracle/). Everything here is brute force in pure Python
float64 (loops, math.exp/log/erf/tanh) and central finite differences for the
gradients, so that it shares no formula with the oracle's closed forms: a
dropped term, a wrong sign, a transposed operand or an off-by-one in the
vocabulary offset shows up as a mismatch.

    python tests/golden/make_golden.py

The reference package is not imported (it cannot be on this torch: it needs
torch._six) and nothing of it is copied; the definitions below are the
mathematical ones the reference's tests check against (A @ W + b, LayerNorm,
softmax cross-entropy).
"""
import json
import math
import os
import random

HERE = os.path.dirname(os.path.abspath(__file__))


def rnd_matrix(rng, r, c, scale=1.0):
    return [[round(rng.gauss(0.0, scale), 4) for _ in range(c)] for _ in range(r)]


def rnd_vector(rng, n, scale=1.0):
    return [round(rng.gauss(0.0, scale), 4) for _ in range(n)]


def act(x, kind):
    if kind == "none":
        return x
    if kind == "relu":
        return x if x > 0 else 0.0
    if kind == "gelu_erf":
        return 0.5 * x * (1.0 + math.erf(x / math.sqrt(2.0)))
    if kind == "gelu_tanh":
        return 0.5 * x * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))
    raise ValueError(kind)


def gemm_case(rng, layout, M, N, K, steps, kind, with_addend):
    A = [rnd_matrix(rng, K if layout == "TN" else M, M if layout == "TN" else K) for _ in range(steps)]
    B = [rnd_matrix(rng, N if layout == "NT" else K, K if layout == "NT" else N, 0.5) for _ in range(steps)]
    bias = rnd_vector(rng, N, 0.5)
    addend = rnd_matrix(rng, M, N) if with_addend else None
    pre = [[0.0] * N for _ in range(M)]
    for s in range(steps):
        for m in range(M):
            for n in range(N):
                acc = 0.0
                for k in range(K):
                    a = A[s][k][m] if layout == "TN" else A[s][m][k]
                    b = B[s][n][k] if layout == "NT" else B[s][k][n]
                    acc += a * b
                pre[m][n] += acc
    for m in range(M):
        for n in range(N):
            pre[m][n] += bias[n] + (addend[m][n] if addend else 0.0)
    out = [[act(v, kind) for v in row] for row in pre]
    return {"layout": layout, "A": A, "B": B, "bias": bias, "addend": addend, "act": kind, "preact": pre, "out": out}


def layernorm_fwd(x, gamma, beta, eps):
    out = []
    for row in x:
        h = len(row)
        mean = sum(row) / h
        var = sum((v - mean) ** 2 for v in row) / h
        out.append([gamma[c] * (row[c] - mean) / math.sqrt(var + eps) + beta[c] for c in range(h)])
    return out


def layernorm_case(rng, R, H, eps):
    x = rnd_matrix(rng, R, H)
    gamma = [round(1.0 + rng.uniform(-0.1, 0.1), 4) for _ in range(H)]
    beta = rnd_vector(rng, H, 0.1)
    dy = rnd_matrix(rng, R, H)
    y = layernorm_fwd(x, gamma, beta, eps)

    def loss(xx, gg, bb):
        yy = layernorm_fwd(xx, gg, bb, eps)
        return sum(dy[r][c] * yy[r][c] for r in range(R) for c in range(H))

    hstep = 1e-6
    dx = [[0.0] * H for _ in range(R)]
    for r in range(R):
        for c in range(H):
            xp = [row[:] for row in x]
            xm = [row[:] for row in x]
            xp[r][c] += hstep
            xm[r][c] -= hstep
            dx[r][c] = (loss(xp, gamma, beta) - loss(xm, gamma, beta)) / (2 * hstep)
    dgamma, dbeta = [], []
    for c in range(H):
        gp, gm = gamma[:], gamma[:]
        gp[c] += hstep
        gm[c] -= hstep
        dgamma.append((loss(x, gp, beta) - loss(x, gm, beta)) / (2 * hstep))
        bp, bm = beta[:], beta[:]
        bp[c] += hstep
        bm[c] -= hstep
        dbeta.append((loss(x, gamma, bp) - loss(x, gamma, bm)) / (2 * hstep))
    # local partials of the first half of the columns, as a q = 2 row group splits them
    half = H // 2
    stats_local = [[sum(row[:half]), sum(v * v for v in row[:half])] for row in x]
    stats_peer = [[sum(row[half:]), sum(v * v for v in row[half:])] for row in x]
    return {"x": x, "gamma": gamma, "beta": beta, "dy": dy, "eps": eps, "y": y, "dx": dx, "dgamma": dgamma,
            "dbeta": dbeta, "stats_local": stats_local, "stats_peer": stats_peer}


def ce_losses(logits, targets):
    out = []
    for row, t in zip(logits, targets):
        m = max(row)
        lse = m + math.log(sum(math.exp(v - m) for v in row))
        out.append(lse - row[t])
    return out


def ce_case(rng, T, V, p):
    logits = rnd_matrix(rng, T, V * p, 2.0)
    # targets on slice borders and inside slices
    targets = [min(t, V * p - 1) for t in (0, V - 1, V, V * p - 1, 2 * V + 1, V + V // 2)][:T]
    while len(targets) < T:
        targets.append(rng.randrange(V * p))
    dloss = [round(rng.uniform(0.5, 1.5), 4) for _ in range(T)]
    loss = ce_losses(logits, targets)
    hstep = 1e-6
    grad = [[0.0] * (V * p) for _ in range(T)]
    for r in range(T):
        for c in range(V * p):
            lp = [row[:] for row in logits]
            lm = [row[:] for row in logits]
            lp[r][c] += hstep
            lm[r][c] -= hstep
            fp = sum(d * l for d, l in zip(dloss, ce_losses(lp, targets)))
            fm = sum(d * l for d, l in zip(dloss, ce_losses(lm, targets)))
            grad[r][c] = (fp - fm) / (2 * hstep)
    # per-slice integer bookkeeping, by definition
    masks, shifted, preds, maxes = [], [], [], []
    for r in range(p):
        start, end = r * V, (r + 1) * V
        masks.append([0 if start <= t < end else 1 for t in targets])
        shifted.append([t - start if start <= t < end else 0 for t in targets])
        preds.append([logits[i][t] if start <= t < end else 0.0 for i, t in enumerate(targets)])
        maxes.append([max(row[start:end]) for row in logits])
    return {"logits": logits, "targets": targets, "slices": p, "dloss": dloss, "loss": loss, "grad": grad,
            "mask": masks, "shifted": shifted, "pred": preds, "max": maxes}


def main():
    rng = random.Random(20240607)
    data = {
        "gemm": [
            gemm_case(rng, "NN", 3, 4, 5, 2, "gelu_tanh", False),
            gemm_case(rng, "NT", 4, 3, 6, 1, "gelu_erf", True),
            gemm_case(rng, "TN", 5, 2, 4, 3, "relu", True),
            gemm_case(rng, "NN", 2, 2, 3, 2, "none", False),
        ],
        "layernorm": [layernorm_case(rng, 3, 8, 1e-5), layernorm_case(rng, 2, 6, 1e-12)],
        "cross_entropy": [ce_case(rng, 6, 4, 3), ce_case(rng, 5, 7, 2)],
    }
    path = os.path.join(HERE, "golden_small.json")
    with open(path, "w") as f:
        json.dump(data, f, indent=None, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
