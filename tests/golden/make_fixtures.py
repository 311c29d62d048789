"""Writes the small committed fixtures under tests/golden/.

Run from the repository root:  python tests/golden/make_fixtures.py

ep_recipe_seed{42,43}.npz re-create the fixture RECIPE of the reference's own
dispatch/combine test (tests/test_ep.py:54-59,71-78,88-90 with
tests/utils.py:11-16, rank 0): seed -> eight nn.Linear(36, 36) experts with
U(0,1) weights, re-seed, then 4 iterations of randn inputs [128, 36], randint
expert ids [256] and rand routing weights [256, 1].  The expected outputs are
NOT produced by the oracle: they are the per-token definition
  y[t] = sum_j w[t,j] * (W[e] x[t] + b[e]),  e = idx[2t+j]
evaluated in float64 numpy, so that the oracle's sort / bincount / scatter
restatement is checked against something it does not share code with.

gate_small.npz holds a brute-force float64 router result on a tiny input.
"""
import os
import random

import numpy as np
import torch
import torch.nn as nn

HERE = os.path.dirname(os.path.abspath(__file__))

N_TOKENS, N_ITER, HIDDEN, E, K = 128, 4, 36, 8, 2


def set_seed(seed):
    torch.manual_seed(seed)
    np.random.seed(seed)
    random.seed(seed)


def ep_recipe(seed):
    set_seed(seed)
    ws, bs = [], []
    for _ in range(E):
        lin = nn.Linear(HIDDEN, HIDDEN)
        nn.init.uniform_(lin.weight, a=0.0, b=1.0)
        ws.append(lin.weight.detach().clone())
        bs.append(lin.bias.detach().clone())
    set_seed(seed + 0)  # rank 0
    out = {"expert_w": torch.stack(ws).numpy(), "expert_b": torch.stack(bs).numpy()}
    for it in range(N_ITER):
        inp = torch.randn(N_TOKENS, HIDDEN)
        idx = torch.randint(0, E, (N_TOKENS * K,))
        wts = torch.rand(N_TOKENS * K, 1)
        x64 = inp.double().numpy()
        W64 = out["expert_w"].astype(np.float64)
        b64 = out["expert_b"].astype(np.float64)
        y = np.zeros((N_TOKENS, HIDDEN))
        for t in range(N_TOKENS):
            for j in range(K):
                e = int(idx[t * K + j])
                y[t] += float(wts[t * K + j, 0]) * (W64[e] @ x64[t] + b64[e])
        out[f"inp{it}"] = inp.numpy()
        out[f"idx{it}"] = idx.numpy()
        out[f"w{it}"] = wts.numpy()
        out[f"y{it}"] = y
    return out


def gate_small():
    rng = np.random.default_rng(7)
    n, d, e, k = 37, 24, 8, 2
    x = rng.standard_normal((n, d)).astype(np.float32)
    w = (rng.standard_normal((e, d)) * 0.3).astype(np.float32)
    logits = x.astype(np.float64) @ w.astype(np.float64).T
    p = np.exp(logits - logits.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    order = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    topw = np.take_along_axis(p, order, -1)
    return {"x": x, "w": w, "idx": order.astype(np.int64), "weight": topw,
            "weight_norm": topw / (topw.sum(-1, keepdims=True) + 1e-20), "logits": logits}


if __name__ == "__main__":
    for seed in (42, 43):
        np.savez_compressed(os.path.join(HERE, f"ep_recipe_seed{seed}.npz"), **ep_recipe(seed))
    np.savez_compressed(os.path.join(HERE, "gate_small.npz"), **gate_small())
    print("fixtures written to", HERE)
