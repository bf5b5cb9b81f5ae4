"""Writes recurrent_float64.json.  Run from the repository root: python tests/golden/make_recurrent_golden.py

Nothing here calls the oracle or the library.  Small seeded f32 inputs (f16-valued where the runtime
keeps f16) and what the textbook form of each recurrence gives for them in float64, one token and one
head at a time with plain matrix expressions:

* v4 (src/shaders/time_mix_v4.wgsl) without its exponent shift: a <- e^w a + e^k v, b <- e^w b + e^k,
  y = sigmoid(r) (a + e^(u+k) v) / (b + e^(u+k)); the state rows hold aa, bb, pp with a = aa e^pp, b = bb e^pp
* v5 / v6 (time_mix_v5.wgsl, time_mix_v6.wgsl): y = r^T (diag(u) k v^T + S), S <- diag(w) S + k v^T
* v7 (time_mix_v7.wgsl): sa = S^T (-kk), S <- diag(e^(-e^(-1/2) sigmoid(w))) S + k v^T + (kk a) sa^T, y = S^T r

Runs: the tokens of two requests stacked ((slot, count) pairs); row 0 of a request's state takes the
layer input x at its last token.
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
RUNS = [(1, 3), (0, 2)]
H, S, B = 1, 32, 2  # one head of 32: the smallest head every version's kernel is built for
f = np.float64


def tokens():
    out = []
    for slot, n in RUNS:
        out += [(slot, i == n - 1) for i in range(n)]
    return out


def lst(a):
    a = np.asarray(a)
    if a.dtype == np.float32:  # inputs: the shortest decimal that reads back as the same f32 (readers convert to float32)
        return [float(str(v)) for v in a.reshape(-1)]
    return [float(f"{v:.10g}") for v in a.astype(np.float64).reshape(-1)]  # results: ten significant digits


def wkv56(w_per_token, rng):
    A, C = len(tokens()), H * S
    k, v, r, x = (rng.standard_normal((A, H, S)).astype(np.float16).astype(np.float32) * np.float32(0.5) for _ in range(4))
    w = np.exp(-np.exp(rng.standard_normal((A, H, S) if w_per_token else (H, S)).astype(np.float32))).astype(np.float32)
    u = (0.3 * rng.standard_normal((H, S))).astype(np.float32)
    state = (0.1 * rng.standard_normal((B, S + 1, C))).astype(np.float32)
    st, y = state.astype(f).copy(), np.zeros((A, H, S))
    for t, (slot, last) in enumerate(tokens()):
        if last:
            st[slot, 0] = x[t].astype(f).reshape(-1)
        for h in range(H):
            Sm = st[slot, 1:, h * S:(h + 1) * S]
            kv = np.outer(k[t, h].astype(f), v[t, h].astype(f))
            y[t, h] = r[t, h].astype(f) @ (u[h].astype(f)[:, None] * kv + Sm)
            wt = (w[t, h] if w_per_token else w[h]).astype(f)
            st[slot, 1:, h * S:(h + 1) * S] = wt[:, None] * Sm + kv
    return {"k": lst(k), "v": lst(v), "r": lst(r), "x": lst(x), "time_decay": lst(w), "time_first": lst(u), "state": lst(state), "y": lst(y), "state_after": lst(st)}


def wkv7(rng):
    A, C = len(tokens()), H * S
    r, k, v, x = (rng.standard_normal((A, H, S)).astype(np.float16).astype(np.float32) * np.float32(0.5) for _ in range(4))
    w = rng.standard_normal((A, H, S)).astype(np.float16).astype(np.float32)
    a = rng.random((A, H, S)).astype(np.float16).astype(np.float32)
    kk = rng.standard_normal((A, H, S))
    kk = (kk / np.sqrt((kk * kk).sum(axis=-1, keepdims=True))).astype(np.float16).astype(np.float32)
    state = (0.1 * rng.standard_normal((B, S + 1, C))).astype(np.float32)
    st, y = state.astype(f).copy(), np.zeros((A, H, S))
    for t, (slot, last) in enumerate(tokens()):
        if last:
            st[slot, 0] = x[t].astype(f).reshape(-1)
        for h in range(H):
            Sm = st[slot, 1:, h * S:(h + 1) * S]
            ww = np.exp(-np.exp(-0.5) / (1.0 + np.exp(-w[t, h].astype(f))))
            sa = Sm.T @ (-kk[t, h].astype(f))
            Sn = ww[:, None] * Sm + np.outer(k[t, h].astype(f), v[t, h].astype(f)) + np.outer(kk[t, h].astype(f) * a[t, h].astype(f), sa)
            y[t, h] = Sn.T @ r[t, h].astype(f)
            st[slot, 1:, h * S:(h + 1) * S] = Sn
    return {"r": lst(r), "w": lst(w), "n": lst(np.stack([k, v, a, kk])), "x": lst(x), "state": lst(state), "y": lst(y), "state_after": lst(st)}


def wkv4(rng):
    A, C = len(tokens()), H * S
    k, v, r, x = (rng.standard_normal((A, C)).astype(np.float16).astype(np.float32) for _ in range(4))
    w = (-np.exp(rng.standard_normal(C).astype(np.float32))).astype(np.float32)
    u = (0.3 * rng.standard_normal(C)).astype(np.float32)
    state = rng.standard_normal((B, 4, C)).astype(np.float32)
    state[:, 2] = np.abs(state[:, 2]) + np.float32(0.5)
    state[0, 1:] = np.array([[0] * C, [0] * C, [-1e30] * C], dtype=np.float32)  # slot 0 starts fresh
    a = state[:, 1].astype(f) * np.exp(state[:, 3].astype(f))
    b = state[:, 2].astype(f) * np.exp(state[:, 3].astype(f))
    row0, y = state[:, 0].astype(f).copy(), np.zeros((A, C))
    for t, (slot, last) in enumerate(tokens()):
        if last:
            row0[slot] = x[t].astype(f)
        ek, eu = np.exp(k[t].astype(f)), np.exp(u.astype(f) + k[t].astype(f))
        y[t] = (a[slot] + eu * v[t].astype(f)) / (b[slot] + eu) / (1 + np.exp(-r[t].astype(f)))
        a[slot] = np.exp(w.astype(f)) * a[slot] + ek * v[t].astype(f)
        b[slot] = np.exp(w.astype(f)) * b[slot] + ek
    return {"k": lst(k), "v": lst(v), "r": lst(r), "x": lst(x), "time_decay": lst(w), "time_first": lst(u), "state": lst(state), "y": lst(y),
            "numerator_after": lst(a), "denominator_after": lst(b), "row0_after": lst(row0)}


if __name__ == "__main__":
    rng = np.random.default_rng(0x57525200)
    out = {"H": H, "S": S, "B": B, "runs": RUNS, "v4": wkv4(rng), "v5": wkv56(False, rng), "v6": wkv56(True, rng), "v7": wkv7(rng)}
    with open(os.path.join(HERE, "recurrent_float64.json"), "w") as fh:
        json.dump(out, fh)
    print("wrote recurrent_float64.json")
