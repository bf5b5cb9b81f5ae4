"""Writes the fixtures of this folder.  Run from the repository root: python tests/golden/make_golden.py

Nothing here calls the oracle or the library.  Expected values come from exact rational
arithmetic (`fractions.Fraction`) on the closed forms that the reference's own unit tests
state, and from the literal tuples of its schedule tests:

* int8 packing  code = round(255 (v - min) / (max - min)) per 128-block, scales = (min, max)
  as f16                                   (src/tensor/ops.rs:2939-2962)
* nf4 packing   nibble = nearest table entry of v / absmax per 64-block, first wins, two
  nibbles per byte, low nibble first        (src/tensor/ops.rs:3114-3144)
* products      out[t][r] = sum_k deq(W[r][k]) x[t][k] with deq = u / 255 (max - min) + min
  (ops.rs:3011-3016) or table[nibble] * absmax (ops.rs:3199-3211)
* RnnIter       the expected tuples of test_run_iter / test_advance (src/runtime/infer/rnn.rs:362-507)

The reference evaluates these forms in f32 on the GPU; a code or nibble whose exact value lies
within 1e-4 of a rounding boundary may legitimately differ there and is flagged in `sensitive`.
Products are exact rationals rounded once to float64.
"""
import json
import os
from fractions import Fraction

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
NF4 = [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453, -0.28444138169288635,
       -0.18477343022823334, -0.09105003625154495, 0.0, 0.07958029955625534, 0.16093020141124725,
       0.24611230194568634, 0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
       0.7229568362236023, 1.0]
NF4_F32 = [float(np.float32(v)) for v in NF4]


def f16_values(rng, n, std):
    return (rng.standard_normal(n, dtype=np.float32) * np.float32(std)).astype(np.float16)


def pack_int8(w16):
    """exact codes of a flat f16 array, 128 per block"""
    codes, minmax, sensitive = [], [], []
    for b in range(0, len(w16), 128):
        blk = [Fraction(float(v)) for v in w16[b:b + 128]]
        mn, mx = min(blk), max(blk)
        minmax += [mn, mx]
        for v in blk:
            s = 255 * (v - mn) / (mx - mn)
            fl = s.numerator // s.denominator
            frac = s - fl
            codes.append(int(fl + (1 if frac >= Fraction(1, 2) else 0)))
            sensitive.append(bool(abs(frac - Fraction(1, 2)) < Fraction(1, 10000)))
    return codes, minmax, sensitive


def pack_nf4(w16, table):
    tab = [Fraction(v) for v in table]
    nibbles, absmax, sensitive = [], [], []
    for b in range(0, len(w16), 64):
        blk = [Fraction(float(v)) for v in w16[b:b + 64]]
        am = max(abs(v) for v in blk)
        absmax.append(am)
        for v in blk:
            x = v / am
            d = [abs(x - q) for q in tab]
            best = min(range(16), key=lambda j: (d[j], j))  # nearest, first wins
            ds = sorted(d)
            nibbles.append(best)
            sensitive.append(bool(ds[1] - ds[0] < Fraction(1, 10000)))
    return nibbles, absmax, sensitive


def case(seed, kind, K, R, T):
    rng = np.random.default_rng(seed)
    w = f16_values(rng, R * K, 0.02)
    x = f16_values(rng, T * K, 1.0)
    out = {"kind": kind, "K": K, "R": R, "T": T, "w_f16_bits": w.view(np.uint16).tolist(), "x_f16_bits": x.view(np.uint16).tolist()}
    wq = []
    if kind == "int8":
        codes, minmax, sens = pack_int8(w)
        out["codes"] = codes
        out["minmax_f16_bits"] = np.array([float(v) for v in minmax], dtype=np.float16).view(np.uint16).tolist()
        for i, u in enumerate(codes):
            mn, mx = minmax[2 * (i // 128)], minmax[2 * (i // 128) + 1]
            wq.append(Fraction(u, 255) * (mx - mn) + mn)
    else:
        nib, absmax, sens = pack_nf4(w, NF4_F32)
        out["bytes"] = [nib[2 * i] | (nib[2 * i + 1] << 4) for i in range(len(nib) // 2)]
        out["absmax_f16_bits"] = np.array([float(v) for v in absmax], dtype=np.float16).view(np.uint16).tolist()
        for i, n in enumerate(nib):
            wq.append(Fraction(NF4_F32[n]) * absmax[i // 64])
    out["sensitive"] = [i for i, s in enumerate(sens) if s]
    xs = [Fraction(float(v)) for v in x]
    out["product_f64"] = [[float(sum(wq[r * K + k] * xs[t * K + k] for k in range(K))) for r in range(R)] for t in range(T)]
    return out


RNN_KATS = {
    "source": "src/runtime/infer/rnn.rs:362-507 (test_run_iter, test_advance): batch lengths, chunk size, expected tokens per slot of successive runs",
    "run_iter": {"lengths": [139, 1, 0, 65], "chunk": 128, "runs": [[65, 1, 0, 62], [60, 1, 0, 3], [14, 1, 0, 1], [1, 1, 0, 1], [1, 1, 0, 1]]},
    "advance": {"lengths": [139, 1, 0, 65], "chunk": 128, "after_one_step_first_run": [61, 0, 0, 3]},
    "advance_refilled": {"lengths": [61, 1, 0, 3], "chunk": 128, "runs": [[60, 1, 0, 3]]},
}

if __name__ == "__main__":
    cases = [case(0x57525100 + i, kind, K, R, T)
             for i, (kind, K, R, T) in enumerate([("int8", 256, 8, 1), ("int8", 384, 4, 4), ("nf4", 256, 8, 1), ("nf4", 192, 4, 4)])]
    with open(os.path.join(HERE, "exact_pack_and_products.json"), "w") as f:
        json.dump({"nf4_table": NF4_F32, "cases": cases}, f)
    with open(os.path.join(HERE, "rnn_iter_kats.json"), "w") as f:
        json.dump(RNN_KATS, f, indent=1)
    print("wrote", len(cases), "cases")
    # data_movement_kats.json beside these holds the literal buffers of test_blit / test_transpose
    # (src/tensor/ops.rs:3302-3365); it is data copied by hand, nothing computes it
