"""A small whole RWKV-v6 model (embedding, 7 layers with the residual halved after the sixth, head) on the
GPU through the library: a 32-token prompt as one run (the chunk kernels), then greedy decode steps, against
the numpy composition of the oracle's restatements on the same tokens; once with every layer as the
reference's op list, once with the fused small ops for the short runs."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close, int8_dequant64, nf4_dequant64
from test_v6_layer import layer_numpy

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525604


def run_numpy(lop, w, layers_q, tokens, slot, state, H, S, rescale=6):
    f64 = np.float64
    A = len(tokens)
    cursors = lop.pack_cursors([(slot, A)])
    x = lop.layer_norm(w["embed_ln_w"], w["embed_ln_b"], w["embed"][np.asarray(tokens)], 1e-5)
    for i, lw in enumerate(layers_q):
        x = layer_numpy(lop, lw, x, state[i], cursors, H, S)
        if (i + 1) % rescale == 0:
            x = lop.affine(x, 0.5, 0.0)
    hx = lop.layer_norm(w["head_ln_w"], w["head_ln_b"], x[A - 1:A], 1e-5)
    return (hx.astype(f64) @ w["head"].astype(f64).T).astype(np.float32)[0]


@pytest.mark.gpu
@pytest.mark.parametrize("quant", ["int8", "nf4"])
@pytest.mark.parametrize("fused", [False, True], ids=["op list", "fused small ops"])
def test_v6_model_prompt_and_greedy_decode(gpu, oracle, quant, fused):
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v6 = importlib.import_module(gpu.__name__ + ".v6")
    L, H, S, hidden, V, B, slot = 7, 4, 64, 1024, 8192, 3, 2
    PROMPT, DECODE = 32, 12
    C = H * S
    print("small v6 model", quant, "fused" if fused else "op list", flush=True)
    rng = np.random.default_rng(SEED)
    w = v6.random_model_weights(rng, L, C, H, S, hidden, V)
    model = v6.Model(torch, w, quant, H, S, hidden, B, dispatch=v6.dispatch_layer_auto if fused else v6.dispatch_layer)
    layers_q = []
    for lw, layer in zip(w["layers"], model.layers):
        q = dict(lw)
        for name in v6.QUANTIZED:
            mtx = layer.m[name]
            if quant == "int8":
                q[name] = int8_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy())
            else:
                q[name] = nf4_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy(), np.array(gpu.NF4_QUANT, dtype=np.float32))
        layers_q.append(q)
    state = [np.zeros((B, S + 2, C), dtype=np.float32) for _ in range(L)]
    run = [int(t) for t in rng.integers(0, V, PROMPT)]
    worst = 0.0
    for step in range(DECODE + 1):
        got = model.run(run, slot).cpu().numpy()
        want = run_numpy(lop, w, layers_q, run, slot, state, H, S)
        # f16 buffers between the ops of 7 layers: a few f16 ulps of O(1) activations per layer
        assert_close(got, want, 5e-3, f"logits of run {step}")
        worst = max(worst, float(np.abs(got - want).max()))
        token = int(got.argmax())
        assert want[token] >= want.max() - 5e-3 * max(1.0, abs(float(want.max()))), f"greedy token of run {step}"
        run = [token]
    print("largest logit difference", worst, flush=True)
    for i in range(L):
        assert_close(model.state[i].cpu().numpy(), state[i], 5e-3, f"state of layer {i} after the runs")
        assert not model.state[i][:2].any()  # the other slots were never touched
