"""The small whole-model configuration: an RWKV-v5-shaped random-init model (12 layers, 768 channels,
12 heads of 64, feed-forward width 2688, vocabulary 65536, all layers Int8), one request: a 32-token
seeded prompt in one run (the chunk kernels: 32 tokens is a multiple of the chunk unit), then greedy
decode steps, every op through the library as the reference dispatches them
(src/runtime/v5.rs:541-930).  The CPU side is the numpy composition of the oracle's restatements on
the same tokens: the logits of every run are compared, and the token the GPU picked must be a maximum
of the CPU's logits up to the comparison's tolerance (the runs are teacher-forced with the GPU's
choices, so one near-tie cannot derail the comparison)."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close, int8_dequant64
from test_v5_layer import layer_numpy

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525101  # configuration 1


def run_numpy(lop, w, layers_q, tokens, slot, state, H, S, rescale=6):
    f16, f64 = np.float16, np.float64
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
def test_v5_model_prompt_and_greedy_decode(gpu, oracle):
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v5 = importlib.import_module(gpu.__name__ + ".v5")
    L, H, S, hidden, V, B, slot = 12, 12, 64, 2688, 65536, 2, 1
    PROMPT, DECODE = 32, 128
    C = H * S
    print("v5-shape model, int8: prompt", PROMPT, "then", DECODE, "greedy tokens", flush=True)
    rng = np.random.default_rng(SEED)
    w = v5.random_model_weights(rng, L, C, H, S, hidden, V)
    model = v5.Model(torch, w, "int8", H, S, hidden, B)
    layers_q = []
    for lw, layer in zip(w["layers"], model.layers):
        q = dict(lw)
        for name in v5.QUANTIZED:
            q[name] = int8_dequant64(layer.m[name].w.cpu().numpy(), layer.m[name].m.cpu().numpy())
        layers_q.append(q)
    state = [np.zeros((B, S + 2, C), dtype=np.float32) for _ in range(L)]

    run = [int(t) for t in rng.integers(0, V, PROMPT)]
    picked = []
    worst = 0.0
    for step in range(DECODE + 1):
        got = model.run(run, slot).cpu().numpy()
        want = run_numpy(lop, w, layers_q, run, slot, state, H, S)
        # 12 layers of f16 buffers between the ops: a few f16 ulps of O(1) activations per layer
        assert_close(got, want, 1e-2, f"logits of run {step}")
        worst = max(worst, float(np.abs(got - want).max()))
        token = int(got.argmax())
        assert want[token] >= want.max() - 1e-2 * max(1.0, abs(float(want.max()))), f"greedy token of run {step}"
        picked.append(token)
        if step % 16 == 0:
            print("run", step, "largest logit difference so far", worst, flush=True)
        run = [token]
    print("largest logit difference", worst, "tokens", picked[:8], flush=True)
    for i in range(L):
        assert_close(model.state[i].cpu().numpy(), state[i], 2e-2, f"state of layer {i} after the runs")
        assert not model.state[i][0].any()  # the other slot was never touched


@pytest.mark.gpu
def test_v5_model_packed_token_shifts_equal_the_op_list(gpu):
    # one token shift per half of a layer (factors stacked and repeated over the tokens with `broadcast`)
    # against the reference's four and two: the same logits and states, bit for bit
    import torch

    v5 = importlib.import_module(gpu.__name__ + ".v5")
    L, H, S, hidden, V, B = 3, 12, 64, 2688, 4096, 2
    print("v5-shape model, packed token shifts", flush=True)
    rng = np.random.default_rng(SEED + 1)
    w = v5.random_model_weights(rng, L, H * S, H, S, hidden, V)
    models = [v5.Model(torch, w, "int8", H, S, hidden, B, packed_shifts=p) for p in (False, True)]
    for tokens in ([int(t) for t in rng.integers(0, V, 32)], [7], [9, 11, 13]):
        a, b = (m.run(tokens, 1).cpu().numpy() for m in models)
        assert np.array_equal(a, b), f"logits after a run of {len(tokens)}"
    for sa, sb in zip(models[0].state, models[1].state):
        assert torch.equal(sa, sb)


@pytest.mark.gpu
def test_sparse_input_statistics_of_ffn_value(gpu):
    # `matmul_vec_*` with SPARSE_INPUT (src/shaders/matmul_vec_int8.wgsl:80-84, matmul_vec_nf4.wgsl:110-120) skips a group of
    # 4 (int8) or 8 (nf4) weights per row when all their activations are zero; the one call site is ffn.value, whose input
    # is the squared ReLU of ffn.key (src/runtime/v5.rs:854-859).  The library accepts the flag and skips nothing: its
    # kernels are bound by the weight bytes crossing HBM, which only aligned runs of zeros as long as a memory sector of
    # a weight row (64 activations for int8) could save.  This measures, on the activations of this model's decode steps,
    # how often such runs occur.
    import torch

    v5 = importlib.import_module(gpu.__name__ + ".v5")
    L, H, S, hidden, V = 12, 12, 64, 2688, 65536
    rng = np.random.default_rng(SEED)
    model = v5.Model(torch, v5.random_model_weights(rng, L, H * S, H, S, hidden, V), "int8", H, S, hidden, 2)
    seen = []
    model.hook = lambda i, buf: seen.append(buf.ffn_k.detach().clone())
    run = [int(t) for t in rng.integers(0, V, 32)]
    for step in range(17):
        logits = model.run(run, 1)
        run = [int(logits.argmax())]
    decode = [k.cpu().numpy().reshape(-1, hidden) for k in seen[L:]]  # the 16 one-token runs
    k = np.concatenate(decode)  # [16 * 12, hidden]
    zero = k == 0
    stats = {g: float(zero.reshape(k.shape[0], hidden // g, g).all(axis=2).mean()) for g in (4, 8, 16, 64)}
    print("ffn.value input: zero elements", float(zero.mean()), "all-zero aligned groups of 4 / 8 / 16 / 64:", stats, flush=True)
    assert 0.3 < zero.mean() < 0.7  # a squared ReLU of a roughly symmetric pre-activation
    assert stats[4] < 0.2 and stats[64] == 0.0  # zeros do not cluster: no sector of a weight row could be skipped
