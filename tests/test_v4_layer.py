"""One whole RWKV-v4 layer, dispatched op by op like the reference (src/runtime/v4.rs:620-791), on
the GPU through the library against a numpy composition of the oracle's restatements."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close, int8_dequant64, nf4_dequant64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525400


def layer_numpy(lop, w, x, state, cursors):
    """The layer on the CPU: every buffer rounded to the type the reference's runtime gives it
    (f16 except aux_x and att_k / v / r: src/runtime/v4.rs:234-256)."""
    f16, f32, f64 = np.float16, np.float32, np.float64
    mm = lambda a, W, dt: (a.astype(f64) @ W.astype(f64).T).astype(dt)
    att_x = lop.layer_norm(w["att_ln_w"], w["att_ln_b"], x, 1e-5)
    kx, vx, rx = (lop.token_shift(cursors, w[n], state[:, 0], att_x, f16, reversed=False)[0] for n in ("time_mix_k", "time_mix_v", "time_mix_r"))
    k, v, r = mm(kx, w["att_w_k"], f32), mm(vx, w["att_w_v"], f32), mm(rx, w["att_w_r"], f32)
    att = np.ascontiguousarray(state[:, :4])
    aux = lop.time_mix_v4(cursors, w["time_decay"], w["time_first"], att, k, v, r, att_x.astype(f32))
    state[:, :4] = att
    x = lop.binary("add", mm(aux.astype(f16), w["att_w_o"], f16), x)
    ffn_x = lop.layer_norm(w["ffn_ln_w"], w["ffn_ln_b"], x, 1e-5)
    ffn_state = np.ascontiguousarray(state[:, 4])
    fkx = lop.token_shift(cursors, w["ffn_time_mix_k"], ffn_state, ffn_x, f16, reversed=False)[0]
    frx = lop.token_shift(cursors, w["ffn_time_mix_r"], ffn_state, ffn_x, f16, reversed=False)[0]
    fk = lop.activation(1, mm(fkx, w["ffn_w_k"], f32)).astype(f16)
    fv = mm(fk, w["ffn_w_v"], f16)
    fr = mm(frx, w["ffn_w_r"], f16)
    ffn_x = lop.channel_mix(cursors, ffn_state, fr, fv, ffn_x)
    state[:, 4] = ffn_state
    return lop.binary("add", ffn_x, x)


@pytest.mark.gpu
@pytest.mark.parametrize("quant", ["int8", "nf4"])
@pytest.mark.parametrize("runs", [[(2, 3), (0, 1), (5, 4)], [(1, 20), (3, 12)], [(4, 1)]], ids=["8 tokens", "32 tokens (chunk kernels)", "1 token"])
def test_v4_layer_against_numpy(gpu, oracle, quant, runs):
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v4 = importlib.import_module(gpu.__name__ + ".v4")
    print("v4 layer on the GPU", quant, runs, flush=True)
    C, hidden, B = 512, 2048, 6
    rng = np.random.default_rng(SEED + len(runs))
    w = v4.random_layer_weights(rng, C, hidden, layer=7)
    cursors = lop.pack_cursors(runs)
    A = len(cursors)
    x = rng.standard_normal((A, C)).astype(np.float16)
    state = (0.1 * rng.standard_normal((B, 5, C))).astype(np.float32)
    state[:, 2] = np.abs(state[:, 2]) + 0.5  # the denominator of the running average

    layer = v4.Layer(torch, w, quant)
    wq = dict(w)  # the CPU side works on what the packed matrices represent
    for name in v4.QUANTIZED:
        mtx = layer.m[name]
        if quant == "int8":
            wq[name] = int8_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy())
        else:
            wq[name] = nf4_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy(), np.array(gpu.NF4_QUANT, dtype=np.float32))
    want_state = state.copy()
    want = layer_numpy(lop, wq, x, want_state, cursors)

    buf = v4.Runtime(torch, C, hidden, A)
    buf.x.copy_(torch.from_numpy(x).cuda().reshape(1, A, C))
    sd = torch.from_numpy(state.copy()).cuda()
    v4.dispatch_layer(layer, buf, sd, torch.from_numpy(cursors.view(np.int32)).cuda(), A, C)
    torch.cuda.synchronize()
    assert_close(buf.x.cpu().numpy()[0], want, 1e-2, "layer output")
    assert_close(sd.cpu().numpy(), want_state, 1e-2, "state after the run")
    untouched = [b for b in range(B) if b not in [s for s, _ in runs]]
    assert np.array_equal(sd.cpu().numpy()[untouched], state[untouched])
