"""One whole RWKV-v5 layer, dispatched op by op like the reference (src/runtime/v5.rs:651-890),
on the GPU through the library against a numpy composition of the oracle's restatements; the layer
of the small model configuration: 768 channels, 12 heads of 64, feed-forward width 2688."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close, int8_dequant64, nf4_dequant64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525500


def layer_numpy(lop, w, x, state, cursors, H, S):
    """The layer on the CPU: every buffer rounded to the type the reference's runtime gives it
    (f16 except aux_x and att_k / v / r: src/runtime/v5.rs:258-283)."""
    f16, f32, f64 = np.float16, np.float32, np.float64
    A, C = x.shape
    mm = lambda a, W, dt: (a.astype(f64) @ W.astype(f64).T).astype(dt)
    att_x = lop.layer_norm(w["att_ln_w"], w["att_ln_b"], x, 1e-5)
    kx, vx, rx, gx = (lop.token_shift(cursors, w[n], state[:, 0], att_x, f16, reversed=False)[0] for n in ("time_mix_k", "time_mix_v", "time_mix_r", "time_mix_g"))
    k, v, r = mm(kx, w["att_w_k"], f32), mm(vx, w["att_w_v"], f32), mm(rx, w["att_w_r"], f32)
    g = mm(gx, w["att_w_g"], f16)
    att = np.ascontiguousarray(state[:, :S + 1])
    aux = lop.time_mix_v5(cursors, w["time_decay"], w["time_first"], att, k.reshape(A, H, S), v.reshape(A, H, S), r.reshape(A, H, S),
                          att_x.astype(f32).reshape(A, H, S))
    state[:, :S + 1] = att
    aux = lop.group_norm(w["gn_w"], w["gn_b"], aux, 64e-5)
    att_x = lop.binary("mul", g, aux.reshape(A, C).astype(f16), act_x=7)
    x = lop.binary("add", mm(att_x, w["att_w_o"], f16), x)
    ffn_x = lop.layer_norm(w["ffn_ln_w"], w["ffn_ln_b"], x, 1e-5)
    ffn_state = np.ascontiguousarray(state[:, S + 1])
    fkx = lop.token_shift(cursors, w["ffn_time_mix_k"], ffn_state, ffn_x, f16, reversed=False)[0]
    frx = lop.token_shift(cursors, w["ffn_time_mix_r"], ffn_state, ffn_x, f16, reversed=False)[0]
    fk = lop.activation(1, mm(fkx, w["ffn_w_k"], f32)).astype(f16)
    fv = mm(fk, w["ffn_w_v"], f16)
    fr = mm(frx, w["ffn_w_r"], f16)
    ffn_x = lop.channel_mix(cursors, ffn_state, fr, fv, ffn_x)
    state[:, S + 1] = ffn_state
    return lop.binary("add", ffn_x, x)


@pytest.mark.gpu
@pytest.mark.parametrize("quant", ["int8", "nf4"])
@pytest.mark.parametrize("runs", [[(2, 3), (0, 1), (5, 4)], [(1, 32)], [(4, 1)]], ids=["8 tokens", "32-token prompt (chunk kernels)", "1 token"])
def test_v5_layer_against_numpy(gpu, oracle, quant, runs):
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v5 = importlib.import_module(gpu.__name__ + ".v5")
    print("v5 layer on the GPU", quant, runs, flush=True)
    H, S, hidden, B = 12, 64, 2688, 6
    C = H * S
    rng = np.random.default_rng(SEED + len(runs))
    w = v5.random_layer_weights(rng, C, H, S, hidden, layer=7)
    cursors = lop.pack_cursors(runs)
    A = len(cursors)
    x = rng.standard_normal((A, C)).astype(np.float16)
    state = (0.1 * rng.standard_normal((B, S + 2, C))).astype(np.float32)

    layer = v5.Layer(torch, w, quant)
    # the CPU side works on what the packed matrices represent
    wq = dict(w)
    for name in v5.QUANTIZED:
        mtx = layer.m[name]
        if quant == "int8":
            wq[name] = int8_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy())
        else:
            wq[name] = nf4_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy(), np.array(gpu.NF4_QUANT, dtype=np.float32))
    want_state = state.copy()
    want = layer_numpy(lop, wq, x, want_state, cursors, H, S)

    buf = v5.Runtime(torch, C, hidden, A)
    buf.x.copy_(torch.from_numpy(x).cuda().reshape(1, A, C))
    sd = torch.from_numpy(state.copy()).cuda()
    v5.dispatch_layer(layer, buf, sd, torch.from_numpy(cursors.view(np.int32)).cuda(), A, H, S)
    torch.cuda.synchronize()
    got = buf.x.cpu().numpy()[0]
    # f16 buffers between the ops: a few f16 ulps of the O(1) activations
    assert_close(got, want, 1e-2, "layer output")
    assert_close(sd.cpu().numpy(), want_state, 1e-2, "state after the run")
    untouched = [b for b in range(B) if b not in [s for s, _ in runs]]
    assert np.array_equal(sd.cpu().numpy()[untouched], state[untouched])
