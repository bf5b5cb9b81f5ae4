"""One whole RWKV-v6 layer, dispatched op by op like the reference (src/runtime/v6.rs:758-955),
on the GPU through the library against a numpy composition of the oracle's restatements."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close, int8_dequant64, nf4_dequant64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525300


def layer_numpy(lop, w, x, state, cursors, H, S):
    """The layer on the CPU: every buffer rounded to the type the reference's runtime gives it
    (f16 except aux_x, att_k / v / r and time_decay: src/runtime/v6.rs:270-303)."""
    f16, f32, f64 = np.float16, np.float32, np.float64
    A, C = x.shape
    mm = lambda a, W, dt: (a.astype(f64) @ W.astype(f64).T).astype(dt)
    att_x = lop.layer_norm(w["att_ln_w"], w["att_ln_b"], x, 1e-5)
    att_xx = lop.token_shift(cursors, w["time_mix_x"], state[:, 0], att_x, f16, reversed=True)[0]
    tmx = np.tanh(mm(att_xx, w["time_mix_w1"], f64)).astype(f16).reshape(A, 5, 32)
    tmt = np.swapaxes(tmx, 0, 1)
    time_mix = np.stack([mm(tmt[b], w["time_mix_w2"][b], f16) for b in range(5)])
    time_mix = lop.binary("add", w["time_mix"], time_mix)
    att_sx = lop.token_shift(cursors, time_mix, state[:, 0], att_x, f16, counts=5, reversed=True)
    k, v, r = (mm(att_sx[i], w[n], f32) for i, n in ((1, "att_w_k"), (2, "att_w_v"), (3, "att_w_r")))
    g = mm(att_sx[4], w["att_w_g"], f16)
    att_w = np.tanh(mm(att_sx[0], w["time_decay_w1"], f64)).astype(f16)
    decay = lop.activation(3, lop.binary("add", w["time_decay"], mm(att_w, w["time_decay_w2"], f32)))
    att = np.ascontiguousarray(state[:, :S + 1])
    aux = lop.time_mix_v6(cursors, decay.reshape(A, H, S), w["time_first"], att, k.reshape(A, H, S), v.reshape(A, H, S), r.reshape(A, H, S),
                          att_x.astype(f32).reshape(A, H, S))
    state[:, :S + 1] = att
    aux = lop.group_norm(w["gn_w"], w["gn_b"], aux, 64e-5)
    att_x = lop.binary("mul", g, aux.reshape(A, C).astype(f16), act_x=7)
    x = lop.binary("add", mm(att_x, w["att_w_o"], f16), x)
    ffn_x = lop.layer_norm(w["ffn_ln_w"], w["ffn_ln_b"], x, 1e-5)
    ffn_state = np.ascontiguousarray(state[:, S + 1])
    kx = lop.token_shift(cursors, w["ffn_time_mix_k"], ffn_state, ffn_x, f16, reversed=True)[0]
    rx = lop.token_shift(cursors, w["ffn_time_mix_r"], ffn_state, ffn_x, f16, reversed=True)[0]
    fk = lop.activation(1, mm(kx, w["ffn_w_k"], f32)).astype(f16)
    fv = mm(fk, w["ffn_w_v"], f16)
    fr = mm(rx, w["ffn_w_r"], f16)
    ffn_x = lop.channel_mix(cursors, ffn_state, fr, fv, ffn_x)
    state[:, S + 1] = ffn_state
    return lop.binary("add", ffn_x, x)


@pytest.mark.gpu
@pytest.mark.parametrize("quant", ["int8", "nf4"])
@pytest.mark.parametrize("runs", [[(2, 3), (0, 1), (5, 4)], [(1, 20), (3, 12)], [(4, 1)]], ids=["8 tokens", "32 tokens (chunk kernels)", "1 token"])
def test_v6_layer_against_numpy(gpu, oracle, quant, runs):
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v6 = importlib.import_module(gpu.__name__ + ".v6")
    print("v6 layer on the GPU", quant, runs, flush=True)
    H, S, hidden, B = 4, 64, 512, 6
    C = H * S
    rng = np.random.default_rng(SEED + len(runs))
    w = v6.random_layer_weights(rng, C, H, S, hidden, layer=7)
    cursors = lop.pack_cursors(runs)
    A = len(cursors)
    x = rng.standard_normal((A, C)).astype(np.float16)
    state = (0.1 * rng.standard_normal((B, S + 2, C))).astype(np.float32)

    layer = v6.Layer(torch, w, quant)
    # the CPU side works on what the packed matrices represent
    wq = dict(w)
    for name in v6.QUANTIZED:
        mtx = layer.m[name]
        if quant == "int8":
            wq[name] = int8_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy())
        else:
            wq[name] = nf4_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy(), np.array(gpu.NF4_QUANT, dtype=np.float32))
    want_state = state.copy()
    want = layer_numpy(lop, wq, x, want_state, cursors, H, S)

    buf = v6.Runtime(torch, C, hidden, A)
    buf.x.copy_(torch.from_numpy(x).cuda().reshape(1, A, C))
    sd = torch.from_numpy(state.copy()).cuda()
    v6.dispatch_layer(layer, buf, sd, torch.from_numpy(cursors.view(np.int32)).cuda(), A, H, S)
    torch.cuda.synchronize()
    got = buf.x.cpu().numpy()[0]
    # f16 buffers between 35 ops: a few f16 ulps of the O(1) activations
    assert_close(got, want, 1e-2, "layer output")
    assert_close(sd.cpu().numpy(), want_state, 1e-2, "state after the run")
    untouched = [b for b in range(B) if b not in [s for s, _ in runs]]
    assert np.array_equal(sd.cpu().numpy()[untouched], state[untouched])


@pytest.mark.gpu
@pytest.mark.parametrize("quant", ["int8", "nf4"])
@pytest.mark.parametrize("runs", [[(2, 3), (0, 1), (5, 4)], [(1, 20), (3, 12)], [(4, 1)]], ids=["8 tokens", "32 tokens (chunk kernels)", "1 token"])
def test_v6_layer_fused_equals_op_list(gpu, oracle, quant, runs):
    # the 12-launch form of the layer against the op list: same buffers, same roundings
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v6 = importlib.import_module(gpu.__name__ + ".v6")
    print("v6 layer, fused, on the GPU", quant, runs, flush=True)
    H, S, hidden, B = 4, 64, 512, 6
    C = H * S
    rng = np.random.default_rng(SEED + 100 + len(runs))
    layer = v6.Layer(torch, v6.random_layer_weights(rng, C, H, S, hidden, layer=3), quant)
    cursors = lop.pack_cursors(runs)
    A = len(cursors)
    curd = torch.from_numpy(cursors.view(np.int32)).cuda()
    x = rng.standard_normal((A, C)).astype(np.float16)
    state = (0.1 * rng.standard_normal((B, S + 2, C))).astype(np.float32)
    outs = []
    for fused in (False, True):
        buf = v6.Runtime(torch, C, hidden, A)
        buf.x.copy_(torch.from_numpy(x).cuda().reshape(1, A, C))
        sd = torch.from_numpy(state.copy()).cuda()
        (v6.dispatch_layer_fused if fused else v6.dispatch_layer)(layer, buf, sd, curd, A, H, S, rescale_now=True)
        torch.cuda.synchronize()
        outs.append((buf.x.cpu().numpy()[0].astype(np.float32), sd.cpu().numpy()))
    # f32 sums in another order flip an f16 rounding here and there: a few f16 ulps after 35 ops
    assert_close(outs[1][0], outs[0][0], 4e-3, "layer output, fused vs op list")
    assert_close(outs[1][1], outs[0][1], 4e-3, "state, fused vs op list")
    assert np.mean(outs[1][0] == outs[0][0]) > 0.9  # and most outputs are the same f16 value
