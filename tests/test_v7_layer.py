"""Two consecutive RWKV-v7 layers (the first keeps its values as `v0`, the second mixes its own with
them), dispatched op by op like the reference (src/runtime/v7.rs:704-1006), on the GPU through the
library against a numpy composition of the oracle's restatements."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close, int8_dequant64, nf4_dequant64

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525700


def layer_numpy(lop, w, x, v0, state, cursors, H, S, index):
    """The layer on the CPU, every buffer rounded to f16 as the reference's runtime keeps it
    (src/runtime/v7.rs:281-320).  Returns the new x and the values the first layer hands on."""
    f16, f64 = np.float16, np.float64
    A, C = x.shape
    mm = lambda a, W: (a.astype(f64) @ W.astype(f64).T)
    att_x = lop.layer_norm(w["att_ln_w"], w["att_ln_b"], x, 1e-5)
    rx, wx, kx, vx, ax, gx = (lop.token_shift(cursors, w[n], state[:, 0], att_x, f16, reversed=True)[0] for n in ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g"))
    r, k, v = mm(rx, w["att_w_r"]).astype(f16), mm(kx, w["att_w_k"]).astype(f16), mm(vx, w["att_w_v"]).astype(f16)
    aux_w = np.tanh(mm(wx, w["w1"])).astype(f16)
    att_w = lop.binary("add", w["w0"], mm(aux_w, w["w2"]).astype(f16))
    aux_a = mm(ax, w["a1"]).astype(f16)
    att_a = lop.binary("add", w["a0"], mm(aux_a, w["a2"]).astype(f16), act_out=6)
    aux_g = lop.activation(6, mm(gx, w["g1"]).astype(np.float32)).astype(f16)
    att_g = mm(aux_g, w["g2"]).astype(f16)
    kk = lop.binary("mul", w["k_k"], k)
    kk = lop.l2_norm(kk.reshape(A, H, S), 1e-12).reshape(A, C)
    k = lop.control_k_v7(w["k_a"], att_a, k)
    if index == 0:
        v0 = v.copy()
    else:
        aux_v = mm(vx, w["v1"]).astype(f16)
        vv = lop.binary("add", w["v0"], mm(aux_v, w["v2"]).astype(f16), act_out=6)
        v = lop.lerp(v0, v, vv, reversed=True)
    n = np.stack([k, v, att_a, kk]).reshape(4, A, H, S)
    att = np.ascontiguousarray(state[:, :S + 1])
    y = lop.time_mix_v7(cursors, att, r.reshape(A, H, S), att_w.reshape(A, H, S), n, att_x.reshape(A, H, S))
    state[:, :S + 1] = att
    y = lop.group_norm(w["gn_w"], w["gn_b"], y, 64e-5)
    y = lop.time_first_v7(w["r_k"], r.reshape(A, H, S), n, y)
    att_x = lop.binary("mul", att_g, y.reshape(A, C))
    x = lop.binary("add", mm(att_x, w["att_w_o"]).astype(f16), x)
    ffn_x = lop.layer_norm(w["ffn_ln_w"], w["ffn_ln_b"], x, 1e-5)
    ffn_state = np.ascontiguousarray(state[:, S + 1])
    fkx = lop.token_shift(cursors, w["ffn_x_k"], ffn_state, ffn_x, f16, reversed=True)[0]
    fk = lop.activation(1, mm(fkx, w["ffn_w_k"]).astype(np.float32)).astype(f16)
    fv = mm(fk, w["ffn_w_v"]).astype(f16)
    ffn_x = lop.channel_mix_v7(cursors, ffn_state, fv, ffn_x)
    state[:, S + 1] = ffn_state
    return lop.binary("add", ffn_x, x), v0


@pytest.mark.gpu
@pytest.mark.parametrize("quant", ["int8", "nf4"])
@pytest.mark.parametrize("runs", [[(2, 3), (0, 1), (5, 4)], [(1, 20), (3, 12)], [(4, 1)]], ids=["8 tokens", "32 tokens (chunk kernels)", "1 token"])
def test_v7_layers_against_numpy(gpu, oracle, quant, runs):
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v7 = importlib.import_module(gpu.__name__ + ".v7")
    print("v7 layers on the GPU", quant, runs, flush=True)
    H, S, hidden, B, L = 4, 64, 1024, 6, 2
    C = H * S
    rng = np.random.default_rng(SEED + len(runs))
    cursors = lop.pack_cursors(runs)
    A = len(cursors)
    x = rng.standard_normal((A, C)).astype(np.float16)
    curd = torch.from_numpy(cursors.view(np.int32)).cuda()
    buf = v7.Runtime(torch, C, hidden, A)
    buf.x.copy_(torch.from_numpy(x).cuda().reshape(1, A, C))
    want, v0 = x, None
    for index in range(L):
        w = v7.random_layer_weights(rng, C, H, S, hidden)
        state = (0.1 * rng.standard_normal((B, S + 2, C))).astype(np.float32)
        layer = v7.Layer(torch, w, quant)
        wq = dict(w)  # the CPU side works on what the packed matrices represent
        for name in v7.QUANTIZED:
            mtx = layer.m[name]
            if quant == "int8":
                wq[name] = int8_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy())
            else:
                wq[name] = nf4_dequant64(mtx.w.cpu().numpy(), mtx.m.cpu().numpy(), np.array(gpu.NF4_QUANT, dtype=np.float32))
        want_state = state.copy()
        want, v0 = layer_numpy(lop, wq, want, v0, want_state, cursors, H, S, index)
        sd = torch.from_numpy(state.copy()).cuda()
        v7.dispatch_layer(layer, buf, sd, curd, A, H, S, index)
        torch.cuda.synchronize()
        got = buf.x.cpu().numpy()[0]
        # f16 buffers between 50 ops: a few f16 ulps of the O(1) activations
        assert_close(got, want, 1.5e-2, f"output of layer {index}")
        assert_close(sd.cpu().numpy(), want_state, 1.5e-2, f"state of layer {index} after the run")
        untouched = [b for b in range(B) if b not in [s for s, _ in runs]]
        assert np.array_equal(sd.cpu().numpy()[untouched], state[untouched])
        want = got  # the next layer starts from the device's x on both sides


@pytest.mark.gpu
@pytest.mark.parametrize("runs", [[(2, 3), (0, 1), (5, 4)], [(1, 32)], [(4, 1)]], ids=["8 tokens", "32 tokens", "1 token"])
def test_v7_layer_packed_token_shifts_equal_the_op_list(gpu, runs):
    # the six token shifts in one launch (factors stacked and repeated over the tokens with `broadcast`): bit-equal
    import torch

    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    v7 = importlib.import_module(gpu.__name__ + ".v7")
    print("v7 layer, packed token shifts", runs, flush=True)
    H, S, hidden, B = 4, 64, 1024, 6
    C = H * S
    rng = np.random.default_rng(SEED + 50 + len(runs))
    cursors = lop.pack_cursors(runs)
    A = len(cursors)
    curd = torch.from_numpy(cursors.view(np.int32)).cuda()
    layer = v7.Layer(torch, v7.random_layer_weights(rng, C, H, S, hidden), "int8")
    x = rng.standard_normal((A, C)).astype(np.float16)
    state = (0.1 * rng.standard_normal((B, S + 2, C))).astype(np.float32)
    outs = []
    for packed in (False, True):
        buf = v7.Runtime(torch, C, hidden, A)
        buf.x.copy_(torch.from_numpy(x).cuda().reshape(1, A, C))
        buf.att_v0.copy_(torch.from_numpy(x[::-1].copy()).cuda().reshape(1, A, C))
        sd = torch.from_numpy(state.copy()).cuda()
        v7.dispatch_layer(layer, buf, sd, curd, A, H, S, 1, shifts=v7.PackedShifts(torch, layer, A) if packed else None)
        torch.cuda.synchronize()
        outs.append((buf.x.cpu().numpy(), sd.cpu().numpy()))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
