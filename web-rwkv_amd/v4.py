"""Host-side mirror of one RWKV-v4 layer as the reference dispatches it (src/runtime/v4.rs:620-791):
the same ops in the same order on the same buffers, every op one library call on torch's current
stream.  Weights are random-init tensors of the reference's shapes (src/runtime/v4.rs:60-100);
nothing here loads a checkpoint."""
import importlib

import numpy as np

_pkg = importlib.import_module(__name__.rsplit(".", 1)[0])
LayerOp, Matrix, turbo, matmul_vec_group = _pkg.LayerOp, _pkg.Matrix, _pkg.turbo, _pkg.matmul_vec_group
ACT_NONE, ACT_SQUARED_RELU = _pkg.ACT_NONE, _pkg.ACT_SQUARED_RELU

LN_EPS = 1.0e-5  # Model::LN_EPS, src/runtime/v4.rs:45

QUANTIZED = ("att_w_k", "att_w_v", "att_w_r", "att_w_o", "ffn_w_k", "ffn_w_v", "ffn_w_r")


def random_layer_weights(rng, C, hidden, layer=0):
    """numpy weights of one layer: matrices [out, in] f16 ~ N(0, 0.02) (att.output and ffn.value with the
    loader's 2^-(layer / 6) discount), vectors of plausible ranges; time_decay as the loader leaves it,
    -exp(w) (src/runtime/loader.rs:436-470)."""
    h16 = lambda *s, std=0.02: (rng.standard_normal(s, dtype=np.float32) * np.float32(std)).astype(np.float16)
    disc = np.float32(2.0 ** -(layer // 6))
    w = {
        "att_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "att_ln_b": h16(C, std=0.1),
        "ffn_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "ffn_ln_b": h16(C, std=0.1),
        "time_decay": (-np.exp((-1.0 + 0.5 * rng.standard_normal(C)).astype(np.float32))).astype(np.float32),
        "time_first": (0.3 * rng.standard_normal(C)).astype(np.float32),
    }
    for name in ("time_mix_k", "time_mix_v", "time_mix_r", "ffn_time_mix_k", "ffn_time_mix_r"):
        w[name] = rng.random(C).astype(np.float16)
    for name, (R, K) in {"att_w_k": (C, C), "att_w_v": (C, C), "att_w_r": (C, C), "att_w_o": (C, C), "ffn_w_k": (hidden, C), "ffn_w_v": (C, hidden),
                         "ffn_w_r": (C, C)}.items():
        m = rng.standard_normal((R, K), dtype=np.float32) * np.float32(0.02)
        if name in ("att_w_o", "ffn_w_v"):
            m = m * disc
        w[name] = m.astype(np.float16)
    return w


class Layer:
    def __init__(self, torch, weights, quant):
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.t = {k: dev(v) for k, v in weights.items() if k not in QUANTIZED}
        pack = Matrix.quant_u8 if quant == "int8" else Matrix.quant_nf4
        self.m = {k: pack(dev(weights[k])) for k in QUANTIZED}


class Runtime:
    """The buffers of a run of `A` tokens (`Runtime<F>`, src/runtime/v4.rs:234-285), F = f16."""

    def __init__(self, torch, C, hidden, A):
        z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device="cuda")
        f32 = torch.float32
        self.x, self.att_x, self.att_kx, self.att_vx, self.att_rx, self.att_o = (z(1, A, C) for _ in range(6))
        self.aux_x, self.att_k, self.att_v, self.att_r = (z(1, A, C, dt=f32) for _ in range(4))
        self.ffn_x, self.ffn_kx, self.ffn_rx, self.ffn_v, self.ffn_r = (z(1, A, C) for _ in range(5))
        self.ffn_k = z(1, A, hidden)


def dispatch_layer(layer, buf, state, cursors, A, C, rescale_now=False):
    """src/runtime/v4.rs:620-791.  `state`: this layer's f32 rows (B, 5, C): rows 0..3 the attention
    state (`State::att`, :175-179), row 4 the feed-forward one (`State::ffn`, :181-184)."""
    t, m = layer.t, layer.m
    B = state.shape[0]
    fast = turbo(A)
    att_state = ((C, 4, B), (C, 5, B), (0, 0, 0))
    ffn_state = ((C, 1, B), (C, 5, B), (0, 4, 0))

    LayerOp.blit(buf.x, buf.att_x)
    LayerOp.layer_norm(t["att_ln_w"], t["att_ln_b"], buf.att_x, LN_EPS)
    for name, out in (("time_mix_k", buf.att_kx), ("time_mix_v", buf.att_vx), ("time_mix_r", buf.att_rx)):
        LayerOp.token_shift(cursors, t[name], state, buf.att_x, out, False, state_view=att_state)
    matmul_vec_group([(m["att_w_k"], buf.att_kx, buf.att_k, ACT_NONE, False, {}), (m["att_w_v"], buf.att_vx, buf.att_v, ACT_NONE, False, {}),
                      (m["att_w_r"], buf.att_rx, buf.att_r, ACT_NONE, False, {})])
    LayerOp.blit(buf.att_x, buf.aux_x)
    LayerOp.time_mix_v4(cursors, t["time_decay"], t["time_first"], state, buf.att_k, buf.att_v, buf.att_r, buf.aux_x, state_view=att_state)
    LayerOp.blit(buf.aux_x, buf.att_x)
    m["att_w_o"].matmul_op(buf.att_x, buf.att_o, ACT_NONE, fast)
    LayerOp.add(buf.att_o, buf.x)

    LayerOp.blit(buf.x, buf.ffn_x)
    LayerOp.layer_norm(t["ffn_ln_w"], t["ffn_ln_b"], buf.ffn_x, LN_EPS)
    LayerOp.token_shift(cursors, t["ffn_time_mix_k"], state, buf.ffn_x, buf.ffn_kx, False, state_view=ffn_state)
    LayerOp.token_shift(cursors, t["ffn_time_mix_r"], state, buf.ffn_x, buf.ffn_rx, False, state_view=ffn_state)
    matmul_vec_group([(m["ffn_w_k"], buf.ffn_kx, buf.ffn_k, ACT_SQUARED_RELU, False, {}), (m["ffn_w_r"], buf.ffn_rx, buf.ffn_r, ACT_NONE, False, {})])
    m["ffn_w_v"].matmul_op_sparse(buf.ffn_k, buf.ffn_v, ACT_NONE, fast)
    LayerOp.channel_mix(cursors, state, buf.ffn_r, buf.ffn_v, buf.ffn_x, state_view=ffn_state)
    LayerOp.add(buf.ffn_x, buf.x)
    if rescale_now:
        LayerOp.affine(buf.x, 0.5, 0.0)
