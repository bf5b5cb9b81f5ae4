"""Host-side mirror of one RWKV-v7 layer as the reference dispatches it (src/runtime/v7.rs:704-1006):
the same ops in the same order on the same buffers, every op one library call on torch's current
stream.  Weights are random-init tensors of the reference's shapes (src/runtime/v7.rs:77-128);
nothing here loads a checkpoint."""
import importlib

import numpy as np

_pkg = importlib.import_module(__name__.rsplit(".", 1)[0])
LayerOp, Matrix, turbo, matmul_vec_group = _pkg.LayerOp, _pkg.Matrix, _pkg.turbo, _pkg.matmul_vec_group
ACT_NONE, ACT_SQUARED_RELU, ACT_TANH, ACT_SIGMOID = _pkg.ACT_NONE, _pkg.ACT_SQUARED_RELU, _pkg.ACT_TANH, _pkg.ACT_SIGMOID

L2_EPS = 1.0e-12  # Model::L2_EPS, src/runtime/v7.rs:46
LN_EPS = 1.0e-5   # Model::LN_EPS, src/runtime/v7.rs:47
GN_EPS = 64.0e-5  # Model::GN_EPS, src/runtime/v7.rs:48
RANK_W, RANK_A, RANK_G, RANK_V = 64, 64, 128, 32  # inner sizes of the four adapters (read from the tensors by the reference)

QUANTIZED = ("att_w_r", "att_w_k", "att_w_v", "att_w_o", "ffn_w_k", "ffn_w_v")
ADAPTERS = ("w1", "w2", "a1", "a2", "g1", "g2", "v1", "v2")


def random_layer_weights(rng, C, H, S, hidden):
    """numpy weights of one layer: matrices [out, in] f16 ~ N(0, 0.02), adapters a little larger, vectors
    of plausible ranges (v7 models are loaded without the per-layer discount: the default rescale is 1024,
    src/runtime/v7.rs:50)."""
    h16 = lambda *s, std=0.02: (rng.standard_normal(s, dtype=np.float32) * np.float32(std)).astype(np.float16)
    w = {
        "att_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "att_ln_b": h16(C, std=0.1),
        "ffn_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "ffn_ln_b": h16(C, std=0.1),
        "w0": (-1.0 + 0.5 * rng.standard_normal(C)).astype(np.float16), "a0": h16(C, std=0.5), "v0": h16(C, std=0.5),
        "r_k": h16(H, S, std=0.3), "k_k": (0.5 + 0.3 * rng.standard_normal(C)).astype(np.float16), "k_a": rng.random(C).astype(np.float16),
        "gn_w": (1.0 + 0.1 * rng.standard_normal((H, S))).astype(np.float16), "gn_b": h16(H, S, std=0.1),
        "w1": h16(RANK_W, C, std=0.05), "w2": h16(C, RANK_W, std=0.1), "a1": h16(RANK_A, C, std=0.05), "a2": h16(C, RANK_A, std=0.1),
        "g1": h16(RANK_G, C, std=0.05), "g2": h16(C, RANK_G, std=0.1), "v1": h16(RANK_V, C, std=0.05), "v2": h16(C, RANK_V, std=0.1),
    }
    for name in ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g", "ffn_x_k"):
        w[name] = rng.random(C).astype(np.float16)
    for name, (R, K) in {"att_w_r": (C, C), "att_w_k": (C, C), "att_w_v": (C, C), "att_w_o": (C, C), "ffn_w_k": (hidden, C), "ffn_w_v": (C, hidden)}.items():
        w[name] = h16(R, K)
    return w


class Layer:
    """Device weights of one layer: the six big matrices quantised (`quant`: "int8" or "nf4"), the
    adapters as `Matrix::Fp16`, vectors as the reference keeps them."""

    def __init__(self, torch, weights, quant):
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.t = {k: dev(v) for k, v in weights.items() if k not in QUANTIZED}
        pack = Matrix.quant_u8 if quant == "int8" else Matrix.quant_nf4
        self.m = {k: pack(dev(weights[k])) for k in QUANTIZED}
        for k in ADAPTERS:
            self.m[k] = Matrix.fp16(self.t[k])


class Runtime:
    """The buffers of a run of `A` tokens (`Runtime<F>`, src/runtime/v7.rs:281-370), F = f16."""

    def __init__(self, torch, C, hidden, A):
        z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")
        for name in ("x", "att_x", "att_v0", "att_rx", "att_wx", "att_kx", "att_vx", "att_ax", "att_gx", "att_r", "att_w", "att_k", "att_v", "att_a",
                     "att_g", "att_o", "att_kk", "att_vv", "ffn_x", "ffn_kx", "ffn_v"):
            setattr(self, name, z(1, A, C))
        self.att_n = z(4, A, C)
        self.aux_w, self.aux_a, self.aux_g, self.aux_v = z(1, A, RANK_W), z(1, A, RANK_A), z(1, A, RANK_G), z(1, A, RANK_V)
        self.ffn_k = z(1, A, hidden)


class PackedShifts:
    """The six token-shift factors of a layer's attention half stacked and repeated over the tokens of a run
    (`[C, A, 6]`, made once per layer and run length with `TensorOp::broadcast`), so that one `token_shift`
    in the reference's per-token form (src/tensor/ops.rs:1409-1414) replaces six launches."""

    NAMES = ("x_r", "x_w", "x_k", "x_v", "x_a", "x_g")

    def __init__(self, torch, layer, A):
        C = layer.t["x_r"].numel()
        self.mix = torch.empty((6, A, C), dtype=torch.float16, device="cuda")
        LayerOp.broadcast(torch.stack([layer.t[n] for n in self.NAMES]).view(6, 1, C), self.mix)
        self.sx = torch.zeros_like(self.mix)


def dispatch_layer(layer, buf, state, cursors, A, H, S, index, rescale_now=False, shifts=None):
    """src/runtime/v7.rs:704-1006.  `state`: this layer's f32 tensor (B, S + 2, C): rows 0..S the
    attention state, row S + 1 the feed-forward one; `index`: the layer's number (layer 0 keeps its
    values as `att_v0`, the later ones mix theirs with it)."""
    t, m, C = layer.t, layer.m, H * S
    B = state.shape[0]
    fast = turbo(A)
    att_state = ((C, S + 1, B), (C, S + 2, B), (0, 0, 0))
    ffn_state = ((C, 1, B), (C, S + 2, B), (0, S + 1, 0))
    heads = lambda x: x.view(A, H, S)
    plane = lambda i: ((C, A, 1), (C, A, 4), (0, 0, i))

    LayerOp.blit(buf.x, buf.att_x)
    LayerOp.layer_norm(t["att_ln_w"], t["att_ln_b"], buf.att_x, LN_EPS)
    if shifts is None:
        for name, out in (("x_r", buf.att_rx), ("x_w", buf.att_wx), ("x_k", buf.att_kx), ("x_v", buf.att_vx), ("x_a", buf.att_ax), ("x_g", buf.att_gx)):
            LayerOp.token_shift(cursors, t[name], state, buf.att_x, out, True, state_view=att_state)
        rx, wx, kx, vx, ax, gx = ((b, {}) for b in (buf.att_rx, buf.att_wx, buf.att_kx, buf.att_vx, buf.att_ax, buf.att_gx))
    else:
        # one launch for the six shifts; the products read their slice of the stack through views
        LayerOp.token_shift(cursors, shifts.mix, state, buf.att_x, shifts.sx, True, state_view=att_state)
        rx, wx, kx, vx, ax, gx = ((shifts.sx, dict(input_view=((C, A, 1), (C, A, 6), (0, 0, i)))) for i in range(6))
    # the three independent projections in one call: the library's form of a `TensorOp::List` of them
    matmul_vec_group([(m["att_w_r"], rx[0], buf.att_r, ACT_NONE, False, rx[1]), (m["att_w_k"], kx[0], buf.att_k, ACT_NONE, False, kx[1]),
                      (m["att_w_v"], vx[0], buf.att_v, ACT_NONE, False, vx[1])])
    m["w1"].matmul_op(wx[0], buf.aux_w, ACT_TANH, fast, **wx[1])
    m["w2"].matmul_op(buf.aux_w, buf.att_w, ACT_NONE, fast)
    LayerOp.add(t["w0"], buf.att_w)
    m["a1"].matmul_op(ax[0], buf.aux_a, ACT_NONE, fast, **ax[1])
    m["a2"].matmul_op(buf.aux_a, buf.att_a, ACT_NONE, fast)
    LayerOp.add_activate(t["a0"], buf.att_a, ACT_NONE, ACT_NONE, ACT_SIGMOID)
    m["g1"].matmul_op(gx[0], buf.aux_g, ACT_SIGMOID, fast, **gx[1])
    m["g2"].matmul_op(buf.aux_g, buf.att_g, ACT_NONE, fast)
    LayerOp.blit(buf.att_k, buf.att_kk)
    LayerOp.mul(t["k_k"], buf.att_kk)
    LayerOp.l2_norm(heads(buf.att_kk), L2_EPS)
    LayerOp.control_k_v7(t["k_a"], buf.att_a, buf.att_k)
    if index == 0:
        LayerOp.blit(buf.att_v, buf.att_v0)
    else:
        m["v1"].matmul_op(vx[0], buf.aux_v, ACT_NONE, fast, **vx[1])
        m["v2"].matmul_op(buf.aux_v, buf.att_vv, ACT_NONE, fast)
        LayerOp.add_activate(t["v0"], buf.att_vv, ACT_NONE, ACT_NONE, ACT_SIGMOID)
        LayerOp.lerp(buf.att_v0, buf.att_v, buf.att_vv, True)
    for i, src in enumerate((buf.att_k, buf.att_v, buf.att_a, buf.att_kk)):
        LayerOp.blit(src, buf.att_n, output_view=plane(i))
    LayerOp.time_mix_v7(cursors, state, heads(buf.att_r), heads(buf.att_w), buf.att_n.view(4, A, H, S), heads(buf.att_x), state_view=att_state)
    LayerOp.group_norm(t["gn_w"], t["gn_b"], heads(buf.att_x), GN_EPS)
    LayerOp.time_first_v7(t["r_k"], heads(buf.att_r), buf.att_n.view(4, A, H, S), heads(buf.att_x))
    LayerOp.mul(buf.att_g, buf.att_x)
    m["att_w_o"].matmul_op(buf.att_x, buf.att_o, ACT_NONE, fast)
    LayerOp.add(buf.att_o, buf.x)

    LayerOp.blit(buf.x, buf.ffn_x)
    LayerOp.layer_norm(t["ffn_ln_w"], t["ffn_ln_b"], buf.ffn_x, LN_EPS)
    LayerOp.token_shift(cursors, t["ffn_x_k"], state, buf.ffn_x, buf.ffn_kx, True, state_view=ffn_state)
    m["ffn_w_k"].matmul_op(buf.ffn_kx, buf.ffn_k, ACT_SQUARED_RELU, fast)
    m["ffn_w_v"].matmul_op_sparse(buf.ffn_k, buf.ffn_v, ACT_NONE, fast)
    LayerOp.channel_mix_v7(cursors, state, buf.ffn_v, buf.ffn_x, state_view=ffn_state)
    LayerOp.add(buf.ffn_x, buf.x)
    if rescale_now:
        LayerOp.affine(buf.x, 0.5, 0.0)
