"""Host-side mirror of one RWKV-v6 layer as the reference dispatches it (src/runtime/v6.rs:700-958):
the same ops in the same order on the same buffers, every op one library call on torch's current
stream.  Weights are random-init tensors of the reference's shapes (src/runtime/v6.rs:76-108,
:1040-1132); nothing here loads a checkpoint."""
import importlib

import numpy as np

_pkg = importlib.import_module(__name__.rsplit(".", 1)[0])
LayerOp, Matrix, turbo, matmul_vec_group, FusedV6 = _pkg.LayerOp, _pkg.Matrix, _pkg.turbo, _pkg.matmul_vec_group, _pkg.FusedV6
ACT_NONE, ACT_SQUARED_RELU, ACT_TANH, ACT_STABLE_EXP, ACT_SILU = _pkg.ACT_NONE, _pkg.ACT_SQUARED_RELU, _pkg.ACT_TANH, _pkg.ACT_STABLE_EXP, _pkg.ACT_SILU

LN_EPS = 1.0e-5   # Model::LN_EPS, src/runtime/v6.rs:46
GN_EPS = 64.0e-5  # Model::GN_EPS, src/runtime/v6.rs:47
TIME_MIX_LORA, TIME_DECAY_LORA = 32, 64


def random_layer_weights(rng, C, H, S, hidden, layer=0):
    """numpy weights of one layer: matrices [out, in] f16 ~ N(0, 0.02) (att.output and ffn.value with the
    loader's 2^-(layer / 6) discount, src/runtime/loader.rs:660-661), vectors of plausible ranges."""
    h16 = lambda *s, std=0.02: (rng.standard_normal(s, dtype=np.float32) * np.float32(std)).astype(np.float16)
    disc = np.float32(2.0 ** -(layer // 6))
    w = {
        "att_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "att_ln_b": h16(C, std=0.1),
        "ffn_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "ffn_ln_b": h16(C, std=0.1),
        "time_mix_x": rng.random(C).astype(np.float16), "time_mix": rng.random((5, 1, C)).astype(np.float16),
        "time_mix_w1": h16(5 * TIME_MIX_LORA, C), "time_mix_w2": h16(5, C, TIME_MIX_LORA, std=0.1),
        "time_decay": (-1.0 + 0.5 * rng.standard_normal(C)).astype(np.float16),
        "time_decay_w1": h16(TIME_DECAY_LORA, C), "time_decay_w2": h16(C, TIME_DECAY_LORA, std=0.1),
        "time_first": (0.3 * rng.standard_normal((H, S))).astype(np.float32),
        "gn_w": (1.0 + 0.1 * rng.standard_normal((H, S))).astype(np.float16), "gn_b": h16(H, S, std=0.1),
        "ffn_time_mix_k": rng.random(C).astype(np.float16), "ffn_time_mix_r": rng.random(C).astype(np.float16),
    }
    for name, (R, K) in {"att_w_k": (C, C), "att_w_v": (C, C), "att_w_r": (C, C), "att_w_g": (C, C), "att_w_o": (C, C),
                         "ffn_w_k": (hidden, C), "ffn_w_v": (C, hidden), "ffn_w_r": (C, C)}.items():
        m = rng.standard_normal((R, K), dtype=np.float32) * np.float32(0.02)
        if name in ("att_w_o", "ffn_w_v"):
            m = m * disc
        w[name] = m.astype(np.float16)
    return w


QUANTIZED = ("att_w_k", "att_w_v", "att_w_r", "att_w_g", "att_w_o", "ffn_w_k", "ffn_w_v", "ffn_w_r")


class Layer:
    """Device weights of one layer: the eight big matrices quantised (`quant`: "int8" or "nf4"), the
    low-rank adapters as `Matrix::Fp16`, vectors as the reference keeps them."""

    def __init__(self, torch, weights, quant):
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.t = {k: dev(v) for k, v in weights.items() if k not in QUANTIZED}
        pack = Matrix.quant_u8 if quant == "int8" else Matrix.quant_nf4
        self.m = {k: pack(dev(weights[k])) for k in QUANTIZED}
        for k in ("time_mix_w1", "time_mix_w2", "time_decay_w1", "time_decay_w2"):
            self.m[k] = Matrix.fp16(self.t[k])


class Runtime:
    """The buffers of a run of `A` tokens (`Runtime<F>`, src/runtime/v6.rs:270-345), F = f16."""

    def __init__(self, torch, C, hidden, A):
        z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device="cuda")
        f32 = torch.float32
        self.x, self.att_x, self.att_xx, self.att_g, self.att_o = (z(1, A, C) for _ in range(5))
        self.aux_x, self.att_k, self.att_v, self.att_r, self.time_decay = (z(1, A, C, dt=f32) for _ in range(5))
        self.att_sx, self.time_mix = z(5, A, C), z(5, A, C)
        self.att_w = z(1, A, TIME_DECAY_LORA)
        self.time_mix_x, self.time_mix_t = z(A, 5, TIME_MIX_LORA), z(5, A, TIME_MIX_LORA)
        self.ffn_x, self.ffn_kx, self.ffn_rx, self.ffn_v, self.ffn_r = (z(1, A, C) for _ in range(5))
        self.ffn_k = z(1, A, hidden)
        self.x2 = z(1, A, C)  # the residual between the two halves of a layer on the fused path


def dispatch_layer(layer, buf, state, cursors, A, H, S, rescale_now=False):
    """src/runtime/v6.rs:758-955.  `state`: this layer's f32 tensor (B, S + 2, C): rows 0..S the
    attention state (`State::att`, :187-191), row S + 1 the feed-forward one (`State::ffn`, :193-197)."""
    t, m, C = layer.t, layer.m, H * S
    B = state.shape[0]
    fast = turbo(A)
    att_state = ((C, S + 1, B), (C, S + 2, B), (0, 0, 0))
    ffn_state = ((C, 1, B), (C, S + 2, B), (0, S + 1, 0))
    heads = lambda x: x.view(A, H, S)
    slice_of = lambda i: ((C, A, 1), (C, A, 5), (0, 0, i))

    LayerOp.blit(buf.x, buf.att_x)
    LayerOp.layer_norm(t["att_ln_w"], t["att_ln_b"], buf.att_x, LN_EPS)
    LayerOp.token_shift(cursors, t["time_mix_x"], state, buf.att_x, buf.att_xx, True, state_view=att_state)
    m["time_mix_w1"].matmul_op(buf.att_xx, buf.time_mix_x.view(1, A, 5 * TIME_MIX_LORA), ACT_TANH, fast)
    LayerOp.transpose(buf.time_mix_x, buf.time_mix_t)
    m["time_mix_w2"].matmul_op(buf.time_mix_t, buf.time_mix, ACT_NONE, fast)
    LayerOp.add(t["time_mix"], buf.time_mix)
    LayerOp.token_shift(cursors, buf.time_mix, state, buf.att_x, buf.att_sx, True, state_view=att_state)
    # the four independent projections in one call: the library's form of a `TensorOp::List` of them
    matmul_vec_group([(m[n], buf.att_sx, out, ACT_NONE, False, dict(input_view=slice_of(i)))
                      for n, out, i in (("att_w_k", buf.att_k, 1), ("att_w_v", buf.att_v, 2), ("att_w_r", buf.att_r, 3), ("att_w_g", buf.att_g, 4))])
    m["time_decay_w1"].matmul_op(buf.att_sx, buf.att_w, ACT_TANH, fast, input_view=slice_of(0))
    m["time_decay_w2"].matmul_op(buf.att_w, buf.time_decay, ACT_NONE, fast)
    LayerOp.add(t["time_decay"], buf.time_decay)
    LayerOp.activate(buf.time_decay, ACT_STABLE_EXP)
    LayerOp.blit(buf.att_x, buf.aux_x)
    LayerOp.time_mix_v6(cursors, heads(buf.time_decay), t["time_first"], state, heads(buf.att_k), heads(buf.att_v), heads(buf.att_r), heads(buf.aux_x),
                        state_view=att_state)
    LayerOp.group_norm(t["gn_w"], t["gn_b"], heads(buf.aux_x), GN_EPS)
    LayerOp.blit(buf.aux_x, buf.att_x)
    LayerOp.mul_activate(buf.att_g, buf.att_x, ACT_SILU, ACT_NONE, ACT_NONE)
    m["att_w_o"].matmul_op(buf.att_x, buf.att_o, ACT_NONE, fast)
    LayerOp.add(buf.att_o, buf.x)

    LayerOp.blit(buf.x, buf.ffn_x)
    LayerOp.layer_norm(t["ffn_ln_w"], t["ffn_ln_b"], buf.ffn_x, LN_EPS)
    LayerOp.token_shift(cursors, t["ffn_time_mix_k"], state, buf.ffn_x, buf.ffn_kx, True, state_view=ffn_state)
    LayerOp.token_shift(cursors, t["ffn_time_mix_r"], state, buf.ffn_x, buf.ffn_rx, True, state_view=ffn_state)
    matmul_vec_group([(m["ffn_w_k"], buf.ffn_kx, buf.ffn_k, ACT_SQUARED_RELU, False, {}), (m["ffn_w_r"], buf.ffn_rx, buf.ffn_r, ACT_NONE, False, {})])
    m["ffn_w_v"].matmul_op_sparse(buf.ffn_k, buf.ffn_v, ACT_NONE, fast)
    LayerOp.channel_mix(cursors, state, buf.ffn_r, buf.ffn_v, buf.ffn_x, state_view=ffn_state)
    LayerOp.add(buf.ffn_x, buf.x)
    if rescale_now:
        LayerOp.affine(buf.x, 0.5, 0.0)


def dispatch_layer_fused(layer, buf, state, cursors, A, H, S, rescale_now=False):
    """The same layer in 12 launches: the 8 quantized products (3 launches for the independent ones, 2
    alone), the first halves of the two adapters, and 5 fused launches for the 27 small ops
    (`wrq_v6_*`).  Same buffers and results as `dispatch_layer` up to f32 summation order."""
    t, m, C = layer.t, layer.m, H * S
    B = state.shape[0]
    fast = turbo(A)
    att_state = ((C, S + 1, B), (C, S + 2, B), (0, 0, 0))
    ffn_state = ((C, 1, B), (C, S + 2, B), (0, S + 1, 0))
    slice_of = lambda i: ((C, A, 1), (C, A, 5), (0, 0, i))

    FusedV6.pre(C, A, cursors, buf.x, None, None, t["att_ln_w"], t["att_ln_b"], LN_EPS, state, att_state, [t["time_mix_x"]], buf.att_x, [buf.att_xx])
    m["time_mix_w1"].matmul_op(buf.att_xx, buf.time_mix_x.view(1, A, 5 * TIME_MIX_LORA), ACT_TANH, fast)
    FusedV6.time_mix(C, A, TIME_MIX_LORA, cursors, buf.time_mix_x, t["time_mix_w2"], t["time_mix"], state, att_state, buf.att_x, buf.att_sx)
    matmul_vec_group([(m[n], buf.att_sx, out, ACT_NONE, False, dict(input_view=slice_of(i)))
                      for n, out, i in (("att_w_k", buf.att_k, 1), ("att_w_v", buf.att_v, 2), ("att_w_r", buf.att_r, 3), ("att_w_g", buf.att_g, 4))])
    m["time_decay_w1"].matmul_op(buf.att_sx, buf.att_w, ACT_TANH, fast, input_view=slice_of(0))
    FusedV6.decay(C, A, TIME_DECAY_LORA, buf.att_w, t["time_decay_w2"], t["time_decay"], buf.time_decay)
    FusedV6.wkv_gate(S, H, A, cursors, buf.time_decay, t["time_first"], state, att_state, buf.att_k, buf.att_v, buf.att_r, buf.att_g, t["gn_w"], t["gn_b"],
                     GN_EPS, buf.att_x)
    m["att_w_o"].matmul_op(buf.att_x, buf.att_o, ACT_NONE, fast)
    FusedV6.pre(C, A, cursors, buf.x, buf.att_o, buf.x2, t["ffn_ln_w"], t["ffn_ln_b"], LN_EPS, state, ffn_state, [t["ffn_time_mix_k"], t["ffn_time_mix_r"]],
                buf.ffn_x, [buf.ffn_kx, buf.ffn_rx])
    matmul_vec_group([(m["ffn_w_k"], buf.ffn_kx, buf.ffn_k, ACT_SQUARED_RELU, False, {}), (m["ffn_w_r"], buf.ffn_rx, buf.ffn_r, ACT_NONE, False, {})])
    m["ffn_w_v"].matmul_op_sparse(buf.ffn_k, buf.ffn_v, ACT_NONE, fast)
    FusedV6.post_ffn(C, A, cursors, state, ffn_state, buf.ffn_r, buf.ffn_v, buf.ffn_x, buf.x2, buf.x, rescale_now)


FUSED_MAX_TOKENS = 16  # measured: beyond this the op list's chunked kernels win (the fused ones walk tokens one by one)


def dispatch_layer_auto(layer, buf, state, cursors, A, H, S, rescale_now=False):
    """The fused form for short runs (decode and the tail of a schedule), the op list beyond."""
    if A <= FUSED_MAX_TOKENS and S == 64:
        dispatch_layer_fused(layer, buf, state, cursors, A, H, S, rescale_now)
    else:
        dispatch_layer(layer, buf, state, cursors, A, H, S, rescale_now)


def random_model_weights(rng, num_layer, C, H, S, hidden, vocab):
    """The tensors around the layers (src/runtime/v6.rs:110-135): embedding f16 [vocab, C] with its layer
    norm, the head's layer norm and the f16 head [vocab, C]."""
    h16 = lambda *s, std=0.02: (rng.standard_normal(s, dtype=np.float32) * np.float32(std)).astype(np.float16)
    return {
        "embed": h16(vocab, C, std=0.5), "embed_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "embed_ln_b": h16(C, std=0.1),
        "head_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "head_ln_b": h16(C, std=0.1), "head": h16(vocab, C),
        "layers": [random_layer_weights(rng, C, H, S, hidden, layer=i) for i in range(num_layer)],
    }


class Model:
    """A whole model on the device and one run of it (`Bundle::dispatch`, src/runtime/v6.rs:596-700):
    embedding rows of the run's tokens, their layer norm, the layers (halving the residual after every
    `rescale`-th one), then layer norm and head on the last token of the run's one request.  `dispatch`
    chooses how a layer runs: `dispatch_layer` (the op list), `dispatch_layer_fused` or `dispatch_layer_auto`."""

    def __init__(self, torch, weights, quant, H, S, hidden, slots, rescale=6, dispatch=dispatch_layer_auto):
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.torch, self.H, self.S, self.hidden, self.rescale, self.layer_fn = torch, H, S, hidden, rescale, dispatch
        self.C = H * S
        self.t = {k: dev(v) for k, v in weights.items() if k not in ("layers", "head")}
        self.head = Matrix.fp16(dev(weights["head"]))
        self.layers = [Layer(torch, w, quant) for w in weights["layers"]]
        self.state = [torch.zeros((slots, S + 2, self.C), dtype=torch.float32, device="cuda") for _ in self.layers]
        self.vocab = weights["head"].shape[0]

    def run(self, tokens, slot):
        """One run: `tokens` (up to 255) of the request in `slot`; returns the f32 logits after the last one."""
        torch, C, A = self.torch, self.C, len(tokens)
        buf = Runtime(torch, C, self.hidden, A)
        ids = torch.tensor([list(tokens)], dtype=torch.int32, device="cuda")
        cursors = torch.from_numpy(np.full(A, slot | (A << 24), dtype=np.uint32).view(np.int32)).cuda()
        inp = torch.zeros((1, A, C), dtype=torch.float16, device="cuda")
        head_x = torch.zeros((1, 1, C), dtype=torch.float16, device="cuda")
        logits = torch.zeros((1, 1, self.vocab), dtype=torch.float32, device="cuda")
        LayerOp.embed(ids, self.t["embed"], inp)
        LayerOp.layer_norm(self.t["embed_ln_w"], self.t["embed_ln_b"], inp, LN_EPS)
        LayerOp.blit(inp, buf.x)
        for i, (layer, st) in enumerate(zip(self.layers, self.state)):
            self.layer_fn(layer, buf, st, cursors, A, self.H, self.S, rescale_now=(i + 1) % self.rescale == 0)
        LayerOp.blit(buf.x, head_x, input_view=((C, 1, 1), (C, A, 1), (0, A - 1, 0)))
        LayerOp.layer_norm(self.t["head_ln_w"], self.t["head_ln_b"], head_x, LN_EPS)
        self.head.matmul_op(head_x, logits, ACT_NONE, turbo(1))
        return logits.view(-1)
