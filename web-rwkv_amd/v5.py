"""Host-side mirror of one RWKV-v5 layer as the reference dispatches it (src/runtime/v5.rs:651-890):
the same ops in the same order on the same buffers, every op one library call on torch's current
stream.  Weights are random-init tensors of the reference's shapes (src/runtime/v5.rs:60-105,
:945-1036); nothing here loads a checkpoint."""
import importlib

import numpy as np

_pkg = importlib.import_module(__name__.rsplit(".", 1)[0])
LayerOp, Matrix, turbo, matmul_vec_group = _pkg.LayerOp, _pkg.Matrix, _pkg.turbo, _pkg.matmul_vec_group
ACT_NONE, ACT_SQUARED_RELU, ACT_SILU = _pkg.ACT_NONE, _pkg.ACT_SQUARED_RELU, _pkg.ACT_SILU

LN_EPS = 1.0e-5   # Model::LN_EPS, src/runtime/v5.rs:45
GN_EPS = 64.0e-5  # Model::GN_EPS, src/runtime/v5.rs:46

QUANTIZED = ("att_w_k", "att_w_v", "att_w_r", "att_w_g", "att_w_o", "ffn_w_k", "ffn_w_v", "ffn_w_r")


def random_layer_weights(rng, C, H, S, hidden, layer=0):
    """numpy weights of one layer: matrices [out, in] f16 ~ N(0, 0.02) (att.output and ffn.value with the
    loader's 2^-(layer / 6) discount, src/runtime/loader.rs:660-661), vectors of plausible ranges;
    time_decay as the loader leaves it, exp(-exp(w)) (src/runtime/loader.rs:472-520)."""
    h16 = lambda *s, std=0.02: (rng.standard_normal(s, dtype=np.float32) * np.float32(std)).astype(np.float16)
    disc = np.float32(2.0 ** -(layer // 6))
    w = {
        "att_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "att_ln_b": h16(C, std=0.1),
        "ffn_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "ffn_ln_b": h16(C, std=0.1),
        "time_decay": np.exp(-np.exp((-1.0 + 0.5 * rng.standard_normal((H, S))).astype(np.float32))).astype(np.float32),
        "time_first": (0.3 * rng.standard_normal((H, S))).astype(np.float32),
        "gn_w": (1.0 + 0.1 * rng.standard_normal((H, S))).astype(np.float16), "gn_b": h16(H, S, std=0.1),
    }
    for name in ("time_mix_k", "time_mix_v", "time_mix_r", "time_mix_g", "ffn_time_mix_k", "ffn_time_mix_r"):
        w[name] = rng.random(C).astype(np.float16)
    for name, (R, K) in {"att_w_k": (C, C), "att_w_v": (C, C), "att_w_r": (C, C), "att_w_g": (C, C), "att_w_o": (C, C),
                         "ffn_w_k": (hidden, C), "ffn_w_v": (C, hidden), "ffn_w_r": (C, C)}.items():
        m = rng.standard_normal((R, K), dtype=np.float32) * np.float32(0.02)
        if name in ("att_w_o", "ffn_w_v"):
            m = m * disc
        w[name] = m.astype(np.float16)
    return w


class Layer:
    """Device weights of one layer: the eight matrices quantised (`quant`: "int8" or "nf4"), vectors
    as the reference keeps them."""

    def __init__(self, torch, weights, quant):
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.t = {k: dev(v) for k, v in weights.items() if k not in QUANTIZED}
        pack = Matrix.quant_u8 if quant == "int8" else Matrix.quant_nf4
        self.m = {k: pack(dev(weights[k])) for k in QUANTIZED}


class Runtime:
    """The buffers of a run of `A` tokens (`Runtime<F>`, src/runtime/v5.rs:258-313), F = f16."""

    def __init__(self, torch, C, hidden, A):
        z = lambda *s, dt=torch.float16: torch.zeros(s, dtype=dt, device="cuda")
        f32 = torch.float32
        self.x, self.att_x, self.att_kx, self.att_vx, self.att_rx, self.att_gx, self.att_g, self.att_o = (z(1, A, C) for _ in range(8))
        self.aux_x, self.att_k, self.att_v, self.att_r = (z(1, A, C, dt=f32) for _ in range(4))
        self.ffn_x, self.ffn_kx, self.ffn_rx, self.ffn_v, self.ffn_r = (z(1, A, C) for _ in range(5))
        self.ffn_k = z(1, A, hidden)


def dispatch_layer(layer, buf, state, cursors, A, H, S, rescale_now=False):
    """src/runtime/v5.rs:651-890.  `state`: this layer's f32 tensor (B, S + 2, C): rows 0..S the
    attention state (`State::att`, :175-179), row S + 1 the feed-forward one (`State::ffn`, :181-185)."""
    t, m, C = layer.t, layer.m, H * S
    B = state.shape[0]
    fast = turbo(A)
    att_state = ((C, S + 1, B), (C, S + 2, B), (0, 0, 0))
    ffn_state = ((C, 1, B), (C, S + 2, B), (0, S + 1, 0))
    heads = lambda x: x.view(A, H, S)

    LayerOp.blit(buf.x, buf.att_x)
    LayerOp.layer_norm(t["att_ln_w"], t["att_ln_b"], buf.att_x, LN_EPS)
    for name, out in (("time_mix_k", buf.att_kx), ("time_mix_v", buf.att_vx), ("time_mix_r", buf.att_rx), ("time_mix_g", buf.att_gx)):
        LayerOp.token_shift(cursors, t[name], state, buf.att_x, out, False, state_view=att_state)
    # the four independent projections in one call: the library's form of a `TensorOp::List` of them
    matmul_vec_group([(m["att_w_k"], buf.att_kx, buf.att_k, ACT_NONE, False, {}), (m["att_w_v"], buf.att_vx, buf.att_v, ACT_NONE, False, {}),
                      (m["att_w_r"], buf.att_rx, buf.att_r, ACT_NONE, False, {}), (m["att_w_g"], buf.att_gx, buf.att_g, ACT_NONE, False, {})])
    LayerOp.blit(buf.att_x, buf.aux_x)
    LayerOp.time_mix_v5(cursors, t["time_decay"], t["time_first"], state, heads(buf.att_k), heads(buf.att_v), heads(buf.att_r), heads(buf.aux_x),
                        state_view=att_state)
    LayerOp.group_norm(t["gn_w"], t["gn_b"], heads(buf.aux_x), GN_EPS)
    LayerOp.blit(buf.aux_x, buf.att_x)
    LayerOp.mul_activate(buf.att_g, buf.att_x, ACT_SILU, ACT_NONE, ACT_NONE)
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


class PackedShifts:
    """The four token-shift factors of a layer's attention half and the two of its feed-forward half, each
    stack repeated over the tokens of a run: `[C, A, 4]` and `[C, A, 2]` tensors made once per layer and run
    length with `TensorOp::broadcast`, so that one `token_shift` per half (the reference's form with a factor
    per token and output slice, src/tensor/ops.rs:1409-1414) replaces four and two launches."""

    def __init__(self, torch, layer, A):
        C = layer.t["time_mix_k"].numel()
        att = torch.stack([layer.t[n] for n in ("time_mix_k", "time_mix_v", "time_mix_r", "time_mix_g")]).view(4, 1, C)
        ffn = torch.stack([layer.t[n] for n in ("ffn_time_mix_k", "ffn_time_mix_r")]).view(2, 1, C)
        self.att, self.ffn = torch.empty((4, A, C), dtype=torch.float16, device="cuda"), torch.empty((2, A, C), dtype=torch.float16, device="cuda")
        LayerOp.broadcast(att, self.att)
        LayerOp.broadcast(ffn, self.ffn)
        self.att_sx, self.ffn_sx = torch.zeros_like(self.att), torch.zeros_like(self.ffn)


def dispatch_layer_packed(layer, shifts, buf, state, cursors, A, H, S, rescale_now=False):
    """`dispatch_layer` with the token shifts of each half in one launch (`shifts`: the layer's `PackedShifts`
    for this run length); the products read their slice of the shifted stack through views, as the v6 layer
    does.  Same results, bit for bit: 22 -> 18 launches per layer."""
    t, m, C = layer.t, layer.m, H * S
    B = state.shape[0]
    fast = turbo(A)
    att_state = ((C, S + 1, B), (C, S + 2, B), (0, 0, 0))
    ffn_state = ((C, 1, B), (C, S + 2, B), (0, S + 1, 0))
    heads = lambda x: x.view(A, H, S)
    slice_of = lambda i, n: dict(input_view=((C, A, 1), (C, A, n), (0, 0, i)))

    LayerOp.blit(buf.x, buf.att_x)
    LayerOp.layer_norm(t["att_ln_w"], t["att_ln_b"], buf.att_x, LN_EPS)
    LayerOp.token_shift(cursors, shifts.att, state, buf.att_x, shifts.att_sx, False, state_view=att_state)
    matmul_vec_group([(m[n], shifts.att_sx, out, ACT_NONE, False, slice_of(i, 4))
                      for i, (n, out) in enumerate((("att_w_k", buf.att_k), ("att_w_v", buf.att_v), ("att_w_r", buf.att_r), ("att_w_g", buf.att_g)))])
    LayerOp.blit(buf.att_x, buf.aux_x)
    LayerOp.time_mix_v5(cursors, t["time_decay"], t["time_first"], state, heads(buf.att_k), heads(buf.att_v), heads(buf.att_r), heads(buf.aux_x),
                        state_view=att_state)
    LayerOp.group_norm(t["gn_w"], t["gn_b"], heads(buf.aux_x), GN_EPS)
    LayerOp.blit(buf.aux_x, buf.att_x)
    LayerOp.mul_activate(buf.att_g, buf.att_x, ACT_SILU, ACT_NONE, ACT_NONE)
    m["att_w_o"].matmul_op(buf.att_x, buf.att_o, ACT_NONE, fast)
    LayerOp.add(buf.att_o, buf.x)

    LayerOp.blit(buf.x, buf.ffn_x)
    LayerOp.layer_norm(t["ffn_ln_w"], t["ffn_ln_b"], buf.ffn_x, LN_EPS)
    LayerOp.token_shift(cursors, shifts.ffn, state, buf.ffn_x, shifts.ffn_sx, False, state_view=ffn_state)
    matmul_vec_group([(m["ffn_w_k"], shifts.ffn_sx, buf.ffn_k, ACT_SQUARED_RELU, False, slice_of(0, 2)),
                      (m["ffn_w_r"], shifts.ffn_sx, buf.ffn_r, ACT_NONE, False, slice_of(1, 2))])
    m["ffn_w_v"].matmul_op_sparse(buf.ffn_k, buf.ffn_v, ACT_NONE, fast)
    LayerOp.channel_mix(cursors, state, buf.ffn_r, buf.ffn_v, buf.ffn_x, state_view=ffn_state)
    LayerOp.add(buf.ffn_x, buf.x)
    if rescale_now:
        LayerOp.affine(buf.x, 0.5, 0.0)


def random_model_weights(rng, num_layer, C, H, S, hidden, vocab):
    """The tensors around the layers (src/runtime/v5.rs:104-125): embedding f16 [vocab, C] with its layer
    norm, the head's layer norm and the f16 head [vocab, C]."""
    h16 = lambda *s, std=0.02: (rng.standard_normal(s, dtype=np.float32) * np.float32(std)).astype(np.float16)
    return {
        "embed": h16(vocab, C, std=0.5), "embed_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "embed_ln_b": h16(C, std=0.1),
        "head_ln_w": (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), "head_ln_b": h16(C, std=0.1), "head": h16(vocab, C),
        "layers": [random_layer_weights(rng, C, H, S, hidden, layer=i) for i in range(num_layer)],
    }


class Model:
    """A whole model on the device and one run of it (`Bundle::dispatch`, src/runtime/v5.rs:541-650):
    embedding rows of the run's tokens, their layer norm, the layers (halving the residual after every
    `rescale`-th one), then layer norm and head on the last token of the run's one request."""

    def __init__(self, torch, weights, quant, H, S, hidden, slots, rescale=6, packed_shifts=False):
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
        self.torch, self.H, self.S, self.hidden, self.rescale, self.packed = torch, H, S, hidden, rescale, packed_shifts
        self.C = H * S
        self.t = {k: dev(v) for k, v in weights.items() if k not in ("layers", "head")}
        self.head = Matrix.fp16(dev(weights["head"]))
        self.layers = [Layer(torch, w, quant) for w in weights["layers"]]
        self.state = [torch.zeros((slots, S + 2, self.C), dtype=torch.float32, device="cuda") for _ in self.layers]
        self.vocab = weights["head"].shape[0]
        self._buffers, self._shifts = {}, {}
        self.hook = None  # called as hook(layer index, run buffers) behind every layer, like a `Hook::PostFfn` of the reference (src/runtime/v5.rs:880-885)

    def buffers(self, A):
        """The buffers of runs of `A` tokens, made once per run length (`checkout_buffer`, src/runtime/v5.rs:497-510)."""
        if A not in self._buffers:
            torch, C = self.torch, self.C
            z = lambda *s, dt: torch.zeros(s, dtype=dt, device="cuda")
            self._buffers[A] = (Runtime(torch, C, self.hidden, A), z(1, A, dt=torch.int32), z(A, dt=torch.int32), z(1, A, C, dt=torch.float16),
                                z(1, 1, C, dt=torch.float16), z(1, 1, self.vocab, dt=torch.float32))
            if self.packed:
                self._shifts[A] = [PackedShifts(torch, layer, A) for layer in self.layers]
        return self._buffers[A]

    def dispatch(self, A):
        """The op list of one run of `A` tokens of one request on the buffers of that run length: nothing but
        library calls on the current stream (a HIP graph can record it)."""
        C = self.C
        buf, ids, cursors, inp, head_x, logits = self.buffers(A)
        LayerOp.embed(ids, self.t["embed"], inp)
        LayerOp.layer_norm(self.t["embed_ln_w"], self.t["embed_ln_b"], inp, LN_EPS)
        LayerOp.blit(inp, buf.x)
        for i, (layer, st) in enumerate(zip(self.layers, self.state)):
            if self.packed:
                dispatch_layer_packed(layer, self._shifts[A][i], buf, st, cursors, A, self.H, self.S, rescale_now=(i + 1) % self.rescale == 0)
            else:
                dispatch_layer(layer, buf, st, cursors, A, self.H, self.S, rescale_now=(i + 1) % self.rescale == 0)
            if self.hook is not None:
                self.hook(i, buf)
        LayerOp.blit(buf.x, head_x, input_view=((C, 1, 1), (C, A, 1), (0, A - 1, 0)))
        LayerOp.layer_norm(self.t["head_ln_w"], self.t["head_ln_b"], head_x, LN_EPS)
        self.head.matmul_op(head_x, logits, ACT_NONE, turbo(1))
        return logits.view(-1)

    def run(self, tokens, slot):
        """One run: `tokens` (up to 255) of the request in `slot`; returns the f32 logits after the last one."""
        torch, A = self.torch, len(tokens)
        _, ids, cursors, _, _, _ = self.buffers(A)
        ids.copy_(torch.tensor([list(tokens)], dtype=torch.int32))
        cursors.copy_(torch.from_numpy(np.full(A, slot | (A << 24), dtype=np.uint32).view(np.int32)))
        return self.dispatch(A)
