"""CPU restatement (numpy, f32) of the shaders of the ops between the matrix products.

TEST INFRASTRUCTURE ONLY: tests/ and nothing else import this; the library never does.

Each function follows its shader lane by lane: a workgroup of BLOCK_SIZE threads, each thread a
`vec4<f32>` lane group, strided over the row, then the shader's tree over the threads.
  softmax                 src/shaders/softmax.wgsl:52-110           (BLOCK_SIZE 128, ops.rs:301)
  layer_norm, group_norm  src/shaders/layer_norm.wgsl:27-120        (128 / 32, ops.rs:415, :468)
  add / mul + activations src/shaders/binary.wgsl:36-77, activations src/tensor/ops.rs:205-233
  token_shift, channel_mix(_v7), time_mix_v5 / v6 / v7, time_first_v7, l2_norm, control_k_v7: cited at each function
What pins them: the closed forms of the reference's own tests (softmax ops.rs:2655-2662, layer
norm ops.rs:2726-2746: sequential Welford) and float64 textbook forms, in tests/test_layer_ops.py.
Parity unpinned: group_norm's tree starts at a stride (64) beyond its 32 threads; the reads past
the workgroup arrays are taken to find zero counts (nothing merged), which only a run of the
reference could confirm.  f16 rounding of results: round to nearest even (numpy), as for the
matrix products.
"""
import numpy as np

F = np.float32


def _rows(x):
    """(..., C) array -> (rows, C) f32 copy."""
    a = np.asarray(x)
    return a.reshape(-1, a.shape[-1]).astype(F), a.shape, a.dtype


def _lanes(row, block):
    """Row of C elements -> [iterations, block, 4] vectors as thread `index` meets them
    (`for i = index; i < stride; i += BLOCK_SIZE`), and the validity of every slot."""
    nv = row.size // 4
    iters = (nv + block - 1) // block
    v = np.zeros((iters * block, 4), dtype=F)
    ok = np.zeros(iters * block, dtype=bool)
    v[:nv] = row.reshape(nv, 4)
    ok[:nv] = True
    return v.reshape(iters, block, 4), ok.reshape(iters, block)


def softmax(x, block=128):
    rows, shape, dt = _rows(x)
    out = np.empty_like(rows)
    for r, row in enumerate(rows):
        v, ok = _lanes(row, block)
        mx = np.full((block, 4), F(-1.0e30))
        for it in range(v.shape[0]):
            mx = np.where(ok[it][:, None], np.maximum(mx, v[it]), mx)
        s = 64
        while s >= 1:  # reduce_max(index, 64 .. 1)
            if s < block:
                mx[:s] = np.maximum(mx[:s], mx[s:2 * s])
            s //= 2
        m = F(max(mx[0]))
        sm = np.zeros((block, 4), dtype=F)
        for it in range(v.shape[0]):
            sm = np.where(ok[it][:, None], sm + np.exp(v[it] - m, dtype=F), sm)
        s = 64
        while s >= 1:
            if s < block:
                sm[:s] = sm[:s] + sm[s:2 * s]
            s //= 2
        total = F(((sm[0][0] + sm[0][1]) + sm[0][2]) + sm[0][3])  # dot(sketch[0], 1)
        out[r] = np.exp(row - m, dtype=F) / total
    return out.reshape(shape).astype(dt)


def layer_norm(w, b, x, eps, block=128, group=False):
    """x (..., C); w, b (C,) f16 -- or, group norm, x (A, H, S), w, b (H, S)."""
    rows, shape, dt = _rows(x)
    out = np.empty_like(rows)
    wf = np.asarray(w).astype(F).reshape(-1, rows.shape[1])
    bf = np.asarray(b).astype(F).reshape(-1, rows.shape[1])
    n = F(rows.shape[1])
    for r, row in enumerate(rows):
        v, ok = _lanes(row, block)
        mu = np.zeros((block, 4), dtype=F)
        m2 = np.zeros((block, 4), dtype=F)
        cnt = np.zeros((block, 4), dtype=np.uint32)
        for it in range(v.shape[0]):  # per-lane Welford
            k = ok[it][:, None]
            delta = v[it] - mu
            c1 = cnt + np.uint32(1)
            with np.errstate(divide="ignore", invalid="ignore"):
                mu1 = mu + delta / c1.astype(F)
            m21 = m2 + delta * (v[it] - mu1)
            cnt, mu, m2 = np.where(k, c1, cnt), np.where(k, mu1, mu), np.where(k, m21, m2)
        s = 64
        while s >= 1:  # reduce_step(index, 64 .. 1); strides beyond the workgroup merge nothing
            if s < block:
                mu1, mu2, c1, c2 = mu[:s], mu[s:2 * s], cnt[:s], cnt[s:2 * s]
                delta = mu2 - mu1
                tot = c1 + c2
                with np.errstate(divide="ignore", invalid="ignore"):
                    nm = (mu1 * c1.astype(F) + mu2 * c2.astype(F)) / tot.astype(F)
                    n2 = m2[:s] + m2[s:2 * s] + delta * delta * (c1 * c2).astype(F) / tot.astype(F)
                mu[:s] = np.where(tot > 0, nm, F(0))
                m2[:s] = np.where(tot > 0, n2, F(0))
                cnt[:s] = tot
            s //= 2
        c0 = cnt[0].astype(F)
        mean = F(np.dot(mu[0], c0 / n))
        d = mu[0] - mean
        var = F((F(m2[0].sum(dtype=F)) + F(np.dot(d * d, c0))) / n + F(eps))
        dev = F(1.0) / np.sqrt(var, dtype=F)
        h = r % wf.shape[0] if group else 0
        out[r] = ((row - mean) * dev) * wf[h] + bf[h]
    return out.reshape(shape).astype(dt)


def group_norm(w, b, x, eps):
    return layer_norm(w, b, x, eps, block=32, group=True)


def activation(act, x):
    """Activation::{None, SquaredRelu, Tanh, StableExp, OppositeExp, Softplus, Sigmoid, Silu} on f32."""
    x = np.asarray(x, dtype=F)
    with np.errstate(over="ignore"):
        if act == 0:
            return x
        if act == 1:
            p = np.maximum(x, F(0))
            return p * p
        if act == 2:
            return np.where(x > F(42), F(1), np.tanh(x, dtype=F))
        if act == 3:
            return np.exp(-np.exp(x, dtype=F), dtype=F)
        if act == 4:
            return -np.exp(x, dtype=F)
        if act == 5:
            return np.log(F(1) + np.exp(x, dtype=F), dtype=F)
        if act == 6:
            return F(1) / (F(1) + np.exp(-x, dtype=F))
        if act == 7:
            return x / (F(1) + np.exp(-x, dtype=F))
    raise ValueError(act)


def binary(op, x, y, act_x=0, act_y=0, act_out=0):
    """ACT_OUT(ACT_X(x) op ACT_Y(y)) with numpy broadcasting of x; result in y's type."""
    a, c = activation(act_x, np.asarray(x).astype(F)), activation(act_y, np.asarray(y).astype(F))
    r = activation(act_out, a * c if op == "mul" else a + c)
    return r.astype(np.asarray(y).dtype)


def view(a, shape, offset):
    """The slice a `View` names: numpy array (B, T, C) (last axis = x), reference-order shape / offset."""
    a = np.asarray(a)
    a = a.reshape((1,) * (3 - a.ndim) + a.shape) if a.ndim < 3 else a
    (c, t, b), (oc, ot, ob) = shape[:3], offset[:3]
    return a[ob:ob + b, ot:ot + t, oc:oc + c]


def blit(src, dst):
    """dst[...] = src converted to dst's type (src/shaders/blit.wgsl:35-53); both already sliced."""
    dst[...] = np.asarray(src).astype(F).astype(dst.dtype)


def transpose(src, dst):
    """input [C, T, B] -> output [C, B, T] (src/shaders/reshape.wgsl:58-77): numpy (B, T, C) -> (T, B, C)."""
    dst[...] = np.swapaxes(np.asarray(src), 0, 1).astype(F).astype(dst.dtype)


def affine(x, scale, bias):
    return (F(scale) * np.asarray(x).astype(F) + F(bias)).astype(np.asarray(x).dtype)


def lerp(x, y, f, reversed=False):
    """mix(x, y, f) = x (1 - f) + y f in f32, result in y's type (src/shaders/lerp.wgsl:82-93)."""
    a, c, t = np.asarray(x).astype(F), np.asarray(y).astype(F), np.asarray(f).astype(F)
    r = c * (F(1) - t) + a * t if reversed else a * (F(1) - t) + c * t
    return r.astype(np.asarray(y).dtype)


# ---- ops that carry state -----------------------------------------------------------------------
def pack_cursors(runs):
    """runs: list of (state slot, tokens of that request in the stack), in stack order ->
    u32 per token: slot | first token << 8 | count << 24 (compute_cursor, token_shift.wgsl:44-51)."""
    out, first = [], 0
    for slot, n in runs:
        out += [np.uint32(slot | (first << 8) | (n << 24))] * n
        first += n
    return np.array(out, dtype=np.uint32)


def _cursor(c):
    c = int(c)
    return c & 0xff, (c >> 8) & 0xffff, (c >> 24) & 0xff


def _mix(a, b, t):
    return a * (F(1) - t) + b * t


def token_shift(cursors, time_mix, state_row, x, out_dtype, counts=1, reversed=False):
    """src/shaders/token_shift.wgsl:91-116.  x (A, C); time_mix (counts, A, C), (counts, 1, C) or (C,);
    state_row (B, C) f32 = row 0 of the state view; result (counts, A, C)."""
    x32 = np.asarray(x).astype(F)
    A, C = x32.shape
    tm = np.asarray(time_mix).astype(F)
    tm = np.broadcast_to(tm.reshape((1, 1, C)) if tm.ndim == 1 else tm, (counts, A, C))
    out = np.empty((counts, A, C), dtype=F)
    for a in range(A):
        slot, first, _ = _cursor(cursors[a])
        prev = np.asarray(state_row)[slot].astype(F) if a == first else x32[a - 1]
        for c in range(counts):
            out[c, a] = _mix(x32[a], prev, tm[c, a]) if reversed else _mix(prev, x32[a], tm[c, a])
    return out.astype(out_dtype)


def channel_mix(cursors, state_row, r, v, x):
    """src/shaders/channel_mix.wgsl:83-106: state_row (B, C) f32 updated in place; returns the new x."""
    x = np.asarray(x)
    for a in range(x.shape[0]):
        slot, first, n = _cursor(cursors[a])
        if a - first + 1 == n:
            state_row[slot] = x[a].astype(F)
    rr = F(1) / (F(1) + np.exp(-np.asarray(r).astype(F), dtype=F))
    return (rr * np.asarray(v).astype(F)).astype(x.dtype)


def _fma(a, b, c):
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(F)


def time_mix_v6(cursors, time_decay, time_first, state, k, v, r, x):
    """src/shaders/time_mix_v6.wgsl:83-155.  k, v, r, x, time_decay (A, H, S); time_first (H, S);
    state (B, S + 1, H * S) f32 updated in place (row 0: x at a request's last token; row 1 + j:
    S[j][.]); the sum over j runs in the shader's order, one chain.  Returns the new x."""
    x = np.asarray(x)
    A, H, S = x.shape
    k32, v32, r32, w32, u32 = (np.asarray(t).astype(F) for t in (k, v, r, time_decay, time_first))
    out = np.empty((A, H, S), dtype=F)
    for t in range(A):
        slot, first, n = _cursor(cursors[t])
        if t - first + 1 == n:
            state[slot, 0] = x[first + n - 1].astype(F).reshape(-1)
        y = np.zeros((H, S), dtype=F)
        for j in range(S):
            ss = state[slot, 1 + j].reshape(H, S)
            kv = k32[t, :, j:j + 1] * v32[t]
            y = y + r32[t, :, j:j + 1] * _fma(np.broadcast_to(u32[:, j:j + 1], (H, S)), kv, ss)
            state[slot, 1 + j] = _fma(np.broadcast_to(w32[t, :, j:j + 1], (H, S)), ss, kv).reshape(-1)
        out[t] = y
    return out.astype(x.dtype)


def time_mix_v5(cursors, time_decay, time_first, state, k, v, r, x):
    """src/shaders/time_mix_v5.wgsl:86-155.  k, v, r, x (A, H, S); time_decay, time_first (H, S): the
    decay is a constant of the channel; state (B, S + 1, H * S) f32 updated in place (row 0: x at a
    request's last token; row 1 + j: S[j][.]); the sum over j in the shader's order.  Returns the new x."""
    x = np.asarray(x)
    A, H, S = x.shape
    k32, v32, r32, w32, u32 = (np.asarray(t).astype(F) for t in (k, v, r, time_decay, time_first))
    out = np.empty((A, H, S), dtype=F)
    for t in range(A):
        slot, first, n = _cursor(cursors[t])
        if t - first + 1 == n:
            state[slot, 0] = x[first + n - 1].astype(F).reshape(-1)
        y = np.zeros((H, S), dtype=F)
        for j in range(S):
            ss = state[slot, 1 + j].reshape(H, S)
            kv = k32[t, :, j:j + 1] * v32[t]
            y = y + r32[t, :, j:j + 1] * _fma(np.broadcast_to(u32[:, j:j + 1], (H, S)), kv, ss)
            state[slot, 1 + j] = _fma(np.broadcast_to(w32[:, j:j + 1], (H, S)), ss, kv).reshape(-1)
        out[t] = y
    return out.astype(x.dtype)


def l2_norm(x, eps, block=128):
    """src/shaders/normalize.wgsl:118-152: rows of the last axis; squares summed per lane vector over the
    row's stride, then the shader's tree over the threads; x / sqrt(sum + eps)."""
    rows, shape, dtype = _rows(x)
    out = np.empty_like(rows)
    for i, row in enumerate(rows):
        vec, valid = _lanes(row, block)
        acc = np.zeros((block, 4), dtype=F)
        for it in range(vec.shape[0]):
            acc = np.where(valid[it][:, None], acc + vec[it] * vec[it], acc)
        step = block >> 1
        while step:
            acc[:step] = acc[:step] + acc[step:2 * step]
            step >>= 1
        total = F(F(acc[0, 0] + acc[0, 1]) + acc[0, 2]) + acc[0, 3]
        out[i] = row * (F(1) / np.sqrt(F(total + F(eps)), dtype=F))
    return out.reshape(shape).astype(dtype)


def control_k_v7(p, a, k):
    """src/shaders/control_k_v7.wgsl:64-79: k (1 + (a - 1) p), p (C,) broadcast over tokens."""
    k = np.asarray(k)
    p32, a32, k32 = np.asarray(p).astype(F), np.asarray(a).astype(F), k.astype(F)
    return (k32 * (F(1) + (a32 - F(1)) * p32)).astype(k.dtype)


def time_mix_v7(cursors, state, r, w, n, x):
    """src/shaders/time_mix_v7.wgsl:137-212.  r, w, x (A, H, S); n (4, A, H, S) = k, v, a, kk; state
    (B, S + 1, H * S) f32 updated in place (row 0: x at a request's last token; row 1 + j: S[j][.]);
    both sums over j in the shader's order.  Returns the new x."""
    x = np.asarray(x)
    A, H, S = x.shape
    r32, w32, n32 = (np.asarray(t).astype(F) for t in (r, w, n))
    k32, v32, a32, kk32 = n32
    out = np.empty((A, H, S), dtype=F)
    for t in range(A):
        slot, first, cnt = _cursor(cursors[t])
        if t - first + 1 == cnt:
            state[slot, 0] = x[first + cnt - 1].astype(F).reshape(-1)
        ww = np.exp(F(-0.606531) * (F(1) / (F(1) + np.exp(-w32[t], dtype=F))), dtype=F)
        aa, bb = -kk32[t], kk32[t] * a32[t]
        sa = np.zeros((H, S), dtype=F)
        for j in range(S):
            sa = sa + state[slot, 1 + j].reshape(H, S) * aa[:, j:j + 1]
        y = np.zeros((H, S), dtype=F)
        for j in range(S):
            ss = state[slot, 1 + j].reshape(H, S)
            ss = ss * ww[:, j:j + 1] + k32[t, :, j:j + 1] * v32[t] + sa * bb[:, j:j + 1]
            y = y + r32[t, :, j:j + 1] * ss
            state[slot, 1 + j] = ss.reshape(-1)
        out[t] = y
    return out.astype(x.dtype)


def time_first_v7(u, r, n, x):
    """src/shaders/time_mix_v7.wgsl:214-255: x + (sum_j u[j] k[j] r[j]) v per head and token; the sum
    runs over 4-lane vectors with the shader's tree, then over the four lanes."""
    x = np.asarray(x)
    A, H, S = x.shape
    n32 = np.asarray(n).astype(F)
    prod = np.asarray(u).astype(F)[None] * n32[0] * np.asarray(r).astype(F)  # (A, H, S)
    vec = prod.reshape(A, H, S // 4, 4).copy()
    step = (S // 4) >> 1
    while step:
        vec[:, :, :step] = vec[:, :, :step] + vec[:, :, step:2 * step]
        step >>= 1
    xx = (vec[:, :, 0, 0] + vec[:, :, 0, 1]) + vec[:, :, 0, 2] + vec[:, :, 0, 3]
    return (x.astype(F) + xx[..., None] * n32[1]).astype(x.dtype)


def channel_mix_v7(cursors, state_row, v, x):
    """src/shaders/channel_mix.wgsl:83-106 with V7: state_row (B, C) f32 updated in place; returns v as the new x."""
    x = np.asarray(x)
    for a in range(x.shape[0]):
        slot, first, cnt = _cursor(cursors[a])
        if a - first + 1 == cnt:
            state_row[slot] = x[a].astype(F)
    return np.asarray(v).astype(x.dtype)


def time_mix_v4(cursors, time_decay, time_first, state, k, v, r, x):
    """src/shaders/time_mix_v4.wgsl:67-129.  k, v, r, x (A, C); time_decay, time_first (C,); state
    (B, 4, C) f32 updated in place (row 0: x at a request's last token; rows 1..3: aa, bb, pp).
    Returns the new x."""
    x = np.asarray(x)
    A = x.shape[0]
    k32, v32, r32 = (np.asarray(t).astype(F) for t in (k, v, r))
    u, w = np.asarray(time_first).astype(F), np.asarray(time_decay).astype(F)
    out = np.empty(x.shape, dtype=F)
    for t in range(A):
        slot, first, cnt = _cursor(cursors[t])
        aa, bb, pp = state[slot, 1].copy(), state[slot, 2].copy(), state[slot, 3].copy()
        if t - first + 1 == cnt:  # the shader stores this row at every token of the request, always from its last token
            state[slot, 0] = x[first + cnt - 1].astype(F)
        rr = F(1) / (F(1) + np.exp(-r32[t], dtype=F))
        ww = u + k32[t]
        q = np.maximum(pp, ww)
        e1, e2 = np.exp(pp - q, dtype=F), np.exp(ww - q, dtype=F)
        out[t] = rr * (e1 * aa + e2 * v32[t]) / (e1 * bb + e2)
        ww = w + pp
        q = np.maximum(ww, k32[t])
        e1, e2 = np.exp(ww - q, dtype=F), np.exp(k32[t] - q, dtype=F)
        state[slot, 1], state[slot, 2], state[slot, 3] = e1 * aa + e2 * v32[t], e1 * bb + e2, q
    return out.astype(x.dtype)


def _row_sum_tree(row, block, square):
    """the shaders' row sum: per-lane vectors strided over the row, the tree over the threads, the four lanes"""
    vec, valid = _lanes(row, block)
    acc = np.zeros((block, 4), dtype=F)
    for it in range(vec.shape[0]):
        acc = np.where(valid[it][:, None], acc + (vec[it] * vec[it] if square else vec[it]), acc)
    step = block >> 1
    while step:
        acc[:step] = acc[:step] + acc[step:2 * step]
        step >>= 1
    return F(F(acc[0, 0] + acc[0, 1]) + acc[0, 2]) + acc[0, 3]


def recenter(x, block=128):
    """src/shaders/normalize.wgsl:46-80: x - mean over the last axis."""
    rows, shape, dtype = _rows(x)
    out = np.empty_like(rows)
    for i, row in enumerate(rows):
        out[i] = row - F(_row_sum_tree(row, block, False) / F(row.size))
    return out.reshape(shape).astype(dtype)


def rms_norm(w, b, x, eps, block=128):
    """src/shaders/normalize.wgsl:82-116: fma(x / sqrt(mean(x^2) + eps), w, b)."""
    rows, shape, dtype = _rows(x)
    out = np.empty_like(rows)
    w32, b32 = np.asarray(w).astype(F), np.asarray(b).astype(F)
    for i, row in enumerate(rows):
        norm = F(1) / np.sqrt(F(_row_sum_tree(row, block, True) / F(row.size) + F(eps)), dtype=F)
        out[i] = _fma(row * norm, w32, b32)
    return out.reshape(shape).astype(dtype)


def broadcast(src, dst):
    """src/shaders/reshape.wgsl:35-56: dst (B, T, C) <- src (b, t, C) repeated along batches and tokens."""
    src = np.asarray(src)
    B, T, _ = dst.shape
    dst[...] = src[np.arange(B) % src.shape[0]][:, np.arange(T) % src.shape[1]].astype(F).astype(dst.dtype)


def blend(factor, x, y):
    """src/shaders/blend.wgsl:49-70: factor[0] x + factor[1] y in y's type."""
    f = np.asarray(factor, dtype=F)
    return (f[0] * np.asarray(x).astype(F) + f[1] * np.asarray(y).astype(F)).astype(np.asarray(y).dtype)


def blend_lora(factor, xa, xb, out):
    """src/shaders/blend_lora.wgsl:49-119: out (B, N, M) <- factor[0] xb xa^T + factor[1] out; xa (B, M, K), xb (B, N, K') f16,
    f32 sums over min(K, K') (in float64 here, rounded once: the shader's order of the 4 x 4 block sums is not followed)."""
    f = np.asarray(factor, dtype=F)
    xa, xb, out = np.asarray(xa), np.asarray(xb), np.asarray(out)
    K = min(xa.shape[-1], xb.shape[-1])
    prod = np.einsum("bnk,bmk->bnm", xb[..., :K].astype(np.float64), xa[..., :K].astype(np.float64)).astype(F)
    return (f[0] * prod + f[1] * out.astype(F)).astype(out.dtype)
