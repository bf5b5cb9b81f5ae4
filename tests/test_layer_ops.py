"""The ops between the matrix products: oracle against the closed forms of the reference's own
tests and float64, and -- marked gpu -- the library against the oracle through the C ABI."""
import importlib
import os
import sys

import numpy as np
import pytest

from helpers import assert_close

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SEED = 0x57525200


@pytest.fixture(scope="module")
def lop():
    sys.path.insert(0, ROOT)
    return importlib.import_module("oracle.layer_ops")


def softmax64(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def layer_norm64(w, b, x, eps):
    x = x.astype(np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * w.astype(np.float64) + b.astype(np.float64)


def layer_norm_reference_test_form(w, b, x, eps):
    """ops.rs:2726-2746: sequential f32 Welford over the row, then (x - mean) * deviation * w + b."""
    out = np.empty(x.shape, dtype=np.float32)
    for r, row in enumerate(x.reshape(-1, x.shape[-1]).astype(np.float32)):
        mean, m2 = np.float32(0), np.float32(0)
        for count, v in enumerate(row, start=1):
            delta = v - mean
            mean = np.float32(mean + delta / np.float32(count))
            m2 = np.float32(m2 + delta * (v - mean))
        dev = np.float32(1.0) / np.sqrt(np.float32(m2 / np.float32(row.size) + np.float32(eps)))
        out.reshape(-1, x.shape[-1])[r] = (row - mean) * dev * w.astype(np.float32) + b.astype(np.float32)
    return out


def reference_test_inputs(rng, C=1000, T=3, B=2):
    """the shapes and distributions of test_softmax / test_layer_norm (ops.rs:2636-2646, :2677-2697)"""
    x = (10.0 * (rng.random((B, T, C), dtype=np.float32) - 0.5)).astype(np.float32)
    w = (rng.random(C, dtype=np.float32) - 0.5).astype(np.float16)
    b = (rng.random(C, dtype=np.float32) - 0.5).astype(np.float16)
    return x, w, b


def test_oracle_softmax(lop):
    rng = np.random.default_rng(SEED + 1)
    x, _, _ = reference_test_inputs(rng)
    got = lop.softmax(x)
    assert_close(got, softmax64(x), 1e-6, "softmax vs float64")
    assert np.allclose(got.sum(axis=-1), 1.0, atol=1e-5)
    # invariances of the definition: a shift of the row changes nothing, a constant row is uniform
    assert_close(lop.softmax(x + np.float32(3.0)), got, 1e-5, "shift invariance")
    assert_close(lop.softmax(np.full((2, 64), 7.0, dtype=np.float32)), np.full((2, 64), 1 / 64), 1e-6, "constant row")
    h = lop.softmax(x.astype(np.float16))
    assert h.dtype == np.float16
    assert_close(h, softmax64(x.astype(np.float16)), 1e-3, "f16 rows")


@pytest.mark.parametrize("C", [1000, 4096, 64, 4])
def test_oracle_layer_norm(lop, C):
    rng = np.random.default_rng(SEED + 2 + C)
    x, w, b = reference_test_inputs(rng, C=C)
    got = lop.layer_norm(w, b, x, 1e-5)
    assert_close(got, layer_norm64(w, b, x, 1e-5), 1e-4, "vs float64")
    if C <= 1000:
        assert_close(got, layer_norm_reference_test_form(w, b, x, 1e-5), 1e-3, "vs the reference test's sequential form")  # its own bar
    # a dropped bias, a missing eps or the unbiased variance would show here
    one, zero = np.ones(C, dtype=np.float16), np.zeros(C, dtype=np.float16)
    y = lop.layer_norm(one, zero, x, 0.0).astype(np.float64)
    assert np.allclose(y.mean(axis=-1), 0.0, atol=1e-5) and np.allclose((y ** 2).mean(axis=-1), 1.0, atol=1e-4)
    big = lop.layer_norm(one, zero, np.full((1, C), 5.0, dtype=np.float32), 1e-5)
    assert np.all(big == 0.0)  # zero variance: eps keeps the division finite


def test_oracle_group_norm(lop):
    rng = np.random.default_rng(SEED + 3)
    A, H, S = 5, 8, 64
    x = (4.0 * rng.standard_normal((A, H, S))).astype(np.float32)
    w = rng.standard_normal((H, S)).astype(np.float16)
    b = rng.standard_normal((H, S)).astype(np.float16)
    got = lop.group_norm(w, b, x, 64e-5)
    assert_close(got, layer_norm64(w[None], b[None], x, 64e-5), 1e-4, "vs float64, per head")
    # heads must not share weights: permuting the heads of x, w and b together permutes the result
    p = rng.permutation(H)
    assert_close(lop.group_norm(w[p], b[p], x[:, p], 64e-5), got[:, p], 1e-6, "head permutation")


@pytest.mark.parametrize("op", ["add", "mul"])
def test_oracle_binary(lop, op):
    rng = np.random.default_rng(SEED + 4)
    x = rng.standard_normal((2, 3, 64)).astype(np.float16)
    y = rng.standard_normal((2, 3, 64)).astype(np.float32)
    f = (lambda a, c: a * c) if op == "mul" else (lambda a, c: a + c)
    assert_close(lop.binary(op, x, y), f(x.astype(np.float64), y.astype(np.float64)), 1e-6, "plain")
    # the gate of the attention output (v6.rs:881-887): silu(g) * x
    g = x.astype(np.float64)
    want = g / (1 + np.exp(-g)) * y if op == "mul" else g / (1 + np.exp(-g)) + y
    assert_close(lop.binary(op, x, y, act_x=7), want, 1e-6, "silu on the input")
    # broadcast of a [C, 1, 1] input, the closed forms of every activation at known points
    assert_close(lop.binary(op, x[0, 0], y), f(x[0, 0].astype(np.float64), y.astype(np.float64)), 1e-6, "broadcast")
    pts = np.array([-2.0, 0.0, 0.5, 50.0], dtype=np.float32)
    want = {1: [0, 0, 0.25, 2500], 2: [np.tanh(-2), 0, np.tanh(0.5), 1], 3: [np.exp(-np.exp(-2)), np.exp(-1), np.exp(-np.exp(0.5)), 0],
            4: [-np.exp(-2), -1, -np.exp(0.5), -np.exp(50)], 5: [np.log1p(np.exp(-2)), np.log(2), np.log1p(np.exp(0.5)), 50],
            6: [1 / (1 + np.exp(2)), 0.5, 1 / (1 + np.exp(-0.5)), 1], 7: [-2 / (1 + np.exp(2)), 0, 0.5 / (1 + np.exp(-0.5)), 50]}
    for act, w in want.items():
        assert_close(lop.activation(act, pts), np.array(w, dtype=np.float64), 1e-6, f"activation {act}")


def movement_kats():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "data_movement_kats.json")) as f:
        return json.load(f)


def test_oracle_data_movement_kats(lop):
    k = movement_kats()
    out = np.zeros(k["blit"]["output_shape"][::-1][1:], dtype=np.float32)  # (B, T, C)
    for op in k["blit"]["ops"]:
        src = np.array(op["input"], dtype=np.float32).reshape(op["input_shape"][::-1][1:])
        lop.blit(src, lop.view(out, op["view_shape"], op["view_offset"]))
    assert out.reshape(-1).tolist() == k["blit"]["expected"]
    t = k["transpose"]
    out = np.zeros(t["output_shape"][::-1][1:], dtype=np.float32)
    src = np.array(t["input"], dtype=np.float32).reshape(t["input_shape"][::-1][1:])
    lop.transpose(src, lop.view(out, t["view_shape"], t["view_offset"]))
    assert out.reshape(-1).tolist() == t["expected"]


def test_oracle_lerp_affine(lop):
    rng = np.random.default_rng(SEED + 5)
    x = (rng.random((2, 3, 1000), dtype=np.float32) - 0.5).astype(np.float32)
    y = (rng.random((2, 3, 1000), dtype=np.float32) - 0.5).astype(np.float32)
    f = rng.random((2, 3, 1000), dtype=np.float32)
    want = x.astype(np.float64) * (1 - f.astype(np.float64)) + y.astype(np.float64) * f  # ops.rs:3286-3290
    assert_close(lop.lerp(x, y, f), want, 1e-6, "lerp")
    assert_close(lop.lerp(x, y, f, reversed=True), y.astype(np.float64) * (1 - f.astype(np.float64)) + x.astype(np.float64) * f, 1e-6, "reversed")
    assert np.array_equal(lop.lerp(x, y, np.zeros_like(f)), x) and np.array_equal(lop.lerp(x, y, np.ones_like(f)), y)
    assert_close(lop.affine(x, 0.5, 0.0), x / 2, 0.0, "affine halves exactly")  # the rescale of v6.rs:953-955


RUNS = [(2, 3), (0, 1), (5, 4)]  # (state slot, tokens in the stack): three requests, 8 tokens


def test_oracle_token_shift_channel_mix(lop):
    rng = np.random.default_rng(SEED + 6)
    C, B = 64, 6
    cur = lop.pack_cursors(RUNS)
    A = len(cur)
    x = rng.standard_normal((A, C)).astype(np.float16)
    state = rng.standard_normal((B, C)).astype(np.float32)
    tm = rng.random(C).astype(np.float16)
    got = lop.token_shift(cur, tm, state, x, np.float32, reversed=True)
    # by hand: the token before a request's first token is its state row, else the token before in the stack
    prev = np.stack([state[2], x[0], x[1], state[0], state[5], x[4], x[5], x[6]]).astype(np.float64)
    f = tm.astype(np.float64)
    assert_close(got[0], x.astype(np.float64) * (1 - f) + prev * f, 1e-6, "reversed: mix(x, prev, f)")
    assert_close(lop.token_shift(cur, tm, state, x, np.float32)[0], prev * (1 - f) + x.astype(np.float64) * f, 1e-6, "mix(prev, x, f)")
    # per token and per count factors (the five data-dependent shifts of v6.rs:796-805)
    tm5 = rng.random((5, A, C)).astype(np.float32)
    got5 = lop.token_shift(cur, tm5, state, x, np.float16, counts=5, reversed=True)
    assert got5.shape == (5, A, C) and got5.dtype == np.float16
    assert_close(got5[3], x.astype(np.float64) * (1 - tm5[3]) + prev * tm5[3], 1e-3, "count 3")
    # channel mix: the state takes x at every request's last token, x becomes sigmoid(r) v
    r = rng.standard_normal((A, C)).astype(np.float16)
    v = rng.standard_normal((A, C)).astype(np.float16)
    st = state.copy()
    out = lop.channel_mix(cur, st, r, v, x)
    assert np.array_equal(st[2], x[2].astype(np.float32)) and np.array_equal(st[0], x[3].astype(np.float32)) and np.array_equal(st[5], x[7].astype(np.float32))
    assert np.array_equal(st[[1, 3, 4]], state[[1, 3, 4]])
    assert_close(out, v.astype(np.float64) / (1 + np.exp(-r.astype(np.float64))), 1e-3, "sigmoid(r) v")


def wkv6_float64(cursors, w, u, state, k, v, r, x):
    """textbook form of the recurrence per request and head, in float64, one token at a time:
    y = r^T (diag(u) k v^T + S),  S <- diag(w) S + k v^T"""
    A, H, S = x.shape
    st = state.astype(np.float64).copy()
    out = np.zeros((A, H, S))
    for t in range(A):
        c = int(cursors[t])
        slot, first, n = c & 0xff, (c >> 8) & 0xffff, (c >> 24) & 0xff
        if t - first + 1 == n:
            st[slot, 0] = x[t].astype(np.float64).reshape(-1)
        for h in range(H):
            Sm = st[slot, 1:, h * S:(h + 1) * S]  # [j, i]
            kv = np.outer(k[t, h].astype(np.float64), v[t, h].astype(np.float64))
            out[t, h] = r[t, h].astype(np.float64) @ (u[h].astype(np.float64)[:, None] * kv + Sm)
            st[slot, 1:, h * S:(h + 1) * S] = w[t, h].astype(np.float64)[:, None] * Sm + kv
    return out, st


def wkv6_inputs(rng, A, H, S, B, dtype):
    k = (0.5 * rng.standard_normal((A, H, S))).astype(dtype)
    v = (0.5 * rng.standard_normal((A, H, S))).astype(dtype)
    r = (0.5 * rng.standard_normal((A, H, S))).astype(dtype)
    x = rng.standard_normal((A, H, S)).astype(dtype)
    w = np.exp(-np.exp(rng.standard_normal((A, H, S)).astype(np.float32))).astype(np.float32)  # the decay after StableExp
    u = (0.3 * rng.standard_normal((H, S))).astype(np.float32)
    state = (0.1 * rng.standard_normal((B, S + 1, H * S))).astype(np.float32)
    return k, v, r, x, w, u, state


def test_oracle_time_mix_v6(lop):
    rng = np.random.default_rng(SEED + 7)
    H, S, B = 3, 16, 6
    cur = lop.pack_cursors(RUNS)
    k, v, r, x, w, u, state = wkv6_inputs(rng, len(cur), H, S, B, np.float32)
    st = state.copy()
    got = lop.time_mix_v6(cur, w, u, st, k, v, r, x)
    want, want_state = wkv6_float64(cur, w, u, state, k, v, r, x)
    assert_close(got, want, 1e-5, "y vs float64")
    assert_close(st, want_state, 1e-5, "state vs float64")
    assert np.array_equal(st[[1, 3, 4]], state[[1, 3, 4]])  # requests that are not in the stack keep their state
    # one token, zero state: y = (r . (u k)) v exactly as a closed form; the state becomes k v^T
    z = np.zeros_like(state)
    one = lop.pack_cursors([(1, 1)])
    y1 = lop.time_mix_v6(one, w[:1], u, z, k[:1], v[:1], r[:1], x[:1])
    assert_close(y1[0], (r[0] * u * k[0]).sum(axis=-1, keepdims=True).astype(np.float64) * v[0], 1e-5, "first token")
    assert_close(z[1, 1:, :S], np.outer(k[0, 0], v[0, 0]), 1e-6, "state after the first token")
    # a run of 2 tokens equals two runs of 1 token (the state carries everything)
    s_a, s_b = state.copy(), state.copy()
    two = lop.time_mix_v6(lop.pack_cursors([(4, 2)]), w[:2], u, s_a, k[:2], v[:2], r[:2], x[:2])
    first = lop.time_mix_v6(lop.pack_cursors([(4, 1)]), w[:1], u, s_b, k[:1], v[:1], r[:1], x[:1])
    second = lop.time_mix_v6(lop.pack_cursors([(4, 1)]), w[1:2], u, s_b, k[1:2], v[1:2], r[1:2], x[1:2])
    assert np.array_equal(two, np.concatenate([first, second])) and np.array_equal(s_a, s_b)


# ---------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_gpu_token_shift_channel_mix(gpu, lop, dtype):
    import torch

    print("token shift / channel mix on the GPU", dtype.__name__, flush=True)
    rng = np.random.default_rng(SEED + 50)
    C, B, L = 256, 6, 3
    cur = lop.pack_cursors(RUNS)
    A = len(cur)
    curd = torch.from_numpy(cur.view(np.int32)).cuda()
    x = rng.standard_normal((A, C)).astype(dtype)
    # the state of a model: [C, rows per layer * layers, B]; this layer's row is picked by the view
    rows = 2 * L
    state = rng.standard_normal((B, rows, C)).astype(np.float32)
    row = 3
    sview = ((C, 1, B), (C, rows, B), (0, row, 0))
    sd = torch.from_numpy(state.copy()).cuda()
    xd = torch.from_numpy(x).cuda()
    tm = rng.random((1, 1, C)).astype(np.float16)
    for rev in (True, False):
        for ot in (np.float16, np.float32):
            out = torch.empty((1, A, C), dtype=torch.float16 if ot == np.float16 else torch.float32, device="cuda")
            gpu.LayerOp.token_shift(curd, torch.from_numpy(tm).cuda(), sd, xd.reshape(1, A, C), out, rev, state_view=sview)
            want = lop.token_shift(cur, tm.reshape(C), state[:, row], x, ot, reversed=rev)
            assert_close(out.cpu().numpy(), want, 1e-3 if ot == np.float16 else 1e-6, f"token shift {rev} {ot.__name__}")
    tm5 = rng.random((5, A, C)).astype(np.float32)
    out5 = torch.empty((5, A, C), dtype=torch.float16, device="cuda")
    gpu.LayerOp.token_shift(curd, torch.from_numpy(tm5).cuda(), sd, xd.reshape(1, A, C), out5, True, state_view=sview)
    assert_close(out5.cpu().numpy(), lop.token_shift(cur, tm5, state[:, row], x, np.float16, counts=5, reversed=True), 1e-3, "five shifts")
    r = rng.standard_normal((A, C)).astype(dtype)
    v = rng.standard_normal((A, C)).astype(dtype)
    st = state[:, row].copy()
    want = lop.channel_mix(cur, st, r, v, x)
    xm = torch.from_numpy(x.copy()).cuda().reshape(1, A, C)
    gpu.LayerOp.channel_mix(curd, sd, torch.from_numpy(r).cuda().reshape(1, A, C), torch.from_numpy(v).cuda().reshape(1, A, C), xm, state_view=sview)
    assert_close(xm.cpu().numpy()[0], want, 1e-3 if dtype == np.float16 else 1e-6, "channel mix")
    want_state = state.copy()
    want_state[:, row] = st
    assert np.array_equal(sd.cpu().numpy(), want_state)  # only this layer's row of the requests in the stack changed


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("H,S,runs", [(3, 16, RUNS), (4, 64, RUNS), (64, 64, [(0, 1)]), (2, 128, [(1, 2), (3, 2)]), (8, 64, [(b, 1) for b in range(6)]), (2, 64, [(4, 100)])])
def test_gpu_time_mix_v6(gpu, lop, dtype, H, S, runs):
    import torch

    print("time mix v6 on the GPU", dtype.__name__, H, S, runs[:3], flush=True)
    rng = np.random.default_rng(SEED + 60 + H + S)
    B = 6
    cur = lop.pack_cursors(runs)
    A = len(cur)
    k, v, r, x, w, u, state = wkv6_inputs(rng, A, H, S, B, dtype)
    # the model's state tensor holds S + 1 rows per layer; layer 1 of 2 is used here
    full = np.concatenate([np.zeros_like(state), state], axis=1)
    sview = ((H * S, S + 1, B), (H * S, 2 * (S + 1), B), (0, S + 1, 0))
    sd = torch.from_numpy(full.copy()).cuda()
    xd = torch.from_numpy(x.copy()).cuda()
    gpu.LayerOp.time_mix_v6(torch.from_numpy(cur.view(np.int32)).cuda(), torch.from_numpy(w).cuda(), torch.from_numpy(u).cuda(), sd,
                            torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), torch.from_numpy(r).cuda(), xd, state_view=sview)
    want, want_state = wkv6_float64(cur, w, u, state, k, v, r, x)
    eps = 2e-3 if dtype == np.float16 else 2e-5
    assert_close(xd.cpu().numpy(), want, eps, "y vs float64")
    got_state = sd.cpu().numpy()
    assert_close(got_state[:, S + 1:], want_state, 2e-5, "state vs float64")
    assert np.array_equal(got_state[:, :S + 1], full[:, :S + 1])  # the other layer's rows are untouched
    if A * H * S * S <= 2000000:
        st = state.copy()
        assert_close(xd.cpu().numpy(), lop.time_mix_v6(cur, w, u, st, k, v, r, x), eps, "y vs oracle")
        assert_close(got_state[:, S + 1:], st, 2e-5, "state vs oracle")


# ---------------------------------------------------------------------------------------------
def test_oracle_time_mix_v5(lop):
    # v5 is the recurrence with one decay per channel (src/shaders/time_mix_v5.wgsl:120-152): the
    # float64 textbook form with that decay repeated for every token, and bit equality with the v6
    # restatement on the repeated decay (the shaders differ only in where w comes from)
    rng = np.random.default_rng(SEED + 8)
    H, S, B = 3, 16, 6
    cur = lop.pack_cursors(RUNS)
    A = len(cur)
    k, v, r, x, w, u, state = wkv6_inputs(rng, A, H, S, B, np.float32)
    w5 = w[0]
    wrep = np.broadcast_to(w5, (A, H, S))
    st = state.copy()
    got = lop.time_mix_v5(cur, w5, u, st, k, v, r, x)
    want, want_state = wkv6_float64(cur, wrep, u, state, k, v, r, x)
    assert_close(got, want, 1e-5, "y vs float64")
    assert_close(st, want_state, 1e-5, "state vs float64")
    st6 = state.copy()
    assert np.array_equal(got, lop.time_mix_v6(cur, wrep, u, st6, k, v, r, x)) and np.array_equal(st, st6)
    # n tokens of one request from a zero state with r = 1, u = 0: y_t[i] = sum_j sum_{s<t} w_j^(t-1-s) k_s[j] v_s[i]
    n = 5
    z = np.zeros_like(state)
    ones = np.ones((n, H, S), dtype=np.float32)
    y = lop.time_mix_v5(lop.pack_cursors([(2, n)]), w5, np.zeros_like(u), z, k[:n], v[:n], ones, x[:n])
    w64, k64, v64 = w5.astype(np.float64), k[:n].astype(np.float64), v[:n].astype(np.float64)
    for t in range(n):
        closed = sum(((w64 ** (t - 1 - s)) * k64[s]).sum(axis=-1, keepdims=True) * v64[s] for s in range(t)) if t else np.zeros((H, S))
        assert_close(y[t], closed, 1e-5, f"geometric closed form, token {t}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("H,S,runs", [(3, 16, RUNS), (12, 64, RUNS), (12, 64, [(0, 1)]), (2, 128, [(1, 2), (3, 2)]), (2, 64, [(4, 100)])])
def test_gpu_time_mix_v5(gpu, lop, dtype, H, S, runs):
    import torch

    print("time mix v5 on the GPU", dtype.__name__, H, S, runs[:3], flush=True)
    rng = np.random.default_rng(SEED + 80 + H + S)
    B = 6
    cur = lop.pack_cursors(runs)
    A = len(cur)
    k, v, r, x, w, u, state = wkv6_inputs(rng, A, H, S, B, dtype)
    w5 = np.ascontiguousarray(w[0])
    full = np.concatenate([np.zeros_like(state), state], axis=1)
    sview = ((H * S, S + 1, B), (H * S, 2 * (S + 1), B), (0, S + 1, 0))
    sd = torch.from_numpy(full.copy()).cuda()
    xd = torch.from_numpy(x.copy()).cuda()
    gpu.LayerOp.time_mix_v5(torch.from_numpy(cur.view(np.int32)).cuda(), torch.from_numpy(w5).cuda(), torch.from_numpy(u).cuda(), sd,
                            torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), torch.from_numpy(r).cuda(), xd, state_view=sview)
    want, want_state = wkv6_float64(cur, np.broadcast_to(w5, (A, H, S)), u, state, k, v, r, x)
    eps = 2e-3 if dtype == np.float16 else 2e-5
    assert_close(xd.cpu().numpy(), want, eps, "y vs float64")
    got_state = sd.cpu().numpy()
    assert_close(got_state[:, S + 1:], want_state, 2e-5, "state vs float64")
    assert np.array_equal(got_state[:, :S + 1], full[:, :S + 1])  # the other layer's rows are untouched
    if A * H * S * S <= 2000000:
        st = state.copy()
        assert_close(xd.cpu().numpy(), lop.time_mix_v5(cur, w5, u, st, k, v, r, x), eps, "y vs oracle")
        assert_close(got_state[:, S + 1:], st, 2e-5, "state vs oracle")
    # a per-token decay tensor is the v6 op's operand, not this one's
    if A > 1:
        with pytest.raises(gpu.TensorError):
            gpu.LayerOp.time_mix_v5(torch.from_numpy(cur.view(np.int32)).cuda(), torch.from_numpy(w).cuda(), torch.from_numpy(u).cuda(), sd,
                                    torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), torch.from_numpy(r).cuda(), xd, state_view=sview)


# ---------------------------------------------------------------------------------------------
def wkv4_float64(cursors, w, u, state, k, v, r, x):
    """the v4 recurrence without the exponent shift, in float64 (inputs small enough not to overflow):
    a <- e^w a + e^k v, b <- e^w b + e^k, y = sigmoid(r) (a + e^(u+k) v) / (b + e^(u+k)); a = aa e^pp, b = bb e^pp.
    Returns y, the true (a, b) of every request, and row 0."""
    f = np.float64
    A, C = x.shape
    a = state[:, 1].astype(f) * np.exp(state[:, 3].astype(f))
    b = state[:, 2].astype(f) * np.exp(state[:, 3].astype(f))
    row0 = state[:, 0].astype(f).copy()
    out = np.zeros((A, C))
    for t in range(A):
        c = int(cursors[t])
        slot, first, cnt = c & 0xff, (c >> 8) & 0xffff, (c >> 24) & 0xff
        if t - first + 1 == cnt:
            row0[slot] = x[t].astype(f)
        ek, eu = np.exp(k[t].astype(f)), np.exp(u.astype(f) + k[t].astype(f))
        out[t] = (a[slot] + eu * v[t].astype(f)) / (b[slot] + eu) / (1 + np.exp(-r[t].astype(f)))
        a[slot] = np.exp(w.astype(f)) * a[slot] + ek * v[t].astype(f)
        b[slot] = np.exp(w.astype(f)) * b[slot] + ek
    return out, a, b, row0


def wkv4_inputs(rng, A, C, B, dtype):
    k, v, r, x = (rng.standard_normal((A, C)).astype(dtype) for _ in range(4))
    w = -np.exp(rng.standard_normal(C).astype(np.float32))  # the decay as the loader leaves it: -exp(time_decay)
    u = (0.3 * rng.standard_normal(C)).astype(np.float32)
    state = rng.standard_normal((B, 4, C)).astype(np.float32)
    state[:, 2] = np.abs(state[:, 2]) + 0.5  # a denominator
    state[3] = [[0] * C, [0] * C, [0] * C, [-1e30] * C]  # a fresh request: nothing seen yet
    return k, v, r, x, w, u, state


def check_wkv4_state(got, want_a, want_b, eps):
    f = np.float64
    assert_close(got[:, 1].astype(f) * np.exp(got[:, 3].astype(f)), want_a, eps, "numerator vs float64")
    assert_close(got[:, 2].astype(f) * np.exp(got[:, 3].astype(f)), want_b, eps, "denominator vs float64")


def test_oracle_time_mix_v4(lop):
    rng = np.random.default_rng(SEED + 10)
    C, B = 64, 6
    runs = [(2, 3), (3, 2), (5, 4)]  # slot 3 starts fresh
    cur = lop.pack_cursors(runs)
    k, v, r, x, w, u, state = wkv4_inputs(rng, len(cur), C, B, np.float32)
    st = state.copy()
    got = lop.time_mix_v4(cur, w, u, st, k, v, r, x)
    want, a, b, row0 = wkv4_float64(cur, w, u, state, k, v, r, x)
    assert_close(got, want, 1e-5, "y vs float64")
    check_wkv4_state(st, a, b, 1e-5)
    assert_close(st[:, 0], row0, 0, "row 0")
    assert np.array_equal(st[[0, 1, 4]], state[[0, 1, 4]])
    # the first token of a fresh request returns sigmoid(r) v: the average of one value
    assert_close(got[3], v[3] / (1 + np.exp(-r[3].astype(np.float64))), 1e-6, "fresh request")
    # a run of 2 tokens equals two runs of 1 token
    s_a, s_b = state.copy(), state.copy()
    two = lop.time_mix_v4(lop.pack_cursors([(4, 2)]), w, u, s_a, k[:2], v[:2], r[:2], x[:2])
    first = lop.time_mix_v4(lop.pack_cursors([(4, 1)]), w, u, s_b, k[:1], v[:1], r[:1], x[:1])
    second = lop.time_mix_v4(lop.pack_cursors([(4, 1)]), w, u, s_b, k[1:2], v[1:2], r[1:2], x[1:2])
    assert np.array_equal(two, np.concatenate([first, second])) and np.array_equal(s_a[:, 1:], s_b[:, 1:])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("C,runs", [(64, [(2, 3), (3, 2), (5, 4)]), (768, [(3, 1)]), (1000, [(3, 40), (1, 2)])])
def test_gpu_time_mix_v4(gpu, lop, dtype, C, runs):
    import torch

    print("time mix v4 on the GPU", dtype.__name__, C, runs, flush=True)
    rng = np.random.default_rng(SEED + 70 + C)
    B = 6
    cur = lop.pack_cursors(runs)
    A = len(cur)
    k, v, r, x, w, u, state = wkv4_inputs(rng, A, C, B, dtype)
    # the model's state holds 5 rows per layer (4 attention rows, 1 feed-forward row); the view picks the first 4
    full = np.concatenate([state, np.full((B, 1, C), 7.0, dtype=np.float32)], axis=1)
    sview = ((C, 4, B), (C, 5, B), (0, 0, 0))
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    sd, xd = dev(full), dev(x.reshape(1, A, C))
    gpu.LayerOp.time_mix_v4(dev(cur.view(np.int32)), dev(w), dev(u), sd, dev(k.reshape(1, A, C)), dev(v.reshape(1, A, C)), dev(r.reshape(1, A, C)), xd, state_view=sview)
    want, a, b, row0 = wkv4_float64(cur, w, u, state, k, v, r, x)
    eps = 2e-3 if dtype == np.float16 else 2e-5
    assert_close(xd.cpu().numpy()[0], want, eps, "y vs float64")
    got_state = sd.cpu().numpy()
    check_wkv4_state(got_state[:, :4], a, b, 5e-5)
    assert_close(got_state[:, 0], row0, 0, "row 0")
    assert np.array_equal(got_state[:, 4], full[:, 4])  # the feed-forward row is untouched
    st = state.copy()
    assert_close(xd.cpu().numpy()[0], lop.time_mix_v4(cur, w, u, st, k, v, r, x), eps, "y vs oracle")
    assert_close(got_state[:, 1:4], st[:, 1:], 5e-5, "state vs oracle")


# ---------------------------------------------------------------------------------------------
# the ops an RWKV-v7 layer adds.  The reference has no test of them: the restatements are pinned by
# float64 textbook forms, closed forms of special cases and invariants only (parity unpinned).
def wkv7_float64(cursors, state, r, w, n, x):
    """per request and head in float64, matrices indexed [j, i]:  sa = S^T a,  S <- diag(w) S + k v^T + b sa^T,  y = S^T r
    with a = -kk, b = kk * a_in, w = exp(-exp(-1/2) sigmoid(w_in))"""
    A, H, S = x.shape
    f = np.float64
    st = state.astype(f).copy()
    out = np.zeros((A, H, S))
    k, v, a_in, kk = (t.astype(f) for t in n)
    for t in range(A):
        c = int(cursors[t])
        slot, first, cnt = c & 0xff, (c >> 8) & 0xffff, (c >> 24) & 0xff
        if t - first + 1 == cnt:
            st[slot, 0] = x[t].astype(f).reshape(-1)
        for h in range(H):
            Sm = st[slot, 1:, h * S:(h + 1) * S]
            ww = np.exp(-np.exp(-0.5) / (1.0 + np.exp(-w[t, h].astype(f))))
            sa = Sm.T @ (-kk[t, h])
            Sn = ww[:, None] * Sm + np.outer(k[t, h], v[t, h]) + np.outer(kk[t, h] * a_in[t, h], sa)
            out[t, h] = Sn.T @ r[t, h].astype(f)
            st[slot, 1:, h * S:(h + 1) * S] = Sn
    return out, st


def wkv7_inputs(rng, A, H, S, B, dtype):
    r = (0.5 * rng.standard_normal((A, H, S))).astype(dtype)
    w = rng.standard_normal((A, H, S)).astype(dtype)
    k = (0.5 * rng.standard_normal((A, H, S))).astype(dtype)
    v = (0.5 * rng.standard_normal((A, H, S))).astype(dtype)
    a = rng.random((A, H, S)).astype(dtype)  # a sigmoid's output
    kk = rng.standard_normal((A, H, S))
    kk = (kk / np.sqrt((kk * kk).sum(axis=-1, keepdims=True))).astype(dtype)  # rows of unit length, as after l2_norm
    x = rng.standard_normal((A, H, S)).astype(dtype)
    state = (0.1 * rng.standard_normal((B, S + 1, H * S))).astype(np.float32)
    return r, w, np.stack([k, v, a, kk]), x, state


def test_oracle_v7_ops(lop):
    rng = np.random.default_rng(SEED + 9)
    H, S, B = 3, 16, 6
    cur = lop.pack_cursors(RUNS)
    A = len(cur)
    r, w, n, x, state = wkv7_inputs(rng, A, H, S, B, np.float32)
    st = state.copy()
    got = lop.time_mix_v7(cur, st, r, w, n, x)
    want, want_state = wkv7_float64(cur, state, r, w, n, x)
    assert_close(got, want, 1e-5, "y vs float64")
    assert_close(st, want_state, 1e-5, "state vs float64")
    assert np.array_equal(st[[1, 3, 4]], state[[1, 3, 4]])
    # one token from a zero state: S = k v^T, so y = (r . k) v whatever a and kk are
    z = np.zeros_like(state)
    y1 = lop.time_mix_v7(lop.pack_cursors([(1, 1)]), z, r[:1], w[:1], n[:, :1], x[:1])
    assert_close(y1[0], (r[0] * n[0, 0]).sum(axis=-1, keepdims=True).astype(np.float64) * n[1, 0], 1e-5, "first token")
    # kk = 0 switches the correction off: tokens of one request from a zero state give
    # y_t = sum_{s <= t} (r_t . (prod_{s < q <= t} w_q) k_s) v_s
    n0 = n.copy()
    n0[3] = 0
    z = np.zeros_like(state)
    y = lop.time_mix_v7(lop.pack_cursors([(2, 4)]), z, r[:4], w[:4], n0[:, :4], x[:4])
    wd = np.exp(-np.exp(-0.5) / (1.0 + np.exp(-w[:4].astype(np.float64))))
    for t in range(4):
        closed = np.zeros((H, S))
        for s_ in range(t + 1):
            decay = np.prod(wd[s_ + 1:t + 1], axis=0) if s_ < t else np.ones((H, S))
            closed += (r[t] * decay * n[0, s_]).sum(axis=-1, keepdims=True) * n[1, s_]
        assert_close(y[t], closed, 1e-5, f"decay-only closed form, token {t}")
    # a run of 2 tokens equals two runs of 1 token
    s_a, s_b = state.copy(), state.copy()
    two = lop.time_mix_v7(lop.pack_cursors([(4, 2)]), s_a, r[:2], w[:2], n[:, :2], x[:2])
    first = lop.time_mix_v7(lop.pack_cursors([(4, 1)]), s_b, r[:1], w[:1], n[:, :1], x[:1])
    second = lop.time_mix_v7(lop.pack_cursors([(4, 1)]), s_b, r[1:2], w[1:2], n[:, 1:2], x[1:2])
    assert np.array_equal(two, np.concatenate([first, second])) and np.array_equal(s_a, s_b)

    u = (0.3 * rng.standard_normal((H, S))).astype(np.float16)
    got = lop.time_first_v7(u, r, n, x)
    f = np.float64
    want = x.astype(f) + (u.astype(f) * n[0].astype(f) * r.astype(f)).sum(axis=-1, keepdims=True) * n[1].astype(f)
    assert_close(got, want, 1e-5, "time_first_v7 vs float64")

    rows = rng.standard_normal((5, 7, 64)).astype(np.float32)
    got = lop.l2_norm(rows, 1e-12)
    assert_close(got, rows / np.sqrt((rows.astype(f) ** 2).sum(axis=-1, keepdims=True)), 1e-6, "l2_norm vs float64")
    assert_close((got.astype(f) ** 2).sum(axis=-1), np.ones((5, 7)), 1e-6, "unit length")
    assert np.array_equal(lop.l2_norm(np.zeros((1, 8), dtype=np.float32), 1e-12), np.zeros((1, 8), dtype=np.float32))  # eps keeps 0 / 0 away

    p = rng.random(64).astype(np.float16)
    a, k = rng.random((3, 64)).astype(np.float32), rng.standard_normal((3, 64)).astype(np.float32)
    assert_close(lop.control_k_v7(p, a, k), k.astype(f) * (1 + (a.astype(f) - 1) * p.astype(f)), 1e-6, "control_k_v7 vs float64")
    assert np.array_equal(lop.control_k_v7(np.zeros(64, dtype=np.float16), a, k), k)  # p = 0: k unchanged
    assert_close(lop.control_k_v7(np.ones(64, dtype=np.float16), a, k), k * a, 1e-6, "p = 1: k a")

    cm_state = rng.standard_normal((B, 64)).astype(np.float32)
    keep = cm_state.copy()
    xs, vs_ = rng.standard_normal((A, 64)).astype(np.float16), rng.standard_normal((A, 64)).astype(np.float16)
    out = lop.channel_mix_v7(cur, cm_state, vs_, xs)
    assert np.array_equal(out, vs_)
    first = 0
    for slot, cnt in RUNS:
        assert np.array_equal(cm_state[slot], xs[first + cnt - 1].astype(np.float32))
        first += cnt
    assert np.array_equal(cm_state[[1, 3, 4]], keep[[1, 3, 4]])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("H,S,runs", [(3, 32, RUNS), (4, 64, RUNS), (64, 64, [(0, 1)]), (2, 128, [(1, 2), (3, 2)]), (2, 64, [(4, 100)])])
def test_gpu_time_mix_v7(gpu, lop, dtype, H, S, runs):
    import torch

    print("time mix v7 on the GPU", dtype.__name__, H, S, runs[:3], flush=True)
    rng = np.random.default_rng(SEED + 90 + H + S)
    B = 6
    cur = lop.pack_cursors(runs)
    A = len(cur)
    r, w, n, x, state = wkv7_inputs(rng, A, H, S, B, dtype)
    full = np.concatenate([np.zeros_like(state), state], axis=1)
    sview = ((H * S, S + 1, B), (H * S, 2 * (S + 1), B), (0, S + 1, 0))
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    sd, xd, rd, nd = dev(full), dev(x), dev(r), dev(n)
    gpu.LayerOp.time_mix_v7(dev(cur.view(np.int32)), sd, rd, dev(w), nd, xd, state_view=sview)
    want, want_state = wkv7_float64(cur, state, r, w, n, x)
    eps = 2e-3 if dtype == np.float16 else 5e-5
    assert_close(xd.cpu().numpy(), want, eps, "y vs float64")
    got_state = sd.cpu().numpy()
    assert_close(got_state[:, S + 1:], want_state, 5e-5, "state vs float64")
    assert np.array_equal(got_state[:, :S + 1], full[:, :S + 1])  # the other layer's rows are untouched
    if A * H * S * S <= 2000000:
        st = state.copy()
        assert_close(xd.cpu().numpy(), lop.time_mix_v7(cur, st, r, w, n, x), eps, "y vs oracle")
        assert_close(got_state[:, S + 1:], st, 5e-5, "state vs oracle")
    # time_first_v7 on top of the result
    u = (0.3 * rng.standard_normal((H, S))).astype(np.float16)
    y = xd.cpu().numpy()
    gpu.LayerOp.time_first_v7(dev(u), rd, nd, xd)
    assert_close(xd.cpu().numpy(), lop.time_first_v7(u, r, n, y), eps, "time_first_v7 vs oracle")
    f = np.float64
    assert_close(xd.cpu().numpy(), y.astype(f) + (u.astype(f) * n[0].astype(f) * r.astype(f)).sum(axis=-1, keepdims=True) * n[1].astype(f), eps, "time_first_v7 vs float64")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_gpu_v7_small_ops(gpu, lop, dtype):
    import torch

    print("l2 norm / control k / channel mix v7 on the GPU", dtype.__name__, flush=True)
    rng = np.random.default_rng(SEED + 95)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    eps = 2e-3 if dtype == np.float16 else 1e-6
    f = np.float64
    for shape in ((9, 12, 64), (3, 1, 1000), (1, 2, 2048)):
        rows = rng.standard_normal(shape).astype(dtype)
        xd = dev(rows)
        gpu.LayerOp.l2_norm(xd, 1e-12)
        assert_close(xd.cpu().numpy(), lop.l2_norm(rows, 1e-12), eps, f"l2_norm vs oracle {shape}")
        assert_close(xd.cpu().numpy(), rows.astype(f) / np.sqrt((rows.astype(f) ** 2).sum(axis=-1, keepdims=True)), eps, f"l2_norm vs float64 {shape}")
    C, A, B = 256, 8, 6
    p = rng.random(C).astype(np.float16)
    for adt in (np.float16, np.float32):
        a, k = rng.random((1, A, C)).astype(adt), rng.standard_normal((1, A, C)).astype(dtype)
        kd = dev(k)
        gpu.LayerOp.control_k_v7(dev(p), dev(a), kd)
        assert_close(kd.cpu().numpy(), lop.control_k_v7(p, a, k), eps, "control_k_v7 vs oracle")
    # k as one slice of a larger tensor
    big = rng.standard_normal((3, A, C)).astype(dtype)
    a = rng.random((1, A, C)).astype(dtype)
    bd = dev(big)
    gpu.LayerOp.control_k_v7(dev(p), dev(a), bd, k_view=((C, A, 1), (C, A, 3), (0, 0, 2)))
    want = big.copy()
    want[2] = lop.control_k_v7(p, a[0], big[2])
    assert_close(bd.cpu().numpy(), want, eps, "control_k_v7 on a slice")
    assert np.array_equal(bd.cpu().numpy()[:2], big[:2])
    cur = lop.pack_cursors(RUNS)
    A = len(cur)
    rows_, row = 4, 3
    state = rng.standard_normal((B, rows_, C)).astype(np.float32)
    sview = ((C, 1, B), (C, rows_, B), (0, row, 0))
    x, v = rng.standard_normal((A, C)).astype(dtype), rng.standard_normal((A, C)).astype(dtype)
    sd, xd = dev(state), dev(x.reshape(1, A, C))
    gpu.LayerOp.channel_mix_v7(dev(cur.view(np.int32)), sd, dev(v.reshape(1, A, C)), xd, state_view=sview)
    st = state[:, row].copy()
    assert np.array_equal(xd.cpu().numpy()[0], lop.channel_mix_v7(cur, st, v, x))
    want_state = state.copy()
    want_state[:, row] = st
    assert np.array_equal(sd.cpu().numpy(), want_state)


# ---------------------------------------------------------------------------------------------
# the rest of the op set (no test in the reference: float64 forms and invariants pin the restatements)
def test_oracle_misc_ops(lop):
    rng = np.random.default_rng(SEED + 11)
    f = np.float64
    rows = (3.0 + rng.standard_normal((2, 5, 1000))).astype(np.float32)
    got = lop.recenter(rows)
    assert_close(got, rows.astype(f) - rows.astype(f).mean(axis=-1, keepdims=True), 1e-5, "recenter vs float64")
    assert np.abs(got.astype(f).mean(axis=-1)).max() < 1e-5
    w, b = (1.0 + 0.1 * rng.standard_normal(1000)).astype(np.float16), (0.1 * rng.standard_normal(1000)).astype(np.float16)
    got = lop.rms_norm(w, b, rows, 1e-5)
    want = rows.astype(f) / np.sqrt((rows.astype(f) ** 2).mean(axis=-1, keepdims=True) + 1e-5) * w.astype(f) + b.astype(f)
    assert_close(got, want, 1e-5, "rms_norm vs float64")
    # a row of equal values c: recenter gives 0, rms_norm gives sign(c) w + b (eps aside)
    const = np.full((1, 64), -2.5, dtype=np.float32)
    assert np.array_equal(lop.recenter(const), np.zeros((1, 64), dtype=np.float32))
    assert_close(lop.rms_norm(w[:64], b[:64], const, 0.0), -w[:64].astype(f) + b[:64].astype(f), 1e-6, "rms_norm of a constant row")
    src = rng.standard_normal((2, 3, 8)).astype(np.float16)
    dst = np.zeros((4, 6, 8), dtype=np.float32)
    lop.broadcast(src, dst)
    for bb in range(4):
        for t in range(6):
            assert np.array_equal(dst[bb, t], src[bb % 2, t % 3].astype(np.float32))
    x, y = rng.standard_normal((3, 16)).astype(np.float16), rng.standard_normal((3, 16)).astype(np.float32)
    assert_close(lop.blend([0.25, 1.5, 0, 0], x, y), 0.25 * x.astype(f) + 1.5 * y.astype(f), 1e-6, "blend vs float64")
    assert np.array_equal(lop.blend([0, 1, 0, 0], x, y), y) and np.array_equal(lop.blend([1, 0, 0, 0], x, y), x.astype(np.float32))
    xa, xb = rng.standard_normal((2, 12, 8)).astype(np.float16), rng.standard_normal((2, 20, 8)).astype(np.float16)
    out = rng.standard_normal((2, 20, 12)).astype(np.float16)
    got = lop.blend_lora([0.5, 1.0, 0, 0], xa, xb, out)
    want = 0.5 * np.stack([xb[i].astype(f) @ xa[i].astype(f).T for i in range(2)]) + out.astype(f)
    assert_close(got, want, 2e-3, "blend_lora vs float64")
    eye = np.eye(8, dtype=np.float16)[None]
    assert np.array_equal(lop.blend_lora([1, 0, 0, 0], eye, xb[:1], np.zeros((1, 20, 8), dtype=np.float16)), xb[:1])  # xa = I: the product is xb


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_gpu_misc_ops(gpu, lop, dtype):
    import torch

    print("recenter / rms_norm / broadcast / blend / blend_lora on the GPU", dtype.__name__, flush=True)
    rng = np.random.default_rng(SEED + 96)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    eps = 2e-3 if dtype == np.float16 else 2e-6
    f = np.float64
    for shape in ((2, 5, 1000), (1, 3, 4096), (3, 1, 64)):
        rows = (1.0 + rng.standard_normal(shape)).astype(dtype)
        C = shape[-1]
        w, b = (1.0 + 0.1 * rng.standard_normal(C)).astype(np.float16), (0.1 * rng.standard_normal(C)).astype(np.float16)
        xd = dev(rows)
        gpu.LayerOp.recenter(xd)
        assert_close(xd.cpu().numpy(), lop.recenter(rows), eps, f"recenter vs oracle {shape}")
        assert_close(xd.cpu().numpy(), rows.astype(f) - rows.astype(f).mean(axis=-1, keepdims=True), 2 * eps, f"recenter vs float64 {shape}")
        xd = dev(rows)
        gpu.LayerOp.rms_norm(dev(w), dev(b), xd, 1e-5)
        assert_close(xd.cpu().numpy(), lop.rms_norm(w, b, rows, 1e-5), eps, f"rms_norm vs oracle {shape}")
    src = rng.standard_normal((2, 3, 256)).astype(np.float16)
    big = np.zeros((5, 7, 256), dtype=dtype)
    bd = dev(big)
    gpu.LayerOp.broadcast(dev(src), bd, output_view=((256, 6, 4), (256, 7, 5), (0, 1, 1)))
    want = big.copy()
    lop.broadcast(src, want[1:, 1:])
    assert np.array_equal(bd.cpu().numpy(), want)
    x, y = rng.standard_normal((3, 5, 64)).astype(np.float16), rng.standard_normal((3, 5, 64)).astype(dtype)
    factor = np.array([0.25, 1.5, 0, 0], dtype=np.float32)
    yd = dev(y)
    gpu.LayerOp.blend(dev(factor), dev(x), yd)
    assert_close(yd.cpu().numpy(), lop.blend(factor, x, y), eps, "blend vs oracle")
    with pytest.raises(gpu.TensorError):
        gpu.LayerOp.blend(dev(factor), dev(x[:2]), yd)
    if dtype == np.float16:
        # a rank-32 adapter blended into a 768 x 512 matrix, and into a slice of a stack of matrices
        M, N, K = 512, 768, 32
        xa, xb = (0.1 * rng.standard_normal((1, M, K))).astype(np.float16), (0.1 * rng.standard_normal((1, N, K))).astype(np.float16)
        out = (0.02 * rng.standard_normal((1, N, M))).astype(np.float16)
        factor = np.array([2.0 / K, 1.0, 0, 0], dtype=np.float32)
        od = dev(out)
        gpu.LayerOp.blend_lora(dev(factor), dev(xa), dev(xb), od)
        assert_close(od.cpu().numpy(), lop.blend_lora(factor, xa, xb, out), 2e-3, "blend_lora vs oracle")
        want = factor[0] * (xb[0].astype(f) @ xa[0].astype(f).T) + out[0].astype(f)
        assert_close(od.cpu().numpy()[0], want, 2e-3, "blend_lora vs float64")
        stack = (0.02 * rng.standard_normal((3, 20, 64))).astype(np.float16)
        xa, xb = rng.standard_normal((1, 64, 8)).astype(np.float16), rng.standard_normal((1, 20, 8)).astype(np.float16)
        sd = dev(stack)
        gpu.LayerOp.blend_lora(dev(factor), dev(xa), dev(xb), sd, output_view=((64, 20, 1), (64, 20, 3), (0, 0, 2)))
        want = stack.copy()
        want[2:] = lop.blend_lora(factor, xa, xb, stack[2:])
        assert_close(sd.cpu().numpy(), want, 2e-3, "blend_lora into a slice")
        assert np.array_equal(sd.cpu().numpy()[:2], stack[:2])


# ---------------------------------------------------------------------------------------------
@pytest.mark.gpu
def test_gpu_data_movement_kats(gpu):
    import torch

    print("blit / transpose KATs on the GPU", flush=True)
    k = movement_kats()
    for dt in (torch.float32, torch.float16):
        out = torch.zeros(k["blit"]["output_shape"][::-1][1:], dtype=dt, device="cuda")
        for op in k["blit"]["ops"]:
            src = torch.tensor(op["input"], dtype=torch.float32, device="cuda").reshape(op["input_shape"][::-1][1:])
            gpu.LayerOp.blit(src, out, output_view=(op["view_shape"], k["blit"]["output_shape"], op["view_offset"]))
        assert out.float().reshape(-1).tolist() == k["blit"]["expected"]
        t = k["transpose"]
        out = torch.zeros(t["output_shape"][::-1][1:], dtype=dt, device="cuda")
        src = torch.tensor(t["input"], dtype=torch.float32, device="cuda").reshape(t["input_shape"][::-1][1:])
        gpu.LayerOp.transpose(src, out, output_view=(t["view_shape"], t["output_shape"], t["view_offset"]))
        assert out.float().reshape(-1).tolist() == t["expected"]
    with pytest.raises(gpu.TensorError):
        gpu.LayerOp.transpose(src, torch.zeros((3, 2, 8), dtype=torch.float32, device="cuda"))


@pytest.mark.gpu
def test_gpu_embed(gpu):
    import torch

    print("embed on the GPU", flush=True)
    rng = np.random.default_rng(SEED + 45)
    V, C, T, B = 300, 128, 5, 2
    table = rng.standard_normal((V, C)).astype(np.float16)
    ids = rng.integers(0, V, size=(B, T)).astype(np.int32)
    for dt in (torch.float16, torch.float32):
        out = torch.zeros((B, T, C), dtype=dt, device="cuda")
        gpu.LayerOp.embed(torch.from_numpy(ids).cuda(), torch.from_numpy(table).cuda(), out)
        assert np.array_equal(out.cpu().numpy(), table[ids].astype(out.cpu().numpy().dtype))  # a gather: exact
    with pytest.raises(gpu.TensorError):
        gpu.LayerOp.embed(torch.from_numpy(ids).cuda(), torch.from_numpy(table).cuda(), torch.zeros((B, T + 1, C), dtype=torch.float16, device="cuda"))


@pytest.mark.gpu
def test_gpu_lerp_activate_affine(gpu, lop):
    import torch

    print("lerp / activate / affine on the GPU", flush=True)
    rng = np.random.default_rng(SEED + 40)
    B, T, C = 2, 3, 1000
    x = (rng.random((B, T, C), dtype=np.float32) - 0.5).astype(np.float32)
    y = (rng.random((B, T, C), dtype=np.float32) - 0.5).astype(np.float32)
    for fshape in ((B, T, C), (1, T, C), (B, 1, C), (1, 1, C)):
        f = rng.random(fshape, dtype=np.float32)
        for rev in (False, True):
            for ft, it, ot in ((np.float32, np.float32, np.float32), (np.float16, np.float16, np.float32), (np.float32, np.float16, np.float16)):
                yd = torch.from_numpy(y.astype(ot)).cuda()
                gpu.LayerOp.lerp(torch.from_numpy(x.astype(it)).cuda(), yd, torch.from_numpy(f.astype(ft)).cuda(), rev)
                want = lop.lerp(x.astype(it), y.astype(ot), f.astype(ft), rev)
                assert_close(yd.cpu().numpy(), want, 1e-3 if ot == np.float16 else 1e-6, f"lerp {fshape} {rev} {ot.__name__}")
    for act in range(8):
        for dt in (np.float32, np.float16):
            v = (1.5 * rng.standard_normal((B, T, C))).astype(dt)  # exp stays inside f16
            vd = torch.from_numpy(v.copy()).cuda()
            gpu.LayerOp.activate(vd, act)
            assert_close(vd.cpu().numpy(), lop.activation(act, v.astype(np.float32)).astype(dt), 2e-3 if dt == np.float16 else 2e-6, f"activate {act} {dt.__name__}")
    # a view: only slice 1 of 3 changes
    v = rng.standard_normal((3, T, C)).astype(np.float32)
    vd = torch.from_numpy(v.copy()).cuda()
    gpu.LayerOp.activate(vd, gpu.ACT_STABLE_EXP, view=((C, T, 1), (C, T, 3), (0, 0, 1)))
    want = v.copy()
    want[1] = lop.activation(3, v[1])
    assert_close(vd.cpu().numpy(), want, 2e-6, "activate on a view")
    xd = torch.from_numpy(x.copy()).cuda()
    gpu.LayerOp.affine(xd, 0.5, 0.0)
    assert np.array_equal(xd.cpu().numpy(), x * np.float32(0.5))
    hd = torch.from_numpy(x.astype(np.float16)).cuda()
    gpu.LayerOp.affine(hd, 2.0, 1.0)
    assert_close(hd.cpu().numpy(), lop.affine(x.astype(np.float16), 2.0, 1.0), 1e-3, "affine f16")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("C,T,B", [(1000, 3, 2), (4096, 1, 1), (4096, 128, 1), (65536, 2, 1), (64, 5, 1), (4, 1, 3)])
def test_gpu_softmax_layer_norm(gpu, lop, dtype, C, T, B):
    import torch

    print("softmax / layer norm on the GPU", dtype.__name__, C, T, B, flush=True)
    rng = np.random.default_rng(SEED + 10 + C + T)
    x, w, b = reference_test_inputs(rng, C=C, T=T, B=B)
    x = x.astype(dtype)
    eps_out = 1e-3 if dtype == np.float16 else 2e-5
    xd = torch.from_numpy(x.copy()).cuda()
    gpu.LayerOp.softmax(xd)
    if T * C <= 20000:
        assert_close(xd.cpu().numpy(), lop.softmax(x), eps_out if dtype == np.float16 else 1e-6, "softmax vs oracle")
    assert_close(xd.cpu().numpy(), softmax64(x), eps_out if dtype == np.float16 else 1e-6, "softmax vs float64")
    xd = torch.from_numpy(x.copy()).cuda()
    gpu.LayerOp.layer_norm(torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda(), xd, 1e-5)
    if T * C <= 20000:
        assert_close(xd.cpu().numpy(), lop.layer_norm(w, b, x, 1e-5), eps_out * 2, "layer norm vs oracle")
    assert_close(xd.cpu().numpy(), layer_norm64(w, b, x, 1e-5), 1e-3, "layer norm vs float64")  # the reference's bar (ops.rs:2750)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("A,H,S", [(1, 64, 64), (33, 64, 64), (4, 32, 128), (2, 3, 2048)])
def test_gpu_group_norm(gpu, lop, dtype, A, H, S):
    import torch

    print("group norm on the GPU", dtype.__name__, A, H, S, flush=True)
    rng = np.random.default_rng(SEED + 20 + A + S)
    x = (4.0 * rng.standard_normal((A, H, S))).astype(dtype)
    w = rng.standard_normal((H, S)).astype(np.float16)
    b = rng.standard_normal((H, S)).astype(np.float16)
    xd = torch.from_numpy(x.copy()).cuda()
    gpu.LayerOp.group_norm(torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda(), xd, 64e-5)
    eps = 2e-3 if dtype == np.float16 else 1e-4
    if A * H * S <= 20000:
        assert_close(xd.cpu().numpy(), lop.group_norm(w, b, x, 64e-5), eps, "vs oracle")
    assert_close(xd.cpu().numpy(), layer_norm64(w[None], b[None], x, 64e-5), max(eps, 1e-3), "vs float64")


@pytest.mark.gpu
@pytest.mark.parametrize("op", ["add", "mul"])
def test_gpu_binary(gpu, lop, op):
    import torch

    print("binary ops on the GPU", op, flush=True)
    rng = np.random.default_rng(SEED + 30)
    C, T, B = 256, 5, 2
    fn = gpu.LayerOp.mul_activate if op == "mul" else gpu.LayerOp.add_activate
    for it, ot in ((np.float16, np.float32), (np.float32, np.float16), (np.float16, np.float16), (np.float32, np.float32)):
        y = rng.standard_normal((B, T, C)).astype(ot)
        for xs in ((B, T, C), (B, 1, C), (1, 1, C)):
            x = rng.standard_normal(xs).astype(it)
            for acts in ((0, 0, 0), (7, 0, 0), (2, 6, 1), (0, 3, 5)):
                yd = torch.from_numpy(y.copy()).cuda()
                fn(torch.from_numpy(x).cuda(), yd, *acts)
                want = lop.binary(op, lop.activation(acts[0], x.astype(np.float32)), lop.activation(acts[1], y.astype(np.float32)))
                want = lop.activation(acts[2], want.astype(np.float32)).astype(ot)
                assert_close(yd.cpu().numpy(), want, 2e-3 if ot == np.float16 else 1e-5, f"{op} {it.__name__}->{ot.__name__} {xs} {acts}")
    # views: the input is slice 2 of a [C, T, 5] stack, the output rows 1..3 of a taller tensor
    stack = rng.standard_normal((5, T, C)).astype(np.float16)
    tall = rng.standard_normal((1, T + 2, C)).astype(np.float32)
    td = torch.from_numpy(tall.copy()).cuda()
    fn(torch.from_numpy(stack).cuda(), td, 0, 0, 0, input_view=((C, T, 1), (C, T, 5), (0, 0, 2)), output_view=((C, T, 1), (C, T + 2, 1), (0, 1, 0)))
    want = tall.copy()
    want[0, 1:T + 1] = lop.binary(op, stack[2], tall[0, 1:T + 1])
    assert_close(td.cpu().numpy(), want, 1e-5, "views")
    # the constructor's shape rule
    with pytest.raises(gpu.TensorError):
        fn(torch.zeros((B, T, C // 2), dtype=torch.float16, device="cuda"), torch.zeros((B, T, C), dtype=torch.float16, device="cuda"))
