"""Independent numpy closed forms used to pin the oracle and to judge the HIP path.

None of these call the oracle.  The int8 / nf4 forms are the ones the reference's
own unit tests use (src/tensor/ops.rs:2939-2962, :3004-3018, :3114-3144,
:3199-3211), which differ from the shader arithmetic in documented ways (division
instead of reciprocal, round-half-away instead of the packing builtin, strict `<`).
"""
import numpy as np

NF4_QUANT = np.array(
    [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
     -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
     0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
     0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0],
    dtype=np.float32,
)

EPS = 2e-3  # north-star tolerance for products (f16 output, f32 accumulate)


def is_approx_eps(a, b, eps):
    """|a-b| <= max(eps, eps*max(|a|,|b|)); src/tensor/ops.rs:2614-2618."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) <= np.maximum(eps, np.maximum(np.abs(a), np.abs(b)) * eps)


def assert_close(a, b, eps=EPS, what=""):
    ok = is_approx_eps(a, b, eps)
    if not ok.all():
        bad = np.argwhere(~ok)
        i = tuple(bad[0])
        raise AssertionError(
            f"{what}: {len(bad)} of {ok.size} outside eps={eps}; first at {i}: "
            f"{np.asarray(a)[i]} vs {np.asarray(b)[i]}"
        )


def gen_f16(rng, shape, std):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std)).astype(np.float16)


def int8_test_form(w):
    """Reference test's packer (ops.rs:2939-2962): f32 math, f32::round (half away)."""
    w32 = w.astype(np.float32).reshape(-1, 128)
    mn = w32.min(axis=1, keepdims=True)
    mx = w32.max(axis=1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        q = (w32 - mn) / (mx - mn)
        s = (q * np.float32(255.0)).astype(np.float32)
    # f32::round = half away from zero of the f32 product (s >= 0 here); evaluated in f64 so
    # that the `+ 0.5` itself cannot round
    r = np.floor(s.astype(np.float64) + 0.5)
    tie = (s.astype(np.float64) - np.floor(s.astype(np.float64))) == 0.5
    u8 = np.nan_to_num(r, nan=0.0).astype(np.uint8)
    minmax = np.stack([mn[:, 0], mx[:, 0]], axis=1).reshape(-1).astype(np.float16)
    return u8.reshape(w.shape), minmax, tie.reshape(w.shape)


def int8_f64_form(w):
    """Exact-arithmetic view of the packer: 255*(v-min)/(max-min) in float64."""
    w64 = w.astype(np.float64).reshape(-1, 128)
    mn = w64.min(axis=1, keepdims=True)
    mx = w64.max(axis=1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        s = 255.0 * (w64 - mn) / (mx - mn)
    return s.reshape(w.shape)


def int8_dequant64(u8, minmax):
    """(u8/255)*(max-min)+min per 128-block (ops.rs:3011-3016), in float64."""
    mm = minmax.astype(np.float64).reshape(-1, 2)
    u = u8.astype(np.float64).reshape(-1, 128)
    return (u / 255.0 * (mm[:, 1:2] - mm[:, 0:1]) + mm[:, 0:1]).reshape(u8.shape)


def nf4_test_form(w, quant=NF4_QUANT):
    """Reference test's packer (ops.rs:3114-3144): v/absmax, strict '<' (first wins)."""
    w32 = w.astype(np.float32).reshape(-1, 64)
    am = np.abs(w32).max(axis=1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore"):
        x = (w32 / am).astype(np.float32)
    err = np.abs(x[..., None] - quant[None, None, :]).astype(np.float32)
    err = np.where(np.isnan(err), np.inf, err)
    idx = err.argmin(axis=2).astype(np.uint8)  # argmin returns the first minimum
    idx = idx.reshape(-1)
    packed = (idx[0::2] | (idx[1::2] << 4)).astype(np.uint8)
    return packed.reshape(w.shape[:-1] + (w.shape[-1] // 2,)), am[:, 0].astype(np.float16), x.reshape(w.shape)


def nf4_unpack(packed):
    p = packed.reshape(-1)
    idx = np.empty(p.size * 2, dtype=np.uint8)
    idx[0::2] = p & 0xF
    idx[1::2] = p >> 4
    return idx.reshape(packed.shape[:-1] + (packed.shape[-1] * 2,))


def nf4_dequant64(packed, absmax, quant=NF4_QUANT):
    idx = nf4_unpack(packed)
    q = quant.astype(np.float64)[idx].reshape(-1, 64)
    return (q * absmax.astype(np.float64)[:, None]).reshape(idx.shape)


ACTS = {
    "none": lambda x: x,
    "squared_relu": lambda x: np.maximum(x, 0.0) ** 2,
    "tanh": lambda x: np.where(x > 42.0, 1.0, np.tanh(x)),
    "stable_exp": lambda x: np.exp(-np.exp(x)),
    "opposite_exp": lambda x: -np.exp(x),
    "softplus": lambda x: np.log(1.0 + np.exp(x)),
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "silu": lambda x: x / (1.0 + np.exp(-x)),
}


def truth_matmul(wdeq64, x, act="none"):
    """Textbook product in float64: out[t, r] = act(sum_k W[r, k] x[t, k])."""
    return ACTS[act](x.astype(np.float64) @ wdeq64.T)
