"""ctypes binding of ``libwrq_hip.so`` for tests and benchmarks.

The product is the shared library (C ABI in ``include/wrq.h``); this module only loads it
and wraps torch device tensors into the ``wrq_tensor`` / ``wrq_tensor_view`` structs.  It
never computes anything itself: without the library, or without a GPU, calls fail loudly.

Names mirror the reference (``TensorOp::matmul_vec_int8`` ... in src/tensor/ops.rs,
``Matrix::quant_u8`` ... in src/tensor/matrix.rs).  Shapes are given in the reference's
order, x fastest: a torch tensor of shape ``(B, R, K)`` is the reference's ``[K, R, B, 1]``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libwrq_hip.so")
CSRC = os.path.join(_HERE, "csrc")

INT8_BLOCK_SIZE = 128
NF4_BLOCK_SIZE = 64

OK, ERR_SHAPE, ERR_SIZE, ERR_TYPE, ERR_ALIGNMENT, ERR_UNSUPPORTED, ERR_NULL, ERR_DEVICE = range(8)
F16, F32 = 0, 1

ACTIVATIONS = ["", "squared_relu", "custom_tanh", "stable_exp", "opposite_exp", "softplus", "sigmoid", "silu"]
ACT_NONE, ACT_SQUARED_RELU, ACT_TANH, ACT_STABLE_EXP, ACT_OPPOSITE_EXP, ACT_SOFTPLUS, ACT_SIGMOID, ACT_SILU = range(8)

# Float4Quant::new, src/tensor/matrix.rs:46-70
NF4_QUANT = [
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0,
]

EXPORTS = [
    "wrq_init", "wrq_abi_version", "wrq_abi_minor", "wrq_status_string", "wrq_last_error",
    "wrq_debug_override",
    "wrq_debug_stamps",
    "wrq_quantize_mat_int8", "wrq_quantize_mat_nf4",
    "wrq_matmul_vec_int8", "wrq_matmul_vec_nf4", "wrq_matmul_mat_int8", "wrq_matmul_mat_nf4", "wrq_matmul_mat_int8_noalloc",
    "wrq_matmul_vec_int8_group", "wrq_matmul_vec_nf4_group",
    "wrq_matmul_vec_fp16", "wrq_matmul_mat_fp16",
    "wrq_softmax", "wrq_layer_norm", "wrq_group_norm", "wrq_add_activate", "wrq_mul_activate",
    "wrq_blit", "wrq_transpose", "wrq_activate", "wrq_affine", "wrq_lerp",
    "wrq_token_shift", "wrq_channel_mix", "wrq_time_mix_v4", "wrq_time_mix_v5", "wrq_time_mix_v6", "wrq_embed",
    "wrq_l2_norm", "wrq_control_k_v7", "wrq_time_mix_v7", "wrq_time_first_v7", "wrq_channel_mix_v7",
    "wrq_recenter", "wrq_rms_norm", "wrq_broadcast", "wrq_blend", "wrq_blend_lora",
    "wrq_v6_pre", "wrq_v6_time_mix", "wrq_v6_decay", "wrq_v6_wkv_gate", "wrq_v6_post_ffn",
]
MAX_GROUP = 8


def quantile_student(nu):
    """Float4Quant::new_student (src/tensor/matrix.rs:29-44): the 16-entry SF4 table.

    Quantiles of Student's t at delta + i (0.5 - delta) / 7 (i < 7) and 0.5 + i (0.5 - delta) / 8
    (i < 9), delta = (1/32 + 1/30) / 2, divided by the largest.  The reference uses the `statrs`
    crate's inverse CDF; here the CDF (regularised incomplete beta, continued fraction) is
    inverted by bisection in double precision.
    """
    import math

    def betacf(a, b, x):
        tiny = 1e-300
        qab, qap, qam = a + b, a + 1.0, a - 1.0
        c, d = 1.0, 1.0 - qab * x / qap
        d = 1.0 / (d if abs(d) > tiny else tiny)
        h = d
        for m in range(1, 401):
            m2 = 2 * m
            aa = m * (b - m) * x / ((qam + m2) * (a + m2))
            d = 1.0 + aa * d
            d = 1.0 / (d if abs(d) > tiny else tiny)
            c = 1.0 + aa / c
            c = c if abs(c) > tiny else tiny
            h *= d * c
            aa = -(a + m) * (qab + m) * x / ((a + m2) * (qap + m2))
            d = 1.0 + aa * d
            d = 1.0 / (d if abs(d) > tiny else tiny)
            c = 1.0 + aa / c
            c = c if abs(c) > tiny else tiny
            h *= d * c
            if abs(d * c - 1.0) < 1e-16:
                break
        return h

    def betai(a, b, x):
        if x <= 0.0:
            return 0.0
        if x >= 1.0:
            return 1.0
        bt = math.exp(math.lgamma(a + b) - math.lgamma(a) - math.lgamma(b) + a * math.log(x) + b * math.log(1.0 - x))
        return bt * betacf(a, b, x) / a if x < (a + 1.0) / (a + b + 2.0) else 1.0 - bt * betacf(b, a, 1.0 - x) / b

    def cdf(t):
        tail = 0.5 * betai(0.5 * nu, 0.5, nu / (nu + t * t))
        return 1.0 - tail if t > 0 else tail

    def quantile(p):
        if p == 0.5:
            return 0.0  # the median, exactly (table entry 7)
        lo, hi = -1e6, 1e6
        for _ in range(200):
            mid = 0.5 * (lo + hi)
            if cdf(mid) < p:
                lo = mid
            else:
                hi = mid
        return 0.5 * (lo + hi)

    delta = (1.0 / 32.0 + 1.0 / 30.0) / 2.0
    probs = [delta + (0.5 - delta) / 7.0 * i for i in range(7)] + [0.5 + (1.0 - delta - 0.5) / 8.0 * i for i in range(9)]
    q = [quantile(p) for p in probs]
    most = max(q)
    import numpy as np

    return [float(np.float32(v / most)) for v in q]


class TensorError(RuntimeError):
    """A failed op constructor; ``status`` is the wrq_status code."""

    def __init__(self, status, message):
        super().__init__(message)
        self.status = status


class CTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("shape", C.c_uint32 * 4)]


class CView(C.Structure):
    _fields_ = [("shape", C.c_uint32 * 4), ("stride", C.c_uint32 * 4), ("offset", C.c_uint32 * 4)]


class CTensorView(C.Structure):
    _fields_ = [("data", C.c_void_p), ("view", CView), ("dtype", C.c_int)]


class CVecInt8Op(C.Structure):
    _fields_ = [("matrix", C.POINTER(CTensor)), ("minmax", C.POINTER(CTensor)), ("input", C.POINTER(CTensorView)),
                ("output", C.POINTER(CTensorView)), ("act", C.c_int), ("sparse", C.c_int)]


class CVecNf4Op(C.Structure):
    _fields_ = [("matrix", C.POINTER(CTensor)), ("quant", C.POINTER(CTensor)), ("absmax", C.POINTER(CTensor)),
                ("input", C.POINTER(CTensorView)), ("output", C.POINTER(CTensorView)), ("act", C.c_int), ("sparse", C.c_int)]


def build(verbose=False):
    """Compile every HIP source for gfx950 into ``libwrq_hip.so`` (always recompiles)."""
    r = subprocess.run(["make", "-C", CSRC, "-B", "-j8"], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libwrq_hip.so failed:\n" + r.stdout[-4000:] + r.stderr[-4000:])
    if verbose:
        print(r.stdout[-2000:])
    return LIB_PATH


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc --offload-arch=gfx950); this package has no CPU or eager fallback"
            )
        L = C.CDLL(LIB_PATH)
        T, V, vp, i = C.POINTER(CTensor), C.POINTER(CTensorView), C.c_void_p, C.c_int
        L.wrq_init.restype = i
        L.wrq_abi_version.restype = i
        L.wrq_status_string.restype = C.c_char_p
        L.wrq_status_string.argtypes = [i]
        L.wrq_last_error.restype = C.c_char_p
        L.wrq_debug_override.argtypes = [C.c_char_p, i]
        L.wrq_debug_stamps.argtypes = [vp, C.c_uint64]
        L.wrq_quantize_mat_int8.argtypes = [vp, T, T, T]
        L.wrq_quantize_mat_nf4.argtypes = [vp, T, T, T, T]
        L.wrq_matmul_vec_int8.argtypes = [vp, T, T, V, V, i, i]
        L.wrq_matmul_vec_nf4.argtypes = [vp, T, T, T, V, V, i, i]
        L.wrq_matmul_mat_int8.argtypes = [vp, V, T, V, V, i]
        L.wrq_matmul_mat_int8_noalloc.argtypes = [vp, V, T, V, V, i]
        L.wrq_matmul_mat_nf4.argtypes = [vp, V, T, T, V, V, i]
        L.wrq_matmul_vec_fp16.argtypes = [vp, T, V, V, i, i]
        L.wrq_matmul_mat_fp16.argtypes = [vp, V, V, V, i]
        L.wrq_matmul_vec_int8_group.argtypes = [vp, C.POINTER(CVecInt8Op), i]
        L.wrq_matmul_vec_nf4_group.argtypes = [vp, C.POINTER(CVecNf4Op), i]
        L.wrq_softmax.argtypes = [vp, T, i]
        L.wrq_layer_norm.argtypes = [vp, T, T, T, i, C.c_float]
        L.wrq_group_norm.argtypes = [vp, T, T, T, i, C.c_float]
        L.wrq_add_activate.argtypes = [vp, V, V, i, i, i]
        L.wrq_mul_activate.argtypes = [vp, V, V, i, i, i]
        L.wrq_blit.argtypes = [vp, V, V]
        L.wrq_transpose.argtypes = [vp, V, V]
        L.wrq_activate.argtypes = [vp, V, i]
        L.wrq_affine.argtypes = [vp, T, i, C.c_float, C.c_float]
        L.wrq_lerp.argtypes = [vp, V, V, V, i]
        L.wrq_token_shift.argtypes = [vp, T, V, V, T, i, T, i, i]
        L.wrq_channel_mix.argtypes = [vp, T, V, T, T, T, i]
        L.wrq_time_mix_v4.argtypes = [vp, T, T, T, V, T, T, T, T, i]
        L.wrq_time_mix_v5.argtypes = [vp, T, T, T, V, T, T, T, T, i]
        L.wrq_time_mix_v6.argtypes = [vp, T, T, T, V, T, T, T, T, i]
        L.wrq_l2_norm.argtypes = [vp, T, i, C.c_float]
        L.wrq_control_k_v7.argtypes = [vp, T, V, V]
        L.wrq_time_mix_v7.argtypes = [vp, T, V, T, T, T, T, i]
        L.wrq_time_first_v7.argtypes = [vp, T, T, T, T, i]
        L.wrq_channel_mix_v7.argtypes = [vp, T, V, T, T, i]
        L.wrq_recenter.argtypes = [vp, T, i]
        L.wrq_rms_norm.argtypes = [vp, T, T, T, i, C.c_float]
        L.wrq_broadcast.argtypes = [vp, V, V]
        L.wrq_blend.argtypes = [vp, T, T, i, T, i]
        L.wrq_blend_lora.argtypes = [vp, T, V, V, V]
        L.wrq_embed.argtypes = [vp, T, T, T, i]
        u = C.c_uint32
        L.wrq_v6_pre.argtypes = [vp, u, u, vp, vp, vp, vp, vp, vp, C.c_float, V, i, vp, vp, vp, vp, vp]
        L.wrq_v6_time_mix.argtypes = [vp, u, u, u, vp, vp, vp, vp, V, vp, vp]
        L.wrq_v6_decay.argtypes = [vp, u, u, u, vp, vp, vp, vp]
        L.wrq_v6_wkv_gate.argtypes = [vp, u, u, u, vp, vp, vp, V, vp, vp, vp, vp, vp, vp, C.c_float, vp]
        L.wrq_v6_post_ffn.argtypes = [vp, u, u, vp, V, vp, vp, vp, vp, vp, i]
        for name in EXPORTS:
            if name not in ("wrq_status_string", "wrq_last_error"):
                getattr(L, name).restype = i
        _lib = L
    return _lib


def debug_override(key, value=-1):
    """``wrq_debug_override``: pin (value >= 0) or release (value < 0) one kernel / tile choice."""
    _check(lib().wrq_debug_override(key.encode(), int(value)))


def _check(status):
    if status != OK:
        raise TensorError(status, lib().wrq_last_error().decode())


def _stream():
    import torch

    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def shape_of(t):
    """Reference-order shape [x, y, z, w] of a torch tensor (last dim is x)."""
    s = list(t.shape)[::-1]
    assert len(s) <= 4
    return s + [1] * (4 - len(s))


def as_tensor(t, shape=None):
    """``TensorGpu``: a contiguous device tensor and its shape."""
    assert t.is_contiguous()
    return CTensor(t.data_ptr(), tuple(shape if shape is not None else shape_of(t)))


def _dtype(t):
    import torch

    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.float32:
        return F32
    return 2  # rejected by the library with ERR_TYPE


def as_view(t, view=None, dtype=None):
    """``TensorGpuView``: parent tensor plus (shape, stride, offset); default the whole tensor."""
    assert t.is_contiguous()
    if view is None:
        s = shape_of(t)
        view = (s, s, [0, 0, 0, 0])
    pad = lambda v, f: tuple(v) + (f,) * (4 - len(v))
    cv = CView(pad(view[0], 1), pad(view[1], 1), pad(view[2], 0))
    return CTensorView(t.data_ptr(), cv, _dtype(t) if dtype is None else dtype)


class TensorOp:
    """The six constructors of the path; each enqueues on torch's current stream."""

    INT8_BLOCK_SIZE = INT8_BLOCK_SIZE
    NF4_BLOCK_SIZE = NF4_BLOCK_SIZE

    @staticmethod
    def quantize_mat_int8(input, minmax, output):
        _check(lib().wrq_quantize_mat_int8(_stream(), C.byref(as_tensor(input)), C.byref(as_tensor(minmax)), C.byref(as_tensor(output))))

    @staticmethod
    def quantize_mat_nf4(input, quant, absmax, output):
        _check(lib().wrq_quantize_mat_nf4(_stream(), C.byref(as_tensor(input)), C.byref(as_tensor(quant)), C.byref(as_tensor(absmax)), C.byref(as_tensor(output))))

    @staticmethod
    def matmul_vec_int8(matrix, minmax, input, output, act=ACT_NONE, sparse=False, input_view=None, output_view=None):
        _check(lib().wrq_matmul_vec_int8(_stream(), C.byref(as_tensor(matrix)), C.byref(as_tensor(minmax)),
                                         C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act, int(sparse)))

    @staticmethod
    def matmul_vec_nf4(matrix, quant, absmax, input, output, act=ACT_NONE, sparse=False, input_view=None, output_view=None):
        _check(lib().wrq_matmul_vec_nf4(_stream(), C.byref(as_tensor(matrix)), C.byref(as_tensor(quant)), C.byref(as_tensor(absmax)),
                                        C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act, int(sparse)))

    @staticmethod
    def matmul_mat_int8(matrix, minmax, input, output, act=ACT_NONE, matrix_view=None, input_view=None, output_view=None):
        _check(lib().wrq_matmul_mat_int8(_stream(), C.byref(as_view(matrix, matrix_view, dtype=F16)), C.byref(as_tensor(minmax)),
                                         C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act))

    @staticmethod
    def matmul_mat_int8_noalloc(matrix, minmax, input, output, act=ACT_NONE, matrix_view=None, input_view=None, output_view=None):
        _check(lib().wrq_matmul_mat_int8_noalloc(_stream(), C.byref(as_view(matrix, matrix_view, dtype=F16)), C.byref(as_tensor(minmax)),
                                                 C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act))

    @staticmethod
    def matmul_mat_nf4(matrix, quant, absmax, input, output, act=ACT_NONE, matrix_view=None, input_view=None, output_view=None):
        _check(lib().wrq_matmul_mat_nf4(_stream(), C.byref(as_view(matrix, matrix_view, dtype=F16)), C.byref(as_tensor(quant)), C.byref(as_tensor(absmax)),
                                        C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act))

    @staticmethod
    def matmul_vec_fp16(matrix, input, output, act=ACT_NONE, sparse=False, input_view=None, output_view=None):
        _check(lib().wrq_matmul_vec_fp16(_stream(), C.byref(as_tensor(matrix)), C.byref(as_view(input, input_view)),
                                         C.byref(as_view(output, output_view)), act, int(sparse)))

    @staticmethod
    def matmul_mat_fp16(matrix, input, output, act=ACT_NONE, matrix_view=None, input_view=None, output_view=None):
        _check(lib().wrq_matmul_mat_fp16(_stream(), C.byref(as_view(matrix, matrix_view)), C.byref(as_view(input, input_view)),
                                         C.byref(as_view(output, output_view)), act))


class LayerOp:
    """The row-wise and element-wise ops between the matrix products (src/tensor/ops.rs:300-509,
    :1227-1391); each enqueues on torch's current stream and works in place like the reference."""

    @staticmethod
    def softmax(x):
        _check(lib().wrq_softmax(_stream(), C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def layer_norm(w, b, x, eps):
        _check(lib().wrq_layer_norm(_stream(), C.byref(as_tensor(w)), C.byref(as_tensor(b)), C.byref(as_tensor(x)), _dtype(x), eps))

    @staticmethod
    def group_norm(w, b, x, eps):
        _check(lib().wrq_group_norm(_stream(), C.byref(as_tensor(w)), C.byref(as_tensor(b)), C.byref(as_tensor(x)), _dtype(x), eps))

    @staticmethod
    def add_activate(input, output, act_x=ACT_NONE, act_y=ACT_NONE, act_out=ACT_NONE, input_view=None, output_view=None):
        _check(lib().wrq_add_activate(_stream(), C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act_x, act_y, act_out))

    @staticmethod
    def mul_activate(input, output, act_x=ACT_NONE, act_y=ACT_NONE, act_out=ACT_NONE, input_view=None, output_view=None):
        _check(lib().wrq_mul_activate(_stream(), C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)), act_x, act_y, act_out))

    add = add_activate
    mul = mul_activate

    @staticmethod
    def embed(tokens, input, output):
        _check(lib().wrq_embed(_stream(), C.byref(as_tensor(tokens)), C.byref(as_tensor(input)), C.byref(as_tensor(output)), _dtype(output)))

    @staticmethod
    def blit(input, output, input_view=None, output_view=None):
        _check(lib().wrq_blit(_stream(), C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view))))

    @staticmethod
    def transpose(input, output, input_view=None, output_view=None):
        _check(lib().wrq_transpose(_stream(), C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view))))

    @staticmethod
    def activate(x, act, view=None):
        _check(lib().wrq_activate(_stream(), C.byref(as_view(x, view)), act))

    @staticmethod
    def affine(x, scale, bias):
        _check(lib().wrq_affine(_stream(), C.byref(as_tensor(x)), _dtype(x), scale, bias))

    @staticmethod
    def token_shift(cursors, time_mix, state, input, output, reversed=False, time_mix_view=None, state_view=None):
        _check(lib().wrq_token_shift(_stream(), C.byref(as_tensor(cursors)), C.byref(as_view(time_mix, time_mix_view)), C.byref(as_view(state, state_view)),
                                     C.byref(as_tensor(input)), _dtype(input), C.byref(as_tensor(output)), _dtype(output), int(reversed)))

    @staticmethod
    def channel_mix(cursors, state, r, v, x, state_view=None):
        _check(lib().wrq_channel_mix(_stream(), C.byref(as_tensor(cursors)), C.byref(as_view(state, state_view)), C.byref(as_tensor(r)),
                                     C.byref(as_tensor(v)), C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def time_mix_v4(cursors, time_decay, time_first, state, k, v, r, x, state_view=None):
        _check(lib().wrq_time_mix_v4(_stream(), C.byref(as_tensor(cursors)), C.byref(as_tensor(time_decay)), C.byref(as_tensor(time_first)),
                                     C.byref(as_view(state, state_view)), C.byref(as_tensor(k)), C.byref(as_tensor(v)), C.byref(as_tensor(r)),
                                     C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def time_mix_v5(cursors, time_decay, time_first, state, k, v, r, x, state_view=None):
        _check(lib().wrq_time_mix_v5(_stream(), C.byref(as_tensor(cursors)), C.byref(as_tensor(time_decay)), C.byref(as_tensor(time_first)),
                                     C.byref(as_view(state, state_view)), C.byref(as_tensor(k)), C.byref(as_tensor(v)), C.byref(as_tensor(r)),
                                     C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def time_mix_v6(cursors, time_decay, time_first, state, k, v, r, x, state_view=None):
        _check(lib().wrq_time_mix_v6(_stream(), C.byref(as_tensor(cursors)), C.byref(as_tensor(time_decay)), C.byref(as_tensor(time_first)),
                                     C.byref(as_view(state, state_view)), C.byref(as_tensor(k)), C.byref(as_tensor(v)), C.byref(as_tensor(r)),
                                     C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def recenter(x):
        _check(lib().wrq_recenter(_stream(), C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def rms_norm(w, b, x, eps):
        _check(lib().wrq_rms_norm(_stream(), C.byref(as_tensor(w)), C.byref(as_tensor(b)), C.byref(as_tensor(x)), _dtype(x), eps))

    @staticmethod
    def broadcast(input, output, input_view=None, output_view=None):
        _check(lib().wrq_broadcast(_stream(), C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view))))

    @staticmethod
    def blend(factor, input, output):
        _check(lib().wrq_blend(_stream(), C.byref(as_tensor(factor)), C.byref(as_tensor(input)), _dtype(input), C.byref(as_tensor(output)), _dtype(output)))

    @staticmethod
    def blend_lora(factor, xa, xb, output, xa_view=None, xb_view=None, output_view=None):
        _check(lib().wrq_blend_lora(_stream(), C.byref(as_tensor(factor)), C.byref(as_view(xa, xa_view)), C.byref(as_view(xb, xb_view)),
                                    C.byref(as_view(output, output_view))))

    @staticmethod
    def l2_norm(x, eps):
        _check(lib().wrq_l2_norm(_stream(), C.byref(as_tensor(x)), _dtype(x), eps))

    @staticmethod
    def control_k_v7(p, a, k, a_view=None, k_view=None):
        _check(lib().wrq_control_k_v7(_stream(), C.byref(as_tensor(p)), C.byref(as_view(a, a_view)), C.byref(as_view(k, k_view))))

    @staticmethod
    def time_mix_v7(cursors, state, r, w, n, x, state_view=None):
        _check(lib().wrq_time_mix_v7(_stream(), C.byref(as_tensor(cursors)), C.byref(as_view(state, state_view)), C.byref(as_tensor(r)),
                                     C.byref(as_tensor(w)), C.byref(as_tensor(n)), C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def time_first_v7(u, r, n, x):
        _check(lib().wrq_time_first_v7(_stream(), C.byref(as_tensor(u)), C.byref(as_tensor(r)), C.byref(as_tensor(n)), C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def channel_mix_v7(cursors, state, v, x, state_view=None):
        _check(lib().wrq_channel_mix_v7(_stream(), C.byref(as_tensor(cursors)), C.byref(as_view(state, state_view)), C.byref(as_tensor(v)),
                                        C.byref(as_tensor(x)), _dtype(x)))

    @staticmethod
    def lerp(input, output, factor, reversed=False, input_view=None, output_view=None, factor_view=None):
        _check(lib().wrq_lerp(_stream(), C.byref(as_view(input, input_view)), C.byref(as_view(output, output_view)),
                              C.byref(as_view(factor, factor_view)), int(reversed)))


class FusedV6:
    """The fused forms of a v6 layer's small ops (`wrq_v6_*`); arguments are contiguous torch tensors."""

    @staticmethod
    def _p(t):
        return None if t is None else C.c_void_p(t.data_ptr())

    @staticmethod
    def pre(Cn, A, cursors, x, add, x_out, ln_w, ln_b, eps, state, state_view, factors, ln_out, shifts):
        p = FusedV6._p
        _check(lib().wrq_v6_pre(_stream(), Cn, A, p(cursors), p(x), p(add), p(x_out), p(ln_w), p(ln_b), eps, C.byref(as_view(state, state_view)), len(factors),
                                p(factors[0]), p(factors[1] if len(factors) > 1 else None), p(ln_out), p(shifts[0]), p(shifts[1] if len(shifts) > 1 else None)))

    @staticmethod
    def time_mix(Cn, A, lora_size, cursors, lora, w2, time_mix, state, state_view, att_x, att_sx):
        p = FusedV6._p
        _check(lib().wrq_v6_time_mix(_stream(), Cn, A, lora_size, p(cursors), p(lora), p(w2), p(time_mix), C.byref(as_view(state, state_view)), p(att_x), p(att_sx)))

    @staticmethod
    def decay(Cn, A, lora_size, lora, w2, time_decay, out):
        p = FusedV6._p
        _check(lib().wrq_v6_decay(_stream(), Cn, A, lora_size, p(lora), p(w2), p(time_decay), p(out)))

    @staticmethod
    def wkv_gate(S, H, A, cursors, time_decay, time_first, state, state_view, k, v, r, g, gn_w, gn_b, eps, att_x):
        p = FusedV6._p
        _check(lib().wrq_v6_wkv_gate(_stream(), S, H, A, p(cursors), p(time_decay), p(time_first), C.byref(as_view(state, state_view)), p(k), p(v), p(r), p(g),
                                     p(gn_w), p(gn_b), eps, p(att_x)))

    @staticmethod
    def post_ffn(Cn, A, cursors, state, state_view, r, v, ffn_x, x_in, x_out, rescale):
        p = FusedV6._p
        _check(lib().wrq_v6_post_ffn(_stream(), Cn, A, p(cursors), C.byref(as_view(state, state_view)), p(r), p(v), p(ffn_x), p(x_in), p(x_out), int(rescale)))


def matmul_vec_group(ops):
    """Independent decode products in shared launches (``wrq_matmul_vec_*_group``).

    ``ops``: list of ``(matrix: Matrix, input, output, act, sparse, views: dict)``, all Int8 or all Fp4.
    """
    if not ops:
        return
    kind = ops[0][0].kind
    keep = []  # ctypes structs must outlive the call
    if kind == "Int8":
        arr = (CVecInt8Op * len(ops))()
        for k, (m, x, out, act, sparse, views) in enumerate(ops):
            assert m.kind == kind
            t = (as_tensor(m.w), as_tensor(m.m), as_view(x, views.get("input_view")), as_view(out, views.get("output_view")))
            keep.append(t)
            arr[k] = CVecInt8Op(C.pointer(t[0]), C.pointer(t[1]), C.pointer(t[2]), C.pointer(t[3]), act, int(sparse))
        _check(lib().wrq_matmul_vec_int8_group(_stream(), arr, len(ops)))
    else:
        arr = (CVecNf4Op * len(ops))()
        for k, (m, x, out, act, sparse, views) in enumerate(ops):
            assert m.kind == kind
            t = (as_tensor(m.w), as_tensor(m.q), as_tensor(m.m), as_view(x, views.get("input_view")), as_view(out, views.get("output_view")))
            keep.append(t)
            arr[k] = CVecNf4Op(C.pointer(t[0]), C.pointer(t[1]), C.pointer(t[2]), C.pointer(t[3]), C.pointer(t[4]), act, int(sparse))
        _check(lib().wrq_matmul_vec_nf4_group(_stream(), arr, len(ops)))


class Matrix:
    """``Matrix::{Fp16, Int8, Fp4}`` (src/tensor/matrix.rs:29-44, :80-94): weights plus scales."""

    def __init__(self, kind, w, m, q=None):
        self.kind, self.w, self.m, self.q = kind, w, m, q

    @staticmethod
    def quant_u8(matrix):
        """Matrix::quant_u8, src/tensor/matrix.rs:162-178."""
        import torch

        w = torch.empty(matrix.shape, dtype=torch.uint8, device=matrix.device)
        n = (matrix.numel() * 2 + INT8_BLOCK_SIZE - 1) // INT8_BLOCK_SIZE
        m = torch.empty(n, dtype=torch.float16, device=matrix.device)
        TensorOp.quantize_mat_int8(matrix, m, w)
        return Matrix("Int8", w, m)

    @staticmethod
    def quant_nf4(matrix, quant=None):
        """Matrix::quant_nf4 / quant_sf4 (a caller-supplied table), src/tensor/matrix.rs:180-222."""
        import torch

        q = torch.tensor(NF4_QUANT if quant is None else quant, dtype=torch.float32, device=matrix.device)
        w = torch.empty(matrix.shape[:-1] + (matrix.shape[-1] // 2,), dtype=torch.uint8, device=matrix.device)
        n = (matrix.numel() + NF4_BLOCK_SIZE - 1) // NF4_BLOCK_SIZE
        m = torch.empty(n, dtype=torch.float16, device=matrix.device)
        TensorOp.quantize_mat_nf4(matrix, q, m, w)
        return Matrix("Fp4", w, m, q)

    @staticmethod
    def fp16(matrix):
        """Matrix::Fp16: the f16 tensor as it is."""
        return Matrix("Fp16", matrix, None)

    @staticmethod
    def quant_sf4(matrix, nu):
        """Matrix::quant_sf4, src/tensor/matrix.rs:202-222."""
        return Matrix.quant_nf4(matrix, quantile_student(nu))

    def matmul_vec_op(self, input, output, act=ACT_NONE, sparse=False, **views):
        if self.kind == "Fp16":
            TensorOp.matmul_vec_fp16(self.w, input, output, act, sparse, **views)
        elif self.kind == "Int8":
            TensorOp.matmul_vec_int8(self.w, self.m, input, output, act, sparse, **views)
        else:
            TensorOp.matmul_vec_nf4(self.w, self.q, self.m, input, output, act, sparse, **views)

    def matmul_mat_op(self, input, output, act=ACT_NONE, **views):
        if self.kind == "Fp16":
            TensorOp.matmul_mat_fp16(self.w, input, output, act, **views)
        elif self.kind == "Int8":
            TensorOp.matmul_mat_int8(self.w, self.m, input, output, act, **views)
        else:
            TensorOp.matmul_mat_nf4(self.w, self.q, self.m, input, output, act, **views)

    def matmul_op(self, input, output, act=ACT_NONE, turbo=False, **views):
        """Matrix::matmul_op, src/tensor/matrix.rs:136-147."""
        if turbo:
            self.matmul_mat_op(input, output, act, **views)
        else:
            self.matmul_vec_op(input, output, act, **views)

    def matmul_op_sparse(self, input, output, act=ACT_NONE, turbo=False, **views):
        """Matrix::matmul_op_sparse, src/tensor/matrix.rs:149-160."""
        if turbo:
            self.matmul_mat_op(input, output, act, **views)
        else:
            self.matmul_vec_op(input, output, act, sparse=True, **views)


def turbo(num_token):
    """Kernel choice of the model builders: chunk kernels iff T % 32 == 0 (src/runtime/v6.rs:568-570)."""
    return num_token % 32 == 0
