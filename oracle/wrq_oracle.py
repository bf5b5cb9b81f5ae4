"""numpy front end of the CPU oracle (``libwrq_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by tests, by the smoke check and by the
CPU-baseline leg of the benchmark, never by the library.

Tensors use the reference's shape order (x fastest): a matrix ``[K, R, B]`` is a
numpy array of shape ``(B, R, K)`` (or ``(R, K)`` for B = 1), an input ``[K, T, B]``
is ``(B, T, K)`` / ``(T, K)``, an output ``[R, T, B]`` is ``(B, T, R)`` / ``(T, R)``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwrq_oracle.so")

INT8_BLOCK = 128  # src/tensor/ops.rs:292
NF4_BLOCK = 64  # src/tensor/ops.rs:291

# src/tensor/matrix.rs:50-67 (identical literals at src/tensor/ops.rs:3096-3113)
NF4_QUANT = np.array(
    [
        -1.0,
        -0.6961928009986877,
        -0.5250730514526367,
        -0.39491748809814453,
        -0.28444138169288635,
        -0.18477343022823334,
        -0.09105003625154495,
        0.0,
        0.07958029955625534,
        0.16093020141124725,
        0.24611230194568634,
        0.33791524171829224,
        0.44070982933044434,
        0.5626170039176941,
        0.7229568362236023,
        1.0,
    ],
    dtype=np.float32,
)

ACT_NAMES = [
    "none",
    "squared_relu",
    "tanh",
    "stable_exp",
    "opposite_exp",
    "softplus",
    "sigmoid",
    "silu",
]


class View(C.Structure):
    """shape / stride (= parent shape) / offset; src/tensor/mod.rs:26-43."""

    _fields_ = [("shape", C.c_uint32 * 4), ("stride", C.c_uint32 * 4), ("offset", C.c_uint32 * 4)]

    @classmethod
    def full(cls, x, y=1, z=1, w=1):
        return cls((x, y, z, w), (x, y, z, w), (0, 0, 0, 0))

    @classmethod
    def make(cls, shape, stride, offset):
        pad = lambda s, f: tuple(s) + (f,) * (4 - len(s))
        return cls(pad(shape, 1), pad(stride, 1), pad(offset, 0))


def build():
    """Compile the oracle with gcc (always recompiles)."""
    subprocess.run(["make", "-C", _HERE, "-B", "libwrq_oracle.so"], check=True, capture_output=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        vp, u32, i32, sz = C.c_void_p, C.c_uint32, C.c_int, C.c_size_t
        VP = C.POINTER(View)
        L.wrq_oracle_quant_int8.argtypes = [vp, sz, vp, vp]
        L.wrq_oracle_quant_int8.restype = C.c_uint64
        L.wrq_oracle_quant_nf4.argtypes = [vp, sz, vp, vp, vp]
        L.wrq_oracle_quant_nf4.restype = None
        L.wrq_oracle_matmul_vec_int8.argtypes = [vp, vp, u32, u32, u32, vp, VP, i32, vp, VP, i32, i32, i32]
        L.wrq_oracle_matmul_vec_int8.restype = None
        L.wrq_oracle_matmul_vec_nf4.argtypes = [vp, vp, vp, u32, u32, u32, vp, VP, i32, vp, VP, i32, i32, i32]
        L.wrq_oracle_matmul_vec_nf4.restype = None
        L.wrq_oracle_matmul_mat_int8.argtypes = [vp, VP, vp, vp, VP, i32, vp, VP, i32, i32]
        L.wrq_oracle_matmul_mat_int8.restype = None
        L.wrq_oracle_matmul_mat_nf4.argtypes = [vp, VP, vp, vp, vp, VP, i32, vp, VP, i32, i32]
        L.wrq_oracle_matmul_mat_nf4.restype = None
        L.wrq_oracle_matmul_vec_fp16.argtypes = [vp, u32, u32, u32, vp, VP, i32, vp, VP, i32, i32, i32]
        L.wrq_oracle_matmul_vec_fp16.restype = None
        L.wrq_oracle_matmul_mat_fp16.argtypes = [vp, VP, vp, VP, i32, vp, VP, i32, i32]
        L.wrq_oracle_matmul_mat_fp16.restype = None
        L.wrq_oracle_f32_to_f16.argtypes = [vp, vp, sz]
        L.wrq_oracle_f16_to_f32.argtypes = [vp, vp, sz]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _dt(a):
    if a.dtype == np.float16:
        return 0
    if a.dtype == np.float32:
        return 1
    raise TypeError(a.dtype)


def _act(act):
    return act if isinstance(act, int) else ACT_NAMES.index(act)


def f32_to_f16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.float16)
    lib().wrq_oracle_f32_to_f16(_p(x), _p(out), x.size)
    return out


def f16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.float16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().wrq_oracle_f16_to_f32(_p(x), _p(out), x.size)
    return out


def quant_int8(w):
    """w: f16 array (any shape, size % 128 == 0) -> (u8 same shape, minmax f16 [2*n/128], flagged)."""
    w = np.ascontiguousarray(w, dtype=np.float16)
    assert w.size % INT8_BLOCK == 0
    out = np.empty(w.shape, dtype=np.uint8)
    minmax = np.empty(2 * w.size // INT8_BLOCK, dtype=np.float16)
    flagged = lib().wrq_oracle_quant_int8(_p(w), w.size, _p(minmax), _p(out))
    return out, minmax, int(flagged)


def quant_nf4(w, quant=NF4_QUANT):
    """w: f16 array (..., K) with size % 64 == 0 -> (u8 (..., K/2), absmax f16 [n/64])."""
    w = np.ascontiguousarray(w, dtype=np.float16)
    assert w.size % NF4_BLOCK == 0 and w.shape[-1] % 2 == 0
    quant = np.ascontiguousarray(quant, dtype=np.float32)
    out = np.empty(w.shape[:-1] + (w.shape[-1] // 2,), dtype=np.uint8)
    absmax = np.empty(w.size // NF4_BLOCK, dtype=np.float16)
    lib().wrq_oracle_quant_nf4(_p(w), w.size, _p(quant), _p(absmax), _p(out))
    return out, absmax


def _shape3(a):
    """numpy (B, Y, X) / (Y, X) -> (X, Y, B)."""
    if a.ndim == 2:
        return a.shape[1], a.shape[0], 1
    assert a.ndim == 3
    return a.shape[2], a.shape[1], a.shape[0]


def _mk_out(R, T, B, out_dtype, out, dst):
    if out is None:
        out = np.zeros((B, T, R), dtype=out_dtype)
        dst = View.full(R, T, B)
    return out, dst


def matmul_vec_int8(w, minmax, x, out_dtype=np.float16, act=0, sparse=False, src=None, out=None, dst=None):
    K, R, B = _shape3(w)
    x = np.ascontiguousarray(x)
    if src is None:
        src = View.full(*_shape3(x))
    T = src.shape[1]
    out, dst = _mk_out(R, T, B, out_dtype, out, dst)
    lib().wrq_oracle_matmul_vec_int8(
        _p(w), _p(minmax), K, R, B, _p(x), C.byref(src), _dt(x), _p(out), C.byref(dst), _dt(out), _act(act), int(sparse)
    )
    return out


def matmul_vec_nf4(w, absmax, x, quant=NF4_QUANT, out_dtype=np.float16, act=0, sparse=False, src=None, out=None, dst=None):
    K2, R, B = _shape3(w)
    K = K2 * 2
    x = np.ascontiguousarray(x)
    quant = np.ascontiguousarray(quant, dtype=np.float32)
    if src is None:
        src = View.full(*_shape3(x))
    T = src.shape[1]
    out, dst = _mk_out(R, T, B, out_dtype, out, dst)
    lib().wrq_oracle_matmul_vec_nf4(
        _p(w), _p(quant), _p(absmax), K, R, B, _p(x), C.byref(src), _dt(x), _p(out), C.byref(dst), _dt(out), _act(act), int(sparse)
    )
    return out


def matmul_mat_int8(w, minmax, x, out_dtype=np.float16, act=0, va=None, src=None, out=None, dst=None):
    K, R, B = _shape3(w)
    x = np.ascontiguousarray(x)
    if va is None:
        va = View.full(K, R, B)
    if src is None:
        src = View.full(*_shape3(x))
    out, dst = _mk_out(va.shape[1], src.shape[1], va.shape[2], out_dtype, out, dst)
    lib().wrq_oracle_matmul_mat_int8(
        _p(w), C.byref(va), _p(minmax), _p(x), C.byref(src), _dt(x), _p(out), C.byref(dst), _dt(out), _act(act)
    )
    return out


def matmul_mat_nf4(w, absmax, x, quant=NF4_QUANT, out_dtype=np.float16, act=0, va=None, src=None, out=None, dst=None):
    K2, R, B = _shape3(w)
    x = np.ascontiguousarray(x)
    quant = np.ascontiguousarray(quant, dtype=np.float32)
    if va is None:
        va = View.full(K2, R, B)
    if src is None:
        src = View.full(*_shape3(x))
    out, dst = _mk_out(va.shape[1], src.shape[1], va.shape[2], out_dtype, out, dst)
    lib().wrq_oracle_matmul_mat_nf4(
        _p(w), C.byref(va), _p(quant), _p(absmax), _p(x), C.byref(src), _dt(x), _p(out), C.byref(dst), _dt(out), _act(act)
    )
    return out


def matmul_vec_fp16(w, x, out_dtype=np.float16, act=0, sparse=False, src=None, out=None, dst=None):
    """matmul_vec_fp16: `w` f16 (B, R, K) or (R, K)."""
    K, R, B = _shape3(w)
    w = np.ascontiguousarray(w, dtype=np.float16)
    x = np.ascontiguousarray(x)
    if src is None:
        src = View.full(*_shape3(x))
    T = src.shape[1]
    out, dst = _mk_out(R, T, B, out_dtype, out, dst)
    lib().wrq_oracle_matmul_vec_fp16(
        _p(w), K, R, B, _p(x), C.byref(src), _dt(x), _p(out), C.byref(dst), _dt(out), _act(act), int(sparse)
    )
    return out


def matmul_mat_fp16(w, x, out_dtype=np.float16, act=0, va=None, src=None, out=None, dst=None):
    K, R, B = _shape3(w)
    w = np.ascontiguousarray(w, dtype=np.float16)
    x = np.ascontiguousarray(x)
    if va is None:
        va = View.full(K, R, B)
    if src is None:
        src = View.full(*_shape3(x))
    out, dst = _mk_out(va.shape[1], src.shape[1], va.shape[2], out_dtype, out, dst)
    lib().wrq_oracle_matmul_mat_fp16(
        _p(w), C.byref(va), _p(x), C.byref(src), _dt(x), _p(out), C.byref(dst), _dt(out), _act(act)
    )
    return out
