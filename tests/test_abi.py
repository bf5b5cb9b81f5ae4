"""CPU-side checks of the C ABI: the library loads, exports what include/wrq.h declares,
and rejects bad operands before touching a device (no compute calls here)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "wrq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wrq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(wrq):
    L = wrq.lib()
    names = declared_functions()
    assert set(wrq.EXPORTS) == set(names)
    for n in names:
        assert hasattr(L, n), n
    assert L.wrq_abi_version() == 1
    assert L.wrq_abi_minor() >= 3  # entry points were added since minor 0; signatures never changed
    assert L.wrq_status_string(0) == b"ok"
    assert L.wrq_status_string(1) == b"tensor shape not match"


def test_struct_layouts_match_the_header(wrq):
    # wrq_view is the reference's 48-byte View uniform (src/tensor/mod.rs:26-43)
    assert C.sizeof(wrq.CView) == 48
    assert C.sizeof(wrq.CTensor) == 24
    assert C.sizeof(wrq.CTensorView) == 8 + 48 + 8
    assert wrq.ACTIVATIONS[1] == "squared_relu" and len(wrq.ACTIVATIONS) == 8


FAKE = 0x10000  # never dereferenced: every call below fails its checks first


def T(wrq, shape, ptr=FAKE):
    return wrq.CTensor(ptr, tuple(shape))


def V(wrq, shape, stride=None, offset=(0, 0, 0, 0), dtype=0, ptr=FAKE):
    return wrq.CTensorView(ptr, wrq.CView(tuple(shape), tuple(stride or shape), tuple(offset)), dtype)


def err(wrq):
    return wrq.lib().wrq_last_error().decode()


def test_shape_errors_read_like_the_reference(wrq):
    L = wrq.lib()
    K, R, Tn = 256, 8, 1
    ok_mm = T(wrq, (2 * K * R // 128, 1, 1, 1))
    # minmax of the wrong length -> TensorErrorKind::Shape(got, want) (src/tensor/ops.rs:809)
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (7, 1, 1, 1))),
                              C.byref(V(wrq, (K, Tn, 1, 1))), C.byref(V(wrq, (R, Tn, 1, 1))), 0, 0)
    assert s == wrq.ERR_SHAPE
    assert err(wrq) == "tensor shape not match: (7, 1, 1, 1) vs. (32, 1, 1, 1)"
    # matrix vs input K mismatch (ops.rs:810)
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(ok_mm),
                              C.byref(V(wrq, (K // 2, Tn, 1, 1))), C.byref(V(wrq, (R, Tn, 1, 1))), 0, 0)
    assert s == wrq.ERR_SHAPE and "(256, 8, 1, 1) vs. (128, 8, 1, 1)" in err(wrq)
    # token count mismatch between input and output (ops.rs:811)
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(ok_mm),
                              C.byref(V(wrq, (K, 2, 1, 1))), C.byref(V(wrq, (R, 1, 1, 1))), 0, 0)
    assert s == wrq.ERR_SHAPE and "(256, 2, 1, 1) vs. (256, 1, 1, 1)" in err(wrq)
    # nf4: matrix holds K/2 bytes per row, absmax one per 64 (ops.rs:910-912)
    s = L.wrq_matmul_vec_nf4(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (16, 1, 1, 1))),
                             C.byref(T(wrq, (K * R // 64, 1, 1, 1))), C.byref(V(wrq, (K, Tn, 1, 1))),
                             C.byref(V(wrq, (R, Tn, 1, 1))), 0, 0)
    assert s == wrq.ERR_SHAPE
    # quantize: input and output shapes must agree (ops.rs:2405), minmax = 2 * ceil(len / 128) (ops.rs:2402-2403)
    s = L.wrq_quantize_mat_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(ok_mm), C.byref(T(wrq, (K, R + 4, 1, 1))))
    assert s == wrq.ERR_SHAPE
    s = L.wrq_quantize_mat_nf4(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (16, 1, 1, 1))),
                               C.byref(T(wrq, (K * R // 64 + 1, 1, 1, 1))), C.byref(T(wrq, (K // 2, R, 1, 1))))
    assert s == wrq.ERR_SHAPE and "(33, 1, 1, 1) vs. (32, 1, 1, 1)" in err(wrq)


def test_unchecked_preconditions_of_the_reference_become_errors(wrq):
    L = wrq.lib()
    K = 256
    # R % 4 != 0: the reference's grid R/4 silently drops rows (ops.rs:884)
    R = 6
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 1, 1, 1))), C.byref(V(wrq, (R, 1, 1, 1))), 0, 0)
    assert s == wrq.ERR_ALIGNMENT
    # len % 128 != 0
    s = L.wrq_quantize_mat_int8(None, C.byref(T(wrq, (100, 3, 1, 1))), C.byref(T(wrq, (6, 1, 1, 1))), C.byref(T(wrq, (100, 3, 1, 1))))
    assert s == wrq.ERR_ALIGNMENT
    # chunk kernels: T % 4 (ops.rs:1068-1069)
    R = 8
    s = L.wrq_matmul_mat_int8(None, C.byref(V(wrq, (K, R, 1, 1))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 6, 1, 1))), C.byref(V(wrq, (R, 6, 1, 1))), 0)
    assert s == wrq.ERR_ALIGNMENT
    # sliced matrix views are refused, not mis-executed
    s = L.wrq_matmul_mat_int8(None, C.byref(V(wrq, (K, R, 1, 1), stride=(K, 2 * R, 1, 1))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 8, 1, 1))), C.byref(V(wrq, (R, 8, 1, 1))), 0)
    assert s == wrq.ERR_UNSUPPORTED and "sliced matrix views" in err(wrq)
    # ... also a slice that starts inside the parent (the reference's scale indexing has no consistent meaning for it)
    s = L.wrq_matmul_mat_int8(None, C.byref(V(wrq, (K, R, 1, 1), stride=(K, R, 2, 1), offset=(0, 0, 1, 0))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 8, 1, 1))), C.byref(V(wrq, (R, 8, 1, 1))), 0)
    assert s == wrq.ERR_UNSUPPORTED and "offset 1 along axis 2" in err(wrq)
    # view outside its parent
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 1, 1, 1), stride=(K, 1, 5, 1), offset=(0, 0, 5, 0))), C.byref(V(wrq, (R, 1, 1, 1))), 0, 0)
    assert s == wrq.ERR_SHAPE and "out of range" in err(wrq)
    # dtype outside {F16, F32}, null pointers, unknown activation
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 1, 1, 1), dtype=5)), C.byref(V(wrq, (R, 1, 1, 1))), 0, 0)
    assert s == wrq.ERR_TYPE and err(wrq) == "data type mismatch"
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1), ptr=0)), C.byref(T(wrq, (4, 1, 1, 1))),
                              C.byref(V(wrq, (K, 1, 1, 1))), C.byref(V(wrq, (R, 1, 1, 1))), 0, 0)
    assert s == wrq.ERR_NULL
    s = L.wrq_matmul_vec_int8(None, None, None, None, None, 0, 0)
    assert s == wrq.ERR_NULL
    s = L.wrq_matmul_vec_int8(None, C.byref(T(wrq, (K, R, 1, 1))), C.byref(T(wrq, (2 * K * R // 128, 1, 1, 1))),
                              C.byref(V(wrq, (K, 1, 1, 1))), C.byref(V(wrq, (R, 1, 1, 1))), 99, 0)
    assert s == wrq.ERR_UNSUPPORTED


def test_missing_library_fails_loudly(wrq, monkeypatch, tmp_path):
    monkeypatch.setattr(wrq, "_lib", None)
    monkeypatch.setattr(wrq, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(FileNotFoundError, match="no CPU or eager fallback"):
        wrq.lib()


def test_sf4_table_matches_student_quantiles():
    # Float4Quant::new_student (src/tensor/matrix.rs:29-44).  The reference takes the quantile from
    # the statrs crate, which is not available here: the table is checked against scipy's
    # Student-t quantile instead (equal far inside f32) -- bit parity with statrs is unpinned.
    import importlib

    import numpy as np
    from scipy import stats

    wrq = importlib.import_module("web-rwkv_amd")
    delta = (1 / 32 + 1 / 30) / 2
    probs = [delta + (0.5 - delta) / 7 * i for i in range(7)] + [0.5 + (0.5 - delta) / 8 * i for i in range(9)]
    for nu in (1.0, 2.5, 5.0, 30.0):
        q = np.array(wrq.quantile_student(nu), dtype=np.float32)
        ref = stats.t.ppf(probs, nu)
        ref = (ref / ref.max()).astype(np.float32)
        assert q.shape == (16,) and q[0] == -1.0 and q[7] == 0.0 and q[15] == 1.0
        assert (np.diff(q) > 0).all()
        assert np.abs(q.astype(np.float64) - ref.astype(np.float64)).max() <= 1.2e-7
