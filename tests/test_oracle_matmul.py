"""Pins the oracle's products (CPU only) against textbook float64 matmul on independently
dequantised weights, plus structural invariants (views, sparse flag, vec == mat)."""
import numpy as np
import pytest

from helpers import (ACTS, NF4_QUANT, assert_close, gen_f16, int8_dequant64, nf4_dequant64,
                     truth_matmul)

F32_EPS = 2e-4  # f32 accumulation over K <= 2560 against float64


def _int8_case(oracle, rng, K, R, T, wstd=0.02, xstd=1.0):
    w = gen_f16(rng, (R, K), wstd)
    x = gen_f16(rng, (T, K), xstd)
    u8, minmax, _ = oracle.quant_int8(w)
    return u8, minmax, x, int8_dequant64(u8, minmax)


def _nf4_case(oracle, rng, K, R, T, wstd=0.02, xstd=1.0):
    w = gen_f16(rng, (R, K), wstd)
    x = gen_f16(rng, (T, K), xstd)
    packed, absmax = oracle.quant_nf4(w)
    return packed, absmax, x, nf4_dequant64(packed, absmax)


# (C, R, T) of the reference's tests (ops.rs:3058-3059, :3253-3254) plus small ragged-K cases
SHAPES = [(320, 64, 320), (2560, 2048, 64), (128, 4, 1), (384, 8, 3), (1024, 16, 5)]


@pytest.mark.parametrize("K,R,T", SHAPES)
def test_int8_products_against_float64(oracle, K, R, T):
    rng = np.random.default_rng(K * 31 + R)
    # reference-test scale: weights and inputs ~ 10*(U-0.5) -> outputs of magnitude ~100
    u8, minmax, x, wdeq = _int8_case(oracle, rng, K, R, T, wstd=2.9, xstd=2.9)
    truth = truth_matmul(wdeq, x)
    vec = oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float32)[0]
    scale = np.abs(truth).max()
    assert np.abs(vec - truth).max() <= F32_EPS * scale
    if T % 4 == 0:
        mat = oracle.matmul_mat_int8(u8, minmax, x, out_dtype=np.float32)[0]
        assert np.abs(mat - truth).max() <= F32_EPS * scale
    # f16 output = RNE of the f32 output
    vec16 = oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float16)[0]
    with np.errstate(over="ignore"):
        assert np.array_equal(vec16.view(np.uint16), vec.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("K,R,T", SHAPES)
def test_nf4_products_against_float64(oracle, K, R, T):
    if K % 64:
        pytest.skip("nf4 blocks need K % 64 == 0")
    rng = np.random.default_rng(K * 17 + R)
    packed, absmax, x, wdeq = _nf4_case(oracle, rng, K, R, T, wstd=1.0, xstd=0.58)
    truth = truth_matmul(wdeq, x)
    vec = oracle.matmul_vec_nf4(packed, absmax, x, out_dtype=np.float32)[0]
    scale = np.abs(truth).max()
    assert np.abs(vec - truth).max() <= F32_EPS * scale
    if T % 4 == 0:
        mat = oracle.matmul_mat_nf4(packed, absmax, x, out_dtype=np.float32)[0]
        assert np.abs(mat - truth).max() <= F32_EPS * scale


def test_transposed_operand_would_fail(oracle):
    # a square case where W and W^T give different answers: guards the row/column convention
    rng = np.random.default_rng(5)
    u8, minmax, x, wdeq = _int8_case(oracle, rng, 128, 128, 4)
    vec = oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float32)[0]
    good = truth_matmul(wdeq, x)
    bad = x.astype(np.float64) @ wdeq
    assert np.abs(vec - good).max() < 1e-3 * np.abs(good).max()
    assert np.abs(vec - bad).max() > 0.1 * np.abs(good).max()


@pytest.mark.parametrize("act", list(ACTS))
def test_activations(oracle, act):
    rng = np.random.default_rng(11)
    u8, minmax, x, wdeq = _int8_case(oracle, rng, 256, 16, 4, wstd=0.1)
    packed, absmax, x2, wdeq2 = _nf4_case(oracle, rng, 256, 16, 4, wstd=0.1)
    for got, truth in [
        (oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float32, act=act)[0], truth_matmul(wdeq, x, act)),
        (oracle.matmul_mat_int8(u8, minmax, x, out_dtype=np.float32, act=act)[0], truth_matmul(wdeq, x, act)),
        (oracle.matmul_vec_nf4(packed, absmax, x2, out_dtype=np.float32, act=act)[0], truth_matmul(wdeq2, x2, act)),
        (oracle.matmul_mat_nf4(packed, absmax, x2, out_dtype=np.float32, act=act)[0], truth_matmul(wdeq2, x2, act)),
    ]:
        assert_close(got, truth, 1e-4, act)
    # tanh saturates to exactly 1 above 42 (ops.rs:232-234)
    if act == "tanh":
        big = np.full((1, 256), 60.0, dtype=np.float16)
        w = np.full((4, 256), 1.0, dtype=np.float16)
        w[:, 0] = 0.5
        u8b, mmb, _ = oracle.quant_int8(w)
        assert (oracle.matmul_vec_int8(u8b, mmb, big, out_dtype=np.float32, act=act) == 1.0).all()


def test_sparse_flag_does_not_change_results(oracle):
    rng = np.random.default_rng(13)
    u8, minmax, x, _ = _int8_case(oracle, rng, 512, 32, 3)
    packed, absmax, x2, _ = _nf4_case(oracle, rng, 512, 32, 3)
    x = x.copy(); x2 = x2.copy()
    x[:, 64:256] = 0  # whole groups of zeros, as squared-relu outputs have
    x2[:, 128:384] = 0
    a = oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float32, sparse=False)
    b = oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float32, sparse=True)
    assert np.array_equal(a, b)
    a = oracle.matmul_vec_nf4(packed, absmax, x2, out_dtype=np.float32, sparse=False)
    b = oracle.matmul_vec_nf4(packed, absmax, x2, out_dtype=np.float32, sparse=True)
    assert np.array_equal(a, b)


def test_offset_views_equal_contiguous_copies(oracle):
    # v6 call sites pass att_sx.view(.., .., i, ..) of a [C, T, 5] tensor (src/runtime/v6.rs:806-829)
    rng = np.random.default_rng(17)
    K, R, T = 256, 32, 4
    u8, minmax, _, _ = _int8_case(oracle, rng, K, R, T)
    packed, absmax, _, _ = _nf4_case(oracle, rng, K, R, T)
    parent = gen_f16(rng, (5, T, K), 1.0)
    outp = np.zeros((3, T + 2, R), dtype=np.float32)
    for i in (1, 4):
        src = oracle.View.make((K, T, 1), (K, T, 5), (0, 0, i))
        dst = oracle.View.make((R, T, 1), (R, T + 2, 3), (0, 1, 2))
        for fn, args in [(oracle.matmul_vec_int8, (u8, minmax)), (oracle.matmul_vec_nf4, (packed, absmax)),
                         (oracle.matmul_mat_int8, (u8, minmax)), (oracle.matmul_mat_nf4, (packed, absmax))]:
            outp[:] = -7.0
            fn(*args, parent, out_dtype=np.float32, src=src, out=outp, dst=dst)
            want = fn(*args, np.ascontiguousarray(parent[i]), out_dtype=np.float32)[0]
            assert np.array_equal(outp[2, 1:1 + T], want)
            rest = outp.copy(); rest[2, 1:1 + T] = -7.0
            assert (rest == -7.0).all()  # nothing outside the view is written


def test_f32_input_and_batch_axis(oracle):
    rng = np.random.default_rng(19)
    K, R, T, B = 256, 8, 2, 3
    w = gen_f16(rng, (B, R, K), 0.05)
    x = rng.standard_normal((B, T, K), dtype=np.float32)
    u8, minmax, _ = oracle.quant_int8(w)
    packed, absmax = oracle.quant_nf4(w)
    t8 = np.stack([truth_matmul(int8_dequant64(u8, minmax)[b], x[b]) for b in range(B)])
    t4 = np.stack([truth_matmul(nf4_dequant64(packed, absmax)[b], x[b]) for b in range(B)])
    assert_close(oracle.matmul_vec_int8(u8, minmax, x, out_dtype=np.float32), t8, 1e-4)
    assert_close(oracle.matmul_vec_nf4(packed, absmax, x, out_dtype=np.float32), t4, 1e-4)
    x4 = np.concatenate([x, x], axis=1)
    assert_close(oracle.matmul_mat_int8(u8, minmax, x4, out_dtype=np.float32)[:, :T], t8, 1e-4)
    assert_close(oracle.matmul_mat_nf4(packed, absmax, x4, out_dtype=np.float32)[:, :T], t4, 1e-4)


def test_row_permutation_permutes_outputs(oracle):
    rng = np.random.default_rng(23)
    K, R, T = 256, 16, 2
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    perm = rng.permutation(R)
    u8, mm, _ = oracle.quant_int8(w)
    u8p, mmp, _ = oracle.quant_int8(w[perm])
    a = oracle.matmul_vec_int8(u8, mm, x, out_dtype=np.float32)[0]
    b = oracle.matmul_vec_int8(u8p, mmp, x, out_dtype=np.float32)[0]
    assert np.array_equal(a[:, perm], b)


# ------------------------------------------------------------ plain f16 weights (matmul_*_fp16)


@pytest.mark.parametrize("K,R,T", [(320, 64, 320), (2560, 96, 4), (512, 128, 1), (36, 8, 5)], ids=str)
def test_fp16_products_against_float64(oracle, K, R, T):
    rng = np.random.default_rng(23 + K + R + T)
    w = gen_f16(rng, (R, K), 0.05)
    x = gen_f16(rng, (T, K), 1.0)
    truth = x.astype(np.float64) @ w.astype(np.float64).T
    assert_close(oracle.matmul_vec_fp16(w, x, out_dtype=np.float32)[0], truth, 1e-5, "vec f32 out")
    assert_close(oracle.matmul_vec_fp16(w, x)[0], truth, 1e-3, "vec f16 out")
    if T % 4 == 0:
        assert_close(oracle.matmul_mat_fp16(w, x, out_dtype=np.float32)[0], truth, 1e-5, "mat f32 out")
    # a transposed or row-shuffled weight operand must not pass
    wrong = x.astype(np.float64) @ np.roll(w, 1, axis=0).astype(np.float64).T
    assert not np.allclose(oracle.matmul_vec_fp16(w, x, out_dtype=np.float32)[0], wrong, atol=1e-3)


def test_fp16_views_batch_activation_and_f32_input(oracle):
    rng = np.random.default_rng(29)
    K, R, T, B = 256, 16, 4, 2
    w = gen_f16(rng, (B, R, K), 0.05)
    x = rng.standard_normal((B, T, K), dtype=np.float32)
    truth = np.einsum("btk,brk->btr", x.astype(np.float64), w.astype(np.float64))
    for act, fn in ACTS.items():
        assert_close(oracle.matmul_vec_fp16(w, x, out_dtype=np.float32, act=act), fn(truth), 2e-5, f"vec act {act}")
        assert_close(oracle.matmul_mat_fp16(w, x, out_dtype=np.float32, act=act), fn(truth), 2e-5, f"mat act {act}")
    # offset views, as the att_sx call sites use them (src/runtime/v6.rs:806-829)
    parent = gen_f16(rng, (5, T, K), 1.0)
    outp = np.full((3, T + 2, R), -7.0, dtype=np.float32)
    src = oracle.View.make((K, T, 1), (K, T, 5), (0, 0, 3))
    dst = oracle.View.make((R, T, 1), (R, T + 2, 3), (0, 1, 2))
    for fn in (oracle.matmul_vec_fp16, oracle.matmul_mat_fp16):
        outp[:] = -7.0
        fn(w[0], parent, out_dtype=np.float32, src=src, out=outp, dst=dst)
        want = fn(w[0], np.ascontiguousarray(parent[3]), out_dtype=np.float32)[0]
        assert np.array_equal(outp[2, 1:1 + T], want)
        rest = outp.copy(); rest[2, 1:1 + T] = -7.0
        assert (rest == -7.0).all()
    # sparse flag: skipping all-zero groups changes nothing
    xs = gen_f16(rng, (T, K), 1.0); xs[:, 64:192] = 0
    assert np.array_equal(oracle.matmul_vec_fp16(w[0], xs, sparse=True), oracle.matmul_vec_fp16(w[0], xs, sparse=False))
