"""Parity of the HIP path against the CPU oracle and float64 truth, through the C ABI.

Bars: packed bytes and scale blocks bit-exact; products within
|a - b| <= max(eps, eps * max(|a|, |b|)), eps = 2e-3 (f16 output, f32 accumulate).
"""
import os

import numpy as np
import pytest

from helpers import (ACTS, EPS, NF4_QUANT, assert_close, gen_f16, int8_dequant64, nf4_dequant64,
                     truth_matmul)

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SEED = 0x57525100


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    import torch

    torch.cuda.synchronize()
    return t.cpu().numpy()


def announce(*what):
    print("case:", *what, flush=True)


# ---------------------------------------------------------------- packing


# (R, K): the reference's test shapes, the 1.6B operator-sweep shapes (head 2048 -> 65536 included), the 7B FFN shapes
PACK_SHAPES = [(64, 320), (2048, 2560), (2048, 2048), (2048, 7168), (7168, 2048), (768, 2688), (3, 8, 512),
               (65536, 2048), (14336, 4096), (4096, 14336)]


def special_blocks(rng):
    """Edge cases: constant and zero blocks, +-max f16, subnormals, exact ties, +-absmax."""
    w = gen_f16(rng, (16, 1024), 0.02)
    w[0, :128] = np.float16(0.25)  # constant int8 block -> all codes 0
    w[1, :] = 0  # zero nf4 blocks -> nibble 0, absmax 0
    w[2, :4] = [65504, -65504, 6e-8, -6e-8]
    w[3, :256] = np.linspace(-1, 1, 256).astype(np.float16)  # many exact ties after scaling
    w[4, :64] = 0.5
    w[4, 1] = -0.5
    w[5, :128] = np.arange(128, dtype=np.float16) * np.float16(2.0)  # (v-min)/(max-min)*255 hits n + 0.5 often
    return w


@pytest.mark.parametrize("shape", PACK_SHAPES, ids=str)
def test_quant_int8_bit_exact(gpu, oracle, shape):
    import torch

    announce("quant_int8", shape)
    rng = np.random.default_rng(SEED + 2)
    w = gen_f16(rng, shape, 0.02)
    m = gpu.Matrix.quant_u8(dev(w))
    want_w, want_m, flagged = oracle.quant_int8(w)
    assert np.array_equal(host(m.m).view(np.uint16), want_m.view(np.uint16))
    got = host(m.w)
    assert got.shape == w.shape
    assert np.array_equal(got, want_w), f"{(got != want_w).sum()} bytes differ ({flagged} policy-sensitive)"


def test_quant_int8_edge_cases(gpu, oracle):
    announce("quant_int8 edge cases")
    w = special_blocks(np.random.default_rng(SEED + 20))
    m = gpu.Matrix.quant_u8(dev(w))
    want_w, want_m, _ = oracle.quant_int8(w)
    assert np.array_equal(host(m.m).view(np.uint16), want_m.view(np.uint16))
    assert np.array_equal(host(m.w), want_w)
    assert (host(m.w)[0, :128] == 0).all()


@pytest.mark.parametrize("shape", PACK_SHAPES, ids=str)
def test_quant_nf4_bit_exact(gpu, oracle, shape):
    announce("quant_nf4", shape)
    rng = np.random.default_rng(SEED + 3)
    w = gen_f16(rng, shape, 0.02)
    m = gpu.Matrix.quant_nf4(dev(w))
    want_w, want_m = oracle.quant_nf4(w)
    assert np.array_equal(host(m.m).view(np.uint16), want_m.view(np.uint16))
    got = host(m.w)
    assert got.shape == want_w.shape
    assert np.array_equal(got, want_w), f"{(got != want_w).sum()} bytes differ"
    assert np.array_equal(host(m.q), NF4_QUANT)


def test_quant_nf4_edge_cases_and_custom_table(gpu, oracle):
    announce("quant_nf4 edge cases")
    w = special_blocks(np.random.default_rng(SEED + 30))
    for table in (None, np.linspace(-1, 1, 16).astype(np.float32) ** 3):
        m = gpu.Matrix.quant_nf4(dev(w), None if table is None else table.tolist())
        want_w, want_m = oracle.quant_nf4(w, NF4_QUANT if table is None else table)
        assert np.array_equal(host(m.m).view(np.uint16), want_m.view(np.uint16))
        assert np.array_equal(host(m.w), want_w)
    assert (host(m.w)[1] == 0).all()


def test_quant_every_f16_value(gpu, oracle):
    announce("quant every finite f16")
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    fin = allh[np.isfinite(allh)]
    fin = np.concatenate([fin, np.zeros((-len(fin)) % 128, np.float16)])
    rng = np.random.default_rng(SEED + 40)
    for order in (fin, rng.permutation(fin)):
        w = order.reshape(-1, 128)
        m8, m4 = gpu.Matrix.quant_u8(dev(w)), gpu.Matrix.quant_nf4(dev(w))
        w8, s8, _ = oracle.quant_int8(w)
        w4, s4 = oracle.quant_nf4(w)
        assert np.array_equal(host(m8.w), w8) and np.array_equal(host(m8.m).view(np.uint16), s8.view(np.uint16))
        assert np.array_equal(host(m4.w), w4) and np.array_equal(host(m4.m).view(np.uint16), s4.view(np.uint16))


def test_quant_int8_hard_divisions(gpu, oracle):
    """Blocks whose range max - min is the f32 just below a power of two (all-ones mantissa): the
    reciprocal of such a divisor sits next to a rounding boundary, the hard case of any division
    built from a reciprocal.  Dividends: powers of two, their neighbours and random values."""
    announce("quant_int8 hard divisions")
    rng = np.random.default_rng(SEED + 50)
    rows = []
    for k in range(0, 16):
        mx, mn = np.float16(2.0 ** k), np.float16(2.0 ** (k - 24))
        assert np.float32(mx) - np.float32(mn) == np.nextafter(np.float32(mx), np.float32(0))
        for _ in range(4):
            blk = (rng.random(128) * float(mx)).astype(np.float16)
            p2 = np.float16(2.0) ** rng.integers(k - 24, k, 48)
            blk[:48] = p2.astype(np.float16)
            blk[48:64] = np.nextafter(p2[:16].astype(np.float16), np.float16(0))
            blk[64:80] = np.nextafter(p2[16:32].astype(np.float16), np.float16(65504))
            blk = np.clip(blk, mn, mx)
            blk[rng.integers(0, 128)] = mx
            blk[(np.argmax(blk == mx) + 1) % 128] = mn
            rows.append(blk if rng.random() < 0.5 else -blk)
    w = np.stack(rows).astype(np.float16)
    m = gpu.Matrix.quant_u8(dev(w))
    want_w, want_m, _ = oracle.quant_int8(w)
    assert np.array_equal(host(m.m).view(np.uint16), want_m.view(np.uint16))
    got = host(m.w)
    assert np.array_equal(got, want_w), f"{(got != want_w).sum()} bytes differ"


@pytest.mark.parametrize("table", ["eighths", "sf4", "reversed", "shuffled", "duplicates", "narrow", "close_pair"])
def test_quant_nf4_tables(gpu, oracle, table):
    """Tables on both sides of the packer's choice between threshold search and literal scan.
    `eighths` puts every decision threshold on an f16 value, and blocks holding 1.0 present those
    values unscaled: exact ties, which the scan gives to the later entry."""
    announce("quant_nf4 table", table)
    rng = np.random.default_rng(SEED + 60)
    q = {
        "eighths": np.arange(-8, 8) / 8.0,
        "sf4": np.array(gpu.quantile_student(5.0)),
        "reversed": NF4_QUANT[::-1],
        "shuffled": rng.permutation(NF4_QUANT),
        "duplicates": np.repeat(NF4_QUANT[::2], 2),
        "narrow": NF4_QUANT * 0.2 - 0.7,  # all entries in [-0.9, -0.5]: x above 0.5 is further than the scan's initial bound
        "close_pair": np.concatenate([NF4_QUANT[:8], [NF4_QUANT[8] * 0 + 1e-7], NF4_QUANT[9:]]),
    }[table].astype(np.float32)
    w = gen_f16(rng, (256, 1024), 0.02)
    w[:64] = (rng.integers(-16, 17, (64, 1024)) / 16.0).astype(np.float16)  # thresholds of `eighths` and entries
    w[:64, ::64] = 1.0
    w[64:96] = (rng.random((32, 1024)) * 2 - 1).astype(np.float16)
    w[96:128] = gen_f16(rng, (32, 1024), 30.0)
    m = gpu.Matrix.quant_nf4(dev(w), q.tolist())
    want_w, want_m = oracle.quant_nf4(w, q)
    assert np.array_equal(host(m.m).view(np.uint16), want_m.view(np.uint16))
    got = host(m.w)
    assert np.array_equal(got, want_w), f"{(got != want_w).sum()} bytes differ"


def test_quant_full_size_random_scales(gpu, oracle):
    """A 4096 x 4096 matrix whose blocks span many magnitudes: x = v / absmax then takes f32 values
    all over [-1, 1], next to the nf4 decision thresholds included."""
    announce("quant 4096x4096 mixed scales")
    rng = np.random.default_rng(SEED + 70)
    scale = np.exp2(rng.integers(-20, 12, (4096, 64))).repeat(64, axis=1)
    w = (rng.standard_normal((4096, 4096)) * scale).astype(np.float16)
    m8, m4 = gpu.Matrix.quant_u8(dev(w)), gpu.Matrix.quant_nf4(dev(w))
    w8, s8, _ = oracle.quant_int8(w)
    w4, s4 = oracle.quant_nf4(w)
    assert np.array_equal(host(m8.w), w8) and np.array_equal(host(m8.m).view(np.uint16), s8.view(np.uint16))
    assert np.array_equal(host(m4.w), w4) and np.array_equal(host(m4.m).view(np.uint16), s4.view(np.uint16))


# --------------------------------------------------------------- products


def pack(oracle, kind, w):
    if kind == "int8":
        u8, mm, _ = oracle.quant_int8(w)
        return u8, mm, int8_dequant64(u8, mm)
    p, am = oracle.quant_nf4(w)
    return p, am, nf4_dequant64(p, am)


def gpu_matrix(gpu, kind, wp, scale):
    import torch

    q = torch.tensor(gpu.NF4_QUANT, dtype=torch.float32, device="cuda") if kind == "nf4" else None
    return gpu.Matrix("Int8" if kind == "int8" else "Fp4", dev(wp), dev(scale), q)


def run(gpu, m, x, R, entry, out_dtype=np.float16, act=0, sparse=False):
    import torch

    T = x.shape[-2]
    shape = x.shape[:-2] + (T, R)
    out = torch.full(shape, float("nan"), dtype=torch.float16 if out_dtype == np.float16 else torch.float32, device="cuda")
    xd = dev(x)
    if entry == "vec":
        m.matmul_vec_op(xd, out, act, sparse)
    else:
        m.matmul_mat_op(xd, out, act)
    return host(out)


# (K, R): config-2/3 operator sweep at RWKV-v6 1.6B shapes, 7B shapes, and the v5 config-1 shapes
SWEEP = [(2048, 2048), (2048, 7168), (7168, 2048), (2048, 65536), (4096, 4096), (4096, 14336), (14336, 4096),
         (768, 768), (768, 2688), (2688, 768)]


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("K,R", SWEEP, ids=str)
def test_gemv_against_oracle(gpu, oracle, kind, K, R):
    announce("gemv", kind, K, R)
    rng = np.random.default_rng(SEED + 2 + K * 7 + R)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (1, K), 1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    ofn = oracle.matmul_vec_int8 if kind == "int8" else oracle.matmul_vec_nf4
    for out_dtype in (np.float16, np.float32):
        got = run(gpu, m, x, R, "vec", out_dtype)
        want = ofn(wp, scale, x, out_dtype=out_dtype)[0]
        assert_close(got, want, EPS, f"{kind} {K}x{R} vs oracle")
        assert_close(got, truth_matmul(wdeq, x), EPS, f"{kind} {K}x{R} vs float64")
    if out_dtype == np.float32:  # f32 output: accumulation error only, far inside the bar
        assert_close(got, truth_matmul(wdeq, x), 1e-4, f"{kind} {K}x{R} f32 vs float64")


# every K / 1024 the wave-owns-rows decode kernel is built for
WAVE_ROWS_K = [1024 * b for b in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16)]


@pytest.mark.parametrize("K", WAVE_ROWS_K)
def test_int8_wave_rows_kernel(gpu, oracle, K, overrides):
    # one token, f16 activations, K a multiple of 1024: single products and groups, rows that do not fill the last
    # task, all output types, an activation, a z-offset view, the batch axis -- against the oracle and float64; the
    # kernel it replaces (gemv_waverows=0) is held to the same bar on the same inputs
    import torch

    announce("int8 wave-owns-rows", K)
    rng = np.random.default_rng(SEED + 77 + K)
    rows = [204, 64, 8, 4, 132]  # multiples of 4 (the entry point requires it): ragged last tasks, a single task
    mats, xs, truths, wants = [], [], [], []
    for R in rows:
        w = gen_f16(rng, (R, K), 0.02)
        x = gen_f16(rng, (1, K), 1.0)
        wp, scale, wdeq = pack(oracle, "int8", w)
        mats.append(gpu_matrix(gpu, "int8", wp, scale))
        xs.append(x)
        truths.append(truth_matmul(wdeq, x))
        wants.append(oracle.matmul_vec_int8(wp, scale, x, out_dtype=np.float32)[0])
    # 2: the wave-owns-rows kernel at every K it is built for; 1: the default choice (beyond K = 8192 the K-split kernel);
    # 0: the one-shot kernel they replace
    for waverows in (2, 1, 0):
        overrides(gemv_waverows=waverows)
        for m, x, R, truth, want in zip(mats, xs, rows, truths, wants):
            for out_dtype in (np.float16, np.float32):
                got = run(gpu, m, x, R, "vec", out_dtype)
                assert_close(got, want, EPS, f"K={K} R={R} waverows={waverows} vs oracle")
                assert_close(got, truth, EPS, f"K={K} R={R} waverows={waverows} vs float64")
            got = run(gpu, m, x, R, "vec", np.float32, act=1)
            assert_close(got, np.square(np.maximum(truth, 0.0)), EPS, f"K={K} R={R} squared relu")
        # all five in one grouped launch, mixed output types and activations
        outs = [torch.full((1, R), float("nan"), dtype=torch.float16 if i % 2 else torch.float32, device="cuda") for i, R in enumerate(rows)]
        gpu.matmul_vec_group([(m, dev(x), o, gpu.ACT_SQUARED_RELU if i == 2 else gpu.ACT_NONE, False, {})
                              for i, (m, x, o) in enumerate(zip(mats, xs, outs))])
        for i, (o, truth) in enumerate(zip(outs, truths)):
            assert_close(host(o).astype(np.float32), np.square(np.maximum(truth, 0.0)) if i == 2 else truth, EPS, f"K={K} group member {i}")
        # groups of two to four take a kernel of their own (the first product's descriptor travels with the arguments)
        for n in (2, 3, 4):
            outs = [torch.full((1, R), float("nan"), dtype=torch.float16 if i % 2 else torch.float32, device="cuda") for i, R in enumerate(rows[:n])]
            gpu.matmul_vec_group([(m, dev(x), o, gpu.ACT_SQUARED_RELU if i == 0 else gpu.ACT_NONE, False, {})
                                  for i, (m, x, o) in enumerate(zip(mats[:n], xs[:n], outs))])
            for i, (o, truth) in enumerate(zip(outs, truths[:n])):
                assert_close(host(o).astype(np.float32), np.square(np.maximum(truth, 0.0)) if i == 0 else truth, EPS, f"K={K} group of {n}, member {i}")
    overrides(gemv_waverows=2)
    # a z-offset input view and an offset output view (v6: att_sx.view(.., .., i, ..), src/runtime/v6.rs:806-829)
    parent = gen_f16(rng, (5, 1, K), 1.0)
    out = torch.full((3, 3, rows[0]), -7.0, dtype=torch.float32, device="cuda")
    mats[0].matmul_vec_op(dev(parent), out, input_view=((K, 1, 1), (K, 1, 5), (0, 0, 3)), output_view=((rows[0], 1, 1), (rows[0], 3, 3), (0, 1, 2)))
    got = host(out)
    assert_close(got[2, 1:2], oracle.matmul_vec_int8(host(mats[0].w), host(mats[0].m), parent[3], out_dtype=np.float32)[0], EPS, "offset views")
    got[2, 1:2] = -7.0
    assert (got == -7.0).all(), "wrote outside the output view"
    # batch axis: matrix [K, R, B]
    B, R = 3, 36
    wb = gen_f16(rng, (B, R, K), 0.02)
    xb = gen_f16(rng, (B, 1, K), 1.0)
    wpb, sb, wdq = pack(oracle, "int8", wb)
    truth = np.stack([truth_matmul(wdq[b], xb[b]) for b in range(B)])
    assert_close(run(gpu, gpu_matrix(gpu, "int8", wpb, sb), xb, R, "vec", np.float32), truth, EPS, "batched")


@pytest.mark.parametrize("K", WAVE_ROWS_K)
def test_int8_wave_rows_kernels_on_short_runs(gpu, oracle, K, overrides):
    # runs of 2, 3 and 4 tokens of f16 activations on int8 rows of a multiple of 1024 take the wave-owns-rows layout (up to 8192, the
    # tokens' activations in LDS) or, at three tokens, the K-split layout (10240 .. 14336), all tokens of the run in one pass.
    # Single products and groups, ragged last tasks, both output types, an activation, token strides through views, the batch axis --
    # against the oracle and float64, and the kernel they replace (gemv_rows_tokens = 0) on the same inputs
    import torch

    announce("int8 wave-owns-rows, short runs", K)
    rng = np.random.default_rng(SEED + 177 + K)
    rows = [204, 64, 8, 4, 132]
    packed, mats = [], []
    for R in rows:
        wp, scale, wdeq = pack(oracle, "int8", gen_f16(rng, (R, K), 0.02))
        packed.append((wp, scale, wdeq))
        mats.append(gpu_matrix(gpu, "int8", wp, scale))
    for T in (2, 3, 4):
        xs = [gen_f16(rng, (T, K), 1.0) for _ in rows]
        truths = [truth_matmul(wdeq, x) for (_, _, wdeq), x in zip(packed, xs)]
        wants = [oracle.matmul_vec_int8(wp, scale, x, out_dtype=np.float32)[0] for (wp, scale, _), x in zip(packed, xs)]
        for tokens_kernel in (1, 0):
            overrides(gemv_rows_tokens=tokens_kernel)
            for m, x, R, truth, want in zip(mats, xs, rows, truths, wants):
                for out_dtype in (np.float16, np.float32):
                    got = run(gpu, m, x, R, "vec", out_dtype)
                    assert_close(got, want, EPS, f"K={K} R={R} T={T} tokens_kernel={tokens_kernel} vs oracle")
                    assert_close(got, truth, EPS, f"K={K} R={R} T={T} tokens_kernel={tokens_kernel} vs float64")
                got = run(gpu, m, x, R, "vec", np.float32, act=1)
                assert_close(got, np.square(np.maximum(truth, 0.0)), EPS, f"K={K} R={R} T={T} squared relu")
            outs = [torch.full((T, R), float("nan"), dtype=torch.float16 if i % 2 else torch.float32, device="cuda") for i, R in enumerate(rows)]
            gpu.matmul_vec_group([(m, dev(x), o, gpu.ACT_SQUARED_RELU if i == 2 else gpu.ACT_NONE, False, {})
                                  for i, (m, x, o) in enumerate(zip(mats, xs, outs))])
            for i, (o, truth) in enumerate(zip(outs, truths)):
                assert_close(host(o).astype(np.float32), np.square(np.maximum(truth, 0.0)) if i == 2 else truth, EPS, f"K={K} T={T} group member {i}")
        overrides(gemv_rows_tokens=1)
        # token strides that differ from the row lengths: the i-th of 5 interleaved activation sets (v6: att_sx.view(.., .., i, ..),
        # src/runtime/v6.rs:806-829) into a slice of a wider output
        parent = gen_f16(rng, (5, T, K), 1.0)
        out = torch.full((3, T + 2, rows[0]), -7.0, dtype=torch.float32, device="cuda")
        mats[0].matmul_vec_op(dev(parent), out, input_view=((K, T, 1), (K, T, 5), (0, 0, 3)),
                              output_view=((rows[0], T, 1), (rows[0], T + 2, 3), (0, 1, 2)))
        got = host(out)
        assert_close(got[2, 1:1 + T], oracle.matmul_vec_int8(packed[0][0], packed[0][1], parent[3], out_dtype=np.float32)[0], EPS, f"T={T} offset views")
        got[2, 1:1 + T] = -7.0
        assert (got == -7.0).all(), "wrote outside the output view"
        # batch axis: matrix [K, R, B], activations [K, T, B]
        B, R = 3, 36
        wb = gen_f16(rng, (B, R, K), 0.02)
        xb = gen_f16(rng, (B, T, K), 1.0)
        wpb, sb, wdq = pack(oracle, "int8", wb)
        truth = np.stack([truth_matmul(wdq[b], xb[b]) for b in range(B)])
        assert_close(run(gpu, gpu_matrix(gpu, "int8", wpb, sb), xb, R, "vec", np.float32), truth, EPS, f"T={T} batched")


def test_stamped_builds_of_the_decode_kernels(gpu, oracle):
    # wrq_debug_stamps swaps in builds of the one-token int8 kernels (K = 4096 rows kernel, single and grouped; K = 14336
    # K-split kernel) that also write wall-clock records: results must be bit-identical to the product kernels', every
    # wave of every launch must leave a record with ordered readings, and nothing is written once the hook is off
    import ctypes as C
    import torch

    announce("int8 stamped decode kernels")
    L = gpu.lib()
    L.wrq_debug_stamps.argtypes = [C.c_void_p, C.c_uint64]
    rng = np.random.default_rng(SEED + 79)
    shapes = [(4096, 204), (4096, 64), (14336, 36)]
    mats, xs = [], []
    for K, R in shapes:
        wp, scale, _ = pack(oracle, "int8", gen_f16(rng, (R, K), 0.02))
        mats.append(gpu_matrix(gpu, "int8", wp, scale))
        xs.append(gen_f16(rng, (1, K), 1.0))

    def products():
        outs = [run(gpu, m, x, R, "vec", np.float32) for m, x, (K, R) in zip(mats, xs, shapes)]
        go = [torch.full((1, R), float("nan"), dtype=torch.float32, device="cuda") for K, R in shapes[:2]]
        gpu.matmul_vec_group([(m, dev(x), o, gpu.ACT_NONE, False, {}) for m, x, o in zip(mats[:2], xs[:2], go)])
        return outs + [host(o) for o in go]

    want = products()
    slot = 1 << 20
    buf = torch.zeros(4 * slot, dtype=torch.uint8, device="cuda")
    assert L.wrq_debug_stamps(C.c_void_p(buf.data_ptr()), slot + 5) != 0, "a size that is no multiple of 1 MiB must be refused"
    assert L.wrq_debug_stamps(C.c_void_p(buf.data_ptr()), buf.numel()) == 0, L.wrq_last_error().decode()
    try:
        got = products()
    finally:
        assert L.wrq_debug_stamps(None, 0) == 0
    for a, b in zip(got, want):
        assert np.array_equal(a, b), "stamped build changed a result"
    rec = buf.view(torch.int64).view(4, slot // 32, 4).cpu().numpy()
    waves = [(-(-204 // 4)) * 4, (64 // 4) * 4, -(-36 // 8) * 14, (-(-204 // 4) + 64 // 4) * 4]  # records per launch, in launch order
    for i, n in enumerate(waves):
        r = rec[i]
        assert (r[:n, 0] > 0).all(), f"launch {i}: a wave left no record"
        assert (np.diff(r[:n], axis=1) >= 0).all(), f"launch {i}: readings out of order"
        assert (r[n:] == 0).all(), f"launch {i}: records beyond its waves"
    buf.zero_()
    products()
    assert int(buf.count_nonzero()) == 0, "stamps written with the hook off"


def test_int8_wave_rows_groups_of_mixed_k(gpu, oracle):
    # products of different K in one grouped call: the launch is cut where K changes, every product still gets its result
    import torch

    announce("int8 wave-owns-rows, mixed K in a group")
    rng = np.random.default_rng(SEED + 78)
    shapes = [(4096, 96), (4096, 40), (2048, 72), (1152, 24), (4096, 12), (14336, 20), (14336, 4)]  # R % 4 == 0
    ops, truths, outs = [], [], []
    for K, R in shapes:
        w = gen_f16(rng, (R, K), 0.02)
        x = gen_f16(rng, (1, K), 1.0)
        wp, scale, wdeq = pack(oracle, "int8", w)
        o = torch.full((1, R), float("nan"), dtype=torch.float32, device="cuda")
        ops.append((gpu_matrix(gpu, "int8", wp, scale), dev(x), o, gpu.ACT_NONE, False, {}))
        outs.append(o)
        truths.append(truth_matmul(wdeq, x))
    gpu.matmul_vec_group(ops)
    for (K, R), o, truth in zip(shapes, outs, truths):
        assert_close(host(o), truth, EPS, f"mixed group member {K}x{R}")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("T", [2, 3, 4, 5, 8, 15, 16, 17, 31])
def test_multi_token_vec_entry(gpu, oracle, kind, T):
    # T < 32 or T % 32 != 0 reaches the vec entry point in the reference (grid.y = T)
    announce("vec multi-token", kind, T)
    K, R = 2048, 512
    rng = np.random.default_rng(SEED + 5 + T)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    ofn = oracle.matmul_vec_int8 if kind == "int8" else oracle.matmul_vec_nf4
    got = run(gpu, m, x, R, "vec", np.float32)
    assert_close(got, ofn(wp, scale, x, out_dtype=np.float32)[0], EPS, "vs oracle")
    assert_close(got, truth_matmul(wdeq, x), EPS, "vs float64")
    # K that is no multiple of 128 (blocks straddle rows) stays on the VALU kernels at every T
    K2, R2 = 1056, 64
    w2 = gen_f16(rng, (R2, K2), 0.02)
    x2 = gen_f16(rng, (T, K2), 1.0)
    wp2, scale2, wdeq2 = pack(oracle, kind, w2)
    got2 = run(gpu, gpu_matrix(gpu, kind, wp2, scale2), x2, R2, "vec", np.float32)
    assert_close(got2, ofn(wp2, scale2, x2, out_dtype=np.float32)[0], EPS, "K = 1056 vs oracle")
    assert_close(got2, truth_matmul(wdeq2, x2), EPS, "K = 1056 vs float64")


# (K, R, T) for the chunk kernels: config 3 (T in 32, 128, 256), config 4 (T = 128 at 7B), the
# reference's own test shapes (ops.rs:3058-3059), and T below one MFMA tile
GEMM = [(2048, 2048, 32), (2048, 2048, 128), (2048, 2048, 256), (2048, 7168, 32), (7168, 2048, 128),
        (4096, 4096, 128), (2560, 2048, 64), (320, 64, 320), (768, 2688, 32), (2688, 768, 32), (2048, 512, 4),
        (2048, 512, 20), (2048, 65536, 32),
        (4096, 14336, 128), (14336, 4096, 128), (4096, 4096, 256), (14336, 4096, 256), (2048, 65536, 256),
        # the remaining cells of config 3 (every shape at every token count)
        (7168, 2048, 32), (2048, 7168, 128), (2048, 65536, 128), (2048, 7168, 256), (7168, 2048, 256)]


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("K,R,T", GEMM, ids=str)
def test_gemm_against_truth(gpu, oracle, kind, K, R, T):
    announce("gemm", kind, K, R, T)
    if kind == "nf4" and K % 64:
        pytest.skip("nf4 needs K % 64 == 0")
    rng = np.random.default_rng(SEED + 3 + K * 7 + R + T)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    truth = truth_matmul(wdeq, x)
    for out_dtype in (np.float16, np.float32):
        got = run(gpu, m, x, R, "mat", out_dtype)
        assert_close(got, truth, EPS, f"{kind} {K}x{R}x{T} vs float64")
    assert_close(got, truth, 2e-4, "f32 output vs float64")  # exact operands: only f32 accumulation differs
    if R * T * K <= 2048 * 2048 * 32:
        ofn = oracle.matmul_mat_int8 if kind == "int8" else oracle.matmul_mat_nf4
        assert_close(got, ofn(wp, scale, x, out_dtype=np.float32)[0], EPS, "vs oracle")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("K,R", SWEEP[:4], ids=str)
def test_eight_tokens_on_the_vec_entry(gpu, oracle, kind, K, R):
    # the operator sweep's 8 activation rows at the 1.6B shapes: T = 8 is no multiple of 32, so the model
    # builders send it to the decode entry point (src/runtime/v6.rs:568-570)
    announce("vec entry, 8 tokens", kind, K, R)
    rng = np.random.default_rng(SEED + 8 + K * 3 + R)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (8, K), 1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    truth = truth_matmul(wdeq, x)
    for out_dtype in (np.float16, np.float32):
        assert_close(run(gpu, m, x, R, "vec", out_dtype), truth, EPS, f"{kind} {K}x{R} T=8 vs float64")
    if R <= 7168:
        ofn = oracle.matmul_vec_int8 if kind == "int8" else oracle.matmul_vec_nf4
        assert_close(run(gpu, m, x, R, "vec", np.float32), ofn(wp, scale, x, out_dtype=np.float32)[0], EPS, "vs oracle")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("entry,T", [("mat", 32), ("mat", 128), ("vec", 16), ("vec", 40)])
def test_f32_activations_that_are_no_f16_values(gpu, oracle, kind, entry, T):
    # the reference's Bundle<f32> feeds f32 activations to f32 arithmetic (src/shaders/matmul_mat_int8.wgsl:106-132):
    # random f32 inputs, rows that cancel included, at the longest K of the path, against float64
    announce("f32 activations", kind, entry, T)
    K, R = 14336, 512
    rng = np.random.default_rng(SEED + 77 + T)
    w = gen_f16(rng, (R, K), 0.02)
    x = rng.standard_normal((T, K), dtype=np.float32) * np.float32(1.0009765625)
    x[1] = x[0] * np.float32(-0.99993896484375)  # token 1 nearly cancels token 0 when summed by a caller
    assert (x.astype(np.float16).astype(np.float32) != x).mean() > 0.9
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    truth = truth_matmul(wdeq, x)
    got = run(gpu, m, x, R, entry, np.float32)
    assert_close(got, truth, EPS, f"{kind} {entry} T={T} f32 activations vs float64")
    # weights whose products cancel: w and -w interleaved along K, so every output is a small difference of large sums
    w2 = w.copy()
    w2[:, 1::2] = -w2[:, 0::2]
    x2 = x.copy()
    x2[:, 1::2] = x2[:, 0::2] * np.float32(1.0001220703125)
    wp2, scale2, wdeq2 = pack(oracle, kind, w2)
    got2 = run(gpu, gpu_matrix(gpu, kind, wp2, scale2), x2, R, entry, np.float32)
    assert_close(got2, truth_matmul(wdeq2, x2), EPS, f"{kind} {entry} T={T} cancelling sums")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("T", [1, 16, 40])
def test_f32_activations_beyond_the_f16_range(gpu, oracle, kind, T):
    # f32 activations up to 65535 in magnitude: the matrix-core kernel splits them into two f16 halves and must keep both finite
    # (f16 ends at 65504); the decode kernels take f32 as it is.  The same inputs through both entry points, against float64.
    announce("f32 activations beyond the f16 range", kind, T)
    K, R = 1024, 128
    rng = np.random.default_rng(SEED + 79 + T)
    w = gen_f16(rng, (R, K), 0.02)
    x = rng.standard_normal((T, K), dtype=np.float32)
    big = np.float32([65505.0, -65519.5, 65520.0, -65535.0, 65504.0, 60000.25, -65534.99, 32768.5])
    for t in range(T):
        cols = rng.choice(K, size=len(big), replace=False)
        x[t, cols] = big * np.float32(1.0 if t % 2 == 0 else -1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    truth = truth_matmul(wdeq, x)
    # terms of magnitude 65535 * |w| cancel in these sums.  f32 accumulation (the reference's too) is good to a few 1e-7 of the
    # sum of the terms' magnitudes; the kernels factor the block's scale and offset out of the sum of codes
    # (s * sum((1024 + u) x) + (min - 1024 s) * sum(x)), whose two parts are about 30 times a term, so the bar is the usual
    # one widened by 1e-5 of that sum -- invisible at any activation a model produces, visible at 65535
    terms = np.abs(x.astype(np.float64)) @ np.abs(wdeq.astype(np.float64)).T
    for entry in (("vec", "mat") if T % 4 == 0 else ("vec",)):  # the mat entry takes multiples of 4 tokens
        got = run(gpu, m, x, R, entry, np.float32)
        assert np.isfinite(got).all(), f"{kind} {entry} T={T}: non-finite outputs"
        bound = np.maximum(np.maximum(EPS, EPS * np.abs(truth)), 1e-5 * terms)
        bad = np.abs(got - truth) > bound
        assert not bad.any(), f"{kind} {entry} T={T}: {bad.sum()} outputs off, worst {np.abs(got - truth)[bad].max()} at bound {bound[bad].min()}"


@pytest.mark.parametrize("kind", ["nf4", "int8"])
def test_serving_schedule_run_lengths(gpu, oracle, kind):
    # every distinct run length of the 32-slot serving schedule (prompts 16 .. 1024, chunk 256, 128 decode
    # tokens per slot, cut by the RnnIter restatement in bench.py) on the products of a 7B-shape layer, with
    # the kernel choice of the model builders (chunk kernels iff T % 32 == 0); a sample of rows of every
    # product against float64
    import torch

    import bench

    announce("serving schedule", kind)
    rng = np.random.default_rng(SEED + 5)
    slots, chunk, gen_len = 32, 256, 128
    prompts = rng.integers(16, 1025, size=slots)
    state = [[False, int(p)] for p in prompts]
    to_gen = [gen_len] * slots
    lengths = set()
    while any(read > 0 for _, read in state):
        lens = bench.rnn_iter_next(state, chunk)
        T = sum(lens)
        if T == 0:
            break
        lengths.add(T)
        for i in range(slots):
            state[i][0] = False
            if lens[i] > 0 and state[i][1] == 0 and to_gen[i] > 0:
                to_gen[i] -= 1
                state[i][1] = 1 if to_gen[i] > 0 else 0
    assert 256 in lengths and 32 in lengths and min(lengths) < 32
    C, H = 4096, 14336
    mats = []
    for K, R in ((C, C), (C, H), (H, C)):
        w = gen_f16(rng, (R, K), 0.02)
        wp, scale, wdeq = pack(oracle, kind, w)
        rows = np.sort(rng.choice(R, 96, replace=False))
        mats.append((K, R, gpu_matrix(gpu, kind, wp, scale), wdeq[rows], rows))
    for T in sorted(lengths):
        for K, R, m, wsub, rows in mats:
            x = gen_f16(rng, (T, K), 1.0)
            out = torch.full((T, R), float("nan"), dtype=torch.float16, device="cuda")
            m.matmul_op(dev(x), out, turbo=gpu.turbo(T))
            got = host(out)
            assert np.isfinite(got).all(), f"{kind} T={T} {K}x{R}"
            assert_close(got[:, rows], truth_matmul(wsub, x), EPS, f"{kind} T={T} {K}x{R} vs float64")


# (MRT, NTILE, KG) instantiations of the chunk kernel: 64 * MRT / KG rows x 16 * NTILE tokens per
# workgroup, KG k groups of waves that take alternate K steps
TILE_VARIANTS = [(1, 1, 1), (1, 2, 1), (1, 4, 1), (1, 8, 1), (2, 1, 1), (2, 2, 1), (2, 4, 1), (2, 8, 1),
                 (1, 1, 2), (1, 2, 2), (1, 4, 2), (2, 1, 2), (2, 2, 2), (2, 4, 2), (1, 1, 4), (1, 2, 4)]


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("mrt,ntile,kg", TILE_VARIANTS, ids=str)
def test_chunk_tile_variants(gpu, oracle, kind, mrt, ntile, kg, overrides):
    # every tile instantiation of the chunk kernel, with and without split K, on a shape that
    # leaves ragged edges everywhere: 5 steps of K (a partial stage, fewer steps than some k
    # groups get), rows and tokens that do not fill the tiles.  The tile is pinned through the
    # library's test hook (wrq_debug_override).
    announce("chunk tile variant", kind, mrt, ntile, kg)
    K, R, T = 640, 200, 40
    rng = np.random.default_rng(SEED + 11 + mrt * 16 + ntile + 64 * kg)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    truth = truth_matmul(wdeq, x)
    overrides(gemm_kg=kg, gemm_mrt=mrt, gemm_ntile=ntile)
    for ksplit in (1, 2, 5):
        overrides(gemm_ksplit=ksplit)
        for out_dtype in (np.float16, np.float32):
            got = run(gpu, m, x, R, "mat", out_dtype, act=1)
            assert_close(got, np.square(np.maximum(truth, 0.0)), EPS, f"{kind} tile ({mrt},{ntile},{kg}) ksplit {ksplit}")
        got32 = run(gpu, m, x.astype(np.float32), R, "mat", np.float32)
        assert_close(got32, truth, EPS, f"{kind} tile ({mrt},{ntile},{kg}) ksplit {ksplit} f32 in")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("T", [8, 24, 100, 200])
def test_chunk_k_groups_by_default(gpu, oracle, kind, T):
    # shapes that the tile choice sends to k groups without any override: a 4096-row product
    # (nf4: k groups instead of a split of K) and groups of about 256 and 288 row tiles of 64
    # at narrow token tiles (two k groups per workgroup)
    import torch

    announce("chunk k groups by default", kind, T)
    rng = np.random.default_rng(SEED + 41 + T)
    K = 1152
    packed = {}
    for R in (4096, 14336):
        w = gen_f16(rng, (R, K), 0.02)
        wp, scale, wdeq = pack(oracle, kind, w)
        packed[R] = (gpu_matrix(gpu, kind, wp, scale), wdeq)
    x = gen_f16(rng, (T, K), 1.0)
    m, wdeq = packed[4096]
    assert_close(run(gpu, m, x, 4096, "mat", np.float32), truth_matmul(wdeq, x), EPS, f"{kind} 4096 rows T={T}")
    for rows in ([4096] * 4, [14336, 4096]):
        xs = [gen_f16(rng, (T, K), 1.0) for _ in rows]
        xd = [dev(v) for v in xs]
        outs = [torch.full((T, R), float("nan"), dtype=torch.float32, device="cuda") for R in rows]
        gpu.matmul_vec_group([(packed[R][0], xv, o, gpu.ACT_NONE, False, {}) for R, xv, o in zip(rows, xd, outs)])
        for R, xv, o in zip(rows, xs, outs):
            assert_close(host(o), truth_matmul(packed[R][1], xv), EPS, f"{kind} group {rows} T={T}")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("C,H", [(2560, 8960), (5120, 17920)], ids=str)
def test_decode_tasks_from_the_measured_table(gpu, oracle, kind, C, H, overrides):
    # runs of 1 .. 4 tokens on the launches of model sizes whose lanes and rows per task come from the measured
    # table of the one-shot kernels (csrc/gemv_tuned.inc), against float64 on sampled rows; once more with the
    # table switched off (gemv_table = 0)
    import torch

    announce("decode tasks from the table", kind, C, H)
    rng = np.random.default_rng(SEED + 53 + C)
    mats = {}
    for R, K in ((C, C), (H, C), (C, H)):
        w = gen_f16(rng, (R, K), 0.02)
        wp, scale, wdeq = pack(oracle, kind, w)
        rows = np.sort(rng.choice(R, 64, replace=False))
        mats[(R, K)] = (gpu_matrix(gpu, kind, wp, scale), wdeq[rows], rows)
    for table in (1, 0):
        overrides(gemv_table=table)
        for T in (1, 2, 3, 4):
            for group in ([(C, C)] * 4, [(C, C)], [(H, C), (C, C)], [(C, H)]):
                xs = [gen_f16(rng, (T, K), 1.0) for _, K in group]
                outs = [torch.full((T, R), float("nan"), dtype=torch.float32 if i % 2 else torch.float16, device="cuda") for i, (R, _) in enumerate(group)]
                if len(group) == 1:
                    mats[group[0]][0].matmul_op(dev(xs[0]), outs[0], turbo=False)
                else:
                    gpu.matmul_vec_group([(mats[g][0], dev(x), o, gpu.ACT_NONE, False, {}) for g, x, o in zip(group, xs, outs)])
                for g, x, o in zip(group, xs, outs):
                    _, wsub, rows = mats[g]
                    got = host(o)
                    assert np.isfinite(got).all(), f"{kind} {group} T={T} table={table}"
                    assert_close(got[:, rows], truth_matmul(wsub, x), EPS, f"{kind} {group} T={T} table={table} vs float64")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("C,H", [(1024, 3584), (2048, 7168), (2560, 8960), (2176, 7296)], ids=str)
def test_chunk_tiles_from_the_measured_table(gpu, oracle, kind, C, H, overrides):
    # the launches of the smaller model sizes take their tile shape and split from the measured table
    # (csrc/gemm_tuned.inc): {k, v, r, g}, att.output, {ffn.key, ffn.receptance} and ffn.value at run lengths
    # in several buckets, against float64 on sampled rows -- and once more with the table switched off
    # (gemm_table = 0), where the rules pick the tile.  2176 / 7296 is no model size: its rows and K lie within
    # 7 % of the 2048 / 7168 entries and take them, with row and K counts that fill no tile evenly
    import torch

    announce("chunk tiles from the table", kind, C, H)
    rng = np.random.default_rng(SEED + 47 + C)
    mats = {}
    for R, K in ((C, C), (H, C), (C, H)):
        w = gen_f16(rng, (R, K), 0.02)
        wp, scale, wdeq = pack(oracle, kind, w)
        rows = np.sort(rng.choice(R, 64, replace=False))
        mats[(R, K)] = (gpu_matrix(gpu, kind, wp, scale), wdeq[rows], rows)
    for table in (1, 0):
        overrides(gemm_table=table)
        for T in (6, 24, 40, 96, 130, 256, 300, 500):
            for group in ([(C, C)] * 4, [(C, C)], [(H, C), (C, C)], [(C, H)]):
                xs = [gen_f16(rng, (T, K), 1.0) for _, K in group]
                outs = [torch.full((T, R), float("nan"), dtype=torch.float32 if i % 2 else torch.float16, device="cuda") for i, (R, _) in enumerate(group)]
                if len(group) == 1:
                    mats[group[0]][0].matmul_op(dev(xs[0]), outs[0], turbo=gpu.turbo(T))
                else:
                    gpu.matmul_vec_group([(mats[g][0], dev(x), o, gpu.ACT_NONE, False, {}) for g, x, o in zip(group, xs, outs)])
                for g, x, o in zip(group, xs, outs):
                    _, wsub, rows = mats[g]
                    got = host(o)
                    assert np.isfinite(got).all(), f"{kind} {group} T={T} table={table}"
                    assert_close(got[:, rows], truth_matmul(wsub, x), EPS, f"{kind} {group} T={T} table={table} vs float64")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("T,ksplit", [(128, 2), (256, 1), (252, 1)], ids=str)
def test_chunk_grid_a_little_above_two_workgroups_per_cu(gpu, oracle, kind, T, ksplit, overrides):
    # 576 workgroups (288 tiles of 128 rows x 64 tokens split in two, or 576 tiles) run as two launches:
    # the first 512 as they are, the tiles of the rest with K split 8 ways further, one finish launch
    # for both kinds.  The group {14336, 4096} rows and a single product of 18432 rows both have that
    # grid; with the cut switched off (gemm_tail=0) the results must agree to the same bound.
    import torch

    announce("chunk grid tail", kind, T, ksplit)
    rng = np.random.default_rng(SEED + 43 + T)
    K = 2048
    packed = {}
    for R in (4096, 14336, 18432):
        w = gen_f16(rng, (R, K), 0.02)
        wp, scale, wdeq = pack(oracle, kind, w)
        packed[R] = (gpu_matrix(gpu, kind, wp, scale), wdeq)
    overrides(gemm_kg=1, gemm_mrt=2, gemm_ntile=4, gemm_ksplit=ksplit)
    for tail in (1, 0):
        overrides(gemm_tail=tail)
        for x_dtype in (np.float16, np.float32):
            rows = [14336, 4096]
            xs = [gen_f16(rng, (T, K), 1.0).astype(x_dtype) for _ in rows]
            outs = [torch.full((T, R), float("nan"), dtype=torch.float16 if R == 4096 else torch.float32, device="cuda") for R in rows]
            gpu.matmul_vec_group([(packed[R][0], dev(xv), o, gpu.ACT_SQUARED_RELU if R == 14336 else gpu.ACT_NONE, False, {})
                                  for R, xv, o in zip(rows, xs, outs)])
            for R, xv, o in zip(rows, xs, outs):
                truth = truth_matmul(packed[R][1], xv)
                if R == 14336:
                    truth = np.square(np.maximum(truth, 0.0))
                assert_close(host(o), truth, EPS, f"{kind} group {rows} T={T} tail={tail} {np.dtype(x_dtype).name}")
        m, wdeq = packed[18432]
        x = gen_f16(rng, (T, K), 1.0)
        assert_close(run(gpu, m, x, 18432, "mat", np.float32), truth_matmul(wdeq, x), EPS, f"{kind} 18432 rows T={T} tail={tail}")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
def test_reference_test_data_scale(gpu, oracle, kind):
    # the reference's unit tests draw weights/inputs of magnitude ~1..5, outputs ~100 (ops.rs:2929-2937, 3072-3093)
    announce("reference test scale", kind)
    K, R, T = 2560, 2048, 64
    rng = np.random.default_rng(42)
    w = gen_f16(rng, (R, K), 1.0)
    x = (2.0 * rng.random((T, K), dtype=np.float32) - 1.0).astype(np.float16)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    truth = truth_matmul(wdeq, x)
    assert_close(run(gpu, m, x, R, "mat", np.float32), truth, EPS, "mat")
    assert_close(run(gpu, m, x[:8], R, "vec", np.float32), truth[:8], EPS, "vec")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("act", list(ACTS))
def test_activations(gpu, oracle, kind, act):
    announce("activation", kind, act)
    K, R = 1024, 256
    rng = np.random.default_rng(SEED + 11)
    w = gen_f16(rng, (R, K), 0.03)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    code = list(ACTS).index(act)
    for T, entry in ((1, "vec"), (3, "vec"), (32, "mat")):
        x = gen_f16(rng, (T, K), 1.0)
        got = run(gpu, m, x, R, entry, np.float32, act=code)
        assert_close(got, truth_matmul(wdeq, x, act), EPS, f"{act} {entry} T={T}")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
def test_offset_views_f32_and_batch(gpu, oracle, kind):
    import torch

    announce("views", kind)
    K, R, T = 1024, 128, 4
    rng = np.random.default_rng(SEED + 17)
    w = gen_f16(rng, (R, K), 0.02)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    # v6: att_sx.view(.., .., i, ..) of a [C, T, 5] tensor (src/runtime/v6.rs:806-829), f32 outputs for k/v/r
    for in_dtype in (np.float16, np.float32):
        parent = rng.standard_normal((5, T, K), dtype=np.float32).astype(in_dtype)
        pd = dev(parent)
        for entry in ("vec", "mat"):
            for i in (1, 4):
                out = torch.full((3, T + 2, R), -7.0, dtype=torch.float32, device="cuda")
                views = dict(input_view=((K, T, 1), (K, T, 5), (0, 0, i)), output_view=((R, T, 1), (R, T + 2, 3), (0, 1, 2)))
                (m.matmul_vec_op if entry == "vec" else m.matmul_mat_op)(pd, out, **views)
                got = host(out)
                assert_close(got[2, 1:1 + T], truth_matmul(wdeq, parent[i]), EPS, f"{entry} view {i}")
                got[2, 1:1 + T] = -7.0
                assert (got == -7.0).all(), "wrote outside the output view"
    # batch axis B > 1: matrix [K, R, B], per-batch inputs
    B = 3
    wb = gen_f16(rng, (B, R, K), 0.02)
    xb = gen_f16(rng, (B, T, K), 1.0)
    wpb, sb, wdq = pack(oracle, kind, wb)
    mb = gpu_matrix(gpu, kind, wpb, sb)
    truth = np.stack([truth_matmul(wdq[b], xb[b]) for b in range(B)])
    assert_close(run(gpu, mb, xb, R, "vec", np.float32), truth, EPS, "batched vec")
    assert_close(run(gpu, mb, xb, R, "mat", np.float32), truth, EPS, "batched mat")
    # a matrix view of the leading batches: the one kind of slice for which the reference's scale check (sized by the
    # view) and scale indexing (by the position in the parent) agree
    blocks = 2 * R * K // (64 if kind == "nf4" else 128) * (1 if kind == "nf4" else 2)
    lead = gpu.Matrix(mb.kind, mb.w, mb.m[:blocks].contiguous(), mb.q)
    out2 = torch.full((2, T, R), float("nan"), dtype=torch.float32, device="cuda")
    kx = K // 2 if kind == "nf4" else K
    lead.matmul_mat_op(dev(xb[:2]), out2, matrix_view=((kx, R, 2), (kx, R, B), (0, 0, 0)))
    assert_close(host(out2), truth[:2], EPS, "leading batches of a matrix view")
    with pytest.raises(gpu.TensorError) as e:
        lead.matmul_mat_op(dev(xb[:2]), out2, matrix_view=((kx, R, 2), (kx, R, B), (0, 0, 1)))
    assert e.value.status == gpu.ERR_UNSUPPORTED


@pytest.mark.parametrize("kind", ["int8", "nf4"])
def test_sparse_flag_and_turbo_dispatch(gpu, oracle, kind):
    announce("sparse/turbo", kind)
    K, R = 2688, 768  # ffn.value of the v5 config: sparse (squared-relu) input
    rng = np.random.default_rng(SEED + 19)
    w = gen_f16(rng, (R, K), 0.02)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    x = np.maximum(gen_f16(rng, (1, K), 1.0), 0).astype(np.float16) ** 2
    a = run(gpu, m, x, R, "vec", np.float32, sparse=False)
    b = run(gpu, m, x, R, "vec", np.float32, sparse=True)
    assert np.array_equal(a, b)
    assert_close(a, truth_matmul(wdeq, x), EPS, "sparse input")
    # Matrix::matmul_op picks the chunk kernel iff T % 32 == 0 (src/runtime/v6.rs:568-570)
    import torch

    assert gpu.turbo(32) and gpu.turbo(128) and not gpu.turbo(1) and not gpu.turbo(31)
    for T in (1, 31, 32):
        xt = gen_f16(rng, (T, K), 1.0)
        out = torch.empty((T, R), dtype=torch.float16, device="cuda")
        m.matmul_op_sparse(dev(xt), out, turbo=gpu.turbo(T))
        assert_close(host(out), truth_matmul(wdeq, xt), EPS, f"matmul_op T={T}")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
def test_full_size_properties(gpu, oracle, kind):
    # size-independent checks at a 7B shape: linearity in x, and row permutation of W permutes outputs
    import torch

    announce("full-size properties", kind)
    K, R = 4096, 14336
    g = torch.Generator(device="cuda").manual_seed(SEED)
    w = (torch.randn((R, K), generator=g, device="cuda") * 0.02).half()
    m = gpu.Matrix.quant_u8(w) if kind == "int8" else gpu.Matrix.quant_nf4(w)
    x1 = torch.randn((1, K), generator=g, device="cuda").half()
    x2 = torch.randn((1, K), generator=g, device="cuda").half()
    xs = (x1.float() + x2.float())  # exact in f32
    o1, o2, os_ = (torch.empty((1, R), dtype=torch.float32, device="cuda") for _ in range(3))
    m.matmul_vec_op(x1, o1)
    m.matmul_vec_op(x2, o2)
    m.matmul_vec_op(xs, os_)
    assert_close(host(os_), host(o1 + o2), 1e-4, "linearity")
    perm = torch.randperm(R, generator=g, device="cuda")
    mp = gpu.Matrix.quant_u8(w[perm].contiguous()) if kind == "int8" else gpu.Matrix.quant_nf4(w[perm].contiguous())
    assert torch.equal(mp.w, m.w[perm])  # K % 128 == 0: blocks never straddle rows, packing is per row
    op = torch.empty((1, R), dtype=torch.float32, device="cuda")
    mp.matmul_vec_op(x1, op)
    assert torch.equal(op, o1[:, perm])
    # chunk kernel agrees with the decode kernel on the same tokens
    xt = torch.randn((32, K), generator=g, device="cuda").half()
    ov, om = (torch.empty((32, R), dtype=torch.float32, device="cuda") for _ in range(2))
    for t in range(32):
        m.matmul_vec_op(xt[t:t + 1].contiguous(), ov[t:t + 1])
    m.matmul_mat_op(xt, om)
    assert_close(host(om), host(ov), 2e-4, "mat vs vec")


@pytest.mark.parametrize("kind", ["int8", "nf4"])
@pytest.mark.parametrize("T", [2, 3, 4])
@pytest.mark.parametrize("K,R", [(14336, 516), (4096, 2060), (2048, 16388)], ids=str)
def test_short_runs_on_decode_kernels(gpu, oracle, kind, K, R, T):
    # 2 - 4 tokens share one pass of the decode kernels: long rows (two chunks per lane), row
    # counts that leave a partial task, enough rows for 8 per task, f16 output with an activation
    announce("short run", kind, K, R, T)
    rng = np.random.default_rng(SEED + 29 + T + K)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    wp, scale, wdeq = pack(oracle, kind, w)
    m = gpu_matrix(gpu, kind, wp, scale)
    got = run(gpu, m, x, R, "vec", np.float16, act=gpu.ACT_SILU)
    assert got.shape == (T, R)
    assert_close(got, truth_matmul(wdeq, x, "silu"), EPS, "vs float64")
    one = np.concatenate([run(gpu, m, x[t:t + 1], R, "vec", np.float16, act=gpu.ACT_SILU) for t in range(T)])
    assert_close(got, one, 1e-3, "vs one call per token")  # same arithmetic up to the last f16 ulp


@pytest.mark.parametrize("T,x_dtype", [(1, np.float16), (2, np.float16), (3, np.float32), (32, np.float16), (40, np.float16)])
def test_grouped_nf4_products_keep_their_own_tables(gpu, oracle, T, x_dtype):
    # every Matrix::Fp4 owns its table tensor (src/tensor/matrix.rs:180-222): ops of one group may
    # carry different tables -- here even different contents -- on every kernel family
    # (one-shot, resident with f32 activations, matrix cores)
    import torch

    announce("grouped nf4, own tables", T, x_dtype.__name__)
    K, R = 1024, 768
    rng = np.random.default_rng(SEED + 31 + T)
    tables = [NF4_QUANT, (np.arange(-8, 8) / 8.0).astype(np.float32), NF4_QUANT.copy()]
    x = gen_f16(rng, (T, K), 1.0).astype(x_dtype)
    xd = dev(x)
    ops, outs, truths = [], [], []
    for tab in tables:
        w = gen_f16(rng, (R, K), 0.02)
        p, am = oracle.quant_nf4(w, tab)
        m = gpu.Matrix("Fp4", dev(p), dev(am), torch.tensor(tab, dtype=torch.float32, device="cuda"))
        out = torch.full((T, R), float("nan"), dtype=torch.float32, device="cuda")
        ops.append((m, xd, out, gpu.ACT_NONE, False, {}))
        outs.append(out)
        truths.append(truth_matmul(nf4_dequant64(p, am, tab), x))
    gpu.matmul_vec_group(ops)
    for j, (out, truth) in enumerate(zip(outs, truths)):
        assert_close(host(out), truth, EPS, f"op {j} vs float64 with its own table")


@pytest.mark.parametrize("T", [1, 2, 3, 4, 5, 32])
@pytest.mark.parametrize("kind", ["int8", "nf4"])
def test_grouped_decode_products_equal_single_calls(gpu, oracle, kind, T):
    # the independent products of a layer in shared launches: same results as one call each;
    # one token on the decode kernels, several on the matrix-core kernel (products of one K
    # share a launch there as well)
    import torch

    announce("grouped", kind, T)
    C, H = 1024, 3584
    rng = np.random.default_rng(SEED + 23 + T)
    shapes = [(C, C), (C, C), (C, C), (C, C), (C, H), (H, C)]  # (K, R); the last two differ in K
    mats, truths = [], []
    att_sx = gen_f16(rng, (5, T, C), 1.0)
    xh = gen_f16(rng, (T, H), 1.0)
    for j, (K, R) in enumerate(shapes):
        w = gen_f16(rng, (R, K), 0.02)
        wp, scale, wdeq = pack(oracle, kind, w)
        mats.append(gpu_matrix(gpu, kind, wp, scale))
        x = att_sx[j + 1] if j < 4 else (att_sx[0] if K == C else xh)
        truths.append(truth_matmul(wdeq, x, "squared_relu" if j == 4 else "none"))
    sxd, xhd = dev(att_sx), dev(xh)
    outs_dt = [torch.float32, torch.float32, torch.float32, torch.float16, torch.float16, torch.float16]
    single = [torch.empty((T, R), dtype=dt, device="cuda") for (K, R), dt in zip(shapes, outs_dt)]
    group = [torch.full((T, R), float("nan"), dtype=dt, device="cuda") for (K, R), dt in zip(shapes, outs_dt)]
    ops = []
    for j, (K, R) in enumerate(shapes):
        if j < 4:
            x, views = sxd, dict(input_view=((C, T, 1), (C, T, 5), (0, 0, j + 1)))
        elif K == C:
            x, views = sxd, dict(input_view=((C, T, 1), (C, T, 5), (0, 0, 0)))
        else:
            x, views = xhd, {}
        act = gpu.ACT_SQUARED_RELU if j == 4 else gpu.ACT_NONE
        mats[j].matmul_vec_op(x, single[j], act, **views)
        ops.append((mats[j], x, group[j], act, j == 5, views))
    gpu.matmul_vec_group(ops)
    for j in range(len(shapes)):
        assert_close(host(group[j]), truths[j], EPS, f"group op {j} vs float64")
        # same arithmetic; only the lane count of the final reduction may differ with the group's shapes
        assert_close(host(group[j]), host(single[j]), 1e-3, f"group op {j} vs the single call")  # <= 1 f16 ulp
    # mixed token counts and a chunk-shaped op inside one list are split, not rejected
    x32 = gen_f16(rng, (32, C), 1.0)
    o32 = torch.empty((32, C), dtype=torch.float16, device="cuda")
    o1 = torch.empty((1, C), dtype=torch.float16, device="cuda")
    gpu.matmul_vec_group([(mats[0], dev(x32), o32, 0, False, {}), (mats[1], dev(x32[:1]), o1, 0, False, {})])
    w0 = truth_matmul  # noqa: F841
    torch.cuda.synchronize()
    assert torch.isfinite(o32).all() and torch.isfinite(o1).all()
    # an invalid op anywhere in the list fails the whole call before any launch
    bad = torch.empty((1, C + 4), dtype=torch.float16, device="cuda")
    group[0].fill_(7.0)
    with pytest.raises(gpu.TensorError) as e:
        gpu.matmul_vec_group([ops[0], (mats[1], sxd, bad, 0, False, dict(input_view=((C, T, 1), (C, T, 5), (0, 0, 2))))])
    assert e.value.status == gpu.ERR_SHAPE
    torch.cuda.synchronize()
    assert (group[0] == 7.0).all()

@pytest.mark.parametrize("kind", ["int8", "nf4"])
def test_v5_shape_layer_sequence(gpu, oracle, kind):
    # The quantized call sites of a v5-shape layer (768 wide, FFN 2688) in the order and with the
    # kernel choice of the model builder (src/runtime/v5.rs: att k/v/r/g, att out, ffn key with
    # SquaredRelu, ffn value on the sparse path, ffn receptance; chunk kernels iff T % 32 == 0):
    # a 32-token prompt run, then single-token runs.  Every product is checked against the
    # oracle on the inputs the GPU chain actually produced.
    import torch

    announce("v5-shape layer sequence", kind)
    C, H, LAYERS = 768, 2688, 2
    rng = np.random.default_rng(SEED + 1)
    names = [("att_k", C, C), ("att_v", C, C), ("att_r", C, C), ("att_g", C, C), ("att_o", C, C),
             ("ffn_k", C, H), ("ffn_v", H, C), ("ffn_r", C, C)]
    layers = []
    for _ in range(LAYERS):
        L = {}
        for name, K, R in names:
            wp, scale, _ = pack(oracle, kind, gen_f16(rng, (R, K), 0.02))
            L[name] = (wp, scale, gpu_matrix(gpu, kind, wp, scale))
        layers.append(L)

    def product(entry, name, xd, R, act=0, sparse=False, turbo=False):
        wp, scale, m = entry[name]
        T = xd.shape[0]
        out = torch.full((T, R), float("nan"), dtype=torch.float16, device="cuda")
        if sparse:
            m.matmul_op_sparse(xd, out, act, turbo=turbo)
        else:
            m.matmul_op(xd, out, act, turbo=turbo)
        x = host(xd)
        if turbo:
            ofn = oracle.matmul_mat_int8 if kind == "int8" else oracle.matmul_mat_nf4
            want = ofn(wp, scale, x, act=act)[0]
        else:
            ofn = oracle.matmul_vec_int8 if kind == "int8" else oracle.matmul_vec_nf4
            want = ofn(wp, scale, x, act=act, sparse=sparse)[0]
        assert_close(host(out), want, EPS, f"{kind} {name} T={T}")
        return out

    for T in (32, 1, 1):
        turbo = gpu.turbo(T)
        x = dev(gen_f16(rng, (T, C), 1.0))
        for L in layers:
            k = product(L, "att_k", x, C, turbo=turbo)
            v = product(L, "att_v", x, C, turbo=turbo)
            r = product(L, "att_r", x, C, turbo=turbo)
            g = product(L, "att_g", x, C, turbo=turbo)
            mixed = (torch.sigmoid(r.float()) * (k.float() * v.float()) + g.float()).half()
            x = (x.float() + product(L, "att_o", mixed, C, turbo=turbo).float()).half()
            kk = product(L, "ffn_k", x, H, act=1, turbo=turbo)  # SquaredRelu
            vv = product(L, "ffn_v", kk, C, sparse=True, turbo=turbo)
            rr = product(L, "ffn_r", x, C, turbo=turbo)
            x = (x.float() + torch.sigmoid(rr.float()) * vv.float()).half()


# ---------------------------------------------------------------- plain f16 weights


FP16_CASES = [(2048, 512, 1), (2048, 512, 2), (2048, 516, 3), (4096, 16388, 4), (1056, 64, 7), (4096, 1024, 1), (324, 64, 5), (1056, 64, 3), (2048, 512, 17),
              (2048, 2048, 32), (2560, 2048, 64), (4096, 4096, 128), (2048, 65536, 1), (2048, 65536, 32),
              (32, 4096, 128), (64, 4100, 37), (128, 516, 4), (32, 160, 5)]  # short rows over runs: the adapters' shapes


@pytest.mark.parametrize("K,R,T", FP16_CASES, ids=str)
def test_fp16_matrix_products(gpu, oracle, K, R, T):
    # matmul_vec_fp16 / matmul_mat_fp16 (head and low-rank matrices): one-token kernel, generic
    # kernel (K % 8 != 0), per-token fallback (K % 128 != 0) and the matrix-core kernel
    import torch

    announce("fp16 matrix", K, R, T)
    rng = np.random.default_rng(SEED + 13 + K + R + T)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    m = gpu.Matrix.fp16(dev(w))
    truth = x.astype(np.float64) @ w.astype(np.float64).T
    for entry in (["vec", "mat"] if T % 4 == 0 else ["vec"]):
        for out_dtype in (np.float16, np.float32):
            got = run(gpu, m, x, R, entry, out_dtype)
            assert_close(got, truth, EPS, f"fp16 {K}x{R}x{T} {entry} vs float64")
        assert_close(got, truth, 2e-4, "f32 output vs float64")
    if R * T * K <= 2048 * 2048 * 32:
        assert_close(got, oracle.matmul_vec_fp16(w, x, out_dtype=np.float32)[0], EPS, "vs oracle")
        xf = x.astype(np.float32) * np.float32(1.0009765625)  # f32 activations that are not f16 values
        got32 = run(gpu, m, xf, R, "vec", np.float32, act=1)
        want = np.square(np.maximum(xf.astype(np.float64) @ w.astype(np.float64).T, 0.0))
        assert_close(got32, want, EPS, "f32 activations, squared relu")


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_all_routes(gpu, oracle, seed):
    """Seeded random walk over formats, shapes, token counts, operand types, activations and entry
    points: whatever kernel a call is routed to, the result is the float64 product of the
    dequantised weights."""
    import torch

    rng = np.random.default_rng(SEED + 1000 + seed)
    acts = list(ACTS)
    for case in range(28):
        kind = ["int8", "nf4", "fp16"][int(rng.integers(0, 3))]
        K = int(rng.choice([128, 256, 384, 1024, 2048, 4096, 64, 192, 320, 1056, 96, 2080]))
        if kind == "nf4" and K % 64:
            K += 64 - K % 64
        R = int(rng.choice([4, 8, 36, 64, 132, 512, 1028, 2048]))
        if kind != "fp16":
            while (R * K) % 128:  # whole scale blocks
                R += 4
        T = int(rng.choice([1, 1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 31, 32, 40]))
        x_dtype = np.float16 if rng.random() < 0.7 else np.float32
        out_dtype = np.float16 if rng.random() < 0.5 else np.float32
        act = int(rng.integers(0, len(acts)))
        mat_ok = T % 4 == 0 and K % (64 if kind == "nf4" else 32) == 0 and x_dtype == np.float16
        entry = "mat" if mat_ok and rng.random() < 0.4 else "vec"
        announce("fuzz", seed, case, kind, K, R, T, x_dtype.__name__, out_dtype.__name__, acts[act], entry)
        w = gen_f16(rng, (R, K), 0.05)
        x = gen_f16(rng, (T, K), 1.0).astype(x_dtype)
        if kind == "fp16":
            m, wdeq = gpu.Matrix.fp16(dev(w)), w.astype(np.float64)
        else:
            wp, scale, wdeq = pack(oracle, kind, w)
            m = gpu_matrix(gpu, kind, wp, scale)
        truth = truth_matmul(wdeq, x, acts[act])
        if acts[act] in ("stable_exp", "opposite_exp", "softplus") and not np.isfinite(truth).all():
            continue
        got = run(gpu, m, x, R, entry, out_dtype, act=act)
        assert_close(got, truth, EPS, f"{kind} K={K} R={R} T={T} {entry} act={acts[act]}")


def test_entry_points_from_several_threads(gpu, oracle):
    # ops are built on worker threads in the reference (src/runtime/mod.rs:138-166): the entry
    # points keep no shared mutable state (errors are per thread); every thread drives its own
    # stream and its own decode products here
    import threading

    import torch

    announce("threads")
    K, R = 2048, 512
    rng = np.random.default_rng(SEED + 31)
    cases = []
    for j in range(4):
        kind = "int8" if j % 2 == 0 else "nf4"
        w = gen_f16(rng, (R, K), 0.02)
        x = gen_f16(rng, (1, K), 1.0)
        wp, scale, wdeq = pack(oracle, kind, w)
        cases.append((gpu_matrix(gpu, kind, wp, scale), dev(x), truth_matmul(wdeq, x)))
    torch.cuda.synchronize()
    results, errors = [None] * 4, []

    def work(j):
        try:
            m, xd, _ = cases[j]
            stream = torch.cuda.Stream()
            outs = []
            with torch.cuda.stream(stream):
                for _ in range(50):
                    out = torch.empty((1, R), dtype=torch.float32, device="cuda")
                    m.matmul_vec_op(xd, out)
                    outs.append(out)
                # a failing call on this thread reports this thread's message
                bad = torch.empty((1, R + 4), dtype=torch.float32, device="cuda")
                try:
                    m.matmul_vec_op(xd, bad)
                    errors.append((j, "shape error not raised"))
                except gpu.TensorError as e:
                    if e.status != gpu.ERR_SHAPE or str(R + 4) not in str(e):
                        errors.append((j, str(e)))
            stream.synchronize()
            results[j] = [o.cpu().numpy() for o in outs]
        except Exception as e:  # noqa: BLE001
            errors.append((j, repr(e)))

    threads = [threading.Thread(target=work, args=(j,)) for j in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for j in range(4):
        for o in results[j]:
            assert_close(o, cases[j][2], EPS, f"thread {j}")


def test_split_products_on_several_streams(gpu, oracle, overrides):
    # split-K products keep partial sums in library scratch memory: every stream has a slice of its own, so products of
    # different streams may overlap in time; a stream beyond the slices runs unsplit.  Six streams (more than the slices),
    # each with its own weights and inputs and a pinned 8-way split, launched interleaved; every result against float64.
    import torch

    announce("split-K on several streams")
    K, R, T = 4096, 1024, 32
    rng = np.random.default_rng(SEED + 91)
    overrides(gemm_ksplit=8)
    streams = [torch.cuda.Stream() for _ in range(6)]
    cases = []
    for j, _ in enumerate(streams):
        kind = "int8" if j % 2 == 0 else "nf4"
        w = gen_f16(rng, (R, K), 0.02)
        x = gen_f16(rng, (T, K), 1.0)
        wp, scale, wdeq = pack(oracle, kind, w)
        cases.append((gpu_matrix(gpu, kind, wp, scale), dev(x), truth_matmul(wdeq, x), []))
    torch.cuda.synchronize()
    for rep in range(12):
        for st, (m, xd, _, outs) in zip(streams, cases):
            with torch.cuda.stream(st):
                out = torch.full((T, R), float("nan"), dtype=torch.float32, device="cuda")
                m.matmul_mat_op(xd, out)
                outs.append(out)
    torch.cuda.synchronize()
    for j, (_, _, truth, outs) in enumerate(cases):
        for rep, out in enumerate(outs):
            assert_close(host(out), truth, EPS, f"stream {j} repetition {rep}")


def test_overrides_are_refused_after_the_first_launch_outside_tests():
    # wrq_debug_override is a process-wide table that launches read without a lock: a process that has not declared itself
    # a test (WRQ_TEST_HOOKS) may set overrides before its first launch and is refused afterwards
    import subprocess
    import sys

    announce("override gate")
    code = r'''
import importlib, os, sys
os.environ.pop("WRQ_TEST_HOOKS", None)
import torch
wrq = importlib.import_module("web-rwkv_amd")
assert wrq.lib().wrq_init() == 0
assert wrq.lib().wrq_debug_override(b"gemm_ksplit", 2) == 0          # before any launch: allowed
assert wrq.lib().wrq_debug_override(b"gemm_ksplit", -1) == 0
w = (torch.randn((64, 256), device="cuda") * 0.02).half()
m = wrq.Matrix.quant_u8(w)                                           # launches the packer
torch.cuda.synchronize()
s = wrq.lib().wrq_debug_override(b"gemm_ksplit", 2)
assert s == wrq.ERR_UNSUPPORTED, s
assert b"WRQ_TEST_HOOKS" in wrq.lib().wrq_last_error()
print("gate ok")
'''
    env = {k: v for k, v in os.environ.items() if k != "WRQ_TEST_HOOKS"}
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "gate ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
