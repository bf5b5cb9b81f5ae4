"""Pins the oracle's packers (CPU only).

Checks are independent of the oracle's own formulas: the reference tests' closed forms,
exact float64 arithmetic, invariants, and brute force over every finite f16 value.
"""
import numpy as np
import pytest

from helpers import (NF4_QUANT, gen_f16, int8_dequant64, int8_f64_form, int8_test_form,
                     nf4_dequant64, nf4_test_form, nf4_unpack)


def test_f16_conversions_match_numpy(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10,
        rng.standard_normal(200000).astype(np.float32) * 1e-5,  # subnormal range
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0**-24, 2.0**-25,
                  2.0**-25 * 1.0001, 5.96e-8, 6.1e-5, np.inf, -np.inf], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    got = oracle.f32_to_f16(x)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # every f16 bit pattern widens exactly
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    got32 = oracle.f16_to_f32(allh)
    want32 = allh.astype(np.float32)
    assert np.array_equal(got32.view(np.uint32)[~np.isnan(want32)], want32.view(np.uint32)[~np.isnan(want32)])
    assert np.isnan(got32[np.isnan(want32)]).all()


@pytest.mark.parametrize("shape,std", [((64, 320), 2.9), ((256, 2560), 2.9), ((128, 2048), 0.02)])
def test_int8_against_reference_test_form(oracle, shape, std):
    rng = np.random.default_rng(42)
    # the reference test draws 10*(U-0.5); any finite f16 data exercises the same formula
    w = (10.0 * (rng.random(shape, dtype=np.float32) - 0.5)).astype(np.float16) if std == 2.9 else gen_f16(rng, shape, std)
    u8, minmax, flagged = oracle.quant_int8(w)
    want_u8, want_mm, tie = int8_test_form(w)
    # scales bit-exact, (min, max) interleaved (ops.rs:2963-2966)
    assert np.array_equal(minmax.view(np.uint16), want_mm.view(np.uint16))
    diff = u8.astype(np.int32) - want_u8.astype(np.int32)
    assert np.abs(diff).max() <= 1  # the reference's own bar (ops.rs:2995-3000)
    # away-from-zero vs half-even can only differ on exact ties of the f32 product
    assert not (diff != 0)[~tie].any()
    assert flagged >= int(tie.sum())
    assert flagged < 5e-3 * w.size + 4


def test_int8_against_exact_arithmetic(oracle):
    rng = np.random.default_rng(7)
    w = gen_f16(rng, (512, 1024), 0.02)
    u8, minmax, _ = oracle.quant_int8(w)
    s = int8_f64_form(w)
    frac = s - np.floor(s)
    clear = np.abs(frac - 0.5) > 1e-3  # f32 rounding of the quotient cannot cross these
    assert clear.mean() > 0.99
    assert np.array_equal(u8[clear], np.rint(s[clear]).astype(np.uint8))
    # invariants: block min -> 0, block max -> 255, round trip within half a step
    w64 = w.astype(np.float64).reshape(-1, 128)
    b = u8.reshape(-1, 128)
    assert (b[np.arange(len(b)), w64.argmin(axis=1)] == 0).all()
    assert (b[np.arange(len(b)), w64.argmax(axis=1)] == 255).all()
    deq = int8_dequant64(u8, minmax).reshape(-1, 128)
    step = (w64.max(axis=1) - w64.min(axis=1)) / 255.0
    assert (np.abs(deq - w64) <= 0.5 * step[:, None] * (1 + 1e-5) + 1e-12).all()


def test_int8_every_f16_value_in_a_block(oracle):
    # blocks [min=-a, max=a, 126 probes]: all finite f16 magnitudes up to a pass through the packer
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    for a in (1.0, 0.0731, 37.5):
        probes = allh[np.isfinite(allh) & (np.abs(allh.astype(np.float32)) <= a)]
        pad = (-len(probes)) % 126
        probes = np.concatenate([probes, np.zeros(pad, dtype=np.float16)]).reshape(-1, 126)
        blocks = np.concatenate([np.full((len(probes), 1), -a, np.float16),
                                 np.full((len(probes), 1), a, np.float16), probes], axis=1)
        u8, minmax, _ = oracle.quant_int8(blocks)
        s = int8_f64_form(blocks)
        frac = s - np.floor(s)
        clear = np.abs(frac - 0.5) > 1e-3
        assert np.array_equal(u8[clear], np.rint(s[clear]).astype(np.uint8))
        assert np.abs(u8.astype(np.float64) - s).max() <= 0.5 + 1e-3


def test_int8_constant_block_policy(oracle):
    w = np.full((2, 128), 0.25, dtype=np.float16)
    w[1, 5] = 0.5
    u8, minmax, flagged = oracle.quant_int8(w)
    assert (u8[0] == 0).all()  # 0/0 -> NaN -> clamp gives 0: dequantises to min exactly
    assert minmax[0] == minmax[1] == np.float16(0.25)
    assert u8[1, 5] == 255 and (np.delete(u8[1], 5) == 0).all()
    assert flagged >= 128


@pytest.mark.parametrize("shape", [(64, 320), (128, 2560)])
def test_nf4_against_reference_test_form(oracle, shape):
    rng = np.random.default_rng(42)
    w = rng.standard_normal(shape, dtype=np.float32).astype(np.float16)  # N(0,1) as ops.rs:3072-3083
    packed, absmax = oracle.quant_nf4(w)
    want_packed, want_am, x = nf4_test_form(w)
    assert np.array_equal(absmax.view(np.uint16), want_am.view(np.uint16))
    got, want = nf4_unpack(packed), nf4_unpack(want_packed)
    # nibble order: byte p = idx[2p] | idx[2p+1] << 4 (ops.rs:3139-3141)
    mism = got != want
    # v*(1/a) vs v/a and '<=' vs '<' may only disagree within a few ulp of a midpoint
    mid = ((NF4_QUANT[1:] + NF4_QUANT[:-1]) / 2).astype(np.float64)
    dist = np.abs(x.astype(np.float64)[..., None] - mid).min(axis=-1)
    assert (dist[mism] < 1e-6).all()
    assert mism.mean() < 1e-4
    assert np.abs(got.astype(int) - want.astype(int)).max() <= 1


def test_nf4_every_f16_value(oracle):
    allh = np.arange(65536, dtype=np.uint16).view(np.float16)
    q64 = NF4_QUANT.astype(np.float64)
    mid = (q64[1:] + q64[:-1]) / 2
    for a in (1.0, 0.0731, 37.5):
        probes = allh[np.isfinite(allh) & (np.abs(allh.astype(np.float32)) <= a)]
        pad = (-len(probes)) % 63
        probes = np.concatenate([probes, np.zeros(pad, dtype=np.float16)]).reshape(-1, 63)
        blocks = np.concatenate([np.full((len(probes), 1), a, np.float16), probes], axis=1)
        packed, absmax = oracle.quant_nf4(blocks)
        assert (absmax == np.float16(a)).all()
        idx = nf4_unpack(packed)
        x = blocks.astype(np.float64) / float(np.float16(a))
        want = np.searchsorted(mid, x)  # nearest quantile in exact arithmetic
        clear = np.abs(x[..., None] - mid).min(axis=-1) > 1e-6
        assert np.array_equal(idx[clear], want[clear].astype(np.uint8))
        assert np.abs(idx.astype(int) - want).max() <= 1


def test_nf4_special_values(oracle):
    w = np.zeros((3, 64), dtype=np.float16)
    w[1, 0], w[1, 1], w[1, 2] = 0.5, -0.5, 0.0
    w[2, :] = 0.0  # all-zero block: 1/0 = inf, 0*inf = NaN, no comparison succeeds -> nibble 0
    w[0, :] = np.linspace(-1, 1, 64).astype(np.float16)
    packed, absmax = oracle.quant_nf4(w)
    idx = nf4_unpack(packed)
    assert idx[1, 0] == 15 and idx[1, 1] == 0 and idx[1, 2] == 7
    assert (idx[1, 3:] == 7).all()
    assert (packed[2] == 0).all() and absmax[2] == 0
    assert idx[0, 0] == 0 and idx[0, -1] == 15
    assert (np.diff(idx[0].astype(int)) >= 0).all()
    # custom table is honoured (SF4 swaps the table, src/tensor/matrix.rs:202-222)
    table = np.linspace(-1, 1, 16).astype(np.float32)
    packed2, _ = oracle.quant_nf4(w[:1], table)
    x = w[0].astype(np.float64)
    want = np.abs(x[:, None] - table.astype(np.float64)[None, :]).argmin(axis=1)
    got = nf4_unpack(packed2)[0]
    assert (np.abs(got.astype(int) - want) <= 1).all() and (got == want).mean() > 0.9


def test_nf4_round_trip_error_bound(oracle):
    rng = np.random.default_rng(3)
    w = gen_f16(rng, (256, 1024), 0.02)
    packed, absmax = oracle.quant_nf4(w)
    deq = nf4_dequant64(packed, absmax).reshape(-1, 64)
    w64 = w.astype(np.float64).reshape(-1, 64)
    half_gap = np.diff(NF4_QUANT.astype(np.float64)).max() / 2
    assert (np.abs(deq - w64) <= absmax.astype(np.float64)[:, None] * half_gap * (1 + 1e-6)).all()
