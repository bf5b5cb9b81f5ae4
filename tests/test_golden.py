"""The committed fixtures of tests/golden (exact rational arithmetic on the closed forms of the
reference's unit tests, and the literal tuples of its schedule tests; see make_golden.py) against
the oracle, the schedule restatement used by bench.py, and -- marked gpu -- the HIP library."""
import importlib
import json
import os
import sys

import numpy as np
import pytest

from helpers import EPS, assert_close

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
with open(os.path.join(HERE, "golden", "exact_pack_and_products.json")) as f:
    GOLDEN = json.load(f)
with open(os.path.join(HERE, "golden", "rnn_iter_kats.json")) as f:
    RNN = json.load(f)
CASES = GOLDEN["cases"]
IDS = [f"{c['kind']}-{c['K']}x{c['R']}x{c['T']}" for c in CASES]


def arrays(c):
    w = np.array(c["w_f16_bits"], dtype=np.uint16).view(np.float16).reshape(c["R"], c["K"])
    x = np.array(c["x_f16_bits"], dtype=np.uint16).view(np.float16).reshape(c["T"], c["K"])
    return w, x


def check_packing(c, packed, scales):
    """codes / nibbles equal the exact ones except where the exact value sits on a rounding boundary"""
    sens = np.zeros(c["R"] * c["K"], dtype=bool)
    sens[c["sensitive"]] = True
    if c["kind"] == "int8":
        want = np.array(c["codes"], dtype=np.uint8)
        got = np.asarray(packed).reshape(-1)
        want_scale = np.array(c["minmax_f16_bits"], dtype=np.uint16)
    else:
        by = np.asarray(packed).reshape(-1)
        got = np.stack([by & 15, by >> 4], axis=1).reshape(-1)
        wb = np.array(c["bytes"], dtype=np.uint8)
        want = np.stack([wb & 15, wb >> 4], axis=1).reshape(-1)
        want_scale = np.array(c["absmax_f16_bits"], dtype=np.uint16)
    assert np.array_equal(np.asarray(scales).reshape(-1).view(np.uint16), want_scale), "scales bit-exact"
    diff = got != want
    assert not (diff & ~sens).any(), f"{int((diff & ~sens).sum())} codes differ away from rounding boundaries"
    assert np.abs(got.astype(int) - want.astype(int))[diff].max(initial=0) <= 1
    assert sens.sum() < 0.01 * sens.size  # the fixture is decisive for > 99 % of the elements


@pytest.mark.parametrize("c", CASES, ids=IDS)
def test_oracle_against_exact_fixtures(oracle, c):
    w, x = arrays(c)
    if c["kind"] == "int8":
        p, s, _flagged = oracle.quant_int8(w)
        out = oracle.matmul_vec_int8(p, s, x, out_dtype=np.float32)[0]
        mat = oracle.matmul_mat_int8(p, s, x, out_dtype=np.float32)[0]
    else:
        p, s = oracle.quant_nf4(w, np.array(GOLDEN["nf4_table"], dtype=np.float32))
        out = oracle.matmul_vec_nf4(p, s, x, out_dtype=np.float32)[0]
        mat = oracle.matmul_mat_nf4(p, s, x, out_dtype=np.float32)[0]
    check_packing(c, p, s)
    if not c["sensitive"]:  # products of the exact codes: comparable when no code is ambiguous
        assert_close(out, np.array(c["product_f64"]), EPS, "vec vs exact product")
        if c["T"] % 4 == 0:  # the mat entry points take multiples of 4 tokens (ops.rs:1068-1070, 1146-1149)
            assert_close(mat, np.array(c["product_f64"]), EPS, "mat vs exact product")
    else:
        assert_close(out, np.array(c["product_f64"]), 5e-3, "vec vs exact product (codes within 1 at boundaries)")


def test_schedule_restatement_against_reference_tuples():
    sys.path.insert(0, ROOT)
    bench = importlib.import_module("bench")
    k = RNN["run_iter"]
    state = [[False, n] for n in k["lengths"]]
    for want in k["runs"]:
        assert bench.rnn_iter_next(state, k["chunk"]) == want
    k = RNN["advance_refilled"]
    state = [[False, n] for n in k["lengths"]]
    assert bench.rnn_iter_next(state, k["chunk"]) == k["runs"][0]
    # test_advance: what is left to read after the first run is taken off the input
    k = RNN["advance"]
    state = [[False, n] for n in k["lengths"]]
    first = bench.rnn_iter_next(state, k["chunk"])
    left = [n - t for n, t in zip(k["lengths"], first)]
    state = [[False, n] for n in left]
    assert bench.rnn_iter_next(state, k["chunk"]) == k["after_one_step_first_run"]


@pytest.mark.gpu
@pytest.mark.parametrize("c", CASES, ids=IDS)
def test_library_against_exact_fixtures(gpu, c):
    import torch

    print("golden fixture on the GPU", c["kind"], c["K"], c["R"], c["T"], flush=True)
    w, x = arrays(c)
    wd = torch.from_numpy(w.copy()).cuda()
    xd = torch.from_numpy(x.copy()).cuda()
    if c["kind"] == "int8":
        m = gpu.Matrix.quant_u8(wd)
        packed, scales = m.w.cpu().numpy(), m.m.cpu().numpy()
    else:
        m = gpu.Matrix.quant_nf4(wd, np.array(GOLDEN["nf4_table"], dtype=np.float32))
        packed, scales = m.w.cpu().numpy(), m.m.cpu().numpy()
    check_packing(c, packed, scales)
    want = np.array(c["product_f64"])
    eps = EPS if not c["sensitive"] else 5e-3
    for entry in ("vec", "mat") if c["T"] % 4 == 0 else ("vec",):
        out = torch.empty((c["T"], c["R"]), dtype=torch.float32, device="cuda")
        (m.matmul_vec_op if entry == "vec" else m.matmul_mat_op)(xd, out)
        assert_close(out.cpu().numpy(), want, eps, f"{entry} vs exact product")


# ---------------------------------------------------------------------------------------------
# the recurrences of the four model versions against committed float64 vectors
# (tests/golden/recurrent_float64.json, written by make_recurrent_golden.py beside it)
with open(os.path.join(HERE, "golden", "recurrent_float64.json")) as f:
    REC = json.load(f)


def rec_arrays(version):
    c, H, S, B = REC[version], REC["H"], REC["S"], REC["B"]
    A = sum(n for _, n in REC["runs"])
    f32 = lambda key, *shape: np.array(c[key], dtype=np.float32).reshape(shape)
    f64 = lambda key, *shape: np.array(c[key], dtype=np.float64).reshape(shape)
    return c, H, S, B, A, f32, f64


def run_recurrence(version, ops, cursors, to_dev, to_host, dtype):
    """`ops`: the oracle module or the library's LayerOp; returns (y, state after) as numpy arrays."""
    c, H, S, B, A, f32, f64 = rec_arrays(version)
    C = H * S
    cast = lambda a: a.astype(dtype)
    if version == "v4":
        state = f32("state", B, 4, C)
        k, v, r, x = (cast(f32(n, A, C)) for n in ("k", "v", "r", "x"))
        w, u = f32("time_decay", C), f32("time_first", C)
        return state, (k, v, r, x, w, u)
    state = f32("state", B, S + 1, C)
    if version == "v7":
        return state, (cast(f32("r", A, H, S)), cast(f32("w", A, H, S)), cast(f32("n", 4, A, H, S)), cast(f32("x", A, H, S)))
    wshape = (A, H, S) if version == "v6" else (H, S)
    k, v, r, x = (cast(f32(n, A, H, S)) for n in ("k", "v", "r", "x"))
    return state, (k, v, r, x, f32("time_decay", *wshape), f32("time_first", H, S))


def check_recurrence(version, y, state_after, eps_y, eps_state):
    c, H, S, B, A, f32, f64 = rec_arrays(version)
    C = H * S
    if version == "v4":
        assert_close(y, f64("y", A, C), eps_y, "v4 y vs float64 fixture")
        st = state_after.astype(np.float64)
        assert_close(st[:, 1] * np.exp(st[:, 3]), f64("numerator_after", B, C), eps_state, "v4 numerator")
        assert_close(st[:, 2] * np.exp(st[:, 3]), f64("denominator_after", B, C), eps_state, "v4 denominator")
        assert_close(st[:, 0], f64("row0_after", B, C), 1e-7, "v4 row 0")
        return
    assert_close(y, f64("y", A, H, S), eps_y, f"{version} y vs float64 fixture")
    assert_close(state_after, f64("state_after", B, S + 1, C), eps_state, f"{version} state vs float64 fixture")


@pytest.mark.parametrize("version", ["v4", "v5", "v6", "v7"])
def test_oracle_recurrences_against_float64_fixtures(version):
    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    cursors = lop.pack_cursors([tuple(r) for r in REC["runs"]])
    state, a = run_recurrence(version, lop, cursors, None, None, np.float32)
    if version == "v4":
        k, v, r, x, w, u = a
        y = lop.time_mix_v4(cursors, w, u, state, k, v, r, x)
    elif version == "v7":
        r, w, n, x = a
        y = lop.time_mix_v7(cursors, state, r, w, n, x)
    else:
        k, v, r, x, w, u = a
        y = (lop.time_mix_v5 if version == "v5" else lop.time_mix_v6)(cursors, w, u, state, k, v, r, x)
    check_recurrence(version, y, state, 2e-5, 2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("version", ["v4", "v5", "v6", "v7"])
def test_library_recurrences_against_float64_fixtures(gpu, version, dtype):
    import torch

    print("recurrence fixture on the GPU", version, dtype.__name__, flush=True)
    sys.path.insert(0, ROOT)
    lop = importlib.import_module("oracle.layer_ops")
    cursors = lop.pack_cursors([tuple(r) for r in REC["runs"]])
    state, a = run_recurrence(version, None, cursors, None, None, dtype)
    dev = lambda t: torch.from_numpy(np.ascontiguousarray(t)).cuda()
    cur, sd = dev(cursors.view(np.int32)), dev(state)
    if version == "v4":
        k, v, r, x, w, u = a
        A, C = x.shape
        xd = dev(x.reshape(1, A, C))
        gpu.LayerOp.time_mix_v4(cur, dev(w), dev(u), sd, dev(k.reshape(1, A, C)), dev(v.reshape(1, A, C)), dev(r.reshape(1, A, C)), xd)
        y = xd.cpu().numpy()[0]
    elif version == "v7":
        r, w, n, x = a
        xd = dev(x)
        gpu.LayerOp.time_mix_v7(cur, sd, dev(r), dev(w), dev(n), xd)
        y = xd.cpu().numpy()
    else:
        k, v, r, x, w, u = a
        xd = dev(x)
        (gpu.LayerOp.time_mix_v5 if version == "v5" else gpu.LayerOp.time_mix_v6)(cur, dev(w), dev(u), sd, dev(k), dev(v), dev(r), xd)
        y = xd.cpu().numpy()
    # f16 operands are the fixture's values exactly (they were drawn as f16); an f16 result carries its rounding
    check_recurrence(version, y, sd.cpu().numpy(), 2e-3 if dtype == np.float16 else 5e-5, 5e-5)
