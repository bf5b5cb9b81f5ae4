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
