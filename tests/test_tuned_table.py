"""The measured tile table of the chunk kernel (web-rwkv_amd/csrc/gemm_tuned.inc) is well formed.

A CPU check of generated data: every filled bucket names a tile shape the kernel is instantiated for and
a split the launcher takes, and no product is listed twice.
"""
import importlib
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rows_of_table():
    text = open(os.path.join(ROOT, "web-rwkv_amd", "csrc", "gemm_tuned.inc")).read()
    pat = re.compile(r"^\{(\d+),\s*(\d+)u,\s*(\d+)u,\s*\{([^}]*)\}\},\s*$", re.M)
    return [(int(q), int(r), int(k), [int(c, 0) for c in cells.split(",")]) for q, r, k, cells in pat.findall(text)]


def test_every_bucket_names_an_instantiated_tile():
    tune = importlib.import_module("web-rwkv_amd.tune_gemm")
    rows = rows_of_table()
    assert rows, "empty table"
    seen = set()
    for quant, r, k, cells in rows:
        assert quant in (0, 1) and r > 0 and k > 0 and k % 128 == 0
        assert (quant, r, k) not in seen, f"product listed twice: {(quant, r, k)}"
        seen.add((quant, r, k))
        assert len(cells) == len(tune.T_GRID)
        assert any(cells), "a row without any filled bucket"
        for bucket, c in zip(tune.T_GRID, cells):
            if c == 0:
                continue
            mrt, ntile, kg, split = c & 15, (c >> 4) & 15, (c >> 8) & 15, c >> 12
            assert (mrt, ntile, kg) in tune.TILES, f"{(quant, r, k)} bucket {bucket}: no kernel for tile {(mrt, ntile, kg)}"
            assert split in tune.SPLITS
            assert 16 * ntile < 2 * max(bucket, 16), f"{(quant, r, k)} bucket {bucket}: token tile wider than the run"


def test_every_decode_cell_names_a_task_shape_the_kernels_have():
    tune = importlib.import_module("web-rwkv_amd.tune_gemm")
    text = open(os.path.join(ROOT, "web-rwkv_amd", "csrc", "gemv_tuned.inc")).read()
    pat = re.compile(r"^\{(\d+),\s*(\d+)u,\s*(\d+)u,\s*\{([^}]*)\}\},\s*$", re.M)
    rows = [(int(q), int(r), int(k), [int(c, 0) for c in cells.split(",")]) for q, r, k, cells in pat.findall(text)]
    assert rows, "empty table"
    seen = set()
    for quant, r, k, cells in rows:
        assert quant in (0, 1) and r > 0 and k > 0
        assert (quant, r, k) not in seen
        seen.add((quant, r, k))
        assert len(cells) == len(tune.DECODE_T) and any(cells)
        for c in cells:
            if c:
                assert (c & 0xfff) in tune.DECODE_LANES and (c >> 12) in tune.DECODE_ROWS


def test_table_generation_keeps_the_rules_where_they_are_close(tmp_path, capsys):
    # `table` fills a bucket only where the fastest combination beats the rules by more than 4 %, prefers the smallest
    # grid among near ties, and lets a second-pass (refined) measurement replace the first pass of its case
    import json

    tune = importlib.import_module("web-rwkv_amd.tune_gemm")
    base = {"quant": "int8", "kind": "x", "C": 256, "H": 512, "n": 1}
    recs = []
    for T, rule, cands in ((8, 10.0, {(1, 1, 2, 1): 9.8, (2, 1, 1, 4): 9.7}),  # within 4 %: the rules stay
                           (16, 10.0, {(1, 1, 2, 1): 8.00, (2, 1, 1, 4): 7.95}),  # near tie: the unsplit one
                           (24, 10.0, {(1, 2, 2, 1): 6.0})):
        recs.append(dict(base, rows=256, K=256, T=T, cfg="rule", us=rule))
        recs += [dict(base, rows=256, K=256, T=T, cfg=list(c), us=u) for c, u in cands.items()]
    # second pass of the last case: the first-pass winner does not hold up
    recs.append(dict(base, rows=256, K=256, T=24, cfg="rule", us=10.0, refined=1))
    recs.append(dict(base, rows=256, K=256, T=24, cfg=[1, 2, 2, 1], us=9.9, refined=1))
    path = tmp_path / "sweep.jsonl"
    path.write_text("".join(json.dumps(r) + "\n" for r in recs))

    class Args:
        files = [str(path)]

    tune.table(Args)
    out = capsys.readouterr().out
    row = [line for line in out.splitlines() if line.startswith("{0,")]
    assert len(row) == 1
    cells = [int(c, 0) for c in re.search(r"\{([^{}]*)\}\},", row[0]).group(1).split(",")]
    assert cells[0] == 0 and cells[2] == 0
    assert cells[1] == (1 | 1 << 4 | 2 << 8 | 1 << 12)
