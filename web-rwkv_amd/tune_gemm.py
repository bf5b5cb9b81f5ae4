"""Sweep of the chunk kernel's tile shapes, and the table the library picks them from.

The matrix-core kernel (csrc/gemm.hip) exists in sixteen tile shapes (rows per workgroup, tokens per
workgroup, K groups inside a workgroup), each with K split 1, 2, 4 or 8 ways over the grid.  Which
one is fastest depends on the product's rows, its K, the run length and the format, and follows no
simple rule at the small end.  This tool measures all of them for the launch kinds of the RWKV model
sizes and writes the winners as a table:

  python3 web-rwkv_amd/tune_gemm.py sweep --out sweep.jsonl     (on an MI355X, about 20 minutes)
  python3 web-rwkv_amd/tune_gemm.py sweep --out refined.jsonl --refine sweep.jsonl
  python3 web-rwkv_amd/tune_gemm.py table sweep.jsonl refined.jsonl > web-rwkv_amd/csrc/gemm_tuned.inc

The one-shot decode kernels (csrc/gemv.hip, runs of 1 .. 4 tokens on products the wave-owns-rows and K-split
kernels do not take) have two such choices, lanes per task and rows per task; `sweep --decode` and
`table --decode` do the same for them (gemv_tuned.inc).

`sweep` pins every combination through wrq_debug_override (WRQ_TEST_HOOKS) and times one HIP graph
of back-to-back launches over enough copies of the packed weights that none is cached; with --refine
it measures the rules and the three fastest combinations of a first pass again, in turn and for
longer, so that drift between short measurements does not pick the winner.  `table`
keeps, per (format, rows, K, run-length bucket), the fastest combination wherever it beats the library's
rules by more than 4 %; the library looks a launch up by format, rows (within 7 %), K (within 7 %) and
the first bucket that holds its run, and falls back to its rules when nothing matches.
"""
import argparse
import collections
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

TILES = [(1, 1, 1), (1, 2, 1), (1, 4, 1), (1, 8, 1), (2, 1, 1), (2, 2, 1), (2, 4, 1), (2, 8, 1), (1, 1, 2), (1, 2, 2), (1, 4, 2), (2, 1, 2), (2, 2, 2),
         (2, 4, 2), (1, 1, 4), (1, 2, 4)]  # (MRT, NTILE, KG): the instantiations of gemm_kernel
SPLITS = (1, 2, 4, 8)
KEYS = ("gemm_mrt", "gemm_ntile", "gemm_kg", "gemm_ksplit")
T_GRID = (8, 16, 24, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256, 320, 384, 448, 512)  # a run of T tokens takes the first bucket >= T

# (C, H, kinds): kinds of launches swept for a model size.  A kind is a list of (rows, K) products that share one launch.
FULL = ("att4", "att3", "att_o", "ffn2", "ffn_k", "ffn_v", "head")
MAIN = ("att4", "att3", "att_o", "ffn2", "ffn_v")
WIDE = ("ffn_k", "ffn_v")  # the layers with FFN = 4 x d_model (v7) share everything else with the 3.5 x ones
SIZES = [(768, 2688, FULL), (1024, 3584, MAIN), (2048, 7168, FULL), (2560, 8960, MAIN), (4096, 14336, FULL), (5120, 17920, MAIN),
         (768, 3072, WIDE), (1024, 4096, WIDE), (2048, 8192, WIDE), (2560, 10240, WIDE), (4096, 16384, WIDE)]


def products(kind, C, H):
    return {"att4": [(C, C)] * 4, "att3": [(C, C)] * 3, "att_o": [(C, C)], "ffn2": [(H, C), (C, C)], "ffn_k": [(H, C)], "ffn_v": [(C, H)],
            "head": [(65536, C)]}[kind]


def sweep(args):
    os.environ.setdefault("WRQ_TEST_HOOKS", "1")
    sys.path.insert(0, ROOT)
    import torch

    wrq = importlib.import_module("web-rwkv_amd")
    f16 = torch.float16
    gen = torch.Generator(device="cuda").manual_seed(7)
    out = open(args.out, "a")
    wrq.debug_override("gemm_table", 0)  # the "rule" rows: the library without its table
    last = [time.time()]
    shortlist = load(args.refine.split(",")) if args.refine else None

    def timed(fn, launches, min_ms=0.0):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps, ms = 3, 0.0
        for attempt in range(2):  # a second, longer pass when the first one was shorter than min_ms
            g.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(reps):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            if ms >= min_ms:
                break
            reps = int(reps * min_ms / max(ms, 1e-3)) + 1
        return ms * 1e3 / reps / launches

    sizes = [s for s in SIZES if not args.sizes or f"{s[0]}x{s[1]}" in args.sizes.split(",")]
    for quant in args.quant.split(","):
        pack = wrq.Matrix.quant_u8 if quant == "int8" else wrq.Matrix.quant_nf4
        for C, H, kinds in sizes:
            for kind in kinds:
                if args.kinds and kind not in args.kinds.split(","):
                    continue
                prods = products(kind, C, H)
                nbytes = sum(r * k for r, k in prods) // (1 if quant == "int8" else 2)
                copies = max(8, min(256, (1 << 30) // nbytes + 1))  # a gigabyte of weights: nothing stays cached
                mats = [[pack((torch.randn((r, k), generator=gen, device="cuda") * 0.02).half()) for r, k in prods] for _ in range(copies)]
                rows, K = sum(r for r, _ in prods), prods[0][1]
                for T in T_GRID:
                    if args.tokens and str(T) not in args.tokens.split(","):
                        continue
                    xs = [torch.randn((T, K), generator=gen, device="cuda").to(f16) for _ in prods]
                    outs = [torch.empty((T, r), dtype=f16, device="cuda") for r, _ in prods]
                    turbo = wrq.turbo(T)

                    def fn():
                        for ms in mats:
                            if len(ms) == 1:
                                ms[0].matmul_op(xs[0], outs[0], turbo=turbo)
                            else:
                                wrq.matmul_vec_group([(m, x, o, wrq.ACT_NONE, False, {}) for m, x, o in zip(ms, xs, outs)])

                    maxnt = 1
                    while maxnt * 16 < T:
                        maxnt *= 2
                    timed(fn, copies)
                    rule = timed(fn, copies)
                    rec = {"quant": quant, "kind": kind, "C": C, "H": H, "rows": rows, "K": K, "n": len(prods), "T": T}
                    out.write(json.dumps(dict(rec, cfg="rule", us=round(rule, 3))) + "\n")
                    wrq.debug_override("gemm_table", -1)
                    tab = timed(fn, copies)  # what the library does by itself, with the table it was built with
                    wrq.debug_override("gemm_table", 0)
                    out.write(json.dumps(dict(rec, cfg="table", us=round(tab, 3))) + "\n")
                    best = (rule, "rule")
                    if shortlist is not None:
                        # second pass: the rules and the three fastest combinations of the first pass, measured in turn, three rounds of
                        # at least 20 ms each, so that drift between measurements does not pick the winner
                        e = shortlist.get((quant, rows, K, T), {})
                        cands = sorted((c for c in e if not isinstance(c, str)), key=e.get)[:3]
                        acc = collections.defaultdict(list)
                        for _ in range(3):
                            wrq.debug_override("gemm_table", 0)
                            acc["rule"].append(timed(fn, copies, 20.0))
                            for c in cands:
                                for k, v in zip(KEYS, c):
                                    wrq.debug_override(k, v)
                                acc[c].append(timed(fn, copies, 20.0))
                                for k in KEYS:
                                    wrq.debug_override(k, -1)
                        for c, v in acc.items():
                            us = sorted(v)[1]  # median of three
                            out.write(json.dumps(dict(rec, cfg=c if isinstance(c, str) else list(c), us=round(us, 3), refined=1)) + "\n")
                            if us < best[0] or best[1] == "rule" and c == "rule":
                                best = (us, c)
                        print(f"{quant} {C:4d}x{H:5d} {kind:6s} rows={rows:6d} K={K:5d} T={T:3d}  rule {acc['rule'][1]:8.2f} us  best {best[0]:8.2f} us {best[1]}", flush=True)
                        out.flush()
                        del xs, outs
                        continue
                    for mrt, nt, kg in TILES:
                        if nt > maxnt or args.defaults_only:
                            continue
                        for ks in SPLITS:
                            wgs = -(-rows * kg // (64 * mrt)) * -(-T // (16 * nt)) * ks
                            if ks > 1 and (wgs > 4096 or K // 128 // ks < 2):
                                continue
                            for k, v in zip(KEYS, (mrt, nt, kg, ks)):
                                wrq.debug_override(k, v)
                            try:
                                us = timed(fn, copies)
                            except Exception as e:  # a combination the library refuses
                                us = None
                                out.write(json.dumps(dict(rec, cfg=[mrt, nt, kg, ks], err=str(e)[:80])) + "\n")
                            for k in KEYS:
                                wrq.debug_override(k, -1)
                            if us is None:
                                continue
                            out.write(json.dumps(dict(rec, cfg=[mrt, nt, kg, ks], us=round(us, 3))) + "\n")
                            if us < best[0]:
                                best = (us, (mrt, nt, kg, ks))
                            if time.time() - last[0] > 20:
                                last[0] = time.time()
                                out.flush()
                                print(f"... {quant} {C}x{H} {kind} T={T}", flush=True)
                    print(f"{quant} {C:4d}x{H:5d} {kind:6s} rows={rows:6d} K={K:5d} T={T:3d}  rule {rule:8.2f} us  table {tab:8.2f} us  best {best[0]:8.2f} us {best[1]}", flush=True)
                    out.flush()
                    del xs, outs
                del mats
                torch.cuda.empty_cache()


DECODE_T = (1, 2, 3, 4)  # run lengths of the one-shot decode kernels
DECODE_LANES = (64, 128, 256, 512)
DECODE_ROWS = (4, 8)


def sweep_decode(args):
    """Lanes per task and rows per task of the one-shot decode kernels (gemv_*_oneshot_kernel), per launch kind and run length:
    the library's own choice and the eight combinations, three rounds in turn of at least 20 ms each, median."""
    os.environ.setdefault("WRQ_TEST_HOOKS", "1")
    sys.path.insert(0, ROOT)
    import torch

    wrq = importlib.import_module("web-rwkv_amd")
    gen = torch.Generator(device="cuda").manual_seed(7)
    out = open(args.out, "a")
    wrq.debug_override("gemv_table", 0)

    def timed(fn, launches, min_ms=20.0):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps, ms = 3, 0.0
        for attempt in range(2):
            g.replay()
            torch.cuda.synchronize()
            e0.record()
            for _ in range(reps):
                g.replay()
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            if ms >= min_ms:
                break
            reps = int(reps * min_ms / max(ms, 1e-3)) + 1
        return ms * 1e3 / reps / launches

    sizes = [s for s in SIZES if not args.sizes or f"{s[0]}x{s[1]}" in args.sizes.split(",")]
    for quant in args.quant.split(","):
        pack = wrq.Matrix.quant_u8 if quant == "int8" else wrq.Matrix.quant_nf4
        for C, H, kinds in sizes:
            for kind in kinds:
                if args.kinds and kind not in args.kinds.split(","):
                    continue
                prods = products(kind, C, H)
                nbytes = sum(r * k for r, k in prods) // (1 if quant == "int8" else 2)
                copies = max(8, min(256, (1 << 30) // nbytes + 1))
                mats = [[pack((torch.randn((r, k), generator=gen, device="cuda") * 0.02).half()) for r, k in prods] for _ in range(copies)]
                rows, K = sum(r for r, _ in prods), prods[0][1]
                for T in DECODE_T:
                    xs = [torch.randn((T, K), generator=gen, device="cuda").half() for _ in prods]
                    outs = [torch.empty((T, r), dtype=torch.float16, device="cuda") for r, _ in prods]

                    def fn():
                        for ms in mats:
                            if len(ms) == 1:
                                ms[0].matmul_op(xs[0], outs[0], turbo=False)
                            else:
                                wrq.matmul_vec_group([(m, x, o, wrq.ACT_NONE, False, {}) for m, x, o in zip(ms, xs, outs)])

                    timed(fn, copies, 5.0)
                    acc = collections.defaultdict(list)
                    for _ in range(3):
                        acc["rule"].append(timed(fn, copies))
                        for nt in DECODE_LANES:
                            for nrows in DECODE_ROWS:
                                wrq.debug_override("gemv_nt", nt)
                                wrq.debug_override("gemv_rows", nrows)
                                acc[(nt, nrows)].append(timed(fn, copies))
                                wrq.debug_override("gemv_nt", -1)
                                wrq.debug_override("gemv_rows", -1)
                    rec = {"quant": quant, "kind": kind, "C": C, "H": H, "rows": rows, "K": K, "n": len(prods), "T": T, "decode": 1}
                    med = {c: sorted(v)[1] for c, v in acc.items()}
                    for c, us in med.items():
                        out.write(json.dumps(dict(rec, cfg=c if isinstance(c, str) else list(c), us=round(us, 3))) + "\n")
                    best = min((c for c in med if c != "rule"), key=med.get)
                    print(f"{quant} {C:4d}x{H:5d} {kind:6s} rows={rows:6d} K={K:5d} T={T}  rule {med['rule']:7.2f} us  best {med[best]:7.2f} us {best}", flush=True)
                    out.flush()
                    del xs, outs
                del mats
                torch.cuda.empty_cache()


def table_decode(args):
    data = load(args.files, decode=True)
    shapes = sorted({(q, rows, K) for q, rows, K, _ in data})
    print("// Generated by web-rwkv_amd/tune_gemm.py (sweep --decode, table --decode) on an MI355X; do not edit by hand.")
    print("// One row per (format, rows of the launch, K): for runs of 1, 2, 3 and 4 tokens on the one-shot decode kernels the fastest")
    print("// lanes per task | rows per task << 12 where it beats the rules by more than 4 %; 0 = the rules decide.")
    filled = 0
    for q, rows, K in shapes:
        cells = []
        for T in DECODE_T:
            e = data.get((q, rows, K, T), {})
            cands = {c: u for c, u in e.items() if not isinstance(c, str)}
            if not cands or "rule" not in e:
                cells.append("0")
                continue
            best = min(cands, key=cands.get)
            near = [c for c, u in cands.items() if u <= cands[best] * 1.01]
            best = min(near, key=lambda c: (c[0], c[1]))  # the smallest task among near ties
            if e["rule"] < cands[best] * 1.04:
                cells.append("0")
                continue
            filled += 1
            cells.append("0x%04x" % (best[0] | best[1] << 12))
        if any(c != "0" for c in cells):
            print("{%d, %6du, %6du, {%s}}," % (0 if q == "int8" else 1, rows, K, ", ".join(cells)))
    print(f"// {filled} cells filled")


def load(paths, decode=False):
    d = collections.defaultdict(dict)
    refined = set()
    for p in paths:
        for line in open(p):
            r = json.loads(line)
            if "us" not in r:
                continue
            if bool(r.get("decode")) != decode:
                continue
            key = (r["quant"], r["rows"], r["K"], r["T"])
            if r.get("refined") and key not in refined:  # a second-pass measurement replaces the first pass of its case
                refined.add(key)
                d[key] = {}
            if key in refined and not r.get("refined"):
                continue
            cfg = r["cfg"] if isinstance(r["cfg"], str) else tuple(r["cfg"])
            d[key].setdefault(cfg, []).append(r["us"])
    return {k: {c: sum(v) / len(v) for c, v in e.items()} for k, e in d.items()}


def table(args):
    data = load(args.files)
    shapes = sorted({(q, rows, K) for q, rows, K, _ in data})
    print("// Generated by web-rwkv_amd/tune_gemm.py from a sweep of every tile shape and split on an MI355X; do not edit by hand.")
    print("// One row per (format, rows of the launch, K): for each run-length bucket (" + ", ".join(str(t) for t in T_GRID[:10]) + ",")
    print("// " + ", ".join(str(t) for t in T_GRID[10:]) + " tokens) the fastest combination, packed as MRT | NTILE << 4 | KG << 8 | split << 12; 0 = the rules decide.")
    gain = []
    for q, rows, K in shapes:
        cells = []
        for T in T_GRID:
            e = data.get((q, rows, K, T))
            if not e:
                cells.append("0")
                continue
            cands = {c: u for c, u in e.items() if not isinstance(c, str)}
            if not cands:
                cells.append("0")
                continue
            best = min(cands, key=cands.get)
            # the smallest grid among those within 1 % of the fastest: the less scratch and the fewer workgroups the better
            near = [c for c, u in cands.items() if u <= cands[best] * 1.01]
            best = min(near, key=lambda c: (c[3], c[2], -c[0] * c[1]))
            if "rule" in e and e["rule"] < cands[best] * 1.04:
                # the rules are within 4 % (two measurements' noise) of the fastest: they stay in charge of this bucket
                cells.append("0")
                continue
            cells.append("0x%04x" % (best[0] | best[1] << 4 | best[2] << 8 | best[3] << 12))
            if "rule" in e:
                gain.append((e["rule"] / cands[best] - 1, q, rows, K, T))
        if any(c != "0" for c in cells):
            print("{%d, %6du, %6du, {%s}}," % (0 if q == "int8" else 1, rows, K, ", ".join(cells)))
    if gain:
        mean = sum(g[0] for g in gain) / len(gain)
        print(f"// {len(gain)} buckets filled (the rules keep the others): {100 * mean:.1f} % faster than the rules on average at sweep time, at most {100 * max(gain)[0]:.0f} %")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    s = sub.add_parser("sweep")
    s.add_argument("--out", required=True)
    s.add_argument("--quant", default="int8,nf4")
    s.add_argument("--sizes", default="", help="comma-separated CxH subset, e.g. 4096x14336")
    s.add_argument("--tokens", default="", help="comma-separated run-length buckets, e.g. 320,384 (chunk sweep)")
    s.add_argument("--kinds", default="", help="comma-separated launch kinds, e.g. att3,ffn_k")
    s.add_argument("--decode", action="store_true", help="sweep the one-shot decode kernels (lanes and rows per task at 1 .. 4 tokens) instead of the chunk kernel")
    s.add_argument("--refine", default="", help="comma-separated sweep files: measure only their three fastest combinations per case, longer and in turn")
    s.add_argument("--defaults-only", action="store_true", help="time only the library's own choices, with and without the table")
    t = sub.add_parser("table")
    t.add_argument("--decode", action="store_true", help="write gemv_tuned.inc from a sweep --decode")
    t.add_argument("files", nargs="+")
    args = ap.parse_args()
    if args.cmd == "sweep":
        (sweep_decode if args.decode else sweep)(args)
    else:
        (table_decode if args.decode else table)(args)


if __name__ == "__main__":
    main()
