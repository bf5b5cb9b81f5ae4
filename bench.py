#!/usr/bin/env python3
"""Benchmark of the quantized-weight matrix path on one MI355X.

Default workload (config 4 of the baseline): one decode step, batch 1, of an RWKV-v6
7B-shaped model (32 layers, d_model 4096, FFN 14336) with every layer Int8-quantized.  A
"step" streams all packed weights of the path once: per layer the products att.key /
value / receptance / gate / output (4096 -> 4096), ffn.key (4096 -> 14336, squared ReLU),
ffn.value (14336 -> 4096, sparse hint) and ffn.receptance, with the reference's operand
types and views (src/runtime/v6.rs:806-829, :880-885, :920-938).  Only this path is timed:
the recurrent, normalisation and head ops of the model are not part of this library.

Weights are random-init f16 ~ N(0, 0.02) (att.output and ffn.value pre-multiplied by
2^-(layer / 6), src/runtime/loader.rs:734-762) packed on the GPU by the library itself;
inputs are resident in HBM before the timed region.

Prints one JSON line: metric / value (tok/s of the path) / unit / n_gpus / steps / warmup /
ms_per_step / dtype / config, `roofline` (algorithmic bytes per launch over the average launch
duration against 8 TB/s, measured HBM traffic) and `cpu_baseline` (the CPU restatement on the
host cores).  `--sweep` prints per-operator figures instead, `--schedule` a multi-slot serving
schedule, `--tokens N` steps of N tokens, `--with-head` adds the f16 head.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense f16 matrix cores
SEED = 0x57525100


def int8_bytes(K, R, T=1, out_size=2):
    """Algorithmic bytes of one int8 product: weights + (min,max) pairs + input + output."""
    return K * R + 4 * K * R // 128 + 2 * K * T + out_size * R * T


def fp16_bytes(K, R, T=1, out_size=2):
    """Plain f16 weights (head, low-rank matrices): 2 bytes per weight."""
    return 2 * K * R + 2 * K * T + out_size * R * T


def nf4_bytes(K, R, T=1, out_size=2):
    return K * R // 2 + 2 * K * R // 64 + 64 + 2 * K * T + out_size * R * T


MODEL_SHAPES = {"0b4": (1024, 3584, 24), "1b6": (2048, 7168, 24), "3b": (2560, 8960, 32), "7b": (4096, 14336, 32), "14b": (5120, 17920, 61)}  # d_model, FFN, layers (v6)


class Layer:
    pass


def build_model(wrq, torch, quant, n_layer, C, H, rescale=6):
    """Random-init packed weights of the eight quantized matrices per layer."""
    g = torch.Generator(device="cuda").manual_seed(SEED + 4)
    pack = wrq.Matrix.quant_u8 if quant == "int8" else wrq.Matrix.quant_nf4
    layers = []
    for i in range(n_layer):
        discount = 2.0 ** -(i // rescale)
        L = Layer()

        def mat(R, K, scale=1.0):
            w = (torch.randn((R, K), generator=g, device="cuda") * (0.02 * scale)).half()
            return pack(w)

        L.att_k, L.att_v, L.att_r, L.att_g = (mat(C, C) for _ in range(4))
        L.att_o = mat(C, C, discount)
        L.ffn_k = mat(H, C)
        L.ffn_v = mat(C, H, discount)
        L.ffn_r = mat(C, C)
        layers.append(L)
    torch.cuda.synchronize()
    return layers


class Decode:
    """The op list of one run of the quantized path for T tokens (Appendix-B call sites of v6)."""

    def __init__(self, wrq, torch, layers, C, H, T):
        self.wrq, self.layers, self.C, self.H, self.T = wrq, layers, C, H, T
        g = torch.Generator(device="cuda").manual_seed(SEED + 5)
        f16, f32 = torch.float16, torch.float32
        self.att_sx = torch.randn((5, T, C), generator=g, device="cuda").to(f16)  # [C, T, 5]
        self.att_x = torch.randn((T, C), generator=g, device="cuda").to(f16)
        self.ffn_kx = torch.randn((T, C), generator=g, device="cuda").to(f16)
        self.ffn_rx = torch.randn((T, C), generator=g, device="cuda").to(f16)
        self.att_k = torch.empty((T, C), dtype=f32, device="cuda")
        self.att_v = torch.empty((T, C), dtype=f32, device="cuda")
        self.att_r = torch.empty((T, C), dtype=f32, device="cuda")
        self.att_g = torch.empty((T, C), dtype=f16, device="cuda")
        self.att_o = torch.empty((T, C), dtype=f16, device="cuda")
        self.ffn_k = torch.empty((T, H), dtype=f16, device="cuda")
        self.ffn_v = torch.empty((T, C), dtype=f16, device="cuda")
        self.ffn_r = torch.empty((T, C), dtype=f16, device="cuda")
        self.turbo = wrq.turbo(T)
        self.launches = 8 * len(layers)

    def step_grouped(self):
        """The same products with the independent ones of a layer sharing launches: {k, v, r, g},
        then output, then {ffn.key, ffn.receptance}, then ffn.value."""
        wrq, C, T = self.wrq, self.C, self.T
        sq, no = wrq.ACT_SQUARED_RELU, wrq.ACT_NONE
        for L in self.layers:
            wrq.matmul_vec_group([
                (m, self.att_sx, out, no, False, dict(input_view=((C, T, 1), (C, T, 5), (0, 0, i))))
                for i, (m, out) in enumerate(((L.att_k, self.att_k), (L.att_v, self.att_v), (L.att_r, self.att_r), (L.att_g, self.att_g)), 1)])
            L.att_o.matmul_op(self.att_x, self.att_o, turbo=self.turbo)
            wrq.matmul_vec_group([(L.ffn_k, self.ffn_kx, self.ffn_k, sq, False, {}), (L.ffn_r, self.ffn_rx, self.ffn_r, no, False, {})])
            L.ffn_v.matmul_op_sparse(self.ffn_k, self.ffn_v, turbo=self.turbo)

    def step(self):
        wrq, C, T, turbo = self.wrq, self.C, self.T, self.turbo
        sq = wrq.ACT_SQUARED_RELU
        for L in self.layers:
            for i, (m, out) in enumerate(((L.att_k, self.att_k), (L.att_v, self.att_v), (L.att_r, self.att_r), (L.att_g, self.att_g)), 1):
                m.matmul_op(self.att_sx, out, turbo=turbo, input_view=((C, T, 1), (C, T, 5), (0, 0, i)))
            L.att_o.matmul_op(self.att_x, self.att_o, turbo=turbo)
            L.ffn_k.matmul_op(self.ffn_kx, self.ffn_k, sq, turbo=turbo)
            L.ffn_v.matmul_op_sparse(self.ffn_k, self.ffn_v, turbo=turbo)
            L.ffn_r.matmul_op(self.ffn_rx, self.ffn_r, turbo=turbo)

    def bytes_per_step(self, quant):
        f = int8_bytes if quant == "int8" else nf4_bytes
        C, H, T = self.C, self.H, self.T
        per_layer = 3 * f(C, C, T, 4) + 3 * f(C, C, T, 2) + f(C, H, T, 2) + f(H, C, T, 2)
        return per_layer * len(self.layers)


def time_steps(torch, fn, steps, warmup):
    """ms per step over exactly `steps` calls, bracketed by synchronisation; HIP events on the launch stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_time(e1) / steps, wall_ms / steps


def cpu_baseline(wrq, torch, layers, dec, quant, sample_layers, seconds=10.0):
    """The oracle (a port of the reference's kernels, OpenMP over rows) on the host cores, on a
    bounded sample: `sample_layers` layers of the same decode step, scaled to the full depth."""
    from oracle import wrq_oracle as oracle

    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    vec = oracle.matmul_vec_int8 if quant == "int8" else oracle.matmul_vec_nf4
    host = []
    for L in layers[:sample_layers]:
        host.append([(m.w.cpu().numpy(), m.m.cpu().numpy()) for m in (L.att_k, L.att_v, L.att_r, L.att_g, L.att_o, L.ffn_k, L.ffn_v, L.ffn_r)])
    xc = dec.att_x[:1].cpu().numpy()
    xh = np.maximum(dec.ffn_k[:1].cpu().numpy(), 0)
    tokens = 0
    t0 = time.perf_counter()
    while True:
        for mats in host:
            for j, (w, s) in enumerate(mats):
                x = xh if j == 6 else xc
                vec(w, s, x, act=1 if j == 5 else 0, sparse=(j == 6))
        tokens += 1
        dt = time.perf_counter() - t0
        if dt > seconds or tokens >= 64:
            break
    tok_s = tokens / (dt * len(layers) / sample_layers)
    return {
        "value": round(tok_s, 4), "unit": "tok/s", "cores": cores, "kind": "port",
        "sample": f"{tokens} pass(es) over {sample_layers} of {len(layers)} layers of the same decode step ({dt:.1f} s of CPU work), scaled to full depth; "
                  "CPU restatement of the reference kernels, not lavapipe",
    }


def dominant_kernel(quant, tokens):
    """The library kernel that takes most of a step of `tokens` tokens through the vec entry point."""
    if quant == "int8":
        if tokens == 1:
            return "gemv_int8_rows_group4_kernel"  # K = 4096 and 14336 are multiples of 1024: the wave-owns-rows kernel (single products: gemv_int8_rows_single_kernel)
        return "gemv_int8_rows_tokens_kernel" if tokens <= 4 else "gemm_kernel"  # the same layout with 2 or 4 tokens per pass
    return "gemv_nf4_oneshot_kernel" if tokens <= 3 else "gemm_kernel"


# What a plain streaming read of the same bytes reaches in the same kind of graph on this machine (measured with the probe kernels):
# a dependent dispatch costs about 1.45 us and the stream runs at about 7.2 TB/s.
PLAIN_READ_DISPATCH_US, PLAIN_READ_GBPS = 1.45, 7200.0


def plain_read_frac(nbytes, launches):
    """Fraction of the HBM peak that `launches` plain reads of `nbytes` in total would reach: the ceiling of the launch structure."""
    us = launches * PLAIN_READ_DISPATCH_US + nbytes / PLAIN_READ_GBPS / 1e3
    return round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)


def read_traffic(quant):
    """HBM bytes per launch of the default decode step from profiles/gemv_<quant>_decode_7b_hbm_traffic.txt
    (the line `traffic_bytes_per_launch: N`), or None."""
    path = os.path.join(ROOT, "profiles", f"gemv_{quant}_decode_7b_hbm_traffic.txt")
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return int(line.split(":", 1)[1].split()[0].replace(",", ""))
    except OSError:
        pass
    return None


PROBE_SRC = os.path.join(ROOT, "bench_probe.hip")
PROBE_LIB = os.path.join(ROOT, "bench_probe.so")


def build_probe():
    """Compiles the measurement probes (bench_probe.hip: a plain copy and a streaming read) for gfx950."""
    import subprocess

    hipcc, arch = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), os.environ.get("ARCH", "gfx950")  # the Makefile's variables
    cmd = [hipcc, f"--offload-arch={arch}", "-O3", "-std=c++17", "-fPIC", "-shared",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-o", PROBE_LIB, PROBE_SRC]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building bench_probe.so failed:\n" + r.stdout[-2000:] + r.stderr[-2000:])
    return PROBE_LIB


def run_probe(torch):
    """Plain copy and streaming read of 256 MiB with the probe kernels; returns their GB/s."""
    import ctypes as C

    if not os.path.exists(PROBE_LIB):
        build_probe()
    L = C.CDLL(PROBE_LIB)
    L.wrq_probe_read.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int]
    L.wrq_probe_copy.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64]
    n = 256 << 20
    src = torch.randint(0, 127, (4, n), dtype=torch.uint8, device="cuda")
    dst = torch.empty(n, dtype=torch.uint8, device="cuda")
    sink = torch.zeros(16, dtype=torch.int32, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    it = [0]

    def copy():
        L.wrq_probe_copy(st, C.c_void_p(dst.data_ptr()), C.c_void_p(src[it[0] % 4].data_ptr()), n)
        it[0] += 1

    def read():
        L.wrq_probe_read(st, C.c_void_p(src[it[0] % 4].data_ptr()), C.c_void_p(sink.data_ptr()), n, 2, 1)
        it[0] += 1

    ms_copy, _ = time_steps(torch, copy, 8, 2)
    ms_read, _ = time_steps(torch, read, 8, 2)
    return {"bytes": n, "copy_GBps": round(2 * n / ms_copy / 1e6, 1), "read_GBps": round(n / ms_read / 1e6, 1)}


def sweep_pack(wrq, torch, quant, w):
    """Packing one f16 matrix (quant_mat_int8 / quant_mat_nf4): microseconds and HBM bytes per
    second, 2 B read + 1 or 0.5 B written per element plus the scale blocks; inputs rotate so
    that none is still cached."""
    R, K = w.shape
    nin = min(16, max(2, int(1.0e9 // (w.numel() * 2)) + 1))
    ins = [w] + [w.clone() for _ in range(nin - 1)]
    if quant == "int8":
        out = torch.empty((R, K), dtype=torch.uint8, device="cuda")
        scale = torch.empty(2 * R * K // wrq.INT8_BLOCK_SIZE, dtype=torch.float16, device="cuda")
        calls = [lambda x=x: wrq.TensorOp.quantize_mat_int8(x, scale, out) for x in ins]
    else:
        out = torch.empty((R, K // 2), dtype=torch.uint8, device="cuda")
        scale = torch.empty(R * K // wrq.NF4_BLOCK_SIZE, dtype=torch.float16, device="cuda")
        table = torch.tensor(wrq.NF4_QUANT, dtype=torch.float32, device="cuda")
        calls = [lambda x=x: wrq.TensorOp.quantize_mat_nf4(x, table, scale, out) for x in ins]
    reps = max(nin, 24)
    calls[0]()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(reps):
            calls[i % nin]()
    ms, _ = time_steps(torch, graph.replay, 5, 2)
    us = ms * 1e3 / reps
    nbytes = w.numel() * 2 + out.numel() + scale.numel() * 2
    return {"op": "pack", "quant": quant, "K": K, "R": R, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
            "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3), "copies": nin}


def sweep(wrq, torch, args):
    """Per-operator figures of configs 2 and 3: cold (rotating weight copies) GB/s per shape."""
    import ctypes as C

    rows = []
    probe = None
    if args.probe:
        if not os.path.exists(PROBE_LIB):
            build_probe()
        probe = C.CDLL(PROBE_LIB)
        probe.wrq_probe_read.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int]
        sink = torch.zeros(16, dtype=torch.int32, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(SEED + 2)
    shapes = [(2048, 2048), (2048, 7168), (7168, 2048), (2048, 65536), (4096, 4096), (4096, 14336), (14336, 4096)]
    for quant in ("int8", "nf4", "fp16"):
        for K, R in (shapes if quant != "fp16" else [(2048, 65536), (4096, 65536), (4096, 4096)]):
            w = (torch.randn((R, K), generator=g, device="cuda") * 0.02).half()
            if quant != "fp16":
                rows.append(sweep_pack(wrq, torch, quant, w))
                print(json.dumps(rows[-1]), flush=True)
            m0 = wrq.Matrix.quant_u8(w) if quant == "int8" else wrq.Matrix.quant_nf4(w) if quant == "nf4" else wrq.Matrix.fp16(w)
            del w
            wbytes = m0.w.numel() * m0.w.element_size()
            ncopy = max(2, int(1.5e9 // wbytes) + 1)
            ncopy = min(ncopy, 64)
            mats = [m0] + [wrq.Matrix(m0.kind, m0.w.clone(), None if m0.m is None else m0.m.clone(), m0.q) for _ in range(ncopy - 1)]
            for T in ([1] if quant != "nf4" and not args.all_t else [1, 8, 32, 128, 256]):
                x = torch.randn((T, K), generator=g, device="cuda").half()
                out = torch.empty((T, R), dtype=torch.float16, device="cuda")
                turbo = wrq.turbo(T)
                it = [0]

                def fn():
                    mats[it[0] % ncopy].matmul_op(x, out, turbo=turbo)
                    it[0] += 1

                # one HIP graph of `reps` back-to-back launches over rotating weight copies, so
                # that neither host launch cost nor cache reuse enters the figure
                reps = max(ncopy, 50)
                fn()
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for _ in range(reps):
                        fn()
                ms, _ = time_steps(torch, graph.replay, 5, 2)
                us = ms * 1e3 / reps
                nbytes = (int8_bytes if quant == "int8" else nf4_bytes if quant == "nf4" else fp16_bytes)(K, R, T)
                flops = 2.0 * K * R * T
                rows.append({"quant": quant, "K": K, "R": R, "T": T, "us": round(us, 2),
                             "GBps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3),
                             "TFLOPs": round(flops / us / 1e6, 1), "copies": ncopy})
                if T == 1 and probe is not None:
                    # what a launch of this size can reach at all: the probe's plain streaming read of the same
                    # packed weights, in the same graph of back-to-back launches over the same rotating copies
                    it[0] = 0

                    def rd():
                        wt = mats[it[0] % ncopy].w
                        st = C.c_void_p(torch.cuda.current_stream().cuda_stream)  # the capture stream, inside a capture
                        probe.wrq_probe_read(st, C.c_void_p(wt.data_ptr()), C.c_void_p(sink.data_ptr()), wt.numel() * wt.element_size(), 2, 1)
                        it[0] += 1

                    rd()
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        for _ in range(reps):
                            rd()
                    ms, _ = time_steps(torch, graph.replay, 5, 2)
                    rows[-1]["plain_read_us"] = round(ms * 1e3 / reps, 2)
                    rows[-1]["of_plain_read"] = round(ms * 1e3 / reps / us, 3)
                print(json.dumps(rows[-1]), flush=True)
            del mats, m0
            torch.cuda.empty_cache()
    return rows


MIN_TOKEN_CHUNK_SIZE = 32


def rnn_iter_next(state, chunk):
    """One RnnIter step (src/runtime/infer/rnn.rs:280-335): how many tokens of each slot enter
    the next run.  `state` is a list of [generating, tokens_to_read]; updated in place."""
    remains = [1 if gen else read for gen, read in state]
    num_token = min(sum(remains), chunk)
    if num_token > MIN_TOKEN_CHUNK_SIZE:
        num_token -= num_token % MIN_TOKEN_CHUNK_SIZE
    lens = [0] * len(state)
    while num_token > 0:
        live = [r for r in remains if r > 0]
        if not live:
            break
        mid = min(live)
        for i, r in enumerate(remains):
            if r == 0:
                continue
            take = min(mid, num_token)
            num_token -= take
            lens[i] += take
            remains[i] -= take
    for i, n in enumerate(lens):
        if n > 0:
            state[i][0] = remains[i] == 0
            state[i][1] = remains[i]
    return lens


def schedule(wrq, torch, args, layers, C, H):
    """Config 5: a serving schedule instead of one step size.  `slots` requests with prompts of
    16..1024 tokens arrive together, the reference's RnnIter cuts every run (chunk 256), every
    request then decodes 128 tokens; a finished request leaves its slot empty.  The matrix path
    of every run is replayed from a HIP graph per distinct run length T: chunk kernels for
    T % 32 == 0, decode kernels otherwise (src/runtime/v6.rs:568-570)."""
    rng = np.random.default_rng(SEED + 5)
    slots, chunk, gen_len = args.slots, 256, 128
    chunk = max(chunk, MIN_TOKEN_CHUNK_SIZE)
    prompts = rng.integers(16, 1025, size=slots)
    state = [[False, int(p)] for p in prompts]  # RnnIter state per slot
    to_gen = [gen_len] * slots
    runs = []  # tokens per run
    while True:
        if not any(read > 0 for _, read in state):
            break
        lens = rnn_iter_next(state, chunk)
        T = sum(lens)
        if T == 0:
            break
        runs.append(T)
        for i in range(slots):
            # every run starts from a fresh iterator over what is left to read (JobInput::step,
            # rnn.rs:233-240); a slot whose input is exhausted emitted a token, which is fed back
            # as its next input while the request lasts
            state[i][0] = False
            if lens[i] > 0 and state[i][1] == 0 and to_gen[i] > 0:
                to_gen[i] -= 1
                state[i][1] = 1 if to_gen[i] > 0 else 0
    graphs = {}
    for T in sorted(set(runs)):
        dec = Decode(wrq, torch, layers, C, H, T)
        step = dec.step_grouped
        step()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            step()
        graphs[T] = (g, dec)
    for g, _ in graphs.values():
        g.replay()
    torch.cuda.synchronize()
    phases = {"prefill (T = 256)": [0, 0.0], "mixed (32 < T < 256)": [0, 0.0], "all slots decoding (T = 32)": [0, 0.0], "tail (T < 32)": [0, 0.0]}
    t0 = time.perf_counter()
    evs = []
    for T in runs:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graphs[T][0].replay()
        e1.record()
        evs.append((T, e0, e1))
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    nbytes = 0
    for T, e0, e1 in evs:
        ms = e0.elapsed_time(e1)
        key = "prefill (T = 256)" if T == 256 else "all slots decoding (T = 32)" if T == 32 else "tail (T < 32)" if T < 32 else "mixed (32 < T < 256)"
        phases[key][0] += T
        phases[key][1] += ms
        nbytes += graphs[T][1].bytes_per_step(args.quant)
    total_tokens = sum(runs)
    gpu_ms = sum(v[1] for v in phases.values())
    out = {
        "metric": "config 5: serving schedule of the quantized matrix path, tokens/s over all runs",
        "value": round(total_tokens / wall, 1), "unit": "tok/s", "n_gpus": 1,
        "config": {"workload": f"config 5: RWKV-v6 7B-shape, {args.layers} layers {args.quant}, {slots} slots, prompts 16..1024 (seeded), chunk 256, "
                               f"{gen_len} decode tokens per slot, runs cut by RnnIter", "runs": len(runs), "distinct_T": len(graphs)},
        "tokens": total_tokens, "wall_ms": round(wall * 1e3, 2), "gpu_ms": round(gpu_ms, 2),
        "packed_GBps": round(nbytes / gpu_ms / 1e6, 1),
        "phases": {k: {"tokens": v[0], "ms": round(v[1], 2), "tok_per_s": round(v[0] / v[1] * 1e3, 1) if v[1] else None} for k, v in phases.items()},
        "data": "synthetic",
    }
    print(json.dumps(out), flush=True)


def stamps_timeline(wrq, torch, args, layers, C, H):
    """Timeline of one Int8 decode step from wall-clock stamps written by stamped builds of the same kernels
    (wrq_debug_stamps): per launch of a layer, when its first wave started and its last wave ended, the gap to
    the launch before, and where a wave's lifetime goes.  Stamps cost time: the step is slower than the product's."""
    import ctypes as C_
    assert args.quant == "int8" and args.tokens == 1, "--stamps covers the Int8 one-token step"
    L = wrq.lib()
    L.wrq_debug_stamps.argtypes = [C_.c_void_p, C_.c_uint64]
    dec = Decode(wrq, torch, layers, C, H, 1)
    n_launch = 4 * len(layers)
    slot = 1 << 20
    buf = torch.zeros(n_launch * slot, dtype=torch.uint8, device="cuda")

    def graph_of(fn):
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        return g

    plain = graph_of(dec.step_grouped)
    plain_ms, _ = time_steps(torch, plain.replay, args.steps, args.warmup)
    assert L.wrq_debug_stamps(C_.c_void_p(buf.data_ptr()), buf.numel()) == 0, L.wrq_last_error().decode()
    dec.step_grouped()  # warm the stamped kernels (slots 0..n_launch-1)
    torch.cuda.synchronize()
    assert L.wrq_debug_stamps(C_.c_void_p(buf.data_ptr()), buf.numel()) == 0  # restart the slot counter
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        dec.step_grouped()
    stamped_ms, _ = time_steps(torch, g.replay, args.steps, args.warmup)
    torch.cuda.synchronize()
    assert L.wrq_debug_stamps(None, 0) == 0
    rec = buf.view(torch.int64).view(n_launch, slot // 32, 4).cpu().numpy()
    kinds = [("{att.w_k, w_v, w_r, w_g}", 4 * C // 4, 4), ("att.w_o", C // 4, 4), ("{ffn.w_k, ffn.w_r}", (H + C) // 4, 4), ("ffn.w_v", C // 8, 14)]
    tick_us = 0.01  # the wall-clock counter runs at 100 MHz
    import numpy as np
    rows = {k: [] for k in range(4)}
    xcd_ends = {k: [] for k in range(4)}
    xcd_starts = {k: [] for k in range(4)}
    last_end = None
    for i in range(n_launch):
        name, wgs, waves = kinds[i % 4]
        r = rec[i, :wgs * waves].astype(np.float64) * tick_us
        assert (r[:, 0] > 0).all() and (r[:, 3] >= r[:, 0]).all(), "launch %d left stamp records unwritten" % i
        first, end = r[:, 0].min(), r[:, 3].max()
        if i >= 4:  # the first layer starts from an idle machine
            life = r[:, 3] - r[:, 0]
            xcd = (np.arange(wgs * waves) // waves) % 8  # workgroup b runs on XCD b mod 8
            xcd_end = np.array([r[xcd == q, 3].max() for q in range(8)])
            xcd_ends[i % 4].append(xcd_end - first)
            xcd_starts[i % 4].append(np.array([r[xcd == q, 0].min() for q in range(8)]) - first)
            rows[i % 4].append(dict(span=end - first, gap=first - last_end, xcd_spread=float(xcd_end.max() - xcd_end.min()),
                                    last_start=r[:, 0].max() - first, issue=np.median(r[:, 1] - r[:, 0]),
                                    data=np.median(r[:, 2] - r[:, 1]), finish=np.median(r[:, 3] - r[:, 2]), life=np.median(life),
                                    life95=np.percentile(life, 95), first_done=r[:, 2].min() - first))
        last_end = end
    step_span = (rec[n_launch - 1, :kinds[3][1] * kinds[3][2], 3].max() - rec[0, :kinds[0][1] * kinds[0][2], 0].min()) * tick_us
    print("Int8 decode step, %d layers, graph replay: %.4f ms with the product kernels, %.4f ms with the stamped builds; "
          "first stamp to last stamp of the stamped step %.4f ms" % (len(layers), plain_ms, stamped_ms, step_span / 1e3))
    print("per launch, microseconds, mean over layers 1..%d (medians over the waves of a launch where marked):" % (len(layers) - 1))
    hdr = "%-26s %6s %6s %9s %9s %10s %9s %9s %9s %9s %9s %10s %10s" % ("launch", "wgs", "waves", "gap", "span", "last_start", "issue~", "data~", "finish~", "life~", "life95", "first_done", "xcd_spread")
    print(hdr)
    out = {}
    tot_gap = tot_span = 0.0
    for k in range(4):
        name, wgs, waves = kinds[k]
        m = {f: float(np.mean([r[f] for r in rows[k]])) for f in rows[k][0]}
        out[name] = {f: round(v, 3) for f, v in m.items()}
        tot_gap += m["gap"]
        tot_span += m["span"]
        print("%-26s %6d %6d %9.2f %9.2f %10.2f %9.2f %9.2f %9.2f %9.2f %9.2f %10.2f %10.2f" % (name, wgs, wgs * waves, m["gap"], m["span"], m["last_start"], m["issue"],
              m["data"], m["finish"], m["life"], m["life95"], m["first_done"], m["xcd_spread"]))
    for k in range(4):
        print("%-26s last wave end per XCD 0..7, after the launch's first start: %s; first wave start: %s" % (
            kinds[k][0], " ".join("%.2f" % v for v in np.mean(xcd_ends[k], axis=0)), " ".join("%.2f" % v for v in np.mean(xcd_starts[k], axis=0))))
    print("layer: gaps %.2f us + spans %.2f us = %.2f us (stamped); the product step is %.2f us per layer" % (tot_gap, tot_span, tot_gap + tot_span, plain_ms * 1e3 / len(layers)))
    print("gap: first wave start minus last wave end of the launch before; span: first wave start to last wave end; last_start: when the last wave of")
    print("the launch started, after the first; issue~: entry to every load requested; data~: from there to every row accumulated; finish~: reduction")
    print("and store; life~/life95: wave lifetime, median and 95th percentile; first_done: first wave anywhere with every row accumulated, after the first start;")
    print("xcd_spread: between the XCD whose last wave ends first and the one whose last wave ends last.")
    print(json.dumps({"stamps": out, "plain_ms": round(plain_ms, 4), "stamped_ms": round(stamped_ms, 4)}))


def full_layers(wrq, torch, args, C, H):
    """Every op of the v6 layers, dispatched like the reference (src/runtime/v6.rs:758-955): 35 ops
    per layer, 8 of them the quantized products.  One run of `--tokens` tokens of one request per
    step, replayed from a HIP graph.  Model tok/s without embedding and head."""
    v6 = importlib.import_module("web-rwkv_amd.v6")
    heads, S, slots = C // 64, 64, 4
    rng = np.random.default_rng(SEED + 7)
    layers, states = [], []
    for i in range(args.layers):
        layers.append(v6.Layer(torch, v6.random_layer_weights(rng, C, heads, S, H, layer=i), args.quant))
        states.append(torch.zeros((slots, S + 2, C), dtype=torch.float32, device="cuda"))
    A = args.tokens
    buf = v6.Runtime(torch, C, H, A)
    buf.x.copy_(torch.randn((1, A, C), device="cuda").half())
    # one request in slot 0 whose A tokens fill the stack (the reference packs the count into 8 bits)
    cursors = torch.from_numpy(np.full(A, (min(A, 255) << 24), dtype=np.uint32).view(np.int32)).cuda()
    x0 = buf.x.clone()
    dispatch = v6.dispatch_layer_auto if args.fused else v6.dispatch_layer
    model = args.full_model
    if model:
        # the ends of the model (src/runtime/v6.rs:625-640, :960-1000): embedding + its layer norm in front,
        # layer norm + f16 head (65536 x C) on the run's last token + softmax behind
        V = 65536
        g = torch.Generator(device="cuda").manual_seed(SEED + 8)
        embed = (torch.randn((V, C), generator=g, device="cuda") * 0.5).half()
        head = wrq.Matrix.fp16((torch.randn((V, C), generator=g, device="cuda") * 0.02).half())
        ln = [(1.0 + 0.1 * torch.randn(C, generator=g, device="cuda")).half(), (0.1 * torch.randn(C, generator=g, device="cuda")).half()]
        ids = torch.randint(0, V, (1, A), generator=g, device="cuda", dtype=torch.int32)
        inp = torch.zeros((1, A, C), dtype=torch.float16, device="cuda")
        head_x = torch.zeros((1, 1, C), dtype=torch.float16, device="cuda")
        logits = torch.zeros((1, 1, V), dtype=torch.float32, device="cuda")

    def step():
        if model:
            wrq.LayerOp.embed(ids, embed, inp)
            wrq.LayerOp.layer_norm(ln[0], ln[1], inp, v6.LN_EPS)
            wrq.LayerOp.blit(inp, buf.x)
        else:
            buf.x.copy_(x0)  # the embedding of the next token would land here
        for i, (layer, st) in enumerate(zip(layers, states)):
            dispatch(layer, buf, st, cursors, A, heads, S, rescale_now=(i + 1) % 6 == 0)
        if model:
            wrq.LayerOp.blit(buf.x, head_x, input_view=((C, 1, 1), (C, A, 1), (0, A - 1, 0)))
            wrq.LayerOp.layer_norm(ln[0], ln[1], head_x, v6.LN_EPS)
            head.matmul_op(head_x, logits, turbo=False)
            wrq.LayerOp.softmax(logits)

    step()
    torch.cuda.synchronize()
    if args.no_graph:
        fn = step
    else:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        fn = graph.replay
    ms, wall_ms = time_steps(torch, fn, args.steps, args.warmup)
    assert torch.isfinite(buf.x.float()).all()
    what = "RWKV-v6 7B-shape model step, every op (embedding, layers, head on the last token, softmax), tokens/s" if model else \
        "RWKV-v6 7B-shape layers, every op (no embedding, no head), tokens/s"
    print(json.dumps({"metric": what, "value": round(A * 1e3 / wall_ms, 2), "unit": "tok/s",
                      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4), "gpu_ms_per_step": round(ms, 4),
                      "config": {"workload": f"{args.layers} v6 layers ({C} x {H}, {heads} heads), {args.quant}, {A} token(s) of one request per step, "
                                             + ("12 launches per layer (fused small ops)" if args.fused and A <= v6.FUSED_MAX_TOKENS else "35 ops per layer"),
                                 "hip_graph": not args.no_graph}, "data": "synthetic"}))


def v5_model(wrq, torch, args):
    """Config 1 on the GPU: the v5-shape model, every op of a run through the library
    (src/runtime/v5.rs:541-930), one request; the 32-token prompt run and the one-token decode run,
    each a HIP graph."""
    v5 = importlib.import_module("web-rwkv_amd.v5")
    L, heads, S, hidden, V = 12, 12, 64, 2688, 65536
    rng = np.random.default_rng(SEED + 1)
    model = v5.Model(torch, v5.random_model_weights(rng, L, heads * S, heads, S, hidden, V), args.quant, heads, S, hidden, 1, packed_shifts=args.packed_shifts)
    out = {}
    for A in (32, 1):
        model.run([int(t) for t in rng.integers(0, V, A)], 0)
        torch.cuda.synchronize()
        if args.no_graph:
            fn = lambda A=A: model.dispatch(A)
        else:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                model.dispatch(A)
            fn = graph.replay
        ms, wall_ms = time_steps(torch, fn, args.steps, args.warmup)
        out[A] = (ms, wall_ms)
        assert torch.isfinite(model.buffers(A)[5]).all()
    packed = sum(m.w.numel() * m.w.element_size() + m.m.numel() * 2 for layer in model.layers for m in layer.m.values())
    print(json.dumps({"metric": "RWKV-v5-shape model (config 1), every op, decode tokens/s, batch 1", "value": round(1e3 / out[1][1], 2), "unit": "tok/s",
                      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(out[1][1], 4), "gpu_ms_per_step": round(out[1][0], 4),
                      "prompt_32_tokens_ms": round(out[32][1], 4), "prompt_tok_s": round(32e3 / out[32][1], 1),
                      "config": {"workload": f"{L} v5 layers (768 x {hidden}, {heads} heads), {args.quant}, embedding, head 65536 x 768 f16 on the last token; "
                                             + ("21 ops per layer (token shifts of a half in one launch)" if args.packed_shifts else "27 ops per layer"), "hip_graph": not args.no_graph, "packed_bytes": packed}, "data": "synthetic"}))


def loader_bench(args):
    """Writes the eight matrices of `--layers` 7B-shape layers (f16, 450 MB per layer) as a safetensors file
    under the temporary directory and times the C++ loader on it (tests/cpp/test_host --loader-bench)."""
    import subprocess
    import tempfile

    from safetensors.numpy import save_file

    binary = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "cpp", "test_host")
    assert os.path.exists(binary), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    C, H = 4096, 14336
    rng = np.random.default_rng(SEED + 11)
    layers = min(args.layers, 4)
    tensors = {}
    for i in range(layers):
        for name, (R, K) in {"att.key": (C, C), "att.value": (C, C), "att.receptance": (C, C), "att.gate": (C, C), "att.output": (C, C),
                             "ffn.key": (H, C), "ffn.value": (C, H), "ffn.receptance": (C, C)}.items():
            tensors[f"blocks.{i}.{name}.weight"] = (rng.standard_normal((R, K), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "layers.st")
        save_file(tensors, path)
        r = subprocess.run([binary, "--loader-bench", path], capture_output=True, text=True, timeout=600)
    sys.stdout.write(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr


def v7_layers(wrq, torch, args):
    """RWKV-v7 layers at the 7B shape, every op through the library (src/runtime/v7.rs:704-1006), one
    request, one HIP graph per step."""
    v7 = importlib.import_module("web-rwkv_amd.v7")
    C, heads, S, hidden, A = 4096, 64, 64, 16384, args.tokens
    rng = np.random.default_rng(SEED + 9)
    layers = [v7.Layer(torch, v7.random_layer_weights(rng, C, heads, S, hidden), args.quant) for _ in range(args.layers)]
    states = [torch.zeros((1, S + 2, C), dtype=torch.float32, device="cuda") for _ in layers]
    buf = v7.Runtime(torch, C, hidden, A)
    x0 = torch.randn((1, A, C), device="cuda").half()
    cursors = torch.from_numpy(np.full(A, (min(A, 255) << 24), dtype=np.uint32).view(np.int32)).cuda()
    shifts = [v7.PackedShifts(torch, layer, A) for layer in layers] if args.packed_shifts else None

    def step():
        buf.x.copy_(x0)  # the embedding of the next token would land here
        for i, (layer, st) in enumerate(zip(layers, states)):
            v7.dispatch_layer(layer, buf, st, cursors, A, heads, S, i, shifts=shifts[i] if shifts else None)

    step()
    torch.cuda.synchronize()
    if args.no_graph:
        fn = step
    else:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        fn = graph.replay
    ms, wall_ms = time_steps(torch, fn, args.steps, args.warmup)
    assert torch.isfinite(buf.x.float()).all()
    print(json.dumps({"metric": "RWKV-v7 7B-shape layers, every op (no embedding, no head), tokens/s", "value": round(A * 1e3 / wall_ms, 2), "unit": "tok/s",
                      "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4), "gpu_ms_per_step": round(ms, 4),
                      "config": {"workload": f"{args.layers} v7 layers ({C} x {hidden}, {heads} heads), {args.quant}, {A} token(s) of one request per step, "
                                             + ("46 ops per layer (the six token shifts in one launch)" if args.packed_shifts else "51 ops per layer (47 in the first)") + ", the three independent projections in one launch", "hip_graph": not args.no_graph}, "data": "synthetic"}))


def ops_table(wrq, torch, args, C):
    """Time of every layer op alone at the 7B layer shape, A tokens (HIP graph of 20 calls)."""
    LayerOp = wrq.LayerOp
    A, S = args.tokens, 64
    heads = C // S
    h = lambda *s: torch.randn(s, device="cuda").half()
    f = lambda *s: torch.randn(s, device="cuda")
    cur = torch.from_numpy(np.full(A, (min(A, 255) << 24), dtype=np.uint32).view(np.int32)).cuda()
    state = torch.zeros((4, S + 2, C), dtype=torch.float32, device="cuda")
    att = ((C, S + 1, 4), (C, S + 2, 4), (0, 0, 0))
    ffn = ((C, 1, 4), (C, S + 2, 4), (0, S + 1, 0))
    x, y, w, b, x5, tm5 = h(1, A, C), h(1, A, C), h(C), h(C), h(5, A, C), h(5, A, C)
    k, v, r, aux, decay, u = f(A, heads, S), f(A, heads, S), f(A, heads, S), f(A, heads, S), torch.rand((A, heads, S), device="cuda"), f(heads, S)
    gw, gb = h(heads, S), h(heads, S)
    r16, w16, n16, u16 = h(A, heads, S), h(A, heads, S), 0.1 * h(4, A, heads, S), h(heads, S)  # the v7 operands are f16
    cases = {
        "layer_norm": (lambda: LayerOp.layer_norm(w, b, x, 1e-5), 2 * A * C * 2),
        "group_norm": (lambda: LayerOp.group_norm(gw, gb, aux, 64e-5), 2 * A * C * 4),
        "token_shift (1)": (lambda: LayerOp.token_shift(cur, w, state, x, y, True, state_view=att), 2 * A * C * 2),
        "token_shift (5)": (lambda: LayerOp.token_shift(cur, tm5, state, x, x5, True, state_view=att), 11 * A * C * 2),
        "add": (lambda: LayerOp.add(x, y), 3 * A * C * 2),
        "mul_activate silu": (lambda: LayerOp.mul_activate(x, y, wrq.ACT_SILU), 3 * A * C * 2),
        "blit f16 -> f32": (lambda: LayerOp.blit(x, aux.view(1, A, C)), A * C * 6),
        "activate stable_exp": (lambda: LayerOp.activate(decay.view(1, A, C), wrq.ACT_STABLE_EXP), 2 * A * C * 4),
        "channel_mix": (lambda: LayerOp.channel_mix(cur, state, x, y, x5[0:1], state_view=ffn), 4 * A * C * 2),
        "time_mix_v6": (lambda: LayerOp.time_mix_v6(cur, decay, u, state, k, v, r, aux, state_view=att), 5 * A * C * 4 + 2 * S * C * 4),
        "time_mix_v5": (lambda: LayerOp.time_mix_v5(cur, decay[0], u, state, k, v, r, aux, state_view=att), 4 * A * C * 4 + 2 * S * C * 4),
        "time_mix_v7": (lambda: LayerOp.time_mix_v7(cur, state, r16, w16, n16, x.view(A, heads, S), state_view=att), 7 * A * C * 2 + 2 * S * C * 4),
        "time_first_v7": (lambda: LayerOp.time_first_v7(u16, r16, n16, x.view(A, heads, S)), 5 * A * C * 2),
        "l2_norm (heads)": (lambda: LayerOp.l2_norm(x.view(A, heads, S), 1e-12), 2 * A * C * 2),
        "control_k_v7": (lambda: LayerOp.control_k_v7(w, x, y), 3 * A * C * 2),
        "channel_mix_v7": (lambda: LayerOp.channel_mix_v7(cur, state, x, y, state_view=ffn), 2 * A * C * 2),
        "softmax (65536)": (lambda: LayerOp.softmax(f(1, 1, 65536)), 0),
    }
    for name, (fn, nbytes) in cases.items():
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        if name.startswith("softmax"):
            logits = f(1, 1, 65536)
            fn = lambda: LayerOp.softmax(logits)
            nbytes = 2 * 65536 * 4
            fn()
            torch.cuda.synchronize()
        with torch.cuda.graph(g):
            for _ in range(20):
                fn()
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / 200
        print(json.dumps({"op": name, "tokens": A, "us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1)}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--quant", choices=["int8", "nf4"], default="int8")
    ap.add_argument("--tokens", type=int, default=1, help="tokens per step (1 = decode; 128 = a prefill chunk)")
    ap.add_argument("--layers", type=int, default=None, help="default: the model's depth (32 for the 7B shape of the metric)")
    ap.add_argument("--model", choices=sorted(MODEL_SHAPES), default="7b",
                    help="layer shape of the step; 7b is the metric's config 4, 1b6 the shape of configs 2 and 3")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-group", action="store_true", help="one launch per product instead of grouped launches of independent products")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--main-only", action="store_true", help="leave the ungrouped and NF4 figures out of the default line (for profiler runs of one workload)")
    ap.add_argument("--cpu-sample-layers", type=int, default=8)
    ap.add_argument("--cpu-seconds", type=float, default=3.0,
                    help="seconds of CPU work for the cpu_baseline sample (whole passes over the sampled layers; at least one)")
    ap.add_argument("--probe", action="store_true",
                    help="also run the plain copy (256 MiB) and stream-read probes: the dispatches rocprofv3's FETCH_SIZE / WRITE_SIZE are scaled against")
    ap.add_argument("--sweep", action="store_true", help="per-operator sweep (configs 2 and 3) instead of the decode step")
    ap.add_argument("--all-t", action="store_true", help="with --sweep: all token counts for int8 too")
    ap.add_argument("--with-head", action="store_true", help="add the fp16 head (65536 x 4096, matmul_vec_fp16 / matmul_mat_fp16) to every step")
    ap.add_argument("--schedule", action="store_true", help="config 5: multi-slot serving schedule (use with --quant nf4) instead of one step size")
    ap.add_argument("--slots", type=int, default=32)
    ap.add_argument("--full-layers", action="store_true", help="every op of the v6 layers (35 per layer), not only the quantized products")
    ap.add_argument("--ops", action="store_true", help="time of every layer op alone at the 7B layer shape")
    ap.add_argument("--fused", action="store_true", help="with --full-layers / --full-model: the fused small ops (12 launches per layer instead of 35)")
    ap.add_argument("--full-model", action="store_true", help="--full-layers plus embedding, head and softmax: a whole model step")
    ap.add_argument("--v7-layers", action="store_true",
                    help="every op of RWKV-v7 layers at the 7B shape (4096 channels, 64 heads, FFN 16384): --layers of them, --tokens per step")
    ap.add_argument("--packed-shifts", action="store_true", help="with --v5-model / --v7-layers: the token shifts of each half of a layer in one launch")
    ap.add_argument("--loader", action="store_true",
                    help="the C++ loader: the f16 matrices of --layers 7B-shape layers from a safetensors file into Int8 matrices (file -> device -> pack)")
    ap.add_argument("--v5-model", action="store_true",
                    help="config 1: the RWKV-v5-shape model (12 layers, 768 channels, FFN 2688, vocabulary 65536), every op: a 32-token prompt run, then decode steps")
    ap.add_argument("--stamps", action="store_true",
                    help="timeline of the Int8 decode step from wall-clock stamps written by stamped builds of its kernels (sets WRQ_TEST_HOOKS=1)")
    args = ap.parse_args()
    if args.stamps:
        os.environ["WRQ_TEST_HOOKS"] = "1"
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus above 1 is not supported: the path would shard by weight rows, one all-gather of the outputs per product")

    if args.loader:
        loader_bench(args)
        return

    import torch

    wrq = importlib.import_module("web-rwkv_amd")
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    torch.cuda.set_device(0)
    assert wrq.lib().wrq_init() == 0, wrq.lib().wrq_last_error().decode()

    if args.sweep:
        sweep(wrq, torch, args)
        return
    probe = run_probe(torch) if args.probe else None

    C, H, depth = MODEL_SHAPES[args.model]
    if args.layers is None:
        args.layers = depth
    if args.ops:
        ops_table(wrq, torch, args, C)
        return
    if args.full_layers or args.full_model:
        full_layers(wrq, torch, args, C, H)
        return
    if args.v5_model:
        v5_model(wrq, torch, args)
        return
    if args.v7_layers:
        v7_layers(wrq, torch, args)
        return
    layers = build_model(wrq, torch, args.quant, args.layers, C, H)
    if args.schedule:
        schedule(wrq, torch, args, layers, C, H)
        return
    if args.stamps:
        stamps_timeline(wrq, torch, args, layers, C, H)
        return
    dec = Decode(wrq, torch, layers, C, H, args.tokens)

    def graph_ms(step_fn):
        """ms per step (device, wall) of `step_fn` captured once and replayed."""
        step_fn()
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            step_fn()
        return time_steps(torch, gr.replay, args.steps, args.warmup)

    grouped = not args.no_group
    step = dec.step_grouped if grouped else dec.step
    if grouped:
        dec.launches = 4 * len(layers)
    head_bytes = 0
    if args.with_head:
        # the head of the model (src/runtime/v6.rs:982-987): plain f16, one product per step on
        # the last token of the run (decode) -- here on all T tokens of the step
        gh = torch.Generator(device="cuda").manual_seed(SEED + 6)
        head = wrq.Matrix.fp16((torch.randn((65536, C), generator=gh, device="cuda") * 0.02).half())
        head_x = torch.randn((args.tokens, C), generator=gh, device="cuda").half()
        head_out = torch.empty((args.tokens, 65536), dtype=torch.float32, device="cuda")
        body = step

        def step():
            body()
            head.matmul_op(head_x, head_out, turbo=dec.turbo)

        head_bytes = fp16_bytes(C, 65536, args.tokens, 4)
        dec.launches += 1
    if args.no_graph:
        fn = step
    else:
        # the launches of one step are captured once and replayed: the per-step host cost of
        # 256 launches otherwise bounds batch-1 decode
        step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        fn = graph.replay

    ms, wall_ms = time_steps(torch, fn, args.steps, args.warmup)
    nbytes = dec.bytes_per_step(args.quant) + head_bytes
    tok_s = args.tokens * 1e3 / wall_ms
    launch_us = ms * 1e3 / dec.launches
    achieved = nbytes / dec.launches / launch_us / 1e3  # GB/s
    # HBM bytes per launch: not measurable inside this process (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE are
    # counter runs of their own, scaled by the same counters on a 256 MiB plain copy).  The figure is read
    # from the tracked summary of those runs for this workload, which states its commands; null without one.
    traffic = None
    if args.tokens == 1 and grouped and not args.with_head and args.layers == 32 and args.model == "7b":
        traffic = read_traffic(args.quant)
    kernel = dominant_kernel(args.quant, args.tokens)
    out = {
        "metric": "Int8/NF4 matmul HBM GB/s (% of peak); RWKV-7B-shape decode tok/s, batch 1",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8" if args.quant == "int8" else "u4",
        "data": "synthetic",
        "config": {
            "workload": f"{'config 4: ' if args.model == '7b' else ''}RWKV-v6 {args.model.upper().replace('B', '.', 1) + 'B' if 'b' in args.model[:-1] else args.model.upper()}-shape ({args.layers} layers, d_model {C}, FFN {H}), all layers {args.quant}, "
                        f"batch 1, {args.tokens} token(s) per step, quantized-matrix path only (8 products per layer)",
            "quant": args.quant, "tokens_per_step": args.tokens, "hip_graph": not args.no_graph, "grouped_launches": grouped,
            "fp16_head": bool(args.with_head),
        },
        "hbm_gbps": round(nbytes / (ms * 1e-3) / 1e9, 1),
        "bytes_per_step": nbytes,
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
            "traffic_source": None if traffic is None else f"tracked rocprofv3 --pmc summary profiles/gemv_{args.quant}_decode_7b_hbm_traffic.txt (not measured in this run)",
            "kernel": kernel, "launches_per_step": dec.launches,
            "avg_launch_us": round(launch_us, 3), "bytes_per_launch": nbytes // dec.launches,
            "plain_read_model_frac": plain_read_frac(nbytes, dec.launches),
        },
    }
    default_line = (args.quant == "int8" and args.tokens == 1 and grouped and not args.no_graph and not args.with_head and not args.main_only)
    if default_line:
        # the literal call pattern of the reference's layer (src/runtime/v6.rs:806-938): eight separate products per layer
        ms_u, wall_u = graph_ms(dec.step)
        out["ungrouped"] = {"value": round(1e3 / wall_u, 2), "unit": "tok/s", "ms_per_step": round(wall_u, 4), "launches_per_step": 8 * len(layers),
                            "frac": round(nbytes / (ms_u * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                            "plain_read_model_frac": plain_read_frac(nbytes, 8 * len(layers))}
        # the other half of the metric: the same step with every layer NF4
        del graph
        layers4 = build_model(wrq, torch, "nf4", args.layers, C, H)
        dec4 = Decode(wrq, torch, layers4, C, H, 1)
        ms4, wall4 = graph_ms(dec4.step_grouped)
        nbytes4 = dec4.bytes_per_step("nf4")
        n4 = 4 * len(layers4)
        out["nf4"] = {"value": round(1e3 / wall4, 2), "unit": "tok/s", "ms_per_step": round(wall4, 4), "dtype": "u4",
                      "hbm_gbps": round(nbytes4 / (ms4 * 1e-3) / 1e9, 1), "bytes_per_step": nbytes4,
                      "roofline": {"bound": "hbm", "achieved": round(nbytes4 / (ms4 * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                   "frac": round(nbytes4 / (ms4 * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                                   "traffic": read_traffic("nf4") if args.layers == 32 and args.model == "7b" else None,
                                   "kernel": dominant_kernel("nf4", 1), "launches_per_step": n4,
                                   "avg_launch_us": round(ms4 * 1e3 / n4, 3), "bytes_per_launch": nbytes4 // n4,
                                   "plain_read_model_frac": plain_read_frac(nbytes4, n4)}}
        del dec4, layers4
    # from some token count on the matrix cores bound a step, not HBM: 2 K R T flops per product against the
    # dense f16 peak take longer than the packed bytes against the HBM peak
    flops = 2.0 * args.tokens * len(layers) * (5 * C * C + 2 * C * H + C * C) + (2.0 * args.tokens * C * 65536 if args.with_head else 0.0)
    if flops / (MFMA_F16_PEAK_TFLOPS * 1e12) > nbytes / (HBM_PEAK_GBPS * 1e9):
        tflops = flops / dec.launches / launch_us / 1e6
        out["roofline"].update({"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "flops_per_launch": int(flops // dec.launches)})
    if probe:
        out["probe"] = probe
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wrq, torch, layers, dec, args.quant, min(args.cpu_sample_layers, args.layers), args.cpu_seconds)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
