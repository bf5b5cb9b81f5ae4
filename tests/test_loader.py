"""The C++ loader (include/wrq_loader.hpp: safetensors file -> discount -> packed device matrix,
src/runtime/loader.rs:44-74, :389-392, :651-762) against a model file written here with the
`safetensors` package and what numpy and the CPU restatement of the packers make of the same tensors."""
import os
import subprocess

import numpy as np
import pytest

from test_host_cpp import BIN, build_host_tests

SEED = 0x57524c44


def write_model(tmp_path, oracle):
    from safetensors.numpy import save_file

    rng = np.random.default_rng(SEED)
    out_w = (rng.standard_normal((256, 256), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    ffn_v = (rng.standard_normal((256, 384), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    # values that the discount takes into and through the subnormal range of f16, and ties of the rounding
    ffn_v[0, :8] = np.array([6.1e-5, 1.2e-7, 5.96e-8, -3.0e-5, 65504.0, -65504.0, 0.0, 1.0009765625], dtype=np.float16)
    tensors = {"blocks.6.att.output.weight": out_w, "blocks.6.ffn.value.weight": ffn_v,
               "blocks.6.att.time_first": rng.standard_normal((4, 64)).astype(np.float32)}
    path = str(tmp_path / "model.st")
    save_file(tensors, path, metadata={"note": 'a "quoted" word'})
    with open(path, "rb") as f:
        whole = f.read()
    with open(tmp_path / "cut.st", "wb") as f:
        f.write(whole[:-100])
    # a header whose extents multiply to 2^65 bytes: in 64-bit arithmetic that is 0, the size of its data range
    import json
    import struct

    header = json.dumps({"huge": {"dtype": "F16", "shape": [2 ** 31, 2 ** 31, 4], "data_offsets": [0, 0]}}).encode()
    with open(tmp_path / "wraps.st", "wb") as f:
        f.write(struct.pack("<Q", len(header)) + header)
    for name in ("blocks.6.att.output.weight", "blocks.6.ffn.value.weight"):
        for tag, d in ((".half.f16", 0.5), (".x03.f16", 0.3)):
            # Loader::load_matrix_f16_discount: f16::from_f32(discount * x.to_f32()), src/runtime/loader.rs:660-661
            (np.float32(d) * tensors[name].astype(np.float32)).astype(np.float16).tofile(tmp_path / (name + tag))
    # an adapter file (src/runtime/loader.rs:355-386): low-rank halves `<stem>.lora.0` [in, rank] and `.lora.1` [out, rank] for
    # ffn.value, a whole tensor of the same name for att.output; blended with LoraBlend::full(0.5): out = alpha / rank * xa^T xb + w
    rank, alpha = 8, np.float32(0.5)
    xa = (rng.standard_normal((384, rank), dtype=np.float32) * np.float32(0.1)).astype(np.float16)  # [in, rank]
    xb = (rng.standard_normal((256, rank), dtype=np.float32) * np.float32(0.1)).astype(np.float16)  # [out, rank]
    ov = (rng.standard_normal((256, 256), dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    save_file({"blocks.6.ffn.value.lora.0": xa, "blocks.6.ffn.value.lora.1": xb, "blocks.6.att.output.weight": ov}, str(tmp_path / "lora.st"))
    for tag, d in ((".lora.f16", np.float32(1.0)), (".lora_half.f16", np.float32(0.5))):
        base = (d * ffn_v.astype(np.float32)).astype(np.float16).astype(np.float32)  # the discounted matrix is an f16 tensor before the blend
        low = xb.astype(np.float32) @ xa.astype(np.float32).T  # [out, in]
        (np.float32(d * alpha / rank) * low + base).astype(np.float16).tofile(tmp_path / ("blocks.6.ffn.value.weight" + tag))
        base = (d * out_w.astype(np.float32)).astype(np.float16).astype(np.float32)
        (np.float32(d * alpha) * ov.astype(np.float32) + base).astype(np.float16).tofile(tmp_path / ("blocks.6.att.output.weight" + tag))
    if oracle is not None:
        name = "blocks.6.ffn.value.weight"
        half = (np.float32(0.5) * ffn_v.astype(np.float32)).astype(np.float16)
        w, m, _ = oracle.quant_int8(half)
        w.tofile(tmp_path / (name + ".int8.w")), m.tofile(tmp_path / (name + ".int8.m"))
        w, m = oracle.quant_nf4(half)
        w.tofile(tmp_path / (name + ".nf4.w")), m.tofile(tmp_path / (name + ".nf4.m"))
    return path


def run(flag, path, tmp_path):
    if not os.path.exists(BIN):
        build_host_tests()
    r = subprocess.run([BIN, flag, path, str(tmp_path)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host tests ok" in r.stdout


def test_loader_reads_and_discounts(tmp_path):
    run("--loader", write_model(tmp_path, None), tmp_path)


@pytest.mark.gpu
def test_loader_packs_on_the_gpu(tmp_path, oracle):
    print("case: C++ loader, safetensors file -> discount -> int8 / nf4 / sf4 / f16 matrices", flush=True)
    run("--loader-gpu", write_model(tmp_path, oracle), tmp_path)
