"""wrq_matmul_mat_int8_noalloc: the chunk product whose split-K partial sums live in a fixed array of
the library (for callers that cannot allocate), against wrq_matmul_mat_int8 through the C ABI.

The two entry points run the same kernels, so where they take the same split outputs must agree to the
last bit; the bar that counts is the product bar, |a - b| <= max(eps, eps * max(|a|, |b|)), eps = 2e-3,
also held against the float64 product of the dequantised weights."""
import numpy as np
import pytest

from helpers import EPS, assert_close, gen_f16, int8_dequant64, truth_matmul

pytestmark = pytest.mark.gpu

SEED = 0x57525100


def _case(gpu, oracle, torch, K, R, T, seed):
    rng = np.random.default_rng(seed)
    w = gen_f16(rng, (R, K), 0.02)
    x = gen_f16(rng, (T, K), 1.0)
    u8, mm, _ = oracle.quant_int8(w)
    wd, md, xd = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (u8, mm, x))
    want = torch.full((T, R), float("nan"), dtype=torch.float32, device="cuda")
    got = torch.full((T, R), float("nan"), dtype=torch.float32, device="cuda")
    gpu.TensorOp.matmul_mat_int8(wd, md, xd, want)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]  # hipMemGetInfo: what the device has left, whoever allocates
    gpu.TensorOp.matmul_mat_int8_noalloc(wd, md, xd, got)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the no-alloc entry point changed the device's free memory"
    return got.cpu().numpy(), want.cpu().numpy(), truth_matmul(int8_dequant64(u8, mm), x)


def test_no_alloc_entry_matches_plain_entry_twice(gpu, oracle):
    import torch

    # first call: 4096 x 4096 at 32 tokens -- 32 row tiles on 256 CUs, so K is split over workgroups and
    # the partial sums pass through the fixed array; second call: a smaller product right behind it,
    # which finds the first call's partial sums in the array and must not read them
    for K, R, T in ((4096, 4096, 32), (1024, 512, 16)):
        print("case: no_alloc", K, R, T, flush=True)
        got, want, truth = _case(gpu, oracle, torch, K, R, T, SEED + K + R + T)
        assert np.isfinite(got).all()
        assert_close(got, want, EPS, f"noalloc vs plain entry {K}x{R}x{T}")
        assert np.array_equal(got, want), "same kernels, same split: expected bit-equal outputs"
        assert_close(got, truth, EPS, f"noalloc vs float64 {K}x{R}x{T}")


def test_no_alloc_entry_takes_fewer_splits_where_the_preferred_split_does_not_fit(gpu, oracle):
    import torch

    # 4096 rows x 14336 at 192 tokens: the preferred 8-way split would put 24 MiB of partial sums into the 16 MiB array;
    # the entry point splits 4 ways instead (the plain one, with more room, keeps 8): same bar, different summation order
    K, R, T = 14336, 4096, 192
    print("case: no_alloc, fewer splits", K, R, T, flush=True)
    got, want, truth = _case(gpu, oracle, torch, K, R, T, SEED + 77)
    assert np.isfinite(got).all()
    assert_close(got, want, EPS, f"noalloc vs plain entry {K}x{R}x{T}")
    assert_close(got, truth, EPS, f"noalloc vs float64 {K}x{R}x{T}")


def test_no_alloc_entry_refuses_a_pinned_split_that_does_not_fit(gpu, oracle, overrides):
    import torch

    # 65536 rows x 32 tokens with the split pinned to 8 would need 64 MiB of partial sums: the fixed array holds 16
    K, R, T = 1024, 65536, 32
    rng = np.random.default_rng(SEED + 9)
    wd = torch.from_numpy(rng.integers(0, 256, (R, K), dtype=np.uint8)).cuda()
    md = torch.from_numpy(np.tile(np.array([-0.05, 0.05], np.float16), R * K // 128)).cuda()
    xd = torch.from_numpy(gen_f16(rng, (T, K), 1.0)).cuda()
    out = torch.full((T, R), 7.0, dtype=torch.float32, device="cuda")
    overrides(gemm_ksplit=8)
    with pytest.raises(gpu.TensorError) as e:
        gpu.TensorOp.matmul_mat_int8_noalloc(wd, md, xd, out)
    assert e.value.status == gpu.ERR_SIZE and "scratch" in str(e.value)
    torch.cuda.synchronize()
    assert (out == 7.0).all(), "a refused call must not launch anything"
    gpu.TensorOp.matmul_mat_int8(wd, md, xd, out)  # the plain entry point takes fewer splits instead
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
