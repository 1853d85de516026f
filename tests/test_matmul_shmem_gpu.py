"""GPU parity tests of matmul_shmem (the SIMT, no-matrix-core path) through the C ABI.

Bars: int32 is exact (the reference's own <int,int> test uses atol 0, matmul_shmem.cu:306-307);
fp32 is bit-identical to the oracle's sequential fused-multiply-add loop and within
|C - Cref| <= 1e-4 * (|Cref| + 1) of the oracle's multiply-then-add loop (the reference's CPU check);
fp16 in/out with fp32 accumulation equals the fused loop rounded once to half.
"""
import numpy as np
import pytest
import torch

from tests import gpu_util as G

pytestmark = pytest.mark.gpu

RTOL_F32 = 1e-4

LEGAL = [(32, 2), (32, 4), (32, 8), (32, 16), (32, 32), (64, 1), (64, 2), (64, 4), (64, 8), (64, 16), (128, 2), (128, 4), (128, 8)]


def run(ck, dtype, a, b, M, N, K, tile, br, bt):
    da, db = G.to_dev(a), G.to_dev(b)
    tdt = {ck.DT_F32: torch.float32, ck.DT_I32: torch.int32, ck.DT_F16: torch.float16}[dtype]
    dc = torch.full((M, N), -9, dtype=tdt, device="cuda")
    ck.matmul_shmem(dtype, da, db, dc, M, N, K, tile, br, bt)
    torch.cuda.synchronize()
    return dc.cpu().numpy()


@pytest.mark.parametrize("bt", [False, True])
def test_int32_exact_all_tilings(ck, oracle, bt):
    # reference: 256^3, values in [-10, 10], atol 0
    M = N = K = 256
    a = ck.fill_int(ck.DT_I32, (M, K), 17, 0, -10, 10)
    b = ck.fill_int(ck.DT_I32, (N, K) if bt else (K, N), 17, 1, -10, 10)
    want = oracle.matmul(oracle.DT_I32, a, b, bt)
    assert np.array_equal(want, (a.astype(np.int64) @ (b.T if bt else b).astype(np.int64)).astype(np.int32))
    for tile, br in LEGAL:
        assert ck.check_matmul_shmem_tuning(tile, br) == ck.OK
        got = run(ck, ck.DT_I32, a, b, M, N, K, tile, br, bt)
        assert np.array_equal(got, want), (tile, br)


@pytest.mark.parametrize("bt", [False, True])
def test_fp32_bit_identical_to_fused_loop(ck, oracle, bt):
    M, N, K = 256, 384, 512
    a = ck.fill_uniform(ck.DT_F32, (M, K), 18, 0)
    b = ck.fill_uniform(ck.DT_F32, (N, K) if bt else (K, N), 18, 1)
    fused = oracle.matmul(oracle.DT_F32, a, b, bt, fused=True)
    plain = oracle.matmul(oracle.DT_F32, a, b, bt, fused=False)
    for tile, br in LEGAL:
        got = run(ck, ck.DT_F32, a, b, M, N, K, tile, br, bt)
        assert np.array_equal(got.view(np.uint32), fused.view(np.uint32)), (tile, br)
        n, worst = oracle.count_outside_rel(plain, got, RTOL_F32)
        assert n == 0, (tile, br, worst)
        assert oracle.count_incorrect(plain, got, 0.1) == 0  # the reference's criterion (matmul_shmem.cu:300)


def test_fp16_in_out_fp32_accumulate(ck, oracle):
    M = N = K = 256
    a = ck.fill_uniform(ck.DT_F16, (M, K), 19, 0)
    b = ck.fill_uniform(ck.DT_F16, (K, N), 19, 1)
    want = oracle.matmul(oracle.DT_F16, a, b, False, fused=True).astype(np.float16)
    for tile, br in ((32, 8), (64, 4), (128, 2), (128, 8)):
        got = run(ck, ck.DT_F16, a, b, M, N, K, tile, br, False)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), (tile, br)


@pytest.mark.parametrize("block_rows", [4, 2])   # 4: the instance bench.py times and profiles/ records (8 x 4 micro-tile)
def test_config2_fp32_4096_b_transposed(ck, oracle, block_rows):
    M = N = K = 4096
    a = ck.fill_uniform(ck.DT_F32, (M, K), 0xC0FFEE02, 0)
    b = ck.fill_uniform(ck.DT_F32, (N, K), 0xC0FFEE02, 1)
    got = run(ck, ck.DT_F32, a, b, M, N, K, 128, block_rows, True)
    if block_rows == 4:
        # the benchmarked instance: the whole matrix, bit for bit, against the oracle's fused multiply-add loop
        fused = oracle.matmul(oracle.DT_F32, a, b, True, fused=True)
        assert np.array_equal(got.view(np.uint32), fused.view(np.uint32))
    else:
        # eight rows of every tile row (at a different height in each), and the last eight rows
        bands = [r0 + (r0 // 128 * 24) % 120 for r0 in range(0, M, 128)] + [M - 8]
        for r0 in bands:
            fused = oracle.matmul(oracle.DT_F32, a, b, True, fused=True, rows=(r0, r0 + 8))
            assert np.array_equal(got[r0:r0 + 8].view(np.uint32), fused.view(np.uint32)), r0
    for r0 in (0, 2048, 4088):
        plain = oracle.matmul(oracle.DT_F32, a, b, True, fused=False, rows=(r0, r0 + 8))
        n, worst = oracle.count_outside_rel(plain, got[r0:r0 + 8], RTOL_F32)
        assert n == 0, worst
    # linearity checksum over the whole matrix in float64
    lhs = got.astype(np.float64).sum(axis=1)
    rhs = a.astype(np.float64) @ b.astype(np.float64).sum(axis=0)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64).sum(axis=0) + 1.0
    assert np.max(np.abs(lhs - rhs) / scale) < 1e-5


def test_cpp_driver_through_the_matmul_shmem_template(ck):
    # the C++ face (ckopt::matmul_shmem<DT, DT_ACC>) driven by a test main in the role of the reference's own
    # (matmul_shmem.cu:176-325): all three element types over every legal (tile_dim, block_rows), <int, int> at
    # tolerance 0, then the TFLOPS lines
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "build", "matmul_shmem_driver")
    assert os.path.exists(exe), "tests/cpp/build/matmul_shmem_driver is not built (make -C tests/cpp)"
    r = subprocess.run([exe, "all", "2048"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "PASSED" in r.stdout and "failed" not in r.stdout
    for name in ("<half, float>, correctness", "<float, float>, correctness", "<int, int>, correctness", "<int, int>, [TFLOPS]"):
        assert name in r.stdout
    passed = [l for l in r.stdout.splitlines() if l.endswith(": passed")]
    rates = [l for l in r.stdout.splitlines() if l.startswith("(") and "): " in l and not l.endswith("ed")]
    assert len(passed) >= 3 * 2 * 10 and len(rates) >= 3 * 10 and all(float(l.split("): ")[1]) > 0.1 for l in rates)
