"""Pins the CPU oracle (oracle/matmul_oracle.c) before anything is compared against it.

Every check here is independent of the oracle's own formula: closed forms the reference's tests
hold (constant matrices, matmul_test.h:279-288), exact integer arithmetic in numpy int64, special
operands (identity, one-hot) that reduce the product to a copy, library conversions (numpy fp16,
torch bf16), the README's accumulator table, set-bijection of the tile order, and the shared-memory
figures that follow from the reference's formula (port_2.cu:1057-1086).
"""
import numpy as np
import pytest
import torch

from tests.gpu_util import bf16_bits_to_f32, f32_to_bf16_bits


def test_half_decode_matches_numpy_for_all_bit_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().oracle_half_to_float(int(b)) for b in bits[::7]], dtype=np.float32)
    w = want[::7]
    both_nan = np.isnan(w) & np.isnan(got)
    assert np.array_equal(w[~both_nan].view(np.uint32), got[~both_nan].view(np.uint32))


def test_bf16_decode_matches_torch(oracle):
    bits = np.arange(0, 65536, 5, dtype=np.uint16)
    want = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy()
    got = np.array([oracle.lib().oracle_bf16_to_float(int(b)) for b in bits], dtype=np.float32)
    both_nan = np.isnan(want) & np.isnan(got)
    assert np.array_equal(want[~both_nan].view(np.uint32), got[~both_nan].view(np.uint32))


@pytest.mark.parametrize("blocked", [False, True])
@pytest.mark.parametrize("K", [64, 1024, 4096])
def test_constant_matrices_closed_form(oracle, blocked, K):
    # reference fixture: A == 1, B == 10, C == 1  ->  alpha * 10 * K + beta (matmul_test.h:229, :280-281)
    M, N = 48, 80
    a = np.full((M, K), 1, dtype=np.float16)
    bt = np.full((N, K), 10, dtype=np.float16)
    c = np.ones((M, N), dtype=np.float32)
    for alpha, beta in ((1.0, 1.0), (2.0, 0.0), (0.5, 3.0)):
        out = oracle.gemm(oracle.DT_F16, a, bt, c, alpha, beta, blocked=blocked)
        assert np.all(out == np.float32(alpha * 10 * K + beta))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(33, 47, 129), (64, 64, 256), (5, 260, 77)])
def test_small_integer_inputs_are_exact(oracle, dtype, shape):
    M, N, K = shape
    rng = np.random.default_rng(7)
    ai = rng.integers(-3, 4, size=(M, K))
    bi = rng.integers(-3, 4, size=(N, K))
    want = (ai.astype(np.int64) @ bi.astype(np.int64).T).astype(np.float32)
    if dtype == "f16":
        a, bt, dt = ai.astype(np.float16), bi.astype(np.float16), oracle.DT_F16
    else:
        a, bt, dt = f32_to_bf16_bits(ai.astype(np.float32)), f32_to_bf16_bits(bi.astype(np.float32)), oracle.DT_BF16
    for blocked in (False, True):
        got = oracle.gemm(dt, a, bt, blocked=blocked)
        assert np.array_equal(got, want)


def test_blocked_equals_scalar_bit_for_bit(oracle):
    rng = np.random.default_rng(3)
    M, N, K = 37, 301, 515
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    bt = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    c = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    s = oracle.gemm(oracle.DT_F16, a, bt, c, 1.25, -0.5, blocked=False)
    b = oracle.gemm(oracle.DT_F16, a, bt, c, 1.25, -0.5, blocked=True)
    assert np.array_equal(s.view(np.uint32), b.view(np.uint32))
    # a row range gives the same rows
    r = oracle.gemm(oracle.DT_F16, a, bt, c, 1.25, -0.5, rows=(5, 19), blocked=True)
    assert np.array_equal(r.view(np.uint32), s[5:19].view(np.uint32))


def test_identity_and_one_hot_operands(oracle):
    rng = np.random.default_rng(11)
    K = 96
    a = rng.uniform(-1, 1, (40, K)).astype(np.float16)
    eye = np.eye(K, dtype=np.float16)           # Bt = I  ->  D = A
    out = oracle.gemm(oracle.DT_F16, a, eye)
    assert np.array_equal(out, a.astype(np.float32))
    # Bt row j one-hot at k = perm[j] with weight w[j]: D[i, j] = a[i, perm[j]] * w[j] (one exact product)
    perm = rng.permutation(K)[:50]
    w = rng.uniform(-2, 2, 50).astype(np.float16)
    bt = np.zeros((50, K), dtype=np.float16)
    bt[np.arange(50), perm] = w
    out = oracle.gemm(oracle.DT_F16, a, bt)
    assert np.array_equal(out, a[:, perm].astype(np.float32) * w.astype(np.float32)[None, :])


def test_random_inputs_close_to_float64(oracle):
    rng = np.random.default_rng(5)
    M, N, K = 64, 96, 2048
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    bt = rng.uniform(-1, 1, (N, K)).astype(np.float16)
    out = oracle.gemm(oracle.DT_F16, a, bt)
    ref = a.astype(np.float64) @ bt.astype(np.float64).T
    # sequential fp32 summation of K exact products: error bound ~ K * eps * sum|terms|
    assert np.max(np.abs(out - ref)) < 2e-3


def test_bt_stride_is_k_for_non_square(oracle):
    # the reference indexes Bt with stride dim.n (matmul_test.h:296), valid only for square problems;
    # a non-square product must still equal the textbook one
    rng = np.random.default_rng(9)
    ai = rng.integers(-2, 3, size=(16, 40))
    bi = rng.integers(-2, 3, size=(24, 40))
    got = oracle.gemm(oracle.DT_F16, ai.astype(np.float16), bi.astype(np.float16))
    assert np.array_equal(got, (ai @ bi.T).astype(np.float32))


@pytest.mark.parametrize("b_transposed", [False, True])
def test_matmul_shmem_oracle_int_exact_and_float(oracle, b_transposed):
    rng = np.random.default_rng(13)
    M, N, K = 24, 40, 64
    ai = rng.integers(-10, 11, size=(M, K)).astype(np.int32)
    bi = rng.integers(-10, 11, size=(N, K) if b_transposed else (K, N)).astype(np.int32)
    want = ai.astype(np.int64) @ (bi.T if b_transposed else bi).astype(np.int64)
    got = oracle.matmul(oracle.DT_I32, ai, bi, b_transposed)
    assert np.array_equal(got, want.astype(np.int32))
    # float inputs holding the same integers: both the mul+add and the fused variant are exact
    for fused in (False, True):
        gotf = oracle.matmul(oracle.DT_F32, ai.astype(np.float32), bi.astype(np.float32), b_transposed, fused)
        assert np.array_equal(gotf, want.astype(np.float32))
    # fused differs from mul+add only by rounding on real-valued data
    af = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    bf = rng.uniform(-1, 1, (N, K) if b_transposed else (K, N)).astype(np.float32)
    ref = af.astype(np.float64) @ (bf.T if b_transposed else bf).astype(np.float64)
    for fused in (False, True):
        assert np.max(np.abs(oracle.matmul(oracle.DT_F32, af, bf, b_transposed, fused) - ref)) < 1e-4


def test_count_incorrect_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    e = rng.uniform(-5, 5, 1000).astype(np.float32)
    r = e + rng.uniform(-0.2, 0.2, 1000).astype(np.float32)
    assert oracle.count_incorrect(e, r, 0.1) == int(np.sum(np.abs(e - r) > np.float32(0.1)))
    n, worst = oracle.count_outside_rel(e, r, 1e-2)
    ratio = np.abs(r - e) / (np.abs(e) + 1)
    assert n == int(np.sum(~(ratio <= np.float32(1e-2))))
    assert abs(worst - float(ratio.max())) < 1e-6


def test_num_acc_matches_readme_table(oracle):
    # readme/compiler_mapped_workload.jpg: 64/8 -> 2, 64/4 -> 4, 128/8 -> 8, 128/4 -> 16
    L = oracle.lib()
    assert [L.oracle_get_num_acc(64, 8), L.oracle_get_num_acc(64, 4), L.oracle_get_num_acc(128, 8),
            L.oracle_get_num_acc(128, 4)] == [2, 4, 8, 16]
    # warp tile rows x cols: 1x2, 2x2, 2x4, 4x4
    assert [L.oracle_get_warp_tile_rows(64, 8), L.oracle_get_warp_tile_rows(64, 4), L.oracle_get_warp_tile_rows(128, 8),
            L.oracle_get_warp_tile_rows(128, 4)] == [1, 2, 2, 4]


@pytest.mark.parametrize("M,N,t,g", [(512, 512, 128, 1), (1024, 768, 128, 3), (640, 1280, 64, 4), (256, 256, 64, 6)])
def test_tile_order_is_a_bijection_onto_tile_origins(oracle, M, N, t, g):
    L = oracle.lib()
    tiles = (M // t) * (N // t)
    got = sorted(L.oracle_get_tile_offset_cd(M, N, t, g, tc) for tc in range(tiles))
    want = sorted(r * t * N + c * t for r in range(M // t) for c in range(N // t))
    assert got == want
    # brute-force statement of the grouped order: groups of g tile rows, column-major inside a group
    order = []
    for first in range(0, M // t, g):
        rows = min(g, M // t - first)
        for c in range(N // t):
            for r in range(rows):
                order.append((first + r) * t * N + c * t)
    assert [L.oracle_get_tile_offset_cd(M, N, t, g, tc) for tc in range(tiles)] == order


def test_reference_shared_memory_figures(oracle):
    L = oracle.lib()
    # tile mode, t = 128, sk = 64, half / float: 2*128*(64+16)*2 = 40960 per stage + barriers
    f = lambda S, sk=64: L.oracle_get_shmem_req(2, 4, 128, sk, 0, 0, 128, 128, S, 4)
    # S = 1: 5 barriers = 40 B, + 40 % 32 = 8 -> 48; the C/D tile (128*128*4 = 65536) dominates
    assert f(1) == 65536 + 48
    # S = 2: 9 barriers = 72 B, + 72 % 32 = 8 -> 80; two stages of 40960
    assert f(2) == 2 * 40960 + 80
    # S = 3: 13 barriers = 104 B, + 104 % 32 = 8 -> 112
    assert f(3) == 3 * 40960 + 112
    assert f(2, 128) == 2 * 2 * 128 * (128 + 16) * 2 + 80
    # the "+ size % 32" quirk is not a round-up to 32
    assert (104 + 104 % 32) % 32 != 0
