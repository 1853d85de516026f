"""GPU parity tests of gemm_shmem_tc_async_opt_port (all through the C ABI) against the CPU oracle.

Bars: bit-exact wherever the arithmetic is exact (constant matrices, small integers, identity,
one-hot); |D - Dref| <= 1e-2 * (|Dref| + 1) for random fp16/bf16 inputs with fp32 accumulation, the
tolerance BASELINE states. The three test kinds follow the reference's own drivers:
constant-matrix correctness sweeps (port_2.cu:1171-1279), random accuracy counts (:1281-1391) and
full-size runs checked through sampled rows and size-independent identities.
"""
import itertools

import os

import numpy as np
import pytest
import torch

from tests import gpu_util as G

pytestmark = pytest.mark.gpu

RTOL = 1e-2  # |D - Dref| <= RTOL * (|Dref| + 1), fp16/bf16 inputs, fp32 accumulation


def assert_close(oracle, ref, got, rtol=RTOL):
    n, worst = oracle.count_outside_rel(ref, got, rtol)
    assert n == 0, "%d elements outside tolerance, worst ratio %g" % (n, worst)


def mode_rows(ck, t, mode):
    if mode == "tile":
        return t["tile_dim"], t["tile_dim"]
    if mode == "wave":
        return G.wave_mode_rows(ck, t)
    return 16, 16


def all_modes(ck, tile, cw):
    """(mode, bar_steps_a, bar_steps_b) tuples legal for this tile / consumer count."""
    wtr = ck.get_warp_tile_rows(tile, cw)
    wtc = ck.get_num_acc(tile, cw) // wtr
    out = [("tile", 0, 0)]
    out += [("wave", sa, sb) for sa in range(cw // 2 + 1) for sb in range(3)]
    out += [("acc", sa, sb) for sa in sorted({0, wtr // 2, wtr - 1}) for sb in sorted({0, wtc // 2, wtc - 1})]
    return out


def make_tuning(ck, tile, sk, stages, p, c, mode="tile", sa=0, sb=0, group=4, cus=256):
    t = G.tuning(tile_dim=tile, segment_dim_k=sk, num_stages=stages, num_producer_warps=p, num_consumer_warps=c,
                 bar_steps_a=sa, bar_steps_b=sb, tile_group_m=group, num_sms=cus)
    t["bar_step_rows_a"], t["bar_step_rows_b"] = mode_rows(ck, t, mode)
    return t


def legal(ck, t):
    return ck.check_gemm_tuning(t["tile_dim"], t["segment_dim_k"], t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"],
                                t["bar_step_rows_b"], t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                t["num_consumer_warps"], t["num_sms"]) == ck.OK


# ---- config 1: fp16 512^3, uniform[-1,1), seeded, checked against the full CPU reference -------------
@pytest.mark.parametrize("tile,sk,stages,p,c", [(64, 64, 3, 2, 4), (128, 64, 2, 2, 4), (128, 64, 3, 4, 8),
                                                 (128, 32, 4, 2, 8), (128, 128, 2, 8, 4), (256, 32, 4, 4, 8),
                                                 (256, 64, 2, 2, 8)])
def test_config1_fp16_512_uniform(ck, oracle, tile, sk, stages, p, c):
    M = N = K = 512
    a = ck.fill_uniform(ck.DT_F16, (M, K), 0xC0FFEE01, 0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 0xC0FFEE01, 1)
    ref = oracle.gemm(oracle.DT_F16, a, bt)
    d = G.run_gemm(ck, ck.DT_F16, a, bt, t=make_tuning(ck, tile, sk, stages, p, c))
    assert_close(oracle, ref, d)
    # the reference's accuracy criterion: count of |err| > 0.1 (matmul_test.h:320) must be zero too
    assert oracle.count_incorrect(ref, d, 0.1) == 0


# ---- constant matrices: the reference's correctness sweep, closed form alpha*1*10*K + beta*1 -------------
def constant_sweep(ck):
    tuples = []
    for tile, c in ((64, 4), (64, 8), (128, 4), (128, 8), (256, 8)):
        for sk in (32, 64, 128):
            for (mode, sa, sb) in all_modes(ck, tile, c):
                for stages, p, group in ((1, 2, 1), (3, 4, 3), (2, 8, 6)):
                    t = make_tuning(ck, tile, sk, stages, p, c, mode, sa, sb, group)
                    if legal(ck, t):
                        tuples.append(t)
    return tuples


def test_constant_matrices_sweep(ck):
    dim_max = 1024
    a = G.to_dev(ck.fill_constant(ck.DT_F16, (dim_max * dim_max,), 1.0))
    bt = G.to_dev(ck.fill_constant(ck.DT_F16, (dim_max * dim_max,), 10.0))
    c = G.to_dev(ck.fill_constant(ck.DT_F32, (dim_max * dim_max,), 1.0))
    d = torch.empty(dim_max * dim_max, dtype=torch.float32, device="cuda")
    rng = np.random.default_rng(0xC0FFEE)
    tuples = constant_sweep(ck)
    assert len(tuples) > 150
    # every 5th tuple at a random tile-multiple sub-dimension (reference: GetMatDim, matmul_test.h:263-268)
    for idx, t in enumerate(tuples[::3]):
        tile = t["tile_dim"]
        dim = dim_max if idx % 5 else max(tile, int(rng.integers(0, dim_max + 1)) // tile * tile)
        d.fill_(0)
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, a, bt, c, d, 1.0, 1.0, dim, dim, dim, t["tile_dim"], t["segment_dim_k"],
                                        t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                        t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                        t["num_consumer_warps"], t["num_sms"])
        assert ck.device_status() == 0, t
        got = d[: dim * dim]
        want = 10.0 * dim + 1.0
        assert bool(torch.all(got == want)), (t, dim, float(got.min()), float(got.max()))
        assert bool(torch.all(d[dim * dim:] == 0)), "wrote past the dim x dim result"


# ---- small integers: exact for every summation order, so any race or misplaced fragment shows ----------
@pytest.mark.parametrize("tile,c", [(64, 4), (64, 8), (128, 4), (128, 8), (256, 8)])
def test_small_integers_bit_exact_all_sync_modes(ck, tile, c):
    M, N, K = 2 * tile, 3 * tile, 640
    a = ck.fill_int(ck.DT_F16, (M, K), 21, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 21, 1, -2, 2)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    n = 0
    for (mode, sa, sb), (sk, stages, p) in itertools.product(all_modes(ck, tile, c), ((32, 4, 2), (64, 2, 4), (128, 1, 2))):
        t = make_tuning(ck, tile, sk, stages, p, c, mode, sa, sb, group=2)
        if not legal(ck, t):
            continue
        d = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
        assert np.array_equal(d, want), (t, int((d != want).sum()))
        n += 1
    assert n >= 20


def test_more_stages_than_segments_and_single_segment(ck):
    # K / seg_k < num_stages: some stages are never filled
    a = ck.fill_int(ck.DT_F16, (256, 128), 3, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (256, 128), 3, 1, -2, 2)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    for sk, stages in ((128, 2), (64, 4), (32, 9)):
        for mode, sa, sb in (("tile", 0, 0), ("wave", 1, 1), ("acc", 1, 2)):
            d = G.run_gemm(ck, ck.DT_F16, a, bt, t=make_tuning(ck, 128, sk, stages, 2, 4, mode, sa, sb))
            assert np.array_equal(d, want)


def test_identity_and_one_hot(ck):
    K = 256
    a = ck.fill_uniform(ck.DT_F16, (384, K), 5, 0)
    eye = np.eye(K, dtype=np.float16)
    d = G.run_gemm(ck, ck.DT_F16, a, eye, t=make_tuning(ck, 128, 64, 2, 2, 4))
    assert np.array_equal(d, a.astype(np.float32))
    rng = np.random.default_rng(2)
    perm = rng.permutation(K)
    bt = np.zeros((K, K), dtype=np.float16)
    bt[np.arange(K), perm] = 2.0
    d = G.run_gemm(ck, ck.DT_F16, a, bt, t=make_tuning(ck, 64, 32, 3, 2, 8, "acc", 0, 1))
    assert np.array_equal(d, 2.0 * a[:, perm].astype(np.float32))


@pytest.mark.parametrize("alpha,beta", [(1.0, 1.0), (1.5, -0.75), (0.0, 2.0), (-2.0, 0.0)])
def test_alpha_beta_textbook_form(ck, oracle, alpha, beta):
    # D = alpha*A*Bt^T + beta*C as the CPU check states it (matmul_test.h:298), not alpha*(beta*C + A*Bt^T)
    M, N, K = 384, 256, 512
    a = ck.fill_uniform(ck.DT_F16, (M, K), 8, 0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 8, 1)
    c = ck.fill_uniform(ck.DT_F32, (M, N), 8, 2)
    ref = oracle.gemm(oracle.DT_F16, a, bt, c, alpha, beta)
    for t in (make_tuning(ck, 128, 64, 2, 2, 4), make_tuning(ck, 256, 32, 4, 4, 8, "wave", 2, 1)):
        d = G.run_gemm(ck, ck.DT_F16, a, bt, c, alpha, beta, t=t)
        assert_close(oracle, ref, d)


def test_bf16_uniform_and_exact(ck, oracle):
    M, N, K = 512, 384, 768
    a = ck.fill_uniform(ck.DT_BF16, (M, K), 9, 0)
    bt = ck.fill_uniform(ck.DT_BF16, (N, K), 9, 1)
    ref = oracle.gemm(oracle.DT_BF16, a, bt)
    for t in (make_tuning(ck, 128, 64, 3, 4, 8), make_tuning(ck, 256, 64, 2, 2, 8), make_tuning(ck, 64, 128, 2, 2, 4, "acc", 1, 1)):
        assert_close(oracle, ref, G.run_gemm(ck, ck.DT_BF16, a, bt, t=t))
    ai = ck.fill_int(ck.DT_BF16, (M, K), 9, 2, -3, 3)
    bi = ck.fill_int(ck.DT_BF16, (N, K), 9, 3, -3, 3)
    want = (G.as_f64(True, ai) @ G.as_f64(True, bi).T).astype(np.float32)
    assert np.array_equal(G.run_gemm(ck, ck.DT_BF16, ai, bi, t=make_tuning(ck, 128, 32, 4, 2, 8, "wave", 1, 2)), want)


@pytest.mark.parametrize("M,N,K", [(200, 136, 104), (129, 257, 72), (1, 1, 8), (513, 64, 1000), (6143, 4097, 3072)])
def test_ragged_edges_aligned_k(ck, oracle, M, N, K):
    # M, N not multiples of the tile and K not a multiple of the segment: edges zero-filled / masked.
    # The result lives in a larger allocation whose guard band must stay untouched.
    a = ck.fill_int(ck.DT_F16, (M, K), 31, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 31, 1, -2, 2)
    da, db = G.to_dev(a), G.to_dev(bt)
    guard = 4096
    buf = torch.full((M * N + 2 * guard,), -7.0, dtype=torch.float32, device="cuda")
    d = buf[guard: guard + M * N]
    big = M > 2000
    for t in ([make_tuning(ck, 256, 64, 2, 4, 8)] if big else
              [make_tuning(ck, 64, 32, 3, 2, 4), make_tuning(ck, 128, 64, 2, 2, 8, "wave", 1, 1),
               make_tuning(ck, 256, 32, 4, 4, 8), make_tuning(ck, 128, 128, 1, 2, 4, "acc", 2, 2)]):
        buf.fill_(-7.0)
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                        t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                        t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                        t["num_consumer_warps"], t["num_sms"])
        assert ck.device_status() == 0
        assert bool(torch.all(buf[:guard] == -7.0)) and bool(torch.all(buf[guard + M * N:] == -7.0))
        got = d.cpu().numpy().reshape(M, N)
        if big:
            # exact integer identity instead of a full CPU product: row sums and column sums of D
            ai, bi = a.astype(np.int64), bt.astype(np.int64)
            assert np.array_equal(got.astype(np.int64).sum(axis=1), ai @ bi.sum(axis=0))
            assert np.array_equal(got.astype(np.int64).sum(axis=0), bi @ ai.sum(axis=0))
            rows = (0, 2000, M - 1)
            for r in rows:
                assert np.array_equal(got[r], (ai[r] @ bi.T).astype(np.float32))
        else:
            assert np.array_equal(got, (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32))


@pytest.mark.parametrize("tile,c", [(64, 4), (64, 8), (128, 4), (128, 8), (256, 8)])
def test_fused_variant_no_producer_waves(ck, oracle, tile, c):
    # num_producer_waves == 0: every wave loads its share and multiplies; exact on small integers for every
    # segment size and ring depth, ragged too
    a = ck.fill_int(ck.DT_F16, (2 * tile, 640), 51, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (3 * tile, 640), 51, 1, -2, 2)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    ar = ck.fill_int(ck.DT_F16, (tile + 40, 72), 51, 2, -2, 2)
    br = ck.fill_int(ck.DT_F16, (tile - 24, 72), 51, 3, -2, 2)
    wantr = (ar.astype(np.int64) @ br.astype(np.int64).T).astype(np.float32)
    n = 0
    for sk in (32, 64, 128):
        for stages in (1, 2, 3, 4, 5, 6):
            t = make_tuning(ck, tile, sk, stages, 0, c)
            if not legal(ck, t):
                continue
            assert np.array_equal(G.run_gemm(ck, ck.DT_F16, a, bt, t=t), want), t
            assert np.array_equal(G.run_gemm(ck, ck.DT_F16, ar, br, t=t), wantr), t
            n += 1
    assert n >= 5
    # granularities other than tile have no fused instance
    t = make_tuning(ck, tile, 32, 2, 0, c, "wave", 1, 1)
    assert not legal(ck, t)
    # random data, alpha/beta, bf16
    M, N, K = 2 * tile, 2 * tile, 1024
    a2 = ck.fill_uniform(ck.DT_BF16, (M, K), 52, 0)
    b2 = ck.fill_uniform(ck.DT_BF16, (N, K), 52, 1)
    c2 = ck.fill_uniform(ck.DT_F32, (M, N), 52, 2)
    ref = oracle.gemm(oracle.DT_BF16, a2, b2, c2, 1.5, -0.5)
    assert_close(oracle, ref, G.run_gemm(ck, ck.DT_BF16, a2, b2, c2, 1.5, -0.5, t=make_tuning(ck, tile, 32, 4, 0, c)))


@pytest.mark.parametrize("dt_name", ["f16", "bf16"])
def test_synchronous_single_stage_partner(ck, oracle, dt_name):
    # num_producer_waves 0 with ONE stage: load, barrier, multiply, barrier (the schedule of the reference's first
    # tensor-core kernel, matmul_shmem_tc.cu:176-209), every tile size / segment size / wave count it is built for
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    odt = oracle.DT_F16 if dt_name == "f16" else oracle.DT_BF16
    is_bf = dt_name == "bf16"
    M, N, K = 300, 520, 328          # ragged in M and N; K ends inside a segment for every segment size
    a = ck.fill_int(dt, (M, K), 53, 0, -2, 2)
    bt = ck.fill_int(dt, (N, K), 53, 1, -2, 2)
    c = ck.fill_int(ck.DT_F32, (M, N), 53, 2, -3, 3)
    want = (2.0 * (G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T) - c).astype(np.float32)
    au = ck.fill_uniform(dt, (512, 1024), 54, 0)
    bu = ck.fill_uniform(dt, (768, 1024), 54, 1)
    ref = oracle.gemm(odt, au, bu)
    n = 0
    for tile, cw in ((64, 4), (64, 8), (128, 4), (128, 8), (256, 8)):
        for sk in (32, 64, 128):
            t = make_tuning(ck, tile, sk, 1, 0, cw, group=3, cus=7)
            assert legal(ck, t), t
            assert np.array_equal(G.run_gemm(ck, dt, a, bt, c, 2.0, -1.0, t=t), want), t
            t["num_sms"] = 256
            assert_close(oracle, ref, G.run_gemm(ck, dt, au, bu, t=t))
            n += 1
    assert n == 15


def test_port_0_and_port_1_entry_points(ck):
    M, N, K = 256, 384, 512
    a = ck.fill_int(ck.DT_F16, (M, K), 41, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 41, 1, -2, 2)
    want = torch.from_numpy((a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)).cuda()
    da, db = G.to_dev(a), G.to_dev(bt)
    d = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    ck.gemm_shmem_tc_async_opt_port_0(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, 128, 64, 3, 2, 2, 4, 256)
    assert ck.device_status() == 0 and bool(torch.equal(d, want))
    for rows_a, rows_b in ((128, 128), (64, 64), (16, 16)):
        d.zero_()
        ck.gemm_shmem_tc_async_opt_port_1(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, 128, 64, rows_a, rows_b, 3, 2, 4, 4, 256)
        assert ck.device_status() == 0 and bool(torch.equal(d, want))


def _exact_case(ck, M, N, K, seed):
    a = ck.fill_int(ck.DT_F16, (M, K), seed, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), seed, 1, -2, 2)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    return G.to_dev(a), G.to_dev(bt), want


@pytest.mark.parametrize("M,N,K", [(256, 384, 512), (700, 520, 1000), (1280, 1536, 256)])   # whole tiles; ragged in M, N and K; 120 tiles on 16 workgroups
def test_port_0_legal_set_single_producer_and_low_precision(ck, M, N, K):
    """port_0's own legal set: one producer warp (port_0.cu:538, one wave streams A then Bt of every segment), and the
    <half, half> instance (port_0.cu:866, :906); also through the port_1 launcher (port_1.cu:1292). Exact on small integers."""
    da, db, want = _exact_case(ck, M, N, K, 43)
    cus = 16 if M * N > 1 << 20 else 256
    for p, tile, sk, stages, c in ((1, 128, 64, 3, 4), (1, 64, 32, 4, 8), (1, 128, 128, 1, 8), (1, 256, 64, 2, 8), (8, 128, 64, 2, 8)):
        d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_0(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, tile, sk, 3, stages, p, c, cus)
        assert ck.device_status() == 0 and np.array_equal(d.cpu().numpy(), want), (p, tile, sk, stages, c)
    h = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    for p in (1, 2):
        h.zero_()
        ck.gemm_shmem_tc_async_opt_port_0_lp(ck.DT_F16, da, db, None, h, 1.0, 0.0, M, N, K, 128, 64, 3, 2, p, 4, cus)
        assert ck.device_status() == 0 and np.array_equal(h.cpu().numpy(), want.astype(np.float16))
    for rows in (128, 64, 16):
        h.zero_()
        ck.gemm_shmem_tc_async_opt_port_1_lp(ck.DT_F16, da, db, None, h, 1.0, 0.0, M, N, K, 128, 64, rows, rows, 3, 2, 4, 4, cus)
        assert ck.device_status() == 0 and np.array_equal(h.cpu().numpy(), want.astype(np.float16))
        d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_1(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, 128, 64, rows, rows, 3, 2, 4, 4, cus)
        assert ck.device_status() == 0 and np.array_equal(d.cpu().numpy(), want)


@pytest.mark.parametrize("M,N,K", [(256, 384, 1024), (200, 136, 1000)])
def test_segments_256_deep(ck, M, N, K):
    """segment_dim_k 256, the upper end of the reference drivers' sweep (port_2.cu:1520-1564): producer/consumer kernels
    on 64 and 128 tiles, every synchronisation granularity; exact on small integers."""
    da, db, want = _exact_case(ck, M, N, K, 47)
    for tile, c, stages in ((128, 4, 1), (128, 8, 1), (64, 4, 2), (64, 8, 2)):
        for mode, sa, sb in all_modes(ck, tile, c):
            t = make_tuning(ck, tile, 256, stages, 2, c, mode, sa, sb)
            if not legal(ck, t):
                continue
            d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, tile, 256, sa, sb, t["bar_step_rows_a"],
                                            t["bar_step_rows_b"], 4, stages, 2, c, 256)
            assert ck.device_status() == 0 and np.array_equal(d.cpu().numpy(), want), (tile, c, stages, mode, sa, sb)
    with pytest.raises(ck.CkoptError) as e:   # a legal depth without an instance
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da, db, None, d, 1.0, 0.0, M, N, K, 128, 192, 0, 0, 128, 128, 4, 1, 2, 4, 256)
    assert e.value.code == ck.ERR_NO_INSTANCE


def test_errors_with_device_pointers(ck):
    a = torch.zeros(1 << 16, dtype=torch.float16, device="cuda")
    d = torch.zeros(1 << 16, dtype=torch.float32, device="cuda")
    t = G.tuning()
    args = (t["tile_dim"], t["segment_dim_k"], t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
            t["tile_group_m"], t["num_stages"], t["num_producer_warps"], t["num_consumer_warps"], t["num_sms"])
    with pytest.raises(ck.CkoptError) as e:  # LDS over budget is the launcher's check here, not the caller's
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, a, a, None, d, 1.0, 0.0, 128, 128, 128, 128, 128, 0, 0, 128, 128, 4, 3, 2, 4, 256)
    assert e.value.code == ck.ERR_LDS_BUDGET
    ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, a, a, None, d, 1.0, 0.0, 128, 128, 128, *args)
    assert ck.device_status() == 0


def test_launch_is_deterministic_and_swizzle_is_transparent(ck):
    M = N = K = 1024
    a = ck.fill_uniform(ck.DT_F16, (M, K), 77, 0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 77, 1)
    t = make_tuning(ck, 256, 64, 2, 4, 8)
    d1 = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
    d2 = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
    assert np.array_equal(d1.view(np.uint32), d2.view(np.uint32))
    prev = ck.set_option(ck.OPT_SWIZZLE, 0)
    try:
        d3 = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
    finally:
        ck.set_option(ck.OPT_SWIZZLE, prev)
    assert np.array_equal(d1.view(np.uint32), d3.view(np.uint32))


# ---- full-size configurations: the whole matrix against the oracle + exact integer identities --------------
def full_size_check(ck, oracle, dtype, odt, M, N, K, tunings, fill):
    """Every tuning's result against the blocked oracle over ALL rows (one oracle pass per configuration)."""
    a, bt = fill(0, (M, K)), fill(1, (N, K))
    ref = oracle.gemm(odt, a, bt)
    bis16 = dtype == ck.DT_BF16
    rhs = G.as_f64(bis16, a) @ G.as_f64(bis16, bt).sum(axis=0)
    scale = (np.abs(G.as_f64(bis16, a)) @ np.abs(G.as_f64(bis16, bt)).sum(axis=0)) + 1.0
    for t in tunings:
        d = G.run_gemm(ck, dtype, a, bt, t=t)
        n, worst = oracle.count_outside_rel(ref, d, RTOL)
        assert n == 0, "%d elements outside tolerance, worst ratio %g, tuning %s" % (n, worst, t)
        # linearity checksum in float64: D @ 1 == A @ (Bt^T @ 1)
        assert np.max(np.abs(d.astype(np.float64).sum(axis=1) - rhs) / scale) < 1e-4, t


def suggested_tuning(ck, M, N, K, cus=256):
    """The tuple bench.py times for this size (ckopt_suggest_gemm_tuning)."""
    return dict(ck.suggest_gemm_tuning(M, N, K, cus))


def test_config3_fp16_8192_headline(ck, oracle):
    M = N = K = 8192
    headline = suggested_tuning(ck, M, N, K)
    assert (headline["tile_dim"], headline["segment_dim_k"], headline["num_stages"], headline["num_producer_warps"],
            headline["num_consumer_warps"]) == (256, 32, 5, 0, 8)
    pc = make_tuning(ck, 256, 64, 2, 2, 8)   # the reference's design: dedicated producer waves
    full_size_check(ck, oracle, ck.DT_F16, oracle.DT_F16, M, N, K, (headline, pc),
                    lambda s, shape: ck.fill_uniform(ck.DT_F16, shape, 0xC0FFEE03, s))
    # exact: small integers at full size
    a = ck.fill_int(ck.DT_F16, (M, K), 0xC0FFEE03, 2, -1, 1)
    bt = ck.fill_int(ck.DT_F16, (N, K), 0xC0FFEE03, 3, -1, 1)
    ai, bi = a.astype(np.int64), bt.astype(np.int64)
    for t in (headline, pc):
        d = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
        assert np.array_equal(d.astype(np.int64).sum(axis=1), ai @ bi.sum(axis=0))
        assert np.array_equal(d.astype(np.int64).sum(axis=0), bi @ ai.sum(axis=0))
        assert np.array_equal(d[4095], (ai[4095] @ bi.T).astype(np.float32))


def test_config4_long_k_shift_sync_regime(ck, oracle):
    M = N = 2048
    K = 32768
    fill = lambda s, shape: ck.fill_normal(ck.DT_F16, shape, 0xC0FFEE04, s, 0.0, 0.1)
    # the first tuple is what bench.py times: the straight-line kernel, 64 tiles of 256 x 256, K cut into 4 slices
    full_size_check(ck, oracle, ck.DT_F16, oracle.DT_F16, M, N, K,
                    (suggested_tuning(ck, M, N, K), make_tuning(ck, 128, 64, 4, 4, 8), make_tuning(ck, 128, 64, 4, 4, 8, "wave", 4, 2),
                     make_tuning(ck, 128, 64, 4, 4, 8, "acc", 1, 3)), fill)


# ---- K not a multiple of 8 / operands off a 16-byte boundary: zero-padded repack in front of the kernel ----
@pytest.mark.parametrize("M,N,K", [(64, 64, 1), (130, 70, 7), (257, 129, 33), (200, 136, 1001)])
def test_k_not_multiple_of_8_small(ck, M, N, K):
    a = ck.fill_int(ck.DT_F16, (M, K), 61, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 61, 1, -2, 2)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    for t in (make_tuning(ck, 64, 32, 3, 2, 4), make_tuning(ck, 128, 64, 2, 2, 8, "wave", 1, 1),
              make_tuning(ck, 256, 32, 4, 0, 8), make_tuning(ck, 128, 64, 2, 4, 4, "acc", 2, 2)):
        assert np.array_equal(G.run_gemm(ck, ck.DT_F16, a, bt, t=t), want), t


def test_operands_off_16_byte_boundary(ck):
    # A and Bt start 2 bytes into their allocations (K % 8 == 0): same repack path, same result
    M, N, K = 192, 320, 256
    a = ck.fill_int(ck.DT_F16, (M, K), 62, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 62, 1, -2, 2)
    want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
    da = torch.zeros(M * K + 8, dtype=torch.float16, device="cuda")
    db = torch.zeros(N * K + 8, dtype=torch.float16, device="cuda")
    da[1: 1 + M * K] = torch.from_numpy(a.reshape(-1)).cuda()
    db[3: 3 + N * K] = torch.from_numpy(bt.reshape(-1)).cuda()
    d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    t = make_tuning(ck, 128, 64, 2, 2, 4)
    ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da.data_ptr() + 2, db.data_ptr() + 6, None, d, 1.0, 0.0, M, N, K,
                                    t["tile_dim"], t["segment_dim_k"], 0, 0, t["bar_step_rows_a"], t["bar_step_rows_b"],
                                    t["tile_group_m"], t["num_stages"], t["num_producer_warps"], t["num_consumer_warps"],
                                    t["num_sms"])
    assert ck.device_status() == 0
    assert np.array_equal(d.cpu().numpy(), want)


def test_config5_bf16_6143x4097x3071(ck, oracle):
    # every dimension ragged, rows of 3071 bf16 values (6142 bytes): the whole matrix against the CPU
    # oracle within the stated tolerance, and the row-sum identity over the whole result
    M, N, K = 6143, 4097, 3071
    fill = lambda s, shape: ck.fill_uniform(ck.DT_BF16, shape, 0xC0FFEE05, s)
    full_size_check(ck, oracle, ck.DT_BF16, oracle.DT_BF16, M, N, K,
                    (suggested_tuning(ck, M, N, K), make_tuning(ck, 256, 64, 2, 2, 8), make_tuning(ck, 256, 64, 2, 0, 8),
                     make_tuning(ck, 128, 64, 4, 4, 8, "wave", 2, 1)), fill)
    # exact at full size on small integers
    a = ck.fill_int(ck.DT_BF16, (M, K), 0xC0FFEE05, 2, -1, 1)
    bt = ck.fill_int(ck.DT_BF16, (N, K), 0xC0FFEE05, 3, -1, 1)
    ai, bi = G.as_f64(True, a).astype(np.int64), G.as_f64(True, bt).astype(np.int64)
    for t in (make_tuning(ck, 256, 64, 2, 2, 8), make_tuning(ck, 256, 32, 5, 0, 8)):
        d = G.run_gemm(ck, ck.DT_BF16, a, bt, t=t)
        assert np.array_equal(d.astype(np.int64).sum(axis=1), ai @ bi.sum(axis=0))
        assert np.array_equal(d[M - 1], (ai[M - 1] @ bi.T).astype(np.float32))


def test_fused_variant_full_size(ck, oracle):
    M = N = K = 8192
    full_size_check(ck, oracle, ck.DT_F16, oracle.DT_F16, M, N, K, (make_tuning(ck, 256, 64, 2, 0, 8), make_tuning(ck, 256, 32, 5, 0, 8)),
                    lambda s, shape: ck.fill_uniform(ck.DT_F16, shape, 0xC0FFEE03, s))


def test_inner_loop_ceiling_probe_runs(ck):
    # measurement aid of bench.py (libckmeasure.so, outside the product library): finite positive rates
    import bench
    r = {(rnd, ld): bench.mfma_ceiling(rnd, ld, 20000) for rnd in (0, 1) for ld in (0, 1)}
    assert all(np.isfinite(v) and 50.0 < v < 2600.0 for v in r.values()), r
    with pytest.raises(RuntimeError):
        bench.mfma_ceiling(0, 0, 1)


def test_cpp_driver_through_the_launcher_templates(ck):
    # the C++ face (include/ckopt.hpp: the reference's launcher templates over the C ABI) driven by a test
    # main in the role of the reference's own: constant-matrix sweep, accuracy counts, tuple-per-line timing
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "build", "gemm_driver")
    assert os.path.exists(exe), "tests/cpp/build/gemm_driver is not built (make -C tests/cpp)"
    r = subprocess.run([exe, "all", "2048"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "PASSED" in r.stdout and "correctness:" in r.stdout and "accuracy:" in r.stdout
    lines = [l for l in r.stdout.splitlines() if l.startswith("(") and "): " in l]
    assert len(lines) >= 8 and all(float(l.split("): ")[1]) > 1.0 for l in lines)


# ---- the <half, half> role: C and D in the operands' 16-bit type, fp32 accumulation, one rounding ----------
@pytest.mark.parametrize("dt_name", ["f16", "bf16"])
def test_low_precision_output_instance(ck, oracle, dt_name):
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    odt = oracle.DT_F16 if dt_name == "f16" else oracle.DT_BF16
    is_bf = dt_name == "bf16"
    tdt = torch.bfloat16 if is_bf else torch.float16

    def run(a, bt, c16, alpha, beta, t, M, N, K):
        da, db = G.to_dev(a), G.to_dev(bt)
        dc = None if c16 is None else G.to_dev(c16)
        dd = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_lp(dt, da, db, dc, dd, alpha, beta, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                           t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                           t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                           t["num_consumer_warps"], t["num_sms"])
        assert ck.device_status() == 0
        return dd.float().cpu().numpy()

    # exact: small integers, every value representable in 16 bits (|sum| <= 4 * 48 = 192 < 256)
    M, N, K = 200, 264, 48
    a = ck.fill_int(dt, (M, K), 71, 0, -2, 2)
    bt = ck.fill_int(dt, (N, K), 71, 1, -2, 2)
    want = (G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T).astype(np.float32)
    for t in (make_tuning(ck, 128, 32, 2, 2, 4), make_tuning(ck, 256, 64, 2, 0, 8), make_tuning(ck, 64, 32, 3, 2, 8, "wave", 1, 1)):
        assert np.array_equal(run(a, bt, None, 1.0, 0.0, t, M, N, K), want), t
    # random, alpha / beta with a 16-bit C: fp32 result of the oracle, rounded once
    M, N, K = 384, 512, 1024
    a = ck.fill_uniform(dt, (M, K), 72, 0)
    bt = ck.fill_uniform(dt, (N, K), 72, 1)
    c16 = ck.fill_uniform(dt, (M, N), 72, 2)
    cf = (G.bf16_bits_to_f32(c16) if is_bf else c16.astype(np.float32))
    ref = oracle.gemm(odt, a, bt, cf, 0.75, -1.25)
    ref16 = torch.from_numpy(ref).to(tdt).float().numpy()
    for t in (make_tuning(ck, 256, 64, 2, 2, 8), make_tuning(ck, 128, 64, 3, 0, 4)):
        got = run(a, bt, c16, 0.75, -1.25, t, M, N, K)
        assert_close(oracle, ref, got)
        # one rounding of an fp32 sum that differs from the oracle's only in summation order: at most 1 ulp apart
        ulp = np.abs(ref16) * (2.0 ** -7 if is_bf else 2.0 ** -10) + 1e-3
        assert np.all(np.abs(got - ref16) <= ulp)


@pytest.mark.parametrize("tile,c", [(64, 4), (64, 8), (128, 4), (128, 8), (256, 8)])
def test_tile_sync_through_the_workgroup_barrier(ck, oracle, tile, c):
    # option 5: dedicated producers, one hardware barrier per segment instead of LDS counters
    prev = ck.set_option(ck.OPT_TILE_SYNC_BARRIER, 1)
    try:
        a = ck.fill_int(ck.DT_F16, (2 * tile, 640), 81, 0, -2, 2)
        bt = ck.fill_int(ck.DT_F16, (3 * tile, 640), 81, 1, -2, 2)
        want = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32)
        ar = ck.fill_int(ck.DT_F16, (tile + 40, 72), 81, 2, -2, 2)
        br = ck.fill_int(ck.DT_F16, (tile - 24, 72), 81, 3, -2, 2)
        wantr = (ar.astype(np.int64) @ br.astype(np.int64).T).astype(np.float32)
        n = 0
        for sk, stages, p in itertools.product((32, 64, 128), (2, 3, 4), (2, 4, 8)):
            t = make_tuning(ck, tile, sk, stages, p, c)
            if not legal(ck, t):
                continue
            assert np.array_equal(G.run_gemm(ck, ck.DT_F16, a, bt, t=t), want), t
            assert np.array_equal(G.run_gemm(ck, ck.DT_F16, ar, br, t=t), wantr), t
            n += 1
        assert n >= 4
        M, N, K = 2 * tile, 2 * tile, 1024
        a2 = ck.fill_uniform(ck.DT_BF16, (M, K), 82, 0)
        b2 = ck.fill_uniform(ck.DT_BF16, (N, K), 82, 1)
        c2 = ck.fill_uniform(ck.DT_F32, (M, N), 82, 2)
        ref = oracle.gemm(oracle.DT_BF16, a2, b2, c2, 1.5, -0.5)
        assert_close(oracle, ref, G.run_gemm(ck, ck.DT_BF16, a2, b2, c2, 1.5, -0.5, t=make_tuning(ck, tile, 32, 4, 4 if tile > 64 else 2, c)))
    finally:
        ck.set_option(ck.OPT_TILE_SYNC_BARRIER, prev)


STRAIGHT_LINE = dict(tile=256, sk=32, stages=5, p=0, c=8)


def _straight_line_tuning(ck, cus=256, group=4):
    t = make_tuning(ck, STRAIGHT_LINE["tile"], STRAIGHT_LINE["sk"], STRAIGHT_LINE["stages"], STRAIGHT_LINE["p"], STRAIGHT_LINE["c"])
    t["num_sms"] = cus
    t["tile_group_m"] = group
    return t


@pytest.mark.parametrize("M,N,K,cus,group", [
    (256, 256, 64, 256, 4),      # one tile, one loop body: prologue, one body, epilogue
    (256, 256, 192, 256, 4),     # odd number of bodies: the ring position at a tile's end varies
    (512, 768, 320, 256, 4),
    (1024, 1024, 64, 3, 4),      # many tiles per workgroup, every body follows an epilogue
    (1024, 1024, 192, 5, 4),
    (1024, 1280, 1152, 7, 3),    # group size that does not divide the tile rows
    (2048, 2048, 1024, 256, 4),
    (300, 260, 128, 256, 4),     # ragged tiles: rows past the edge read as zeros, element-wise stores
    (777, 515, 192, 3, 4),       # N not a multiple of 4: no vector stores anywhere
    (100, 50, 64, 256, 4),
    (1279, 1025, 320, 7, 3),
])
def test_straight_line_kernel_bit_exact(ck, M, N, K, cus, group):
    t = _straight_line_tuning(ck, cus, group)
    assert legal(ck, t)
    for dt in (ck.DT_F16, ck.DT_BF16):
        a = ck.fill_int(dt, (M, K), 91, 0, -2, 2)
        bt = ck.fill_int(dt, (N, K), 91, 1, -2, 2)
        want = (G.as_f64(dt == ck.DT_BF16, a) @ G.as_f64(dt == ck.DT_BF16, bt).T).astype(np.float32)
        for every_kstep in (0, 1):   # both schedules: barrier in the odd k-step only / in every k-step (default)
            prev = ck.set_option(ck.OPT_BARRIER_EVERY_KSTEP, every_kstep)
            try:
                got = G.run_gemm(ck, dt, a, bt, t=t)
            finally:
                ck.set_option(ck.OPT_BARRIER_EVERY_KSTEP, prev)
            assert np.array_equal(got, want), every_kstep


@pytest.mark.parametrize("M,N,K", [(300, 260, 200), (512, 256, 8), (256, 520, 1001), (130, 70, 4100), (257, 513, 80), (520, 300, 1112),
                                   (256, 256, 96), (700, 512, 4136), (384, 256, 112), (256, 300, 120)])
def test_straight_line_kernel_any_k(ck, M, N, K):
    # K that is not a multiple of 64: a multiple of 8 is masked in the kernel's last loop body (every remainder 8 .. 56
    # occurs below), anything else in zero-padded operand copies with whole loop bodies; either way the launch takes
    # the straight-line kernel. Exact on small integers, with and without C, every element written (D starts as NaN);
    # a chunk read past the end of K is the head of the next row and would show in the sums
    for dt in (ck.DT_F16, ck.DT_BF16):
        a = ck.fill_int(dt, (M, K), 98, 0, -2, 2)
        bt = ck.fill_int(dt, (N, K), 98, 1, -2, 2)
        c = ck.fill_int(ck.DT_F32, (M, N), 98, 2, -3, 3)
        exact = G.as_f64(dt == ck.DT_BF16, a) @ G.as_f64(dt == ck.DT_BF16, bt).T
        for cus, width in ((256, 0), (3, 0), (256, 2), (3, 2)):   # 256 x 256 tiles and 256 x 128 tiles
            t = _straight_line_tuning(ck, cus)
            prev = ck.set_option(ck.OPT_HALF_WIDTH, width)
            try:
                assert np.array_equal(G.run_gemm(ck, dt, a, bt, t=t), exact.astype(np.float32)), (M, N, K, dt, cus, width)
                assert np.array_equal(G.run_gemm(ck, dt, a, bt, c, -1.0, 2.0, t=t), (2.0 * c - exact).astype(np.float32)), (width,)
            finally:
                ck.set_option(ck.OPT_HALF_WIDTH, prev)
    order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b",
                            "tile_group_m", "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
    if K % 8:
        assert ck.gemm_workspace_bytes(M, N, K, True, *order) >= (M + N) * ((K + 63) // 64 * 64) * 2
    else:
        assert ck.gemm_workspace_bytes(M, N, K, True, *order) == 0    # K % 64 != 0 is masked inside the kernel


@pytest.mark.parametrize("N", [512, 516, 301])   # rows of D on 128-byte lines / on 16-byte boundaries only / anywhere
def test_d_store_policy_exact(ck, N):
    """Non-temporal and ordinary stores of D (the launcher chooses by the alignment of D's rows; the option forces
    either): same exact small-integer results from the straight-line kernel, a general kernel, split-K planes and the
    16-bit epilogues, whole matrix, every element written (D starts as NaN)."""
    M, K = 520, 2048
    for dt in (ck.DT_F16, ck.DT_BF16):
        is_bf = dt == ck.DT_BF16
        a = ck.fill_int(dt, (M, K), 55, 0, -1, 1)
        bt = ck.fill_int(dt, (N, K), 55, 1, -1, 1)
        c = ck.fill_int(ck.DT_F32, (M, N), 55, 2, -3, 3)
        exact = G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T
        tdt = torch.bfloat16 if is_bf else torch.float16
        for policy in (0, 1, 2):
            prev = ck.set_option(ck.OPT_D_STORE_POLICY, policy)
            try:
                for t in (_straight_line_tuning(ck), make_tuning(ck, 128, 64, 2, 2, 8), make_tuning(ck, 128, 64, 2, 0, 4)):
                    assert np.array_equal(G.run_gemm(ck, dt, a, bt, t=t), exact.astype(np.float32)), (policy, t)
                    assert np.array_equal(G.run_gemm(ck, dt, a, bt, c, -1.0, 2.0, t=t), (2.0 * c - exact).astype(np.float32)), (policy, t)
                before = ck.set_option(ck.OPT_SPLIT_K, 2)   # K = 2048: two slices of 1024 through the planes
                try:
                    assert np.array_equal(G.run_gemm(ck, dt, a, bt, t=_straight_line_tuning(ck)), exact.astype(np.float32)), policy
                finally:
                    ck.set_option(ck.OPT_SPLIT_K, before)
                # 16-bit C and D (|sums| stay far below 2048, so every result is representable)
                small = exact[:, :] * 0.0625
                for t in (_straight_line_tuning(ck), make_tuning(ck, 128, 64, 2, 2, 8)):
                    da, db = G.to_dev(a), G.to_dev(bt)
                    dd = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
                    ck.gemm_shmem_tc_async_opt_port_lp(dt, da, db, None, dd, 0.0625, 0.0, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                                       t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                                       t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                                       t["num_consumer_warps"], t["num_sms"])
                    assert ck.device_status() == 0
                    want16 = torch.from_numpy(small.astype(np.float32)).to(tdt).float().numpy()
                    assert np.array_equal(dd.float().cpu().numpy(), want16), (policy, t)
            finally:
                ck.set_option(ck.OPT_D_STORE_POLICY, prev)


@pytest.mark.parametrize("M,N,K,cus", [
    (1280, 1280, 192, 24),   # 25 tiles on 24 workgroups: 2 rounds, even rounds take 16 workgroups
    (1279, 1025, 320, 12),   # ragged, 25 tiles on 12: 3 rounds, 9 -> 12 workgroups (rounded up to whole XCDs, capped)
    (2304, 2048, 128, 40),   # 72 tiles on 40: 2 rounds of 36 -> 40
])
def test_even_rounds_grid_gives_the_same_result(ck, M, N, K, cus):
    """The persistent grid with even rounds (fewer workgroups, same number of rounds) against min(tiles, num_sms):
    exact small-integer products, both kernels' tile loops."""
    a = ck.fill_int(ck.DT_F16, (M, K), 17, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 17, 1, -2, 2)
    want = (G.as_f64(False, a) @ G.as_f64(False, bt).T).astype(np.float32)
    tunings = [_straight_line_tuning(ck, cus, 4)]
    if K % 64 == 0:
        general = make_tuning(ck, 128, 64, 2, 2, 8)   # producer/consumer kernel, 128 x 128 tiles
        general["num_sms"] = cus
        general["tile_group_m"] = 3
        tunings.append(general)
    for t in tunings:
        assert legal(ck, t)
        for even in (0, 1):
            prev = ck.set_option(ck.OPT_EVEN_ROUNDS, even)
            try:
                got = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
            finally:
                ck.set_option(ck.OPT_EVEN_ROUNDS, prev)
            assert np.array_equal(got, want), (even, t)


def test_straight_line_kernel_epilogue_and_general_kernel_agree(ck, oracle):
    # beta != 0 (the epilogue reads C: the store accounting of the waits is off), 16-bit C/D, and the
    # same launches through the general fused kernel (option 6 off) give the same bits
    M, N, K = 768, 512, 448
    t = _straight_line_tuning(ck, cus=2)
    a = ck.fill_uniform(ck.DT_F16, (M, K), 92, 0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 92, 1)
    c = ck.fill_uniform(ck.DT_F32, (M, N), 92, 2)
    got = G.run_gemm(ck, ck.DT_F16, a, bt, c, 1.5, -0.5, t=t)
    assert_close(oracle, oracle.gemm(oracle.DT_F16, a, bt, c, 1.5, -0.5), got)
    ai = ck.fill_int(ck.DT_F16, (M, K), 93, 0, -2, 2)
    bi = ck.fill_int(ck.DT_F16, (N, K), 93, 1, -2, 2)
    ci = ck.fill_int(ck.DT_F32, (M, N), 93, 2, -3, 3)
    want = 2.0 * (ai.astype(np.int64) @ bi.astype(np.int64).T) - ci.astype(np.float64)
    assert np.array_equal(G.run_gemm(ck, ck.DT_F16, ai, bi, ci, 2.0, -1.0, t=t), want.astype(np.float32))
    prev = ck.set_option(ck.OPT_STRAIGHT_LINE, 0)
    try:
        general = G.run_gemm(ck, ck.DT_F16, a, bt, c, 1.5, -0.5, t=t)
    finally:
        ck.set_option(ck.OPT_STRAIGHT_LINE, prev)
    assert_close(oracle, general, got)


@pytest.mark.parametrize("dt_name", ["f16", "bf16"])
@pytest.mark.parametrize("N", [776, 772])   # rows of D on 16-byte boundaries (16 bytes per lane and store) and not
def test_straight_line_kernel_16_bit_output(ck, oracle, dt_name, N):
    # the <half, half> role through the straight-line kernel: interior tiles take the 16-byte store path
    # (two blocks exchanged between lanes), edge tiles and unaligned rows the general one
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    odt = oracle.DT_F16 if dt_name == "f16" else oracle.DT_BF16
    is_bf = dt_name == "bf16"
    tdt = torch.bfloat16 if is_bf else torch.float16

    def run(a, bt, c16, alpha, beta, M, K, cus, schedule=1, straight_line=1):
        t = _straight_line_tuning(ck, cus=cus)
        da, db = G.to_dev(a), G.to_dev(bt)
        dc = None if c16 is None else G.to_dev(c16)
        dd = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
        prev = ck.set_option(ck.OPT_BARRIER_EVERY_KSTEP, schedule), ck.set_option(ck.OPT_STRAIGHT_LINE, straight_line)
        try:
            ck.gemm_shmem_tc_async_opt_port_lp(dt, da, db, dc, dd, alpha, beta, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                               t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                               t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                               t["num_consumer_warps"], t["num_sms"])
        finally:
            ck.set_option(ck.OPT_BARRIER_EVERY_KSTEP, prev[0])
            ck.set_option(ck.OPT_STRAIGHT_LINE, prev[1])
        assert ck.device_status() == 0
        return dd.float().cpu().numpy()

    # exact: small integers, every value representable in 16 bits (|sum| <= 4 * 64 = 256)
    M, K = 520, 64
    a = ck.fill_int(dt, (M, K), 171, 0, -2, 2)
    bt = ck.fill_int(dt, (N, K), 171, 1, -2, 2)
    want = (G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T).astype(np.float32)
    for cus in (256, 2):          # one tile per workgroup, and several (the next tile's waits count the stores)
        for schedule in (1, 0):
            assert np.array_equal(run(a, bt, None, 1.0, 0.0, M, K, cus, schedule), want), (cus, schedule)
    assert np.array_equal(run(a, bt, None, -0.5, 0.0, M, K, 3), -0.5 * want)
    # a one-hot Bt copies columns of A: position errors cannot cancel
    K = 1024
    a = ck.fill_uniform(dt, (M, K), 172, 0)
    eye = np.zeros((N, K), dtype=np.float32)
    eye[np.arange(N), (np.arange(N) * 7 + 5) % K] = 1.0
    eye = G.f32_to_bf16_bits(eye) if is_bf else eye.astype(np.float16)
    af = G.bf16_bits_to_f32(a) if is_bf else a.astype(np.float32)
    assert np.array_equal(run(a, eye, None, 1.0, 0.0, M, K, 4), af[:, (np.arange(N) * 7 + 5) % K])
    # random operands, long K, several tiles per workgroup: the same bits as the general fused kernel, with
    # and without a C operand, and the oracle's fp32 result rounded once (at most 1 ulp apart)
    bt = ck.fill_uniform(dt, (N, K), 172, 1)
    c16 = ck.fill_uniform(dt, (M, N), 172, 2)
    cf = G.bf16_bits_to_f32(c16) if is_bf else c16.astype(np.float32)
    for c, alpha, beta in ((None, 1.0, 0.0), (c16, 0.75, -1.25)):
        got = run(a, bt, c, alpha, beta, M, K, 3)
        assert np.array_equal(got, run(a, bt, c, alpha, beta, M, K, 3, straight_line=0))
        ref = oracle.gemm(odt, a, bt, None if c is None else cf, alpha, beta)
        assert_close(oracle, ref, got)
        ref16 = torch.from_numpy(ref).to(tdt).float().numpy()
        assert np.all(np.abs(got - ref16) <= np.abs(ref16) * (2.0 ** -7 if is_bf else 2.0 ** -10) + 1e-3)


def test_straight_line_kernel_headline_size_properties(ck):
    # 8192^3 in the headline configuration: constant operands have a closed form (every output
    # alpha * 10 * K), and a one-hot Bt picks columns of A exactly
    M = N = K = 8192
    t = _straight_line_tuning(ck)
    a = ck.fill_constant(ck.DT_F16, (M, K), 1.0)
    bt = ck.fill_constant(ck.DT_F16, (N, K), 10.0)
    d = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
    assert float(d.min()) == float(d.max()) == 10.0 * K
    a = ck.fill_int(ck.DT_F16, (M, K), 94, 0, -8, 8)
    eye = np.zeros((N, K), dtype=np.float16)
    eye[np.arange(N), (np.arange(N) * 5 + 3) % K] = 1.0
    d = G.run_gemm(ck, ck.DT_F16, a, eye, t=t)
    assert np.array_equal(d, a[:, (np.arange(N) * 5 + 3) % K].astype(np.float32))


@pytest.mark.parametrize("M,N,K,slices,cus,dt_name", [
    (2048, 1024, 4096, 4, 256, "f16"),
    (2048, 1024, 4096, 2, 5, "f16"),      # several items per workgroup, slices of different tiles in turn
    (2048, 1024, 8192, 8, 256, "bf16"),
    (2048, 2048, 4096, 1, 256, "f16"),    # automatic: 64 tiles on 256 CUs
    (2000, 1020, 4096, 4, 256, "f16"),    # ragged tiles
    (512, 768, 8192, 1, 256, "f16"),      # 6 tiles: fewer than one XCD round, automatic slicing (8 slices)
    (700, 300, 4096, 3, 4, "bf16"),       # 6 ragged tiles on 4 workgroups; 3 slices asked, 4096 has no 3 whole ones: 2
    (1536, 1536, 8192, 1, 256, "f16"),    # 36 tiles (neither fewer than 32 nor whole runs of 32): automatic, 4 slices
    (700, 301, 8192, 4, 256, "bf16"),     # N not a multiple of 4: rows of the planes and of D on 4-byte boundaries
    (2048, 1100, 4096, 2, 7, "f16"),      # 40 tiles, two slices, seven workgroups
])
def test_split_k_bit_exact(ck, M, N, K, slices, cus, dt_name):
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    t = _straight_line_tuning(ck, cus)
    a = ck.fill_int(dt, (M, K), 95, 0, -2, 2)
    bt = ck.fill_int(dt, (N, K), 95, 1, -2, 2)
    c = ck.fill_int(ck.DT_F32, (M, N), 95, 2, -3, 3)
    want = (2.0 * (G.as_f64(dt == ck.DT_BF16, a) @ G.as_f64(dt == ck.DT_BF16, bt).T) - c.astype(np.float64)).astype(np.float32)
    prev = ck.set_option(ck.OPT_SPLIT_K, slices)
    try:
        got = G.run_gemm(ck, dt, a, bt, c, 2.0, -1.0, t=t)
    finally:
        ck.set_option(ck.OPT_SPLIT_K, prev)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("M,N,K,cus,opts", [
    (2048, 4096, 4096, 256, dict(split_k=2)),            # 128 tiles, two slices: every workgroup one item
    (512, 512, 8192, 256, dict(split_k=4)),              # 4 tiles x 4 slices
    (700, 520, 6144, 256, dict(split_k=3)),              # ragged tiles, three slices
    (512, 768, 16384, 256, dict(split_k=16)),            # 6 tiles x 16 slices
    (1024, 1280, 8192, 16, dict()),                      # the partly filled last round: 16 whole tiles + 4 sliced, one launch
    (2048, 1280, 8192, 16, dict()),                      # two full rounds + 8 sliced tiles
    (1000, 640, 8192, 8, dict(half_width=2)),            # 256 x 128 tiles: 4 x 5 on 8 workgroups, ragged in M
    (1400, 1200, 4096, 8, dict(tail_round=0)),
    (512, 768, 8192, 6, dict(split_k=4)),                # 6 tiles x 4 slices on 6 workgroups: four sliced items each, one after the other
    (512, 500, 6144, 6, dict(split_k=3, half_width=3)),  # 256 x 192 tiles: 2 x 3 tiles x 3 slices on 6 workgroups, ragged in N
])
def test_slices_reduced_in_the_kernel_exact(ck, M, N, K, cus, opts):
    """K slices added inside the straight-line kernel (no second kernel; of a wave tile's slices the wave that arrives last
    adds them all, in slice order, and writes D): fp32 and 16-bit output, with and without C, exact on small integers, any
    number of sliced items per workgroup."""
    t = _straight_line_tuning(ck, cus)
    tup = tuple(t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                               "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms"))
    a = ck.fill_int(ck.DT_F16, (M, K), 97, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 97, 1, -2, 2)
    c = ck.fill_int(ck.DT_F32, (M, N), 97, 2, -3, 3)
    prod = (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float64)
    da, db, dc = G.to_dev(a), G.to_dev(bt), G.to_dev(c)
    dc16 = G.to_dev(c.astype(np.float16))
    # fused_reduction 2: in the kernel wherever that is possible, whatever the cost model says; 256 x 256 tiles unless the case says otherwise
    o = ck.launch_options(fused_reduction=2, **dict(dict(half_width=0), **opts))
    plan = ck.gemm_launch_plan(M, N, K, True, *tup, options=o)
    if opts.get("tail_round", 1):
        assert plan["sliced_tiles"] > 0 and plan["reduced_in_kernel"], plan
    for rep_ in range(2):   # twice: the counters are cleared by every launch
        d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, da, db, dc, d, 2.0, -1.0, M, N, K, *tup, options=o)
        assert ck.device_status() == 0
        assert np.array_equal(d.cpu().numpy(), (2.0 * prod - c).astype(np.float32)), plan
    h = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F16, da, db, dc16, h, 1.0, 1.0, M, N, K, *tup, options=o)
    assert ck.device_status() == 0
    assert np.array_equal(h.cpu().numpy(), (prod + c).astype(np.float16)), plan
    # on a caller-owned workspace of exactly the size the query gives, poisoned
    need = ck.gemm_workspace_bytes(M, N, K, True, *tup, options=o)
    ws = torch.full((max(need, 1),), 0xA5, dtype=torch.uint8, device="cuda")
    d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, da, db, None, d, 1.0, 0.0, M, N, K, *tup, options=o, workspace=ws if need else None,
                                       workspace_bytes=need)
    assert ck.device_status() == 0 and np.array_equal(d.cpu().numpy(), prod.astype(np.float32))
    if need > 256:
        with pytest.raises(ck.CkoptError) as e:
            ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, da, db, None, d, 1.0, 0.0, M, N, K, *tup, options=o, workspace=ws,
                                               workspace_bytes=need - 257)
        assert e.value.code == ck.ERR_TOO_LARGE


@pytest.mark.parametrize("M,N,K,slices", [(2048, 4096, 4096, 2), (2048, 2048, 8192, 4), (1024, 768, 6144, 3)])
def test_slices_reduced_in_the_kernel_against_the_second_pass(ck, oracle, M, N, K, slices):
    """Random fp16 data: both forms of the reduction add the slices of an element in slice order - in the kernel
    whichever wave arrives last - so they agree bit for bit, run after run; and both are within tolerance of the oracle."""
    t = _straight_line_tuning(ck, 256)
    tup = tuple(t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                               "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms"))
    a = ck.fill_uniform(ck.DT_F16, (M, K), 99, 0, -1.0, 1.0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 99, 1, -1.0, 1.0)
    da, db = G.to_dev(a), G.to_dev(bt)
    out = []
    for fused in (2, 0, 2):
        o = ck.launch_options(split_k=slices, fused_reduction=fused, half_width=0)
        plan = ck.gemm_launch_plan(M, N, K, True, *tup, options=o)
        assert plan["reduced_in_kernel"] == bool(fused) and plan["k_slices"] == slices, plan
        d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, da, db, None, d, 1.0, 0.0, M, N, K, *tup, options=o)
        assert ck.device_status() == 0
        out.append(d.cpu().numpy())
    assert np.array_equal(out[0], out[1]) and np.array_equal(out[0], out[2])
    ref = oracle.gemm(oracle.DT_F16, a, bt, rows=(0, 256))
    assert_close(oracle, ref, out[0][:256])


def test_two_streams_reduce_in_the_kernel_at_once(ck):
    """Launches that add their K slices inside the kernel, issued on two streams at the same time: each needs the whole
    device (256 work items), so their workgroups compete for the CUs and neither launch is resident as a whole. No wave
    waits for another in that reduction, so both finish and both are exact."""
    M, N, K = 2048, 2048, 8192
    t = _straight_line_tuning(ck, 256)
    tup = tuple(t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                               "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms"))
    o = ck.launch_options(split_k=4, fused_reduction=2, half_width=0)
    assert ck.gemm_launch_plan(M, N, K, True, *tup, options=o)["reduced_in_kernel"]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ops, wants, outs = [], [], []
    for i in range(2):
        a = ck.fill_int(ck.DT_F16, (M, K), 300 + i, 0, -2, 2)
        bt = ck.fill_int(ck.DT_F16, (N, K), 300 + i, 1, -2, 2)
        wants.append((a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32))
        ops.append((G.to_dev(a), G.to_dev(bt)))
        outs.append(torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda"))
    torch.cuda.synchronize()
    for rep_ in range(6):
        for i in range(2):
            ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, ops[i][0], ops[i][1], None, outs[i], 1.0, 0.0, M, N, K, *tup, options=o,
                                               stream=streams[i])
    torch.cuda.synchronize()
    assert ck.device_status() == 0
    for i in range(2):
        assert np.array_equal(outs[i].cpu().numpy(), wants[i]), i


def test_two_host_threads_with_different_options(ck):
    """Launch options are an argument of the _ex entry points (in the reference every knob is a launcher parameter,
    port_2.cu:1088-1109): two host threads launch at the same time on their own streams with different options - one cuts
    K and reduces in the kernel on 256 x 128 tiles, the other runs whole 256 x 256 tiles - and both get exact results,
    whatever the process-wide switches are set to meanwhile."""
    import threading
    M, N, K = 1024, 1024, 4096
    t = _straight_line_tuning(ck, 256)
    tup = tuple(t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                               "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms"))
    da, db, want = _exact_case(ck, M, N, K, 101)
    variants = [ck.launch_options(split_k=4, half_width=2, fused_reduction=2), ck.launch_options(split_k=0, half_width=0)]
    plans = [ck.gemm_launch_plan(M, N, K, True, *tup, options=o) for o in variants]
    assert plans[0]["k_slices"] == 4 and plans[0]["tile_cols"] == 128 and plans[1]["k_slices"] == 1 and plans[1]["tile_cols"] == 256
    errors = []

    def worker(i):
        try:
            torch.cuda.set_device(0)
            stream = torch.cuda.Stream()
            d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            for _ in range(40):
                with torch.cuda.stream(stream):
                    d.fill_(float("nan"))
                ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, da, db, None, d, 1.0, 0.0, M, N, K, *tup, options=variants[i], stream=stream)
                stream.synchronize()
                if not np.array_equal(d.cpu().numpy(), want):
                    errors.append("thread %d: wrong result" % i)
                    return
        except Exception as e:   # noqa: BLE001 - reported to the main thread
            errors.append("thread %d: %r" % (i, e))

    def flipper(stop):
        while not stop.is_set():
            for key in (ck.OPT_SPLIT_K, ck.OPT_HALF_WIDTH):
                prev = ck.set_option(key, 0)
                ck.set_option(key, prev)

    stop = threading.Event()
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)] + [threading.Thread(target=flipper, args=(stop,))]
    for th in threads:
        th.start()
    for th in threads[:2]:
        th.join()
    stop.set()
    threads[2].join()
    assert not errors, errors
    assert ck.device_status() == 0


@pytest.mark.parametrize("M,N,K,cus,opts,dt_name,out16,beta", [
    (256, 192, 64, 256, {}, "f16", False, 0.0),                      # one tile, one loop body
    (512, 768, 1024, 256, {}, "f16", False, 1.0),
    (700, 500, 1000, 256, {}, "f16", False, 0.0),                    # ragged in M and N, K % 64 != 0: the instance that masks the end of K
    (700, 500, 1001, 256, {}, "bf16", False, 0.0),                   # K % 8 != 0: zero-padded copies
    (1024, 1920, 512, 8, {}, "f16", False, 0.0),                     # 40 tiles on 8 workgroups
    (1024, 1920, 512, 8, dict(barrier_every_kstep=0), "f16", False, -1.0),
    (700, 500, 1000, 256, dict(barrier_every_kstep=0), "bf16", False, 0.0),
    (512, 776, 256, 256, {}, "f16", True, 0.0),                      # 16-bit C / D: block by block (no groups of four block columns)
    (512, 776, 256, 256, {}, "f16", True, 1.0),
    (512, 772, 256, 256, {}, "bf16", True, -1.0),
    (512, 768, 8192, 256, dict(split_k=4, fused_reduction=0), "f16", False, 0.0),     # K slices, second pass
    (512, 768, 8192, 256, dict(split_k=4, fused_reduction=2), "f16", False, 1.0),     # K slices, added in the kernel
    (512, 768, 6144, 256, dict(split_k=3, fused_reduction=2), "f16", True, 1.0),
    (1024, 1920, 8192, 16, dict(fused_reduction=2), "f16", False, 0.0),               # partly filled last round at this width
])
def test_three_quarter_width_tiles_exact(ck, M, N, K, cus, opts, dt_name, out16, beta):
    """256 x 192 tiles of the straight-line kernel (wave tiles of 64 x 96), forced: half of the waves issue a load pair that
    fetches nothing, the 16-bit epilogue goes block by block; every path exact on small integers, every element written."""
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    t = _straight_line_tuning(ck, cus)
    tup = tuple(t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                               "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms"))
    o = ck.launch_options(half_width=3, **opts)
    plan = ck.gemm_launch_plan(M, N, K, K % 8 == 0, *tup, options=o)
    assert plan["tile_cols"] == 192, plan
    a = ck.fill_int(dt, (M, K), 103, 0, -2, 2)
    bt = ck.fill_int(dt, (N, K), 103, 1, -2, 2)
    c = ck.fill_int(ck.DT_F32, (M, N), 103, 2, -3, 3)
    prod = G.as_f64(dt == ck.DT_BF16, a) @ G.as_f64(dt == ck.DT_BF16, bt).T
    da, db = G.to_dev(a), G.to_dev(bt)
    if out16:
        tdt = torch.float16 if dt == ck.DT_F16 else torch.bfloat16
        dc = torch.from_numpy(c).to(tdt).cuda() if beta else None
        d = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_ex(dt, dt, da, db, dc, d, 1.0, beta, M, N, K, *tup, options=o)
        got = d.float().cpu().numpy()
        want = torch.from_numpy(prod + beta * c).to(tdt).float().numpy()
    else:
        dc = G.to_dev(c) if beta else None
        d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        ck.gemm_shmem_tc_async_opt_port_ex(dt, ck.DT_F32, da, db, dc, d, 1.0, beta, M, N, K, *tup, options=o)
        got = d.cpu().numpy()
        want = (prod + beta * c).astype(np.float32)
    assert ck.device_status() == 0
    assert np.array_equal(got, want), plan


def test_three_quarter_width_tiles_chosen_and_within_tolerance(ck, oracle):
    """3072^3 (144 tiles of 256 x 256: 0.56 of a round): the launcher takes 192 tiles of 256 x 192; random fp16 data against the
    oracle over sampled rows of every tile row."""
    M = N = K = 3072
    t = suggested_tuning(ck, M, N, K)
    order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                            "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
    assert ck.gemm_launch_plan(M, N, K, True, *order)["tile_cols"] == 192
    a = ck.fill_uniform(ck.DT_F16, (M, K), 105, 0, -1.0, 1.0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 105, 1, -1.0, 1.0)
    got = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
    assert not np.isnan(got).any()
    for r0 in list(range(0, M, 256)) + [M - 4]:
        ref = oracle.gemm(oracle.DT_F16, a, bt, rows=(r0, r0 + 4))
        assert_close(oracle, ref, got[r0:r0 + 4])


@pytest.mark.parametrize("M,N,K", [(512, 512, 256), (700, 390, 1024), (1024, 768, 4096), (260, 1000, 200)])
def test_half_width_tiles_exact(ck, M, N, K):
    """256 x 128 tiles of the straight-line kernel, forced: fp32 and 16-bit C / D (whole-line and element-wise epilogues),
    with and without C, K slices, few and many workgroups; exact on small integers, every element written."""
    prev = ck.set_option(ck.OPT_HALF_WIDTH, 2)
    try:
        for dt in (ck.DT_F16, ck.DT_BF16):
            is_bf = dt == ck.DT_BF16
            tdt = torch.bfloat16 if is_bf else torch.float16
            a = ck.fill_int(dt, (M, K), 61, 0, -1, 1)
            bt = ck.fill_int(dt, (N, K), 61, 1, -1, 1)
            c = ck.fill_int(ck.DT_F32, (M, N), 61, 2, -3, 3)
            exact = G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T
            for cus in (256, 6):
                t = _straight_line_tuning(ck, cus)
                for split in (0, 1, 2):
                    before = ck.set_option(ck.OPT_SPLIT_K, split)
                    try:
                        assert np.array_equal(G.run_gemm(ck, dt, a, bt, t=t), exact.astype(np.float32)), (dt, cus, split)
                        assert np.array_equal(G.run_gemm(ck, dt, a, bt, c, 0.5, -2.0, t=t), (0.5 * exact - 2.0 * c).astype(np.float32)), (dt, cus, split)
                        da, db = G.to_dev(a), G.to_dev(bt)
                        dd = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
                        ck.gemm_shmem_tc_async_opt_port_lp(dt, da, db, None, dd, 0.0625, 0.0, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                                           t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                                           t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                                           t["num_consumer_warps"], t["num_sms"])
                        assert ck.device_status() == 0
                        want16 = torch.from_numpy((exact * 0.0625).astype(np.float32)).to(tdt).float().numpy()
                        assert np.array_equal(dd.float().cpu().numpy(), want16), (dt, cus, split)
                    finally:
                        ck.set_option(ck.OPT_SPLIT_K, before)
    finally:
        ck.set_option(ck.OPT_HALF_WIDTH, prev)


@pytest.mark.parametrize("M,N,K", [(512, 512, 128), (700, 520, 128), (256, 1024, 192)])
def test_straight_line_16_bit_output_with_c(ck, M, N, K):
    """16-bit C and D with beta != 0 on the straight-line kernel: interior tiles read C in the accumulators' layout and
    store whole lines, edge tiles go element by element; both tile widths; exact (every value is a small integer)."""
    for dt in (ck.DT_F16, ck.DT_BF16):
        is_bf = dt == ck.DT_BF16
        tdt = torch.bfloat16 if is_bf else torch.float16
        a = ck.fill_int(dt, (M, K), 63, 0, -1, 1)
        bt = ck.fill_int(dt, (N, K), 63, 1, -1, 1)
        c = ck.fill_int(ck.DT_F32, (M, N), 63, 2, -3, 3)
        want = (G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T - 2.0 * c).astype(np.float32)   # |.| <= 192 + 6: exact in 16 bits
        dc = torch.from_numpy(c).to(tdt).cuda()
        da, db = G.to_dev(a), G.to_dev(bt)
        for width in (0, 2):
            prev = ck.set_option(ck.OPT_HALF_WIDTH, width)
            try:
                for cus in (256, 3):
                    t = _straight_line_tuning(ck, cus)
                    dd = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
                    ck.gemm_shmem_tc_async_opt_port_lp(dt, da, db, dc, dd, 1.0, -2.0, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                                       t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                                       t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                                       t["num_consumer_warps"], t["num_sms"])
                    assert ck.device_status() == 0
                    assert np.array_equal(dd.float().cpu().numpy(), want), (dt, width, cus)
            finally:
                ck.set_option(ck.OPT_HALF_WIDTH, prev)


def test_half_width_tiles_chosen_for_100_tiles_full_size(ck, oracle):
    # 2560^3: 100 tiles of 256 x 256 on 256 CUs; the launcher takes 256 x 128 tiles by itself. Whole matrix against the oracle.
    M = N = K = 2560
    full_size_check(ck, oracle, ck.DT_F16, oracle.DT_F16, M, N, K, (_straight_line_tuning(ck),), lambda s, shape: ck.fill_uniform(ck.DT_F16, shape, 0xC0FFEE09, s))


def test_automatic_split_k_of_128_tiles_exact(ck):
    # 128 tiles on 256 CUs with a deep K: with 256 x 256 tiles only, the automatic rule cuts K in two (256 work items);
    # with both widths it takes 256 tiles of 256 x 128 and no slices. Exact on small integers either way.
    M, N, K = 2048, 4096, 8192
    t = _straight_line_tuning(ck)
    order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b",
                            "tile_group_m", "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
    a = ck.fill_int(ck.DT_F16, (M, K), 97, 0, -1, 1)
    bt = ck.fill_int(ck.DT_F16, (N, K), 97, 1, -1, 1)
    want = (a.astype(np.float32) @ bt.astype(np.float32).T)   # sums of at most 8192 terms of -1, 0, 1: exact in fp32
    for width, planes in ((0, 2), (1, 0)):
        prev = ck.set_option(ck.OPT_HALF_WIDTH, width)
        try:
            # (the two slices are added by the second pass: two planes of M x N fp32)
            assert ck.gemm_workspace_bytes(M, N, K, True, *order) == (planes * M * N * 4 + 256 if planes else 0)
            assert ck.gemm_launch_plan(M, N, K, True, *order)["k_slices"] == (planes if planes else 1)
            assert np.array_equal(G.run_gemm(ck, ck.DT_F16, a, bt, t=t), want), width
        finally:
            ck.set_option(ck.OPT_HALF_WIDTH, prev)


def test_split_k_against_the_oracle_and_the_single_pass(ck, oracle):
    # uniform data: the sliced sum differs from the single pass in rounding only
    M, N, K = 2048, 1024, 4096
    t = _straight_line_tuning(ck)
    a = ck.fill_uniform(ck.DT_F16, (M, K), 96, 0)
    bt = ck.fill_uniform(ck.DT_F16, (N, K), 96, 1)
    ref = oracle.gemm(oracle.DT_F16, a, bt, None, 1.0, 0.0)
    out = {}
    for slices in (0, 4):
        prev = ck.set_option(ck.OPT_SPLIT_K, slices)
        try:
            out[slices] = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
        finally:
            ck.set_option(ck.OPT_SPLIT_K, prev)
        assert_close(oracle, ref, out[slices])
    assert_close(oracle, out[0], out[4], rtol=1e-4)


def test_straight_line_kernel_random_shapes(ck):
    # seeded sweep over shapes, grid sizes, tile orders, schedules, epilogue forms and split-K: exact on
    # small integers whatever the summation order (D starts out as NaN: every element must be written).
    rng = np.random.default_rng(20240607)
    for case in range(24):
        M = int(rng.integers(1, 1100))
        N = int(rng.integers(1, 1100))
        K = 64 * int(rng.integers(1, 20))
        if case % 6 == 5:  # a shape split-K accepts: a multiple of 32 whole-or-ragged tiles, deep K
            M, N, K = 2048 - int(rng.integers(0, 200)), 1024 - int(rng.integers(0, 50)) * 4, 1024 * int(rng.integers(2, 5))
        cus = int(rng.choice([1, 2, 3, 5, 8, 64, 256]))
        group = int(rng.integers(1, 7))
        dt = ck.DT_F16 if case % 2 == 0 else ck.DT_BF16
        beta = float(rng.choice([0.0, 0.0, -1.0, 2.0]))
        every_kstep = int(rng.integers(0, 2))
        slices = int(rng.choice([0, 1, 2, 4]))
        t = _straight_line_tuning(ck, cus, group)
        a = ck.fill_int(dt, (M, K), 97 + case, 0, -2, 2)
        bt = ck.fill_int(dt, (N, K), 97 + case, 1, -2, 2)
        c = ck.fill_int(ck.DT_F32, (M, N), 97 + case, 2, -3, 3) if beta else None
        want = 2.0 * (G.as_f64(dt == ck.DT_BF16, a) @ G.as_f64(dt == ck.DT_BF16, bt).T)
        if beta:
            want = want + beta * c.astype(np.float64)
        prev = (ck.set_option(ck.OPT_BARRIER_EVERY_KSTEP, every_kstep), ck.set_option(ck.OPT_SPLIT_K, slices))
        try:
            got = G.run_gemm(ck, dt, a, bt, c, 2.0, beta, t=t)
        finally:
            ck.set_option(ck.OPT_BARRIER_EVERY_KSTEP, prev[0])
            ck.set_option(ck.OPT_SPLIT_K, prev[1])
        assert np.array_equal(got, want.astype(np.float32)), (case, M, N, K, cus, group, dt, beta, every_kstep, slices)


# ---- split-K through every form of the reduction pass -----------------------------------------------------
@pytest.mark.parametrize("dt_name", ["f16", "bf16"])
@pytest.mark.parametrize("policy", [1, 4])          # automatic (8 slices for this shape) and four slices asked for
@pytest.mark.parametrize("with_c", [False, True])
def test_split_k_16_bit_output(ck, oracle, dt_name, policy, with_c):
    # the <half, half> role on a shape that the straight-line kernel cuts along K: 4 tiles, K = 8192
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    odt = oracle.DT_F16 if dt_name == "f16" else oracle.DT_BF16
    is_bf = dt_name == "bf16"
    tdt = torch.bfloat16 if is_bf else torch.float16
    M, N, K = 512, 512, 8192
    t = _straight_line_tuning(ck)
    alpha, beta = (2.0, -1.0) if with_c else (1.0, 0.0)

    def to16(x32):
        return torch.from_numpy(np.ascontiguousarray(x32, dtype=np.float32)).to(tdt)

    def run(a, bt, c16, split):
        da, db = G.to_dev(a), G.to_dev(bt)
        dc = None if c16 is None else c16.cuda()
        dd = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
        prev = ck.set_option(ck.OPT_SPLIT_K, split)
        try:
            ck.gemm_shmem_tc_async_opt_port_lp(dt, da, db, dc, dd, alpha, beta, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                               t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                               t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                               t["num_consumer_warps"], t["num_sms"])
        finally:
            ck.set_option(ck.OPT_SPLIT_K, prev)
        assert ck.device_status() == 0
        return dd.cpu()

    # small integers: every partial sum is exact in fp32, so slices and single pass round the same number once
    a = ck.fill_int(dt, (M, K), 181, 0, -2, 2)
    bt = ck.fill_int(dt, (N, K), 181, 1, -2, 2)
    c16 = to16(ck.fill_int(ck.DT_F32, (M, N), 181, 2, -3, 3)) if with_c else None
    exact = alpha * (G.as_f64(is_bf, a) @ G.as_f64(is_bf, bt).T)
    if with_c:
        exact = exact + beta * c16.double().numpy()
    want = to16(exact)   # |exact| < 2^24: the float32 step is exact, one rounding to 16 bits
    got = run(a, bt, c16, policy)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.equal(got.view(torch.int16), run(a, bt, c16, 0).view(torch.int16))
    # uniform data: the oracle's fp32 result rounded once, at most 1 ulp apart
    a = ck.fill_uniform(dt, (M, K), 182, 0)
    bt = ck.fill_uniform(dt, (N, K), 182, 1)
    c16 = to16(ck.fill_uniform(ck.DT_F32, (M, N), 182, 2)) if with_c else None
    got = run(a, bt, c16, policy).float().numpy()
    ref = oracle.gemm(odt, a, bt, None if c16 is None else c16.float().numpy(), alpha, beta)
    assert_close(oracle, ref, got)
    ref16 = to16(ref).float().numpy()
    assert np.all(np.abs(got - ref16) <= np.abs(ref16) * (2.0 ** -7 if is_bf else 2.0 ** -10) + 1e-3)


@pytest.mark.parametrize("with_c", [False, True])
def test_split_k_fp32_output_off_a_16_byte_boundary(ck, with_c):
    # D (and C) four bytes into their allocations: the reduction pass takes its one-element-per-thread form
    M, N, K = 512, 768, 8192
    t = _straight_line_tuning(ck)
    a = ck.fill_int(ck.DT_F16, (M, K), 183, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 183, 1, -2, 2)
    c = ck.fill_int(ck.DT_F32, (M, N), 183, 2, -3, 3)
    alpha, beta = (2.0, -1.0) if with_c else (1.0, 0.0)
    want = alpha * (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float64)
    if with_c:
        want = want + beta * c
    da, db = G.to_dev(a), G.to_dev(bt)
    dbuf = torch.full((M * N + 8,), float("nan"), dtype=torch.float32, device="cuda")
    cbuf = torch.zeros((M * N + 8,), dtype=torch.float32, device="cuda")
    cbuf[1:1 + M * N] = torch.from_numpy(c.reshape(-1)).cuda()
    for policy in (1, 4):
        dbuf.fill_(float("nan"))
        prev = ck.set_option(ck.OPT_SPLIT_K, policy)
        try:
            ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da, db, cbuf.data_ptr() + 4 if with_c else None, dbuf.data_ptr() + 4, alpha, beta,
                                            M, N, K, t["tile_dim"], t["segment_dim_k"], 0, 0, t["bar_step_rows_a"], t["bar_step_rows_b"],
                                            t["tile_group_m"], t["num_stages"], t["num_producer_warps"], t["num_consumer_warps"],
                                            t["num_sms"])
        finally:
            ck.set_option(ck.OPT_SPLIT_K, prev)
        assert ck.device_status() == 0
        h = dbuf.cpu().numpy()
        assert np.isnan(h[0]) and np.isnan(h[1 + M * N:]).all()          # nothing outside D is touched
        assert np.array_equal(h[1:1 + M * N].reshape(M, N), want.astype(np.float32))


# ---- 16384^3: the size the reference's own performance driver times (port_2.cu:1554-1556) -----------------------
def test_16384_cubed_exact(ck):
    M = N = K = 16384
    t = suggested_tuning(ck, M, N, K)
    # a one-hot Bt copies columns of A: every tile offset, every row and column position
    a = ck.fill_int(ck.DT_F16, (M, K), 191, 0, -8, 8)
    cols = (np.arange(N, dtype=np.int64) * 5 + 3) % K
    eye = np.zeros((N, K), dtype=np.float16)
    eye[np.arange(N), cols] = 1.0
    d = G.run_gemm(ck, ck.DT_F16, a, eye, t=t)
    assert np.array_equal(d, a[:, cols].astype(np.float32))
    del eye
    # small integers summed over the whole K: row and column sums of the exact product, and single rows
    bt = ck.fill_int(ck.DT_F16, (N, K), 191, 1, -1, 1)
    ai, bi = a.astype(np.int64), bt.astype(np.int64)      # |sum| <= 8 * 16384 < 2^24: exact in fp32
    d = G.run_gemm(ck, ck.DT_F16, a, bt, t=t)
    assert np.array_equal(d.astype(np.int64).sum(axis=1), ai @ bi.sum(axis=0))
    assert np.array_equal(d.astype(np.int64).sum(axis=0), bi @ ai.sum(axis=0))
    for r in (0, 8191, 16383):
        assert np.array_equal(d[r], (ai[r] @ bi.T).astype(np.float32))


def test_16384_cubed_alpha_beta_one_exact(ck):
    """The reference driver's own performance case: 16384^3 with alpha = beta = 1 and a C tile read in the epilogue
    (port_2.cu:1559-1564), on small integers: every element exact."""
    M = N = K = 16384
    t = suggested_tuning(ck, M, N, K)
    a = ck.fill_int(ck.DT_F16, (M, K), 193, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 193, 1, -1, 1)
    c = ck.fill_int(ck.DT_F32, (M, N), 193, 2, -100, 100)
    d = G.run_gemm(ck, ck.DT_F16, a, bt, c, 1.0, 1.0, t=t)
    d -= c                                                  # exact: all values are small integers
    ai, bi = a.astype(np.int64), bt.astype(np.int64)
    assert np.array_equal(d.astype(np.int64).sum(axis=1), ai @ bi.sum(axis=0))
    assert np.array_equal(d.astype(np.int64).sum(axis=0), bi @ ai.sum(axis=0))
    for r in (0, 255, 256, 8191, 16383):
        assert np.array_equal(d[r], (ai[r] @ bi.T).astype(np.float32))


# ---- caller-owned workspace: the launcher allocates nothing -------------------------------------------------
@pytest.mark.parametrize("name,dt_name,M,N,K", [
    ("config 4", "f16", 2048, 2048, 32768),             # split-K planes: 4 x 16 MiB
    ("config 5", "bf16", 6143, 4097, 3071),             # zero-padded operand copies: 60 MiB
    ("copies and planes", "f16", 300, 520, 4090),       # both
    ("16-bit C and D", "bf16", 512, 512, 8192),         # the <half, half> role through split-K
])
def test_workspace_entry_matches_the_allocating_launcher(ck, name, dt_name, M, N, K):
    dt = ck.DT_F16 if dt_name == "f16" else ck.DT_BF16
    lp = name == "16-bit C and D"
    t = suggested_tuning(ck, M, N, K)
    order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b",
                            "tile_group_m", "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
    a = ck.fill_uniform(dt, (M, K), 201, 0)
    bt = ck.fill_uniform(dt, (N, K), 201, 1)
    da, db = G.to_dev(a), G.to_dev(bt)
    tdt = torch.float32 if not lp else (torch.bfloat16 if dt == ck.DT_BF16 else torch.float16)
    want = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    (ck.gemm_shmem_tc_async_opt_port_lp if lp else ck.gemm_shmem_tc_async_opt_port)(dt, da, db, None, want, 1.0, 0.0, M, N, K, *order)
    assert ck.device_status() == 0
    need = ck.gemm_workspace_bytes(M, N, K, True, *order)
    assert need > 0, "this launch is expected to need scratch memory"
    ws = torch.empty(need + 64, dtype=torch.uint8, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=tdt, device="cuda")
    cd = dt if lp else ck.DT_F32
    ck.gemm_shmem_tc_async_opt_port_ws(dt, cd, da, db, None, got, 1.0, 0.0, M, N, K, *order, ws.data_ptr() + 48, need)   # any alignment
    assert ck.device_status() == 0
    assert torch.equal(got.view(torch.int16 if lp else torch.int32), want.view(torch.int16 if lp else torch.int32))
    # one byte short, or no workspace at all: an error before anything is written
    for wptr, wbytes in ((ws.data_ptr() + 48, need - 257), (None, 0)):
        got.fill_(7.0)
        with pytest.raises(ck.CkoptError) as e:
            ck.gemm_shmem_tc_async_opt_port_ws(dt, cd, da, db, None, got, 1.0, 0.0, M, N, K, *order, wptr, wbytes)
        assert e.value.code == ck.ERR_TOO_LARGE
        torch.cuda.synchronize()
        assert float(got.float().min()) == float(got.float().max()) == 7.0


def test_workspace_query_and_launches_that_need_none(ck):
    # aligned operands, K a multiple of 8, enough tiles: no scratch, a NULL workspace is fine
    M, N, K = 1024, 1024, 512
    t = suggested_tuning(ck, M, N, K)
    order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b",
                            "tile_group_m", "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
    assert ck.gemm_workspace_bytes(M, N, K, True, *order) == 0
    assert ck.gemm_workspace_bytes(M, N, K, False, *order) >= (M + N) * K * 2      # unaligned operands are copied
    assert ck.gemm_workspace_bytes(M, N, K - 3, True, *order) >= (M + N) * ((K - 3 + 7) // 8 * 8) * 2
    a = ck.fill_int(ck.DT_F16, (M, K), 202, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 202, 1, -2, 2)
    d = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    ck.gemm_shmem_tc_async_opt_port_ws(ck.DT_F16, ck.DT_F32, G.to_dev(a), G.to_dev(bt), None, d, 1.0, 0.0, M, N, K, *order, None, 0)
    assert ck.device_status() == 0
    assert np.array_equal(d.cpu().numpy(), (a.astype(np.int64) @ bt.astype(np.int64).T).astype(np.float32))
    with pytest.raises(ck.CkoptError):
        ck.gemm_workspace_bytes(M, N, K, True, 100, *order[1:])


def test_random_tunings_entry_points_and_options_exact(ck):
    # seeded sweep over every kernel design, synchronisation granularity, grid size, the process-wide options and the
    # three homes of the scratch memory (stream-ordered allocation, caller's workspace, the library's static array):
    # exact on small integers whatever the summation order; D starts out as NaN, so every element must be written.
    # CKOPT_SWEEP_SEED / CKOPT_SWEEP_CASES run the same sweep from another seed or for longer.
    seed, cases = int(os.environ.get("CKOPT_SWEEP_SEED", "20251126")), int(os.environ.get("CKOPT_SWEEP_CASES", "260"))
    rng = np.random.default_rng(seed)
    ran = 0
    for case in range(cases):
        if rng.random() < 0.35:
            t = G.tuning(tile_dim=256, segment_dim_k=32, num_stages=5, num_producer_warps=0, num_consumer_warps=8,
                         tile_group_m=int(rng.integers(1, 7)), num_sms=int(rng.choice([1, 3, 8, 40, 256])))
        else:
            tile = int(rng.choice([64, 128, 256]))
            cw = 8 if tile == 256 else int(rng.choice([4, 8]))
            p = int(rng.choice([0, 0, 2, 4, 8]))
            t = G.tuning(tile_dim=tile, segment_dim_k=int(rng.choice([32, 64, 128])), num_stages=int(rng.integers(1, 6)),
                         num_producer_warps=p, num_consumer_warps=cw, tile_group_m=int(rng.integers(1, 7)),
                         num_sms=int(rng.choice([1, 3, 8, 40, 256])))
            mode = "tile" if p == 0 else str(rng.choice(["tile", "wave", "acc"]))
            wtr = ck.get_warp_tile_rows(tile, cw)
            wtc = ck.get_num_acc(tile, cw) // wtr
            if mode == "wave":
                t["bar_step_rows_a"], t["bar_step_rows_b"] = wtr * 16, wtc * 16
                t["bar_steps_a"], t["bar_steps_b"] = int(rng.integers(0, cw // 2 + 1)), int(rng.integers(0, 3))
            elif mode == "acc":
                t["bar_step_rows_a"] = t["bar_step_rows_b"] = 16
                t["bar_steps_a"], t["bar_steps_b"] = int(rng.integers(0, wtr)), int(rng.integers(0, wtc))
        order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b",
                                "tile_group_m", "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
        M, N = int(rng.integers(1, 700)), int(rng.integers(1, 700))
        K = int(rng.choice([int(rng.integers(1, 1500)), 8 * int(rng.integers(1, 200)), 64 * int(rng.integers(1, 40)), 1024 * int(rng.integers(1, 7))]))
        dt = ck.DT_F16 if rng.random() < 0.5 else ck.DT_BF16
        alpha, beta = float(rng.choice([1.0, 2.0, -0.5])), float(rng.choice([0.0, 0.0, -1.0, 2.0]))
        opts = {ck.OPT_SPLIT_K: int(rng.choice([0, 1, 1, 2, 3, 4, 8])), ck.OPT_BARRIER_EVERY_KSTEP: int(rng.integers(0, 2)),
                ck.OPT_EVEN_ROUNDS: int(rng.integers(0, 2)), ck.OPT_TILE_SYNC_BARRIER: int(rng.integers(0, 2)),
                ck.OPT_HALF_WIDTH: int(rng.integers(0, 4)), ck.OPT_D_STORE_POLICY: int(rng.integers(0, 3)),
                ck.OPT_FUSED_REDUCTION: int(rng.integers(0, 3)), ck.OPT_TAIL_ROUND: int(rng.integers(0, 2))}
        entry = int(rng.integers(0, 3))
        if ck.check_gemm_tuning(*order) != ck.OK:
            continue
        a = ck.fill_int(dt, (M, K), 3000 + case, 0, -2, 2)
        bt = ck.fill_int(dt, (N, K), 3000 + case, 1, -2, 2)
        c = ck.fill_int(ck.DT_F32, (M, N), 3000 + case, 2, -3, 3) if beta else None
        want = alpha * (G.as_f64(dt == ck.DT_BF16, a) @ G.as_f64(dt == ck.DT_BF16, bt).T)
        if beta:
            want = want + beta * c.astype(np.float64)
        prev = {k: ck.set_option(k, v) for k, v in opts.items()}
        try:
            da, db = G.to_dev(a), G.to_dev(bt)
            dc = None if c is None else G.to_dev(c)
            dd = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
            try:
                if entry == 0:
                    ck.gemm_shmem_tc_async_opt_port(dt, da, db, dc, dd, alpha, beta, M, N, K, *order)
                elif entry == 1:
                    need = ck.gemm_workspace_bytes(M, N, K, True, *order)
                    ws = torch.empty(need + 64, dtype=torch.uint8, device="cuda")
                    ck.gemm_shmem_tc_async_opt_port_ws(dt, ck.DT_F32, da, db, dc, dd, alpha, beta, M, N, K, *order,
                                                       ws.data_ptr() + int(rng.integers(0, 48)), need)
                else:
                    ck.gemm_shmem_tc_async_opt_port_noalloc(dt, da, db, dc, dd, alpha, beta, M, N, K, *order)
            except ck.CkoptError as e:
                assert e.code == ck.ERR_NO_INSTANCE, (case, order, e)
                continue
            assert ck.device_status() == 0
            assert np.array_equal(dd.cpu().numpy(), want.astype(np.float32)), (case, (M, N, K), dt, alpha, beta, order, opts, entry)
            ran += 1
        finally:
            for k, v in prev.items():
                ck.set_option(k, v)
    assert ran >= 0.55 * cases
