"""The entry point that allocates nothing (ckopt_gemm_shmem_tc_async_opt_port_2_noalloc) against the allocating
port_2 entry point, through the C ABI: two calls in a row on the same device, the second with a smaller input,
bit for bit (both run the same kernels in the same order, only the home of the scratch memory differs)."""
import numpy as np
import pytest
import torch

from tests import gpu_util as G

pytestmark = pytest.mark.gpu

STRAIGHT_LINE = dict(tile_dim=256, segment_dim_k=32, num_stages=5, num_producer_warps=0, num_consumer_warps=8)


def launch(fn, ck, dtype, da, db, dc, M, N, K, alpha, beta, t):
    dd = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    fn(dtype, da, db, dc, dd, alpha, beta, M, N, K, t["tile_dim"], t["segment_dim_k"], t["bar_steps_a"], t["bar_steps_b"],
       t["bar_step_rows_a"], t["bar_step_rows_b"], t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
       t["num_consumer_warps"], t["num_sms"])
    assert ck.device_status() == 0
    return dd.cpu().numpy()


def both(ck, dtype, a, bt, c, alpha, beta, t):
    M, K = a.shape
    N = bt.shape[0]
    da, db = G.to_dev(a), G.to_dev(bt)
    dc = None if c is None else G.to_dev(c)
    want = launch(ck.gemm_shmem_tc_async_opt_port, ck, dtype, da, db, dc, M, N, K, alpha, beta, t)
    got = launch(ck.gemm_shmem_tc_async_opt_port_noalloc, ck, dtype, da, db, dc, M, N, K, alpha, beta, t)
    return want, got


def test_no_alloc_entry_matches_port_2_on_two_calls_in_a_row(ck, oracle):
    t = G.tuning(**STRAIGHT_LINE)
    prev = ck.set_option(ck.OPT_SPLIT_K, 4)   # cut K into four slices wherever that is legal: the planes are scratch
    try:
        # first call: 8 tiles x 4 slices, 8 MiB of planes, uniform data (the sliced sums round like port_2's)
        M, N, K = 512, 1024, 8192
        a = ck.fill_uniform(ck.DT_F16, (M, K), 301, 0)
        bt = ck.fill_uniform(ck.DT_F16, (N, K), 301, 1)
        c = ck.fill_uniform(ck.DT_F32, (M, N), 301, 2)
        want, got = both(ck, ck.DT_F16, a, bt, c, 1.5, -0.5, t)
        assert np.array_equal(got, want)
        n, worst = oracle.count_outside_rel(oracle.gemm(oracle.DT_F16, a, bt, c, 1.5, -0.5), got, 1e-2)
        assert n == 0, worst
        # second call, smaller, on the array the first one left behind: ragged tiles, rows of 4090 bf16 elements
        # (not a multiple of 8: zero-padded copies of both operands AND four planes share the scratch), small integers
        M, N, K = 300, 200, 4090
        a = ck.fill_int(ck.DT_BF16, (M, K), 302, 0, -2, 2)
        bt = ck.fill_int(ck.DT_BF16, (N, K), 302, 1, -2, 2)
        want, got = both(ck, ck.DT_BF16, a, bt, None, 1.0, 0.0, t)
        assert np.array_equal(got, want)
        exact = (G.as_f64(True, a) @ G.as_f64(True, bt).T).astype(np.float32)
        assert np.array_equal(got, exact)
    finally:
        ck.set_option(ck.OPT_SPLIT_K, prev)


def test_no_alloc_entry_other_kernels_and_the_size_limit(ck):
    # a launch that needs no scratch at all (producer/consumer kernel, aligned operands) goes through unchanged
    t = G.tuning(tile_dim=128, segment_dim_k=64, num_stages=2, num_producer_warps=2, num_consumer_warps=4)
    a = ck.fill_int(ck.DT_F16, (384, 512), 303, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (256, 512), 303, 1, -2, 2)
    want, got = both(ck, ck.DT_F16, a, bt, None, 1.0, 0.0, t)
    assert np.array_equal(got, want)
    # beyond the array: 4 slices x 4096 x 2048 x 4 bytes = 128 MiB of planes -> a clear error, D untouched
    t = G.tuning(**STRAIGHT_LINE)
    M, N, K = 4096, 2048, 4096
    da = torch.zeros((M, K), dtype=torch.float16, device="cuda")
    db = torch.zeros((N, K), dtype=torch.float16, device="cuda")
    dd = torch.full((M, N), 7.0, dtype=torch.float32, device="cuda")
    assert 4 * M * N * 4 > ck.NOALLOC_SCRATCH_BYTES
    prev = ck.set_option(ck.OPT_SPLIT_K, 4)
    try:
        with pytest.raises(ck.CkoptError) as e:
            ck.gemm_shmem_tc_async_opt_port_noalloc(ck.DT_F16, da, db, None, dd, 1.0, 0.0, M, N, K, 256, 32, 0, 0, 256, 256, 4, 5, 0,
                                                    8, 256)
        assert e.value.code == ck.ERR_TOO_LARGE
        torch.cuda.synchronize()
        assert float(dd.min()) == float(dd.max()) == 7.0
        ck.set_option(ck.OPT_SPLIT_K, 0)   # without slices the same launch needs no scratch
        ck.gemm_shmem_tc_async_opt_port_noalloc(ck.DT_F16, da, db, None, dd, 1.0, 0.0, M, N, K, 256, 32, 0, 0, 256, 256, 4, 5, 0, 8,
                                                256)
        assert ck.device_status() == 0
        assert float(dd.min()) == float(dd.max()) == 0.0
    finally:
        ck.set_option(ck.OPT_SPLIT_K, prev)


def test_no_alloc_entry_leaves_free_device_memory_unchanged(ck):
    # after one call has loaded what the runtime loads lazily, further calls must not move the free-memory figure
    t = G.tuning(**STRAIGHT_LINE)
    M, N, K = 512, 512, 4090   # zero-padded copies + planes
    a = G.to_dev(ck.fill_int(ck.DT_F16, (M, K), 304, 0, -2, 2))
    bt = G.to_dev(ck.fill_int(ck.DT_F16, (N, K), 304, 1, -2, 2))
    dd = torch.empty((M, N), dtype=torch.float32, device="cuda")
    prev = ck.set_option(ck.OPT_SPLIT_K, 4)
    try:
        def call():
            ck.gemm_shmem_tc_async_opt_port_noalloc(ck.DT_F16, a, bt, None, dd, 1.0, 0.0, M, N, K, 256, 32, 0, 0, 256, 256, 4, 5,
                                                    0, 8, 256)
        call()
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        for _ in range(5):
            call()
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        assert free1 == free0
    finally:
        ck.set_option(ck.OPT_SPLIT_K, prev)


@pytest.mark.parametrize("M,N,K", [(700, 520, 1031), (1024, 1024, 8192)])
def test_no_alloc_entry_in_a_captured_graph(ck, M, N, K):
    """What the entry point is for: a launch recorded into a HIP graph (operand copies for the odd K, K slices and the
    reduction pass for the few tiles - kernels only, nothing allocated, nothing cleared by a memset node) and replayed
    several times with eager work and synchronisations between the replays; every replay exact on small integers."""
    t = G.tuning(**STRAIGHT_LINE)
    order = [t[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b",
                            "tile_group_m", "num_stages", "num_producer_warps", "num_consumer_warps", "num_sms")]
    a = ck.fill_int(ck.DT_F16, (M, K), 31, 0, -2, 2)
    bt = ck.fill_int(ck.DT_F16, (N, K), 31, 1, -2, 2)
    exact = (a.astype(np.float64) @ bt.astype(np.float64).T).astype(np.float32)
    da, db = G.to_dev(a), G.to_dev(bt)
    dd = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):   # a first eager call: kernel attributes and the array's address are looked up outside the capture
        ck.gemm_shmem_tc_async_opt_port_noalloc(ck.DT_F16, da, db, None, dd, 1.0, 0.0, M, N, K, *order, side)
    side.synchronize()
    assert np.array_equal(dd.cpu().numpy(), exact)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ck.gemm_shmem_tc_async_opt_port_noalloc(ck.DT_F16, da, db, None, dd, 1.0, 0.0, M, N, K, *order, torch.cuda.current_stream())
    for replay in range(3):
        dd.fill_(float("nan"))          # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(dd.cpu().numpy(), exact), replay
    assert ck.device_status() == 0
