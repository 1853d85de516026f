"""Helpers shared by the GPU parity tests: device buffers via torch, launches via the C ABI."""
import numpy as np
import torch


def to_dev(x):
    """numpy array (float16 / uint16 bf16 bits / float32 / int32) -> device tensor with the same bytes."""
    x = np.ascontiguousarray(x)
    if x.dtype == np.uint16:
        return torch.from_numpy(x.view(np.int16)).cuda()
    return torch.from_numpy(x).cuda()


def tuning(tile_dim=128, segment_dim_k=64, bar_steps_a=0, bar_steps_b=0, bar_step_rows_a=None, bar_step_rows_b=None,
           tile_group_m=4, num_stages=2, num_producer_warps=2, num_consumer_warps=4, num_sms=256):
    return dict(tile_dim=tile_dim, segment_dim_k=segment_dim_k, bar_steps_a=bar_steps_a, bar_steps_b=bar_steps_b,
                bar_step_rows_a=tile_dim if bar_step_rows_a is None else bar_step_rows_a,
                bar_step_rows_b=tile_dim if bar_step_rows_b is None else bar_step_rows_b,
                tile_group_m=tile_group_m, num_stages=num_stages, num_producer_warps=num_producer_warps,
                num_consumer_warps=num_consumer_warps, num_sms=num_sms)


def wave_mode_rows(ck, t):
    wtr = ck.get_warp_tile_rows(t["tile_dim"], t["num_consumer_warps"])
    wtc = ck.get_num_acc(t["tile_dim"], t["num_consumer_warps"]) // wtr
    return wtr * 16, wtc * 16


def run_gemm(ck, dtype, a, bt, c=None, alpha=1.0, beta=0.0, t=None, poison=True):
    """Launches the port_2 entry point on device copies of the numpy inputs; returns D as numpy (M,N)."""
    t = t or tuning()
    M, K = a.shape
    N = bt.shape[0]
    da, db = to_dev(a), to_dev(bt)
    dc = None if c is None else to_dev(np.asarray(c, dtype=np.float32))
    dd = torch.full((M, N), float("nan") if poison else 0.0, dtype=torch.float32, device="cuda")
    ck.gemm_shmem_tc_async_opt_port(dtype, da, db, dc, dd, alpha, beta, M, N, K, t["tile_dim"], t["segment_dim_k"],
                                    t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"],
                                    t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                    t["num_consumer_warps"], t["num_sms"])
    status = ck.device_status()
    assert status == 0, "device status %d (a bounded flag wait gave up)" % status
    return dd.cpu().numpy()


def bf16_bits_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    """round-to-nearest-even float32 -> bf16 bit patterns (finite inputs)"""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def as_f64(dtype_is_bf16, x):
    return (bf16_bits_to_f32(x) if dtype_is_bf16 else x.astype(np.float32)).astype(np.float64)
