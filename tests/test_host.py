"""CPU-only tests of the host side: the C ABI loads and exports what include/ckopt.h declares,
parameter legality mirrors the reference launcher's asserts, the index helpers agree with the oracle's
restatement of the reference on the reference's domain, and the seeded generator is reproducible.
No kernel is launched here.
"""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ckopt.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ckopt_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(ck):
    lib = ctypes.CDLL(ck.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 18
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(ck.EXPORTED_SYMBOLS) == names


def test_num_acc_and_warp_tile_rows_match_reference_closed_forms(ck, oracle):
    L = oracle.lib()
    for t in (64, 128):
        for c in (4, 8):
            assert ck.get_num_acc(t, c) == L.oracle_get_num_acc(t, c)
            assert ck.get_warp_tile_rows(t, c) == L.oracle_get_warp_tile_rows(t, c)
    # extension to 256: (C/2) x 2 wave tiles of 16x16 blocks
    assert ck.get_num_acc(256, 8) == 32 and ck.get_warp_tile_rows(256, 8) == 4
    with pytest.raises(ck.CkoptError):
        ck.get_num_acc(96, 4)


@pytest.mark.parametrize("M,N,t,g", [(512, 512, 128, 1), (1024, 768, 128, 3), (640, 1280, 64, 4), (256, 256, 64, 6),
                                     (2048, 2048, 256, 4)])
def test_tile_offset_matches_reference_order(ck, oracle, M, N, t, g):
    L = oracle.lib()
    for tc in range((M // t) * (N // t)):
        assert ck.get_tile_offset_cd(M, N, t, g, tc) == L.oracle_get_tile_offset_cd(M, N, t, g, tc)


def test_tile_offset_ragged_is_a_bijection_and_64_bit(ck):
    M, N, t, g = 6143, 4097, 128, 5
    tm, tn = -(-M // t), -(-N // t)
    got = sorted(ck.get_tile_offset_cd(M, N, t, g, tc) for tc in range(tm * tn))
    assert got == sorted(r * t * N + c * t for r in range(tm) for c in range(tn))
    # past int32: 65536 x 65536, last tile
    big = ck.get_tile_offset_cd(65536, 65536, 256, 4, 256 * 256 - 1)
    assert big == (65536 - 256) * 65536 + (65536 - 256)


def test_lds_req_layout(ck):
    # flag region rounded to 1 KiB + stages x 2 operands x tile x seg_k x 2 bytes, no padding
    assert ck.get_lds_req(128, 64, 0, 0, 128, 128, 2, 4) == 1024 + 2 * 2 * 128 * 64 * 2
    assert ck.get_lds_req(256, 32, 0, 0, 256, 256, 4, 8) == 1024 + 4 * 2 * 256 * 32 * 2
    # wave mode: 2*(sa+1) + 2*(sb+1) counters per stage; acc mode: 2*(C/2)*(sa+1) + 2*2*(sb+1)
    assert ck.get_lds_req(128, 64, 2, 2, 64, 64, 3, 4) == 1024 + 3 * 2 * 128 * 64 * 2
    assert ck.get_lds_req(256, 32, 3, 7, 16, 16, 16, 8) == 4096 + 16 * 2 * 256 * 32 * 2
    with pytest.raises(ck.CkoptError):
        ck.get_lds_req(128, 64, 0, 0, 48, 48, 2, 4)  # not one of the three granularities


def tup(**kw):
    d = dict(tile_dim=128, segment_dim_k=64, bar_steps_a=0, bar_steps_b=0, bar_step_rows_a=128, bar_step_rows_b=128,
             tile_group_m=4, num_stages=2, num_producer_waves=2, num_consumer_waves=4, num_cus=256)
    d.update(kw)
    return d


def test_tuning_legality_mirrors_reference_asserts(ck):
    ok = lambda **kw: ck.check_gemm_tuning(**tup(**kw))
    assert ok() == ck.OK
    assert ok(tile_dim=96, bar_step_rows_a=96, bar_step_rows_b=96) == ck.ERR_BAD_PARAM     # port_2.cu:1112
    assert ok(segment_dim_k=48) == ck.ERR_BAD_PARAM                                          # :1113
    # every multiple of 64 is legal in the reference (port_2.cu:1113; its drivers sweep 64 -> 256, :1520-1564): depths
    # without a kernel instance are "no instance", not "bad parameter"; 256 has instances on 64 and 128 tiles
    assert ok(segment_dim_k=192, num_stages=1) == ck.ERR_NO_INSTANCE
    assert ok(segment_dim_k=256, num_stages=1) == ck.OK                       # 128 tile, one stage: 1 KiB + 128 KiB
    assert ok(segment_dim_k=256, num_stages=2) == ck.ERR_LDS_BUDGET
    assert ok(tile_dim=64, bar_step_rows_a=64, bar_step_rows_b=64, segment_dim_k=256, num_stages=2) == ck.OK
    assert ok(segment_dim_k=256, num_stages=1, num_producer_waves=0) == ck.ERR_NO_INSTANCE   # producer/consumer kernels only
    assert ok(segment_dim_k=320, num_stages=1) == ck.ERR_LDS_BUDGET
    assert ok(segment_dim_k=96, num_stages=1) == ck.ERR_NO_INSTANCE
    assert ok(segment_dim_k=0) == ck.ERR_BAD_PARAM and ok(segment_dim_k=-64) == ck.ERR_BAD_PARAM
    assert ok(num_producer_waves=1) == ck.ERR_BAD_PARAM      # one producer warp is legal in port_0 only (port_0.cu:538)
    assert ok(num_producer_waves=3) == ck.ERR_BAD_PARAM                                      # :1122
    assert ok(num_producer_waves=0) == ck.OK                 # fused variant (extension), tile granularity only
    assert ok(num_producer_waves=0, bar_step_rows_a=64, bar_step_rows_b=64) == ck.ERR_NO_INSTANCE
    assert ok(num_producer_waves=0, num_stages=1) == ck.OK   # one stage: the synchronous load / barrier / multiply / barrier kernel
    assert ok(num_consumer_waves=6) == ck.ERR_BAD_PARAM                                      # :1123
    assert ok(num_stages=0) == ck.ERR_BAD_PARAM                                              # :1121
    assert ok(tile_group_m=0) == ck.ERR_BAD_PARAM
    # barrier-mode triple (:1116-1120): wave-tile mode t=128, C=4 -> rows 64, cols 64, steps <= 2 / <= 2
    assert ok(bar_step_rows_a=64, bar_step_rows_b=64, bar_steps_a=2, bar_steps_b=2) == ck.OK
    assert ok(bar_step_rows_a=64, bar_step_rows_b=64, bar_steps_a=3, bar_steps_b=2) == ck.ERR_BAD_PARAM
    assert ok(bar_step_rows_a=64, bar_step_rows_b=32) == ck.ERR_BAD_PARAM
    # accumulator mode: steps strictly below wave tile rows / cols (4 x 4 for t=128, C=4)
    assert ok(bar_step_rows_a=16, bar_step_rows_b=16, bar_steps_a=3, bar_steps_b=3) == ck.OK
    assert ok(bar_step_rows_a=16, bar_step_rows_b=16, bar_steps_a=4, bar_steps_b=0) == ck.ERR_BAD_PARAM
    # LDS budget: 160 KiB
    assert ok(num_stages=4) == ck.OK                                   # 1 KiB + 128 KiB
    assert ok(num_stages=5) == ck.ERR_LDS_BUDGET
    assert ok(tile_dim=256, bar_step_rows_a=256, bar_step_rows_b=256, num_consumer_waves=8, segment_dim_k=64, num_stages=3) == ck.ERR_LDS_BUDGET
    # register budget: a 256 tile with 4 consumer waves needs 256 accumulator registers per wave;
    # 8 producers + 8 consumers at tile 256 exceed the instance's wave count (the reference's own
    # P=8, C=8 launch failure, port_1.cu:35-42, becomes an error code)
    assert ok(tile_dim=256, bar_step_rows_a=256, bar_step_rows_b=256, num_consumer_waves=4) == ck.ERR_NO_INSTANCE
    assert ok(tile_dim=256, bar_step_rows_a=256, bar_step_rows_b=256, num_consumer_waves=8, num_producer_waves=8,
              segment_dim_k=32) == ck.ERR_NO_INSTANCE
    assert ok(tile_dim=256, bar_step_rows_a=256, bar_step_rows_b=256, num_consumer_waves=8, num_producer_waves=4,
              segment_dim_k=32, num_stages=4) == ck.OK


def test_launch_rejects_bad_arguments_before_touching_the_gpu(ck):
    # null pointers and illegal shapes are reported without any HIP call
    args = dict(tile_dim=128, segment_dim_k=64, bar_steps_a=0, bar_steps_b=0, bar_step_rows_a=128, bar_step_rows_b=128,
                tile_group_m=4, num_stages=2, num_producer_warps=2, num_consumer_warps=4, num_sms=256)
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, None, None, None, None, 1.0, 0.0, 256, 256, 256, **args)
    assert e.value.code == ck.ERR_NULL
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F32, 16, 16, None, 16, 1.0, 0.0, 256, 256, 256, **args)
    assert e.value.code == ck.ERR_BAD_PARAM
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, 16, 16, None, 16, 1.0, 0.0, 0, 256, 256, **args)
    assert e.value.code == ck.ERR_BAD_PARAM
    with pytest.raises(ck.CkoptError) as e:  # beta != 0 needs C
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, 16, 16, None, 16, 1.0, 1.0, 256, 256, 256, **args)
    assert e.value.code == ck.ERR_NULL
    with pytest.raises(ck.CkoptError) as e:  # A not even 2-byte aligned
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, 17, 16, None, 16, 1.0, 0.0, 256, 256, 256, **args)
    assert e.value.code == ck.ERR_ALIGNMENT
    # port_0 takes one producer warp (port_0.cu:538): the tuple passes validation and the call stops at the null pointers;
    # the port_1 / port_2 launchers do not (port_2.cu:1122)
    p0 = dict(tile_dim=128, segment_dim_k=64, tile_group_m=4, num_stages=2, num_producer_warps=1, num_consumer_warps=4, num_sms=256)
    for fn in (ck.gemm_shmem_tc_async_opt_port_0, ck.gemm_shmem_tc_async_opt_port_0_lp):
        with pytest.raises(ck.CkoptError) as e:
            fn(ck.DT_F16, None, None, None, None, 1.0, 0.0, 256, 256, 256, **p0)
        assert e.value.code == ck.ERR_NULL
        with pytest.raises(ck.CkoptError) as e:
            fn(ck.DT_F16, None, None, None, None, 1.0, 0.0, 256, 256, 256, **dict(p0, num_producer_warps=3))
        assert e.value.code == ck.ERR_BAD_PARAM
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, None, None, None, None, 1.0, 0.0, 256, 256, 256, **dict(args, num_producer_warps=1))
    assert e.value.code == ck.ERR_BAD_PARAM
    p1 = dict(tile_dim=128, segment_dim_k=64, bar_step_rows_a=64, bar_step_rows_b=64, tile_group_m=4, num_stages=2, num_producer_warps=2,
              num_consumer_warps=4, num_sms=256)
    for fn in (ck.gemm_shmem_tc_async_opt_port_1, ck.gemm_shmem_tc_async_opt_port_1_lp):
        with pytest.raises(ck.CkoptError) as e:
            fn(ck.DT_F16, None, None, None, None, 1.0, 0.0, 256, 256, 256, **p1)
        assert e.value.code == ck.ERR_NULL
        with pytest.raises(ck.CkoptError) as e:
            fn(ck.DT_F16, None, None, None, None, 1.0, 0.0, 256, 256, 256, **dict(p1, num_producer_warps=1))
        assert e.value.code == ck.ERR_BAD_PARAM


def test_matmul_shmem_tuning_legality(ck):
    # reference: tile % block_rows == 0, accumulators per thread bounded, tile*block_rows <= max threads
    # (matmul_shmem.cu:153-155, :198-206)
    assert ck.check_matmul_shmem_tuning(32, 8) == ck.OK
    assert ck.check_matmul_shmem_tuning(128, 2) == ck.OK       # 64 accumulators per thread (extension)
    assert ck.check_matmul_shmem_tuning(128, 4) == ck.OK
    assert ck.check_matmul_shmem_tuning(128, 16) == ck.ERR_NO_INSTANCE   # 2048 threads
    assert ck.check_matmul_shmem_tuning(64, 3) == ck.ERR_BAD_PARAM
    assert ck.check_matmul_shmem_tuning(48, 4) == ck.ERR_BAD_PARAM
    assert ck.check_matmul_shmem_tuning(32, 1) == ck.ERR_NO_INSTANCE     # 32 threads: less than a wavefront
    assert ck.matmul_shmem_lds_req(ck.DT_F32, 128) == 2 * 2 * 16 * 132 * 4
    with pytest.raises(ck.CkoptError) as e:
        ck.matmul_shmem(ck.DT_F32, 16, 16, 16, 100, 128, 128, 32, 8)
    assert e.value.code == ck.ERR_BAD_PARAM


def test_splitmix64_known_answers(oracle):
    # first outputs of SplitMix64 seeded with 1234567 (Vigna's reference implementation)
    z = oracle.splitmix64_at(1234567, np.arange(5))
    assert [int(v) for v in z] == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                   4593380528125082431, 16408922859458223821]


def test_uniform_generator_matches_numpy_restatement_and_is_seeded(ck, oracle):
    n = 10000
    for seed, stream in ((0xC0FFEE01, 0), (0xC0FFEE01, 1), (42, 7)):
        f32 = ck.fill_uniform(ck.DT_F32, (n,), seed, stream, -1.0, 1.0)
        want = oracle.uniform_f32(n, seed, stream, -1.0, 1.0)
        assert np.array_equal(f32, want)
        f16 = ck.fill_uniform(ck.DT_F16, (n,), seed, stream, -1.0, 1.0)
        assert np.array_equal(f16.view(np.uint16), want.astype(np.float16).view(np.uint16))   # RNE to half
        b16 = ck.fill_uniform(ck.DT_BF16, (n,), seed, stream, -1.0, 1.0)
        tb = torch.from_numpy(want).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(b16, tb)                                                          # RNE to bf16
    a = ck.fill_uniform(ck.DT_F32, (n,), 1, 0)
    assert np.array_equal(a, ck.fill_uniform(ck.DT_F32, (n,), 1, 0))
    assert not np.array_equal(a, ck.fill_uniform(ck.DT_F32, (n,), 2, 0))
    assert not np.array_equal(a, ck.fill_uniform(ck.DT_F32, (n,), 1, 1))
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(float(a.mean())) < 0.03
    # a sub-range reproduces the same values: element i depends on (seed, stream, i) only
    assert np.array_equal(ck.fill_uniform(ck.DT_F32, (100,), 1, 0), a[:100])


def test_half_rounding_edge_cases(ck):
    vals = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8, 2.98e-8, 2.99e-8, 6.1e-5, 1.0009765625, 1.00048828125,
                     -3.14159, 1e6, -1e6], dtype=np.float32)
    for v in vals:
        got = ck.fill_constant(ck.DT_F16, (1,), float(v)).view(np.uint16)[0]
        with np.errstate(over="ignore"):
            want = np.float32(v).astype(np.float16).view(np.uint16)
        assert got == want, (v, hex(got), hex(want))


def test_normal_and_int_generators(ck):
    x = ck.fill_normal(ck.DT_F32, (200000,), 5, 0, 0.0, 0.1)
    assert abs(float(x.mean())) < 2e-3 and abs(float(x.std()) - 0.1) < 2e-3
    assert np.array_equal(x, ck.fill_normal(ck.DT_F32, (200000,), 5, 0, 0.0, 0.1))
    k = ck.fill_int(ck.DT_I32, (50000,), 9, 3, -10, 10)
    assert k.min() == -10 and k.max() == 10 and len(np.unique(k)) == 21
    h = ck.fill_int(ck.DT_F16, (1000,), 9, 3, -2, 2)
    assert set(np.unique(h.astype(np.int32))) == {-2, -1, 0, 1, 2}
    c = ck.fill_constant(ck.DT_BF16, (8,), 10.0)
    assert np.all(c == 0x4120)


def test_option_keys_reject_values_outside_their_range(ck):
    # process-wide switches: a bad value changes nothing and reports the error
    for key, bad in ((ck.OPT_NUM_XCD, 0), (ck.OPT_PRIO_MODE, 3), (ck.OPT_PRODUCER_NAP, -1), (ck.OPT_SPLIT_K, 17), (ck.OPT_D_STORE_POLICY, 3), (ck.OPT_HALF_WIDTH, 4), (99, 1),
                     (15, 1), (-1, 0), (ck.OPT_SPIN_LIMIT, 0)):
        with pytest.raises(ck.CkoptError):
            ck.set_option(key, bad)
    prev = ck.set_option(ck.OPT_SPLIT_K, 0)
    assert ck.set_option(ck.OPT_SPLIT_K, prev) == 0
    prev = ck.set_option(ck.OPT_STRAIGHT_LINE, 0)
    assert ck.set_option(ck.OPT_STRAIGHT_LINE, prev) == 0
    prev = ck.set_option(ck.OPT_EVEN_ROUNDS, 0)
    assert prev == 1 and ck.set_option(ck.OPT_EVEN_ROUNDS, prev) == 0
    prev = ck.set_option(ck.OPT_D_STORE_POLICY, 2)
    assert prev == 0 and ck.set_option(ck.OPT_D_STORE_POLICY, prev) == 2


def test_suggested_tunings_are_legal_and_follow_the_measured_rules(ck):
    # every suggestion passes the launcher's own validation; the BASELINE shapes get the tuples bench.py uses
    import itertools
    for M, N, K in itertools.product((1, 100, 512, 1024, 2048, 3000, 8192), (4, 130, 1024, 4097), (8, 64, 1000, 3071, 32768)):
        t = ck.suggest_gemm_tuning(M, N, K)
        assert ck.check_gemm_tuning(t["tile_dim"], t["segment_dim_k"], t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"],
                                    t["bar_step_rows_b"], t["tile_group_m"], t["num_stages"], t["num_producer_warps"],
                                    t["num_consumer_warps"], t["num_sms"]) == 0, (M, N, K, t)
    straight = dict(tile_dim=256, segment_dim_k=32, num_stages=5, num_producer_warps=0, num_consumer_warps=8)
    def picks(M, N, K):
        t = ck.suggest_gemm_tuning(M, N, K)
        return {k: t[k] for k in straight}
    assert picks(8192, 8192, 8192) == straight          # config 3
    assert picks(2048, 2048, 32768) == straight         # config 4: 64 tiles, four slices of 8192
    assert picks(6143, 4097, 3071) == straight          # config 5: K is 3072 after the repack
    assert picks(16384, 16384, 16384) == straight
    assert picks(1024, 1024, 8192) == straight          # 16 tiles, eight slices of 1024
    assert picks(2048, 2048, 2048)["tile_dim"] == 128   # 64 tiles of 256 and K too shallow to cut four times
    assert picks(512, 512, 512)["tile_dim"] == 64       # config 1
    assert picks(8192, 8192, 8200) == straight          # any K: its end is masked in the kernel (or in the operand copies)
    # K a multiple of 8 but not of 64 runs on K itself (no copies), where no slice count is legal: few tiles with such a K
    # must be judged as one pass over 16 tiles, not as the slices a K padded to 8256 would allow
    assert ck.gemm_launch_plan(1024, 1024, 8200, True, *(straight[k] for k in ("tile_dim", "segment_dim_k")), 0, 0, 256, 256, 4, 5, 0, 8, 256)["k_slices"] == 1
    assert picks(1024, 1024, 8200)["tile_dim"] in (64, 128)
    assert picks(1024, 1024, 8192) == straight
    prev = ck.set_option(ck.OPT_STRAIGHT_LINE, 0)
    try:
        assert picks(8192, 8192, 8192)["num_producer_warps"] == 2 and picks(8192, 8192, 8192)["tile_dim"] == 256
    finally:
        ck.set_option(ck.OPT_STRAIGHT_LINE, prev)
    with pytest.raises(ck.CkoptError):
        ck.suggest_gemm_tuning(0, 1, 1)


def test_matmul_shmem_multiply_adds_avoid_one_bank_operands(tmp_path):
    """A v_fmac_f32 whose three registers lie in one register bank (number mod 4) issues at half rate on
    gfx950. The kernel keeps accumulator rows as aligned runs of four, rotated by one against the run of
    four a 16-byte LDS read delivers, so no multiply-add of an instance with an even-width row may have all
    three in one bank (rows of two columns: pairs, 8-byte reads). Checked on the compiled code of the kernel's own translation unit."""
    import importlib.util
    import subprocess
    spec = importlib.util.spec_from_file_location("ckopt_build", os.path.join(ROOT, "cuda-kernel-opt_amd", "build.py"))
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    src = os.path.join(ROOT, "cuda-kernel-opt_amd", "csrc", "simt_launch.hip")
    out = str(tmp_path / "simt.s")
    flags = [f for f in b.DEVICE_FLAGS if f != "-fPIC"]
    r = subprocess.run([b.HIPCC] + flags + ["-S", "--cuda-device-only", src, "-o", out], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    text = open(out).read()
    names = re.findall(r"^(_ZN2ck19matmul_shmem_kernelIfLi(\d+)ELi(\d+)ELi(\d+)ELb[01]EEEvNS_8SimtArgsE):", text, re.M)
    assert len(names) >= 20
    checked = 0
    for name, tile, rm, rn in names:
        if int(rn) % 2:
            continue
        body = text[text.index("\n" + name + ":"):]
        body = body[:body.index("s_endpgm")]
        ops = re.findall(r"v_fmac_f32_e32 v(\d+), v(\d+), v(\d+)", body)
        assert len(ops) >= int(rm) * int(rn)
        bad = [o for o in ops if int(o[0]) % 4 == int(o[1]) % 4 == int(o[2]) % 4]
        assert not bad, "%s: %d of %d multiply-adds with all registers in one bank" % (name, len(bad), len(ops))
        checked += 1
    assert checked >= 16


def test_straight_line_kernel_main_loops_hold_no_wait_of_the_compilers(tmp_path):
    """The ring's loads are issued from asm, so the compiler does not know of them: a vector-memory wait it inserts
    into the main loop on its own account (for a load of C it believes in flight on some path out of the epilogue)
    is a wait for everything (vmcnt(0)), and it empties the load queue once per k-step. The kernel's own waits sit
    inside asm statements; in the compiled code of the default instances (both element types, the three tile widths,
    and the K-tail form) no block with MFMAs may hold any other."""
    import importlib.util
    import subprocess
    spec = importlib.util.spec_from_file_location("ckopt_build", os.path.join(ROOT, "cuda-kernel-opt_amd", "build.py"))
    b = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(b)
    csrc = os.path.join(ROOT, "cuda-kernel-opt_amd", "csrc")
    unit = tmp_path / "stream_instances.hip"
    wanted = [("f16_tag", "false", 8), ("bf16_tag", "false", 8), ("f16_tag", "true", 8), ("bf16_tag", "true", 8),
              ("f16_tag", "false", 6), ("bf16_tag", "false", 6), ("f16_tag", "false", 4), ("bf16_tag", "false", 4)]
    unit.write_text('#include "gemm_stream_kernel.hip.h"\nnamespace ck {\n' + "".join(
        "template __global__ void gemm_stream_kernel<%s, false, %s, %d>(const GemmArgs);\n" % w for w in wanted) + "}\n")
    out = str(tmp_path / "stream.s")
    flags = [f for f in b.DEVICE_FLAGS if f != "-fPIC"]
    r = subprocess.run([b.HIPCC] + flags + ["-I", csrc, "-S", "--cuda-device-only", str(unit), "-o", out], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    kernel, block, in_asm, loops = None, None, False, {}
    for line in open(out):
        m = re.match(r"^(_ZN2ck18gemm_stream_kernel\S*):", line)
        if m:
            kernel, block = m.group(1), "entry"
            continue
        m = re.match(r"^(\.LBB\d+_\d+):", line)
        if m:
            block = m.group(1)
            continue
        if kernel is None:
            continue
        if "#ASMSTART" in line or "#ASMEND" in line:
            in_asm = "#ASMSTART" in line
            continue
        entry = loops.setdefault((kernel, block), [0, []])
        if "v_mfma" in line:
            entry[0] += 1
        if not in_asm and "s_waitcnt" in line and "vmcnt" in line:
            entry[1].append(line.strip())
    main_loops = {k: v for k, v in loops.items() if v[0] >= 32}   # one loop body: two k-steps of 16, 24 or 32 MFMAs
    assert len({k[0] for k in main_loops}) == len(wanted)
    for (kernel, block), (mfmas, waits) in main_loops.items():
        assert not waits, "%s %s (%d MFMAs): %s" % (kernel, block, mfmas, waits)


def test_workspace_query_follows_the_launcher_rules(ck):
    # pure host arithmetic (no GPU call): what a launch takes from a caller-owned workspace
    straight = (256, 32, 0, 0, 256, 256, 4, 5, 0, 8, 256)
    pc = (128, 64, 0, 0, 128, 128, 4, 2, 2, 4, 256)
    r256 = lambda n: (n + 255) // 256 * 256
    # aligned operands, enough tiles: nothing
    assert ck.gemm_workspace_bytes(8192, 8192, 8192, True, *straight) == 0
    assert ck.gemm_workspace_bytes(512, 512, 512, True, *pc) == 0
    # config 4: 64 tiles on 256 CUs -> four slices of 2048 x 2048 fp32, plus room to align the caller's pointer
    assert ck.gemm_workspace_bytes(2048, 2048, 32768, True, *straight) == 4 * 2048 * 2048 * 4 + 256
    # config 5: rows of 3071 elements -> zero-padded copies of both operands with rows of 3072; 408 tiles are not cut
    assert ck.gemm_workspace_bytes(6143, 4097, 3071, True, *straight) == r256((6143 + 4097) * 3072 * 2) + 256
    # operands off a 16-byte boundary are copied whatever K is; other kernels never cut K
    assert ck.gemm_workspace_bytes(512, 512, 512, False, *pc) == r256(2 * 512 * 512 * 2) + 256
    assert ck.gemm_workspace_bytes(256, 256, 32768, True, *pc) == 0
    # copies and planes together (2 x 3 tiles, K 4090 -> 4096, four slices)
    assert ck.gemm_workspace_bytes(300, 520, 4090, True, *straight) == r256((300 + 520) * 4096 * 2) + r256(4 * 300 * 520 * 4) + 256
    # K 8200 (a multiple of 8): no copies, the straight-line kernel masks the end of K itself; K 8201: copies, with rows
    # of 8256 (whole loop bodies of 64) for the straight-line tuple and of 8208 for the others
    assert ck.gemm_workspace_bytes(8192, 8192, 8200, True, *straight) == 0
    assert ck.gemm_workspace_bytes(8192, 8192, 8201, True, *straight) == r256(2 * 8192 * 8256 * 2) + 256
    assert ck.gemm_workspace_bytes(8192, 8192, 8201, True, *pc) == r256(2 * 8192 * 8208 * 2) + 256
    # 36 tiles (1536^2) with a deep K are cut as well: four slices
    assert ck.gemm_workspace_bytes(1536, 1536, 8192, True, *straight) == 4 * 1536 * 1536 * 4 + 256
    # the automatic slice count follows the launcher's cost model: 128 tiles with a deep K are cut in two (256 items),
    # with K 4096 not at all (the reduction pass would cost more than the idle half of the CUs); 81 tiles in three;
    # 144 tiles never (two slices would be 288 items: two rounds). The slices are added by the second pass (planes of
    # M x N fp32) unless the option asks for the reduction inside the kernel: then per tile and slice one tile of fp32
    # (every slice's waves store their partial sums) behind eight 128-byte counter lines per tile
    assert ck.gemm_workspace_bytes(2048, 4096, 16384, True, *straight) == 2 * 2048 * 4096 * 4 + 256
    assert ck.gemm_workspace_bytes(2048, 4096, 16384, True, *straight, options=ck.launch_options(fused_reduction=0)) == 2 * 2048 * 4096 * 4 + 256
    assert (ck.gemm_workspace_bytes(2048, 4096, 16384, True, *straight, options=ck.launch_options(fused_reduction=2))
            == 128 * 8 * 128 + 2 * 128 * 256 * 256 * 4 + 256)
    assert ck.gemm_workspace_bytes(2048, 4096, 4096, True, *straight) == 0
    assert ck.gemm_workspace_bytes(2304, 2304, 12288, True, *straight) == 3 * 2304 * 2304 * 4 + 256
    assert ck.gemm_workspace_bytes(3072, 3072, 8192, True, *straight) == 0
    # the split-K switch is part of the rule
    prev = ck.set_option(ck.OPT_SPLIT_K, 0)
    try:
        assert ck.gemm_workspace_bytes(2048, 2048, 32768, True, *straight) == 0
    finally:
        ck.set_option(ck.OPT_SPLIT_K, prev)
    for bad in ((0, 1, 1), (1, 0, 1), (1, 1, 0)):
        with pytest.raises(ck.CkoptError):
            ck.gemm_workspace_bytes(*bad, True, *straight)


def test_launch_plan_reports_what_a_launch_will_run(ck):
    # pure host arithmetic: kernel form, tile width, K slices, operand copies - the launcher's own rules
    straight = (256, 32, 0, 0, 256, 256, 4, 5, 0, 8, 256)
    pc = (128, 64, 0, 0, 128, 128, 4, 2, 2, 4, 256)
    def plan(*a, **kw):
        return ck.gemm_launch_plan(*a, **kw)
    assert plan(8192, 8192, 8192, True, *straight) == dict(straight_line=True, tile_cols=256, k_slices=1, operand_copies=False, sliced_tiles=0,
                                                           reduced_in_kernel=False, grid=256)
    assert plan(2048, 2048, 32768, True, *straight) == dict(straight_line=True, tile_cols=256, k_slices=4, operand_copies=False, sliced_tiles=64,
                                                            reduced_in_kernel=False, grid=256)
    assert plan(2048, 4096, 16384, True, *straight) == dict(straight_line=True, tile_cols=256, k_slices=2, operand_copies=False, sliced_tiles=128,
                                                            reduced_in_kernel=False, grid=256)
    assert plan(2048, 4096, 16384, True, *straight, options=ck.launch_options(fused_reduction=2))["reduced_in_kernel"]
    assert plan(6143, 4097, 3071, True, *straight) == dict(straight_line=True, tile_cols=256, k_slices=1, operand_copies=True, sliced_tiles=0,
                                                           reduced_in_kernel=False, grid=208)
    assert plan(2560, 2560, 2560, True, *straight) == dict(straight_line=True, tile_cols=128, k_slices=1, operand_copies=False, sliced_tiles=0,
                                                           reduced_in_kernel=False, grid=200)
    assert plan(8192, 8192, 8192, False, *pc) == dict(straight_line=False, tile_cols=128, k_slices=1, operand_copies=True, sliced_tiles=0,
                                                      reduced_in_kernel=False, grid=0)
    # the partly filled last round: 20 tiles on 16 workgroups with a deep K -> 16 whole tiles, then 4 tiles in K slices
    # added inside the kernel, all in one launch of 16 workgroups; switched off: 2 rounds of 10
    tail = (256, 32, 0, 0, 256, 256, 4, 5, 0, 8, 16)
    p = plan(1024, 1280, 8192, True, *tail, options=ck.launch_options(half_width=0))
    assert p["sliced_tiles"] == 4 and p["k_slices"] in (2, 3, 4) and p["reduced_in_kernel"] and p["grid"] == 16
    p = plan(1024, 1280, 8192, True, *tail, options=ck.launch_options(tail_round=0))
    assert p["sliced_tiles"] == 0 and p["k_slices"] == 1 and p["grid"] <= 16 and p["tile_cols"] in (256, 192)
    prev = ck.set_option(ck.OPT_HALF_WIDTH, 0)
    try:
        assert ck.gemm_launch_plan(2560, 2560, 2560, True, *straight)["tile_cols"] == 256
    finally:
        ck.set_option(ck.OPT_HALF_WIDTH, prev)
    # 256 x 192 tiles where the other widths fill the last round badly: 6144^3 is 576 tiles of 256 x 256 (2.25 rounds) but 768 of
    # 256 x 192 (exactly 3); 3072^3 is 144 of 256 (0.56 of a round) but 192 of 192 (0.75)
    assert plan(6144, 6144, 6144, True, *straight)["tile_cols"] == 192 and plan(6144, 6144, 6144, True, *straight)["grid"] == 256
    assert plan(3072, 3072, 3072, True, *straight)["tile_cols"] == 192
    assert plan(3072, 3072, 3072, True, *straight, options=ck.launch_options(half_width=0))["tile_cols"] == 256
    assert plan(8192, 8192, 8192, True, *straight, options=ck.launch_options(half_width=3))["tile_cols"] == 192
    prev = ck.set_option(ck.OPT_STRAIGHT_LINE, 0)
    try:
        assert ck.gemm_launch_plan(8192, 8192, 8192, True, *straight)["straight_line"] is False
    finally:
        ck.set_option(ck.OPT_STRAIGHT_LINE, prev)
    with pytest.raises(ck.CkoptError):
        ck.gemm_launch_plan(0, 1, 1, True, *straight)


def test_bench_refuses_more_than_one_gpu():
    # every box of this build has one GPU and the GEMM path has no collective: --gpus 2 exits with a message that says so
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_query_and_plan_are_pure_functions_of_their_arguments(ck):
    """The _ex queries take the launch options as an argument (in the reference every knob is a launcher parameter,
    port_2.cu:1088-1109): what they answer depends on that argument alone, whatever the process-wide switches say."""
    straight = (256, 32, 0, 0, 256, 256, 4, 5, 0, 8, 256)
    shapes = [(2048, 2048, 32768), (2048, 4096, 16384), (6143, 4097, 3071), (2560, 2560, 2560), (300, 520, 4090), (8192, 8192, 8192)]
    variants = [dict(), dict(split_k=0), dict(split_k=2), dict(half_width=0), dict(half_width=2), dict(fused_reduction=0),
                dict(straight_line=0), dict(even_rounds=0), dict(tail_round=0)]
    frozen = [ck.launch_options(**v) for v in variants]       # taken while the process-wide switches have their defaults
    want = [[(ck.gemm_workspace_bytes(*s, True, *straight, options=o), ck.gemm_launch_plan(*s, True, *straight, options=o)) for s in shapes]
            for o in frozen]
    assert len({repr(w) for w in want}) > 4                    # the options do matter
    changed = [(ck.OPT_SPLIT_K, 0), (ck.OPT_HALF_WIDTH, 2), (ck.OPT_STRAIGHT_LINE, 0), (ck.OPT_FUSED_REDUCTION, 0), (ck.OPT_EVEN_ROUNDS, 0)]
    prev = [ck.set_option(k, v) for k, v in changed]
    try:
        got = [[(ck.gemm_workspace_bytes(*s, True, *straight, options=o), ck.gemm_launch_plan(*s, True, *straight, options=o)) for s in shapes]
               for o in frozen]
        assert got == want
        # no options argument: the process-wide switches
        assert ck.gemm_launch_plan(8192, 8192, 8192, True, *straight)["straight_line"] is False
        assert ck.gemm_workspace_bytes(2048, 2048, 32768, True, *straight) == 0
        # ckopt_launch_options_init reads them
        assert ck.launch_options().split_k == 0 and ck.launch_options().half_width == 2
    finally:
        for (k, _), v in zip(changed, prev):
            ck.set_option(k, v)
    assert ck.launch_options().split_k == 1 and ck.launch_options().straight_line == 1
    # a struct of another size, or a field outside its key's range, is refused
    bad = ck.launch_options()
    bad.struct_bytes = 8
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_workspace_bytes(2048, 2048, 32768, True, *straight, options=bad)
    assert e.value.code == ck.ERR_BAD_PARAM
    bad = ck.launch_options()
    bad.split_k = 17
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_launch_plan(2048, 2048, 32768, True, *straight, options=bad)
    assert e.value.code == ck.ERR_BAD_PARAM
    with pytest.raises(ck.CkoptError) as e:   # the launch refuses it too, before any pointer is looked at
        ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, None, None, None, None, 1.0, 0.0, 256, 256, 256, *straight, options=bad)
    assert e.value.code == ck.ERR_BAD_PARAM
    with pytest.raises(ck.CkoptError) as e:
        ck.gemm_shmem_tc_async_opt_port_ex(ck.DT_F16, ck.DT_F32, None, None, None, None, 1.0, 0.0, 256, 256, 256, *straight, options=ck.launch_options())
    assert e.value.code == ck.ERR_NULL
