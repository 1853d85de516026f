#!/usr/bin/env python3
"""Headline benchmark: fp16 GEMM M=N=K=8192 (fp32 accumulate/output) on one MI355X through the C ABI.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [tuning flags]

A step is one launch of gemm_shmem_tc_async_opt_port over seeded synthetic A and Bt that are already
resident in HBM. Prints ONE JSON line: whole-job TFLOP/s, the MFMA roofline of the kernel (flops per
launch / average launch duration measured with HIP events on the launch stream, against the 2.5 PFLOP/s
dense fp16 peak) and the CPU oracle timed on a bounded sample of the same workload.
"""
import argparse
import importlib.util
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"mfma_f16": 2500.0, "valu_f32": 157.3}

WORKLOADS = {
    # name: (kind, dtype, M, N, K, distribution)
    "config1_fp16_512": ("gemm", "f16", 512, 512, 512, "uniform"),
    "config2_fp32_4096_simt": ("simt", "f32", 4096, 4096, 4096, "uniform"),
    "config3_fp16_8192": ("gemm", "f16", 8192, 8192, 8192, "uniform"),
    "config4_fp16_2048x2048x32768": ("gemm", "f16", 2048, 2048, 32768, "normal"),
    "config5_bf16_6143x4097x3071": ("gemm", "bf16", 6143, 4097, 3071, "uniform"),
    # not a BASELINE config: the size the reference's own performance driver times (port_2.cu:1554-1556)
    "config6_fp16_16384": ("gemm", "f16", 16384, 16384, 16384, "uniform"),
}


# (tile_dim, segment_dim_k, num_stages, num_producer_warps, num_consumer_warps) per GEMM workload
TUNED = {
    "config1_fp16_512": (64, 128, 4, 0, 8),
    "config3_fp16_8192": (256, 32, 5, 0, 8),
    "config4_fp16_2048x2048x32768": (256, 32, 5, 0, 8),
    "config5_bf16_6143x4097x3071": (256, 32, 5, 0, 8),
    "config6_fp16_16384": (256, 32, 5, 0, 8),
}


def load_package():
    name = "ckopt_amd"
    if name in sys.modules:
        return sys.modules[name]
    path = os.path.join(ROOT, "cuda-kernel-opt_amd", "__init__.py")
    spec = importlib.util.spec_from_file_location(name, path, submodule_search_locations=[os.path.dirname(path)])
    mod = importlib.util.module_from_spec(spec)
    sys.modules[name] = mod
    spec.loader.exec_module(mod)
    return mod


def mfma_ceiling(random_operands, with_loads, ksteps=400000, waves=8):
    """TFLOP/s the bare inner loop of the 256 x 256 tile GEMM sustains on the current device (no synchronisation, no
    waiting for data, no epilogue): cuda-kernel-opt_amd/lib/libckmeasure.so, a measurement aid outside the product
    library. waves: 8 (wave tiles of 64 x 128, the kernels' shape) or 4 (128 x 128, one wave per SIMD).
    int ckmeasure_mfma_ceiling_shape(int waves, int random_operands, int with_loads, int ksteps, double* tflops_out)."""
    import ctypes
    path = os.path.join(ROOT, "cuda-kernel-opt_amd", "lib", "libckmeasure.so")
    if not os.path.exists(path):
        raise RuntimeError("libckmeasure.so is not built; run `python cuda-kernel-opt_amd/build.py`")
    lib = ctypes.CDLL(path)
    lib.ckmeasure_mfma_ceiling_shape.restype = ctypes.c_int
    lib.ckmeasure_mfma_ceiling_shape.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    out = ctypes.c_double(0.0)
    rc = lib.ckmeasure_mfma_ceiling_shape(int(waves), int(bool(random_operands)), int(bool(with_loads)), int(ksteps), ctypes.byref(out))
    if rc != 0:
        raise RuntimeError("ckmeasure_mfma_ceiling_shape failed (%d)" % rc)
    return out.value


def valu_ceiling(random_operands, iters=400000):
    """TFLOP/s of the bare fp32 multiply-add stream of the matmul_shmem micro-tile on every CU (no LDS, no loads):
    int ckmeasure_valu_ceiling(int random_operands, int iters, double* tflops_out) of libckmeasure.so."""
    import ctypes
    lib = ctypes.CDLL(os.path.join(ROOT, "cuda-kernel-opt_amd", "lib", "libckmeasure.so"))
    lib.ckmeasure_valu_ceiling.restype = ctypes.c_int
    lib.ckmeasure_valu_ceiling.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    out = ctypes.c_double(0.0)
    rc = lib.ckmeasure_valu_ceiling(int(bool(random_operands)), int(iters), ctypes.byref(out))
    if rc != 0:
        raise RuntimeError("ckmeasure_valu_ceiling failed (%d)" % rc)
    return out.value


HWMON_GLOB = "/sys/class/drm/card*/device/hwmon/hwmon*"


class PowerSampler:
    """Board power of the first GPU from the amdgpu hwmon files (power1_input, microwatts; power1_cap is the limit in
    force), sampled by a thread every few milliseconds while `running` is set. Where the files cannot be read the
    sampler reports that and nothing else."""

    def __init__(self, period_s=0.005):
        import glob
        import threading
        self.period_s = period_s
        self.path = None
        self.cap_w = None
        for d in sorted(glob.glob(HWMON_GLOB)):
            f = os.path.join(d, "power1_input")
            if os.path.exists(f) and os.access(f, os.R_OK):
                self.path = f
                try:
                    self.cap_w = int(open(os.path.join(d, "power1_cap")).read()) / 1e6
                except (OSError, ValueError):
                    self.cap_w = None
                break
        self.samples = []          # (label, watts)
        self.label = None
        self._stop = threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True) if self.path else None
        if self._thread:
            self._thread.start()

    def read_w(self):
        try:
            return int(open(self.path).read()) / 1e6
        except (OSError, ValueError, TypeError):
            return None

    def _run(self):
        while not self._stop.is_set():
            label = self.label
            if label is not None:
                w = self.read_w()
                if w is not None:
                    self.samples.append((label, w))
            time.sleep(self.period_s)

    def stop(self):
        self._stop.set()
        if self._thread:
            self._thread.join()

    def summary(self, label):
        ws = sorted(w for l, w in self.samples if l == label)
        if not ws:
            return None
        return {"samples": len(ws), "mean_w": round(sum(ws) / len(ws), 1), "median_w": round(ws[len(ws) // 2], 1), "max_w": round(ws[-1], 1)}


def power_report(ck, torch, cus, stream):
    """--power: board power, the power limit in force and the shader clock while the device runs (1) the headline GEMM on
    its random operands, (2) the same launches on constant operands, (3) the bare inner loop of the same tile shape on
    random operands - each for about two seconds, after half a second of the same load. One JSON line."""
    M = N = K = 8192
    tup = ck.suggest_gemm_tuning(M, N, K, cus)
    order = [tup[k] for k in ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
                              "num_stages", "num_producer_warps", "num_consumer_warps")] + [cus]
    dd = torch.empty((M, N), dtype=torch.float32, device="cuda")
    sampler = PowerSampler()
    out = {"power_report": "fp16 8192^3, tuple %s" % (order,), "hwmon": sampler.path, "power_cap_w": sampler.cap_w,
           "idle_w": sampler.read_w() if sampler.path else None, "cases": {}}
    if not sampler.path:
        out["note"] = "no readable power1_input under %s: board power is not observable from this process" % HWMON_GLOB
    flops = 2.0 * M * N * K

    def gemm_case(name, a, b):
        da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
        step = lambda: ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da, db, None, dd, 1.0, 0.0, M, N, K, *order, stream)
        for _ in range(600):      # about half a second of the same load first
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        sampler.label = name
        e0.record(stream)
        for _ in range(2500):
            step()
        e1.record(stream)
        torch.cuda.synchronize()
        sampler.label = None
        ms = e0.elapsed_time(e1) / 2500
        cyc, ticks = ck.last_launch_clocks(stream)
        out["cases"][name] = {"launches": 2500, "ms_per_launch": round(ms, 5), "tflops": round(flops / ms * 1e-9, 1),
                              "shader_clock_mhz": round(cyc / ticks * 100.0, 1) if ticks else None, "board_power": sampler.summary(name)}

    gemm_case("gemm_random_operands", ck.fill_uniform(ck.DT_F16, (M, K), 0xC0FFEE03, 0, -1.0, 1.0), ck.fill_uniform(ck.DT_F16, (N, K), 0xC0FFEE03, 1, -1.0, 1.0))
    gemm_case("gemm_constant_operands", ck.fill_constant(ck.DT_F16, (M, K), 1.0), ck.fill_constant(ck.DT_F16, (N, K), 1.0))
    mfma_ceiling(1, 1, 1000000)   # half a second of the bare loop first
    sampler.label = "bare_inner_loop_random_operands"
    tf = mfma_ceiling(1, 1, 4000000)
    sampler.label = None
    out["cases"]["bare_inner_loop_random_operands"] = {"tflops": round(tf, 1), "board_power": sampler.summary("bare_inner_loop_random_operands")}
    sampler.stop()
    if ck.device_status() != 0:
        print("device status non-zero", file=sys.stderr)
        return 4
    print(json.dumps(out))
    return 0


def cpu_baseline(ck, kind, dtype, a, b, M, N, K, budget_s=12.0):
    """Times the CPU oracle on a bounded row sample of the same operands; returns the JSON object."""
    from oracle import oracle as o
    threads = o.lib().oracle_num_threads()

    def run(rows):
        t0 = time.perf_counter()
        if kind == "gemm":
            o.gemm(o.DT_F16 if dtype == "f16" else o.DT_BF16, a, b, rows=(0, rows), blocked=True)
        else:
            o.matmul(o.DT_F32, a, b, True, False, rows=(0, rows))
        return time.perf_counter() - t0

    rows = min(M, 16)
    dt = run(rows)
    while dt < budget_s / 4 and rows < M:
        rows = min(M, max(rows * 2, int(rows * (budget_s / 2) / max(dt, 1e-3)) // 16 * 16))
        dt = run(rows)
    tflops = 2.0 * rows * N * K / dt * 1e-12
    out = {"value": round(tflops, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
           "sample": "first %d of %d rows of the same seeded operands (%.1f s), sequential-k fp32 loop of "
                     "matmul_test.h:289-302 vectorised across output columns, %d OpenMP threads" % (rows, M, dt, threads)}
    # what the reference itself runs: its scalar check loop on one thread at its own CPU-runnable size (config 1)
    m1 = 512
    a1 = ck.fill_uniform(ck.DT_F16, (m1, m1), 0xC0FFEE01, 0, -1.0, 1.0)
    b1 = ck.fill_uniform(ck.DT_F16, (m1, m1), 0xC0FFEE01, 1, -1.0, 1.0)
    t0 = time.perf_counter()
    o.gemm(o.DT_F16, a1, b1, blocked=False, threads=1)
    dt1 = time.perf_counter() - t0
    out["single_thread_config1"] = {"value": round(2.0 * m1 ** 3 / dt1 * 1e-12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                                    "sample": "fp16 512^3, all rows, scalar loop of matmul_test.h:289-302 on one thread (%.2f s)" % dt1}
    return out


def sweep(ck, torch, args, ckdt, da, db, dd, M, N, K, cus, stream):
    """Times a list of tuning tuples: (tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
    bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps): TFLOP/s per line, the
    format of the reference's performance loops, then one JSON line with all of them and the best."""
    tuples = []
    for tile, c in ((256, 8), (128, 8), (128, 4), (64, 8), (64, 4)):
        wtr = ck.get_warp_tile_rows(tile, c)
        wave_rows = (wtr * 16, ck.get_num_acc(tile, c) // wtr * 16)
        for segk, stages, p in ((32, 5, 0), (32, 4, 0), (64, 2, 0), (128, 2, 0), (64, 2, 2), (64, 2, 4), (32, 4, 4), (64, 4, 2), (64, 4, 4), (128, 2, 2),
                                 (64, 1, 2),    # one stage with producer waves: loads and MFMAs alternate
                                 (64, 1, 0), (128, 1, 0)):   # one stage, no producers: the synchronous kernel (load, barrier, multiply,
                                                             # barrier), the no-pipeline / no-specialisation partner of every other line
            tuples.append((tile, segk, 0, 0, tile, tile, args.group, stages, p, c))
        if tile >= 128:   # the finer synchronisation granularities of port_1 / port_2 (producer/consumer kernels only)
            tuples.append((tile, 64, 2, 1, wave_rows[0], wave_rows[1], args.group, 2 if tile == 256 else 4, 2, c))
            tuples.append((tile, 64, c // 2, 2, wave_rows[0], wave_rows[1], args.group, 2 if tile == 256 else 4, 2, c))
            tuples.append((tile, 64, 1, 3 if tile == 256 or c == 4 else 1, 16, 16, args.group, 2 if tile == 256 else 4, 2, c))
    for g in (1, 2, 8):   # tile order: row-major (1) and other group sizes, on the suggested tuple
        sg = ck.suggest_gemm_tuning(M, N, K, cus)
        tuples.append((sg["tile_dim"], sg["segment_dim_k"], 0, 0, sg["bar_step_rows_a"], sg["bar_step_rows_b"], g, sg["num_stages"],
                       sg["num_producer_warps"], sg["num_consumer_warps"]))
    flops = 2.0 * M * N * K
    reps = max(args.steps // 10, 5)
    rows = []
    warm = tuples[0]   # bring the device to its steady clock before the first tuple is timed
    for _ in range(max(args.warmup, 1) * 3):
        ck.gemm_shmem_tc_async_opt_port(ckdt, da, db, None, dd, 1.0, 0.0, M, N, K, *warm, cus, stream)
    torch.cuda.synchronize()
    for t in tuples:
        if ck.check_gemm_tuning(*t, cus) != 0:
            continue
        def step():
            ck.gemm_shmem_tc_async_opt_port(ckdt, da, db, None, dd, 1.0, 0.0, M, N, K, t[0], t[1], t[2], t[3], t[4], t[5], t[6], t[7], t[8],
                                            t[9], cus, stream)
        try:
            for _ in range(3):
                step()
        except ck.CkoptError:
            continue   # no instance for this tuple
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record(stream)
        for _ in range(reps):
            step()
        ev1.record(stream)
        torch.cuda.synchronize()
        if ck.device_status() != 0:
            print("device status non-zero for %s" % (t,), file=sys.stderr)
            return 4
        tf = flops / (ev0.elapsed_time(ev1) / reps * 1e-3) * 1e-12
        print("(%s): %.2f" % (", ".join(str(v) for v in t), tf), flush=True)
        rows.append({"tuple": list(t), "tflops": round(tf, 2)})
    best = max(rows, key=lambda r: r["tflops"])
    print(json.dumps({"sweep": args.workload, "unit": "TFLOP/s", "reps": reps, "tuple_order": "tile_dim, segment_dim_k, bar_steps_a, "
                      "bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps",
                      "results": rows, "best": best}))
    return 0


GRID_SHAPES = [(512, 512, 512), (1024, 1024, 1024), (1536, 1536, 1536), (2048, 2048, 2048), (2560, 2560, 2560), (3072, 3072, 3072), (4096, 4096, 4096),
               (6144, 6144, 6144), (8192, 8192, 8192), (1024, 1024, 8192), (1024, 8192, 1024), (8192, 1024, 1024), (512, 8192, 8192), (8192, 8192, 512),
               (8192, 8192, 1024), (256, 16384, 4096), (16384, 256, 4096), (4096, 4096, 256), (2048, 2048, 32768), (1024, 1024, 65536), (2048, 4096, 16384),
               (2304, 2304, 12288), (6143, 4097, 3071), (5000, 5000, 5000), (3000, 7000, 2000), (8192, 4096, 2048), (12288, 4096, 4096), (4096, 11008, 4096),
               (2048, 8192, 8192)]


def grid(ck, torch, cus, stream):
    """fp16 products of many shapes, each on the tuple the library suggests for it, with the vendor library's GEMM
    (torch.mm, fp32 output) on the same operands beside it: one text line per shape, then one JSON line."""
    def timeit(fn, flops):
        n = max(10, int(0.02 / (flops / 1.0e15)))
        for _ in range(max(20, n // 2)):
            fn()
        torch.cuda.synchronize()
        best = None
        for _ in range(2):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for _ in range(n):
                fn()
            e1.record(stream)
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / n * 1e3
            best = us if best is None else min(best, us)
        return best
    rows = []
    for M, N, K in GRID_SHAPES:
        a = ck.fill_uniform(ck.DT_F16, (M, K), 11, 0, -1.0, 1.0)
        b = ck.fill_uniform(ck.DT_F16, (N, K), 11, 1, -1.0, 1.0)
        da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
        dd = torch.empty((M, N), dtype=torch.float32, device="cuda")
        t = ck.suggest_gemm_tuning(M, N, K, cus)
        tup = (t["tile_dim"], t["segment_dim_k"], t["bar_steps_a"], t["bar_steps_b"], t["bar_step_rows_a"], t["bar_step_rows_b"], t["tile_group_m"],
               t["num_stages"], t["num_producer_warps"], t["num_consumer_warps"])
        flops = 2.0 * M * N * K
        ours = timeit(lambda: ck.gemm_shmem_tc_async_opt_port(ck.DT_F16, da, db, None, dd, 1.0, 0.0, M, N, K, *tup, cus, stream), flops)
        tb = db.t()
        try:
            vend = timeit(lambda: torch.mm(da, tb, out_dtype=torch.float32), flops)
        except Exception:   # a torch without out_dtype
            vend = None
        if ck.device_status() != 0:
            print("device status non-zero at %s" % ((M, N, K),), file=sys.stderr)
            return 4
        row = {"M": M, "N": N, "K": K, "tuple": list(tup), "us": round(ours, 1), "tflops": round(flops / ours * 1e-6, 1),
               "vendor_us": None if vend is None else round(vend, 1), "vendor_tflops": None if vend is None else round(flops / vend * 1e-6, 1)}
        rows.append(row)
        print("%6d x %6d x %6d  (%s): %8.1f us %7.1f TFLOP/s | vendor library %s" % (
            M, N, K, ", ".join(str(v) for v in tup), ours, row["tflops"],
            "not timed" if vend is None else "%8.1f us %7.1f TFLOP/s, ours / vendor %.2f" % (vend, row["vendor_tflops"], vend / ours)), flush=True)
    print(json.dumps({"grid": "fp16, uniform[-1,1), fp32 output; suggested tuple per shape; vendor = torch.mm(A, Bt.T, out_dtype=float32)", "rows": rows}))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="config3_fp16_8192", choices=sorted(WORKLOADS))
    ap.add_argument("--shape", default=None, metavar="M,N,K",
                    help="an fp16 GEMM of this shape (uniform[-1,1) inputs) instead of a named workload, e.g. 2560,2560,2560")
    # tuning flags default to the best measured tuple of the workload (TUNED below)
    ap.add_argument("--tile", type=int, default=None)
    ap.add_argument("--segk", type=int, default=None)
    ap.add_argument("--stages", type=int, default=None)
    ap.add_argument("--producers", type=int, default=None, help="0 selects the fused (barrier-synchronised) variant")
    ap.add_argument("--consumers", type=int, default=None)
    ap.add_argument("--group", type=int, default=4)
    ap.add_argument("--mode", default="tile", choices=["tile", "wave", "acc"])
    ap.add_argument("--beta", type=float, default=0.0,
                    help="GEMM workloads: D = A Bt^T + beta C with a seeded fp32 C (the reference's own performance driver runs alpha = beta = 1, "
                         "port_2.cu:1559-1564); default 0: no C, as the configurations are stated")
    ap.add_argument("--bar-steps-a", type=int, default=0)
    ap.add_argument("--bar-steps-b", type=int, default=0)
    ap.add_argument("--cus", type=int, default=0, help="persistent grid size (default: all compute units)")
    ap.add_argument("--block-rows", type=int, default=4, help="matmul_shmem: block_rows (SIMT workload only)")
    ap.add_argument("--simt-tile", type=int, default=128)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 1 GiB device copy kernel (reads 1 GiB, writes 1 GiB): the reference "
                         "reading for FETCH_SIZE / WRITE_SIZE counter runs")
    ap.add_argument("--ceiling", action="store_true",
                    help="run only the bare inner-loop probe (libckmeasure.so): what the device sustains with "
                         "constant / random operands, without / with the direct-to-LDS loads")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the bare inner-loop probe of the headline workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE",
                    help="ckopt_set_option(KEY, VALUE) before anything is launched (e.g. 0=0: LDS swizzle off, 2=1: no XCD remap, "
                         "8=0: one barrier per loop body); repeatable")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip timing the vendor library's GEMM (hipBLASLt through torch.mm, fp32 output) on the same operands")
    ap.add_argument("--power", action="store_true",
                    help="board power (amdgpu hwmon), power limit and shader clock under the headline GEMM on random and on constant "
                         "operands and under the bare inner loop; one JSON line")
    ap.add_argument("--no-settle", action="store_true",
                    help="skip the set-up launches that bring the device to its sustained clock before warm-up")
    ap.add_argument("--grid", action="store_true",
                    help="fp16 products of many shapes on the tuple the library suggests for each, with the vendor library's GEMM beside it")
    ap.add_argument("--sweep", action="store_true",
                    help="time a list of tuning tuples on the workload (the role of the reference drivers' performance "
                         "loops, port_2.cu:1463-1480): one line per tuple in the reference's format, then one JSON line")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has one MI355X and the GEMM path has no "
              "collective; run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    if not torch.cuda.is_available():
        print("no GPU visible: bench.py needs an MI355X", file=sys.stderr)
        return 3
    ck = load_package()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.ceiling:
        res = {}
        for rnd in (0, 1):
            for loads in (0, 1):
                key = "%s_operands_%s" % ("random" if rnd else "constant", "with_loads" if loads else "no_loads")
                res[key] = round(mfma_ceiling(rnd, loads, 400000), 1)
                # the same loop with one wave per SIMD and wave tiles of 128 x 128 (a third fewer LDS bytes per MFMA)
                res["four_waves_128x128_" + key] = round(mfma_ceiling(rnd, loads, 400000, waves=4), 1)
            res["fp32_valu_%s_operands" % ("random" if rnd else "constant")] = round(valu_ceiling(rnd), 1)
        print(json.dumps({"probe": "bare inner loop of the 256x256 tile GEMM, 8 waves per CU, ~0.2 s per case",
                          "unit": "TFLOP/s", "nominal_peak": PEAK_TFLOPS["mfma_f16"], **res}))
        return 0
    if args.calibrate_copy:
        n = 1 << 28  # fp32 elements: 1 GiB
        src = torch.ones(n, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(max(args.steps, 1)):
            torch.add(src, 1.0, out=dst)  # one elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "elementwise copy kernel", "bytes_read": n * 4, "bytes_written": n * 4,
                          "launches": max(args.steps, 1)}))
        return 0
    cus = args.cus or torch.cuda.get_device_properties(0).multi_processor_count
    options = {}
    for kv in args.option:
        k, v = kv.split("=")
        ck.set_option(int(k), int(v))
        options[int(k)] = int(v)
    if args.grid:
        return grid(ck, torch, cus, torch.cuda.current_stream())
    if args.power:
        return power_report(ck, torch, cus, torch.cuda.current_stream())

    if args.shape:
        sm, sn, sk = (int(v) for v in args.shape.split(","))
        args.workload = "shape_fp16_%dx%dx%d" % (sm, sn, sk)
        WORKLOADS[args.workload] = ("gemm", "f16", sm, sn, sk, "uniform")
    kind, dtype, M, N, K, dist = WORKLOADS[args.workload]
    # tuning flags default to what the library suggests for the shape (ckopt_suggest_gemm_tuning); TUNED records
    # what that is for the named workloads and is checked against it
    sug = ck.suggest_gemm_tuning(M, N, K, cus)
    tuned = (sug["tile_dim"], sug["segment_dim_k"], sug["num_stages"], sug["num_producer_warps"], sug["num_consumer_warps"])
    if kind == "gemm" and args.workload in TUNED and tuned != TUNED[args.workload]:
        print("note: suggestion %s differs from the recorded tuple %s" % (tuned, TUNED[args.workload]), file=sys.stderr)
    for name, val in zip(("tile", "segk", "stages", "producers", "consumers"), tuned):
        if getattr(args, name) is None:
            setattr(args, name, val)
    seed = 0xC0FFEE00 + (7 if args.shape else int(args.workload[6]))
    ckdt = {"f16": ck.DT_F16, "bf16": ck.DT_BF16, "f32": ck.DT_F32}[dtype]
    if dist == "uniform":
        a = ck.fill_uniform(ckdt, (M, K), seed, 0, -1.0, 1.0)
        b = ck.fill_uniform(ckdt, (N, K), seed, 1, -1.0, 1.0)
    else:
        a = ck.fill_normal(ckdt, (M, K), seed, 0, 0.0, 0.1)
        b = ck.fill_normal(ckdt, (N, K), seed, 1, 0.0, 0.1)

    def to_dev(x):
        return torch.from_numpy(x.view(np.int16) if x.dtype == np.uint16 else x).to(dev)

    da, db = to_dev(a), to_dev(b)
    dd = torch.empty((M, N), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream()

    if kind == "gemm" and args.sweep:
        return sweep(ck, torch, args, ckdt, da, db, dd, M, N, K, cus, stream)
    if kind == "gemm":
        rows_a = rows_b = args.tile
        if args.mode == "wave":
            wtr = ck.get_warp_tile_rows(args.tile, args.consumers)
            rows_a, rows_b = wtr * 16, ck.get_num_acc(args.tile, args.consumers) // wtr * 16
        elif args.mode == "acc":
            rows_a = rows_b = 16

        c_host = ck.fill_uniform(ck.DT_F32, (M, N), seed, 2, -1.0, 1.0) if args.beta != 0.0 else None
        dc = None if c_host is None else torch.from_numpy(c_host).to(dev)

        def step():
            ck.gemm_shmem_tc_async_opt_port(ckdt, da, db, dc, dd, 1.0, args.beta, M, N, K, args.tile, args.segk,
                                            args.bar_steps_a, args.bar_steps_b, rows_a, rows_b, args.group, args.stages,
                                            args.producers, args.consumers, cus, stream)
        peak, bound_name, arith = PEAK_TFLOPS["mfma_f16"], "mfma", dtype
        if (args.producers == 0 and args.tile == 256 and args.segk == 32 and args.stages == 5 and args.consumers == 8
                and options.get(6, 1) and options.get(0, 1)):
            plan = ck.gemm_launch_plan(M, N, K, True, args.tile, args.segk, args.bar_steps_a, args.bar_steps_b, rows_a, rows_b, args.group,
                                       args.stages, args.producers, args.consumers, cus)
            kernel = "gemm_stream_kernel<%s, tile %s, five 32-deep quarters, 8 waves, pair fetch>" % (
                dtype, "256" if plan["tile_cols"] == 256 else "256 x 128")
            if plan["k_slices"] > 1:
                kernel += " with K in %d slices and a reduction pass" % plan["k_slices"]
            if plan["operand_copies"]:
                kernel += " behind zero-padded operand copies"
        elif args.producers == 0:
            kernel = "gemm_fused_kernel<%s, tile %d, seg_k %d, %d waves, workgroup barrier per segment>" % (
                dtype, args.tile, args.segk, args.consumers)
        else:
            kernel = "gemm_pc_kernel<%s, tile %d, seg_k %d, %dC+%dP waves, %s sync>" % (
                dtype, args.tile, args.segk, args.consumers, args.producers, args.mode)
    else:
        def step():
            ck.matmul_shmem(ck.DT_F32, da, db, dd, M, N, K, args.simt_tile, args.block_rows, True, stream)
        peak, bound_name, arith = PEAK_TFLOPS["valu_f32"], "valu_f32", "f32"
        kernel = "matmul_shmem_kernel<f32, tile %d, %d accumulators/thread>" % (args.simt_tile, args.simt_tile // args.block_rows)

    # Set-up, outside warm-up and the timed region: bring the device to the state a running job sees. A fresh
    # process finds the device idle at its top clock; under the matrix cores' load the power controller first
    # undershoots (launches 3 to 6 take 1.1 ms at 8192^3) and needs about 50 ms to come back to the clock it
    # then holds (0.79 ms). Batches of about 25 ms of launches are repeated until two consecutive batches agree
    # within 1 % (at least 75 ms in all).
    settle = {"launches": 0, "first_batch_ms": None, "last_batch_ms": None}
    # What a job of a few launches sees, before any of that: the first 21 launches of this process one by one. Launch 1
    # carries the runtime's first-launch work; launches 2 to 21 run on a device that comes from idle (top clock, then the
    # power controller's undershoot).
    cold = {"first_launch_ms": None, "cold_first_20_ms": None}
    sampler = PowerSampler()
    if not args.no_settle:
        cev = [torch.cuda.Event(enable_timing=True) for _ in range(22)]
        cev[0].record(stream)
        for i in range(21):
            step()
            cev[i + 1].record(stream)
        torch.cuda.synchronize()
        cold["first_launch_ms"] = round(cev[0].elapsed_time(cev[1]), 5)
        cold["cold_first_20_ms"] = round(cev[1].elapsed_time(cev[21]) / 20.0, 5)
        settle["launches"] += 21
    if not args.no_settle:
        sev0, sev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        sampler.label = "settle"

        def timed_batch(n):
            sev0.record(stream)
            for _ in range(n):
                step()
            sev1.record(stream)
            sev1.synchronize()
            settle["launches"] += n
            return sev0.elapsed_time(sev1) / n

        settle["first_batch_ms"] = round(timed_batch(4), 5)    # cold: includes the runtime's first-launch work
        cur = timed_batch(4)
        batch = max(4, min(400, int(25.0 / max(cur, 1e-3))))   # about 25 ms of launches: the controller's time scale
        prev, spent_ms = None, 0.0
        for _ in range(40):
            cur = timed_batch(batch)
            spent_ms += cur * batch
            settle["last_batch_ms"] = round(cur, 5)
            if prev is not None and spent_ms >= 75.0 and abs(cur - prev) <= 0.01 * prev:
                break
            prev = cur
        sampler.label = None

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        step()
    ev1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps   # HIP events on the launch stream; launches are back to back
    if ck.device_status() != 0:
        print("device status non-zero after the timed region: a bounded flag wait gave up", file=sys.stderr)
        return 4

    flops = 2.0 * M * N * K
    value = flops / (wall_ms * 1e-3) * 1e-12
    achieved = flops / (kern_ms * 1e-3) * 1e-12

    # after the timed region: the same launches once more with an event between every two, for the spread
    # (median, min, max of single launches), and the clock workgroup 0 of a launch actually ran at
    nper = max(5, min(args.steps, 50))
    pev = [torch.cuda.Event(enable_timing=True) for _ in range(nper + 1)]
    sampler.label = "after"
    pev[0].record(stream)
    for i in range(nper):
        step()
        pev[i + 1].record(stream)
    torch.cuda.synchronize()
    sampler.label = None
    sampler.stop()
    per = sorted(pev[i].elapsed_time(pev[i + 1]) for i in range(nper))
    launch_ms = {"n": nper, "median": round(per[nper // 2], 5), "min": round(per[0], 5), "max": round(per[-1], 5)}
    shader_mhz = None
    if kind == "gemm":
        cyc, ticks = ck.last_launch_clocks(stream)
        if ticks:
            shader_mhz = round(cyc / ticks * 100.0, 1)

    # parity check of what was just timed (oracle = checker, outside the timed region): the whole matrix where the
    # blocked oracle finishes in seconds, else the first and last rows of every tile row
    check = None
    if not args.no_check:
        from oracle import oracle as o
        got = dd.cpu().numpy()
        if 2.0 * M * N * K <= 1.2e12:
            row_sets = [(0, M)]
        else:
            row_sets = [(r, min(r + 2, M)) for r in range(0, M, 256)] + [(M - 2, M)]
        nbad, worst, nrows = 0, 0.0, 0
        for r0, r1 in row_sets:
            if kind == "gemm":
                ref = o.gemm(o.DT_F16 if dtype == "f16" else o.DT_BF16, a, b, c_host, 1.0, args.beta, rows=(r0, r1))
                nb_, w_ = o.count_outside_rel(ref, got[r0:r1], 1e-2)
            else:
                ref = o.matmul(o.DT_F32, a, b, True, False, rows=(r0, r1))
                nb_, w_ = o.count_outside_rel(ref, got[r0:r1], 1e-4)
            nbad += nb_
            worst = max(worst, w_)
            nrows += r1 - r0
        check = {"rows_checked": nrows, "of_rows": M, "outside_tolerance": nbad, "worst_ratio": round(worst, 8),
                 "tolerance": "|D-Dref| <= %g (|Dref|+1)" % (1e-2 if kind == "gemm" else 1e-4)}
        if nbad:
            print("parity check failed: %d elements outside tolerance" % nbad, file=sys.stderr)
            return 5

    traffic, traffic_commit = None, None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        try:
            tj = json.load(open(tpath))
            traffic = tj.get(args.workload)
            traffic_commit = tj.get("_commit")
        except Exception:
            traffic = None

    out = {
        "metric": "fp16_gemm_8192_tflops" if args.workload == "config3_fp16_8192" else args.workload + "_tflops",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": arith, "data": "synthetic",
        "pct_of_peak": round(100.0 * value / peak, 2),
        "config": {"workload": "%s: %s %dx%dx%d, A MxK and Bt NxK row-major, %s inputs from seed, fp32 accumulate/output"
                               % (args.workload, dtype, M, N, K, "uniform[-1,1)" if dist == "uniform" else "N(0,1)*0.1"),
                   "kernel": kernel, **({"tile_group_m": args.group, "num_stages": args.stages, "grid_cus": cus} if kind == "gemm" else
                                        {"tile_dim": args.simt_tile, "block_rows": args.block_rows, "b_transposed": True})},
        "roofline": {"bound": "mfma" if bound_name == "mfma" else "valu", "achieved": round(achieved, 2), "peak": peak,
                     "unit": "TFLOP/s", "frac": round(achieved / peak, 4), "traffic": traffic,
                     "traffic_source": None if traffic is None else "recorded: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                                       "command (profiles/hbm_traffic.json, taken at commit %s), not measured in this run" % traffic_commit,
                     "kernel_ms": round(kern_ms, 5), "flops_per_launch": flops, "launch_ms": launch_ms,
                     "shader_clock_mhz": shader_mhz,
                     # the same fraction against the peak at the clock the kernel actually ran at (nominal 2400 MHz): what the
                     # schedule achieves; frac / frac_at_measured_clock is the clock's share of the gap
                     "frac_at_measured_clock": None if not shader_mhz else round(achieved / (peak * shader_mhz / 2400.0), 4),
                     "board_power": {"cap_w": sampler.cap_w, "set_up_launches": sampler.summary("settle"), "launches_after_timed_region": sampler.summary("after"),
                                     "source": sampler.path or "no readable amdgpu hwmon power1_input",
                                     "note": "the driver's reading follows the load over about a second: phases of tens of milliseconds read low; "
                                             "`python bench.py --power` holds each load for seconds (profiles/power_config3.txt)"}},
        "setup": {"settle": settle, "cold": cold, "effective_warmup_launches": settle["launches"] + args.warmup,
                  "note": "set-up launches before warm-up, until the device holds its sustained clock; `cold` is what a fresh process sees: "
                          "launch 1 alone, then the mean of launches 2 to 21 (value at that rate: %s TFLOP/s)"
                          % (None if not cold["cold_first_20_ms"] else round(flops / cold["cold_first_20_ms"] * 1e-9, 1))},
    }
    if kind == "gemm" and args.workload == "config3_fp16_8192" and not args.no_ceiling:
        # what the bare inner loop of this tile shape sustains on this device with random operands and the
        # loads of the real data flow (no synchronisation, no waiting, no epilogue): the device's power limit
        # keeps it well below the nominal peak, and no kernel of this shape can exceed it
        try:   # a measurement aid in its own library: without it the line is printed without the ceiling
            ceil = mfma_ceiling(1, 1, 400000)
            out["roofline"]["measured_ceiling"] = round(ceil, 1)
            out["roofline"]["frac_of_measured_ceiling"] = round(achieved / ceil, 4)
        except (RuntimeError, OSError) as e:
            out["roofline"]["measured_ceiling"] = None
            print("ceiling probe not run: %s" % e, file=sys.stderr)
    if kind == "simt" and not args.no_ceiling:
        # the same for the vector ALUs: the micro-tile's multiply-add stream with random operands and nothing to feed it
        try:
            ceil = valu_ceiling(1)
            out["roofline"]["measured_ceiling"] = round(ceil, 1)
            out["roofline"]["frac_of_measured_ceiling"] = round(achieved / ceil, 4)
        except (RuntimeError, OSError) as e:
            out["roofline"]["measured_ceiling"] = None
            print("ceiling probe not run: %s" % e, file=sys.stderr)
    if kind == "gemm" and not args.no_vendor and args.beta == 0.0:
        # for orientation, outside the timed region: the vendor library's kernel for the same product on the same operands
        # (fp16 in, fp32 out), timed the same way right after ours, i.e. at the same sustained clock
        try:
            ta, tb = (da, db.t()) if dtype == "f16" else (da.view(torch.bfloat16), db.view(torch.bfloat16).t())
            for _ in range(100):   # the other kernel draws different power: let the clock find its level again
                torch.mm(ta, tb, out_dtype=torch.float32)
            vev0, vev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            vev0.record(stream)
            for _ in range(args.steps):
                vout = torch.mm(ta, tb, out_dtype=torch.float32)
            vev1.record(stream)
            torch.cuda.synchronize()
            vms = vev0.elapsed_time(vev1) / args.steps
            out["vendor_library"] = {"what": "torch.mm(A, Bt.T, out_dtype=float32) = hipBLASLt, same operands, same steps, timed right "
                                             "after the timed region", "value": round(flops / (vms * 1e-3) * 1e-12, 2), "unit": "TFLOP/s",
                                     "ms": round(vms, 5), "max_abs_diff_to_ours": round(float((vout - dd).abs().max()), 6)}
            del vout
        except Exception as e:   # an older torch without out_dtype: the comparison is simply left out
            out["vendor_library"] = {"error": repr(e)[:200]}
    if options:
        out["config"]["options"] = options
    if kind == "gemm" and args.beta != 0.0:
        out["config"]["beta"] = args.beta
    if check is not None:
        out["parity_check"] = check
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(ck, kind, dtype, a, b, M, N, K)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
