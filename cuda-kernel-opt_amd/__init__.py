"""Python host side of the MI355X GEMM hot path: a ctypes binding of lib/libckopt.so.

The functions mirror the reference's host launchers (same names, parameter order and meaning;
matmul_shmem.cu:143-152, matmul_shmem_tc_async_opt_port_{0,1,2}.cu launchers) and raise CkoptError
where the reference asserts. They take raw device pointers (ints), so any allocator works; torch
tensors are accepted for convenience and only their data_ptr() is used.

The directory name contains a hyphen, so load it with importlib (see __graft_entry__.load_package()).
There is no CPU fallback: if the HIP library is missing, importing this module fails.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# CKOPT_LIB selects another build of the same library (e.g. a measurement variant)
LIB_PATH = os.environ.get("CKOPT_LIB") or os.path.join(HERE, "lib", "libckopt.so")

DT_F16, DT_BF16, DT_F32, DT_I32 = 0, 1, 2, 3
OK, ERR_BAD_PARAM, ERR_LDS_BUDGET, ERR_NO_INSTANCE, ERR_HIP, ERR_ALIGNMENT, ERR_NULL, ERR_TOO_LARGE = 0, -1, -2, -3, -4, -5, -6, -7
OPT_SWIZZLE, OPT_SPIN_LIMIT, OPT_NUM_XCD, OPT_PRIO_MODE, OPT_PRODUCER_NAP, OPT_TILE_SYNC_BARRIER, OPT_STRAIGHT_LINE, OPT_SPLIT_K, OPT_BARRIER_EVERY_KSTEP = 0, 1, 2, 3, 4, 5, 6, 7, 8
OPT_EVEN_ROUNDS = 9
OPT_TAIL_ROUND = 12       # the partly filled last round of the straight-line kernel as K-sliced items of the same launch (default 1)
OPT_FUSED_REDUCTION = 13  # K slices are added inside the straight-line kernel: 1 where possible and estimated cheaper (default), 2 wherever possible, 0 never
OPT_BATCHED_EMPTY_READS = 14  # wave-tile granularity: producers read all "released" counters of a stage in one look (default 1)
OPT_HALF_WIDTH = 11  # tile width of the straight-line kernel: 0 always 256 x 256, 1 what the cost model prefers (default), 2 always 256 x 128, 3 always 256 x 192
OPT_D_STORE_POLICY = 10  # 0: non-temporal stores of D where its rows lie on 128-byte lines (default), 1: always, 2: never

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libckopt.so is not built (%s); run `python cuda-kernel-opt_amd/build.py` - there is no CPU fallback" % LIB_PATH)

_lib = ctypes.CDLL(LIB_PATH)
_i, _f, _p, _i64, _u64 = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64

_lib.ckopt_gemm_shmem_tc_async_opt_port_2.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_2.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 14 + [_p]
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_lp.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_lp.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 14 + [_p]
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_noalloc.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_noalloc.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 14 + [_p]
_lib.ckopt_gemm_workspace_bytes.restype = _i64
_lib.ckopt_gemm_workspace_bytes.argtypes = [_i] * 15
_lib.ckopt_gemm_launch_plan.restype = _i
_lib.ckopt_gemm_launch_plan.argtypes = [_i] * 15 + [ctypes.POINTER(ctypes.c_int)]


class LaunchOptions(ctypes.Structure):
    """ckopt_launch_options: the launch options as a per-call argument (fields = the ckopt_set_option keys in order)."""
    _fields_ = [(n, ctypes.c_int) for n in (
        "struct_bytes", "lds_swizzle", "spin_limit", "num_xcd", "prio_mode", "producer_nap", "tile_sync_barrier", "straight_line",
        "split_k", "barrier_every_kstep", "even_rounds", "d_store_policy", "half_width", "tail_round", "fused_reduction", "batched_empty_reads")]


_lib.ckopt_launch_options_init.restype = _i
_lib.ckopt_launch_options_init.argtypes = [ctypes.POINTER(LaunchOptions)]
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_ex.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_ex.argtypes = [_i, _i, _p, _p, _p, _p, _f, _f] + [_i] * 14 + [ctypes.POINTER(LaunchOptions), _p, ctypes.c_size_t, _p]
_lib.ckopt_gemm_workspace_bytes_ex.restype = _i64
_lib.ckopt_gemm_workspace_bytes_ex.argtypes = [_i] * 15 + [ctypes.POINTER(LaunchOptions)]
_lib.ckopt_gemm_launch_plan_ex.restype = _i
_lib.ckopt_gemm_launch_plan_ex.argtypes = [_i] * 15 + [ctypes.POINTER(LaunchOptions), ctypes.POINTER(ctypes.c_int)]
_lib.ckopt_gemm_shmem_tc_async_opt_port_1_lp.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_1_lp.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 12 + [_p]
_lib.ckopt_gemm_shmem_tc_async_opt_port_0_lp.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_0_lp.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 10 + [_p]
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_ws.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_2_ws.argtypes = [_i, _i, _p, _p, _p, _p, _f, _f] + [_i] * 14 + [_p, ctypes.c_size_t, _p]
_lib.ckopt_gemm_shmem_tc_async_opt_port_1.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_1.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 12 + [_p]
_lib.ckopt_gemm_shmem_tc_async_opt_port_0.restype = _i
_lib.ckopt_gemm_shmem_tc_async_opt_port_0.argtypes = [_i, _p, _p, _p, _p, _f, _f] + [_i] * 10 + [_p]
_lib.ckopt_get_lds_req.restype = _i
_lib.ckopt_get_lds_req.argtypes = [_i] * 8
_lib.ckopt_get_num_acc.restype = _i
_lib.ckopt_get_num_acc.argtypes = [_i, _i]
_lib.ckopt_get_warp_tile_rows.restype = _i
_lib.ckopt_get_warp_tile_rows.argtypes = [_i, _i]
_lib.ckopt_get_tile_offset_cd.restype = _i64
_lib.ckopt_get_tile_offset_cd.argtypes = [_i, _i, _i, _i, _i64]
_lib.ckopt_check_gemm_tuning.restype = _i
_lib.ckopt_check_gemm_tuning.argtypes = [_i] * 11
_lib.ckopt_matmul_shmem.restype = _i
_lib.ckopt_matmul_shmem.argtypes = [_i, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p]
_lib.ckopt_matmul_shmem_lds_req.restype = _i
_lib.ckopt_matmul_shmem_lds_req.argtypes = [_i, _i]
_lib.ckopt_check_matmul_shmem_tuning.restype = _i
_lib.ckopt_check_matmul_shmem_tuning.argtypes = [_i, _i]
_lib.ckopt_trim_scratch_pool.restype = _i
_lib.ckopt_trim_scratch_pool.argtypes = [ctypes.c_size_t]
_lib.ckopt_device_status.restype = _i
_lib.ckopt_device_status.argtypes = [_p]
_lib.ckopt_last_launch_clocks.restype = _i
_lib.ckopt_last_launch_clocks.argtypes = [_p, ctypes.POINTER(_u64), ctypes.POINTER(_u64)]
_lib.ckopt_suggest_gemm_tuning.restype = _i
_lib.ckopt_suggest_gemm_tuning.argtypes = [_i, _i, _i, _i, ctypes.POINTER(ctypes.c_int)]
_lib.ckopt_set_option.restype = _i
_lib.ckopt_set_option.argtypes = [_i, _i]
_lib.ckopt_fill_uniform.restype = _i
_lib.ckopt_fill_uniform.argtypes = [_i, _p, _i64, _u64, _u64, _f, _f]
_lib.ckopt_fill_normal.restype = _i
_lib.ckopt_fill_normal.argtypes = [_i, _p, _i64, _u64, _u64, _f, _f]
_lib.ckopt_fill_int.restype = _i
_lib.ckopt_fill_int.argtypes = [_i, _p, _i64, _u64, _u64, _i, _i]
_lib.ckopt_fill_constant.restype = _i
_lib.ckopt_fill_constant.argtypes = [_i, _p, _i64, _f]
_lib.ckopt_error_string.restype = ctypes.c_char_p
_lib.ckopt_error_string.argtypes = [_i]

EXPORTED_SYMBOLS = [
    "ckopt_gemm_shmem_tc_async_opt_port_2", "ckopt_gemm_shmem_tc_async_opt_port_2_lp", "ckopt_gemm_shmem_tc_async_opt_port_2_noalloc",
    "ckopt_gemm_workspace_bytes", "ckopt_gemm_launch_plan", "ckopt_gemm_shmem_tc_async_opt_port_2_ws",
    "ckopt_launch_options_init", "ckopt_gemm_shmem_tc_async_opt_port_2_ex", "ckopt_gemm_workspace_bytes_ex", "ckopt_gemm_launch_plan_ex",
    "ckopt_gemm_shmem_tc_async_opt_port_1", "ckopt_gemm_shmem_tc_async_opt_port_1_lp",
    "ckopt_gemm_shmem_tc_async_opt_port_0", "ckopt_gemm_shmem_tc_async_opt_port_0_lp", "ckopt_get_lds_req", "ckopt_get_num_acc", "ckopt_get_warp_tile_rows",
    "ckopt_get_tile_offset_cd", "ckopt_check_gemm_tuning", "ckopt_matmul_shmem", "ckopt_matmul_shmem_lds_req",
    "ckopt_check_matmul_shmem_tuning", "ckopt_device_status", "ckopt_last_launch_clocks", "ckopt_trim_scratch_pool",
    "ckopt_suggest_gemm_tuning",
    "ckopt_set_option", "ckopt_fill_uniform",
    "ckopt_fill_normal", "ckopt_fill_int", "ckopt_fill_constant", "ckopt_error_string",
]


class CkoptError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__("%s: %s (%d)" % (where, error_string(code), code))


def error_string(code):
    return _lib.ckopt_error_string(code).decode()


def _check(code, where):
    if code != OK:
        raise CkoptError(code, where)


def _dptr(x):
    if x is None:
        return None
    if isinstance(x, int):
        return ctypes.c_void_p(x)
    return ctypes.c_void_p(x.data_ptr())  # torch tensor


def _stream(stream):
    if stream is None:
        return None
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)  # torch.cuda.Stream


def get_num_acc(tile_dim, num_consumer_waves):
    r = _lib.ckopt_get_num_acc(tile_dim, num_consumer_waves)
    if r < 0:
        raise CkoptError(r, "get_num_acc")
    return r


def get_warp_tile_rows(tile_dim, num_consumer_waves):
    r = _lib.ckopt_get_warp_tile_rows(tile_dim, num_consumer_waves)
    if r < 0:
        raise CkoptError(r, "get_warp_tile_rows")
    return r


def get_tile_offset_cd(M, N, tile_dim, tile_group_m, tile_count):
    r = _lib.ckopt_get_tile_offset_cd(M, N, tile_dim, tile_group_m, tile_count)
    if r < 0:
        raise CkoptError(int(r), "get_tile_offset_cd")
    return int(r)


def get_lds_req(tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, num_stages,
                num_consumer_waves):
    """Role of the reference's get_shmem_req (port_2.cu:1057-1066)."""
    r = _lib.ckopt_get_lds_req(tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b,
                               num_stages, num_consumer_waves)
    if r < 0:
        raise CkoptError(r, "get_lds_req")
    return r


def check_gemm_tuning(tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m,
                      num_stages, num_producer_waves, num_consumer_waves, num_cus):
    return _lib.ckopt_check_gemm_tuning(tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
                                        bar_step_rows_b, tile_group_m, num_stages, num_producer_waves,
                                        num_consumer_waves, num_cus)


def gemm_shmem_tc_async_opt_port(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
                                 bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
                                 num_producer_warps, num_consumer_warps, num_sms, stream=None):
    """port_2 launcher (matmul_shmem_tc_async_opt_port_2.cu:1088-1109). B is passed transposed (N x K)."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_2(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
        bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
        num_consumer_warps, num_sms, _stream(stream)), "gemm_shmem_tc_async_opt_port")


def gemm_shmem_tc_async_opt_port_lp(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
                                    bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
                                    num_producer_warps, num_consumer_warps, num_sms, stream=None):
    """The <half, half> instance of the port_2 launcher (port_2.cu:968-1055): C and D in the operands' 16-bit type."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_2_lp(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
        bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
        num_consumer_warps, num_sms, _stream(stream)), "gemm_shmem_tc_async_opt_port <DT, DT>")


def gemm_workspace_bytes(M, N, K, operands_aligned, tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
                         bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, options=None):
    """Bytes of caller-owned workspace gemm_shmem_tc_async_opt_port_ws / _ex needs for this launch (0: none)."""
    r = _lib.ckopt_gemm_workspace_bytes_ex(M, N, K, int(bool(operands_aligned)), tile_dim, segment_dim_k, bar_steps_a, bar_steps_b,
                                           bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
                                           num_consumer_warps, num_sms, _optr(options))
    if r < 0:
        raise CkoptError(int(r), "gemm_workspace_bytes")
    return int(r)


def launch_options(**fields):
    """The process-wide default options as a LaunchOptions value, with the given fields replaced."""
    o = LaunchOptions()
    _check(_lib.ckopt_launch_options_init(ctypes.byref(o)), "launch_options_init")
    for k, v in fields.items():
        if k not in dict(LaunchOptions._fields_) or k == "struct_bytes":
            raise KeyError(k)
        setattr(o, k, int(v))
    return o


def _optr(options):
    return None if options is None else ctypes.byref(options)


def gemm_launch_plan(M, N, K, operands_aligned, tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
                     bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, options=None):
    """What the launch will run: dict(straight_line, tile_cols, k_slices, operand_copies, sliced_tiles, reduced_in_kernel, grid)."""
    out = (ctypes.c_int * 7)()
    _check(_lib.ckopt_gemm_launch_plan_ex(M, N, K, int(bool(operands_aligned)), tile_dim, segment_dim_k, bar_steps_a, bar_steps_b,
                                          bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
                                          num_consumer_warps, num_sms, _optr(options), out), "gemm_launch_plan")
    return dict(straight_line=bool(out[0]), tile_cols=int(out[1]), k_slices=int(out[2]), operand_copies=bool(out[3]),
                sliced_tiles=int(out[4]), reduced_in_kernel=bool(out[5]), grid=int(out[6]))


def gemm_shmem_tc_async_opt_port_ex(dtype, cd_dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
                                    bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
                                    num_producer_warps, num_consumer_warps, num_sms, options=None, workspace=None, workspace_bytes=0,
                                    stream=None):
    """The port_2 launcher with its options as an argument (a LaunchOptions; None: the process-wide defaults) and,
    optionally, a caller-owned workspace (None: stream-ordered allocations)."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_2_ex(
        dtype, cd_dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
        bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps,
        num_sms, _optr(options), _dptr(workspace), int(workspace_bytes), _stream(stream)), "gemm_shmem_tc_async_opt_port (options)")


def gemm_shmem_tc_async_opt_port_ws(dtype, cd_dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
                                    bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
                                    num_producer_warps, num_consumer_warps, num_sms, workspace, workspace_bytes, stream=None):
    """The port_2 launcher on a caller-owned workspace (nothing is allocated); cd_dtype DT_F32 or the operands' type."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_2_ws(
        dtype, cd_dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
        bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps,
        num_sms, _dptr(workspace), int(workspace_bytes), _stream(stream)), "gemm_shmem_tc_async_opt_port (workspace)")


NOALLOC_SCRATCH_BYTES = 64 << 20


def gemm_shmem_tc_async_opt_port_noalloc(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
                                         bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
                                         num_producer_warps, num_consumer_warps, num_sms, stream=None):
    """The port_2 launcher for callers that cannot allocate: operand copies and split-K planes in the library's
    static device array of NOALLOC_SCRATCH_BYTES; raises CkoptError(ERR_TOO_LARGE) beyond it."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_2_noalloc(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_steps_a,
        bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
        num_consumer_warps, num_sms, _stream(stream)), "gemm_shmem_tc_async_opt_port (no allocation)")


def gemm_shmem_tc_async_opt_port_1(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_step_rows_a,
                                   bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps,
                                   num_sms, stream=None):
    """port_1 launcher (matmul_shmem_tc_async_opt_port_1.cu:889-908)."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_1(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_step_rows_a,
        bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, _stream(stream)),
        "gemm_shmem_tc_async_opt_port_1")


def gemm_shmem_tc_async_opt_port_0(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, tile_group_m,
                                   num_stages, num_producer_warps, num_consumer_warps, num_sms, stream=None):
    """port_0 launcher (matmul_shmem_tc_async_opt_port_0.cu:515-532)."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_0(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, tile_group_m,
        num_stages, num_producer_warps, num_consumer_warps, num_sms, _stream(stream)), "gemm_shmem_tc_async_opt_port_0")


def gemm_shmem_tc_async_opt_port_1_lp(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_step_rows_a,
                                      bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps,
                                      num_sms, stream=None):
    """The <half, half> instance of the port_1 launcher (port_1.cu:1292, :1332): C and D in the operands' 16-bit type."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_1_lp(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_step_rows_a,
        bar_step_rows_b, tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, _stream(stream)),
        "gemm_shmem_tc_async_opt_port_1 <DT, DT>")


def gemm_shmem_tc_async_opt_port_0_lp(dtype, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, tile_group_m,
                                      num_stages, num_producer_warps, num_consumer_warps, num_sms, stream=None):
    """The <half, half> instance of the port_0 launcher (port_0.cu:866, :906)."""
    _check(_lib.ckopt_gemm_shmem_tc_async_opt_port_0_lp(
        dtype, _dptr(A), _dptr(B), _dptr(C), _dptr(D), alpha, beta, M, N, K, tile_dim, segment_dim_k, tile_group_m,
        num_stages, num_producer_warps, num_consumer_warps, num_sms, _stream(stream)), "gemm_shmem_tc_async_opt_port_0 <DT, DT>")


def matmul_shmem(dtype, A, B, C, M, N, K, tile_dim, block_rows, b_transposed=False, stream=None):
    """matmul_shmem launcher (matmul_shmem.cu:143-152); b_transposed selects an N x K B."""
    _check(_lib.ckopt_matmul_shmem(dtype, _dptr(A), _dptr(B), _dptr(C), M, N, K, tile_dim, block_rows,
                                   int(b_transposed), _stream(stream)), "matmul_shmem")


def matmul_shmem_lds_req(dtype, tile_dim):
    r = _lib.ckopt_matmul_shmem_lds_req(dtype, tile_dim)
    if r < 0:
        raise CkoptError(r, "matmul_shmem_lds_req")
    return r


def check_matmul_shmem_tuning(tile_dim, block_rows):
    return _lib.ckopt_check_matmul_shmem_tuning(tile_dim, block_rows)


def trim_scratch_pool(keep_bytes=0):
    """Hands back what the library's stream-ordered scratch pool of the current device holds beyond keep_bytes."""
    _check(_lib.ckopt_trim_scratch_pool(int(keep_bytes)), "trim_scratch_pool")


def device_status(stream=None):
    """Synchronises `stream` and returns (and clears) the device status word; raises on HIP errors."""
    r = _lib.ckopt_device_status(_stream(stream))
    if r < 0:
        raise CkoptError(r, "device_status")
    return r


def last_launch_clocks(stream=None):
    """(shader cycles, 100 MHz reference ticks) workgroup 0 of the last GEMM launch ran for."""
    c, w = _u64(0), _u64(0)
    _check(_lib.ckopt_last_launch_clocks(_stream(stream), ctypes.byref(c), ctypes.byref(w)), "last_launch_clocks")
    return int(c.value), int(w.value)


def suggest_gemm_tuning(M, N, K, num_cus=256):
    """Tuning tuple for a problem size: dict with the launcher's parameter names."""
    out = (ctypes.c_int * 10)()
    _check(_lib.ckopt_suggest_gemm_tuning(M, N, K, num_cus, out), "suggest_gemm_tuning")
    names = ("tile_dim", "segment_dim_k", "bar_steps_a", "bar_steps_b", "bar_step_rows_a", "bar_step_rows_b", "tile_group_m",
             "num_stages", "num_producer_warps", "num_consumer_warps")
    d = dict(zip(names, [int(v) for v in out]))
    d["num_sms"] = num_cus
    return d


def set_option(key, value):
    r = _lib.ckopt_set_option(key, value)
    if r < 0:
        raise CkoptError(r, "set_option")
    return r


# ---- seeded host inputs (numpy arrays; 16-bit types are returned as float16 / uint16 bit patterns) ----
def _np_dtype(dtype):
    import numpy as np
    return {DT_F16: np.float16, DT_BF16: np.uint16, DT_F32: np.float32, DT_I32: np.int32}[dtype]


def _fill(fn, dtype, shape, *args):
    import numpy as np
    out = np.empty(shape, dtype=_np_dtype(dtype))
    _check(fn(dtype, out.ctypes.data_as(ctypes.c_void_p), out.size, *args), fn.__name__)
    return out


def fill_uniform(dtype, shape, seed, stream_id, lo=-1.0, hi=1.0):
    return _fill(_lib.ckopt_fill_uniform, dtype, shape, seed, stream_id, lo, hi)


def fill_normal(dtype, shape, seed, stream_id, mean=0.0, stddev=1.0):
    return _fill(_lib.ckopt_fill_normal, dtype, shape, seed, stream_id, mean, stddev)


def fill_int(dtype, shape, seed, stream_id, lo, hi_inclusive):
    return _fill(_lib.ckopt_fill_int, dtype, shape, seed, stream_id, lo, hi_inclusive)


def fill_constant(dtype, shape, value):
    return _fill(_lib.ckopt_fill_constant, dtype, shape, value)
