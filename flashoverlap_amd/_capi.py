"""ctypes binding of libfo_kernels.so (the C ABI declared in include/flashoverlap.h).

There is no CPU fallback: if the library has not been built, loading raises.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB = os.path.join(_PKG, "lib", "libfo_kernels.so")
SHIM_LIB = os.path.join(_PKG, "lib", "libst_pybinding.so")

F16, BF16 = 0, 1

c_int, c_i64, c_f32, vp = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

# name -> (restype, argtypes); one entry per symbol of include/flashoverlap.h
SIGNATURES = {
    "fo_error_string": (ctypes.c_char_p, [c_int]),
    "fo_version": (c_int, []),
    "fo_algo_count": (c_int, []),
    "fo_algo_info": (c_int, [c_int, vp]),
    "fo_schedule_order": (c_int, [c_int, c_int, c_int, vp]),
    "fo_workgroup_tiles": (c_int, [c_int, c_int, c_int, vp, vp]),
    "fo_gemm_wave_tiles": (c_int, [c_int, c_int, c_int, c_int, vp]),
    "fo_gemm_kernel_info": (c_int, [c_int, c_int, c_int, c_int, c_int, vp]),
    "fo_set": (c_int, [vp, c_int, vp]),
    "fo_wait_groups": (c_int, [c_int, vp, vp, vp]),
    "fo_gemm": (c_int, [c_int, c_int, c_int, c_int, vp, vp, vp, c_int, vp]),
    "fo_gemm_signal": (c_int, [c_int, c_int, c_int, c_int, c_int, vp, c_int, vp, vp, vp, vp, vp,
                               c_int, c_int, vp]),
    "fo_gemm_scatter": (c_int, [c_int, c_int, c_int, c_int, c_int, vp, c_int, vp, vp, vp, vp, vp, vp,
                                c_int, c_int, vp]),
    "fo_wait": (c_int, [c_int, vp, vp]),
    "fo_wait_bounded": (c_int, [c_int, vp, c_i64, vp, vp]),
    "fo_consumer_reduce": (c_int, [c_int, vp, vp, c_i64, vp]),
    "fo_consumer_reduce_rs": (c_int, [c_int, vp, vp, c_i64, c_int, c_i64, vp]),
    "fo_consumer_reduce_rs_own": (c_int, [c_int, vp, vp, c_i64, c_int, c_i64, vp, c_int, vp]),
    "fo_consumer_reduce_rs_groups": (c_int, [c_int, vp, vp, vp, c_int, c_i64, c_i64, c_int, c_i64, vp, c_int, vp]),
    "fo_wait_reduce_groups": (c_int, [c_int, vp, vp, vp, vp, c_int, c_i64, c_int, c_i64, vp, c_int, vp,
                                      c_int, c_int, c_int, vp]),
    "fo_reorder_rmsnorm": (c_int, [c_int, vp, vp, vp, c_int, c_int, c_int, c_int, c_int, vp, c_f32,
                                   vp]),
    "fo_reorder_rmsnorm_rows": (c_int, [c_int, vp, vp, vp, c_int, c_int, c_int, c_int, c_int, c_int, c_int, vp, c_f32,
                                        vp]),
    "fo_norm_rows_kernel_info": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, vp]),
    "fo_rmsnorm": (c_int, [c_int, vp, vp, vp, c_int, c_int, c_f32, vp]),
    "fo_overlap_plan_batches": (c_int, [vp, c_int, c_int, vp]),
    "fo_overlap_plan_norm_rows": (c_int, [vp, c_int, c_int, vp, c_int, c_int, vp, c_int]),
    "fo_overlap_create": (c_int, [ctypes.POINTER(vp)]),
    "fo_overlap_destroy": (c_int, [vp]),
    "fo_overlap_set_gemm_stream": (c_int, [vp, vp]),
    "fo_overlap_init": (c_int, [vp]),
    "fo_overlap_set_world": (c_int, [vp, c_int, c_int]),
    "fo_overlap_set_accumulator": (c_int, [vp, vp, c_i64]),
    "fo_overlap_set_fused_consumer": (c_int, [vp, c_int]),
    "fo_overlap_set_schedule": (c_int, [vp, ctypes.c_double, c_int]),
    "fo_overlap_set_link_rate": (c_int, [vp, ctypes.c_double]),
    "fo_pace": (c_int, [c_i64, vp]),
    "fo_overlap_set_wait_limit": (c_int, [vp, c_i64]),
    "fo_overlap_status": (c_int, [vp, vp]),
    "fo_overlap_comm_stream": (vp, [vp]),
    "fo_overlap_gemm": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, c_int]),
    "fo_overlap_gemm_allreduce": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, c_int,
                                          c_int, c_int, vp, vp, c_int, c_int, c_int]),
    "fo_overlap_gemm_allreduce_norm": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp, c_int,
                                               c_int, c_int, vp, vp, c_int, c_int, c_int, vp, vp, c_f32]),
    "fo_overlap_gemm_reducescatter": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, vp,
                                              vp, c_int, c_int, c_int, vp, vp, c_int, c_int, c_int]),
    "fo_overlap_gemm_allreduce_serial": (c_int, [vp, c_int, c_int, c_int, c_int, vp, vp, vp, c_int]),
    "fo_overlap_seg_allreduce": (c_int, [vp, c_int, vp, c_i64, vp, c_int, c_int]),
    "fo_gemm_set_cu_limit": (c_int, [c_int]),
    "fo_gemm_set_row_waves": (c_int, [c_int]),
    "fo_gemm_allreduce_overlap_static": (c_int, [c_int, c_int, c_int, c_int, vp, vp, vp, vp, vp, c_int, c_int, c_int,
                                                 vp, vp, c_int, c_int, c_int, vp, vp]),
    "fo_static_status": (c_int, [vp, vp, vp]),
}

_lib = None


class FlashOverlapError(RuntimeError):
    def __init__(self, what, code):
        self.code = code
        msg = lib().fo_error_string(code).decode() if _lib is not None else "?"
        super().__init__(f"{what} failed: {msg} (code {code})")


def lib():
    """Load libfo_kernels.so once and attach the prototypes."""
    global _lib
    if _lib is None:
        if not os.path.exists(KERNEL_LIB):
            raise ImportError(
                f"{KERNEL_LIB} is missing: build it with `python -m flashoverlap_amd.build` "
                "(hipcc, gfx950). There is no CPU fallback.")
        L = ctypes.CDLL(KERNEL_LIB)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(code, what):
    if code != 0:
        raise FlashOverlapError(what, code)


def algo_table():
    """The 102 x 12 Algo table as a list of tuples."""
    L = lib()
    out = []
    buf = (ctypes.c_int32 * 12)()
    for a in range(L.fo_algo_count()):
        check(L.fo_algo_info(a, buf), "fo_algo_info")
        out.append(tuple(buf))
    return out


def algo_tile(algo):
    buf = (ctypes.c_int32 * 12)()
    check(lib().fo_algo_info(int(algo), buf), "fo_algo_info")
    return buf[0], buf[1]


def find_algo(bm, bn, swizzle=None, tbk=None, stages=None):
    """First Algo index whose (TbM, TbN[, Swizzle, TbK, Stages]) match."""
    for i, row in enumerate(algo_table()):
        if row[0] == bm and row[1] == bn and (swizzle is None or row[10] == swizzle) and (
                tbk is None or row[2] == tbk) and (stages is None or row[9] == stages):
            return i
    raise ValueError(f"no Algo with tile {bm}x{bn} swizzle={swizzle}")


def schedule_order(algo, M, N):
    """Tile ids in workgroup dispatch order (the analytic hint)."""
    bm, bn = algo_tile(algo)
    T = (M // bm) * (N // bn)
    buf = (ctypes.c_int32 * T)()
    check(lib().fo_schedule_order(int(algo), M, N, buf), "fo_schedule_order")
    return list(buf)


def set_gemm_cu_limit(n):
    """The GEMM launches count on n CUs from here on (0: on all); the schedule order, wave_tiles and
    kernel_info answer for that number, so take them again afterwards."""
    check(lib().fo_gemm_set_cu_limit(int(n)), "fo_gemm_set_cu_limit")


def set_row_waves(on):
    """Raster of the 256x256 launches: waves of whole tile rows where they fit (default) or panels only;
    the schedule order answers for the choice, so take it again afterwards."""
    check(lib().fo_gemm_set_row_waves(int(bool(on))), "fo_gemm_set_row_waves")


def wave_tiles(algo, M, N, dtype=F16):
    """Reorder tiles that complete together: resident workgroups of the persistent
    GEMM x reorder tiles per workgroup (asks the GPU for the kernel's occupancy)."""
    tiles = ctypes.c_int32()
    check(lib().fo_gemm_wave_tiles(int(dtype), int(algo), M, N, ctypes.byref(tiles)), "fo_gemm_wave_tiles")
    return tiles.value


def kernel_info(algo, M, N, epilogue=1, dtype=F16):
    """{resident workgroups, vector registers per lane, LDS bytes, threads} of the main GEMM launch
    for this problem (epilogue 0 plain, 1 signal, 2 scatter); asks the GPU."""
    info = (ctypes.c_int32 * 4)()
    check(lib().fo_gemm_kernel_info(int(dtype), int(algo), M, N, int(epilogue), info), "fo_gemm_kernel_info")
    return {"resident": info[0], "vgprs": info[1], "lds_bytes": info[2], "threads": info[3]}


def norm_rows_kernel_info(dim, reorder=True, BN=128, rldn=1, beside_gemm=True, dtype=F16):
    """{vector registers per lane, LDS bytes per workgroup} of the row-range RMSNorm kernel; asks the GPU."""
    info = (ctypes.c_int32 * 2)()
    check(lib().fo_norm_rows_kernel_info(int(dtype), int(dim), int(bool(reorder)), int(BN), int(rldn),
                                         int(bool(beside_gemm)), info), "fo_norm_rows_kernel_info")
    return {"vgprs": info[0], "lds_bytes": info[1]}


def plan_norm_rows(RA, cseg, wave_tiles):
    """Schedule of the normalisation inside gemm_allreduce_rmsnorm_overlap: list of (batch, first_tile_row,
    end_tile_row).  RA: the reorder table as a [TM, TN] array-like on the host."""
    import numpy as np
    ra = np.ascontiguousarray(np.asarray(RA, dtype=np.int32))
    TM, TN = ra.shape
    G = len(cseg)
    arr = (ctypes.c_int32 * G)(*cseg)
    runs = (ctypes.c_int32 * (3 * TM))()
    n = lib().fo_overlap_plan_norm_rows(ra.ctypes.data_as(ctypes.c_void_p), TM, TN, arr, G, int(wave_tiles), runs, TM)
    if n < 0:
        raise FlashOverlapError("fo_overlap_plan_norm_rows", n)
    return [(runs[3 * i], runs[3 * i + 1], runs[3 * i + 2]) for i in range(n)]


def plan_batches(cseg, wave_tiles):
    """Groups per launch of the per-group consumer path: list of (first_group, end_group)."""
    G = len(cseg)
    arr = (ctypes.c_int32 * G)(*cseg)
    first = (ctypes.c_int32 * (G + 1))()
    n = lib().fo_overlap_plan_batches(arr, G, int(wave_tiles), first)
    if n < 0:
        raise FlashOverlapError("fo_overlap_plan_batches", n)
    return [(first[i], first[i + 1]) for i in range(n)]
