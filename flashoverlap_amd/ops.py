"""torch-tensor front end of the C ABI (ctypes; tensors only provide device memory
and the current stream).  Every function enqueues on `stream` (default: torch's
current stream) and returns immediately."""
import ctypes

import torch

from . import _capi
from ._capi import F16, BF16, check, lib


def dtype_code(t):
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"expected float16 or bfloat16, got {t.dtype}")


def _ptr(t, name="tensor", cuda=True):
    if t is None:
        return None
    if cuda and not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return ctypes.c_void_p(t.data_ptr())


def _i32(t, name, cuda=True):
    if t.dtype != torch.int32:
        raise TypeError(f"{name} must be int32")
    return _ptr(t, name, cuda)


def _stream(stream):
    if stream is None:
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, torch.cuda.Stream):
        return ctypes.c_void_p(stream.cuda_stream)
    return ctypes.c_void_p(int(stream))


def _mnk(A, B, C):
    M, K = A.shape
    N, K2 = B.shape
    if K != K2 or C.numel() != M * N or not (A.dtype == B.dtype == C.dtype):
        raise ValueError("need A[M,K], B[N,K], C with M*N elements, one dtype")
    return M, N, K


def gemm(A, B, C, algo, stream=None):
    M, N, K = _mnk(A, B, C)
    check(lib().fo_gemm(dtype_code(A), M, N, K, _ptr(A, "A"), _ptr(B, "B"), _ptr(C, "C"), int(algo),
                        _stream(stream)), "fo_gemm")


def gemm_signal(A, B, C, MM, RA, cseg_dev, algo, rLDN=1, monitor=False, RE=None, stream=None):
    """Signal GEMM (RE is None) or scatter GEMM (RE given)."""
    M, N, K = _mnk(A, B, C)
    G = cseg_dev.numel()
    common = (dtype_code(A), M, N, K, int(rLDN), _i32(cseg_dev, "cSeg"), G, _ptr(A, "A"),
              _ptr(B, "B"), _ptr(C, "C"), _i32(MM, "MM"), _i32(RA, "RA"))
    if RE is None:
        check(lib().fo_gemm_signal(*common, int(bool(monitor)), int(algo), _stream(stream)),
              "fo_gemm_signal")
    else:
        check(lib().fo_gemm_scatter(*common, _i32(RE, "RE"), int(bool(monitor)), int(algo),
                                    _stream(stream)), "fo_gemm_scatter")


def _counter_ptr(MM, index):
    if MM.dtype != torch.int32 or not MM.is_cuda:
        raise TypeError("MM must be an int32 GPU tensor")
    return ctypes.c_void_p(MM.data_ptr() + 4 * int(index))


def wait(expect, MM, index=0, stream=None):
    check(lib().fo_wait(int(expect), _counter_ptr(MM, index), _stream(stream)), "fo_wait")


def wait_groups(cseg_dev, MM, first=0, count=None, stream=None):
    """One launch that waits for groups first..first+count-1 in turn and resets their counters."""
    count = cseg_dev.numel() - first if count is None else count
    i32 = 4
    check(lib().fo_wait_groups(int(count), ctypes.c_void_p(cseg_dev.data_ptr() + first * i32),
                               _counter_ptr(MM, first), _stream(stream)), "fo_wait_groups")


def wait_bounded(expect, MM, index, max_polls, status, stream=None):
    check(lib().fo_wait_bounded(int(expect), _counter_ptr(MM, index), int(max_polls),
                                _i32(status, "status"), _stream(stream)), "fo_wait_bounded")


def consumer_reduce(src, acc, stream=None):
    check(lib().fo_consumer_reduce(dtype_code(src), _ptr(src, "src"), _ptr(acc, "acc"), src.numel(),
                                   _stream(stream)), "fo_consumer_reduce")


def consumer_reduce_rs(src, acc, W, seg_stride, stream=None):
    check(lib().fo_consumer_reduce_rs(dtype_code(src), _ptr(src, "src"), _ptr(acc, "acc"),
                                      src.numel(), int(W), int(seg_stride), _stream(stream)),
          "fo_consumer_reduce_rs")


def consumer_reduce_rs_own(src, acc, W, seg_stride, own, rank, stream=None):
    check(lib().fo_consumer_reduce_rs_own(dtype_code(src), _ptr(src, "src"), _ptr(acc, "acc"),
                                          src.numel(), int(W), int(seg_stride), _ptr(own, "own"), int(rank),
                                          _stream(stream)), "fo_consumer_reduce_rs_own")


def wait_reduce_groups(C, ACC, MM, cseg_dev, tile_elems, workspace, W=1, seg_stride=0, nblocks=0,
                       slices=0, poll_gap_ns=0, own=None, rank=0, stream=None):
    check(lib().fo_wait_reduce_groups(dtype_code(C), _ptr(C, "C"), _ptr(ACC, "ACC"), _i32(MM, "MM"),
                                      _i32(cseg_dev, "cSeg"), cseg_dev.numel(), int(tile_elems),
                                      int(W), int(seg_stride), _ptr(own, "own"),
                                      int(rank), _i32(workspace, "workspace"),
                                      int(nblocks), int(slices), int(poll_gap_ns), _stream(stream)), "fo_wait_reduce_groups")


def reorder_rmsnorm(X, Y, Wt, BM, BN, rldn, RA, eps=1e-5, stream=None):
    bs, dim = X.shape
    check(lib().fo_reorder_rmsnorm(dtype_code(X), _ptr(X, "X"), _ptr(Y, "Y"), _ptr(Wt, "W"), bs, dim,
                                   int(BM), int(BN), int(rldn), _i32(RA, "RA"), float(eps),
                                   _stream(stream)), "fo_reorder_rmsnorm")


def rmsnorm(X, Y, Wt, eps=1e-5, stream=None):
    bs, dim = X.shape
    check(lib().fo_rmsnorm(dtype_code(X), _ptr(X, "X"), _ptr(Y, "Y"), _ptr(Wt, "W"), bs, dim,
                           float(eps), _stream(stream)), "fo_rmsnorm")


class Overlap:
    """fo_overlap_t handle: the C-ABI counterpart of OverlapImpl (src/overlap_impl.h:12-43)."""

    def __init__(self, rank=0, world=1, gemm_stream=None):
        self._h = ctypes.c_void_p()
        check(lib().fo_overlap_create(ctypes.byref(self._h)), "fo_overlap_create")
        check(lib().fo_overlap_set_world(self._h, rank, world), "fo_overlap_set_world")
        check(lib().fo_overlap_set_gemm_stream(self._h, _stream(gemm_stream)),
              "fo_overlap_set_gemm_stream")
        check(lib().fo_overlap_init(self._h), "fo_overlap_init")
        self._acc = None
        self.rank, self.world = rank, world

    def close(self):
        if self._h:
            lib().fo_overlap_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def comm_stream(self):
        return lib().fo_overlap_comm_stream(self._h)

    def set_accumulator(self, acc):
        self._acc = acc
        if acc is None:
            check(lib().fo_overlap_set_accumulator(self._h, None, 0), "fo_overlap_set_accumulator")
        else:
            check(lib().fo_overlap_set_accumulator(self._h, _ptr(acc, "ACC"), acc.numel()),
                  "fo_overlap_set_accumulator")

    def set_fused_consumer(self, fused):
        check(lib().fo_overlap_set_fused_consumer(self._h, int(fused)),
              "fo_overlap_set_fused_consumer")

    def gemm(self, A, B, C, algo):
        M, N, K = _mnk(A, B, C)
        check(lib().fo_overlap_gemm(self._h, dtype_code(A), M, N, K, _ptr(A), _ptr(B), _ptr(C),
                                    int(algo)), "fo_overlap_gemm")

    def gemm_allreduce_overlap(self, A, B, C, MM, RA, rLDN, cseg_cpu, cseg_gpu, algo,
                               monitor=False):
        M, N, K = _mnk(A, B, C)
        TM, TN = RA.shape
        check(lib().fo_overlap_gemm_allreduce(
            self._h, dtype_code(A), M, N, K, _ptr(A), _ptr(B), _ptr(C), _i32(MM, "MM"),
            _i32(RA, "RA"), TM, TN, int(rLDN), _i32(cseg_cpu, "cSEG_CPU", cuda=False),
            _i32(cseg_gpu, "cSEG_GPU"), cseg_gpu.numel(), int(algo), int(bool(monitor))),
            "fo_overlap_gemm_allreduce")

    def gemm_reducescatter_overlap(self, A, B, C, D, MM, RA, RE, rLDN, cseg_cpu, cseg_gpu, algo,
                                   monitor=False):
        M, N, K = _mnk(A, B, C)
        TM, TN = RA.shape
        check(lib().fo_overlap_gemm_reducescatter(
            self._h, dtype_code(A), M, N, K, _ptr(A), _ptr(B), _ptr(C), _ptr(D), _i32(MM, "MM"),
            _i32(RA, "RA"), _i32(RE, "RE"), TM, TN, int(rLDN),
            _i32(cseg_cpu, "cSEG_CPU", cuda=False), _i32(cseg_gpu, "cSEG_GPU"), cseg_gpu.numel(),
            int(algo), int(bool(monitor))), "fo_overlap_gemm_reducescatter")

    def gemm_allreduce(self, A, B, C, algo):
        M, N, K = _mnk(A, B, C)
        check(lib().fo_overlap_gemm_allreduce_serial(self._h, dtype_code(A), M, N, K, _ptr(A),
                                                     _ptr(B), _ptr(C), int(algo)),
              "fo_overlap_gemm_allreduce_serial")

    def seg_allreduce(self, C, cseg_cpu, seg_num):
        check(lib().fo_overlap_seg_allreduce(self._h, dtype_code(C), _ptr(C), C.numel(),
                                             _i32(cseg_cpu, "cSEG_CPU", cuda=False),
                                             cseg_cpu.numel(), int(seg_num)),
              "fo_overlap_seg_allreduce")
