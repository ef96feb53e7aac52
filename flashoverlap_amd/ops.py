"""torch-tensor front end of the C ABI (ctypes; tensors only provide device memory
and the current stream).  Every function enqueues on `stream` (default: torch's
current stream) and returns immediately."""
import ctypes

import torch

from . import _capi
from ._capi import F16, BF16, check, lib
from .layout import counter_size


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


def _check_signal_buffers(M, N, algo, rLDN, G, MM, RA, RE=None, monitor=False, D=None, W=1):
    """The kernels store and count through raw pointers: every buffer they index by tile, group or row
    must be large enough before anything is launched (the reference checks none of this and, with more
    groups than tile columns, writes past MM: test/test.py:94 allocates TN ints)."""
    bm, bn = _capi.algo_tile(algo)
    if M % bm or N % bn:
        raise ValueError(f"M x N = {M} x {N} is not a multiple of the Algo's tile {bm} x {bn}")
    TM, TN = M // bm, N // bn
    need = counter_size(G, TM, TN, monitor)
    if MM.numel() < need:
        raise ValueError(f"MM holds {MM.numel()} counters, {need} are needed "
                         f"({G} groups, {TM} x {TN} tiles{', monitor' if monitor else ''})")
    if RA.numel() != TM * TN:
        raise ValueError(f"RA holds {RA.numel()} entries, the problem has {TM} x {TN} tiles")
    if rLDN <= 0 or (TM * TN) % rLDN:
        raise ValueError(f"rLDN = {rLDN} does not divide the {TM * TN} tiles")
    if RE is not None and RE.numel() < M * N // (rLDN * bn):
        raise ValueError(f"RE holds {RE.numel()} rows, the reshaped output has {M * N // (rLDN * bn)}")
    if D is not None and D.numel() < M * N // W:
        raise ValueError(f"D holds {D.numel()} elements, M*N/W = {M * N // W} are needed")


def gemm(A, B, C, algo, stream=None):
    M, N, K = _mnk(A, B, C)
    check(lib().fo_gemm(dtype_code(A), M, N, K, _ptr(A, "A"), _ptr(B, "B"), _ptr(C, "C"), int(algo),
                        _stream(stream)), "fo_gemm")


def gemm_signal(A, B, C, MM, RA, cseg_dev, algo, rLDN=1, monitor=False, RE=None, stream=None):
    """Signal GEMM (RE is None) or scatter GEMM (RE given)."""
    M, N, K = _mnk(A, B, C)
    G = cseg_dev.numel()
    _check_signal_buffers(M, N, algo, int(rLDN), G, MM, RA, RE, monitor)
    common = (dtype_code(A), M, N, K, int(rLDN), _i32(cseg_dev, "cSeg"), G, _ptr(A, "A"),
              _ptr(B, "B"), _ptr(C, "C"), _i32(MM, "MM"), _i32(RA, "RA"))
    if RE is None:
        check(lib().fo_gemm_signal(*common, int(bool(monitor)), int(algo), _stream(stream)),
              "fo_gemm_signal")
    else:
        check(lib().fo_gemm_scatter(*common, _i32(RE, "RE"), int(bool(monitor)), int(algo),
                                    _stream(stream)), "fo_gemm_scatter")


def _counter_ptr(MM, index, count=1):
    if MM.dtype != torch.int32 or not MM.is_cuda:
        raise TypeError("MM must be an int32 GPU tensor")
    if index < 0 or count < 1 or index + count > MM.numel():
        raise ValueError(f"counters {index}..{index + count - 1} lie outside MM ({MM.numel()} entries)")
    return ctypes.c_void_p(MM.data_ptr() + 4 * int(index))


def wait(expect, MM, index=0, stream=None):
    check(lib().fo_wait(int(expect), _counter_ptr(MM, index), _stream(stream)), "fo_wait")


def wait_groups(cseg_dev, MM, first=0, count=None, stream=None):
    """One launch that waits for groups first..first+count-1 in turn and resets their counters."""
    count = cseg_dev.numel() - first if count is None else count
    if first < 0 or count < 1 or first + count > cseg_dev.numel():
        raise ValueError(f"groups {first}..{first + count - 1} lie outside cSeg ({cseg_dev.numel()} entries)")
    i32 = 4
    _i32(cseg_dev, "cSeg")
    check(lib().fo_wait_groups(int(count), ctypes.c_void_p(cseg_dev.data_ptr() + first * i32),
                               _counter_ptr(MM, first, count), _stream(stream)), "fo_wait_groups")


def wait_bounded(expect, MM, index, max_polls, status, stream=None):
    check(lib().fo_wait_bounded(int(expect), _counter_ptr(MM, index), int(max_polls),
                                _i32(status, "status"), _stream(stream)), "fo_wait_bounded")


def pace(nanoseconds, stream=None):
    """Holds the stream for the given time (the kernel of the link-rate model alone)."""
    check(lib().fo_pace(int(nanoseconds), _stream(stream)), "fo_pace")


def _same_dtype(*tensors):
    if len({t.dtype for t in tensors if t is not None}) > 1:
        raise TypeError("all value tensors of a call must share one dtype")


def consumer_reduce(src, acc, stream=None):
    _same_dtype(src, acc)
    if acc.numel() < src.numel():
        raise ValueError(f"acc holds {acc.numel()} elements, src {src.numel()}")
    check(lib().fo_consumer_reduce(dtype_code(src), _ptr(src, "src"), _ptr(acc, "acc"), src.numel(),
                                   _stream(stream)), "fo_consumer_reduce")


def _check_rs(src, acc, W, seg_stride, own=None):
    _same_dtype(src, acc, own)
    if W <= 0 or src.numel() % W:
        raise ValueError(f"{src.numel()} elements do not split into W = {W} chunks")
    chunk = src.numel() // W
    if acc.numel() < (W - 1) * seg_stride + chunk:
        raise ValueError(f"acc holds {acc.numel()} elements, chunk {W - 1} ends at {(W - 1) * seg_stride + chunk}")
    if own is not None and own.numel() < chunk:
        raise ValueError(f"own holds {own.numel()} elements, a chunk has {chunk}")


def consumer_reduce_rs(src, acc, W, seg_stride, stream=None):
    _check_rs(src, acc, int(W), int(seg_stride))
    check(lib().fo_consumer_reduce_rs(dtype_code(src), _ptr(src, "src"), _ptr(acc, "acc"),
                                      src.numel(), int(W), int(seg_stride), _stream(stream)),
          "fo_consumer_reduce_rs")


def consumer_reduce_rs_own(src, acc, W, seg_stride, own, rank, stream=None):
    _check_rs(src, acc, int(W), int(seg_stride), own)
    check(lib().fo_consumer_reduce_rs_own(dtype_code(src), _ptr(src, "src"), _ptr(acc, "acc"),
                                          src.numel(), int(W), int(seg_stride), _ptr(own, "own"), int(rank),
                                          _stream(stream)), "fo_consumer_reduce_rs_own")


def wait_reduce_groups(C, ACC, MM, cseg_dev, tile_elems, workspace, W=1, seg_stride=0, nblocks=0,
                       slices=0, poll_gap_ns=0, own=None, rank=0, stream=None):
    G = cseg_dev.numel()
    if MM.numel() < G:
        raise ValueError(f"MM holds {MM.numel()} counters for {G} groups")
    if workspace.numel() < 2:
        raise ValueError("workspace needs two int32 words")
    check(lib().fo_wait_reduce_groups(dtype_code(C), _ptr(C, "C"), _ptr(ACC, "ACC"), _i32(MM, "MM"),
                                      _i32(cseg_dev, "cSeg"), cseg_dev.numel(), int(tile_elems),
                                      int(W), int(seg_stride), _ptr(own, "own"),
                                      int(rank), _i32(workspace, "workspace"),
                                      int(nblocks), int(slices), int(poll_gap_ns), _stream(stream)), "fo_wait_reduce_groups")


def _check_norm(X, Y, Wt):
    _same_dtype(X, Y, Wt)
    if X.dim() != 2 or Y.numel() != X.numel() or Wt.numel() < X.shape[1]:
        raise ValueError("need X[bs, dim], Y with bs*dim elements and a weight of dim elements")


def reorder_rmsnorm(X, Y, Wt, BM, BN, rldn, RA, eps=1e-5, stream=None):
    _check_norm(X, Y, Wt)
    bs, dim = X.shape
    if BM <= 0 or BN <= 0 or bs % BM or dim % BN:
        raise ValueError(f"[{bs}, {dim}] is not a multiple of the tile {BM} x {BN}")
    if RA.numel() < (bs // BM) * (dim // BN):
        raise ValueError(f"RA holds {RA.numel()} entries, the matrix has {(bs // BM) * (dim // BN)} tiles")
    check(lib().fo_reorder_rmsnorm(dtype_code(X), _ptr(X, "X"), _ptr(Y, "Y"), _ptr(Wt, "W"), bs, dim,
                                   int(BM), int(BN), int(rldn), _i32(RA, "RA"), float(eps),
                                   _stream(stream)), "fo_reorder_rmsnorm")


def reorder_rmsnorm_rows(X, Y, Wt, row0, nrows, BM, BN, rldn, RA, eps=1e-5, stream=None):
    """Rows [row0, row0 + nrows) of reorder_rmsnorm (RA None: of rmsnorm) with the kernel that fits beside a GEMM."""
    _check_norm(X, Y, Wt)
    bs, dim = X.shape
    if row0 < 0 or nrows < 0 or row0 + nrows > bs:
        raise ValueError(f"rows {row0}..{row0 + nrows - 1} lie outside the {bs} rows of X")
    if RA is not None:
        if BM <= 0 or BN <= 0 or bs % BM or dim % BN:
            raise ValueError(f"[{bs}, {dim}] is not a multiple of the tile {BM} x {BN}")
        if RA.numel() < (bs // BM) * (dim // BN):
            raise ValueError(f"RA holds {RA.numel()} entries, the matrix has {(bs // BM) * (dim // BN)} tiles")
    check(lib().fo_reorder_rmsnorm_rows(dtype_code(X), _ptr(X, "X"), _ptr(Y, "Y"), _ptr(Wt, "W"), int(row0), int(nrows),
                                        bs, dim, int(BM), int(BN), int(rldn), None if RA is None else _i32(RA, "RA"),
                                        float(eps), _stream(stream)), "fo_reorder_rmsnorm_rows")


def rmsnorm(X, Y, Wt, eps=1e-5, stream=None):
    _check_norm(X, Y, Wt)
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

    def set_schedule(self, in_stream_below_flop=-1.0, fused_from_groups=-1):
        check(lib().fo_overlap_set_schedule(self._h, float(in_stream_below_flop), int(fused_from_groups)),
              "fo_overlap_set_schedule")

    def set_link_rate(self, gigabytes_per_second):
        """Link-rate model: every consumer launch of this handle's calls is followed by a kernel that holds
        its stream for bytes / rate, the link time of the collective it stands in for (0: off)."""
        check(lib().fo_overlap_set_link_rate(self._h, float(gigabytes_per_second)), "fo_overlap_set_link_rate")

    def set_wait_limit(self, max_polls):
        """Bound of every device-side wait of this handle's calls (-1: FO_WAIT_MAX_POLLS, 0: none)."""
        check(lib().fo_overlap_set_wait_limit(self._h, int(max_polls)), "fo_overlap_set_wait_limit")

    def status(self):
        """Synchronises both streams; 1 if a bounded wait gave up since the last query, else 0."""
        out = ctypes.c_int32(0)
        check(lib().fo_overlap_status(self._h, ctypes.byref(out)), "fo_overlap_status")
        return out.value

    def _check_call(self, A, B, C, MM, RA, rLDN, cseg_cpu, cseg_gpu, algo, monitor, RE=None, D=None):
        M, N, K = _mnk(A, B, C)
        if RA.dim() != 2:
            raise ValueError("RA must be [TM, TN]")
        if cseg_cpu.numel() != cseg_gpu.numel():
            raise ValueError("cSEG_CPU and cSEG_GPU differ in length")
        _same_dtype(A, D, self._acc)
        _check_signal_buffers(M, N, algo, int(rLDN), cseg_gpu.numel(), MM, RA, RE, monitor, D, self.world)
        if self._acc is not None and self._acc.numel() < M * N:
            raise ValueError(f"the accumulator holds {self._acc.numel()} elements, M*N = {M * N}")
        return M, N, K

    def gemm(self, A, B, C, algo):
        M, N, K = _mnk(A, B, C)
        check(lib().fo_overlap_gemm(self._h, dtype_code(A), M, N, K, _ptr(A), _ptr(B), _ptr(C),
                                    int(algo)), "fo_overlap_gemm")

    def gemm_allreduce_overlap(self, A, B, C, MM, RA, rLDN, cseg_cpu, cseg_gpu, algo,
                               monitor=False):
        M, N, K = self._check_call(A, B, C, MM, RA, rLDN, cseg_cpu, cseg_gpu, algo, monitor)
        TM, TN = RA.shape
        check(lib().fo_overlap_gemm_allreduce(
            self._h, dtype_code(A), M, N, K, _ptr(A), _ptr(B), _ptr(C), _i32(MM, "MM"),
            _i32(RA, "RA"), TM, TN, int(rLDN), _i32(cseg_cpu, "cSEG_CPU", cuda=False),
            _i32(cseg_gpu, "cSEG_GPU"), cseg_gpu.numel(), int(algo), int(bool(monitor))),
            "fo_overlap_gemm_allreduce")

    def gemm_allreduce_rmsnorm_overlap(self, A, B, C, MM, RA, RA_cpu, rLDN, cseg_cpu, cseg_gpu, algo, Y, Wt,
                                       eps=1e-5, monitor=False):
        """gemm_allreduce_overlap + reorder_rmsnorm(C -> Y) in one call: the rows are normalised on the consumer
        stream as the groups that complete them have been consumed.  RA_cpu: host copy of RA (None: copied here,
        which synchronises)."""
        M, N, K = self._check_call(A, B, C, MM, RA, rLDN, cseg_cpu, cseg_gpu, algo, monitor)
        TM, TN = RA.shape
        if RA_cpu is None:
            RA_cpu = RA.cpu()
        if RA_cpu.is_cuda or RA_cpu.numel() != RA.numel():
            raise ValueError("RA_cpu must be a host copy of RA")
        _same_dtype(A, Y, Wt)
        if Y.numel() != M * N or Wt.numel() < N:
            raise ValueError("need Y with M*N elements and a weight of N elements")
        check(lib().fo_overlap_gemm_allreduce_norm(
            self._h, dtype_code(A), M, N, K, _ptr(A), _ptr(B), _ptr(C), _i32(MM, "MM"), _i32(RA, "RA"),
            _i32(RA_cpu, "RA_cpu", cuda=False), TM, TN, int(rLDN), _i32(cseg_cpu, "cSEG_CPU", cuda=False),
            _i32(cseg_gpu, "cSEG_GPU"), cseg_gpu.numel(), int(algo), int(bool(monitor)), _ptr(Y, "Y"),
            _ptr(Wt, "W"), float(eps)), "fo_overlap_gemm_allreduce_norm")

    def gemm_reducescatter_overlap(self, A, B, C, D, MM, RA, RE, rLDN, cseg_cpu, cseg_gpu, algo,
                                   monitor=False):
        M, N, K = self._check_call(A, B, C, MM, RA, rLDN, cseg_cpu, cseg_gpu, algo, monitor, RE=RE, D=D)
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
        if self._acc is not None and self._acc.numel() < C.numel():
            raise ValueError(f"the accumulator holds {self._acc.numel()} elements, C {C.numel()}")
        check(lib().fo_overlap_seg_allreduce(self._h, dtype_code(C), _ptr(C), C.numel(),
                                             _i32(cseg_cpu, "cSEG_CPU", cuda=False),
                                             cseg_cpu.numel(), int(seg_num)),
              "fo_overlap_seg_allreduce")


def gemm_allreduce_overlap_static(A, B, C, acc, RA, rLDN, cseg_cpu, cseg_gpu, algo, fused=-1, gemm_stream=None,
                                  comm_stream=None):
    """fo_gemm_allreduce_overlap_static: the overlapped all-reduce call without a handle and without MM;
    counters and flag words live in the library's static device array, nothing is allocated.
    comm_stream None keeps the call on the GEMM stream."""
    M, N, K = _mnk(A, B, C)
    if RA.dim() != 2:
        raise ValueError("RA must be [TM, TN]")
    bm, bn = _capi.algo_tile(algo)
    if M % bm or N % bn or RA.numel() != (M // bm) * (N // bn):
        raise ValueError("RA does not match the Algo's tiling of M x N")
    if cseg_cpu.numel() != cseg_gpu.numel():
        raise ValueError("cSEG_CPU and cSEG_GPU differ in length")
    _same_dtype(A, acc)
    if acc is not None and acc.numel() < M * N:
        raise ValueError(f"the accumulator holds {acc.numel()} elements, M*N = {M * N}")
    TM, TN = RA.shape
    gs = _stream(gemm_stream)
    cs = gs if comm_stream is None else _stream(comm_stream)
    check(lib().fo_gemm_allreduce_overlap_static(
        dtype_code(A), M, N, K, _ptr(A, "A"), _ptr(B, "B"), _ptr(C, "C"), _ptr(acc, "ACC"), _i32(RA, "RA"), TM, TN,
        int(rLDN), _i32(cseg_cpu, "cSEG_CPU", cuda=False), _i32(cseg_gpu, "cSEG_GPU"), cseg_gpu.numel(), int(algo),
        int(fused), gs, cs), "fo_gemm_allreduce_overlap_static")


def static_status(gemm_stream=None, comm_stream=None):
    """Synchronises the streams of the allocation-free calls; 1 if one of their bounded waits gave up
    since the last query on this device, else 0."""
    gs = _stream(gemm_stream)
    cs = gs if comm_stream is None else _stream(comm_stream)
    out = ctypes.c_int32(0)
    check(lib().fo_static_status(gs, cs, ctypes.byref(out)), "fo_static_status")
    return out.value
