"""ctypes/numpy front end of the CPU checker in fo_oracle.c.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  The shipped package never imports it.

Arrays are numpy: 16-bit floats travel as uint16 bit patterns (`to_bits` /
`from_bits` convert), index arrays are int32.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libfo_oracle.so")

F16, BF16 = 0, 1

_u16p = ctypes.POINTER(ctypes.c_uint16)
_i32p = ctypes.POINTER(ctypes.c_int32)
_f64p = ctypes.POINTER(ctypes.c_double)


def build(force=False):
    """Compile libfo_oracle.so with the Makefile beside this file."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "fo_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libfo_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.fo_oracle_f16_to_f32.restype = ctypes.c_float
        L.fo_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.fo_oracle_bf16_to_f32.restype = ctypes.c_float
        L.fo_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.fo_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.fo_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.fo_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.fo_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.fo_oracle_interp_latency.restype = ctypes.c_double
        L.fo_oracle_interp_latency.argtypes = [_f64p, _f64p, ctypes.c_int, ctypes.c_double,
                                               ctypes.c_double]
        L.fo_oracle_predict_latency.restype = ctypes.c_double
        L.fo_oracle_predict_latency.argtypes = [
            ctypes.c_int64, ctypes.c_int64, ctypes.c_double, _f64p, _f64p, ctypes.c_int, _i32p,
            ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_double]
        L.fo_oracle_consumer_reduce.restype = None
        L.fo_oracle_consumer_reduce.argtypes = [ctypes.c_int, _u16p, _u16p, ctypes.c_int64]
        L.fo_oracle_host_schedule.argtypes = [ctypes.c_int, ctypes.c_int64, _i32p, ctypes.c_int,
                                              _i32p, _u16p, _u16p, ctypes.c_int, ctypes.c_int64]
        L.fo_oracle_gemm_signal.argtypes = [ctypes.c_int] + [ctypes.c_int] * 6 + [
            _u16p, _u16p, _u16p, _i32p, _i32p, _i32p, _i32p, ctypes.c_int, ctypes.c_int, _i32p]
        L.fo_oracle_unpermute.argtypes = [ctypes.c_int] * 5 + [_u16p, _i32p, _i32p, _u16p]
        L.fo_oracle_reorder_rmsnorm.argtypes = [ctypes.c_int, _u16p, _u16p, _u16p] + [
            ctypes.c_int] * 5 + [_i32p, ctypes.c_float]
        _lib = L
    return _lib


def _u16(a):
    return None if a is None else a.ctypes.data_as(_u16p)


def _i32(a):
    return None if a is None else a.ctypes.data_as(_i32p)


def _as_i32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int32)


# ---------------------------------------------------------------- conversions
def to_bits(x, dtype):
    """float32 ndarray -> uint16 bit patterns of fp16 (numpy RNE) or bf16 (RNE)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dtype == F16:
        with np.errstate(over="ignore"):
            return x.astype(np.float16).view(np.uint16)
    u = x.view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def from_bits(b, dtype):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    if dtype == F16:
        return b.view(np.float16).astype(np.float32)
    return (b.astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------- layout
def reorder_indices(S, hint):
    hint = _as_i32(list(hint))
    RA = np.empty(S, dtype=np.int32)
    rc = lib().fo_oracle_reorder_indices(S, _i32(hint), len(hint), _i32(RA))
    if rc:
        raise ValueError("bad hint")
    return RA


def cseg_from_waves(T, wsize):
    out = np.empty(max(1, (T + wsize - 1) // wsize), dtype=np.int32)
    G = lib().fo_oracle_cseg_from_waves(T, wsize, _i32(out))
    if G < 0:
        raise ValueError("bad T/wsize")
    return out[:G]


def row_mapping(M, N, BM, BN, cseg, W):
    cseg = _as_i32(cseg)
    RE = np.empty(M * N // BN, dtype=np.int32)
    rc = lib().fo_oracle_row_mapping(M, N, BM, BN, _i32(cseg), len(cseg), W, _i32(RE))
    if rc:
        raise ValueError("sum(cseg) must equal the tile count")
    return RE


def rows_by_world_size(M, W):
    out = np.empty(M, dtype=np.int32)
    lib().fo_oracle_rows_by_world_size(M, W, _i32(out))
    return out


def tile_group(cseg, r):
    cseg = _as_i32(cseg)
    return lib().fo_oracle_tile_group(_i32(cseg), len(cseg), int(r))


# ---------------------------------------------------------------- kernels
def gemm_signal(dtype, A, B, BM, BN, RA=None, cseg=None, rLDN=1, RE=None, MM=None,
                monitor=False, order=None):
    """A[M,K], B[N,K] uint16 bits.  Returns (C bits flat [M*N] or [M,N] if RA is None, MM)."""
    M, K = A.shape
    N = B.shape[0]
    A = np.ascontiguousarray(A, dtype=np.uint16)
    B = np.ascontiguousarray(B, dtype=np.uint16)
    C = np.zeros(M * N, dtype=np.uint16)
    RA_ = _as_i32(RA)
    RE_ = _as_i32(RE)
    cs = _as_i32(cseg)
    od = _as_i32(order)
    G = 0 if cs is None else len(cs)
    if RA_ is not None and MM is None:
        TN = N // BN
        MM = np.zeros(max(G, (M // BM + 1) * TN), dtype=np.int32)
    rc = lib().fo_oracle_gemm_signal(dtype, M, N, K, BM, BN, rLDN, _u16(A), _u16(B), _u16(C),
                                     _i32(MM), _i32(RA_), _i32(RE_), _i32(cs), G, int(monitor),
                                     _i32(od))
    if rc:
        raise ValueError(f"oracle gemm_signal rc={rc}")
    if RA_ is None:
        return C.reshape(M, N), None
    return C, MM


def unpermute(Cp, M, N, BM, BN, RA, rLDN=1, RE=None):
    Cp = np.ascontiguousarray(Cp, dtype=np.uint16)
    RA_ = _as_i32(RA)
    RE_ = _as_i32(RE)
    C = np.empty((M, N), dtype=np.uint16)
    rc = lib().fo_oracle_unpermute(M, N, BM, BN, rLDN, _u16(Cp), _i32(RA_), _i32(RE_), _u16(C))
    if rc:
        raise ValueError(f"oracle unpermute rc={rc}")
    return C


def wait_poll(expect, counter):
    """counter: int32 ndarray of length 1 (modified in place). Returns True if released."""
    return bool(lib().fo_oracle_wait_poll(int(expect), _i32(counter)))


def consumer_reduce(dtype, src, acc):
    src = np.ascontiguousarray(src, dtype=np.uint16)
    assert acc.dtype == np.uint16 and acc.flags.c_contiguous and acc.size == src.size
    lib().fo_oracle_consumer_reduce(dtype, _u16(src), _u16(acc), src.size)
    return acc


def host_schedule(dtype, tile_elems, cseg, MM, C, ACC=None, W=1, seg_stride=0):
    cs = _as_i32(cseg)
    assert MM.dtype == np.int32
    return lib().fo_oracle_host_schedule(dtype, tile_elems, _i32(cs), len(cs), _i32(MM), _u16(C),
                                         _u16(ACC), W, seg_stride)


def reorder_rmsnorm(dtype, X, Wt, bs, dim, BM=0, BN=0, rldn=1, RA=None, eps=1e-5):
    X = np.ascontiguousarray(X, dtype=np.uint16)
    Wt = np.ascontiguousarray(Wt, dtype=np.uint16)
    RA_ = _as_i32(RA)
    Y = np.empty((bs, dim), dtype=np.uint16)
    rc = lib().fo_oracle_reorder_rmsnorm(dtype, _u16(X), _u16(Y), _u16(Wt), bs, dim, BM, BN, rldn,
                                         _i32(RA_), eps)
    if rc:
        raise ValueError(f"oracle reorder_rmsnorm rc={rc}")
    return Y


def rmsnorm(dtype, X, Wt, bs, dim, eps=1e-5):
    return reorder_rmsnorm(dtype, X, Wt, bs, dim, RA=None, eps=eps)


# ---------------------------------------------------------------- tables / model
def algo_table():
    out = np.zeros((128, 12), dtype=np.int32)
    n = lib().fo_oracle_algo_table(_i32(out), 128)
    return out[:n].copy()


def interp_latency(sizes, bw, x, bytes_factor):
    s = np.ascontiguousarray(sizes, dtype=np.float64)
    b = np.ascontiguousarray(bw, dtype=np.float64)
    return lib().fo_oracle_interp_latency(s.ctypes.data_as(_f64p), b.ctypes.data_as(_f64p),
                                          len(s), float(x), float(bytes_factor))


def predict_latency(M, N, gemm_dur, sizes, bw, gp, tile_num, wave, full_wave, bytes_factor):
    s = np.ascontiguousarray(sizes, dtype=np.float64)
    b = np.ascontiguousarray(bw, dtype=np.float64)
    g = _as_i32(gp)
    return lib().fo_oracle_predict_latency(M, N, float(gemm_dur), s.ctypes.data_as(_f64p),
                                           b.ctypes.data_as(_f64p), len(s), _i32(g), len(g),
                                           tile_num, wave, full_wave, float(bytes_factor))


def compositions(n):
    out = np.zeros(n * (1 << max(0, n - 1)) + 1, dtype=np.int32)
    lens = np.zeros(1 << max(0, n - 1), dtype=np.int32)
    cnt = lib().fo_oracle_compositions(n, _i32(out), _i32(lens))
    res, pos = [], 0
    for i in range(cnt):
        res.append(out[pos:pos + lens[i]].tolist())
        pos += lens[i]
    return res
