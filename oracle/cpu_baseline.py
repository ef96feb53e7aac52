"""CPU timing of the reference semantics (TEST/BENCH INFRASTRUCTURE, not product):
one rank's K-slice product as example/RowParallelLinear.py:19-20 computes it
(torch.matmul(x, W^T), here with fp32 accumulation on the host cores) followed
by RMSNorm exactly as example/RMSNorm.py:13-18.  Used only by the cpu_baseline
leg of bench.py, on a bounded row sample of the workload."""
import time

import torch


def matmul_rmsnorm(A16, B16, gamma16, eps):
    C = (A16.float() @ B16.float().t()).to(A16.dtype)
    x = C.float()
    y = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)).type_as(C) * gamma16
    return C, y


def time_sample(A16, B16, gamma16, eps, target_seconds=15.0):
    """Times matmul+RMSNorm on the first `rows` rows of A, rows chosen from a
    128-row probe so that the timed call does about target_seconds of work."""
    M, K = A16.shape
    N = B16.shape[0]
    probe = min(128, M)
    matmul_rmsnorm(A16[:probe], B16, gamma16, eps)           # warm-up (thread pool, caches)
    t0 = time.perf_counter()
    matmul_rmsnorm(A16[:probe], B16, gamma16, eps)
    dt = max(time.perf_counter() - t0, 1e-6)
    rows = int(min(M, max(probe, probe * target_seconds / dt)))
    rows -= rows % probe
    # a fast host finishes the whole matrix early: repeat the pass until the
    # sample holds about target_seconds of work
    passes = 0
    t0 = time.perf_counter()
    while True:
        matmul_rmsnorm(A16[:rows], B16, gamma16, eps)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= target_seconds * 0.8:
            break
    return {"rows": rows, "passes": passes, "seconds": dt, "flops": 2.0 * passes * rows * N * K,
            "threads": torch.get_num_threads()}
