"""Wave-group tuning for one GPU: GEMM tile candidates, completion-order hint,
consumer bandwidth curve, exhaustive and predictive search.

Counterpart of tune/gen_config.py:25-86 (GEMM candidates), tune/bandwidth.py:77-111
(size -> bandwidth curve, here of the consumer kernel instead of NCCL),
tune/search.py:83-157 (hint from monitor mode), :180-235 (latency model),
:376-385 (compositions), :387-502 (searches).  The latency model is written for
the general "communication stage with a measured bandwidth curve"; the caller
says how many bytes the stage moves per element.
"""
import numpy as np
import torch

from . import _capi, ops
from .layout import cseg_from_waves, div_up, reorder_indices, counter_size

CONSUMER_BYTES_PER_ELEM = 6.0  # read group + read accumulator + write accumulator, 16-bit each


# ------------------------------------------------------------------ model
def interpolate_latency(curve, x, bytes_per_elem=CONSUMER_BYTES_PER_ELEM):
    """ms for a stage over x elements; curve[:,0] = elements, curve[:,1] = GiB/ms,
    linear interpolation clamped at both ends (tune/search.py:180-205; there the
    byte factor is 2*2*(W-1) for all_reduce and 2*(W-1) for reduce_scatter)."""
    curve = np.asarray(curve, dtype=np.float64)
    bw = float(np.interp(float(x), curve[:, 0], curve[:, 1]))
    return float(x) * bytes_per_elem / bw / (1024 ** 3)


def predict_latency(M, N, gemm_dur, curve, gp, tile_num, wave, full_wave=None,
                    bytes_per_elem=CONSUMER_BYTES_PER_ELEM):
    """Pipeline model of tune/search.py:207-235.  `wave` = tiles per wave while the
    second stream is busy (reference: sm_count-2), `full_wave` = tiles per wave
    of the GEMM alone (reference: sm_count)."""
    full_wave = full_wave or wave
    per_tile = M * N // tile_num
    if len(gp) == 1:
        return interpolate_latency(curve, per_tile * gp[0], bytes_per_elem) + gemm_dur
    old_waves = div_up(tile_num, full_wave)
    new_waves = div_up(tile_num, wave)
    gemm = gemm_dur / old_waves * new_waves
    acc_comm = acc_comp = 0.0
    for i, g in enumerate(gp):
        comm = 0.0 if i == 0 else interpolate_latency(curve, per_tile * gp[i - 1], bytes_per_elem)
        acc_comm = max(acc_comp, acc_comm) + comm
        acc_comp += gemm / new_waves * div_up(g, wave)
    return max(acc_comp, acc_comm) + interpolate_latency(curve, per_tile * gp[-1], bytes_per_elem)


def integer_partitions(n):
    """All compositions (ordered partitions) of n, first part ascending
    (tune/search.py:376-385; 2^(n-1) of them)."""
    out = []

    def rec(rem, path):
        if rem == 0:
            out.append(path)
            return
        for i in range(1, rem + 1):
            rec(rem - i, path + [i])

    rec(n, [])
    return out


def groups_to_cseg(gp, unit, tile_num):
    """Scale a composition (in units of `unit` tiles) to tile counts; the last
    group takes what is left (tune/search.py:423-429, :484-490)."""
    cseg, acc = [], 0
    for j, g in enumerate(gp):
        if j < len(gp) - 1:
            cseg.append(g * unit)
            acc += g * unit
        else:
            cseg.append(min(g * unit, tile_num - acc))
    return cseg


def predictive_search(M, N, gemm_dur, curve, tile_num, wave, full_wave=None,
                      bytes_per_elem=CONSUMER_BYTES_PER_ELEM):
    """Best cSeg under the model (tune/search.py:442-502 without the measuring
    steps): groups are multiples of min_group = ceil(wave_num/10) waves, long
    splits with a big first group are skipped ("cold start")."""
    wave_num = div_up(tile_num, wave)
    min_group = div_up(wave_num, 10)
    best, best_dur = None, float("inf")
    for gp in integer_partitions(div_up(wave_num, min_group)):
        if len(gp) > 5 and gp[0] > 2:
            continue
        cseg = groups_to_cseg(gp, wave * min_group, tile_num)
        if min(cseg) <= 0:
            continue
        dur = predict_latency(M, N, gemm_dur, curve, cseg, tile_num, wave, full_wave, bytes_per_elem)
        if dur < best_dur:
            best, best_dur = cseg, dur
    return best, best_dur


# ------------------------------------------------------------------ measurement (GPU)
def _time_ms(fn, warmup, reps, settle_s=0.0):
    """Mean ms per call from per-call device events.  settle_s > 0 first keeps the GPU busy with
    fn for that long: for the first few dozen launches after an idle gap (allocations, host work)
    the part runs up to 30 % slower, which would otherwise decide between candidates."""
    if settle_s > 0:
        import time
        t_end = time.perf_counter() + settle_s
        while time.perf_counter() < t_end:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    end = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        start[i].record()
        fn()
        end[i].record()
    torch.cuda.synchronize()
    return float(np.mean([s.elapsed_time(e) for s, e in zip(start, end)]))


def profile_gemm_configs(M, N, K, dtype=torch.float16, top=10, warmup=10, reps=100):
    """Time every Algo whose tile divides the shape and return the stage-1 lists
    (BM, BN, dur ms, Algo) of the `top` fastest (tune/gen_config.py:25-67)."""
    A = torch.randn(M, K, device="cuda").to(dtype)
    B = torch.randn(N, K, device="cuda").to(dtype)
    C = torch.empty(M, N, device="cuda", dtype=dtype)
    rows = []
    settle = 0.3  # before the first candidate only: the candidates follow each other without a gap
    for algo, row in enumerate(_capi.algo_table()):
        if M % row[0] or N % row[1]:
            continue
        rows.append((_time_ms(lambda: ops.gemm(A, B, C, algo), warmup, reps, settle), row[0], row[1], algo))
        settle = 0.0
    rows.sort()
    rows = rows[:top]
    return [r[1] for r in rows], [r[2] for r in rows], [r[0] for r in rows], [r[3] for r in rows]


def consumer_bandwidth_curve(dtype=torch.float16, points=36, warmup=5, reps=20, link_gbps=0.0):
    """[points, 2] tensor (elements, GiB/ms) of the consumer over 2^(20+0.25 i)
    elements -- the one-GPU analogue of tune/bandwidth.py:77-111.  link_gbps > 0: the curve of the
    link-rate model (Overlap.set_link_rate), i.e. the consumer's time plus 2 n bytes / rate."""
    sizes = [int(2 ** (20 + 0.25 * i)) // 8 * 8 for i in range(points)]
    buf = torch.zeros(max(sizes), device="cuda", dtype=dtype)
    acc = torch.zeros(max(sizes), device="cuda", dtype=dtype)
    out = torch.empty(points, 2, dtype=torch.float64)
    for i, n in enumerate(sizes):
        ms = _time_ms(lambda: ops.consumer_reduce(buf[:n], acc[:n]), warmup, reps)
        if link_gbps > 0:
            ms += 2.0 * n / (link_gbps * 1e9) * 1e3
        out[i, 0] = n
        out[i, 1] = n * CONSUMER_BYTES_PER_ELEM / (1024 ** 3) / ms
    return out


def measured_hint(M, N, K, algo, wave, dtype=torch.float16, warmup=20, samples=10):
    """Completion-order hint from monitor mode with the reference's consistency
    rule: a tile belongs to wave w only if its stamp fell in
    [w*wave, (w+1)*wave) in every sample, and every wave but the last must be
    full (tune/search.py:96-157).  Returns (consistent, hint)."""
    BM, BN = _capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    cseg = cseg_from_waves(T, wave)
    if len(cseg) > TN - 1:
        raise ValueError("monitor mode needs fewer groups than tile columns")
    cseg_cpu = torch.tensor(cseg, dtype=torch.int32)
    cseg_gpu = cseg_cpu.cuda()
    A = torch.randn(M, K, device="cuda").to(dtype)
    B = torch.randn(N, K, device="cuda").to(dtype)
    C = torch.empty(M, N, device="cuda", dtype=dtype)
    MM = torch.zeros((TM + 1, TN), dtype=torch.int32, device="cuda")
    RA = torch.arange(T, dtype=torch.int32, device="cuda").reshape(TM, TN)
    ov = ops.Overlap()
    for _ in range(warmup):
        ov.gemm_allreduce_overlap(A, B, C, MM, RA, 1, cseg_cpu, cseg_gpu, algo, True)
    stamps = torch.empty((samples, T), dtype=torch.int32, device="cuda")
    for i in range(samples):
        torch.cuda.synchronize()
        MM[0] = 0
        ov.gemm_allreduce_overlap(A, B, C, MM, RA, 1, cseg_cpu, cseg_gpu, algo, True)
        torch.cuda.synchronize()
        stamps[i] = MM[1:].reshape(-1)
    ov.close()
    hint, ok = [], True
    for w in range(len(cseg)):
        inside = ((stamps >= w * wave) & (stamps < (w + 1) * wave)).sum(dim=0) == samples
        idx = torch.where(inside)[0]
        if w < len(cseg) - 1 and idx.numel() < wave:
            ok = False
            break
        hint += idx.tolist()
    return ok, hint


def time_overlap(M, N, K, algo, cseg, hint, dtype=torch.float16, warmup=20, reps=200, fused=False,
                 with_consumer=True, settle_s=0.2, link_gbps=0.0):
    """Mean ms of the overlapped call for one cSeg (tune/search.py:255-347)."""
    BM, BN = _capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    A = torch.randn(M, K, device="cuda").to(dtype)
    B = torch.randn(N, K, device="cuda").to(dtype)
    C = torch.empty(M, N, device="cuda", dtype=dtype)
    MM = torch.zeros(counter_size(len(cseg), TM, TN), dtype=torch.int32, device="cuda")
    RA = reorder_indices(TM * TN, hint).reshape(TM, TN)
    cseg_cpu = torch.tensor(cseg, dtype=torch.int32)
    cseg_gpu = cseg_cpu.cuda()
    ov = ops.Overlap()
    ov.set_fused_consumer(fused)
    ov.set_link_rate(link_gbps)
    if with_consumer:
        ov.set_accumulator(torch.zeros(M * N, device="cuda", dtype=dtype))
    if len(cseg) == 1:
        ms = _time_ms(lambda: ov.gemm_allreduce(A, B, C, algo), warmup, reps, settle_s=settle_s)
    else:
        ms = _time_ms(lambda: ov.gemm_allreduce_overlap(A, B, C, MM, RA, 1, cseg_cpu, cseg_gpu, algo),
                      warmup, reps, settle_s=settle_s)
    torch.cuda.synchronize()
    ov.close()
    return ms


def compare_overlap(M, N, K, algo, csegs, hint, dtype=torch.float16, rounds=2, reps=30, warmup=3,
                    with_consumer=True, link_gbps=0.0):
    """Median ms of the overlapped call for each cSeg of `csegs`, measured on one set of buffers with
    the candidates taking turns (`rounds` passes over all of them, `reps` timed calls each): what is
    left of clock drift and of one-off disturbances falls on all candidates alike.  For deciding
    between splits that differ by a few percent; time_overlap's mean of one run does not resolve that."""
    BM, BN = _capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    A = torch.randn(M, K, device="cuda").to(dtype)
    B = torch.randn(N, K, device="cuda").to(dtype)
    C = torch.empty(M, N, device="cuda", dtype=dtype)
    RA = reorder_indices(TM * TN, hint).reshape(TM, TN)
    MM = torch.zeros(counter_size(max(len(c) for c in csegs), TM, TN), dtype=torch.int32, device="cuda")
    ov = ops.Overlap()
    ov.set_link_rate(link_gbps)
    if with_consumer:
        ov.set_accumulator(torch.zeros(M * N, device="cuda", dtype=dtype))
    calls = []
    for cseg in csegs:
        c_cpu = torch.tensor(cseg, dtype=torch.int32)
        c_gpu = c_cpu.cuda()
        if len(cseg) == 1:
            calls.append(lambda: ov.gemm_allreduce(A, B, C, algo))
        else:
            calls.append(lambda c_cpu=c_cpu, c_gpu=c_gpu: ov.gemm_allreduce_overlap(A, B, C, MM, RA, 1, c_cpu, c_gpu, algo))
    samples = [[] for _ in csegs]
    _time_ms(calls[0], 0, 1, settle_s=0.3)
    for _ in range(rounds):
        for i, fn in enumerate(calls):
            for _ in range(warmup):
                fn()
            start = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
            end = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
            for k in range(reps):
                start[k].record()
                fn()
                end[k].record()
            torch.cuda.synchronize()
            samples[i] += [s.elapsed_time(e) for s, e in zip(start, end)]
    gave_up = ov.status()
    ov.close()
    if gave_up:
        raise RuntimeError("a device-side wait gave up while timing the overlapped call")
    return [float(np.median(x)) for x in samples]


def exhaustive_search(M, N, K, algo, wave, hint, dtype=torch.float16, reps=50, link_gbps=0.0):
    """Measure every composition of the wave count (tune/search.py:387-439)."""
    BM, BN = _capi.algo_tile(algo)
    tile_num = (M // BM) * (N // BN)
    best, best_ms, table = None, float("inf"), []
    for gp in integer_partitions(div_up(tile_num, wave)):
        cseg = groups_to_cseg(gp, wave, tile_num)
        ms = time_overlap(M, N, K, algo, cseg, hint, dtype, warmup=5, reps=reps, link_gbps=link_gbps)
        table.append((cseg, ms))
        if ms < best_ms:
            best, best_ms = cseg, ms
    return best, best_ms, table


def choose_candidate(M, N, K, BMs, BNs, algos, predictive, dtype=torch.float16, measure=None, wave_of=None,
                     order_of=None):
    """Walk down the stage-1 GEMM candidates (the first 5 for the exhaustive search, the first 10 for the
    predictive one) until monitor mode gives a hint that is consistent with the wave structure, as
    tune/search.py:397-411 and :452-468 do; the predictive search asks for consistency in units of its
    smallest group, ceil(waves / 10) waves (:462-465).  Returns (candidate index, hint, consistent).
    Where the reference gives up ("Tuning fails!"), the first candidate is taken with the order its
    persistent launch walks the tiles in, which needs no measurement.  A candidate whose group count
    leaves monitor mode no room for its order counter (groups > TN - 1) cannot be measured and is passed
    over.  measure / wave_of / order_of default to measured_hint, _capi.wave_tiles and
    _capi.schedule_order (arguments for tests)."""
    measure = measure or (lambda algo, wave: measured_hint(M, N, K, algo, wave, dtype))
    wave_of = wave_of or (lambda algo: _capi.wave_tiles(algo, M, N))
    order_of = order_of or (lambda algo: _capi.schedule_order(algo, M, N))
    for t in range(min(10 if predictive else 5, len(algos))):
        BM, BN, algo = BMs[t], BNs[t], algos[t]
        tile_num = (M // BM) * (N // BN)
        wave = wave_of(algo)
        unit = wave * div_up(div_up(tile_num, wave), 10) if predictive else wave
        if div_up(tile_num, unit) > N // BN - 1:   # monitor mode keeps its order counter at MM[TN-1]
            continue
        ok, hint = measure(algo, unit)
        if ok:
            return t, hint, True
    return 0, order_of(algos[0]), False


# ------------------------------------------------------------------ command line
def tune_shape(M, N, K, comm_op="all_reduce", predictive=False, dtype=torch.float16, directory=None,
               candidates=None, reps=100, quiet=False, link_gbps=0.0):
    """The reference's three tuning steps for one shape on one GPU, writing the same
    JSON files: GEMM candidates (tune/gen_config.py), consumer bandwidth curve
    (tune/bandwidth.py), wave-group search (tune/search.py).  Returns the solution dict.
    link_gbps > 0 tunes for the link-rate model (a collective of that algorithm bandwidth) instead of
    the consumer alone."""
    import os
    from . import config
    say = (lambda *a: None) if quiet else print
    BMs, BNs, durs, algos = profile_gemm_configs(M, N, K, dtype, top=candidates or 10, warmup=10, reps=reps)
    path = config.save_gemm_candidates(M, N, K, BMs, BNs, durs, algos, directory=directory)
    say("GEMM candidates ->", path)
    # forced for large outputs, as tune/search.py:519
    predictive = predictive or M * N > 33554432
    curve = None
    if predictive:
        curve = consumer_bandwidth_curve(dtype, link_gbps=link_gbps)
        cdir = directory or config.DEFAULT_DIR
        os.makedirs(cdir, exist_ok=True)
        torch.save(curve, os.path.join(cdir, f"bandwidth_{comm_op}_tp1.pt"))
    t, hint, consistent = choose_candidate(M, N, K, BMs, BNs, algos, predictive, dtype)
    BM, BN, dur, algo = BMs[t], BNs[t], durs[t], algos[t]
    tile_num = (M // BM) * (N // BN)
    wave = _capi.wave_tiles(algo, M, N)
    say("GEMM candidate %d (Algo %d, %dx%d): monitor-mode hint consistent with the wave structure: %s"
        % (t, algo, BM, BN, consistent))
    if predictive:
        cseg, est = predictive_search(M, N, dur, curve.numpy(), tile_num, wave)
        say("predicted latency %.4f ms for cSeg %s" % (est, cseg))
    else:
        cseg, ms, table = exhaustive_search(M, N, K, algo, wave, hint, dtype, reps=max(10, reps // 4),
                                            link_gbps=link_gbps)
        for c, c_ms in table:
            say(c, "%.4f" % c_ms)
    ms = time_overlap(M, N, K, algo, cseg, hint, dtype, warmup=10, reps=reps, link_gbps=link_gbps)
    say("searched latency %.4f ms, best cSeg %s" % (ms, cseg))
    path = config.save_solution(M, N, K, BM, BN, dur, algo, hint, cseg, directory=directory)
    say("solution ->", path)
    return config.load_solution(M, N, K, directory=directory)


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description="wave-group tuning on one GPU (tune/search.py:506-525)")
    ap.add_argument("--m", type=int, default=4096)
    ap.add_argument("--k", type=int, default=8192)
    ap.add_argument("--n", type=int, default=8192)
    ap.add_argument("--comm_op", type=str, default="all_reduce")
    ap.add_argument("--predictive_search", type=bool, default=False)  # any non-empty string is true, as in the reference
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"])
    ap.add_argument("--path", default=None, help="directory of the config JSONs")
    ap.add_argument("--link_gbps", type=float, default=0.0,
                    help="tune for a collective of this algorithm bandwidth (link-rate model) instead of the consumer alone")
    a = ap.parse_args(argv)
    tune_shape(a.m, a.n, a.k, a.comm_op, a.predictive_search,
               torch.float16 if a.dtype == "f16" else torch.bfloat16, a.path, link_gbps=a.link_gbps)


if __name__ == "__main__":
    main()
