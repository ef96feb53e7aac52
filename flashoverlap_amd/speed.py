"""Speed table for one tuned shape on one GPU: the counterpart of test/test.py:325-372.

Reads configs/m{M}n{N}k{K}_{gpu}.json (written by `python -m flashoverlap_amd.tune`),
times the consumer alone ("comm"), the overlapped call and the non-overlapped
baseline (vendor GEMM, then the consumer over the whole output, as
BaselineImpl.gemm_allreduce / gemm_reducescatter, src/baseline_impl.cu:84-96),
and prints the reference's table.  Warm-up 20, 200 repetitions, per-call device
events, mean (test/test.py:17-18, :112-119).

    python -m flashoverlap_amd.speed --m 4096 --n 8192 --k 8192 [--comm_op reduce_scatter --world 8] [--link_gbps 200]

--link_gbps R times all three under the link-rate model (Overlap.set_link_rate): every consumer launch is
followed by bytes / R of link time, as a collective of that algorithm bandwidth would take.
"""
import argparse

import torch

from . import _capi, config, layout, ops

WARM_UP, REP = 20, 200


def _mean_ms(fn, warmup=WARM_UP, reps=REP):
    for _ in range(warmup):
        fn()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    end = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        start[i].record()
        fn()
        end[i].record()
    torch.cuda.synchronize()
    return float(torch.tensor([s.elapsed_time(e) for s, e in zip(start, end)]).mean())


def measure(M, N, K, data, comm_op="all_reduce", world=1, dtype=torch.float16, warmup=WARM_UP, reps=REP,
            link_gbps=0.0):
    """Returns (comm_ms, overlap_ms, baseline_ms) for one stage-2 config dict."""
    BM, BN, algo, cseg, hint = data["BM"], data["BN"], data["Algo"], data["cSeg"], data["hint"]
    TM, TN = M // BM, N // BN
    T = TM * TN
    rs = comm_op == "reduce_scatter"
    W = world if rs else 1
    A = torch.empty(M, K, dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5)   # test/test.py:88-89
    B = torch.empty(N, K, dtype=dtype, device="cuda").normal_(mean=0.0, std=0.5)
    C = torch.empty(M * N, dtype=dtype, device="cuda")
    ACC = torch.zeros(M * N, dtype=dtype, device="cuda")
    D = torch.empty(M // W, N, dtype=dtype, device="cuda") if rs else None
    MM = torch.zeros(layout.counter_size(len(cseg), TM, TN), dtype=torch.int32, device="cuda")
    RA = layout.reorder_indices(T, hint, device="cuda").reshape(TM, TN)
    RE = layout.generate_row_mapping(M, N, BM, BN, cseg, W, device="cuda") if rs else None
    cs_cpu = torch.tensor(cseg, dtype=torch.int32)
    cs_gpu = cs_cpu.cuda()
    ov = ops.Overlap(rank=0, world=W)
    ov.set_accumulator(ACC)
    ov.set_link_rate(link_gbps)
    seg = (M // W) * N
    link_ns = int(2.0 * M * N / link_gbps) if link_gbps > 0 else 0

    def consumer_all(src):
        if rs and W > 1:
            ops.consumer_reduce_rs(src, ACC, W, seg)
        else:
            ops.consumer_reduce(src, ACC)
        if link_ns:
            ops.pace(link_ns)

    def overlapped():
        if len(cseg) == 1:            # one group: no overlap, as test/test.py:104-133
            ov.gemm(A, B, C.view(M, N), algo)
            consumer_all(C)
        elif rs:
            ov.gemm_reducescatter_overlap(A, B, C, D, MM, RA, RE, 1, cs_cpu, cs_gpu, algo)
        else:
            ov.gemm_allreduce_overlap(A, B, C, MM, RA, 1, cs_cpu, cs_gpu, algo)

    def baseline():
        torch.matmul(A, B.t(), out=C.view(M, N))
        consumer_all(C)

    comm = _mean_ms(lambda: consumer_all(C), warmup, reps)
    over = _mean_ms(overlapped, warmup, reps)
    base = _mean_ms(baseline, warmup, reps)
    ov.close()
    return comm, over, base


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--m", type=int, default=4096)
    ap.add_argument("--k", type=int, default=8192)
    ap.add_argument("--n", type=int, default=8192)
    ap.add_argument("--comm_op", type=str, default="all_reduce")
    ap.add_argument("--world", type=int, default=8, help="chunks of the emulated reduce-scatter layout")
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"])
    ap.add_argument("--path", default=None, help="directory of the config JSONs")
    ap.add_argument("--link_gbps", type=float, default=0.0, help="link-rate model: algorithm bandwidth of the collective")
    a = ap.parse_args(argv)
    data = config.load_solution(a.m, a.n, a.k, directory=a.path)
    dtype = torch.float16 if a.dtype == "f16" else torch.bfloat16
    comm, over, base = measure(a.m, a.n, a.k, data, a.comm_op, a.world, dtype, link_gbps=a.link_gbps)
    tile_num = a.m // data["BM"] * a.n // data["BN"]
    rows = [("m", a.m), ("n", a.n), ("k", a.k), ("tile_num", tile_num),
            ("wave_tiles", _capi.wave_tiles(data["Algo"], a.m, a.n)), ("groups", len(data["cSeg"]))]
    print(f"{'Item':<18} {'Value':>15}\n{'-----':<18} {'-----':>15}")
    for k, v in rows:
        print(f"{k:<18} {v:>15}")
    for k, v in [("gemm_dur (ms)", data["dur"]), ("comm_dur (ms)", comm), ("baseline_dur (ms)", base),
                 ("overlap_dur (ms)", over), ("speedup", base / over)]:
        print(f"{k:<18} {v:>15.4f}")


if __name__ == "__main__":
    main()
