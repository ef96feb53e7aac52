"""One-GPU benchmark of the overlap hot path.

A step = one pass of the hot path over one synthetic batch: GEMM + tile signal +
reordered store on the GEMM stream, per-group wait + consumer on the second
stream followed there by reorder+RMSNorm of the rows each wave completed, join.  Workload: the large-square configuration the
headline metric is quoted on (fp16, M=N=K=8192, 128x256 tiles, wave groups of
256 tiles).  Prints one JSON line; `value` is GEMM flops / step time.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c2|c3|c4] [--dtype f16|bf16]

The default run (c5) appends compact records of the c2, c3 and c4 workloads as `other_workloads`.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2516.6   # MI355X dense fp16/bf16 MFMA
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch of the signal GEMM, from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/gemm_c5_hbm_traffic.md (FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000, factors from a 256 MiB copy).
MEASURED_TRAFFIC_BYTES = {("c5", "f16"): 788738.0 * 1024 * 2.0 + 131104.0 * 1024}
# From the counter run summarised in profiles/gemm_c5_mfma_utilisation.md (rocprofv3 --pmc GRBM_GUI_ACTIVE
# SQ_VALU_MFMA_BUSY_CYCLES ...): shader cycles per launch of the signal GEMM (GRBM_GUI_ACTIVE / 8 XCDs) and the
# share of them in which a SIMD's matrix pipe was busy.  Cycles per launch do not depend on the clock, so this
# run's launch time turns them into the clock the kernel ran at: what the part sustains under its power limit,
# against the 2.4 GHz the nominal peak assumes.
MEASURED_GEMM_COUNTERS = {("c5", "f16"): {"cycles_per_launch": 1.3496e6, "mfma_util": 0.777}}


class PowerSampler:
    """Socket power of the GPU from the amdgpu hwmon files (power1_average or power1_input, microwatts;
    power1_cap is the limit), read every 10 ms by a thread while a leg loops.  None where the files are
    missing or unreadable."""

    def __init__(self):
        import glob
        self.path = self.cap_w = self.sclk_path = self.last_sclk_mhz = None
        for h in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*")):
            for name in ("power1_average", "power1_input"):
                f = os.path.join(h, name)
                try:
                    int(open(f).read())
                except (OSError, ValueError):
                    continue
                self.path = f
                try:
                    self.cap_w = int(open(os.path.join(h, "power1_cap")).read()) / 1e6
                except (OSError, ValueError):
                    pass
                self.sclk_path = os.path.join(os.path.dirname(os.path.dirname(h)), "pp_dpm_sclk")
                return

    def sclk_mhz(self):
        """The shader clock level the driver marks as current ('1: 1782Mhz *'), or None."""
        try:
            for line in open(self.sclk_path):
                if "*" in line:
                    return float(line.split(":")[1].lower().split("mhz")[0])
        except (OSError, ValueError, IndexError, AttributeError):
            pass
        return None

    def watts_while(self, fn, seconds, launches_per_sync=50, skip_seconds=0.5):
        """Mean power while fn loops for `seconds` (the first skip_seconds are left out), and ms per launch."""
        import threading
        import torch
        samples, clocks, stop = [], [], threading.Event()

        def sampler():
            k = 0
            while not stop.is_set():
                try:
                    samples.append((time.perf_counter(), int(open(self.path).read())))
                except (OSError, ValueError):
                    pass
                if k % 10 == 5:
                    clocks.append((time.perf_counter(), self.sclk_mhz()))
                k += 1
                time.sleep(0.01)
        th = threading.Thread(target=sampler, daemon=True)
        t0 = time.perf_counter()
        if self.path:
            th.start()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = 0
        e0.record()
        while time.perf_counter() < t0 + seconds:
            for _ in range(launches_per_sync):
                fn()
            n += launches_per_sync
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        stop.set()
        if self.path:
            th.join()
        w = [v for (t, v) in samples if t0 + skip_seconds <= t <= t1]
        c = [v for (t, v) in clocks if t0 + skip_seconds <= t <= t1 and v]
        self.last_sclk_mhz = sum(c) / len(c) if c else None
        return (sum(w) / len(w) / 1e6 if w else None), e0.elapsed_time(e1) / n

WORKLOADS = {
    # name: (M, N, K, BM, BN, dtype, group tiles, W, description)
    "c5": (8192, 8192, 8192, 128, 256, "f16", 256, 0, "large square fp16 8192^3, 128x256 tiles, wave groups of 256 tiles"),
    "c2": (4096, 4096, 512, 128, 128, "f16", 4, 0, "row-parallel K-slice fp16 4096x4096x512, 128x128 tiles, groups of 4 tiles"),
    "c3": (8192, 8192, 3584, 256, 128, "bf16", 512, 0, "MLP down-projection bf16 8192x8192x3584, 256x128 tiles"),
    "c4": (8192, 4096, 4096, 128, 128, "f16", 256, 8, "reduce-scatter layout fp16 8192x4096x4096, 8 row-chunk segments"),
}


def measure(args, workload, compact=False):
    """Time one workload.  compact: the core figures only (the default run reports the other
    BASELINE workloads this way, next to the full record of the headline one)."""
    import torch
    import flashoverlap_amd as fo
    from flashoverlap_amd import ops

    M, N, K, BM, BN, dt, gtiles, W, desc = WORKLOADS[workload]
    gtiles = (args.group_tiles if not compact else 0) or gtiles
    dt = (args.dtype if not compact else None) or dt
    td = torch.float16 if dt == "f16" else torch.bfloat16
    algo = fo._capi.find_algo(BM, BN, swizzle=args.swizzle)
    TM, TN = M // BM, N // BN
    T = TM * TN
    if args.comm_cus and not compact and not args.group_tiles:
        gtiles = fo._capi.wave_tiles(algo, M, N)  # one group per GEMM wave, whatever the CU limit makes of a wave
    if workload == "c3" and (compact or not args.group_tiles):
        # wave-group sizes chosen by the predictive search (tune/search.py:442-502) from a measured
        # GEMM duration and the consumer's measured bandwidth curve
        from flashoverlap_amd import tune
        Ap = torch.randn(M, K, device="cuda").to(td)
        Bp = torch.randn(N, K, device="cuda").to(td)
        Cpp = torch.empty(M, N, device="cuda", dtype=td)
        dur = tune._time_ms(lambda: ops.gemm(Ap, Bp, Cpp, algo), 10, 20)
        curve = tune.consumer_bandwidth_curve(td, points=36, warmup=2, reps=5).numpy()
        cseg, _ = tune.predictive_search(M, N, dur, curve, T, fo._capi.wave_tiles(algo, M, N))
        del Ap, Bp, Cpp
    else:
        cseg = fo.layout.cseg_from_waves(T, gtiles)
    hint = fo._capi.schedule_order(algo, M, N)
    RA = fo.layout.reorder_indices(T, hint, device="cuda").reshape(TM, TN)
    RE = fo.layout.generate_row_mapping(M, N, BM, BN, cseg, W, device="cuda") if W else None

    g = torch.Generator().manual_seed(0)
    if workload == "c5":
        A16 = ((torch.rand(M, K, generator=g) * 2 - 1) * K ** -0.5).to(td)
        B16 = ((torch.rand(N, K, generator=g) * 2 - 1) * K ** -0.5).to(td)
    else:
        A32 = torch.randn(M, K, generator=g)
        if workload == "c3":  # 5 % outlier columns scaled x8
            cols = torch.randperm(K, generator=g)[: (K * 5 + 99) // 100]
            A32[:, cols] *= 8
        A16 = A32.to(td)
        B16 = (torch.randn(N, K, generator=g) * K ** -0.5).to(td)
    gamma16 = (1 + 0.01 * torch.randn(N, generator=g)).to(td)
    A, B, gamma = A16.cuda(), B16.cuda(), gamma16.cuda()
    Cp = torch.empty(M * N, device="cuda", dtype=td)
    Cplain = torch.empty(M, N, device="cuda", dtype=td)
    ACC = torch.zeros(M * N, device="cuda", dtype=td)
    D = torch.empty(M // W, N, device="cuda", dtype=td) if W else None
    bs = M // W if W else M
    Y = torch.empty(bs, N, device="cuda", dtype=td)
    MM = torch.zeros(fo.layout.counter_size(len(cseg), TM, TN), dtype=torch.int32, device="cuda")
    cs_cpu = torch.tensor(cseg, dtype=torch.int32)
    cs_gpu = cs_cpu.cuda()
    eps = 1e-6

    ov = ops.Overlap(rank=0, world=max(W, 1))
    ov.set_accumulator(ACC)
    ov.set_fused_consumer(args.fused)

    def norm():
        if W:  # RMSNorm on segment 0 only
            ops.reorder_rmsnorm(ACC.view(W, bs, N)[0], Y, gamma, BM // W, BN, 1, RA, eps=eps)
        else:
            ops.reorder_rmsnorm(Cp.view(M, N), Y, gamma, BM, BN, 1, RA, eps=eps)

    RA_cpu = RA.cpu()

    def step_overlapped():
        # all-reduce layout: one call, the rows normalised on the consumer stream behind each wave's consumer;
        # reduce-scatter layout: the overlapped call, then the normalisation of segment 0
        if W:
            ov.gemm_reducescatter_overlap(A, B, Cp, D, MM, RA, RE, 1, cs_cpu, cs_gpu, algo)
            norm()
        else:
            ov.gemm_allreduce_rmsnorm_overlap(A, B, Cp, MM, RA, RA_cpu, 1, cs_cpu, cs_gpu, algo, Y, gamma, eps=eps)

    def step_pair():  # the reference's two calls: overlapped GEMM + collective, then reorder_rmsnorm behind the join
        ov.gemm_allreduce_overlap(A, B, Cp, MM, RA, 1, cs_cpu, cs_gpu, algo)
        norm()

    def step_serial():  # signal-free GEMM, whole-C consumer, plain RMSNorm, one stream
        ops.gemm(A, B, Cplain, algo)
        if W:
            ops.consumer_reduce_rs(Cplain.view(-1), ACC, W, (M // W) * N)
            ops.rmsnorm(ACC.view(W, bs, N)[0], Y, gamma, eps=eps)
        else:
            ops.consumer_reduce(Cplain.view(-1), ACC)
            ops.rmsnorm(Cplain, Y, gamma, eps=eps)

    def gemm_alone():
        ops.gemm(A, B, Cplain, algo)

    def gemm_signal_alone():  # counters are not consumed here; cleared afterwards
        ops.gemm_signal(A, B, Cp, MM, RA, cs_gpu, algo, RE=RE)

    def consumer_alone():
        ops.consumer_reduce(Cp, ACC)

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return e0.elapsed_time(e1) / steps, wall

    # Bring the part to its sustained clocks first: for the first few dozen launches after idle
    # the same GEMM runs up to 30 % slower, which would otherwise fall on whatever is timed first.
    def settle(fn, seconds=0.5):
        t_end = time.perf_counter() + seconds
        while time.perf_counter() < t_end:
            for _ in range(20):
                fn()
            torch.cuda.synchronize()

    K_, W_ = (max(5, args.steps // 2), max(3, args.warmup // 2)) if compact else (args.steps, args.warmup)
    if args.steps_only and not compact and args.comm_cus:
        # CU-masked streams: the consumer's stream may use comm_cus CUs (the mask's low bits), the GEMM's
        # all of them or, with --gemm-cus-disjoint, the others (the library was told to plan for that
        # many in main()).  The call that takes both streams from the caller is the one without a handle.
        import ctypes
        if W:
            raise SystemExit("--comm-cus: all-reduce workloads only")
        hip = ctypes.CDLL("libamdhip64.so")
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        nw = (cus + 31) // 32

        def masked_stream(bits):
            words = (ctypes.c_uint32 * nw)(*[(bits >> (32 * i)) & 0xFFFFFFFF for i in range(nw)])
            s = ctypes.c_void_p()
            rc = hip.hipExtStreamCreateWithCUMask(ctypes.byref(s), nw, words)
            if rc:
                raise SystemExit(f"hipExtStreamCreateWithCUMask: error {rc}")
            return torch.cuda.ExternalStream(s.value)

        comm_bits = (1 << args.comm_cus) - 1
        comm_s = masked_stream(comm_bits)
        gemm_s = masked_stream(((1 << cus) - 1) & ~comm_bits) if args.gemm_cus_disjoint else torch.cuda.Stream()
        torch.cuda.synchronize()

        def step_masked():
            ops.gemm_allreduce_overlap_static(A, B, Cp, ACC, RA, 1, cs_cpu, cs_gpu, algo, fused=args.fused,
                                              gemm_stream=gemm_s, comm_stream=comm_s)
            norm()

        ev_g, ev_c = torch.cuda.Event(), torch.cuda.Event()

        def serial_masked():
            # the same consumer on the same few CUs with nothing overlapped: GEMM, whole-C consumer, RMSNorm.
            # With a consumer this slow (a link-like rate instead of the 7 TB/s of all CUs) the schedule has
            # something to hide: test/test.py:325-371 compares the same two on a real interconnect.
            ops.gemm(A, B, Cplain, algo)
            ev_g.record(gemm_s)
            comm_s.wait_event(ev_g)
            ops.consumer_reduce(Cplain.view(-1), ACC, stream=comm_s)
            ev_c.record(comm_s)
            gemm_s.wait_event(ev_c)
            ops.rmsnorm(Cplain, Y, gamma, eps=eps)

        with torch.cuda.stream(gemm_s):
            settle(gemm_alone)
            ms_g, _ = timed(gemm_alone, K_, W_)
            ms, _ = timed(step_masked, K_, W_)
            ms_s, _ = timed(serial_masked, K_, W_)
            ms2, _ = timed(step_masked, K_, W_)
        with torch.cuda.stream(comm_s):
            ms_c, _ = timed(consumer_alone, max(3, K_ // 4), 1)
        assert ops.static_status(gemm_s, comm_s) == 0, "a device-side wait gave up: the step ran on incomplete tiles"
        print(json.dumps({"steps_only": True, "steps": K_, "warmup": W_, "comm_cus": args.comm_cus,
                          "gemm_cus": cus - args.comm_cus if args.gemm_cus_disjoint else cus,
                          "wave_tiles": fo._capi.wave_tiles(algo, M, N), "cseg": cseg,
                          "gemm_alone_ms": ms_g, "ms_per_step": min(ms, ms2), "serial_ms": ms_s,
                          "overlapped_vs_serial": min(ms, ms2) / ms_s,
                          "consumer_GBps_on_its_cus": 6.0 * M * N / (ms_c * 1e-3) / 1e9}))
        return
    if args.steps_only and not compact:
        ms, _ = timed(step_overlapped, K_, W_)
        print(json.dumps({"steps_only": True, "steps": K_, "warmup": W_, "ms_per_step": ms}))
        return
    if args.kernels_only and not compact:
        fns = (gemm_alone, gemm_signal_alone, consumer_alone, norm)
        if args.vendor_gemm:
            fns += (lambda: torch.matmul(A, B.t(), out=Cplain),)
        for fn in fns:
            timed(fn, K_, W_)
            MM.zero_()
        torch.cuda.synchronize()
        print(json.dumps({"kernels_only": True, "steps": K_, "warmup": W_}))
        return
    settle(step_serial, 0.25 if compact else 0.5)
    # The ratios asked for are differences of one to ten percent between runs that drift by as much over a
    # second: overlapped step, serial step, GEMM alone and signal GEMM take turns in `blocks` rounds of
    # W_ + K_ launches each, and every figure is the median of its blocks.
    import statistics
    blocks = 3 if compact else args.blocks
    legs = {"overlapped": step_overlapped, "serial": step_serial, "gemm": gemm_alone, "signal": gemm_signal_alone}
    if not W:
        legs["pair"] = step_pair
    samples = {k: [] for k in legs}
    wall_step = 0.0
    for _ in range(blocks):
        for name, fn in legs.items():
            ms, wall = timed(fn, K_, W_)
            samples[name].append(ms)
            if name == "overlapped":
                wall_step = wall
            if name == "signal":
                MM.zero_()
    med = {k: statistics.median(v) for k, v in samples.items()}
    ms_step, ms_serial, ms_gemm, ms_signal = med["overlapped"], med["serial"], med["gemm"], med["signal"]
    ms_pair = med.get("pair")
    # the vendor library's GEMM on the same operands, same process and clocks: a yardstick only
    def vendor_gemm():
        torch.matmul(A, B.t(), out=Cplain)
    ms_vendor, _ = timed(vendor_gemm, K_, W_)
    # the two bandwidth-bound kernels last tens of microseconds: 200 launches or more per figure, so that the
    # first launch's start-up (several microseconds after a synchronisation) does not weigh on the average
    ms_consumer, _ = timed(consumer_alone, max(200, K_), W_)
    ms_norm, _ = timed(norm, max(200, K_), W_)
    ACC.zero_()
    torch.cuda.synchronize()

    flops = 2.0 * M * N * K
    if compact:
        gave_up = ov.status()
        ov.close()
        return {"workload": f"{workload}: {desc}", "dtype": dt, "cseg": cseg if len(cseg) <= 16 else f"{len(cseg)} x {cseg[0]}",
                "gemm_alone_ms": ms_gemm, "gemm_signal_ms": ms_signal, "frac": flops / (ms_signal * 1e-3) / 1e12 / PEAK_TFLOPS,
                "overlapped_ms": ms_step, "serial_ms": ms_serial, "two_calls_ms": ms_pair, "blocks": blocks,
                "overlapped_vs_gemm_alone": ms_step / ms_gemm, "overlapped_vs_serial": ms_step / ms_serial,
                "consumer_GBps": 6.0 * M * N / (ms_consumer * 1e-3) / 1e9,
                "reorder_rmsnorm_GBps": (4.0 * bs * N + 2.0 * N) / (ms_norm * 1e-3) / 1e9,
                "vendor_gemm_ms": ms_vendor, "waits_gave_up": gave_up}

    # wave-group-size sweep (large square only): group sizes in waves of 256 tiles;
    # 8 and 16 waves are a single group, i.e. the serial path (test/test.py:104)
    sweep = []
    if workload == "c5" and not args.no_group_sweep:
        # group sizes in waves of 256 tiles (one tile per CU, the reference's wave); this GEMM completes 512 of these
        # tiles at a time, and groups that complete together share their launches.  The candidates take turns in
        # three rounds; medians.
        cands = []
        for waves in (1, 2, 4, 8, 16):
            cs = fo.layout.cseg_from_waves(T, 256 * waves)
            if len(cs) == 1:
                sweep.append({"waves_per_group": waves, "groups": 1, "ms": ms_serial, "path": "serial"})
                continue
            c_cpu = torch.tensor(cs, dtype=torch.int32)
            cands.append((waves, cs, c_cpu, c_cpu.cuda(), []))
        for _ in range(3):
            for waves, cs, c_cpu, c_gpu, acc_ms in cands:
                acc_ms.append(timed(lambda: ov.gemm_allreduce_rmsnorm_overlap(A, B, Cp, MM, RA, RA_cpu, 1, c_cpu, c_gpu, algo, Y,
                                                                              gamma, eps=eps), K_, W_)[0])
        for waves, cs, c_cpu, c_gpu, acc_ms in cands:
            ms_g = statistics.median(acc_ms)
            sweep.append({"waves_per_group": waves, "groups": len(cs), "ms": ms_g, "path": "overlapped",
                          "vs_serial": ms_g / ms_serial, "vs_gemm_alone": ms_g / ms_gemm})
        sweep.sort(key=lambda e: e["waves_per_group"])
        ACC.zero_()
        torch.cuda.synchronize()

    # Link-rate model (large square only).  The stand-in consumer runs at HBM speed; the collective it stands in for
    # is bound by the links.  With a rate set on the handle every consumer launch is followed by a kernel that holds
    # its stream for bytes / rate (algorithm bandwidth: message bytes / time of the collective), in the overlapped
    # step behind each wave's consumer, in the serial step behind the whole-C consumer: the comparison of
    # test/test.py:325-371 with the link time modelled instead of measured.  Alternating rounds, medians.
    link_model = []
    rates = [float(x) for x in args.link_gbps.split(",") if x] if workload == "c5" and not W and not args.no_group_sweep else []
    for rate in rates:
        ns_all = int(2.0 * M * N / rate)

        def serial_link():
            ops.gemm(A, B, Cplain, algo)
            ops.consumer_reduce(Cplain.view(-1), ACC)
            ops.pace(ns_all)
            ops.rmsnorm(Cplain, Y, gamma, eps=eps)

        ov.set_link_rate(rate)
        sl = {"overlapped": [], "serial": []}
        for _ in range(3):
            sl["overlapped"].append(timed(step_overlapped, K_, W_)[0])
            sl["serial"].append(timed(serial_link, K_, W_)[0])
        ov.set_link_rate(0)
        mo, msr = statistics.median(sl["overlapped"]), statistics.median(sl["serial"])
        link_model.append({"link_GBps": rate, "link_ms_whole_C": ns_all * 1e-6, "overlapped_ms": mo, "serial_ms": msr,
                           "overlapped_vs_serial": mo / msr, "speedup": msr / mo})
    if rates:
        ACC.zero_()
        torch.cuda.synchronize()

    # Power (large square only): the GEMM runs at the board's power limit, which is what holds its clock
    # below the 2.4 GHz of the nominal peak, and an overlapped step cannot finish before the energy of all its
    # kernels has been delivered at that limit.  Each leg loops for 1.5 s while a thread reads the socket power.
    power = None
    if workload == "c5" and not args.no_group_sweep and not W:
        ps = PowerSampler()
        if ps.path:
            pw = {}
            for name, fn, per_sync in (("gemm_signal", gemm_signal_alone, 50), ("consumer", consumer_alone, 400),
                                       ("reorder_rmsnorm", norm, 400), ("overlapped_step", step_overlapped, 50),
                                       ("serial_step", step_serial, 50)):
                watts, ms = ps.watts_while(fn, 1.5, per_sync)
                MM.zero_()
                pw[name] = {"watts": watts, "ms": ms, "sclk_mhz": ps.last_sclk_mhz}
            time.sleep(0.3)
            idle_w, _ = ps.watts_while(lambda: None, 0.6, 1, skip_seconds=0.2)
            power = {"source": ps.path, "cap_w": ps.cap_w, "idle_w": idle_w, "legs": pw}
            if all(v["watts"] for v in pw.values()) and ps.cap_w:
                # energy above idle of the three kernels run one after the other, delivered at the limit
                dyn = sum((pw[k]["watts"] - idle_w) * pw[k]["ms"] for k in ("gemm_signal", "consumer", "reorder_rmsnorm"))
                power["overlapped_step_bound_ms"] = dyn / (ps.cap_w - idle_w)
                power["bound"] = ("(sum over GEMM, consumer, reorder+RMSNorm of (watts - idle) x ms) / (cap - idle): no "
                                  "schedule of these three kernels finishes sooner at this power limit")
            ACC.zero_()
            torch.cuda.synchronize()

    # bf16 repeat of the large square: the same step with bf16 operands
    bf16_repeat = None
    if workload == "c5" and dt == "f16" and not args.no_group_sweep:
        tb = torch.bfloat16
        Ab, Bb, gb = A16.float().to(tb).cuda(), B16.float().to(tb).cuda(), gamma16.float().to(tb).cuda()
        Cb = torch.empty(M * N, device="cuda", dtype=tb)
        Cbp = torch.empty(M, N, device="cuda", dtype=tb)
        ACCb = torch.zeros(M * N, device="cuda", dtype=tb)
        Yb = torch.empty(M, N, device="cuda", dtype=tb)
        ov.set_accumulator(ACCb)

        def step_b():
            ov.gemm_allreduce_rmsnorm_overlap(Ab, Bb, Cb, MM, RA, RA_cpu, 1, cs_cpu, cs_gpu, algo, Yb, gb, eps=eps)

        def serial_b():
            ops.gemm(Ab, Bb, Cbp, algo)
            ops.consumer_reduce(Cbp.view(-1), ACCb)
            ops.rmsnorm(Cbp, Yb, gb, eps=eps)

        def signal_b():
            ops.gemm_signal(Ab, Bb, Cb, MM, RA, cs_gpu, algo)
        settle(serial_b, 0.3)  # the allocations above left the GPU idle
        sb = {"step": [], "serial": [], "signal": []}
        for _ in range(3):
            sb["step"].append(timed(step_b, K_, W_)[0])
            sb["serial"].append(timed(serial_b, K_, W_)[0])
            sb["signal"].append(timed(signal_b, K_, W_)[0])
            MM.zero_()
        ms_b, ms_sb, ms_gb = (statistics.median(sb[k]) for k in ("step", "serial", "signal"))
        torch.cuda.synchronize()
        bf16_repeat = {"overlapped_step_ms": ms_b, "serial_step_ms": ms_sb, "gemm_signal_alone_ms": ms_gb,
                       "gemm_signal_TFLOPs": 2.0 * M * N * K / (ms_gb * 1e-3) / 1e12,
                       "overlapped_vs_serial": ms_b / ms_sb}
        ov.set_accumulator(ACC)
        del Ab, Bb, Cb, Cbp, ACCb, Yb

    achieved = flops / (ms_signal * 1e-3) / 1e12
    out = {
        "metric": "GEMM+signal+reorder TFLOP/s (% MFMA peak); overlapped vs serial time, 1 GPU",
        "value": flops / (ms_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": K_, "warmup": W_,
        "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{workload}: {desc}", "M": M, "N": N, "K": K, "tile": [BM, BN],
                   "groups": len(cseg), "cseg": cseg if len(cseg) <= 16 else f"{len(cseg)} x {cseg[0]}", "algo": algo,
                   "consumer_launches": "on the GEMM stream behind the GEMM (automatic choice for a GEMM this short)"
                   if (args.fused < 0 and 2.0 * M * N * K < 6.4e10)
                   else "one wait and one consumer launch per GEMM wave" if (args.fused == 0 or (args.fused < 0 and len(cseg) <= 16))
                   else "one"},
        "roofline": {"bound": "mfma", "kernel": "fo_gemm256_kernel (signal epilogue)",
                     "achieved": achieved, "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_TFLOPS,
                     "mfma_util": MEASURED_GEMM_COUNTERS.get((workload, dt), {}).get("mfma_util"),
                     "clock_ghz": (MEASURED_GEMM_COUNTERS[(workload, dt)]["cycles_per_launch"] / (ms_signal * 1e-3) / 1e9
                                   if (workload, dt) in MEASURED_GEMM_COUNTERS else None),
                     "counters_source": "mfma_util and the cycles per launch behind clock_ghz: rocprofv3 --pmc run of this "
                                        "kernel and workload (profiles/gemm_c5_mfma_utilisation.md); clock_ghz = those "
                                        "cycles / this run's launch time" if (workload, dt) in MEASURED_GEMM_COUNTERS else None,
                     "traffic": MEASURED_TRAFFIC_BYTES.get((workload, dt)),
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE counter runs of this kernel and workload "
                                       "(profiles/gemm_c5_hbm_traffic.md), not re-measured in this run; it moves by "
                                       "about 10 % between runs"
                     if (workload, dt) in MEASURED_TRAFFIC_BYTES else None},
        "times_ms": {"overlapped_step": ms_step, "overlapped_step_wall": wall_step,
                     "serial_step": ms_serial, "gemm_alone": ms_gemm, "gemm_signal_alone": ms_signal,
                     "two_calls_step": ms_pair,
                     "consumer_alone": ms_consumer, "reorder_rmsnorm_alone": ms_norm,
                     "vendor_gemm_torch_matmul": ms_vendor},
        "overlapped_vs_gemm_alone": ms_step / ms_gemm,
        "overlapped_vs_serial": ms_step / ms_serial,
        "two_calls_vs_serial": ms_pair / ms_serial if ms_pair else None,
        "timing": {"blocks": blocks, "steps_per_block": K_, "warmup_per_block": W_, "figure": "median of the blocks",
                   "block_ms": {k: [round(x, 4) for x in v] for k, v in samples.items()}},
        "consumer_GBps": 6.0 * M * N / (ms_consumer * 1e-3) / 1e9,
        "reorder_rmsnorm_GBps": (4.0 * bs * N + 2.0 * N) / (ms_norm * 1e-3) / 1e9,
        "hbm_peak_GBps": PEAK_HBM_GBS,
        "group_sweep": sweep,
        "link_model": {"what": "the same overlapped and serial step with a modelled link time (bytes / rate) behind "
                               "every consumer launch; a model of a link-bound collective on one GPU, not a measurement "
                               "of one", "rates": link_model} if link_model else None,
        "power": power,
        "bf16_repeat": bf16_repeat,
    }
    if power and power["legs"]["gemm_signal"]["watts"]:
        out["roofline"]["power_w"] = power["legs"]["gemm_signal"]["watts"]
        out["roofline"]["power_cap_w"] = power["cap_w"]

    out["waits_gave_up"] = ov.status()   # 1: a bounded device-side wait ran out of polls; the timings are then void
    return out, ov, (A16, B16, gamma16, eps, M)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--blocks", type=int, default=5,
                    help="rounds in which the overlapped step, the serial step and the two GEMMs take turns "
                         "(warmup + steps launches each per round); every reported time is the median of its blocks")
    ap.add_argument("--workload", default="c5", choices=sorted(WORKLOADS))
    ap.add_argument("--dtype", default=None, choices=["f16", "bf16"])
    ap.add_argument("--swizzle", type=int, default=4)
    ap.add_argument("--fused", type=int, default=-1,
                    help="-1: library default (one wait+reduce launch above 16 groups), 0: two launches per "
                         "group, 1: one launch")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--group-tiles", type=int, default=0, help="tiles per wave group (0: the workload's default)")
    ap.add_argument("--no-group-sweep", action="store_true", help="skip the wave-group-size sweep (c5 only)")
    ap.add_argument("--link-gbps", default="100,200,400,1000",
                    help="link-rate model (c5 only): algorithm bandwidths, in GB/s, of the collective the consumer "
                         "stands in for; empty: skip")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the compact records of the c2, c3 and c4 workloads that the default c5 run appends")
    ap.add_argument("--kernels-only", action="store_true",
                    help="run each hot kernel alone on one stream and exit: for counter collection, which "
                         "serialises dispatches and would stall a waiter that spins on another queue")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="with --kernels-only: also launch the vendor library's GEMM (torch.matmul) on the same "
                         "operands, for a counter run of the yardstick")
    ap.add_argument("--steps-only", action="store_true",
                    help="enqueue warmup + steps overlapped steps and exit: for a kernel-trace timeline of the "
                         "steady state")
    ap.add_argument("--comm-cus", type=int, default=0,
                    help="with --steps-only: put the consumer on a stream masked to this many CUs (a multiple of 8)")
    ap.add_argument("--gemm-cus-disjoint", action="store_true",
                    help="with --comm-cus: put the GEMM on a stream masked to the other CUs and let the library "
                         "plan its launches for that many (fo_gemm_set_cu_limit)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a 256 MiB device-to-device copy five times (reference point for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the collective is "
              "replaced by a one-GPU consumer); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    os.environ.setdefault("FO_WAIT_MAX_POLLS", "200000000")  # a lost signal must not hang the GPU
    import torch
    import flashoverlap_amd as fo
    from flashoverlap_amd import ops

    torch.cuda.set_device(0)
    if args.comm_cus:
        if not args.steps_only or args.comm_cus % 8 or args.comm_cus <= 0:
            raise SystemExit("--comm-cus wants --steps-only and a positive multiple of 8")
        if args.gemm_cus_disjoint:
            fo._capi.set_gemm_cu_limit(torch.cuda.get_device_properties(0).multi_processor_count - args.comm_cus)
    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel(), "copy_bytes_written": dst.numel(), "copies": 5}))
        return
    res = measure(args, args.workload)
    if res is None:  # --steps-only / --kernels-only printed their own line
        return
    out, ov, (A16, B16, gamma16, eps, M) = res
    if args.workload == "c5" and not args.no_other_workloads:
        ov.close()
        ov = None
        torch.cuda.empty_cache()
        out["other_workloads"] = [measure(args, w, compact=True) for w in ("c2", "c3", "c4")]
    if not args.no_cpu_baseline:
        from oracle import cpu_baseline
        r = cpu_baseline.time_sample(A16, B16, gamma16, eps, target_seconds=15.0)
        out["cpu_baseline"] = {"value": r["flops"] / r["seconds"] / 1e12, "unit": "TFLOP/s",
                               "cores": r["threads"], "kind": "port",
                               "sample": f"torch CPU fp32 matmul + RMSNorm on the first {r['rows']} of "
                                         f"{M} rows of the same A (all of B), {r['passes']} passes, {r['seconds']:.1f} s; "
                                         f"host has {os.cpu_count()} logical cpus"}
    if ov is not None:
        ov.close()
    assert out["waits_gave_up"] == 0 and all(o["waits_gave_up"] == 0 for o in out.get("other_workloads", [])), \
        "a device-side wait gave up: the step ran on incomplete tiles"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
