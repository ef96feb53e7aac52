"""GPU parity tests of the overlapped call that also enqueues the reorder+RMSNorm
(fo_overlap_gemm_allreduce_norm: src/overlap_impl.cu:246-263 followed by
src/rmsnorm/rmsnorm.cu:14-30, the rows normalised on the consumer stream as the groups
that complete them are consumed) and of the row-range kernel it uses
(fo_reorder_rmsnorm_rows, src/rmsnorm/rmsnorm.cuh:64-117).

What must hold: C', the counters and the accumulator are bit for bit what the call without
the normalisation leaves; Y equals, bit for bit, the plain RMSNorm (same kernel, no
reorder table) of the plain GEMM's row-major product, lies within 2 units in the last place
of the CPU checker's reorder_rmsnorm on the GPU's own C', and within 1e-2 of the unrounded
float64 formula."""
import numpy as np
import pytest
import torch

from gpu_util import BF16, F16, TORCH_DTYPE, bits_of, from_bits, max_rel_err, rmsnorm_f64, seeded, ulp_diff_ok

pytestmark = pytest.mark.gpu
REL_TOL = 1e-2
EPS = 1e-6


def _setup(fo, dtype, bm, bn, M, N, K, cseg, seed, hint=None):
    algo = fo._capi.find_algo(bm, bn, swizzle=4)
    TM, TN = M // bm, N // bn
    if hint is None:
        hint = fo._capi.schedule_order(algo, M, N)
    RA = fo.layout.reorder_indices(TM * TN, hint, device="cuda").reshape(TM, TN)
    A, _ = seeded((M, K), dtype, seed)
    B, _ = seeded((N, K), dtype, seed + 1, scale=K ** -0.5)
    gamma = (1 + 0.01 * torch.randn(N, generator=torch.Generator().manual_seed(seed + 2))).to(TORCH_DTYPE[dtype]).cuda()
    MM = torch.zeros(fo.layout.counter_size(len(cseg), TM, TN), dtype=torch.int32, device="cuda")
    cs_cpu = torch.tensor(cseg, dtype=torch.int32)
    return algo, RA, A, B, gamma, MM, cs_cpu, cs_cpu.cuda()


def _run_both(fo, dtype, bm, bn, M, N, K, cseg, fused, seed, hint=None):
    """The call with the normalisation and the call without it followed by reorder_rmsnorm, same inputs."""
    algo, RA, A, B, gamma, MM, cs_cpu, cs_gpu = _setup(fo, dtype, bm, bn, M, N, K, cseg, seed, hint)
    td = TORCH_DTYPE[dtype]
    acc0, _ = seeded((M * N,), dtype, seed + 3, scale=0.5)
    ov = fo.ops.Overlap()
    ov.set_fused_consumer(fused)
    # reference pair
    C_ref = torch.full((M * N,), float("nan"), device="cuda", dtype=td)
    acc_ref = acc0.clone()
    ov.set_accumulator(acc_ref)
    ov.gemm_allreduce_overlap(A, B, C_ref, MM, RA, 1, cs_cpu, cs_gpu, algo)
    Y_pair = torch.empty(M, N, device="cuda", dtype=td)
    fo.ops.reorder_rmsnorm(C_ref.view(M, N), Y_pair, gamma, bm, bn, 1, RA, eps=EPS)
    torch.cuda.synchronize()
    assert (MM == 0).all()
    # the call under test, twice on the same buffers (the second call starts from what the first left)
    C = torch.full((M * N,), float("nan"), device="cuda", dtype=td)
    Y = torch.full((M, N), float("nan"), device="cuda", dtype=td)
    acc = acc0.clone()
    ov.set_accumulator(acc)
    RA_cpu = RA.cpu()
    for rep in range(2):
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA_cpu, 1, cs_cpu, cs_gpu, algo, Y, gamma, eps=EPS)
        # what follows on the GEMM stream sees the complete Y without any synchronisation of the host
        Y_seen = Y.clone()
        torch.cuda.synchronize()
        assert ov.status() == 0 and (MM == 0).all()
        assert torch.equal(C, C_ref)
        if rep == 0:
            assert torch.equal(acc, acc_ref)
        assert torch.equal(Y_seen, Y) and not torch.isnan(Y).any()
        if rep == 0:
            Y.fill_(float("nan"))
            Y_first = Y_seen
        else:
            assert torch.equal(Y, Y_first)
    ov.close()
    plain = torch.empty(M, N, device="cuda", dtype=td)
    fo.ops.gemm(A, B, plain, algo)
    Y_plain = torch.empty(M, N, device="cuda", dtype=td)
    fo.ops.reorder_rmsnorm_rows(plain, Y_plain, gamma, 0, M, 1, 8, 1, None, eps=EPS)
    torch.cuda.synchronize()
    assert torch.equal(fo.layout.unpermute(C, M, N, bm, bn, RA), plain)
    assert torch.equal(Y, Y_plain)                      # the gather is exact: same bits as the plain normalisation
    return C, Y, Y_pair, plain, gamma, RA


@pytest.mark.parametrize("fused", [0, 1, -1])           # per-wave launches, one-launch consumer, automatic (one stream)
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_norm_overlap_against_checker(fo, oracle, dtype, fused):
    bm, bn, M, N, K = 128, 128, 1024, 2048, 256
    cseg = [32, 32, 16, 48]
    C, Y, Y_pair, plain, gamma, RA = _run_both(fo, dtype, bm, bn, M, N, K, cseg, fused, seed=400)
    ref = oracle.reorder_rmsnorm(dtype, bits_of(C), bits_of(gamma), M, N, bm, bn, 1, RA.cpu().numpy().reshape(-1), eps=EPS)
    assert ulp_diff_ok(bits_of(Y), ref, dtype, max_ulp=2, frac=0.99)
    assert ulp_diff_ok(bits_of(Y), bits_of(Y_pair), dtype, max_ulp=2, frac=0.99)
    assert max_rel_err(Y.cpu(), rmsnorm_f64(plain, gamma, EPS)) <= REL_TOL


def test_norm_overlap_with_a_scattered_reorder_table(fo, oracle):
    """A reorder table that is not the schedule order: tile rows complete in no particular order, some only with
    the last group; every row must still be normalised exactly once, after its last tile has been consumed."""
    bm, bn, M, N, K = 128, 128, 2048, 1024, 128
    T = (M // bm) * (N // bn)
    hint = np.random.default_rng(7).permutation(T).tolist()
    C, Y, _, plain, gamma, RA = _run_both(fo, F16, bm, bn, M, N, K, [16, 48, 32, 32], 0, seed=410, hint=hint)
    ref = oracle.reorder_rmsnorm(F16, bits_of(C), bits_of(gamma), M, N, bm, bn, 1, RA.cpu().numpy().reshape(-1), eps=EPS)
    assert ulp_diff_ok(bits_of(Y), ref, F16, max_ulp=2, frac=0.99)
    # tile rows in ascending order of completion: rows finish with different groups
    hint2 = [t for tm in (3, 0, 9, 1, 15, 2) for t in range(tm * (N // bn), (tm + 1) * (N // bn))]
    _run_both(fo, F16, bm, bn, M, N, K, [24, 24, 80], 0, seed=420, hint=hint2)


@pytest.mark.parametrize("name,dtype,M,N,K,bm,bn,gtiles", [
    ("large square", F16, 8192, 8192, 8192, 128, 256, 256),
    ("down-projection", BF16, 8192, 8192, 3584, 256, 128, 512),
])
def test_norm_overlap_at_full_size(fo, name, dtype, M, N, K, bm, bn, gtiles):
    """BASELINE shapes: wave groups, the rows of each wave normalised behind its consumer.  Checked through what
    does not depend on the size: bit equality with the plain normalisation of the plain product, counters back
    at zero, sampled rows against the float64 formula."""
    T = (M // bm) * (N // bn)
    cseg = fo.layout.cseg_from_waves(T, gtiles)
    C, Y, Y_pair, plain, gamma, RA = _run_both(fo, dtype, bm, bn, M, N, K, cseg, -1, seed=430)
    rows = torch.tensor([0, 1, 127, 128, 2047, 2048, 4095, 6143, 8191])
    assert max_rel_err(Y[rows.cuda()].cpu(), rmsnorm_f64(plain[rows.cuda()], gamma, EPS)) <= REL_TOL
    assert ulp_diff_ok(bits_of(Y[rows.cuda()]), bits_of(Y_pair[rows.cuda()]), dtype, max_ulp=2, frac=0.99)
    # the waves of the schedule order are whole tile rows: every wave's rows could follow its consumer
    algo = fo._capi.find_algo(bm, bn, swizzle=4)
    wave = fo._capi.wave_tiles(algo, M, N)
    last_slot = RA.cpu().view(M // bm, N // bn).max(dim=1).values
    first_slot = RA.cpu().view(M // bm, N // bn).min(dim=1).values
    assert torch.equal(last_slot // wave, first_slot // wave)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_row_ranges_of_the_normalisation(fo, oracle, dtype):
    """fo_reorder_rmsnorm_rows on ranges that start and end inside tiles, with rows of 4096 to 16384 elements and
    a row length that is no multiple of the 2048 a workgroup covers per pass; untouched rows stay untouched."""
    for (bm, bn, M, N, rldn) in [(128, 128, 512, 4096, 1), (64, 256, 256, 8192, 1), (16, 128, 64, 16384, 1),
                                 (32, 96, 64, 480, 1), (64, 128, 256, 512, 2), (16, 64, 32, 8256, 1)]:
        TM, TN = M // bm, N // bn
        ra = np.random.default_rng(50).permutation(TM * TN).astype(np.int32)
        X, xb = seeded((M, N), dtype, 51, scale=1.5)
        gamma, wb = seeded((N,), dtype, 52)
        RA = torch.from_numpy(ra).cuda()
        ref = oracle.reorder_rmsnorm(dtype, xb.reshape(-1), wb, M, N, bm, bn, rldn, ra, eps=EPS)
        Y = torch.full((M, N), float("nan"), device="cuda", dtype=TORCH_DTYPE[dtype])
        lo, hi = bm // 2 + 1, M - 3
        fo.ops.reorder_rmsnorm_rows(X, Y, gamma, lo, hi - lo, bm, bn, rldn, RA, eps=EPS)
        torch.cuda.synchronize()
        assert torch.isnan(Y[:lo]).all() and torch.isnan(Y[hi:]).all()
        assert ulp_diff_ok(bits_of(Y[lo:hi]), ref[lo:hi], dtype, max_ulp=2, frac=0.99)
        fo.ops.reorder_rmsnorm_rows(X, Y, gamma, 0, lo, bm, bn, rldn, RA, eps=EPS)
        fo.ops.reorder_rmsnorm_rows(X, Y, gamma, hi, M - hi, bm, bn, rldn, RA, eps=EPS)
        Y_old = torch.empty_like(Y)
        fo.ops.reorder_rmsnorm(X, Y_old, gamma, bm, bn, rldn, RA, eps=EPS)
        torch.cuda.synchronize()
        assert ulp_diff_ok(bits_of(Y), ref, dtype, max_ulp=2, frac=0.99)
        assert ulp_diff_ok(bits_of(Y), bits_of(Y_old), dtype, max_ulp=2, frac=0.99)


@pytest.mark.parametrize("dtype,M,N,bm,bn", [(F16, 8192, 8192, 128, 256), (BF16, 8192, 8192, 256, 128),
                                             (F16, 8192, 4096, 128, 128), (BF16, 4096, 2048, 128, 128)])
def test_row_kernel_fits_beside_the_signalling_gemm(fo, dtype, M, N, bm, bn):
    """The rows of a wave are normalised while the next wave's workgroups hold every CU: one workgroup of the row
    kernel (a wavefront per SIMD) must fit into what a GEMM workgroup leaves of the CU's registers and LDS, or the
    call silently degrades into GEMM first, normalisation afterwards."""
    algo = fo._capi.find_algo(bm, bn, swizzle=4)
    gemm = fo._capi.kernel_info(algo, M, N, epilogue=1, dtype=dtype)
    rows = fo._capi.norm_rows_kernel_info(N, True, bn, 1, True, dtype=dtype)
    per_simd = gemm["threads"] // 256 * (gemm["resident"] // 256)
    assert per_simd * ((gemm["vgprs"] + 7) // 8 * 8) + (rows["vgprs"] + 7) // 8 * 8 <= 512, (gemm, rows)
    assert (gemm["resident"] // 256) * gemm["lds_bytes"] + rows["lds_bytes"] <= 160 * 1024, (gemm, rows)


def test_norm_overlap_refuses_bad_arguments(fo):
    bm, bn, M, N, K = 128, 128, 512, 512, 64
    algo, RA, A, B, gamma, MM, cs_cpu, cs_gpu = _setup(fo, F16, bm, bn, M, N, K, [8, 8], seed=440)
    C = torch.empty(M * N, device="cuda", dtype=torch.float16)
    Y = torch.empty(M, N, device="cuda", dtype=torch.float16)
    ov = fo.ops.Overlap()
    with pytest.raises(ValueError):                       # RA_cpu on the GPU
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA, 1, cs_cpu, cs_gpu, algo, Y, gamma)
    with pytest.raises(ValueError):                       # Y too small
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA.cpu(), 1, cs_cpu, cs_gpu, algo, Y[:8], gamma)
    bad = RA.cpu().clone()
    bad[0, 0] = 16                                        # a slot outside the table
    with pytest.raises(fo.FlashOverlapError):
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, bad, 1, cs_cpu, cs_gpu, algo, Y, gamma)
    torch.cuda.synchronize()
    assert ov.status() == 0 and (MM == 0).all()           # a refused call has enqueued nothing
    ov.close()


def test_dropin_class_exposes_the_call(fo):
    """The same call through torch.classes.flashoverlap_class.OverlapImpl (an addition to the reference's methods)."""
    from flashoverlap_amd import layers
    layers.load_library()
    bm, bn, M, N, K = 128, 128, 1024, 1024, 128
    cseg = [32, 32]
    algo, RA, A, B, gamma, MM, cs_cpu, cs_gpu = _setup(fo, F16, bm, bn, M, N, K, cseg, seed=450)
    impl = torch.classes.flashoverlap_class.OverlapImpl()
    impl.nccl_init(0, 1, [0] * 16)
    impl.cutlass_init()
    impl.overlap_init()
    impl.set_fused_consumer(0)
    C = torch.empty(M, N, device="cuda", dtype=torch.float16)
    Y = torch.full((M, N), float("nan"), device="cuda", dtype=torch.float16)
    impl.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA.cpu(), 1, cs_cpu, cs_gpu, algo, False, Y, gamma, EPS)
    torch.cuda.synchronize()
    plain = torch.empty(M, N, device="cuda", dtype=torch.float16)
    fo.ops.gemm(A, B, plain, algo)
    Y_plain = torch.empty_like(Y)
    fo.ops.reorder_rmsnorm_rows(plain, Y_plain, gamma, 0, M, 1, 8, 1, None, eps=EPS)
    torch.cuda.synchronize()
    assert torch.equal(Y, Y_plain) and (MM == 0).all() and impl.status() == 0


def test_link_rate_model_holds_the_consumer_stream_and_changes_no_result(fo):
    """fo_overlap_set_link_rate: every consumer launch is followed by a kernel that holds its stream for
    bytes / rate.  Results are those of the call without it; the call takes at least the link time of the
    last wave's bytes longer than the GEMM, and the serial call at least the whole matrix's link time."""
    dtype, bm, bn, M, N, K = F16, 128, 256, 2048, 4096, 1024
    T = (M // bm) * (N // bn)
    cseg = [T // 4] * 4
    algo, RA, A, B, gamma, MM, cs_cpu, cs_gpu = _setup(fo, dtype, bm, bn, M, N, K, cseg, 31)
    td = TORCH_DTYPE[dtype]
    acc0, _ = seeded((M * N,), dtype, 34, scale=0.5)
    RA_cpu = RA.cpu()
    ov = fo.ops.Overlap()
    ov.set_fused_consumer(0)
    out = {}
    for rate in (0.0, 20.0):          # 16.8 MB of C at 20 GB/s: 0.84 ms of link time
        C = torch.full((M * N,), float("nan"), device="cuda", dtype=td)
        Y = torch.full((M, N), float("nan"), device="cuda", dtype=td)
        acc = acc0.clone()
        ov.set_accumulator(acc)
        ov.set_link_rate(rate)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA_cpu, 1, cs_cpu, cs_gpu, algo, Y, gamma, eps=EPS)
        torch.cuda.synchronize()
        e0.record()
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA_cpu, 1, cs_cpu, cs_gpu, algo, Y, gamma, eps=EPS)
        e1.record()
        torch.cuda.synchronize()
        assert ov.status() == 0 and (MM == 0).all()
        out[rate] = (C, Y, acc, e0.elapsed_time(e1))
    assert torch.equal(out[0.0][0], out[20.0][0]) and torch.equal(out[0.0][1], out[20.0][1])
    assert torch.equal(out[0.0][2], out[20.0][2])
    link_ms = 2.0 * M * N / 20e9 * 1e3
    assert out[20.0][3] >= link_ms * 0.95 and out[0.0][3] < link_ms * 0.5, (out[0.0][3], out[20.0][3], link_ms)
    # the serial comparator of the handle models the same link
    Cs = torch.empty(M, N, device="cuda", dtype=td)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    ov.gemm_allreduce(A, B, Cs, algo)
    e1.record()
    torch.cuda.synchronize()
    assert e0.elapsed_time(e1) >= link_ms * 0.95
    # the kernel alone, and its limit
    e0.record()
    fo.ops.pace(300_000)
    e1.record()
    torch.cuda.synchronize()
    assert 0.28 <= e0.elapsed_time(e1) < 1.0
    with pytest.raises(RuntimeError):
        fo.ops.pace(2_000_000_000)
    with pytest.raises(RuntimeError):
        ov.set_link_rate(-1.0)
    # a rate that would hold the stream for more than a second is refused before anything is enqueued
    ov.set_link_rate(0.001)
    MM.zero_()
    with pytest.raises(RuntimeError):
        ov.gemm_allreduce_rmsnorm_overlap(A, B, C, MM, RA, RA_cpu, 1, cs_cpu, cs_gpu, algo, Y, gamma, eps=EPS)
    torch.cuda.synchronize()
    assert ov.status() == 0 and (MM == 0).all()
    ov.set_link_rate(0)
    ov.close()
