"""GPU parity tests of the individual kernels, called through the C ABI (ctypes)
and checked against the CPU checker on the same seeded inputs.

Tolerances: integer results (permutation, counts, stamps, addresses) and the
consumer are bit-exact; GEMM and RMSNorm values are compared against the
fp32-accumulating checker with max rel err <= 1e-2 (and, tighter, within a
couple of 16-bit ulps, since both sides accumulate in fp32 and round once)."""
import os

import numpy as np
import pytest
import torch

from gpu_util import (BF16, F16, TORCH_DTYPE, bits_of, from_bits, max_rel_err, rmsnorm_f64, seeded,
                      ulp_diff_ok)

pytestmark = pytest.mark.gpu

REL_TOL = 1e-2  # north-star tolerance for GEMM and RMSNorm values


def _algo(fo, bm, bn, swizzle=1):
    return fo._capi.find_algo(bm, bn, swizzle=swizzle)


# ---------------------------------------------------------------- plain GEMM
@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("bm,bn,M,N,K", [(128, 128, 256, 384, 192), (128, 256, 256, 512, 128),
                                         (256, 128, 512, 256, 64), (128, 128, 1024, 1024, 1024)])
def test_gemm_matches_checker(fo, oracle, dtype, bm, bn, M, N, K):
    A, Ab = seeded((M, K), dtype, 1)
    B, Bb = seeded((N, K), dtype, 2, scale=K ** -0.5)
    C = torch.empty(M, N, device="cuda", dtype=TORCH_DTYPE[dtype])
    fo.ops.gemm(A, B, C, _algo(fo, bm, bn))
    torch.cuda.synchronize()
    ref_bits, _ = oracle.gemm_signal(dtype, Ab, Bb, bm, bn)
    ref = torch.from_numpy(oracle.from_bits(ref_bits, dtype))
    assert max_rel_err(C.float().cpu(), ref) <= REL_TOL
    assert ulp_diff_ok(bits_of(C), ref_bits, dtype, max_ulp=1, frac=0.999)


def test_gemm_exact_special_cases(fo):
    # all ones: every C == K exactly (the reference's own AR test input, correctness_ar.py:24-25)
    M, N, K = 256, 256, 512
    A = torch.ones(M, K, device="cuda", dtype=torch.float16)
    B = torch.ones(N, K, device="cuda", dtype=torch.float16)
    C = torch.zeros(M, N, device="cuda", dtype=torch.float16)
    fo.ops.gemm(A, B, C, _algo(fo, 128, 128))
    assert (C == K).all()
    # identity weight: C == A bit for bit; catches transposed or mis-indexed operands
    A, _ = seeded((256, 256), F16, 3)
    eye = torch.eye(256, device="cuda", dtype=torch.float16)
    fo.ops.gemm(A, eye, C, _algo(fo, 128, 128))
    assert torch.equal(C, A)
    # a one-hot row of B selects a column of A
    B = torch.zeros(256, 256, device="cuda", dtype=torch.float16)
    B[5, 77] = 1.0
    fo.ops.gemm(A, B, C, _algo(fo, 128, 128))
    assert torch.equal(C[:, 5], A[:, 77]) and C[:, :5].abs().sum() == 0


# ---------------------------------------------------------------- signal / scatter GEMM
def _signal_case(fo, oracle, dtype, bm, bn, M, N, K, cseg, rldn=1, W=0, monitor=False, swizzle=1, seed=4):
    algo = _algo(fo, bm, bn, swizzle)
    TM, TN = M // bm, N // bn
    T = TM * TN
    rng = np.random.default_rng(seed)
    hint = rng.permutation(T)[: max(1, T // 2)].tolist()
    RA = (torch.arange(T, dtype=torch.int32) if monitor else
          fo.layout.reorder_indices(T, hint, device="cpu")).reshape(TM, TN).cuda()
    A, Ab = seeded((M, K), dtype, seed + 1)
    B, Bb = seeded((N, K), dtype, seed + 2, scale=K ** -0.5)
    plain = torch.empty(M, N, device="cuda", dtype=TORCH_DTYPE[dtype])
    fo.ops.gemm(A, B, plain, algo)
    Cp = torch.full((M * N,), float("nan"), device="cuda", dtype=TORCH_DTYPE[dtype])
    MM = torch.zeros(fo.layout.counter_size(len(cseg), TM, TN, monitor) + 8, dtype=torch.int32, device="cuda")
    cseg_gpu = torch.tensor(cseg, dtype=torch.int32, device="cuda")
    RE = fo.layout.generate_row_mapping(M, N, bm, bn, cseg, W, device="cuda") if W else None
    fo.ops.gemm_signal(A, B, Cp, MM, RA, cseg_gpu, algo, rLDN=rldn, monitor=monitor, RE=RE)
    torch.cuda.synchronize()
    ra_np = RA.cpu().numpy().reshape(-1)
    re_np = None if RE is None else RE.cpu().numpy()
    # (1) permutation bit-exact: un-permuting with the checker's inverse map gives the plain GEMM
    back = oracle.unpermute(bits_of(Cp), M, N, bm, bn, ra_np, rLDN=rldn, RE=re_np)
    assert (back == bits_of(plain)).all()
    # (2) the package's own torch inverse agrees
    assert torch.equal(fo.layout.unpermute(Cp, M, N, bm, bn, RA, rLDN=rldn, RE=RE), plain)
    # (3) every element was written exactly once (no NaN filler left)
    assert not torch.isnan(Cp).any()
    # (4) signal counts bit-exact
    mm = MM.cpu().numpy()
    if not monitor:
        assert mm[:len(cseg)].tolist() == list(cseg)
        assert (mm[len(cseg):] == 0).all()
    # (5) values against the checker's own reordered buffer
    ref_bits, ref_mm = oracle.gemm_signal(dtype, Ab, Bb, bm, bn, RA=ra_np, cseg=cseg, rLDN=rldn, RE=re_np)
    assert ulp_diff_ok(bits_of(Cp), ref_bits, dtype, max_ulp=1, frac=0.999)
    assert max_rel_err(Cp.float().cpu(), torch.from_numpy(oracle.from_bits(ref_bits, dtype))) <= REL_TOL
    return mm, T, TN


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_signal_gemm_reorder_and_counts(fo, oracle, dtype):
    _signal_case(fo, oracle, dtype, 128, 128, 512, 512, 128, [4, 4, 4, 4])
    _signal_case(fo, oracle, dtype, 128, 128, 512, 512, 128, [1, 15])
    _signal_case(fo, oracle, dtype, 128, 256, 512, 1024, 64, [5, 3, 8], swizzle=4)
    _signal_case(fo, oracle, dtype, 256, 128, 1024, 512, 64, [16], swizzle=8)


def test_signal_gemm_many_groups_and_rldn(fo, oracle):
    # more groups than tile columns (the reference under-allocates MM here, test/test.py:94)
    _signal_case(fo, oracle, F16, 128, 128, 1024, 512, 64, [1] * 32)
    # 70 groups: the group lookup needs more than one 64-wide scan step
    _signal_case(fo, oracle, F16, 128, 128, 1280, 1024, 64, [1] * 60 + [2] * 10)
    # rLDN > 1: the reshaped output is rLDN tiles wide
    _signal_case(fo, oracle, F16, 128, 128, 512, 512, 64, [8, 8], rldn=2)
    _signal_case(fo, oracle, F16, 128, 128, 512, 512, 64, [16], rldn=4)


def test_signal_gemm_persistent_walk(fo, oracle):
    """More tiles than resident workgroups: some workgroups compute several tiles, request
    the next tile's operands before their epilogue and send the previous tile's signal late."""
    # 600 tiles of 128x128 (M is no multiple of 256, so the workgroup tile is 128x128; 512 are resident)
    _signal_case(fo, oracle, F16, 128, 128, 3200, 3072, 128, [100] * 6)
    # one K step per tile: the signal cannot ride in the next tile's K loop and is sent at once
    _signal_case(fo, oracle, BF16, 128, 128, 3200, 3072, 64, [599, 1])
    # 272 workgroup tiles of 256x256 on 256 resident workgroups, four reorder tiles each
    _signal_case(fo, oracle, F16, 128, 128, 4352, 4096, 128, [272] * 4, swizzle=4)
    _signal_case(fo, oracle, F16, 256, 128, 4352, 4096, 192, [300, 244], swizzle=4, W=2)
    # 1089 groups: beyond the group table kept in LDS, the lookup scans cSeg in memory
    _signal_case(fo, oracle, F16, 128, 128, 4224, 4224, 64, [1] * 1089)


@pytest.mark.parametrize("bm,bn,M,N", [(128, 256, 4224, 2048), (256, 128, 2048, 4224)])
@pytest.mark.parametrize("dtype,K,cseg,W", [
    (F16, 64, [264], 0),                 # one K step per tile: nothing can ride in the next tile, signalled at once
    (F16, 192, [100, 100, 64], 0),       # three K steps: exactly the ring's depth, no steady step
    (BF16, 1096, [8, 256], 0),           # seventeen full K steps through the dynamic-slot steady loop, then a partial one
    (F16, 448, [132, 132], 2),           # row-mapped stores, seven K steps
    (BF16, 64, [1] * 264, 0),            # a group per tile
])
def test_signal_gemm_three_slot_shapes_walk_several_tiles(fo, oracle, dtype, K, cseg, W, bm, bn, M, N):
    """The 128x256 and 256x128 workgroup tiles run on rings of three slots.  264 tiles on 256 resident
    workgroups (M or N is no multiple of 256, so the workgroup tile is the Algo's own): eight workgroups
    compute a second tile, whose first stage is requested before the first tile's epilogue, whose first
    wait leaves that epilogue's stores in flight, and from whose first K step the first tile's signal is
    sent while younger operand loads are still outstanding."""
    info = fo._capi.kernel_info(_algo(fo, bm, bn, swizzle=4), M, N, epilogue=2 if W else 1, dtype=dtype)
    assert info["resident"] == 256 and info["lds_bytes"] == 3 * (128 + 256) * 64 * 2
    _signal_case(fo, oracle, dtype, bm, bn, M, N, K, cseg, W=W, swizzle=4, seed=11 + K)


@pytest.mark.parametrize("dtype,bm,bn,K,cseg,W,monitor", [
    (F16, 128, 256, 64, [400, 400], 0, False),         # one K step per tile: every step starts a tile, every epilogue is followed by loads
    (F16, 128, 128, 128, [1] * 600 + [1000], 0, False),  # two K steps: the loader is always in the next tile; groups beyond the register table
    (BF16, 256, 128, 200, [144, 256, 400], 0, False),  # three full K steps and a partial one (zeros from beyond the buffer range)
    (F16, 128, 256, 192, [500, 300], 2, False),        # row-mapped stores
    (F16, 128, 256, 72, [800], 0, True),               # monitor stamps, partial second K step
    (BF16, 128, 128, 328, [800, 800], 4, False),       # row-mapped stores, five full K steps and a partial one
])
def test_signal_gemm_256_tile_walks_several_tiles(fo, oracle, dtype, bm, bn, K, cseg, W, monitor):
    """The 256x256 workgroup tile (four wavefronts, operands straight into LDS through buffer loads, the
    loader running two K steps ahead across tile boundaries).  400 tiles of 256x256 on 256 resident
    workgroups: 144 workgroups compute a second tile, whose operands are requested during the first
    tile's last steps, whose first meeting waits for the first tile's stores, and from whose first K
    step the first tile's signal is sent."""
    M, N = 6400, 4096
    info = fo._capi.kernel_info(_algo(fo, bm, bn, swizzle=4), M, N, epilogue=2 if W else 1, dtype=dtype)
    assert info["resident"] == 256 and info["threads"] == 256 and info["lds_bytes"] == 2 * 65536 + 4 * 16 * 136 * 2
    _signal_case(fo, oracle, dtype, bm, bn, M, N, K, cseg, W=W, monitor=monitor, swizzle=4, seed=21 + K)


def test_signal_gemm_under_a_cu_limit(fo, oracle):
    """fo_gemm_set_cu_limit (the reference plans for sm_count - 2, tune/search.py:404-407): with 96 CUs
    the persistent launch holds 96 workgroups, a wave is 96 x 2 reorder tiles of 128x256, and the 400
    tiles of 256x256 are four full waves and a tail of 16 that a second launch walks in the Algo's own
    tile; counters, reordered stores and values as ever."""
    M, N, bm, bn = 6400, 4096, 128, 256
    algo = _algo(fo, bm, bn, swizzle=4)
    try:
        fo._capi.set_gemm_cu_limit(96)
        info = fo._capi.kernel_info(algo, M, N, epilogue=1, dtype=F16)
        assert info["resident"] == 96
        assert fo._capi.wave_tiles(algo, M, N) == 192
        _signal_case(fo, oracle, F16, bm, bn, M, N, 136, [500, 144, 156], swizzle=4, seed=77)
        _signal_case(fo, oracle, BF16, 128, 128, M, N, 64, [1600], swizzle=4, seed=78, monitor=True)
    finally:
        fo._capi.set_gemm_cu_limit(0)
    assert fo._capi.kernel_info(algo, M, N, epilogue=1, dtype=F16)["resident"] == 256
    assert fo._capi.wave_tiles(algo, M, N) == 512


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("bm,bn,M,N,K", [(128, 128, 256, 384, 8), (128, 128, 256, 384, 72),
                                         (128, 128, 384, 256, 200), (128, 128, 256, 256, 1376),
                                         (128, 256, 256, 512, 104), (256, 128, 512, 256, 136),
                                         (128, 256, 256, 512, 24), (128, 128, 4352, 4096, 88)])
def test_gemm_partial_last_k_step(fo, oracle, dtype, bm, bn, M, N, K):
    """K is any multiple of 8: the chunks of the last K step that lie beyond K are zero-filled on
    chip.  The operands end exactly at the end of a buffer whose tail is NaN, so a read past a
    row's end that reached the accumulators would show (it would bring the next row's head, or
    the NaN tail for the last row)."""
    t = TORCH_DTYPE[dtype]
    A, Ab = seeded((M, K), dtype, 31)
    B, Bb = seeded((N, K), dtype, 32, scale=K ** -0.5)
    bufA = torch.full((M * K + 256,), float("nan"), device="cuda", dtype=t)
    bufB = torch.full((N * K + 256,), float("nan"), device="cuda", dtype=t)
    bufA[:M * K] = A.reshape(-1)
    bufB[:N * K] = B.reshape(-1)
    C = torch.empty(M, N, device="cuda", dtype=t)
    fo.ops.gemm(bufA[:M * K].view(M, K), bufB[:N * K].view(N, K), C, _algo(fo, bm, bn))
    torch.cuda.synchronize()
    ref_bits, _ = oracle.gemm_signal(dtype, Ab, Bb, bm, bn)
    ref = torch.from_numpy(oracle.from_bits(ref_bits, dtype))
    assert not torch.isnan(C).any()
    assert max_rel_err(C.float().cpu(), ref) <= REL_TOL
    assert ulp_diff_ok(bits_of(C), ref_bits, dtype, max_ulp=1, frac=0.999)


def test_signal_gemm_partial_last_k_step(fo, oracle):
    """The partial K step inside the persistent walk: as a tile's only step (requested before
    the previous tile's epilogue), as the second of two, and behind the steady loop."""
    _signal_case(fo, oracle, F16, 128, 128, 3200, 3072, 40, [300, 300])
    _signal_case(fo, oracle, BF16, 128, 128, 3200, 3072, 72, [599, 1])
    _signal_case(fo, oracle, F16, 128, 128, 4352, 4096, 456, [272] * 4, swizzle=4)
    _signal_case(fo, oracle, F16, 256, 128, 4352, 4096, 200, [300, 244], swizzle=4, W=2)
    _signal_case(fo, oracle, F16, 128, 256, 1024, 1024, 328, [16, 16])


def test_scatter_gemm_row_map(fo, oracle):
    _signal_case(fo, oracle, F16, 128, 128, 512, 512, 64, [4, 4, 8], W=4)
    _signal_case(fo, oracle, BF16, 128, 128, 512, 256, 128, [3, 5], W=8)


def test_monitor_stamps(fo, oracle):
    mm, T, TN = _signal_case(fo, oracle, F16, 128, 128, 1024, 1024, 64, [16, 16, 16, 16], monitor=True)
    assert mm[:4].tolist() == [16, 16, 16, 16]
    assert mm[TN - 1] == T
    assert sorted(mm[TN:TN + T].tolist()) == list(range(T))


# ---------------------------------------------------------------- wait
def test_wait_bounded_gives_up_and_flags(fo):
    MM = torch.tensor([3, 0], dtype=torch.int32, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    fo.ops.wait_bounded(4, MM, 0, 2000, status)          # 3 != 4 forever: must give up
    torch.cuda.synchronize()
    assert status.item() == 1 and MM[0].item() == 3       # counter untouched
    status.zero_()
    fo.ops.wait_bounded(3, MM, 0, 2000, status)          # already equal: released and reset
    torch.cuda.synchronize()
    assert status.item() == 0 and MM[0].item() == 0


def test_wait_groups_resets_a_run_of_counters(fo):
    cseg = torch.tensor([3, 5, 7, 9], dtype=torch.int32, device="cuda")
    MM = torch.tensor([3, 5, 7, 9, 11], dtype=torch.int32, device="cuda")
    fo.ops.wait_groups(cseg, MM, first=1, count=2)        # groups 1 and 2 only
    torch.cuda.synchronize()
    assert MM.tolist() == [3, 0, 0, 9, 11]
    fo.ops.wait_groups(cseg, MM, first=3)                 # the rest
    fo.ops.wait_groups(cseg, MM, first=0, count=1)
    torch.cuda.synchronize()
    assert MM.tolist() == [0, 0, 0, 0, 11]


def test_wait_released_by_second_stream(fo):
    MM = torch.zeros(4, dtype=torch.int32, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    done = torch.zeros(1, dtype=torch.int32, device="cuda")
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        # bounded (about a minute) so a broken signal path cannot hang the GPU
        fo.ops.wait_bounded(5, MM, 2, 40_000_000, status, stream=s1)
        done.add_(1)                                     # ordered after the wait on s1
    with torch.cuda.stream(s2):
        for _ in range(5):
            MM[2:3].add_(1)
    torch.cuda.synchronize()
    assert status.item() == 0 and done.item() == 1
    assert MM.tolist() == [0, 0, 0, 0]                   # reset by the CAS


# ---------------------------------------------------------------- consumer
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_consumer_bit_exact(fo, oracle, dtype):
    n = 1 << 18
    src, sb = seeded((n,), dtype, 20)
    acc, ab = seeded((n,), dtype, 21, scale=3.0)
    ref = ab.copy()
    for _ in range(3):
        fo.ops.consumer_reduce(src, acc)
        oracle.consumer_reduce(dtype, sb, ref)
    torch.cuda.synchronize()
    assert (bits_of(acc) == ref).all()
    # closed form on a zeroed accumulator: k calls give k * src when k * src is exact
    acc.zero_()
    fo.ops.consumer_reduce(src, acc)
    fo.ops.consumer_reduce(src, acc)
    assert torch.equal(acc, (src.float() * 2).to(src.dtype))


def test_consumer_reduce_scatter_layout(fo, oracle):
    W, chunk = 4, 4096
    src, sb = seeded((W * chunk,), F16, 22)
    seg = 3 * chunk
    acc = torch.zeros(W * seg, device="cuda", dtype=torch.float16)
    fo.ops.consumer_reduce_rs(src, acc[chunk:], W, seg)     # offset inside every segment
    torch.cuda.synchronize()
    a = acc.view(W, seg)
    for q in range(W):
        assert torch.equal(a[q, chunk:2 * chunk], src[q * chunk:(q + 1) * chunk])
        assert a[q, :chunk].abs().sum() == 0 and a[q, 2 * chunk:].abs().sum() == 0


# ---------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("bs,dim", [(64, 256), (32, 4096), (16, 8192), (8, 1000 * 8), (4, 16384)])
def test_rmsnorm_matches_checker(fo, oracle, dtype, bs, dim):
    X, Xb = seeded((bs, dim), dtype, 30, scale=2.0)
    g = torch.Generator().manual_seed(31)
    W16 = (1 + 0.01 * torch.randn(dim, generator=g)).to(TORCH_DTYPE[dtype])
    Y = torch.empty_like(X)
    fo.ops.rmsnorm(X, Y, W16.cuda(), eps=1e-6)
    torch.cuda.synchronize()
    ref_bits = oracle.rmsnorm(dtype, Xb, bits_of(W16), bs, dim, eps=1e-6)
    assert ulp_diff_ok(bits_of(Y), ref_bits, dtype, max_ulp=2, frac=0.99)
    # 1e-2 against the unrounded formula of example/RMSNorm.py:13-18 (both the GPU and the checker)
    exact = rmsnorm_f64(X, W16, 1e-6)
    assert max_rel_err(Y.cpu(), exact) <= REL_TOL
    assert max_rel_err(torch.from_numpy(oracle.from_bits(ref_bits, dtype)).reshape(bs, dim), exact) <= REL_TOL


def test_rmsnorm_constant_row_closed_form(fo):
    dim, c, eps = 512, 3.0, 1e-5
    X = torch.full((4, dim), c, device="cuda", dtype=torch.float16)
    Wt = torch.linspace(0.5, 1.5, dim).to(torch.float16).cuda()
    Y = torch.empty_like(X)
    fo.ops.rmsnorm(X, Y, Wt, eps=eps)
    xn = torch.tensor(c / np.sqrt(c * c + eps), dtype=torch.float32).to(torch.float16)
    expect = (xn.float() * Wt.float().cpu()).to(torch.float16)
    got = Y[0].cpu()
    assert ((got.view(torch.int16).int() - expect.view(torch.int16).int()).abs() <= 1).all()


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_streaming_forms_give_the_same_bits(fo, dtype):
    """Above 192 MB of footprint the consumer's accumulator and the RMSNorm's rows move with
    non-temporal accesses: the values must be those of the cacheable forms that small inputs use."""
    td = TORCH_DTYPE[dtype]
    M = N = 8192                                             # 268 MB per kernel: streaming
    g = torch.Generator(device="cuda").manual_seed(91)
    src = torch.randn(M * N, device="cuda", generator=g).to(td)
    acc = torch.randn(M * N, device="cuda", generator=g).to(td)
    small = 1 << 20                                          # 4 MB: cacheable
    ref_small = acc[:small].clone()
    fo.ops.consumer_reduce(src[:small], ref_small)
    expect = (acc.float() + src.float()).to(td)              # one rounding of the fp32 sum
    fo.ops.consumer_reduce(src, acc)
    torch.cuda.synchronize()
    assert torch.equal(acc, expect)
    assert torch.equal(acc[:small], ref_small)
    # reorder+RMSNorm: the first tile row of the large run against a run on that tile row alone
    bm, bn = 128, 256
    TM, TN = M // bm, N // bn
    ra = torch.randperm(TN, generator=torch.Generator().manual_seed(92)).to(torch.int32)
    RA = (torch.arange(TM, dtype=torch.int32)[:, None] * TN + ra[None, :]).cuda()   # rows of tiles stay together
    X = src.view(M, N)
    Wt = (1 + 0.01 * torch.randn(N, device="cuda", generator=g)).to(td)
    Y = torch.empty(M, N, device="cuda", dtype=td)
    fo.ops.reorder_rmsnorm(X, Y, Wt, bm, bn, 1, RA, eps=1e-6)
    Ys = torch.empty(bm, N, device="cuda", dtype=td)
    fo.ops.reorder_rmsnorm(X[:bm], Ys, Wt, bm, bn, 1, RA[:1].contiguous(), eps=1e-6)
    torch.cuda.synchronize()
    assert torch.equal(Y[:bm], Ys)
    Yp = torch.empty(M, N, device="cuda", dtype=td)
    fo.ops.rmsnorm(X, Yp, Wt, eps=1e-6)
    Yps = torch.empty(bm, N, device="cuda", dtype=td)
    fo.ops.rmsnorm(X[:bm], Yps, Wt, eps=1e-6)
    torch.cuda.synchronize()
    assert torch.equal(Yp[:bm], Yps)
    # Rows from the middle and the end of a streaming-size matrix whose row count is no multiple of the
    # workgroup's four rows (the last workgroup's spare wavefronts lie beyond it) against runs on those
    # rows alone, which take the cacheable form.
    bs2 = M - 3
    Yq = torch.full((M, N), float("nan"), device="cuda", dtype=td)
    fo.ops.rmsnorm(X[:bs2], Yq[:bs2], Wt, eps=1e-6)
    for lo, hi in ((bs2 - 69, bs2), (4001, 4090)):
        Yqs = torch.empty(hi - lo, N, device="cuda", dtype=td)
        fo.ops.rmsnorm(X[lo:hi], Yqs, Wt, eps=1e-6)
        torch.cuda.synchronize()
        assert torch.equal(Yq[lo:hi], Yqs)
        assert torch.equal(Yp[lo:hi], Yqs)
    assert torch.isnan(Yq[bs2:]).all()                       # nothing written beyond the last row
    lo = 37 * bm                                             # a tile row from the middle, reordered form
    Yrs = torch.empty(bm, N, device="cuda", dtype=td)
    fo.ops.reorder_rmsnorm(X[lo:lo + bm], Yrs, Wt, bm, bn, 1, (RA[37:38] - 37 * TN).contiguous(), eps=1e-6)
    torch.cuda.synchronize()
    assert torch.equal(Y[lo:lo + bm], Yrs)


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_reorder_rmsnorm_undoes_the_permutation(fo, oracle, dtype):
    for (bm, bn, M, N, rldn) in [(128, 128, 256, 1024, 1), (128, 256, 256, 4096, 1), (64, 128, 256, 512, 2),
                                 (16, 128, 64, 8192, 1), (32, 96, 64, 480, 1),   # last: BN no power of two
                                 # 128 and 96 tiles per row (slots handed out from two registers per lane; rows of
                                 # more than 8192 elements), 129 tiles per row (beyond the slot registers: general path)
                                 (16, 128, 32, 16384, 1), (32, 128, 64, 12288, 1), (16, 64, 32, 8256, 1)]:
        TM, TN = M // bm, N // bn
        T = TM * TN
        rng = np.random.default_rng(40)
        ra = rng.permutation(T).astype(np.int32)
        plain, pb = seeded((M, N), dtype, 41, scale=1.5)
        _, wb = seeded((N,), dtype, 42)
        Wt = from_bits(wb, dtype)
        # build the reordered buffer on the host with the checker-independent brute force of the address map
        Cp = np.empty(M * N, dtype=np.uint16)
        ldp = rldn * bn
        view = Cp.reshape(-1, ldp)
        for tm in range(TM):
            for tn in range(TN):
                r = ra[tm * TN + tn]
                view[(r // rldn) * bm:(r // rldn + 1) * bm, (r % rldn) * bn:(r % rldn + 1) * bn] = \
                    pb[tm * bm:(tm + 1) * bm, tn * bn:(tn + 1) * bn]
        X = from_bits(Cp, dtype).reshape(M, N)
        RA = torch.from_numpy(ra).cuda()
        Y = torch.empty(M, N, device="cuda", dtype=TORCH_DTYPE[dtype])
        Yp = torch.empty_like(Y)
        fo.ops.reorder_rmsnorm(X, Y, Wt, bm, bn, rldn, RA, eps=1e-6)
        fo.ops.rmsnorm(plain, Yp, Wt, eps=1e-6)
        torch.cuda.synchronize()
        assert torch.equal(Y, Yp)                       # the gather is exact: same bits as plain RMSNorm
        ref_bits = oracle.reorder_rmsnorm(dtype, Cp, wb, M, N, bm, bn, rldn, ra, eps=1e-6)
        assert ulp_diff_ok(bits_of(Y), ref_bits, dtype, max_ulp=2, frac=0.99)
        assert max_rel_err(Y.cpu(), rmsnorm_f64(plain, Wt, 1e-6)) <= REL_TOL


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_gemm_leaves_registers_for_a_consumer_wavefront(fo, dtype):
    """The consumer kernels are built for one 64-register wavefront per SIMD beside the wavefronts
    of a signalling GEMM workgroup (one per SIMD for the 256x256 tile, two for the smaller ones):
    the GEMM's registers per SIMD (architectural + accumulation, allocated in eights) + 64 must fit
    the 512 of a SIMD, or the overlapped path silently degrades into a serial one."""
    for bm, bn, M, N in ((128, 256, 8192, 8192), (128, 256, 4224, 2048), (128, 128, 4224, 4224)):
        algo = _algo(fo, bm, bn, swizzle=4)
        for epilogue in (1, 2):
            info = fo._capi.kernel_info(algo, M, N, epilogue=epilogue, dtype=dtype)
            per_cu = info["resident"] // 256
            assert info["resident"] == 256 * per_cu and per_cu * info["lds_bytes"] <= 160 * 1024
            per_simd = per_cu * info["threads"] // 256
            assert per_simd * ((info["vgprs"] + 7) // 8 * 8) + 64 <= 512, info


def test_error_codes_on_gpu(fo):
    A = torch.zeros(128, 64, device="cuda", dtype=torch.float16)
    C = torch.zeros(128, 128, device="cuda", dtype=torch.float16)
    with pytest.raises(fo.FlashOverlapError) as e:
        fo.ops.gemm(A, torch.zeros(100, 64, device="cuda", dtype=torch.float16),
                    torch.zeros(128, 100, device="cuda", dtype=torch.float16), 0)
    assert e.value.code == -2
    with pytest.raises(fo.FlashOverlapError) as e:
        fo.ops.gemm(A, A, C, 500)
    assert e.value.code == -3
    with pytest.raises(TypeError):
        fo.ops.gemm(A.float(), A.float(), C.float(), 0)


def test_reorder_table_changed_in_place_between_launches(fo):
    """RA is read through the scalar cache, cSeg into registers at kernel start:
    a launch must see what the tensors hold at that time, not what an earlier launch read."""
    bm, bn, M, N, K = 128, 128, 2048, 2048, 128
    algo = _algo(fo, bm, bn, swizzle=4)
    TM, TN = M // bm, N // bn
    T = TM * TN
    A, _ = seeded((M, K), F16, 31)
    B, _ = seeded((N, K), F16, 32, scale=K ** -0.5)
    plain = torch.empty(M, N, device="cuda", dtype=torch.float16)
    fo.ops.gemm(A, B, plain, algo)
    RA = torch.empty(TM, TN, dtype=torch.int32, device="cuda")
    cseg = torch.empty(4, dtype=torch.int32, device="cuda")
    MM = torch.zeros(fo.layout.counter_size(4, TM, TN), dtype=torch.int32, device="cuda")
    Cp = torch.empty(M * N, device="cuda", dtype=torch.float16)
    rng = np.random.default_rng(9)
    for it in range(4):
        perm = torch.from_numpy(rng.permutation(T).astype(np.int32)).reshape(TM, TN)
        cuts = sorted(rng.choice(np.arange(1, T), size=3, replace=False).tolist())
        groups = [b - a for a, b in zip([0] + cuts, cuts + [T])]
        RA.copy_(perm)                                   # same device buffers, new contents
        cseg.copy_(torch.tensor(groups, dtype=torch.int32))
        Cp.fill_(float("nan"))
        fo.ops.gemm_signal(A, B, Cp, MM, RA, cseg, algo)
        torch.cuda.synchronize()
        assert MM[:4].tolist() == groups
        assert torch.equal(fo.layout.unpermute(Cp, M, N, bm, bn, RA), plain)
        MM.zero_()
