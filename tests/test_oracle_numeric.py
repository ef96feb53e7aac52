"""Pins the arithmetic half of the CPU checker (oracle/fo_oracle.c): 16-bit
conversions against numpy, the signal GEMM against torch's fp32 matmul, exact
special cases, a brute-force address map and the round trip; RMSNorm against the
textbook formula of example/RMSNorm.py:13-18; the consumer, the host schedule and
the latency model against hand-computed cases."""
import numpy as np
import pytest
import torch

F16, BF16 = 0, 1


def _rand_bits(o, shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g) * scale
    return o.to_bits(x.numpy(), dtype)


def _torch_dtype(dtype):
    return torch.float16 if dtype == F16 else torch.bfloat16


def _as_torch(o, bits, dtype):
    return torch.from_numpy(o.from_bits(bits, dtype))


# ---------------------------------------------------------------- conversions
def test_f16_conversions_exhaustive(oracle):
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 7):  # every 7th pattern, both directions
        f = L.fo_oracle_f16_to_f32(int(b))
        if np.isnan(ref[b]):
            assert np.isnan(f)
        else:
            assert f == ref[b]
            assert L.fo_oracle_f32_to_f16(float(ref[b])) == b or ref[b] == 0  # -0/+0 keep sign below
    assert L.fo_oracle_f32_to_f16(-0.0) == 0x8000


def test_f32_to_16bit_rounding_matches_numpy_and_torch(oracle):
    L = oracle.lib()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 4000),
        np.array([0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5,
                  1.0009766, 1.00048828125, 1.00146484375], dtype=np.float32)])
    with np.errstate(over="ignore"):
        ref16 = xs.astype(np.float16).view(np.uint16)
    refbf = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    for x, r16, rbf in zip(xs, ref16, refbf):
        assert L.fo_oracle_f32_to_f16(float(x)) == r16, x
        assert L.fo_oracle_f32_to_bf16(float(x)) == rbf, x
    assert (oracle.to_bits(xs, BF16) == refbf).all()


# ---------------------------------------------------------------- GEMM + reorder + signal
@pytest.mark.parametrize("dtype", [F16, BF16])
def test_gemm_values_match_torch_fp32(oracle, dtype):
    M, N, K, BM, BN = 64, 96, 128, 16, 32
    A = _rand_bits(oracle, (M, K), dtype, 1)
    B = _rand_bits(oracle, (N, K), dtype, 2, scale=K ** -0.5)
    C, _ = oracle.gemm_signal(dtype, A, B, BM, BN)
    ref = _as_torch(oracle, A, dtype) @ _as_torch(oracle, B, dtype).T
    got = _as_torch(oracle, C, dtype)
    # one rounding of an fp32 sum: within one 16-bit ulp of torch's fp32 result
    tol = 2.0 ** (-10 if dtype == F16 else -7)
    assert torch.allclose(got, ref, rtol=tol, atol=tol)
    # transposed-operand or wrong-index mistakes would give errors of order 1
    assert (got - ref).abs().max() < 0.05


def test_gemm_all_ones_is_exactly_K(oracle):
    # the reference's own correctness input (example/correctness_ar.py:24-25)
    M, N, K, BM, BN = 32, 32, 256, 16, 16
    ones = oracle.to_bits(np.ones((M, K), np.float32), F16)
    TM, TN = M // BM, N // BN
    ra = oracle.reorder_indices(TM * TN, [3, 1])
    C, MM = oracle.gemm_signal(F16, ones, ones[:N], BM, BN, RA=ra, cseg=[1, 3])
    assert (oracle.from_bits(C, F16) == K).all()
    assert MM[:2].tolist() == [1, 3]


def test_gemm_identity_weight_copies_A(oracle):
    M, K = 32, 64
    A = _rand_bits(oracle, (M, K), F16, 3)
    eye = oracle.to_bits(np.eye(K, dtype=np.float32), F16)  # B[N=K, K] = I  =>  C = A
    C, _ = oracle.gemm_signal(F16, A, eye, 16, 16)
    assert (C == A).all()


def test_reordered_store_brute_force_and_round_trip(oracle):
    M, N, K, BM, BN = 8, 12, 16, 2, 3
    TM, TN = M // BM, N // BN
    T = TM * TN
    rng = np.random.default_rng(5)
    A = _rand_bits(oracle, (M, K), F16, 6)
    B = _rand_bits(oracle, (N, K), F16, 7)
    plain, _ = oracle.gemm_signal(F16, A, B, BM, BN)
    ra = rng.permutation(T).astype(np.int32)
    for rldn in (1, 2, 4):
        cseg = [5, 4, 7]
        Cp, MM = oracle.gemm_signal(F16, A, B, BM, BN, RA=ra, cseg=cseg, rLDN=rldn)
        ldp = rldn * BN
        for m in range(M):          # element-by-element statement of map_to_d
            for n in range(N):
                r = ra[(m // BM) * TN + n // BN]
                assert Cp[((r // rldn) * BM + m % BM) * ldp + (r % rldn) * BN + n % BN] == plain[m, n]
        assert (oracle.unpermute(Cp, M, N, BM, BN, ra, rLDN=rldn) == plain).all()
        assert MM[:3].tolist() == cseg
    # identity RA with rLDN = TN is plain row-major
    Cp, _ = oracle.gemm_signal(F16, A, B, BM, BN, RA=np.arange(T, dtype=np.int32), cseg=[T], rLDN=TN)
    assert (Cp.reshape(M, N) == plain).all()


def test_scatter_rows_end_to_end_identity(oracle):
    # With BM % W == 0, rank q's [M/W, N] segment is a tile-reordered buffer with tile
    # (BM/W, BN) and the same RA; un-permuted it is rows q, q+W, ... of the full product
    # (example/correctness_rs.py:26,33 + src/overlap_impl.cu:312).
    M, N, K, BM, BN, W = 32, 16, 32, 8, 8, 4
    TM, TN = M // BM, N // BN
    T = TM * TN
    A = _rand_bits(oracle, (M, K), F16, 8)
    B = _rand_bits(oracle, (N, K), F16, 9)
    plain, _ = oracle.gemm_signal(F16, A, B, BM, BN)
    hint = [5, 0, 7, 2]
    ra = oracle.reorder_indices(T, hint)
    cseg = [2, 2, 4]
    re_ = oracle.row_mapping(M, N, BM, BN, cseg, W)
    Cp, MM = oracle.gemm_signal(F16, A, B, BM, BN, RA=ra, cseg=cseg, RE=re_)
    assert MM[:3].tolist() == cseg
    # emulate reduce-scatter of every group into W segments (one rank present)
    D = np.zeros((W, M // W * N), dtype=np.uint16)
    MM2 = MM.copy()
    rc = oracle.host_schedule(F16, BM * BN, cseg, MM2, Cp, ACC=D.reshape(-1), W=W,
                              seg_stride=M // W * N)
    assert rc == 0 and MM2[:3].tolist() == [0, 0, 0]
    for q in range(W):
        seg = oracle.unpermute(D[q], M // W, N, BM // W, BN, ra)
        assert (seg == plain[q::W]).all()
    assert (oracle.unpermute(Cp, M, N, BM, BN, ra, RE=re_) == plain).all()


def test_signal_counts_and_monitor_stamps(oracle):
    M, N, K, BM, BN = 16, 32, 16, 4, 4
    TM, TN = M // BM, N // BN
    T = TM * TN
    A = _rand_bits(oracle, (M, K), F16, 10)
    B = _rand_bits(oracle, (N, K), F16, 11)
    rng = np.random.default_rng(12)
    order = rng.permutation(T).astype(np.int32)      # completion order
    ra = np.arange(T, dtype=np.int32)                # monitor runs use the identity RA
    cseg = oracle.cseg_from_waves(T, 6)
    _, MM = oracle.gemm_signal(F16, A, B, BM, BN, RA=ra, cseg=cseg, monitor=True, order=order)
    assert MM[:len(cseg)].tolist() == cseg.tolist()
    assert MM[TN - 1] == T                                      # the order counter
    stamps = MM[TN:TN + T]
    assert sorted(stamps.tolist()) == list(range(T))            # a permutation of 0..T-1
    assert all(stamps[order[s]] == s for s in range(T))         # tile finished s-th gets stamp s
    with pytest.raises(ValueError):
        oracle.gemm_signal(F16, A, B, BM, BN, RA=ra, cseg=[T - 1])  # sum(cSeg) != T


# ---------------------------------------------------------------- wait / consumer / schedule
def test_wait_poll_semantics(oracle):
    c = np.array([3], dtype=np.int32)
    assert not oracle.wait_poll(4, c) and c[0] == 3     # not yet: untouched, keeps spinning
    c[0] = 4
    assert oracle.wait_poll(4, c) and c[0] == 0         # released and reset
    assert not oracle.wait_poll(4, c)


def test_wait_poll_threaded_counter(oracle):
    import threading
    import time
    c = np.zeros(1, dtype=np.int32)
    released = []

    def waiter():
        while not oracle.wait_poll(5, c):
            time.sleep(0.0005)
        released.append(True)

    t = threading.Thread(target=waiter)
    t.start()
    for _ in range(5):
        time.sleep(0.002)
        assert not released
        c[0] += 1
    t.join(timeout=5)
    assert released and c[0] == 0


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_consumer_closed_form(oracle, dtype):
    src = _rand_bits(oracle, (4096,), dtype, 13)
    acc = np.zeros(4096, dtype=np.uint16)
    oracle.consumer_reduce(dtype, src, acc)
    assert (acc == src).all()                                   # 0 + x = x
    oracle.consumer_reduce(dtype, src, acc)
    two = oracle.to_bits(2 * oracle.from_bits(src, dtype), dtype)
    assert (acc == two).all()                                   # doubling is exact
    oracle.consumer_reduce(dtype, src, acc)                     # 3x: one rounding of the fp32 sum
    t = _torch_dtype(dtype)
    ref = (_as_torch(oracle, two, dtype) + _as_torch(oracle, src, dtype)).to(t)
    assert torch.equal(_as_torch(oracle, acc, dtype).to(t), ref)


def test_host_schedule_detects_missing_signal(oracle):
    cseg = [2, 3]
    MM = np.array([2, 2], dtype=np.int32)       # group 1 is one tile short
    C = np.zeros(5 * 8, dtype=np.uint16)
    assert oracle.host_schedule(F16, 8, cseg, MM, C) == 2    # stuck at group index 1
    assert MM.tolist() == [0, 2]


# ---------------------------------------------------------------- RMSNorm
def _textbook_rmsnorm(x16, w16, eps):
    x = x16.float()
    out = (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)).type_as(x16)
    return out * w16


@pytest.mark.parametrize("dtype", [F16, BF16])
def test_rmsnorm_matches_textbook(oracle, dtype):
    bs, dim = 16, 256
    t = _torch_dtype(dtype)
    X = _rand_bits(oracle, (bs, dim), dtype, 14, scale=3.0)
    W = oracle.to_bits(1 + 0.01 * torch.randn(dim, generator=torch.Generator().manual_seed(15)).numpy(), dtype)
    got = _as_torch(oracle, oracle.rmsnorm(dtype, X, W, bs, dim, eps=1e-6), dtype)
    ref = _textbook_rmsnorm(_as_torch(oracle, X, dtype).to(t), _as_torch(oracle, W, dtype).to(t), 1e-6).float()
    ulp = 2.0 ** (-9 if dtype == F16 else -6)   # rsqrt/sum-order differences move a value by <= 1-2 ulp
    assert torch.allclose(got, ref, rtol=ulp, atol=1e-6)


def test_rmsnorm_constant_row_closed_form(oracle):
    dim, c, eps = 64, 3.0, 1e-5
    X = oracle.to_bits(np.full((1, dim), c, np.float32), F16)
    W = oracle.to_bits(np.linspace(0.5, 1.5, dim).astype(np.float32), F16)
    got = oracle.rmsnorm(F16, X, W, 1, dim, eps=eps)
    xn = np.float32(c) * np.float32(1.0) / np.sqrt(np.float32(c * c) + np.float32(eps))
    xn16 = np.float32(xn).astype(np.float16)
    expect = (xn16.astype(np.float32) * oracle.from_bits(W, F16)).astype(np.float16)
    assert (got.reshape(-1).view(np.float16) == expect).all()


def test_reorder_rmsnorm_equals_rmsnorm_of_unpermuted(oracle):
    M, N, K, BM, BN = 16, 64, 32, 4, 16
    TM, TN = M // BM, N // BN
    T = TM * TN
    A = _rand_bits(oracle, (M, K), F16, 16)
    B = _rand_bits(oracle, (N, K), F16, 17)
    W = _rand_bits(oracle, (N,), F16, 18)
    plain, _ = oracle.gemm_signal(F16, A, B, BM, BN)
    ref = oracle.rmsnorm(F16, plain, W, M, N)
    rng = np.random.default_rng(19)
    ra = rng.permutation(T).astype(np.int32)
    for rldn in (1, 2):
        Cp, _ = oracle.gemm_signal(F16, A, B, BM, BN, RA=ra, cseg=[T], rLDN=rldn)
        got = oracle.reorder_rmsnorm(F16, Cp, W, M, N, BM, BN, rldn, ra)
        assert (got == ref).all()
    ident = np.arange(T, dtype=np.int32)  # identity RA over a row-major buffer (rldn = TN)
    assert (oracle.reorder_rmsnorm(F16, plain, W, M, N, BM, BN, TN, ident) == ref).all()


# ---------------------------------------------------------------- latency model / compositions
def test_compositions(oracle):
    assert oracle.compositions(1) == [[1]]
    assert oracle.compositions(3) == [[1, 1, 1], [1, 2], [2, 1], [3]]
    c8 = oracle.compositions(8)
    assert len(c8) == 128 and all(sum(c) == 8 for c in c8)


def test_predict_latency_hand_cases(oracle):
    GiB = 1024.0 ** 3
    sizes, bw = [1e6, 2e6, 4e6], [1.0, 2.0, 2.0]  # GiB/ms
    # interpolation: clamped left, linear inside, clamped right
    assert oracle.interp_latency(sizes, bw, 5e5, 6.0) == pytest.approx(5e5 * 6 / 1.0 / GiB)
    assert oracle.interp_latency(sizes, bw, 1.5e6, 6.0) == pytest.approx(1.5e6 * 6 / 1.5 / GiB)
    assert oracle.interp_latency(sizes, bw, 8e6, 6.0) == pytest.approx(8e6 * 6 / 2.0 / GiB)
    M = N = 2048
    tiles, wave = 64, 16
    per_tile = M * N // tiles
    comm = lambda t: oracle.interp_latency(sizes, bw, per_tile * t, 6.0)
    # one group: gemm then the whole stage
    assert oracle.predict_latency(M, N, 1.0, sizes, bw, [64], tiles, wave, wave, 6.0) == \
        pytest.approx(1.0 + comm(64))
    # two equal groups, compute-bound: gemm + last group's stage
    assert oracle.predict_latency(M, N, 1.0, sizes, bw, [32, 32], tiles, wave, wave, 6.0) == \
        pytest.approx(1.0 + comm(32))
    # stage slower than compute: first group's compute + both stages back to back
    slow = [1e-3, 1e-3, 1e-3]
    c32 = oracle.interp_latency(sizes, slow, per_tile * 32, 6.0)
    assert oracle.predict_latency(M, N, 1.0, sizes, slow, [32, 32], tiles, wave, wave, 6.0) == \
        pytest.approx(0.5 + 2 * c32)
    # fewer tiles per wave when co-running stretches the GEMM: 64/16=4 -> 64/15 -> 5 waves
    assert oracle.predict_latency(M, N, 1.0, sizes, bw, [30, 34], tiles, 15, 16, 6.0) == \
        pytest.approx(1.25 / 5 * (2 + 3) + comm(34))
