"""The allocation-free entry point against the handle-based call it is a variant of.

fo_gemm_allreduce_overlap_static keeps the group counters and the flag words of fork, join and the
one-launch consumer in a static device array inside the library; fo_overlap_gemm_allreduce gets
the counters from the caller (MM) and the flag words from the workspace its handle allocated.
Same kernels, same operands: the reordered output and the accumulator must agree bit for bit
(integer bar: the permutation; floating point: identical kernels give identical bits).  Two calls
in a row, the second on a smaller problem with fewer groups, so that what the first call left in
the array (counters back at zero, flag words) is what the second one starts from."""
import pytest
import torch

from gpu_util import F16, seeded

pytestmark = pytest.mark.gpu


def _case(fo, M, N, K, bm, bn, cseg, fused, two_streams, seed):
    algo = fo._capi.find_algo(bm, bn, swizzle=4)
    TM, TN = M // bm, N // bn
    T = TM * TN
    assert sum(cseg) == T
    RA = fo.layout.reorder_indices(T, fo._capi.schedule_order(algo, M, N), device="cuda").reshape(TM, TN)
    A, _ = seeded((M, K), F16, seed)
    B, _ = seeded((N, K), F16, seed + 1, scale=K ** -0.5)
    acc0, _ = seeded((M * N,), F16, seed + 2, scale=0.5)
    cs_cpu = torch.tensor(cseg, dtype=torch.int32)
    cs_gpu = cs_cpu.cuda()
    # the existing entry point: handle, caller's MM
    MM = torch.zeros(fo.layout.counter_size(len(cseg), TM, TN), dtype=torch.int32, device="cuda")
    C_ref = torch.full((M * N,), float("nan"), device="cuda", dtype=torch.float16)
    acc_ref = acc0.clone()
    ov = fo.ops.Overlap()
    ov.set_fused_consumer(fused)
    ov.set_accumulator(acc_ref)
    ov.gemm_allreduce_overlap(A, B, C_ref, MM, RA, 1, cs_cpu, cs_gpu, algo)
    torch.cuda.synchronize()
    assert ov.status() == 0 and (MM == 0).all()
    ov.close()
    # the allocation-free entry point: everything allocated before the call, nothing inside it
    C = torch.full((M * N,), float("nan"), device="cuda", dtype=torch.float16)
    acc = acc0.clone()
    comm = torch.cuda.Stream() if two_streams else None
    fo.ops.static_status(comm_stream=comm)       # first use of the library's static array happens here, not below
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]   # the driver's free bytes: sees a hipMalloc that torch's allocator would not
    fo.ops.gemm_allreduce_overlap_static(A, B, C, acc, RA, 1, cs_cpu, cs_gpu, algo, fused=fused, comm_stream=comm)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] >= free_before   # nothing was taken from the device's memory
    assert fo.ops.static_status(comm_stream=comm) == 0   # no bounded wait gave up
    assert torch.equal(C, C_ref)                 # reordered tiles: bit-exact
    assert torch.equal(acc, acc_ref)             # consumer: bit-exact
    plain = torch.empty(M, N, device="cuda", dtype=torch.float16)
    fo.ops.gemm(A, B, plain, algo)
    assert torch.equal(fo.layout.unpermute(C, M, N, bm, bn, RA), plain)


@pytest.mark.parametrize("fused,two_streams", [(0, True), (1, True), (-1, False)])
def test_static_call_matches_the_handle_call_twice_in_a_row(fo, fused, two_streams):
    # first call: 256 tiles in 8 groups; second call, smaller: 64 tiles in 3 groups
    _case(fo, 2048, 2048, 512, 128, 128, [32] * 8, fused, two_streams, seed=300)
    _case(fo, 1024, 1024, 256, 128, 128, [16, 16, 32], fused, two_streams, seed=310)


def test_static_call_rejects_what_it_cannot_hold(fo):
    M = N = 1024
    algo = fo._capi.find_algo(128, 128)
    A, _ = seeded((M, 64), F16, 1)
    C = torch.empty(M * N, device="cuda", dtype=torch.float16)
    RA = torch.arange(64, dtype=torch.int32, device="cuda").reshape(8, 8)
    too_many = torch.ones(4097, dtype=torch.int32)
    with pytest.raises(fo.FlashOverlapError) as e:       # more groups than the static array has counters
        fo.ops.gemm_allreduce_overlap_static(A, A, C, None, RA, 1, too_many, too_many.cuda(), algo)
    assert e.value.code == -7
    bad = torch.tensor([32, 31], dtype=torch.int32)      # does not cover the 64 tiles
    with pytest.raises(fo.FlashOverlapError) as e:
        fo.ops.gemm_allreduce_overlap_static(A, A, C, None, RA, 1, bad, bad.cuda(), algo)
    assert e.value.code == -5
