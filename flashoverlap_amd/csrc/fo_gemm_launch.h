// Launch of one compiled GEMM kernel, shared by the translation units that hold
// kernel instantiations (fo_gemm.hip, fo_gemm256_inst.hip).
#pragma once

#include <atomic>
#include <mutex>

#include "fo_gemm_kernel.h"

namespace fo_gemm_dev {

constexpr int kMaxDevices = 64;

// CUs that the GEMM launches may count on (0: all of the device's).  A caller that keeps CUs for other
// kernels, e.g. with CU-masked streams, says so through fo_gemm_set_cu_limit; the persistent launches
// and the raster (with it the schedule order handed out as the hint) then assume that many CUs, as the
// reference's tuner assumes sm_count - 2 (tune/search.py:404-407).
inline std::atomic<int> &gemm_cu_limit() {
    static std::atomic<int> limit{0};
    return limit;
}

// One compiled shape of the kernel template.  The launch is persistent: as many
// workgroups as the device keeps resident at once (or fewer, if the problem has
// fewer macro tiles); each walks the raster with that stride.
// With `resident_out` set nothing is launched: the call only reports how many workgroups the
// launch would hold, in resident_out[1..3] the kernel's registers per lane, LDS bytes and
// threads per workgroup, and in resident_out[4] how many workgroups stay resident at most.
// expect_resident > 0: refuse (FO_ERR_STATE) unless that many stay resident.
template <auto KERN, int SMEM, int THREADS>
inline int launch_kernel(const GemmArgs &a, hipStream_t stream, int *resident_out, int expect_resident) {
    auto kern = KERN;
    constexpr int smem = SMEM;
    constexpr int threads = THREADS;
    // CUs of each device and workgroups of this instantiation per CU; the LDS attribute is set once per device too.
    static std::mutex mu;
    static int cus_of[kMaxDevices], per_cu_of[kMaxDevices];
    int dev = 0;
    FO_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return FO_ERR_STATE;
    int resident;
    {
        std::lock_guard<std::mutex> lock(mu);
        if (!per_cu_of[dev]) {
            FO_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, smem));
            int cus = 0, per_cu = 0;
            FO_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
            FO_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(kern),
                                                                      threads, smem));
            if (cus <= 0 || per_cu <= 0) return FO_ERR_STATE;
            cus_of[dev] = cus;
            per_cu_of[dev] = per_cu;
        }
        const int limit = gemm_cu_limit().load(std::memory_order_relaxed);
        const int cus = limit > 0 && limit < cus_of[dev] ? limit : cus_of[dev];
        // a multiple of 8 keeps "workgroup id mod 8 = XCD" true for every tile of the walk
        const int r = (cus * per_cu_of[dev]) / 8 * 8;
        resident = r > 0 ? r : cus * per_cu_of[dev];
    }
    // The raster (and with it the schedule order handed to the caller as the hint) was laid out for
    // expect_resident workgroups; a launch that would hold another number walks the tiles differently.
    if (expect_resident > 0 && resident != expect_resident) return FO_ERR_STATE;
    const int ntiles = a.count;
    if (resident_out) {
        hipFuncAttributes attr;
        FO_HIP_CHECK(hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kern)));
        resident_out[0] = ntiles < resident ? ntiles : resident;
        resident_out[1] = attr.numRegs;
        resident_out[2] = smem;
        resident_out[3] = threads;
        resident_out[4] = resident;
        return FO_OK;
    }
    dim3 grid(ntiles < resident ? ntiles : resident), block(threads);
    hipLaunchKernelGGL(kern, grid, block, smem, stream, a);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

// The 256x256 kernel (fo_gemm256_kernel.h) for dtype FO_F16 / FO_BF16 and epilogue MODE_PLAIN /
// MODE_SIGNAL / MODE_SCATTER; same arguments as launch_kernel.  One definition per instantiation
// (fo_gemm256_inst.hip compiled with FO_INST_DTYPE and FO_INST_MODE), dispatched in fo_gemm.hip.
int fo_gemm256_launch(int dtype, int mode, const GemmArgs &a, hipStream_t stream, int *resident_out, int expect_resident);
#define FO_GEMM256_INST_DECL(D_, M_) \
    int fo_gemm256_launch_##D_##_##M_(const GemmArgs &a, hipStream_t stream, int *resident_out, int expect_resident);
FO_GEMM256_INST_DECL(0, 0) FO_GEMM256_INST_DECL(0, 1) FO_GEMM256_INST_DECL(0, 2)
FO_GEMM256_INST_DECL(1, 0) FO_GEMM256_INST_DECL(1, 1) FO_GEMM256_INST_DECL(1, 2)
#undef FO_GEMM256_INST_DECL

}  // namespace fo_gemm_dev
