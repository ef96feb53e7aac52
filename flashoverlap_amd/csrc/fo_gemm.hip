// Host side of the gfx950 MFMA GEMM: picks the kernel shape for a problem and
// launches it (plain, signal and scatter epilogues).  The device code is in
// fo_gemm_kernel.h.
#include "fo_gemm_kernel.h"

namespace {

using namespace fo_gemm_dev;

// One compiled shape of the kernel template.  The launch is persistent: as many
// workgroups as the device keeps resident at once (or fewer, if the problem has
// fewer macro tiles); each walks the raster with that stride.
// With `resident_out` set nothing is launched: the call only reports how many workgroups the
// launch would hold, and in resident_out[1..3] the kernel's registers per lane, LDS bytes
// and threads per workgroup.
template <typename Tag, int MTM, int MTN, int BK, int SA, int SB, int WM, int WN, int MODE>
int launch_variant(const GemmArgs &a, hipStream_t stream, int *resident_out) {
    auto kern = fo_gemm_kernel<Tag, MTM, MTN, BK, SA, SB, WM, WN, MODE>;
    constexpr int smem = smem_bytes<MTM, MTN, BK, SA, SB>();
    constexpr int threads = WM * WN * 64;
    static int resident = 0;  // per instantiation; the attribute is process wide
    if (!resident) {
        FO_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem));
        int dev = 0, cus = 0, per_cu = 0;
        FO_HIP_CHECK(hipGetDevice(&dev));
        FO_HIP_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        FO_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void *>(kern),
                                                                  threads, smem));
        if (cus <= 0 || per_cu <= 0) return FO_ERR_STATE;
        // a multiple of 8 keeps "workgroup id mod 8 = XCD" true for every tile of the walk
        resident = (cus * per_cu) / 8 * 8;
        if (resident <= 0) resident = cus * per_cu;
    }
    const int ntiles = a.count;
    if (resident_out) {
        hipFuncAttributes attr;
        FO_HIP_CHECK(hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(kern)));
        resident_out[0] = ntiles < resident ? ntiles : resident;
        resident_out[1] = attr.numRegs;
        resident_out[2] = smem;
        resident_out[3] = threads;
        return FO_OK;
    }
    dim3 grid(ntiles < resident ? ntiles : resident), block(threads);
    hipLaunchKernelGGL(kern, grid, block, smem, stream, a);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

// Macro tile -> kernel shape.  256x256 (eight wavefronts, three 32 KiB slots for
// the A part and two for the B part of a K step: all 160 KiB) is the workhorse; the smaller shapes serve problems whose M or N is
// not a multiple of 256 or that have too few 256x256 tiles to fill the chip.
template <typename Tag, int MODE>
int launch_tile(const GemmArgs &a, int mtm, int mtn, hipStream_t stream, int *resident_out) {
    if (mtm == 256 && mtn == 256)
        return launch_variant<Tag, 256, 256, 64, 2, 2, 2, 4, MODE>(a, stream, resident_out);
    if (mtm == 128 && mtn == 128)
        return launch_variant<Tag, 128, 128, 64, 2, 2, 2, 2, MODE>(a, stream, resident_out);
    if (mtm == 128 && mtn == 256)
        return launch_variant<Tag, 128, 256, 64, 3, 3, 2, 4, MODE>(a, stream, resident_out);
    if (mtm == 256 && mtn == 128)
        return launch_variant<Tag, 256, 128, 64, 3, 3, 2, 2, MODE>(a, stream, resident_out);
    return FO_ERR_ALGO;
}

template <int MODE>
int launch_dtype(int dtype, const GemmArgs &a, int mtm, int mtn, hipStream_t stream, int *resident_out = nullptr) {
    if (dtype == FO_F16) return launch_tile<fo_f16_tag, MODE>(a, mtm, mtn, stream, resident_out);
    if (dtype == FO_BF16) return launch_tile<fo_bf16_tag, MODE>(a, mtm, mtn, stream, resident_out);
    return FO_ERR_DTYPE;
}

int run_gemm(int mode, int dtype, int M, int N, int K, int rLDN, const int32_t *cseg, int G,
             const void *A, const void *B, void *C, int32_t *MM, const int32_t *RA,
             const int32_t *RE, int monitor, int algo, fo_stream_t stream, bool quiet = false) {
    if (dtype != FO_F16 && dtype != FO_BF16) return FO_ERR_DTYPE;
    const fo_algo_entry *e = fo_algo_lookup(algo);
    if (!e) return FO_ERR_ALGO;
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return FO_ERR_ARG;
    fo_raster r;
    int rc = fo_pick_raster(algo, M, N, &r);
    if (rc) return rc;
    if (K % 8) return FO_ERR_SHAPE;  // operand rows are fetched in 16-byte chunks
    // the epilogue assumes a wavefront's 128 x 64 (or 64 x 64) block lies inside one reorder tile
    if (e->f[0] % 128 || e->f[1] % 128) return FO_ERR_ALGO;
    GemmArgs a;
    a.A = static_cast<const uint16_t *>(A);
    a.B = static_cast<const uint16_t *>(B);
    a.C = static_cast<uint16_t *>(C);
    a.M = M; a.N = N; a.K = K;
    a.lda = K; a.ldb = K;
    a.BM = e->f[0]; a.BN = e->f[1];
    a.TN = N / a.BN;
    a.rLDN = rLDN;
    a.RA = RA; a.RE = RE; a.cseg = cseg; a.G = G; a.MM = MM; a.monitor = monitor;
    a.grid_m = r.grid_m; a.grid_n = r.grid_n; a.panel = r.panel; a.xcd_remap = r.xcd_remap;
    a.first = 0; a.sub_m = a.sub_n = 1;
    a.count = r.grid_m * r.grid_n - r.tail_tiles;
    a.quiet = quiet ? 1 : 0;
    if (mode != MODE_PLAIN) {
        const long T = (long)(M / a.BM) * a.TN;
        if ((!MM && !quiet) || !RA || !cseg) return FO_ERR_ARG;
        if (mode == MODE_SCATTER && !RE) return FO_ERR_ARG;
        if (rLDN <= 0 || T % rLDN) return FO_ERR_SHAPE;
        if (G <= 0 || G > T) return FO_ERR_SEGMENTS;
        if (monitor && G > a.TN - 1) return FO_ERR_SEGMENTS;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto launch = [&](const GemmArgs &g, int mtm, int mtn) {
        switch (mode) {
            case MODE_PLAIN: return launch_dtype<MODE_PLAIN>(dtype, g, mtm, mtn, s);
            case MODE_SIGNAL: return launch_dtype<MODE_SIGNAL>(dtype, g, mtm, mtn, s);
            default: return launch_dtype<MODE_SCATTER>(dtype, g, mtm, mtn, s);
        }
    };
    rc = launch(a, r.mtm, r.mtn);
    if (rc || !r.tail_tiles) return rc;
    // the last, partial wave of 256x256 tiles: the same raster positions in the Algo's own tile
    GemmArgs t = a;
    t.first = a.count;
    t.sub_m = r.tail_sub_m; t.sub_n = r.tail_sub_n;
    t.count = r.tail_tiles * r.tail_sub_m * r.tail_sub_n;
    return launch(t, a.BM, a.BN);
}

}  // namespace

// The reordered (optionally row-mapped) store of the signalling GEMMs without
// their counters, for a caller that orders GEMM and consumer by the stream alone.
int fo_gemm_reordered_quiet(int dtype, int M, int N, int K, int rLDN, const int32_t *cseg_dev, int G,
                            const void *A, const void *B, void *C, const int32_t *RA, const int32_t *RE,
                            int algo, fo_stream_t stream) {
    return run_gemm(RE ? MODE_SCATTER : MODE_SIGNAL, dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, nullptr, RA, RE,
                    0, algo, stream, true);
}

extern "C" int fo_gemm_wave_tiles(int dtype, int algo, int M, int N, int32_t *tiles) {
    if (!tiles) return FO_ERR_ARG;
    const fo_algo_entry *e = fo_algo_lookup(algo);
    if (!e) return FO_ERR_ALGO;
    fo_raster r;
    int rc = fo_pick_raster(algo, M, N, &r);
    if (rc) return rc;
    GemmArgs a = {};
    a.grid_m = r.grid_m;
    a.grid_n = r.grid_n;
    a.count = r.grid_m * r.grid_n - r.tail_tiles;
    int info[4] = {0, 0, 0, 0};
    rc = launch_dtype<MODE_SIGNAL>(dtype, a, r.mtm, r.mtn, nullptr, info);
    if (rc) return rc;
    *tiles = info[0] * (r.mtm / e->f[0]) * (r.mtn / e->f[1]);
    return FO_OK;
}

extern "C" int fo_gemm_kernel_info(int dtype, int algo, int M, int N, int epilogue, int32_t info[4]) {
    if (!info) return FO_ERR_ARG;
    fo_raster r;
    int rc = fo_pick_raster(algo, M, N, &r);
    if (rc) return rc;
    GemmArgs a = {};
    a.grid_m = r.grid_m;
    a.grid_n = r.grid_n;
    a.count = r.grid_m * r.grid_n - r.tail_tiles;
    int out[4] = {0, 0, 0, 0};
    switch (epilogue) {
        case MODE_PLAIN: rc = launch_dtype<MODE_PLAIN>(dtype, a, r.mtm, r.mtn, nullptr, out); break;
        case MODE_SIGNAL: rc = launch_dtype<MODE_SIGNAL>(dtype, a, r.mtm, r.mtn, nullptr, out); break;
        case MODE_SCATTER: rc = launch_dtype<MODE_SCATTER>(dtype, a, r.mtm, r.mtn, nullptr, out); break;
        default: return FO_ERR_ARG;
    }
    if (rc) return rc;
    for (int i = 0; i < 4; i++) info[i] = out[i];
    return FO_OK;
}

extern "C" int fo_gemm(int dtype, int M, int N, int K, const void *A, const void *B, void *C,
                       int algo, fo_stream_t stream) {
    return run_gemm(MODE_PLAIN, dtype, M, N, K, 1, nullptr, 0, A, B, C, nullptr, nullptr, nullptr, 0,
                    algo, stream);
}

extern "C" int fo_gemm_signal(int dtype, int M, int N, int K, int rLDN, const int32_t *cseg_dev,
                              int G, const void *A, const void *B, void *C, int32_t *MM,
                              const int32_t *RA, int monitor, int algo, fo_stream_t stream) {
    return run_gemm(MODE_SIGNAL, dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, MM, RA, nullptr,
                    monitor, algo, stream);
}

extern "C" int fo_gemm_scatter(int dtype, int M, int N, int K, int rLDN, const int32_t *cseg_dev,
                               int G, const void *A, const void *B, void *C, int32_t *MM,
                               const int32_t *RA, const int32_t *RE, int monitor, int algo,
                               fo_stream_t stream) {
    return run_gemm(MODE_SCATTER, dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, MM, RA, RE, monitor,
                    algo, stream);
}
