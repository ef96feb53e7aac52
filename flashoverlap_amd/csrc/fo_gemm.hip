// Host side of the gfx950 MFMA GEMM: picks the kernel shape for a problem and
// launches it (plain, signal and scatter epilogues).  The device code is in
// fo_gemm_kernel.h and fo_gemm256_kernel.h; the latter's six instantiations are
// compiled in translation units of their own (fo_gemm256_inst.hip).
#include <atomic>

#include "fo_gemm_kernel.h"
#include "fo_gemm_launch.h"

namespace {

using namespace fo_gemm_dev;

}  // namespace

int fo_gemm_dev::fo_gemm256_launch(int dtype, int mode, const GemmArgs &a, hipStream_t stream, int *resident_out,
                                   int expect_resident) {
    if (a.lda != a.ldb) return FO_ERR_ARG;  // the kernel addresses both operands with one leading dimension
    const int key = (dtype == FO_BF16 ? 3 : 0) + mode;
    switch (key) {
        case 0: return fo_gemm256_launch_0_0(a, stream, resident_out, expect_resident);
        case 1: return fo_gemm256_launch_0_1(a, stream, resident_out, expect_resident);
        case 2: return fo_gemm256_launch_0_2(a, stream, resident_out, expect_resident);
        case 3: return fo_gemm256_launch_1_0(a, stream, resident_out, expect_resident);
        case 4: return fo_gemm256_launch_1_1(a, stream, resident_out, expect_resident);
        case 5: return fo_gemm256_launch_1_2(a, stream, resident_out, expect_resident);
    }
    return FO_ERR_ARG;
}

namespace {

template <typename Tag, int MTM, int MTN, int BK, int SA, int SB, int WM, int WN, int MODE>
int launch_variant(const GemmArgs &a, hipStream_t stream, int *resident_out, int expect_resident) {
    return launch_kernel<fo_gemm_kernel<Tag, MTM, MTN, BK, SA, SB, WM, WN, MODE>, smem_bytes<MTM, MTN, BK, SA, SB>(),
                         WM * WN * 64>(a, stream, resident_out, expect_resident);
}

// Macro tile -> kernel.  256x256 (fo_gemm256_kernel.h: four wavefronts of 128x128, two 64 KiB slots) is
// the workhorse; the smaller shapes (fo_gemm_kernel.h: three slots for 128x256 and 256x128, two for
// 128x128) serve problems whose M or N is not a multiple of 256 or that have too few 256x256 tiles to
// fill the chip.
template <typename Tag, int MODE>
int launch_tile(const GemmArgs &a, int mtm, int mtn, hipStream_t stream, int *resident_out, int expect_resident) {
    if (mtm == 256 && mtn == 256)
        return fo_gemm256_launch(std::is_same<Tag, fo_bf16_tag>::value ? FO_BF16 : FO_F16, MODE, a, stream, resident_out,
                                 expect_resident);
    if (mtm == 128 && mtn == 128)
        return launch_variant<Tag, 128, 128, 64, 2, 2, 2, 2, MODE>(a, stream, resident_out, expect_resident);
    if (mtm == 128 && mtn == 256)
        return launch_variant<Tag, 128, 256, 64, 3, 3, 2, 4, MODE>(a, stream, resident_out, expect_resident);
    if (mtm == 256 && mtn == 128)
        return launch_variant<Tag, 256, 128, 64, 3, 3, 2, 2, MODE>(a, stream, resident_out, expect_resident);
    return FO_ERR_ALGO;
}

template <int MODE>
int launch_dtype(int dtype, const GemmArgs &a, int mtm, int mtn, hipStream_t stream, int *resident_out = nullptr,
                 int expect_resident = 0) {
    if (dtype == FO_F16) return launch_tile<fo_f16_tag, MODE>(a, mtm, mtn, stream, resident_out, expect_resident);
    if (dtype == FO_BF16) return launch_tile<fo_bf16_tag, MODE>(a, mtm, mtn, stream, resident_out, expect_resident);
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
    if (K > (1 << 21)) return FO_ERR_SHAPE;  // 256 operand rows are addressed through one 31-bit buffer range
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
    a.stream_out = (int64_t)M * N * 2 > kStreamOutAboveBytes ? 1 : 0;
    if (mode != MODE_PLAIN) {
        const long T = (long)(M / a.BM) * a.TN;
        if ((!MM && !quiet) || !RA || !cseg) return FO_ERR_ARG;
        if (mode == MODE_SCATTER && !RE) return FO_ERR_ARG;
        if (rLDN <= 0 || T % rLDN) return FO_ERR_SHAPE;
        if (G <= 0 || G > T) return FO_ERR_SEGMENTS;
        if (monitor && G > a.TN - 1) return FO_ERR_SEGMENTS;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto launch = [&](const GemmArgs &g, int mtm, int mtn, int expect) {
        switch (mode) {
            case MODE_PLAIN: return launch_dtype<MODE_PLAIN>(dtype, g, mtm, mtn, s, nullptr, expect);
            case MODE_SIGNAL: return launch_dtype<MODE_SIGNAL>(dtype, g, mtm, mtn, s, nullptr, expect);
            default: return launch_dtype<MODE_SCATTER>(dtype, g, mtm, mtn, s, nullptr, expect);
        }
    };
    // the tail split was computed for r.resident workgroups of the main launch
    rc = launch(a, r.mtm, r.mtn, r.tail_tiles ? r.resident : 0);
    if (rc || !r.tail_tiles) return rc;
    // the last, partial wave of 256x256 tiles: the same raster positions in the Algo's own tile
    GemmArgs t = a;
    t.first = a.count;
    t.sub_m = r.tail_sub_m; t.sub_n = r.tail_sub_n;
    t.count = r.tail_tiles * r.tail_sub_m * r.tail_sub_n;
    return launch(t, a.BM, a.BN, 0);
}

}  // namespace

// Workgroups of the 256x256 shape that stay resident on the current device: what the
// raster's tail split is computed from.  All epilogues and both dtypes of that shape use
// the same LDS (one workgroup per CU); the launch checks its own instantiation against
// this number.  Without a usable device (host-only callers asking for the schedule order)
// the answer is MI355X's: 256 CUs, one workgroup each.
int fo_main_tile_resident() {
    const int limit = gemm_cu_limit().load(std::memory_order_relaxed);
    const int no_device = limit > 0 && limit < 256 ? limit / 8 * 8 : 256;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return no_device;
    }
    // Asked on every launch: answered from here after the first.  An entry holds the CU limit it was
    // computed under (plus one, in the upper half) and the answer.
    static std::atomic<int> cached[kMaxDevices];
    if (dev >= 0 && dev < kMaxDevices) {
        const int c = cached[dev].load(std::memory_order_relaxed);
        if ((c >> 16) == limit + 1) return c & 0xFFFF;
    }
    GemmArgs a = {};
    a.count = 1 << 30;
    int info[5] = {0, 0, 0, 0, 0};
    if (launch_dtype<MODE_SIGNAL>(FO_F16, a, 256, 256, nullptr, info) != FO_OK || info[4] <= 0 || info[4] > 0xFFFF) {
        (void)hipGetLastError();
        return no_device;
    }
    if (dev >= 0 && dev < kMaxDevices) cached[dev].store((limit + 1) << 16 | info[4], std::memory_order_relaxed);
    return info[4];
}

// The GEMM launches count on n CUs from here on (n <= 0: on all).  Process-wide, read at every launch;
// the caller changes it only while no schedule order taken under the old value is still in use.
extern "C" int fo_gemm_set_cu_limit(int n) {
    if (n > 0 && n < 8) return FO_ERR_ARG;  // the raster wants a workgroup count that is a multiple of the 8 XCDs
    if (n > 0x7FFE) return FO_ERR_ARG;
    gemm_cu_limit().store(n > 0 ? n : 0, std::memory_order_relaxed);
    return FO_OK;
}

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
    int info[5] = {0, 0, 0, 0, 0};
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
    int out[5] = {0, 0, 0, 0, 0};
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
