// Shared declarations of the gfx950 kernel library (internal; the public C ABI
// is include/flashoverlap.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "flashoverlap.h"

#define FO_HIP_CHECK(expr)                        \
    do {                                          \
        hipError_t e__ = (expr);                  \
        if (e__ != hipSuccess) return (int)e__;   \
    } while (0)

// The launch itself reports configuration errors through hipGetLastError.
#define FO_LAUNCH_CHECK()                         \
    do {                                          \
        hipError_t e__ = hipGetLastError();       \
        if (e__ != hipSuccess) return (int)e__;   \
    } while (0)

typedef _Float16 fo_half8 __attribute__((ext_vector_type(8)));
typedef __bf16 fo_bf8 __attribute__((ext_vector_type(8)));
typedef float fo_float4v __attribute__((ext_vector_type(4)));
// Native 16- and 8-byte vectors (HIP's uint4 is a struct that register promotion handles badly).
typedef unsigned int fo_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int fo_u32x2 __attribute__((ext_vector_type(2)));

struct fo_f16_tag {};
struct fo_bf16_tag {};

// 16-bit <-> fp32 element conversions (round to nearest even, hardware cvt).
template <typename Tag> struct fo_elem;
template <> struct fo_elem<fo_f16_tag> {
    typedef _Float16 type;
    typedef fo_half8 vec8;
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return (float)__builtin_bit_cast(_Float16, b);
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        return __builtin_bit_cast(uint16_t, (_Float16)f);
    }
    // D(16x16) += A(16x32) . B(32x16); lane l supplies row l & 15, k-chunk l >> 4 of both
    // operands and holds D[4 * (l >> 4) + v][l & 15], v = 0..3.
    // Written as assembly with the accumulator tied to the destination: the
    // builtin's destination is a free operand for this shape, and with 32
    // accumulator blocks in a doubly unrolled loop the register allocator then
    // rotates them through spare registers and spills.  What the compiler
    // therefore does not see is that the result is late: callers keep VALU reads
    // and writes of the accumulators (zeroing, conversion) 24 wait states away
    // from these instructions (fo_mfma_fence).
    static __device__ __forceinline__ void mfma(fo_u32x4 a, fo_u32x4 b, fo_float4v &c) {
        asm("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
};
template <> struct fo_elem<fo_bf16_tag> {
    typedef __bf16 type;
    typedef fo_bf8 vec8;
    static __device__ __forceinline__ float to_f32(uint16_t b) {
        return __builtin_bit_cast(float, (uint32_t)b << 16);
    }
    static __device__ __forceinline__ uint16_t from_f32(float f) {
        return __builtin_bit_cast(uint16_t, (__bf16)f);
    }
    static __device__ __forceinline__ void mfma(fo_u32x4 a, fo_u32x4 b, fo_float4v &c) {
        asm("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
};

// Wait states between the assembly MFMAs and ordinary VALU code touching their
// accumulators (longest case: an 8-pass MFMA result read by a VALU instruction).
static __device__ __forceinline__ void fo_mfma_fence() {
    __builtin_amdgcn_sched_barrier(0);  // nothing is scheduled across the wait states
    asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Algo table (fo_algo.cpp).
struct fo_algo_entry {
    int32_t f[12];  // TbM,TbN,TbK,WarpM,WarpN,WarpK,InstM,InstN,InstK,Stages,Swizzle,SplitK
};
const fo_algo_entry *fo_algo_lookup(int algo);

// Macro-tile choice and raster shared by the launcher and fo_schedule_order.
struct fo_raster {
    int mtm, mtn;        // macro tile (workgroup tile) in elements
    int grid_m, grid_n;  // macro tiles along M and N
    int panel;           // raster panel height in macro tiles (xcd_remap 2: the packed shape of fo_pack_row_waves)
    int xcd_remap;       // 1: workgroup id is de-interleaved over the 8 XCDs; 2: waves of whole tile rows (below)
    // A last wave of 256x256 tiles that would leave most CUs idle is computed by a
    // second launch instead, with the Algo's own (smaller) tile: the last
    // tail_tiles positions of the raster, each cut into tail_sub_m x tail_sub_n.
    int tail_tiles, tail_sub_m, tail_sub_n;
    int resident;  // workgroups of the 256x256 launch the tail split was computed for (0: not a 256x256 raster)
};
int fo_pick_raster(int algo, int M, int N, fo_raster *r);
// Whether fo_pick_raster lays 256x256 launches out in waves of whole tile rows where that fits (default: yes).
void fo_set_row_waves(bool on);
// Resident workgroups of the 256x256 kernel shape on the current device (fo_gemm.hip).
int fo_main_tile_resident();

// fo_gemm_signal / fo_gemm_scatter (RE != nullptr) without the counters: tiles are
// stored reordered, MM is never touched (fo_gemm.hip; used by fo_overlap.cpp).
int fo_gemm_reordered_quiet(int dtype, int M, int N, int K, int rLDN, const int32_t *cseg_dev, int G,
                            const void *A, const void *B, void *C, const int32_t *RA, const int32_t *RE,
                            int algo, fo_stream_t stream);

// Data that is touched once per step is moved with non-temporal accesses when the
// step's working set cannot stay in the 256 MB memory-side cache anyway; below
// that it is left cacheable, because the next kernel reads it again.
constexpr int64_t kStreamAboveBytes = 192LL << 20;
inline bool fo_streams(int64_t bytes) { return bytes > kStreamAboveBytes; }
// A GEMM output above this size is stored with the non-temporal hint (see store16_nt in fo_gemm_kernel.h).
constexpr int64_t kStreamOutAboveBytes = 96LL << 20;

// The consumer entry points with the accumulator's cache policy chosen by the
// caller (fo_aux.hip; the extern "C" forms decide from their own range).
// beside_gemm: the launch runs while a GEMM with waves still to come holds every
// CU.  It then asks for kBesideGemmLds bytes of LDS it never touches, which, beside
// the GEMM workgroup's 145-148 KB, admits one consumer workgroup per CU instead of
// up to eight: the consumer's loads share each CU's load path with the GEMM's
// operand stream (8192^3: overlapped step 0.842 instead of 0.847 ms).
constexpr int kBesideGemmLds = 12288;
// A streaming all-reduce consumer beside the GEMM also runs with one wavefront per workgroup instead of
// four, i.e. on one of the CU's four SIMDs: same grid, a quarter of the lanes, each moving four times as
// much.  Alone it would be slower; beside the GEMM it takes less from it (8192^3: overlapped step 0.846
// against 0.855 ms, 8192x8192x3584: 0.410 against 0.424, alternating runs on one box).  The
// reduce-scatter layout and cacheable accumulators lose that way and keep four wavefronts.
constexpr int kBesideGemmThreads = 64;
int fo_consumer_reduce_with(int dtype, const void *src, void *acc, int64_t nelem, int W, int64_t seg_stride,
                            void *own, int rank, bool stream_acc, fo_stream_t stream, bool beside_gemm = false);
int fo_consumer_reduce_groups_with(int dtype, const void *src, void *acc, const int32_t *cseg_dev, int ngroups,
                                   int64_t max_group_tiles, int64_t tile_elems, int W, int64_t seg_stride,
                                   void *own, int rank, bool stream_acc, fo_stream_t stream,
                                   bool beside_gemm = false);
int fo_wait_reduce_groups_with(int dtype, const void *C, void *ACC, int32_t *MM, const int32_t *cseg_dev, int G,
                               int64_t tile_elems, int W, int64_t seg_stride, void *own, int rank,
                               int32_t *workspace, int nblocks, int slices, int poll_gap_ns, bool stream_acc,
                               long max_polls, fo_stream_t stream);

// Rows [row0, row0 + nrows) of (reorder+)RMSNorm over X[bs, dim] (RA null: no reorder) with the row
// kernel that fits beside a GEMM (fo_aux.hip).  stream_rows: non-temporal accesses; beside_gemm: at most
// one workgroup per CU; grid: workgroups (0: chosen from the row count).  info != null: nothing is launched,
// info = {registers per lane, LDS bytes per workgroup} of the kernel that would run.
int fo_norm_rows_with(int dtype, const void *X, void *Y, const void *Wt, int row0, int nrows, int bs, int dim, int BM,
                      int BN, int rldn, const int32_t *RA, float eps, bool stream_rows, bool beside_gemm, int grid,
                      fo_stream_t stream, int32_t *info = nullptr);

// The waits with their bound and status word chosen by the caller (fo_aux.hip).
// max_polls < 0: the bound of the environment variable FO_WAIT_MAX_POLLS (none
// when unset); 0: unbounded.  A wait that gives up stores 1 into *status (may be
// null) and leaves its counter as it is.
int fo_wait_with(int expect, int32_t *counter, long max_polls, int32_t *status, fo_stream_t stream);
int fo_wait_groups_with(int count, const int32_t *expect_dev, int32_t *counters, long max_polls, int32_t *status,
                        fo_stream_t stream);
// words[0..n) = value by a small kernel (no memset node under stream capture); word `skip` keeps its value.
int fo_fill_words(int32_t *words, int n, int value, fo_stream_t stream, int skip = -1);
constexpr double kMaxPaceSeconds = 1.0;                // longest stretch fo_pace_with accepts
int fo_pace_with(double seconds, fo_stream_t stream);  // a one-lane kernel that holds the stream that long

// Raster of whole-row waves (xcd_remap == 2).  The persistent launch holds R workgroups, R / 8 on each
// XCD; wave k of the walk (raster positions kR .. kR + R - 1) covers the R / grid_n complete tile rows
// that follow those of wave k - 1, cut into 8 blocks of 2^log_bh x 2^log_bw tiles, one per XCD, 2^log_xc
// blocks side by side: whatever consumes whole output rows (a row-wise normalisation) can follow the GEMM
// wave by wave.  An XCD's concurrent tiles still form one block and share its operand panels in that
// XCD's L2.  Everything but the wave index is shifts and masks.
__host__ __device__ inline int fo_pack_row_waves(int log_bh, int log_bw, int log_xc, int resident) {
    return log_bh | log_bw << 4 | log_xc << 8 | resident << 12;
}
__host__ __device__ inline void fo_row_wave_tile(int t, int packed, int *pm, int *pn) {
    const int log_bh = packed & 15, log_bw = (packed >> 4) & 15, log_xc = (packed >> 8) & 15, R = packed >> 12;
    const int k = t / R, w = t - k * R;
    const int x = w & 7, j = w >> 3;
    const int rows_per_wave = (8 >> log_xc) << log_bh;
    *pm = k * rows_per_wave + ((x >> log_xc) << log_bh) + (j & ((1 << log_bh) - 1));
    *pn = ((x & ((1 << log_xc) - 1)) << log_bw) + (j >> log_bh);
}

// Workgroup id -> macro tile coordinates; identical code on host and device.
__host__ __device__ inline void fo_wg_to_tile(int wg, int grid_m, int grid_n, int panel,
                                              int xcd_remap, int *pm, int *pn) {
    if (xcd_remap == 2) {
        fo_row_wave_tile(wg, panel, pm, pn);
        return;
    }
    int nt = grid_m * grid_n;
    int v = wg;
    if (xcd_remap) {
        // Workgroups (and, in the persistent walk, tile slots) are dealt round-robin to the
        // 8 XCDs; give each XCD one contiguous range of the raster so that its private L2
        // sees neighbouring tiles.  XCD x owns the slots x, x+8, ...: nt/8 of them, one more
        // for the first nt%8 XCDs.
        const int q = nt >> 3, rem = nt & 7, x = wg & 7;
        v = x * q + (x < rem ? x : rem) + (wg >> 3);
    }
    int per_panel = panel * grid_n;
    int p = v / per_panel;
    int first_m = p * panel;
    int rows = grid_m - first_m < panel ? grid_m - first_m : panel;
    int in = v - p * per_panel;
    *pm = first_m + in % rows;
    *pn = in / rows;
}

// Unit u of a launch that covers raster positions first, first + 1, ... with each
// position cut into sub_m x sub_n tiles of its own -> coordinates in those tiles.
__host__ __device__ inline void fo_unit_to_tile(int u, int first, int sub_m, int sub_n, int grid_m,
                                                int grid_n, int panel, int xcd_remap, int *pm, int *pn) {
    const int per = sub_m * sub_n;
    if (per == 1) {
        fo_wg_to_tile(first + u, grid_m, grid_n, panel, xcd_remap, pm, pn);
        return;
    }
    int ppm, ppn;
    fo_wg_to_tile(first + u / per, grid_m, grid_n, panel, xcd_remap, &ppm, &ppn);
    const int s = u % per;
    *pm = ppm * sub_m + s / sub_n;
    *pn = ppn * sub_n + s % sub_n;
}
