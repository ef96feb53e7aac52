// MFMA GEMM for gfx950 with three epilogues: plain row-major store, reordered
// tile store + per-group signal, and reordered store through a row map + signal.
//
//   C[M,N] = A[M,K] . B[N,K]^T   (both operands K-contiguous), fp32 accumulate.
//
// Replaces the CUTLASS kernels behind gemm_func_table / signal_func_table /
// scatter_func_table of the reference (src/gemm/gemm.cu:23-110,
// src/overlap/gemm_signal.cu:15-97, src/overlap/gemm_scatter.cu:15-98; epilogue
// semantics src/overlap/gemm_with_signal.h:236-256, :291-361).
//
// Workgroup = WM x WN wavefronts (64 lanes each) computing an MTM x MTN macro
// tile with v_mfma_f32_32x32x16_{f16,bf16}.  Operand tiles (BK = 64) are staged
// global -> registers -> LDS with a 16-byte XOR swizzle and double buffered, so
// one barrier per K step suffices.  The accumulators leave through LDS so that
// every global store is a 16-byte piece of a contiguous output row.
#include "fo_common.h"

namespace {

constexpr int BK = 64;        // K elements per LDS stage
constexpr int CH = BK / 8;    // 16-byte chunks per tile row

enum { MODE_PLAIN = 0, MODE_SIGNAL = 1, MODE_SCATTER = 2 };

struct GemmArgs {
    const uint16_t *A;
    const uint16_t *B;
    uint16_t *C;
    int M, N, K;
    int BM, BN, TN, rLDN;  // reorder/signal tile, tiles along N, reshaped width in tiles
    const int32_t *RA;
    const int32_t *RE;
    const int32_t *cseg;
    int G;
    int32_t *MM;
    int monitor;
    int grid_m, grid_n, panel, xcd_remap;
};

// Group of storage slot r: smallest g with cseg[0]+..+cseg[g] > r
// (src/overlap/gemm_with_signal.h:343-349), found by one wavefront with a
// 64-wide prefix sum per step instead of a serial scan.  All 64 lanes call it.
__device__ __forceinline__ int find_group(const int32_t *cseg, int G, int r, int lane) {
    int base = 0;
    for (int it = 0; it < G; it += 64) {
        int idx = it + lane;
        int s = idx < G ? cseg[idx] : 0;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            int o = __shfl_up(s, d, 64);
            if (lane >= d) s += o;
        }
        s += base;
        unsigned long long hit = __ballot(idx < G && s > r);
        if (hit) return it + (int)__builtin_ctzll(hit);
        base = __shfl(s, 63, 64);
    }
    return G - 1;  // unreachable when sum(cseg) covers every slot (validated on the host)
}

template <typename Tag, int MTM, int MTN, int WM, int WN, int MODE>
__global__ __launch_bounds__(WM *WN * 64) void fo_gemm_kernel(GemmArgs p) {
    typedef fo_elem<Tag> E;
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = MTM / WM, WTN = MTN / WN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int RP = NT / CH;  // tile rows covered by one pass of the whole workgroup
    constexpr int PA = MTM / RP, PB = MTN / RP;
    static_assert(MTM % RP == 0 && MTN % RP == 0, "tile rows must split evenly over the loaders");
    static_assert(RP % 8 == 0, "swizzle key must be constant per loader thread");

    extern __shared__ fo_u32x4 smem[];
    fo_u32x4 *As = smem;                  // [2][MTM*CH]
    fo_u32x4 *Bs = smem + 2 * MTM * CH;   // [2][MTN*CH]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;

    int pm, pn;
    fo_wg_to_tile(blockIdx.x, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);

    const int ldk = p.K >> 3;  // row stride of A and B in 16-byte chunks
    const fo_u32x4 *Ag = reinterpret_cast<const fo_u32x4 *>(p.A) + (size_t)pm * MTM * ldk;
    const fo_u32x4 *Bg = reinterpret_cast<const fo_u32x4 *>(p.B) + (size_t)pn * MTN * ldk;

    const int lc = tid % CH, lr = tid / CH;
    const int lsw = lc ^ (lr & 7);  // swizzled chunk slot of this loader thread

    // Register staging of the next K step (kept as plain unrolled loops: the
    // arrays must stay in VGPRs).
    fo_u32x4 ra[PA], rb[PB];
#define FO_GLOAD(kt_)                                                                    \
    _Pragma("unroll") for (int i = 0; i < PA; i++)                                       \
        ra[i] = Ag[(size_t)(lr + i * RP) * ldk + (kt_) * CH + lc];                       \
    _Pragma("unroll") for (int i = 0; i < PB; i++)                                       \
        rb[i] = Bg[(size_t)(lr + i * RP) * ldk + (kt_) * CH + lc];
#define FO_LSTORE(s_)                                                                    \
    _Pragma("unroll") for (int i = 0; i < PA; i++)                                       \
        As[(s_) * (MTM * CH) + (lr + i * RP) * CH + lsw] = ra[i];                        \
    _Pragma("unroll") for (int i = 0; i < PB; i++)                                       \
        Bs[(s_) * (MTN * CH) + (lr + i * RP) * CH + lsw] = rb[i];

    fo_float16v acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const int KT = p.K / BK;
    FO_GLOAD(0)
    FO_LSTORE(0)
    __syncthreads();

    // Fragment addressing: lane l supplies row (l & 31), k-chunk (l >> 5) of
    // each 32x16 operand block; the swizzle key is the row's low 3 bits.
    const int frow = lane & 31, fk = lane >> 5;
    const int fkey = frow & 7;

    for (int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        if (kt + 1 < KT) {
            FO_GLOAD(kt + 1)
        }
        const fo_u32x4 *a = As + cur * (MTM * CH) + (wm * WTM + frow) * CH;
        const fo_u32x4 *b = Bs + cur * (MTN * CH) + (wn * WTN + frow) * CH;
#pragma unroll
        for (int kk = 0; kk < BK / 16; kk++) {
            const int slot = (kk * 2 + fk) ^ fkey;
            fo_u32x4 af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; i++) af[i] = a[i * 32 * CH + slot];
#pragma unroll
            for (int j = 0; j < FN; j++) bf[j] = b[j * 32 * CH + slot];
            // The N-side block is the MFMA's first operand, so a lane's four
            // consecutive accumulator values are consecutive output columns.
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++) acc[i][j] = E::mfma(bf[j], af[i], acc[i][j]);
        }
        if (kt + 1 < KT) {
            FO_LSTORE(cur ^ 1)
        }
        __syncthreads();
    }

#undef FO_GLOAD
#undef FO_LSTORE

    // ---- epilogue: accumulators -> 16-bit -> LDS (per-wave strip of 32 rows) -> global
    constexpr int PITCH = WTN + 8;  // halfs; keeps 16-byte alignment, skews banks
    uint16_t *stage = reinterpret_cast<uint16_t *>(smem) + wave * (32 * PITCH);
    constexpr int CPR = WTN / 8;      // 16-byte chunks per strip row
    constexpr int RPP = 64 / CPR;     // strip rows per store pass
    const int srow = lane / CPR, scol = lane % CPR;
    const int ldp = p.rLDN * p.BN;    // leading dimension of the reshaped output

#pragma unroll
    for (int i = 0; i < FM; i++) {
#pragma unroll
        for (int j = 0; j < FN; j++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                uint16_t h0 = E::from_f32(acc[i][j][q * 4 + 0]);
                uint16_t h1 = E::from_f32(acc[i][j][q * 4 + 1]);
                uint16_t h2 = E::from_f32(acc[i][j][q * 4 + 2]);
                uint16_t h3 = E::from_f32(acc[i][j][q * 4 + 3]);
                fo_u32x2 v;
                v.x = (uint32_t)h0 | ((uint32_t)h1 << 16);
                v.y = (uint32_t)h2 | ((uint32_t)h3 << 16);
                *reinterpret_cast<fo_u32x2 *>(stage + frow * PITCH + j * 32 + q * 8 + fk * 4) = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int ps = 0; ps < 32 / RPP; ps++) {
            const int row = ps * RPP + srow;
            fo_u32x4 v = *reinterpret_cast<const fo_u32x4 *>(stage + row * PITCH + scol * 8);
            const int m = pm * MTM + wm * WTM + i * 32 + row;
            const int n = pn * MTN + wn * WTN + scol * 8;
            size_t off;
            if (MODE == MODE_PLAIN) {
                off = (size_t)m * p.N + n;
            } else {
                const int t = (m / p.BM) * p.TN + n / p.BN;
                const int r = p.RA[t];
                long prow = (long)(r / p.rLDN) * p.BM + m % p.BM;
                if (MODE == MODE_SCATTER) prow = p.RE[prow];
                off = (size_t)prow * ldp + (size_t)(r % p.rLDN) * p.BN + n % p.BN;
            }
            *reinterpret_cast<fo_u32x4 *>(p.C + off) = v;
        }
        __syncthreads();
    }

    if (MODE != MODE_PLAIN) {
        // Every lane waits until its own stores are acknowledged, the barrier
        // collects the workgroup, and only then one lane releases at agent
        // scope (L2 write-back) and bumps the group counter.  The reference
        // has no fence here (src/overlap/gemm_with_signal.h:337-351).
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (wave == 0) {
            const int sub_m = MTM / p.BM, sub_n = MTN / p.BN;
            for (int s = 0; s < sub_m * sub_n; s++) {
                const int tm = pm * sub_m + s / sub_n;
                const int tn = pn * sub_n + s % sub_n;
                const int r = p.RA[tm * p.TN + tn];
                const int g = find_group(p.cseg, p.G, r, lane);
                if (lane == 0) {
                    __hip_atomic_fetch_add(p.MM + g, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
                    if (p.monitor) {
                        int o = __hip_atomic_fetch_add(p.MM + (p.TN - 1), 1, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(p.MM + p.TN + r, o, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
        }
    }
}

template <typename Tag, int MTM, int MTN, int WM, int WN, int MODE>
int launch_variant(const GemmArgs &a, hipStream_t stream) {
    auto kern = fo_gemm_kernel<Tag, MTM, MTN, WM, WN, MODE>;
    constexpr int smem = 2 * (MTM + MTN) * BK * 2;
    static bool configured = false;  // per instantiation; the attribute is process wide
    if (!configured) {
        FO_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, smem));
        configured = true;
    }
    dim3 grid(a.grid_m * a.grid_n), block(WM * WN * 64);
    hipLaunchKernelGGL(kern, grid, block, smem, stream, a);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

template <typename Tag, int MODE>
int launch_tile(const GemmArgs &a, int mtm, int mtn, hipStream_t stream) {
    if (mtm == 128 && mtn == 128) return launch_variant<Tag, 128, 128, 2, 2, MODE>(a, stream);
    if (mtm == 128 && mtn == 256) return launch_variant<Tag, 128, 256, 2, 2, MODE>(a, stream);
    if (mtm == 256 && mtn == 128) return launch_variant<Tag, 256, 128, 2, 2, MODE>(a, stream);
    return FO_ERR_ALGO;
}

template <int MODE>
int launch_dtype(int dtype, const GemmArgs &a, int mtm, int mtn, hipStream_t stream) {
    if (dtype == FO_F16) return launch_tile<fo_f16_tag, MODE>(a, mtm, mtn, stream);
    if (dtype == FO_BF16) return launch_tile<fo_bf16_tag, MODE>(a, mtm, mtn, stream);
    return FO_ERR_DTYPE;
}

int run_gemm(int mode, int dtype, int M, int N, int K, int rLDN, const int32_t *cseg, int G,
             const void *A, const void *B, void *C, int32_t *MM, const int32_t *RA,
             const int32_t *RE, int monitor, int algo, fo_stream_t stream) {
    if (dtype != FO_F16 && dtype != FO_BF16) return FO_ERR_DTYPE;
    const fo_algo_entry *e = fo_algo_lookup(algo);
    if (!e) return FO_ERR_ALGO;
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return FO_ERR_ARG;
    fo_raster r;
    int rc = fo_pick_raster(algo, M, N, &r);
    if (rc) return rc;
    if (K % BK) return FO_ERR_SHAPE;
    GemmArgs a;
    a.A = static_cast<const uint16_t *>(A);
    a.B = static_cast<const uint16_t *>(B);
    a.C = static_cast<uint16_t *>(C);
    a.M = M; a.N = N; a.K = K;
    a.BM = e->f[0]; a.BN = e->f[1];
    a.TN = N / a.BN;
    a.rLDN = rLDN;
    a.RA = RA; a.RE = RE; a.cseg = cseg; a.G = G; a.MM = MM; a.monitor = monitor;
    a.grid_m = r.grid_m; a.grid_n = r.grid_n; a.panel = r.panel; a.xcd_remap = r.xcd_remap;
    if (mode != MODE_PLAIN) {
        const long T = (long)(M / a.BM) * a.TN;
        if (!MM || !RA || !cseg) return FO_ERR_ARG;
        if (mode == MODE_SCATTER && !RE) return FO_ERR_ARG;
        if (rLDN <= 0 || T % rLDN) return FO_ERR_SHAPE;
        if (G <= 0 || G > T) return FO_ERR_SEGMENTS;
        if (monitor && G > a.TN - 1) return FO_ERR_SEGMENTS;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (mode) {
        case MODE_PLAIN: return launch_dtype<MODE_PLAIN>(dtype, a, r.mtm, r.mtn, s);
        case MODE_SIGNAL: return launch_dtype<MODE_SIGNAL>(dtype, a, r.mtm, r.mtn, s);
        default: return launch_dtype<MODE_SCATTER>(dtype, a, r.mtm, r.mtn, s);
    }
}

}  // namespace

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
