// Device code of the gfx950 MFMA GEMM with three epilogues: plain row-major
// store, reordered tile store + per-group signal, reordered store through a row
// map + signal.
//
//   C[M,N] = A[M,K] . B[N,K]^T   (both operands K-contiguous), fp32 accumulate.
//
// Replaces the CUTLASS kernels behind gemm_func_table / signal_func_table /
// scatter_func_table of the reference (src/gemm/gemm.cu:23-110,
// src/overlap/gemm_signal.cu:15-97, src/overlap/gemm_scatter.cu:15-98; epilogue
// semantics src/overlap/gemm_with_signal.h:236-256, :291-361).
//
// The kernel is persistent: the launch holds at most as many workgroups as the
// chip keeps resident, and workgroup w computes macro tiles w, w + grid,
// w + 2 grid, ... of the raster.  A workgroup of WM x WN wavefronts computes an
// MTM x MTN macro tile with v_mfma_f32_32x32x16_{f16,bf16}.  Operand tiles of
// BK columns travel HBM -> LDS directly (global_load_lds_dwordx4, 1 KiB per
// wavefront instruction, no VGPR staging) into a ring of STAGES buffers; a slot
// is recycled as soon as every wavefront holds its last fragments of it in
// registers; one s_barrier per K step.  The 16-byte chunks of a tile row are
// XOR-swizzled (by choosing which global chunk each lane fetches) so that the
// 16 lanes a ds_read_b128 serves per clock hit 16 different bank groups.  The
// accumulators leave through LDS so that every global store is a 16-byte piece
// of a contiguous output row.
//
// Tile i+1's first operand stage is requested before tile i's epilogue and
// lands while the epilogue runs; tile i's completion signal is sent from inside
// tile i+1's first K step, at a point where every wavefront has already waited
// for its stores, so neither the store drain nor the signal stalls the MFMAs.
#pragma once

#include <type_traits>

#include "fo_common.h"

namespace fo_gemm_dev {

enum { MODE_PLAIN = 0, MODE_SIGNAL = 1, MODE_SCATTER = 2 };

struct GemmArgs {
    const uint16_t *A;
    const uint16_t *B;
    uint16_t *C;
    int M, N, K;
    int lda, ldb;          // row strides of A and B in elements (multiples of 8)
    int BM, BN, TN, rLDN;  // reorder/signal tile, tiles along N, reshaped width in tiles
    const int32_t *RA;
    const int32_t *RE;
    const int32_t *cseg;
    int G;
    int32_t *MM;
    int monitor;
    int grid_m, grid_n, panel, xcd_remap;
};

constexpr int kMaxSub = 4;        // reorder tiles per macro tile (256x256 over 128x128)
constexpr int kPrefixMax = 1024;  // group search on an LDS table for up to this many groups

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

// The same search on inclusive prefix sums kept in LDS (entry g holds
// cseg[0]+..+cseg[g]): no global memory access, so it can run while operand
// loads are in flight without waiting for them.
__device__ __forceinline__ int find_group_lds(const int *pre, int G, int r, int lane) {
    for (int it = 0; it < G; it += 64) {
        const int idx = it + lane;
        unsigned long long hit = __ballot(idx < G && pre[idx] > r);
        if (hit) return it + (int)__builtin_ctzll(hit);
    }
    return G - 1;
}

// s_waitcnt vmcnt(n) only (expcnt/lgkmcnt left at their maxima); gfx9 encoding:
// vmcnt = imm[15:14]:imm[3:0], expcnt = imm[6:4], lgkmcnt = imm[11:8].
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// 16-byte global stores written as assembly so that the number of vector memory
// instructions in flight is known exactly (the main loop waits on vmcnt with
// non-zero counts; the compiler does not see these instructions in its own
// count, which can only make its waits longer, never shorter).  The
// write-through form (system-scope cache policy) is used for the signalled
// epilogues: the tile must be visible to other XCDs before its counter is
// bumped, and a tile that never becomes dirty in L2 makes the releasing
// write-back that precedes the signal nearly free.  The trailing s_nop covers
// the wait states gfx9 requires between a VMEM store of more than 8 bytes and a
// VALU write of its data registers.
__device__ __forceinline__ void store16_write_through(void *ptr, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(ptr), "v"(v) : "memory");
}
// saddr forms: wave-uniform base (SGPR pair) + 32-bit per-lane byte offset
__device__ __forceinline__ void store16_write_through(char *base, unsigned lane_off, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, %2 sc0 sc1\n\ts_nop 1"
                 :
                 : "v"(lane_off), "v"(v), "s"((__attribute__((address_space(1))) char *)base)
                 : "memory");
}
__device__ __forceinline__ void store16(char *base, unsigned lane_off, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1"
                 :
                 : "v"(lane_off), "v"(v), "s"((__attribute__((address_space(1))) char *)base)
                 : "memory");
}

// One direct-to-LDS load of 16 bytes per lane in the saddr form: global address =
// wave-uniform base (SGPR pair) + 32-bit per-lane byte offset; LDS address =
// M0 + lane * 16.  Written as assembly because the compiler materialises a
// 64-bit VGPR address for the intrinsic (two VALU instructions per load, which
// steal issue slots from the MFMAs).  The s_nop covers the M0 write -> LDS-DMA
// wait state.
__device__ __forceinline__ void dma_load16(const __attribute__((address_space(1))) char *base, unsigned lane_off,
                                           unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(lane_off), "s"(base)
                 : "memory");
}

#define FO_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

template <typename Tag, int MTM, int MTN, int BK, int STAGES, int WM, int WN, int MODE>
__global__ __launch_bounds__(WM *WN * 64) void fo_gemm_kernel(GemmArgs p) {
    typedef fo_elem<Tag> E;
    constexpr int NW = WM * WN;
    constexpr int CH = BK / 8;                  // 16-byte chunks per tile row
    constexpr int SWZ_SHIFT = CH == 8 ? 1 : 2;  // rows sharing one swizzle key: 16 / CH
    constexpr int WTM = MTM / WM, WTN = MTN / WN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BLK = MTM * CH / 64, B_BLK = MTN * CH / 64;  // 1 KiB blocks per stage
    constexpr int PA = A_BLK / NW, PB = B_BLK / NW;              // blocks per wavefront
    constexpr int P = PA + PB;                                   // load instructions per wavefront and stage
    constexpr int STAGE16 = (MTM + MTN) * CH;                    // stage size in 16-byte units
    constexpr int KK = BK / 16;                                  // MFMA k-steps per stage
    constexpr int NM = FM * FN, NR = FM + FN;
    // epilogue: per-wavefront strip of 32 rows x WTN columns in the ring behind slot 0
    constexpr int PITCH = WTN + 8;   // halfs; keeps 16-byte alignment, skews banks
    constexpr int CPR = WTN / 8;     // 16-byte chunks per strip row
    constexpr int RPP = 64 / CPR;    // strip rows per store pass
    constexpr int NST = FM * (32 / RPP);  // store instructions per wavefront and tile
    static_assert(BK == 32 || BK == 64, "BK");
    static_assert(A_BLK % NW == 0 && B_BLK % NW == 0, "tile rows must split evenly over the wavefronts");
    static_assert((NW * (64 / CH)) % 32 == 0, "swizzle key must repeat across a wavefront's blocks");
    static_assert(STAGES >= 2, "ring depth");
    static_assert(NW * 32 * PITCH * 2 <= (STAGES - 1) * STAGE16 * 16, "the epilogue strips must fit behind ring slot 0");
    static_assert((STAGES - 1) * P + NST < 64, "vmcnt range");

    extern __shared__ fo_u32x4 smem[];
    const unsigned smem_lds = (unsigned)(uintptr_t)FO_LDS_PTR(smem);  // LDS byte address of the ring

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int ntiles = p.grid_m * p.grid_n;
    // K is a multiple of 8 (one 16-byte chunk).  A last K step that is not full
    // is loaded with its out-of-range chunks redirected to the step's first
    // chunk (valid memory) and zeroed in LDS before the stage is published.
    const int KT = (p.K + BK - 1) / BK;
    const bool ktail = (p.K % BK) != 0;
    const int KT_full = ktail ? KT - 1 : KT;  // K steps whose loads need no special care

    // Fragment addressing: lane l supplies row (l & 31), k-chunk (l >> 5) of
    // each 32x16 operand block.
    const int frow = lane & 31, fk = lane >> 5;
    const int fkey = (frow >> SWZ_SHIFT) & (CH - 1);
    const int a_off = (wm * WTM + frow) * CH;
    const int b_off = MTM * CH + (wn * WTN + frow) * CH;

    // Loader role of this lane inside a 1 KiB block: LDS slot `lane` is
    // (row lane / CH, physical chunk lane % CH); it must receive logical chunk
    // phys ^ key(row).  Block q of a tile covers rows [q*64/CH, (q+1)*64/CH).
    // A wavefront's blocks are NW*64/CH (a multiple of 32) rows apart, so the key
    // of its first block holds for all of them.
    const int lrow = lane / CH;
    const int lchunk = (lane % CH) ^ (((wave * (64 / CH) + lrow) >> SWZ_SHIFT) & (CH - 1));
    // Global addresses = wave-uniform base (SGPRs, advanced with scalar adds) + one
    // loop-invariant 32-bit per-lane byte offset, so the loads use the saddr form
    // and the K loop carries no vector address arithmetic.
    typedef const __attribute__((address_space(1))) char *gptr_t;
    const unsigned a_lane = (unsigned)(lrow * p.lda * 2 + lchunk * 16);
    const unsigned b_lane = (unsigned)(lrow * p.ldb * 2 + lchunk * 16);
    const size_t a_blk_bytes = (size_t)NW * (64 / CH) * p.lda * 2;  // between a wave's consecutive blocks
    const size_t b_blk_bytes = (size_t)NW * (64 / CH) * p.ldb * 2;
    gptr_t Ab, Bb;  // operand rows of the tile whose loads are issued next
    auto set_tile = [&](int pm_, int pn_) {
        Ab = (gptr_t)(p.A) + ((size_t)pm_ * MTM + wave * (64 / CH)) * p.lda * 2;
        Bb = (gptr_t)(p.B) + ((size_t)pn_ * MTN + wave * (64 / CH)) * p.ldb * 2;
    };
    // Issue the loads of K step kt into ring slot s (P instructions per wavefront).
    auto issue_with = [&](int kt, int s, unsigned al, unsigned bl) {
        const unsigned as = smem_lds + (unsigned)(s * STAGE16 + wave * 64) * 16;  // LDS byte addresses
        const unsigned bs = as + MTM * CH * 16;
        gptr_t ak = Ab + (size_t)kt * (BK * 2), bk = Bb + (size_t)kt * (BK * 2);
#pragma unroll
        for (int i = 0; i < PA; i++) dma_load16(ak + i * a_blk_bytes, al, as + i * NW * 1024);
#pragma unroll
        for (int i = 0; i < PB; i++) dma_load16(bk + i * b_blk_bytes, bl, bs + i * NW * 1024);
    };
    auto issue = [&](int kt, int s) { issue_with(kt, s, a_lane, b_lane); };
    // The partial last K step.  Whether this lane's chunk lies beyond K is
    // recomputed from a laundered lane id, so nothing of it stays live across
    // the K loop.
    auto tail_chunk_out = [&](int *row) {
        int el = lane;
        asm volatile("" : "+v"(el));
        *row = el / CH;
        const int lc = (el % CH) ^ (((wave * (64 / CH) + el / CH) >> SWZ_SHIFT) & (CH - 1));
        return (KT - 1) * BK + lc * 8 >= p.K;
    };
    // Same loads as issue(); a chunk beyond K is fetched from the row's first chunk of this step instead.
    auto issue_any = [&](int kt, int s) {
        if (ktail && kt == KT - 1) {
            int row;
            const bool out = tail_chunk_out(&row);
            issue_with(kt, s, out ? (unsigned)(row * p.lda * 2) : a_lane, out ? (unsigned)(row * p.ldb * 2) : b_lane);
        } else {
            issue(kt, s);
        }
    };
    // Zero this lane's chunks of the partial step in ring slot s.  Called after
    // the lane's own loads of that stage have landed and before the barrier that
    // publishes the stage.
    auto zero_tail = [&](int s) {
        int row;
        if (tail_chunk_out(&row)) {
            int el = lane;
            asm volatile("" : "+v"(el));
            fo_u32x4 *mine = smem + s * STAGE16 + wave * 64 + el;
            const fo_u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < PA; i++) mine[i * NW * 64] = z;
#pragma unroll
            for (int i = 0; i < PB; i++) mine[MTM * CH + i * NW * 64] = z;
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    };

    // ---- signalling state (signal and scatter epilogues)
    const int sub_n = MTN / p.BN, nsub = (MTM / p.BM) * sub_n;  // reorder tiles per macro tile
    typedef const __attribute__((address_space(4))) int32_t *cptr_t;  // read-only for the whole launch: scalar loads
    const cptr_t RAc = (cptr_t)(uintptr_t)p.RA;
    int *pre = reinterpret_cast<int *>(smem + STAGES * STAGE16);  // behind the ring: prefix sums of cseg
    const bool lds_search = p.G <= kPrefixMax;
    if (MODE != MODE_PLAIN && wave == 0 && lds_search) {
        int base = 0;
        for (int it = 0; it < p.G; it += 64) {
            const int idx = it + lane;
            int s = idx < p.G ? p.cseg[idx] : 0;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                int o = __shfl_up(s, d, 64);
                if (lane >= d) s += o;
            }
            s += base;
            if (idx < p.G) pre[idx] = s;  // read back by wavefront 0 only, after later barriers
            base = __shfl(s, 63, 64);
        }
    }
    // Wavefront 0 announces the reorder tiles whose storage slots are rs[0..nsub).
    // Callers guarantee that every wavefront's stores of those tiles are complete:
    // the stores are write-through, each wavefront has waited for their
    // acknowledgement (vmcnt) and a workgroup barrier lies between that wait and
    // this call.  The tile is therefore in memory before the counter moves, and
    // the atomic itself is relaxed: a release here would add an L2 write-back
    // (with nothing of this tile left to write back) and a wait for the operand
    // loads in flight, both paid by the whole workgroup at its next barrier.
    auto announce = [&](const int (&rs)[kMaxSub]) {
#pragma unroll
        for (int s = 0; s < kMaxSub; s++) {
            if (s < nsub) {
                const int r = rs[s];
                const int g = lds_search ? find_group_lds(pre, p.G, r, lane) : find_group(p.cseg, p.G, r, lane);
                if (lane == 0) {
                    __hip_atomic_fetch_add(p.MM + g, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (p.monitor) {
                        int o = __hip_atomic_fetch_add(p.MM + (p.TN - 1), 1, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(p.MM + p.TN + r, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
        }
    };

    // Operand fragments are double buffered in registers: while the MFMAs of
    // k-step kk run, the ds_reads of k-step kk+1 (or of the next stage's first
    // k-step) are in flight.
    fo_float16v acc[FM][FN];
    fo_u32x4 af[2][FM], bf[2][FN];
#define FO_LOAD_FRAGS(buf_, st_, kk_)                                                                 \
    {                                                                                                 \
        const int c_ = ((kk_) * 2 + fk) ^ fkey;                                                       \
        _Pragma("unroll") for (int i = 0; i < FM; i++) af[buf_][i] = (st_)[a_off + i * 32 * CH + c_]; \
        _Pragma("unroll") for (int j = 0; j < FN; j++) bf[buf_][j] = (st_)[b_off + j * 32 * CH + c_]; \
    }
    // The N-side block is the MFMA's first operand, so a lane's four consecutive
    // accumulator values are consecutive output columns.
#define FO_MFMAS(kk_)                                  \
    _Pragma("unroll") for (int i = 0; i < FM; i++)     \
        _Pragma("unroll") for (int j = 0; j < FN; j++) \
            acc[i][j] = E::mfma(bf[(kk_) & 1][j], af[(kk_) & 1][i], acc[i][j]);

    int prev_rs[kMaxSub] = {0, 0, 0, 0};  // slots of the tile whose signal is still owed
    bool owed = false;

    // One K step.  STEADY: at least STAGES further steps exist, so the waits and
    // the refill are unconditional and the body is a single scheduling region
    // per k-step, pinned MFMA-first with the memory instructions in its shadow.
    // With two slots the steady loop is unrolled by two and the slot is a
    // compile-time constant (slot_tag >= 0), which makes every LDS address
    // loop-invariant.  `first` marks a tile's first K step: after its barrier
    // every wavefront has waited for the previous tile's stores (they are older
    // than the loads that wait covers), which is where an owed signal is sent.
    auto kstep = [&](auto steady, auto slot_tag, bool first, int kt, int slot_rt, int nslot_rt) {
        constexpr bool STEADY = decltype(steady)::value;
        constexpr int SLOT_C = decltype(slot_tag)::value;
        const int slot = SLOT_C >= 0 ? SLOT_C : slot_rt;
        const int nslot = SLOT_C >= 0 ? (SLOT_C ^ 1) : nslot_rt;
        const fo_u32x4 *st = smem + slot * STAGE16;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            if (kk + 1 < KK) {
                FO_LOAD_FRAGS((kk + 1) & 1, st, kk + 1)
            } else if (STEADY || kt + 1 < KT) {
                // This wavefront holds all of stage kt in registers.  Make stage
                // kt+1 visible (own loads landed + barrier), then recycle slot kt
                // for stage kt+STAGES and fetch the next stage's first fragments.
                if (STEADY || kt + STAGES - 1 < KT)
                    wait_vmcnt<(STAGES - 2) * P>();
                else
                    wait_vmcnt<0>();
                if (!STEADY) {
                    if (ktail && kt + 2 == KT) zero_tail(nslot);  // all loads of stage KT-1 have landed (vmcnt 0)
                }
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if (!STEADY && MODE != MODE_PLAIN) {
                    if (first && owed && wave == 0) announce(prev_rs);
                }
                if constexpr (STEADY) {
                    issue(kt + STAGES, slot);
                } else {
                    if (kt + STAGES < KT) issue_any(kt + STAGES, slot);
                }
                FO_LOAD_FRAGS((kk + 1) & 1, smem + nslot * STAGE16, 0)
            }
            FO_MFMAS(kk)
            if (STEADY) {
                // issue order inside this k-step: MFMA, ds_read, MFMA, ds_read, ...
                // then (last k-step) the direct-to-LDS loads between the remaining MFMAs
#pragma unroll
                for (int t = 0; t < NM; t++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (t < NR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (kk + 1 == KK) {
                        constexpr int per = (P + NM - 1) / NM;
                        __builtin_amdgcn_sched_group_barrier(0x010, per, 0);
                    }
                }
            }
        }
    };

    // ---- persistent loop over this workgroup's macro tiles
    int tile = blockIdx.x;
    int pm, pn;
    fo_wg_to_tile(tile, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);
    pm = __builtin_amdgcn_readfirstlane(pm);
    pn = __builtin_amdgcn_readfirstlane(pn);
    set_tile(pm, pn);
    issue_any(0, 0);
    bool carried = false;  // stores of an earlier tile may still be in flight

    for (;;) {
        // storage slots of this macro tile's reorder tiles (scalar loads, used by the epilogue)
        int rs[kMaxSub] = {0, 0, 0, 0};
        if (MODE != MODE_PLAIN) {
#pragma unroll
            for (int s = 0; s < kMaxSub; s++)
                if (s < nsub) rs[s] = RAc[(pm * (MTM / p.BM) + s / sub_n) * p.TN + pn * sub_n + s % sub_n];
        }
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

        // Stage 0 of this tile is in flight.  First tile: request the rest of the
        // ring, then wait for stage 0.  Later tiles: stage 0 was requested before
        // the previous epilogue, whose strips lived behind slot 0, so the rest
        // of the ring is requested only after the barrier; the previous tile's
        // NST stores are younger than stage 0 and need not have completed.
        if (!carried) {
#pragma unroll
            for (int s = 1; s < STAGES; s++)
                if (s < KT) issue_any(s, s);
            if (KT >= STAGES)
                wait_vmcnt<(STAGES - 1) * P>();
            else
                wait_vmcnt<0>();
            if (ktail && KT == 1) zero_tail(0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            wait_vmcnt<NST>();
            if (ktail && KT == 1) zero_tail(0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
#pragma unroll
            for (int s = 1; s < STAGES; s++)
                if (s < KT) issue_any(s, s);
        }
        FO_LOAD_FRAGS(0, smem, 0)

        using dyn = std::integral_constant<int, -1>;
        int slot = 0;  // ring slot of K step kt
        int kt = 0;
        for (; kt < STAGES - 1 && kt < KT; kt++) {
            const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
            kstep(std::false_type{}, dyn{}, kt == 0, kt, slot, nslot);
            slot = nslot;
        }
        if (MODE != MODE_PLAIN && KT >= 2) owed = false;  // sent in the first K step
        if constexpr (STAGES == 2) {
            // here kt == 1 (slot 1) when KT > 1
            for (; kt + 1 + STAGES < KT_full; kt += 2) {
                kstep(std::true_type{}, std::integral_constant<int, 1>{}, false, kt, 1, 0);
                kstep(std::true_type{}, std::integral_constant<int, 0>{}, false, kt + 1, 0, 1);
            }
        } else {
            for (; kt + STAGES < KT_full; kt++) {
                const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
                kstep(std::true_type{}, dyn{}, false, kt, slot, nslot);
                slot = nslot;
            }
        }
        for (; kt < KT; kt++) {
            const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
            kstep(std::false_type{}, dyn{}, kt == 0, kt, slot, nslot);
            slot = nslot;
        }

        // every wavefront is done reading the ring (no loads are in flight here)
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");

        // request the next tile's first stage; it lands during the epilogue
        const int cur_pm = pm, cur_pn = pn;
        const int next = tile + gridDim.x;
        const bool has_next = next < ntiles;
        if (has_next) {
            fo_wg_to_tile(next, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);
            pm = __builtin_amdgcn_readfirstlane(pm);
            pn = __builtin_amdgcn_readfirstlane(pn);
            set_tile(pm, pn);
            issue_any(0, 0);
        }

        // ---- epilogue: accumulators -> 16-bit -> LDS (per-wave strip of 32 rows) -> global
        // A wavefront's WTM x WTN block lies inside one reorder tile (BM and BN
        // are multiples of 128), so the tile's slot and base address are scalars
        // and a lane adds one 32-bit offset.  The lane id is laundered through an
        // empty asm so that this addressing is recomputed per tile instead of
        // being hoisted into registers that would stay live across the K loop.
        {
            int el = lane;
            asm volatile("" : "+v"(el));
            const int erow = el & 31, ek = el >> 5;
            uint16_t *strip = reinterpret_cast<uint16_t *>(smem + STAGE16) + wave * (32 * PITCH);
            const int srow = el / CPR, scol = el % CPR;
            const int ldp = MODE == MODE_PLAIN ? p.N : p.rLDN * p.BN;  // leading dimension of the output view
            const int row0 = (wm * WTM) % p.BM, col0 = (wn * WTN) % p.BN;  // of this wavefront inside its reorder tile
            int r = 0;
            if (MODE != MODE_PLAIN) {
                const int s = ((wm * WTM) / p.BM) * sub_n + (wn * WTN) / p.BN;
                r = s == 0 ? rs[0] : s == 1 ? rs[1] : s == 2 ? rs[2] : rs[3];
            }
            const long trow = MODE == MODE_PLAIN ? (long)cur_pm * MTM + wm * WTM
                                                 : (long)(r / p.rLDN) * p.BM + row0;  // first output row of the block
            const long tcol = MODE == MODE_PLAIN ? (long)cur_pn * MTN + wn * WTN
                                                 : (long)(r % p.rLDN) * p.BN + col0;
            char *cbase = reinterpret_cast<char *>(p.C) + (trow * ldp + tcol) * 2;  // wave-uniform
            const unsigned lane_off = (unsigned)(srow * ldp + scol * 8) * 2;
            // scatter: the row map entries of all rows this lane will store, fetched in one batch
            int32_t dest_row[MODE == MODE_SCATTER ? FM * (32 / RPP) : 1];
            if (MODE == MODE_SCATTER) {
#pragma unroll
                for (int i = 0; i < FM; i++)
#pragma unroll
                    for (int ps = 0; ps < 32 / RPP; ps++)
                        dest_row[i * (32 / RPP) + ps] = p.RE[trow + i * 32 + ps * RPP + srow];
            }
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
                        *reinterpret_cast<fo_u32x2 *>(strip + erow * PITCH + j * 32 + q * 8 + ek * 4) = v;
                    }
                }
                // the strip is private to this wavefront: order its LDS writes before its reads
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int ps = 0; ps < 32 / RPP; ps++) {
                    const int row = ps * RPP + srow;
                    fo_u32x4 v = *reinterpret_cast<const fo_u32x4 *>(strip + row * PITCH + scol * 8);
                    if (MODE == MODE_SCATTER) {
                        // rows go through the row map: per-lane 64-bit address
                        const long prow = dest_row[i * (32 / RPP) + ps];
                        store16_write_through(p.C + (size_t)prow * ldp + tcol + scol * 8, v);
                    } else {
                        char *sb = cbase + (size_t)(i * 32 + ps * RPP) * ldp * 2;
                        if (MODE == MODE_PLAIN)
                            store16(sb, lane_off, v);
                        else
                            store16_write_through(sb, lane_off, v);
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);  // strip reads done before the next strip overwrites it
                __builtin_amdgcn_wave_barrier();
            }
        }

        if (MODE != MODE_PLAIN) {
            if (has_next && KT >= 2) {
                // sent from inside the next tile's first K step
                owed = true;
#pragma unroll
                for (int s = 0; s < kMaxSub; s++) prev_rs[s] = rs[s];
            } else {
                // Every lane waits until its own stores are acknowledged, the
                // barrier collects the workgroup, and only then one lane
                // releases at agent scope and bumps the group counter.  The
                // reference has no fence here (src/overlap/gemm_with_signal.h:337-351).
                __builtin_amdgcn_s_waitcnt(0);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if (wave == 0) announce(rs);
            }
        }
        if (!has_next) break;
        carried = true;
        tile = next;
    }
#undef FO_LOAD_FRAGS
#undef FO_MFMAS
}

// Dynamic LDS of one workgroup: the ring (the epilogue strips reuse its last
// slot) and the table of group prefix sums.
template <int MTM, int MTN, int BK, int STAGES>
constexpr int smem_bytes() {
    return STAGES * (MTM + MTN) * BK * 2 + kPrefixMax * 4;
}

}  // namespace fo_gemm_dev
