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
// A workgroup of WM x WN wavefronts computes an MTM x MTN macro tile with
// v_mfma_f32_32x32x16_{f16,bf16}.  Operand tiles of BK columns travel
// HBM -> LDS directly (global_load_lds_dwordx4, 1 KiB per wavefront
// instruction, no VGPR staging) into a ring of STAGES buffers; a slot is
// recycled as soon as every wavefront holds its last fragments of it in
// registers, so up to STAGES K steps are resident; one s_barrier per K step.  The
// 16-byte chunks of a tile row are XOR-swizzled (by choosing which global
// chunk each lane fetches) so that the 16 lanes a ds_read_b128 serves per
// clock hit 16 different bank groups.  The accumulators leave through LDS so
// that every global store is a 16-byte piece of a contiguous output row.
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

// s_waitcnt vmcnt(n) only (expcnt/lgkmcnt left at their maxima); gfx9 encoding:
// vmcnt = imm[15:14]:imm[3:0], expcnt = imm[6:4], lgkmcnt = imm[11:8].
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// 16-byte store that writes through the XCD's L2 to memory (system-scope cache
// policy).  Used for the signalled epilogues: the tile must be visible to other
// XCDs before its counter is bumped, and a tile that never becomes dirty in L2
// makes the releasing write-back that precedes the signal nearly free.  The
// compiler does not count this store in vmcnt; the epilogue waits explicitly.
// The trailing s_nop covers the wait states gfx9 requires between a VMEM store
// of more than 8 bytes and a VALU write of its data registers (the compiler
// inserts them for its own stores but cannot see into inline assembly).
__device__ __forceinline__ void store16_write_through(void *ptr, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" : : "v"(ptr), "v"(v) : "memory");
}

// One direct-to-LDS load of 16 bytes per lane in the saddr form: global address =
// wave-uniform base (SGPR pair) + 32-bit per-lane byte offset; LDS address =
// M0 + lane * 16.  Written as assembly because the compiler materialises a
// 64-bit VGPR address for the intrinsic (two VALU instructions per load, which
// steal issue slots from the MFMAs); it does not track these loads in vmcnt,
// the main loop waits explicitly.  The s_nop covers the M0 write -> LDS-DMA
// wait state.
__device__ __forceinline__ void dma_load16(const __attribute__((address_space(1))) char *base, unsigned lane_off,
                                           unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(lane_off), "s"(base)
                 : "memory");
}

// cache policy bits of the operand loads (gfx940 encoding: 1 = sc0, 2 = nt, 16 = sc1)
#ifndef FO_LOAD_CPOL
#define FO_LOAD_CPOL 0
#endif
#define FO_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
#define FO_GLB_PTR(p) ((const __attribute__((address_space(1))) void *)(p))

template <typename Tag, int MTM, int MTN, int BK, int STAGES, int WM, int WN, int MODE, int LOADER = 0,
          int PFD = 0, int DBG = 0>
__global__ __launch_bounds__(WM *WN * 64) void fo_gemm_kernel(GemmArgs p) {
    typedef fo_elem<Tag> E;
    constexpr int NW = WM * WN;
    constexpr int CH = BK / 8;             // 16-byte chunks per tile row
    constexpr int SWZ_SHIFT = CH == 8 ? 1 : 2;  // rows sharing one swizzle key: 16 / CH
    constexpr int WTM = MTM / WM, WTN = MTN / WN;
    constexpr int FM = WTM / 32, FN = WTN / 32;
    constexpr int A_BLK = MTM * CH / 64, B_BLK = MTN * CH / 64;  // 1 KiB blocks per stage
    constexpr int PA = A_BLK / NW, PB = B_BLK / NW;              // blocks per wavefront
    constexpr int STAGE16 = (MTM + MTN) * CH;                    // stage size in 16-byte units
    static_assert(BK == 32 || BK == 64, "BK");
    static_assert(A_BLK % NW == 0 && B_BLK % NW == 0, "tile rows must split evenly over the wavefronts");
    static_assert((NW * (64 / CH)) % 32 == 0, "swizzle key must repeat across a wavefront's blocks");
    static_assert(STAGES >= 2, "ring depth");

    extern __shared__ fo_u32x4 smem[];
    const unsigned smem_lds = (unsigned)(uintptr_t)FO_LDS_PTR(smem);  // LDS byte address of the ring

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;

    int pm, pn;
    fo_wg_to_tile(blockIdx.x, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);

    const int lda16 = p.lda >> 3, ldb16 = p.ldb >> 3;  // row strides in 16-byte chunks
    const int KT = p.K / BK;
    constexpr int KK = BK / 16;  // MFMA k-steps per stage
    constexpr int NM = FM * FN, NR = FM + FN;

    fo_float16v acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    // Fragment addressing: lane l supplies row (l & 31), k-chunk (l >> 5) of
    // each 32x16 operand block.
    const int frow = lane & 31, fk = lane >> 5;
    const int fkey = (frow >> SWZ_SHIFT) & (CH - 1);
    const int a_off = (wm * WTM + frow) * CH;
    const int b_off = MTM * CH + (wn * WTN + frow) * CH;

    // Operand fragments are double buffered in registers: while the MFMAs of
    // k-step kk run, the ds_reads of k-step kk+1 (or of the next stage's first
    // k-step) are in flight.
    fo_u32x4 af[2][FM], bf[2][FN];
#define FO_LOAD_FRAGS(buf_, st_, kk_)                                                   \
    if (!(DBG & 8)) {                                                                   \
        const int c_ = ((kk_) * 2 + fk) ^ fkey;                                         \
        _Pragma("unroll") for (int i = 0; i < FM; i++) af[buf_][i] = (st_)[a_off + i * 32 * CH + c_]; \
        _Pragma("unroll") for (int j = 0; j < FN; j++) bf[buf_][j] = (st_)[b_off + j * 32 * CH + c_]; \
    }
#define FO_MFMAS(kk_)                                                                   \
    if (!(DBG & 8))                                                                     \
    _Pragma("unroll") for (int i = 0; i < FM; i++)                                      \
        _Pragma("unroll") for (int j = 0; j < FN; j++)                                  \
            acc[i][j] = E::mfma(bf[(kk_) & 1][j], af[(kk_) & 1][i], acc[i][j]);

    // ---- main loop, direct-to-LDS loader
    if constexpr (LOADER == 0) {
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
    gptr_t Ab = (gptr_t)(p.A) + ((size_t)pm * MTM + wave * (64 / CH)) * p.lda * 2;
    gptr_t Bb = (gptr_t)(p.B) + ((size_t)pn * MTN + wave * (64 / CH)) * p.ldb * 2;
    const unsigned a_lane = (unsigned)(lrow * p.lda * 2 + lchunk * 16);
    const unsigned b_lane = (unsigned)(lrow * p.ldb * 2 + lchunk * 16);
    const size_t a_blk_bytes = (size_t)NW * (64 / CH) * p.lda * 2;  // between a wave's consecutive blocks
    const size_t b_blk_bytes = (size_t)NW * (64 / CH) * p.ldb * 2;

    // Issue the loads of K step kt into ring slot s (PA + PB instructions per wavefront).
    auto issue = [&](int kt, int s) {
        const unsigned as = smem_lds + (unsigned)(s * STAGE16 + wave * 64) * 16;  // LDS byte addresses
        const unsigned bs = as + MTM * CH * 16;
        gptr_t ak = Ab + (size_t)kt * (BK * 2), bk = Bb + (size_t)kt * (BK * 2);
#pragma unroll
        for (int i = 0; i < PA; i++) dma_load16(ak + i * a_blk_bytes, a_lane, as + i * NW * 1024);
#pragma unroll
        for (int i = 0; i < PB; i++) dma_load16(bk + i * b_blk_bytes, b_lane, bs + i * NW * 1024);
    };

    constexpr int P = PA + PB;   // load instructions per wavefront and stage

    // L2 prefetch (PFD > 0): the CUs of an XCD that share an operand block run in
    // step, so the first touch of a line makes all of them wait for HBM.  Every
    // K step each lane therefore also touches one cache line of stage
    // kt+STAGES+PFD-1 with a 4-byte direct-to-LDS load into a scratch area that
    // nobody reads (no VGPR to reserve, no data dependency); by the time the
    // real loads of that stage are issued the lines sit in L2.
    constexpr int NPF = PFD > 0 ? (MTM + MTN) / (NW * 64) : 0;
    static_assert(PFD == 0 || (MTM + MTN) % (NW * 64) == 0, "one prefetch lane per tile row");
    static_assert((STAGES - 1) * P + (PFD + STAGES) * NPF < 64, "vmcnt range");
    const char *pf_base[NPF > 0 ? NPF : 1];
    if constexpr (PFD > 0) {
#pragma unroll
        for (int i = 0; i < NPF; i++) {
            const int j = (wave + i * NW) * 64 + lane;  // tile row: A rows first, then B rows
            pf_base[i] = j < MTM ? reinterpret_cast<const char *>(p.A) + ((size_t)pm * MTM + j) * p.lda * 2
                                 : reinterpret_cast<const char *>(p.B) + ((size_t)pn * MTN + (j - MTM)) * p.ldb * 2;
        }
    }
    auto prefetch = [&](int kt) {
        if constexpr (PFD > 0) {
            fo_u32x4 *dump = smem + STAGES * STAGE16 + wave * 16;
#pragma unroll
            for (int i = 0; i < NPF; i++)
                __builtin_amdgcn_global_load_lds(FO_GLB_PTR(pf_base[i] + (size_t)kt * (BK * 2)), FO_LDS_PTR(dump), 4,
                                                 0, 0);
        }
    };

#pragma unroll
    for (int s = 0; s < STAGES; s++)
        if (s < KT) issue(s, s);
#pragma unroll
    for (int s = STAGES; s < STAGES + PFD; s++)
        if (s < KT) prefetch(s);

    if (KT >= STAGES + PFD)
        wait_vmcnt<(STAGES - 1) * P + PFD * NPF>();
    else
        wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    FO_LOAD_FRAGS(0, smem, 0)

    // One K step.  STEADY: at least STAGES further steps exist, so the waits and
    // the refill are unconditional and the body is a single scheduling region
    // per k-step, pinned MFMA-first with the memory instructions in its shadow.
    // STEADY additionally means kt >= STAGES-1 and that a prefetch is still due,
    // so the number of younger loads in flight at the wait is a constant.
    // With two slots the loop is unrolled by two and the slot is a compile-time
    // constant (slot_tag >= 0), which makes every LDS address loop-invariant.
    auto kstep = [&](auto steady, auto slot_tag, int kt, int slot_rt, int nslot_rt) {
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
                if (!(DBG & 1)) {
                if (STEADY)
                    wait_vmcnt<(STAGES - 2) * P + (STAGES - 1) * NPF>();
                else if (kt + STAGES - 1 < KT)
                    wait_vmcnt<(STAGES - 2) * P>();  // conservative: also waits for prefetches
                else
                    wait_vmcnt<0>();
                __builtin_amdgcn_s_barrier();
                }
                asm volatile("" ::: "memory");
                if (!(DBG & 2)) if (STEADY || kt + STAGES < KT) issue((DBG & 4) ? (kt & 1) : kt + STAGES, slot);
                if (STEADY || kt + STAGES + PFD < KT) prefetch(kt + STAGES + PFD);
                FO_LOAD_FRAGS((kk + 1) & 1, smem + nslot * STAGE16, 0)
            }
            // The N-side block is the MFMA's first operand, so a lane's four
            // consecutive accumulator values are consecutive output columns.
            FO_MFMAS(kk)
            if (STEADY) {
                // issue order inside this k-step: MFMA, ds_read, MFMA, ds_read, ...
                // then (last k-step) the direct-to-LDS loads between the remaining MFMAs
#pragma unroll
                for (int t = 0; t < NM; t++) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (t < NR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if (kk + 1 == KK) {
                        constexpr int per = (P + NPF + NM - 1) / NM;
                        __builtin_amdgcn_sched_group_barrier(0x010, per, 0);
                    }
                }
            }
        }
    };

    using dyn = std::integral_constant<int, -1>;
    int slot = 0;  // ring slot of K step kt
    int kt = 0;
    for (; kt < STAGES - 1 && kt < KT; kt++) {
        const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
        kstep(std::false_type{}, dyn{}, kt, slot, nslot);
        slot = nslot;
    }
    if constexpr (STAGES == 2) {
        // here kt == 1 (slot 1) when KT > 1
        for (; kt + 1 + STAGES + PFD < KT; kt += 2) {
            kstep(std::true_type{}, std::integral_constant<int, 1>{}, kt, 1, 0);
            kstep(std::true_type{}, std::integral_constant<int, 0>{}, kt + 1, 0, 1);
        }
    } else {
        for (; kt + STAGES + PFD < KT; kt++) {
            const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
            kstep(std::true_type{}, dyn{}, kt, slot, nslot);
            slot = nslot;
        }
    }
    for (; kt < KT; kt++) {
        const int nslot = slot + 1 == STAGES ? 0 : slot + 1;
        kstep(std::false_type{}, dyn{}, kt, slot, nslot);
        slot = nslot;
    }
    }

    // ---- main loop, register-staged loader: HBM -> VGPR -> LDS (ds_write_b128), two
    // LDS slots.  Per K step: the fragments of k-step kk+1 are fetched while the
    // MFMAs of kk run; in the second-to-last k-step the next stage (already in
    // registers) is written to the other slot; before the last k-step one barrier
    // publishes it, after which the next stage's first fragments and the global
    // loads of the stage after that are issued in the shadow of the last MFMAs.
    if constexpr (LOADER == 1) {
        constexpr int NT = NW * 64;
        constexpr int RP = NT / CH;  // tile rows covered by one pass of the whole workgroup
        constexpr int LA = MTM / RP, LB = MTN / RP;
        static_assert(RP % 32 == 0 && MTM % RP == 0 && MTN % RP == 0, "loader split");
        const int lc = tid % CH, lr = tid / CH;
        const int lsw = lc ^ ((lr >> SWZ_SHIFT) & (CH - 1));
        const fo_u32x4 *Ag = reinterpret_cast<const fo_u32x4 *>(p.A) + ((size_t)pm * MTM + lr) * lda16 + lc;
        const fo_u32x4 *Bg = reinterpret_cast<const fo_u32x4 *>(p.B) + ((size_t)pn * MTN + lr) * ldb16 + lc;
        const size_t apass = (size_t)RP * lda16, bpass = (size_t)RP * ldb16;
        fo_u32x4 ra[LA], rb[LB];
#define FO_GLOAD(kt_)                                                                          \
    _Pragma("unroll") for (int i = 0; i < LA; i++) ra[i] = Ag[i * apass + (size_t)(kt_) * CH]; \
    _Pragma("unroll") for (int i = 0; i < LB; i++) rb[i] = Bg[i * bpass + (size_t)(kt_) * CH];
#define FO_LSTORE(slot_)                                                                       \
    _Pragma("unroll") for (int i = 0; i < LA; i++)                                             \
        smem[(slot_) * STAGE16 + (lr + i * RP) * CH + lsw] = ra[i];                            \
    _Pragma("unroll") for (int i = 0; i < LB; i++)                                             \
        smem[(slot_) * STAGE16 + MTM * CH + (lr + i * RP) * CH + lsw] = rb[i];

        FO_GLOAD(0)
        FO_LSTORE(0)
        if (KT > 1) {
            FO_GLOAD(1)
        }
        __syncthreads();
        FO_LOAD_FRAGS(0, smem, 0)

        auto kstep = [&](auto steady, int kt) {
            constexpr bool STEADY = decltype(steady)::value;  // kt + 2 < KT
            const int slot = kt & 1;
            const fo_u32x4 *st = smem + slot * STAGE16;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) {
                if (kk + 1 < KK) {
                    FO_LOAD_FRAGS((kk + 1) & 1, st, kk + 1)
                }
                if (kk == KK - 2 && (STEADY || kt + 1 < KT)) {
                    FO_LSTORE(slot ^ 1)
                }
                if (kk == KK - 1 && (STEADY || kt + 1 < KT)) {
                    // own reads of this slot and own writes of the other one are
                    // complete; the barrier makes that true for the workgroup
                    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    FO_LOAD_FRAGS((kk + 1) & 1, smem + (slot ^ 1) * STAGE16, 0)
                    if (STEADY || kt + 2 < KT) {
                        FO_GLOAD(kt + 2)
                    }
                }
                FO_MFMAS(kk)
                if (STEADY) {
                    constexpr int NL = LA + LB;
#pragma unroll
                    for (int t = 0; t < NM; t++) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        if (t < NR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        if (kk == KK - 2) __builtin_amdgcn_sched_group_barrier(0x200, (NL + NM - 1) / NM, 0);
                        if (kk == KK - 1) __builtin_amdgcn_sched_group_barrier(0x020, (NL + NM - 1) / NM, 0);
                    }
                }
            }
        };
        int kt = 0;
        for (; kt + 2 < KT; kt++) kstep(std::true_type{}, kt);
        for (; kt < KT; kt++) kstep(std::false_type{}, kt);
#undef FO_GLOAD
#undef FO_LSTORE
    }

    // ---- main loop, register-staged loader with two register sets (LOADER == 2):
    // HBM -> VGPR -> LDS through ds_write_b128 (128 B/clk, twice the rate at which
    // direct-to-LDS loads occupy the LDS), two LDS slots.  Stage s is requested
    // in K step s-3 (k-steps 2,3), written to LDS in K step s-1 (k-steps 0,1)
    // and consumed in K step s, so a load has about 1.5 K steps to arrive and
    // the memory instructions are spread evenly between the MFMAs.
    if constexpr (LOADER == 2 || LOADER == 3) {
        constexpr int NSETS = LOADER == 2 ? 2 : 1;  // register sets: a load has NSETS - 0.5 K steps to arrive
        static_assert(KK == 4, "the two-set loader is scheduled for BK = 64");
        constexpr int NT = NW * 64;
        constexpr int RP = NT / CH;  // tile rows covered by one pass of the whole workgroup
        constexpr int LA = MTM / RP, LB = MTN / RP, NL = LA + LB;
        static_assert(RP % 32 == 0 && MTM % RP == 0 && MTN % RP == 0 && NL % 2 == 0, "loader split");
        const int lc = tid % CH, lr = tid / CH;
        const int lsw = lc ^ ((lr >> SWZ_SHIFT) & (CH - 1));
        // Addresses as a wave-uniform base (SGPRs, advanced with scalar adds) plus one
        // 32-bit per-lane byte offset, so the loads use the saddr form and no VGPRs
        // are spent on 64-bit pointers.
        const char *Ab = reinterpret_cast<const char *>(p.A) + (size_t)pm * MTM * p.lda * 2;
        const char *Bb = reinterpret_cast<const char *>(p.B) + (size_t)pn * MTN * p.ldb * 2;
        const unsigned a_lane = (unsigned)(lr * p.lda * 2 + lc * 16);
        const unsigned b_lane = (unsigned)(lr * p.ldb * 2 + lc * 16);
        const size_t apass = (size_t)RP * p.lda * 2, bpass = (size_t)RP * p.ldb * 2;  // bytes
        fo_u32x4 rs[NSETS][NL];
        // loads / stores i in [lo_, hi_) of one stage; i < LA are A rows, the rest B rows
#define FO_GLOAD2(set_, kt_, lo_, hi_)                                                          \
    _Pragma("unroll") for (int i = (lo_); i < (hi_); i++)                                       \
        rs[set_][i] = i < LA ? *reinterpret_cast<const fo_u32x4 *>(Ab + i * apass + (size_t)(kt_) * (BK * 2) + a_lane) \
                             : *reinterpret_cast<const fo_u32x4 *>(Bb + (i - LA) * bpass + (size_t)(kt_) * (BK * 2) + b_lane);
#define FO_LSTORE2(set_, slot_, lo_, hi_)                                                       \
    _Pragma("unroll") for (int i = (lo_); i < (hi_); i++)                                       \
        smem[(slot_) * STAGE16 + (i < LA ? (lr + i * RP) * CH : MTM * CH + (lr + (i - LA) * RP) * CH) + lsw] = \
            rs[set_][i];

        FO_GLOAD2(0, 0, 0, NL)
        if (NSETS == 2 && KT > 1) {
            FO_GLOAD2(NSETS - 1, 1, 0, NL)
        }
        FO_LSTORE2(0, 0, 0, NL)
        if (KT > NSETS) {
            FO_GLOAD2(0, NSETS, 0, NL)
        }
        __syncthreads();
        FO_LOAD_FRAGS(0, smem, 0)

        // K step kt with parity PAR = kt & 1; the set that holds stage kt+1 is PAR ^ 1.
        auto kstep = [&](auto steady, auto parity, int kt) {
            constexpr bool STEADY = decltype(steady)::value;  // kt + 3 < KT
            constexpr int PAR = decltype(parity)::value;
            constexpr int NXT = PAR ^ 1;               // LDS slot of stage kt+1
            constexpr int SET = NSETS == 2 ? NXT : 0;  // register set of stage kt+1, refilled with stage kt+1+NSETS
            const fo_u32x4 *st = smem + PAR * STAGE16;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) {
                if (kk + 1 < KK) {
                    FO_LOAD_FRAGS((kk + 1) & 1, st, kk + 1)
                }
                if (kk < 2 && (STEADY || kt + 1 < KT)) {
                    FO_LSTORE2(SET, NXT, kk * (NL / 2), (kk + 1) * (NL / 2))
                }
                if (kk == 2 && (STEADY || kt + 1 + NSETS < KT)) {
                    FO_GLOAD2(SET, kt + 1 + NSETS, 0, NL / 2)
                }
                if (kk == 3 && (STEADY || kt + 1 < KT)) {
                    // own reads of this slot and own writes of the other one are
                    // complete; the barrier makes that true for the workgroup
                    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    FO_LOAD_FRAGS((kk + 1) & 1, smem + NXT * STAGE16, 0)
                }
                if (kk == 3 && (STEADY || kt + 1 + NSETS < KT)) {
                    FO_GLOAD2(SET, kt + 1 + NSETS, NL / 2, NL)
                }
                FO_MFMAS(kk)
                if (STEADY && !(DBG & 16)) {
                    constexpr int NO = NL / 2;  // ds_writes (k-steps 0,1) or global loads (2,3) in this region
                    static_assert(NR <= NM && NO <= NM, "at most one read and one write/load per MFMA");
#pragma unroll
                    for (int t = 0; t < NM; t++) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                        if (((t + 1) * NR) / NM > (t * NR) / NM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        if (((t + 1) * NO) / NM > (t * NO) / NM) {
                            if (kk < 2)
                                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
                            else
                                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                        }
                    }
                }
            }
        };
        int kt = 0;
        for (; kt + 4 < KT; kt += 2) {
            kstep(std::true_type{}, std::integral_constant<int, 0>{}, kt);
            kstep(std::true_type{}, std::integral_constant<int, 1>{}, kt + 1);
        }
        for (; kt < KT; kt++) {
            if (kt & 1)
                kstep(std::false_type{}, std::integral_constant<int, 1>{}, kt);
            else
                kstep(std::false_type{}, std::integral_constant<int, 0>{}, kt);
        }
#undef FO_GLOAD2
#undef FO_LSTORE2
    }

#undef FO_LOAD_FRAGS
#undef FO_MFMAS
    __syncthreads();  // every wavefront is done reading the ring: reuse it for the epilogue

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
        // the strip is private to this wavefront: order its LDS writes before its reads
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
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
            if (MODE == MODE_PLAIN)
                *reinterpret_cast<fo_u32x4 *>(p.C + off) = v;
            else
                store16_write_through(p.C + off, v);
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // strip reads done before the next strip overwrites it
        __builtin_amdgcn_wave_barrier();
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

// Dynamic LDS of one workgroup: the ring plus 4 KiB of prefetch scratch.
template <int MTM, int MTN, int BK, int STAGES>
constexpr int smem_bytes() {
    return STAGES * (MTM + MTN) * BK * 2 + 4096;
}

}  // namespace fo_gemm_dev
