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
// This template serves the 128x128, 128x256 and 256x128 workgroup tiles; the
// 256x256 tile has a kernel of its own (fo_gemm256_kernel.h), which shares the
// arguments, the raster and the helpers defined here.
//
// The kernel is persistent: the launch holds at most as many workgroups as the
// chip keeps resident, and workgroup w computes macro tiles w, w + grid,
// w + 2 grid, ... of the raster.  A workgroup of WM x WN wavefronts computes an
// MTM x MTN macro tile with v_mfma_f32_16x16x32_{f16,bf16}: in an MFMA-only
// loop under this part's power limit that form sustains 14 % more than
// 32x32x16 (a quarter of the accumulator registers per instruction, half of
// their traffic per flop), and the whole kernel is power-limited.
//
// Operand tiles of BK columns travel HBM -> LDS directly
// (global_load_lds_dwordx4, 1 KiB per wavefront instruction, no VGPR staging)
// into two rings, SA slots for the A part of a K step and SB <= SA slots for
// the B part; one s_barrier per K step, placed behind the last LDS read of the
// step, recycles both slots.  (SA = SB + 1 = 3 is all that 160 KiB of LDS allow
// for a 256x256x64 step: the A part is then requested two K steps ahead.  It
// measured 4 % faster with all-zero operands and no faster with real ones, and
// is not used.)  The 16-byte chunks of a tile row are XOR-swizzled (by choosing
// which global chunk each lane fetches) so that the 16 lanes a ds_read_b128
// serves per clock hit 16 different bank groups.  Fragments stream through a
// short register ring (see the K step), 32 accumulator blocks of 16x16 stay in
// place, and the accumulators leave through LDS so that every global store is
// a 16-byte piece of a contiguous output row.
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
    int grid_m, grid_n, panel, xcd_remap;  // the raster of this launch's parent tiles
    int first, sub_m, sub_n, count;        // this launch: positions from `first`, each cut into sub_m x sub_n macro tiles, `count` of them
    int quiet;                             // signalling epilogues: store the tiles reordered, touch no counter
    int stream_out;                        // 256x256 kernel: store the output with the non-temporal hint
};

constexpr int kMaxSub = 4;        // reorder tiles per macro tile (256x256 over 128x128)
constexpr int kPrefixRegs = 256;  // group search on prefix sums held in registers (one per 64 groups) up to this many groups

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

// 16-byte global stores written as assembly so that the number of vector memory
// instructions in flight is known exactly (the main loop waits on vmcnt with
// non-zero counts; the compiler does not see these instructions in its own
// count, which can only make its waits longer, never shorter).  The
// write-through form (system-scope cache policy) is used for the signalled
// epilogues: the tile must be visible to other XCDs before its counter is
// bumped, and a tile that never becomes dirty in L2 needs no releasing
// write-back before the signal.  The trailing s_nop covers
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
// The same with the non-temporal hint, for outputs too large to be found in a cache by whoever reads them
// next (GemmArgs::stream_out): the resident workgroups finish their tiles together and store 128 KB each
// at once, and output lines that took room in the L2 would push out the operand panels the next tile's
// first K steps are about to share.  8192^3: GEMM alone 1.7 % faster, the overlapped step unchanged; on
// the 8192x4096 output (67 MB), which the consumer finds in the memory-side cache, the hint made the
// overlapped step 2 % and the serial step 8 % slower, so smaller outputs stay cacheable.
__device__ __forceinline__ void store16_write_through_nt(void *ptr, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt\n\ts_nop 1" : : "v"(ptr), "v"(v) : "memory");
}
__device__ __forceinline__ void store16_write_through_nt(char *base, unsigned lane_off, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, %2 sc0 sc1 nt\n\ts_nop 1"
                 :
                 : "v"(lane_off), "v"(v), "s"((__attribute__((address_space(1))) char *)base)
                 : "memory");
}
__device__ __forceinline__ void store16_nt(char *base, unsigned lane_off, fo_u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, %2 nt\n\ts_nop 1"
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

template <typename Tag, int MTM, int MTN, int BK, int SA, int SB, int WM, int WN, int MODE>
__global__ __launch_bounds__(WM *WN * 64) void fo_gemm_kernel(GemmArgs p) {
    typedef fo_elem<Tag> E;
    constexpr int NW = WM * WN;
    constexpr int CH = BK / 8;                  // 16-byte chunks per tile row
    constexpr int SWZ_SHIFT = CH == 8 ? 1 : 2;  // rows sharing one swizzle key: 16 / CH
    constexpr int WTM = MTM / WM, WTN = MTN / WN;
    constexpr int FM = WTM / 16, FN = WTN / 16;  // 16x16 accumulator blocks per wavefront
    constexpr int FMB = WTM / 32;                // 32-row groups of the epilogue
    constexpr int A_BLK = MTM * CH / 64, B_BLK = MTN * CH / 64;  // 1 KiB blocks per stage
    constexpr int PA = A_BLK / NW, PB = B_BLK / NW;              // blocks per wavefront
    constexpr int P = PA + PB;                                   // load instructions per wavefront and stage
    constexpr int A16 = MTM * CH;                                // A part of a stage in 16-byte units
    constexpr int STAGE16 = (MTM + MTN) * CH;                    // stage size in 16-byte units
    // LDS: stage-major, A part then B part; with SA = SB + 1 the last stage has an A part only
    constexpr int RING16 = SB * STAGE16 + (SA - SB) * A16;
    // vector memory instructions that may stay in flight when the next K step's operands are needed:
    // everything requested after that step's last part (request order per step: B part, then A part).
    // Waiting with a non-zero count relies on vmcnt retiring this wavefront's loads and stores in
    // issue order, as it does on gfx9-family parts (one counter for both, decremented in order): when
    // vmcnt(n) returns, everything but the youngest n instructions has completed.
    constexpr int ALLOW = (SA - SB) * PA + (SB - 2) * P;
    constexpr int KK = BK / 32;                                  // MFMA k-steps per stage
    // epilogue: per-wavefront strip of 32 rows x WTN columns in the ring behind slot 0
    constexpr int PITCH = WTN + 8;   // halfs; keeps 16-byte alignment, skews banks
    constexpr int CPR = WTN / 8;     // 16-byte chunks per strip row
    constexpr int RPP = 64 / CPR;    // strip rows per store pass
    constexpr int NST = FMB * (32 / RPP);  // store instructions per wavefront and tile
    static_assert(BK == 64, "BK: two MFMA k-steps per stage (the B fragment buffers alternate with their parity)");
    static_assert(A_BLK % NW == 0 && B_BLK % NW == 0, "tile rows must split evenly over the wavefronts");
    static_assert((NW * (64 / CH)) % 32 == 0, "swizzle key must repeat across a wavefront's blocks");
    static_assert(SB >= 2 && (SA == SB || SA == SB + 1), "ring depths");
    static_assert(NW * 32 * PITCH * 2 <= (RING16 - STAGE16) * 16, "the epilogue strips must fit behind stage 0");
    static_assert(SA * PA + SB * PB + NST < 64, "vmcnt range");

    extern __shared__ fo_u32x4 smem[];
    const unsigned smem_lds = (unsigned)(uintptr_t)FO_LDS_PTR(smem);  // LDS byte address of the ring

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int ntiles = p.count;
    // K is a multiple of 8 (one 16-byte chunk).  A last K step that is not full
    // is loaded with its out-of-range chunks redirected to the step's first
    // chunk (valid memory) and zeroed in LDS before the stage is published.
    const int KT = (p.K + BK - 1) / BK;
    const bool ktail = (p.K % BK) != 0;
    const int KT_full = ktail ? KT - 1 : KT;  // K steps whose loads need no special care

    // Fragment addressing: lane l supplies row (l & 15), k-chunk (l >> 4) of
    // each 16x32 operand block.
    const int frow = lane & 15, fk = lane >> 4;
    const int fkey = (frow >> SWZ_SHIFT) & (CH - 1);
    // LDS byte addresses of this lane's 16 bytes in the first block of the A
    // part / B part of stage 0 for MFMA k-step 0.  Everything else is derived
    // from them inside a K step (slot: + multiple of the stage size, k-step:
    // flip bit 2 of the chunk index, block: + immediate), from copies the compiler
    // cannot see through: as loop invariants the derived addresses would occupy
    // sixteen registers for the whole K loop.
    const unsigned la = smem_lds + (unsigned)((wm * WTM + frow) * CH + (fk ^ fkey)) * 16;
    const unsigned lb = smem_lds + (unsigned)(MTM * CH + (wn * WTN + frow) * CH + (fk ^ fkey)) * 16;
    constexpr unsigned STAGE_B = STAGE16 * 16, BLOCK_B = 16 * CH * 16, KSTEP_X = 4 * 16;
    static_assert(STAGE_B % (2 * KSTEP_X) == 0, "adding a slot offset must not disturb the k-step bit");
    typedef const __attribute__((address_space(3))) fo_u32x4 *lds16_t;

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
    // Request the A part / B part of K step kt into slot s of its ring (PA / PB
    // instructions per wavefront).
    auto issue_a_with = [&](int kt, int s, unsigned al) {
        const unsigned as = smem_lds + (unsigned)(s * STAGE16 + wave * 64) * 16;  // LDS byte address
        gptr_t ak = Ab + (size_t)kt * (BK * 2);
#pragma unroll
        for (int i = 0; i < PA; i++) dma_load16(ak + i * a_blk_bytes, al, as + i * NW * 1024);
    };
    auto issue_b_with = [&](int kt, int s, unsigned bl) {
        const unsigned bs = smem_lds + (unsigned)(s * STAGE16 + A16 + wave * 64) * 16;
        gptr_t bk = Bb + (size_t)kt * (BK * 2);
#pragma unroll
        for (int i = 0; i < PB; i++) dma_load16(bk + i * b_blk_bytes, bl, bs + i * NW * 1024);
    };
    auto issue_a = [&](int kt, int s) { issue_a_with(kt, s, a_lane); };
    auto issue_b = [&](int kt, int s) { issue_b_with(kt, s, b_lane); };
    // Load number q of the P a wavefront requests per K step (the B part of step
    // kb into slot sb first, then the A part of step ka into slot sa), so that
    // the steady loop can place them one by one between its MFMAs.
    auto issue_one = [&](int q, int kb, int sb, int ka, int sa) {
        if (q < PB) {
            const unsigned bs = smem_lds + (unsigned)(sb * STAGE16 + A16 + wave * 64) * 16;
            dma_load16(Bb + (size_t)kb * (BK * 2) + q * b_blk_bytes, b_lane, bs + q * NW * 1024);
        } else {
            const unsigned as = smem_lds + (unsigned)(sa * STAGE16 + wave * 64) * 16;
            dma_load16(Ab + (size_t)ka * (BK * 2) + (q - PB) * a_blk_bytes, a_lane, as + (q - PB) * NW * 1024);
        }
    };
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
    // Same loads; in the partial step a chunk beyond K is fetched from the row's first chunk of that step instead.
    auto issue_a_any = [&](int kt, int s) {
        if (ktail && kt == KT - 1) {
            int row;
            const bool out = tail_chunk_out(&row);
            issue_a_with(kt, s, out ? (unsigned)(row * p.lda * 2) : a_lane);
        } else {
            issue_a(kt, s);
        }
    };
    auto issue_b_any = [&](int kt, int s) {
        if (ktail && kt == KT - 1) {
            int row;
            const bool out = tail_chunk_out(&row);
            issue_b_with(kt, s, out ? (unsigned)(row * p.ldb * 2) : b_lane);
        } else {
            issue_b(kt, s);
        }
    };
    // Zero this lane's chunks of the partial step (A part in slot sa, B part in
    // slot sb).  Called after the lane's own loads of that step have landed and
    // before the barrier that publishes it.
    auto zero_tail = [&](int sa, int sb) {
        int row;
        if (tail_chunk_out(&row)) {
            int el = lane;
            asm volatile("" : "+v"(el));
            fo_u32x4 *mine_a = smem + sa * STAGE16 + wave * 64 + el;
            fo_u32x4 *mine_b = smem + sb * STAGE16 + A16 + wave * 64 + el;
            const fo_u32x4 z = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < PA; i++) mine_a[i * NW * 64] = z;
#pragma unroll
            for (int i = 0; i < PB; i++) mine_b[i * NW * 64] = z;
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    };
    // Everything of a tile that is requested ahead of its first K step, except
    // stage 0, in the order the K loop's waits assume: the A parts that run one
    // step further ahead than the B parts first, then per step its B part and
    // the A part requested with it.
    auto issue_rest_of_prologue = [&]() {
#pragma unroll
        for (int k = 1; k <= SA - SB; k++)
            if (k < KT) issue_a_any(k, k);
#pragma unroll
        for (int k = 1; k < SB; k++) {
            if (k < KT) issue_b_any(k, k);
            if (k + SA - SB < KT) issue_a_any(k + SA - SB, k + SA - SB);
        }
    };

    // ---- signalling state (signal and scatter epilogues)
    const int sub_n = MTN / p.BN, nsub = (MTM / p.BM) * sub_n;  // reorder tiles per macro tile
    typedef const __attribute__((address_space(4))) int32_t *cptr_t;  // read-only for the whole launch: scalar loads
    const cptr_t RAc = (cptr_t)(uintptr_t)p.RA;
    // Inclusive prefix sums of cseg, entries lane, lane + 64, ... in kPrefixRegs / 64
    // registers of every lane (the search below is a ballot over them: no memory
    // access, so it never waits behind operand loads in flight).  More than
    // kPrefixRegs groups are searched in memory.
    constexpr int NPRE = kPrefixRegs / 64;
    int pre[NPRE];
#pragma unroll
    for (int q = 0; q < NPRE; q++) pre[q] = 0;
    const bool reg_search = p.G <= kPrefixRegs;
    const bool signalling = MODE != MODE_PLAIN && !p.quiet;
    if (signalling && reg_search) {
        int base = 0;
#pragma unroll
        for (int q = 0; q < NPRE; q++) {
            int v = q * 64 + lane < p.G ? p.cseg[q * 64 + lane] : 0;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                int o = __shfl_up(v, d, 64);
                if (lane >= d) v += o;
            }
            pre[q] = v + base;
            base = __shfl(pre[q], 63, 64);
        }
    }
    auto group_of = [&](int r) {
        if (reg_search) {
#pragma unroll
            for (int q = 0; q < NPRE; q++) {
                unsigned long long hit = __ballot(q * 64 + lane < p.G && pre[q] > r);
                if (hit) return q * 64 + (int)__builtin_ctzll(hit);
            }
            return p.G - 1;
        }
        return find_group(p.cseg, p.G, r, lane);
    };
    // Wavefront 0 announces the reorder tiles whose storage slots are rs[0..nsub)
    // and whose groups are gs[0..nsub).  (The groups are looked up by the caller,
    // at the end of the epilogue: the lookup inside a K step measured 3 us per
    // tile, the counter update alone nothing.)  Callers guarantee that every wavefront's stores of those tiles are complete:
    // the stores are write-through, each wavefront has waited for their
    // acknowledgement (vmcnt) and a workgroup barrier lies between that wait and
    // this call.  The tile is therefore in memory before the counter moves, and
    // the atomic itself is relaxed: a release here would add an L2 write-back
    // (with nothing of this tile left to write back) and a wait for the operand
    // loads in flight, both paid by the whole workgroup at its next barrier.
    auto groups_of = [&](const int (&rs)[kMaxSub], int (&gs)[kMaxSub]) {
#pragma unroll
        for (int s = 0; s < kMaxSub; s++) gs[s] = s < nsub ? group_of(rs[s]) : 0;
    };
    auto announce = [&](const int (&rs)[kMaxSub], const int (&gs)[kMaxSub]) {
#pragma unroll
        for (int s = 0; s < kMaxSub; s++) {
            if (s < nsub) {
                const int r = rs[s];
                const int g = gs[s];
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

    // Operand fragments.  A K step is walked as KK * FM "rows": the FN MFMAs of
    // one A fragment (16 rows of A, 32 columns of K).  An A fragment is dead after
    // its row, so the A side is a short ring: the fragment of row r + AHEAD is
    // fetched right behind row r into the registers row r - 1 used.  The B
    // fragments of an MFMA k-step are live for its FM rows; the next k-step's are
    // fetched during its last FN rows into a second set.
    constexpr int AHEAD = (FM >= 8 ? 7 : 3), ARING = AHEAD + 1;
    // The step's P direct-to-LDS loads are dealt over the rows behind its barrier
    // instead of being issued in one burst (measured: 3 % faster over four rows
    // with AHEAD = 3; AHEAD = 7 with the loads over eight rows another 0.7-1 %,
    // for 16 more registers, where a k-step has eight A fragments).
    constexpr int DMA_ROWS = AHEAD + 1;
    constexpr int ROWS = KK * FM;
    static_assert(FM % ARING == 0 && FN <= FM && AHEAD < FM, "row pipeline");
    fo_float4v acc[FM][FN];
    fo_u32x4 af[ARING], bf[2][FN];
    // base = la or lb (or a laundered copy) + slot * STAGE_B
    auto load_a = [&](int slot, unsigned base, int kk, int i) {
        af[slot] = *reinterpret_cast<lds16_t>((base ^ (kk * KSTEP_X)) + i * BLOCK_B);
    };
    auto load_b = [&](int buf, unsigned base, int kk, int j) {
        bf[buf][j] = *reinterpret_cast<lds16_t>((base ^ (kk * KSTEP_X)) + j * BLOCK_B);
    };

    int prev_rs[kMaxSub] = {0, 0, 0, 0};  // slots and groups of the tile whose signal is still owed
    int prev_gs[kMaxSub] = {0, 0, 0, 0};
    bool owed = false;

    // One K step kt, whose A part is in slot sa of the A ring and whose B part is
    // in slot sb of the B ring.  STEADY: at least SA further full steps exist, so
    // the waits and the refill are unconditional and the body is a single
    // scheduling region per k-step, pinned MFMA-first with the memory
    // instructions in its shadow.  In the unrolled steady loops the slots are
    // compile-time constants (tags >= 0), which makes every LDS address
    // loop-invariant.  `first` marks a tile's first K step: after its barrier
    // every wavefront has waited for the previous tile's stores (they are older
    // than the loads that wait covers), which is where an owed signal is sent.
    auto kstep = [&](auto steady, auto tag_a, auto tag_b, bool first, int kt, int sa_rt, int sb_rt) {
        constexpr bool STEADY = decltype(steady)::value;
        constexpr int SA_C = decltype(tag_a)::value, SB_C = decltype(tag_b)::value;
        const int sa = SA_C >= 0 ? SA_C : sa_rt;
        const int sb = SB_C >= 0 ? SB_C : sb_rt;
        const int nsa = sa + 1 == SA ? 0 : sa + 1;
        const int nsb = sb + 1 == SB ? 0 : sb + 1;
        unsigned la_ = la, lb_ = lb;
        asm volatile("" : "+v"(la_), "+v"(lb_));
        const unsigned sta = la_ + sa * STAGE_B, stb = lb_ + sb * STAGE_B;
        const unsigned nsta = la_ + nsa * STAGE_B, nstb = lb_ + nsb * STAGE_B;
        const bool more = STEADY || kt + 1 < KT;  // a further K step follows in this tile
        // Row SYNC is the last whose fetches read step kt (the A fragment of the
        // step's last row; the last B fragments were fetched in the k-step
        // before).  Behind them the workgroup meets: every wavefront has issued
        // its last reads of step kt, so the two slots can be recycled, and step
        // kt+1 is made visible (own loads landed + barrier) for the fetches of
        // the remaining rows, which already belong to it.
        constexpr int SYNC = ROWS - 1 - AHEAD;
        static_assert(FN <= AHEAD + 1 && SYNC >= ROWS - FM, "the rows behind SYNC fetch the next step's first B fragments");
#pragma unroll
        for (int r = 0; r < ROWS; r++) {
            const int kk = r / FM, i = r % FM;
            const bool last = kk + 1 == KK;
            // One row is one scheduling region: its FN MFMAs, the A fragment of
            // row r + AHEAD, one B fragment of the next k-step in the rows that
            // fetch those, and behind SYNC a share of the direct-to-LDS loads.
            // Nothing may move across a row: a fetch hoisted above the MFMAs that
            // still read the registers it replaces would cost a second register set.
#pragma unroll
            for (int j = 0; j < FN; j++) E::mfma(bf[kk & 1][j], af[r % ARING], acc[i][j]);
            if (r + AHEAD < ROWS) load_a((r + AHEAD) % ARING, sta, (r + AHEAD) / FM, (r + AHEAD) % FM);
            if (!last && i >= FM - FN) load_b((kk + 1) & 1, stb, kk + 1, i - (FM - FN));
            if (r >= SYNC && more) {
                if (r == SYNC) {
                    if (STEADY || kt + SA - 1 < KT)
                        wait_vmcnt<ALLOW>();
                    else
                        wait_vmcnt<0>();
                    if (!STEADY) {
                        if (ktail && kt + 2 == KT) zero_tail(nsa, nsb);  // all loads of step KT-1 have landed (vmcnt 0)
                    }
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    if (!STEADY && MODE != MODE_PLAIN) {
                        if (first && owed && wave == 0) announce(prev_rs, prev_gs);  // never owed when quiet
                    }
                    if constexpr (!STEADY) {
                        if (kt + SB < KT) issue_b_any(kt + SB, sb);
                        if (kt + SA < KT) issue_a_any(kt + SA, sa);
                    }
                }
                if (r > SYNC) load_a((r + AHEAD) % ARING, nsta, 0, r + AHEAD - ROWS);
                if (r - SYNC < FN) load_b(KK & 1, nstb, 0, r - SYNC);
                if constexpr (STEADY) {
#pragma unroll
                    for (int q = 0; q < P; q++)
                        if (q * DMA_ROWS / P == r - SYNC) issue_one(q, kt + SB, sb, kt + SA, sa);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- persistent loop over this workgroup's macro tiles
    int tile = blockIdx.x;
    int pm, pn;
    fo_unit_to_tile(tile, p.first, p.sub_m, p.sub_n, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);
    pm = __builtin_amdgcn_readfirstlane(pm);
    pn = __builtin_amdgcn_readfirstlane(pn);
    set_tile(pm, pn);
    issue_a_any(0, 0);
    issue_b_any(0, 0);
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
                for (int v = 0; v < 4; v++) acc[i][j][v] = 0.f;
        fo_mfma_fence();

        // Stage 0 of this tile is in flight.  First tile: request the rest of the
        // prologue, then wait for stage 0.  Later tiles: stage 0 was requested
        // before the previous epilogue, whose strips lived behind stage 0, so the
        // rest is requested only after the barrier; the previous tile's NST
        // stores are younger than stage 0 and need not have completed.
        if (!carried) {
            issue_rest_of_prologue();
            if (KT >= SA)
                wait_vmcnt<(SA - 1) * PA + (SB - 1) * PB>();
            else
                wait_vmcnt<0>();
            if (ktail && KT == 1) zero_tail(0, 0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            wait_vmcnt<NST>();
            if (ktail && KT == 1) zero_tail(0, 0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            issue_rest_of_prologue();
        }
#pragma unroll
        for (int j = 0; j < FN; j++) load_b(0, lb, 0, j);
#pragma unroll
        for (int i = 0; i < AHEAD; i++) load_a(i, la, 0, i);

        using dyn = std::integral_constant<int, -1>;
        using yes = std::true_type;
        using no = std::false_type;
#define FO_SLOT(n_) std::integral_constant<int, (n_)>{}
        int sa = 0, sb = 0;  // ring slots of K step kt
        int kt = 0;
        auto advance = [&]() {
            sa = sa + 1 == SA ? 0 : sa + 1;
            sb = sb + 1 == SB ? 0 : sb + 1;
            kt++;
        };
        // the first step is never a steady one: it may carry the previous tile's signal
        if (kt < KT) {
            kstep(no{}, dyn{}, dyn{}, true, kt, sa, sb);
            advance();
        }
        if (MODE != MODE_PLAIN && KT >= 2) owed = false;  // sent in the first K step
        // steady loops start at kt == 1, slots 1 and 1
        if constexpr (SA == 2 && SB == 2) {
            for (; kt + 1 + SA < KT_full; kt += 2) {
                kstep(yes{}, FO_SLOT(1), FO_SLOT(1), false, kt, 1, 1);
                kstep(yes{}, FO_SLOT(0), FO_SLOT(0), false, kt + 1, 0, 0);
            }
        } else if constexpr (SA == 3 && SB == 2) {
            for (; kt + 5 + SA < KT_full; kt += 6) {
                kstep(yes{}, FO_SLOT(1), FO_SLOT(1), false, kt, 1, 1);
                kstep(yes{}, FO_SLOT(2), FO_SLOT(0), false, kt + 1, 2, 0);
                kstep(yes{}, FO_SLOT(0), FO_SLOT(1), false, kt + 2, 0, 1);
                kstep(yes{}, FO_SLOT(1), FO_SLOT(0), false, kt + 3, 1, 0);
                kstep(yes{}, FO_SLOT(2), FO_SLOT(1), false, kt + 4, 2, 1);
                kstep(yes{}, FO_SLOT(0), FO_SLOT(0), false, kt + 5, 0, 0);
            }
        } else {
            for (; kt + SA < KT_full;) {
                kstep(yes{}, dyn{}, dyn{}, false, kt, sa, sb);
                advance();
            }
        }
        while (kt < KT) {
            kstep(no{}, dyn{}, dyn{}, false, kt, sa, sb);
            advance();
        }
#undef FO_SLOT


        fo_mfma_fence();
        // every wavefront is done reading the ring (no loads are in flight here)
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");

        // The next tile's first stage is requested before the epilogue and lands
        // while it runs.  (Scatter epilogue: after its row map entries have
        // arrived, so that their wait does not include these loads.)
        const int cur_pm = pm, cur_pn = pn;
        const int next = tile + gridDim.x;
        const bool has_next = next < ntiles;
        auto request_next = [&]() {
            if (has_next) {
                fo_unit_to_tile(next, p.first, p.sub_m, p.sub_n, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);
                pm = __builtin_amdgcn_readfirstlane(pm);
                pn = __builtin_amdgcn_readfirstlane(pn);
                set_tile(pm, pn);
                issue_a_any(0, 0);
                issue_b_any(0, 0);
            }
        };
        if (MODE != MODE_SCATTER) request_next();

        // ---- epilogue: accumulators -> 16-bit -> LDS (per-wave strip of 32 rows) -> global
        // A wavefront's WTM x WTN block lies inside one reorder tile (BM and BN
        // are multiples of 128), so the tile's slot and base address are scalars
        // and a lane adds one 32-bit offset.  The lane id is laundered through an
        // empty asm so that this addressing is recomputed per tile instead of
        // being hoisted into registers that would stay live across the K loop.
        {
            int el = lane;
            asm volatile("" : "+v"(el));
            const int erow = el & 15, ek = el >> 4;  // accumulator block: row erow, columns 4*ek .. 4*ek+3
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
            int32_t dest_row[MODE == MODE_SCATTER ? FMB * (32 / RPP) : 1];
            if (MODE == MODE_SCATTER) {
#pragma unroll
                for (int i = 0; i < FMB; i++)
#pragma unroll
                    for (int ps = 0; ps < 32 / RPP; ps++)
                        dest_row[i * (32 / RPP) + ps] = p.RE[trow + i * 32 + ps * RPP + srow];
                wait_vmcnt<0>();
                request_next();
            }
#pragma unroll
            for (int i = 0; i < FMB; i++) {  // 32 output rows = two rows of accumulator blocks
#pragma unroll
                for (int ii = 0; ii < 2; ii++) {
#pragma unroll
                    for (int j = 0; j < FN; j++) {
                        const fo_float4v a4 = acc[i * 2 + ii][j];
                        uint16_t h0 = E::from_f32(a4[0]);
                        uint16_t h1 = E::from_f32(a4[1]);
                        uint16_t h2 = E::from_f32(a4[2]);
                        uint16_t h3 = E::from_f32(a4[3]);
                        fo_u32x2 v;
                        v.x = (uint32_t)h0 | ((uint32_t)h1 << 16);
                        v.y = (uint32_t)h2 | ((uint32_t)h3 << 16);
                        *reinterpret_cast<fo_u32x2 *>(strip + (ii * 16 + erow) * PITCH + j * 16 + ek * 4) = v;
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

        if (signalling) {
            int gs[kMaxSub] = {0, 0, 0, 0};
            if (wave == 0) groups_of(rs, gs);
            if (has_next && KT >= 2) {
                // sent from inside the next tile's first K step
                owed = true;
#pragma unroll
                for (int s = 0; s < kMaxSub; s++) {
                    prev_rs[s] = rs[s];
                    prev_gs[s] = gs[s];
                }
            } else {
                // Every lane waits until its own write-through stores are
                // acknowledged, the barrier collects the workgroup, and only then
                // one lane bumps the group counter (a relaxed atomic: the tile is
                // in memory already, there is nothing left to release).  The
                // reference has no fence here (src/overlap/gemm_with_signal.h:337-351).
                __builtin_amdgcn_s_waitcnt(0);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if (wave == 0) announce(rs, gs);
            }
        }
        if (!has_next) break;
        carried = true;
        tile = next;
    }
}

// Dynamic LDS of one workgroup: the two rings (the epilogue strips reuse the
// space behind stage 0).
template <int MTM, int MTN, int BK, int SA, int SB>
constexpr int smem_bytes() {
    return (SB * (MTM + MTN) + (SA - SB) * MTM) * BK * 2;
}

}  // namespace fo_gemm_dev
