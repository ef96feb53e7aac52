// The 256x256 workgroup tile of the gfx950 MFMA GEMM (plain, signal and scatter
// epilogues; same arguments, raster and epilogue semantics as fo_gemm_kernel.h,
// whose reference citations hold here too:
// src/overlap/gemm_with_signal.h:236-256, :291-361, src/overlap/gemm_scatter.cu:15-98).
//
// Four wavefronts, one per SIMD, each computing 128x128 of the tile with
// v_mfma_f32_16x16x32_{f16,bf16}: 64 accumulator blocks = all 256 accumulation
// registers of a lane, operand fragments in about 110 architectural registers.
// One wavefront per SIMD issues its instructions strictly in order, so whatever
// is not an MFMA has to leave in an MFMA's shadow: the K step is written as 128
// MFMAs with at most two other vector-memory or LDS instructions behind each
// (a fragment fetch, or the M0 update + load of an operand block), and a burst
// of such instructions anywhere shows up as idle matrix pipe.
//
// Operands travel HBM/L2 -> LDS directly (buffer_load_dwordx4 ... lds, 1 KiB per
// wavefront instruction) into two slots of 64 KiB (BK = 64: 256 rows of A and
// 256 of B, 128 bytes each, the 16-byte chunks XOR-swizzled by the choice of the
// global chunk each lane fetches, exactly as in fo_gemm_kernel.h).  The buffer
// descriptor covers the tile's rows only, and the chunks of a last, partial K
// step that lie beyond K are requested out of its range: the hardware writes
// zeros for them, nothing outside A or B is ever addressed.
//
// A K step has sixteen rows (one A fragment x eight B fragments) and two
// meetings of the workgroup:
//   FREE (behind row 9): every wavefront has fetched its last fragment of the
//     step's slot (the A ring runs seven rows ahead; the second k-step's B
//     fragments are fetched in rows 0-3), so the slot may be refilled.  The
//     sixteen loads of the stage two steps ahead follow, two per row in rows
//     10-13, then one per row until row 5 of the next step.
//   PUB (behind row 12): the other slot's loads, requested one step earlier,
//     have landed (vmcnt) in every wavefront; rows 13-15 fetch the next step's
//     first fragments from it.
// With one meeting for both, a stage's loads would have to leave within a few
// rows (the load path of a CU delivers a stage in about half a K step, and a
// wavefront that presents loads faster than they drain stalls with its MFMAs
// behind them) or land within a few rows.  The loader runs on across tile
// boundaries (the last two steps of a tile request the next tile's first two
// stages), so only the epilogue itself separates two tiles' MFMAs.
//
// Epilogue: accumulators -> 16-bit -> LDS strip of 16 rows per wavefront (behind
// the two slots) -> 16-byte stores of contiguous output-row pieces.  A tile's
// completion signal is sent from the next tile's first PUB meeting: its wait
// covers loads requested behind the tile's stores, hence the stores (vmcnt
// retires a wavefront's vector memory instructions in issue order on
// gfx9-family parts), in every wavefront, and the meeting's barrier lies between
// that wait and the counter update.
#pragma once

#include "fo_gemm_kernel.h"

namespace fo_gemm_dev {

typedef unsigned int fo_srd_t __attribute__((ext_vector_type(4)));  // buffer descriptor

// 16 bytes per lane, global -> LDS: address = descriptor base + soff + voff (out of range: zeros),
// LDS address = lds_addr + lane * 16 (through M0; the s_nop is the wait state between an M0 write and its use).
__device__ __forceinline__ void dma_buf16(fo_srd_t srd, unsigned voff, unsigned soff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(srd), "s"(soff)
                 : "memory");
}

// The MFMAs of this kernel: accumulator in the accumulation registers, tied to the destination
// (see fo_elem::mfma for why they are assembly); `go_load` carries a direct-to-LDS load in the
// MFMA's shadow: the M0 update in front of the MFMA, which also separates it from its use, the
// load behind it.
template <typename Tag> struct fo_mfma256;
#define FO_MFMA256(TAG_, OPC_)                                                                                        \
    template <> struct fo_mfma256<TAG_> {                                                                             \
        static __device__ __forceinline__ void go(fo_u32x4 a, fo_u32x4 b, fo_float4v &c) {                            \
            asm("v_mfma_f32_16x16x32_" OPC_ " %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));                            \
        }                                                                                                             \
        template <unsigned LDS_OFF>                                                                                   \
        static __device__ __forceinline__ void go_load(fo_u32x4 a, fo_u32x4 b, fo_float4v &c, unsigned lds_base,      \
                                                       fo_srd_t srd, unsigned voff, unsigned soff) {                  \
            asm volatile("s_add_u32 m0, %4, %5\n\tv_mfma_f32_16x16x32_" OPC_                                          \
                         " %0, %1, %2, %0\n\tbuffer_load_dwordx4 %3, %6, %7 offen lds"                                \
                         : "+a"(c)                                                                                    \
                         : "v"(a), "v"(b), "v"(voff), "s"(lds_base), "n"(LDS_OFF), "s"(srd), "s"(soff)                \
                         : "memory", "scc");                                                                          \
        }                                                                                                             \
    };
FO_MFMA256(fo_f16_tag, "f16")
FO_MFMA256(fo_bf16_tag, "bf16")
#undef FO_MFMA256

// Direct-to-LDS loads per wavefront in the rows behind FREE (rows 10, 11, ... wrapping into the next step).
constexpr int kLoadRows256[] = {2, 2, 2, 2, 1, 1, 1, 1, 1, 1, 1, 1};
constexpr int kLoadSpan256 = sizeof(kLoadRows256) / sizeof(int);
constexpr int loads_in_row256(int d) { return d >= 0 && d < kLoadSpan256 ? kLoadRows256[d] : 0; }
constexpr int loads_before_row256(int d) {
    int s = 0;
    for (int e = 0; e < d && e < kLoadSpan256; e++) s += kLoadRows256[e];
    return s;
}

constexpr int kSmem256 = 2 * 65536 + 4 * 16 * (128 + 8) * 2;  // two slots + four strips of 16 padded rows

template <typename Tag, int MODE>
__global__ __launch_bounds__(256) void fo_gemm256_kernel(GemmArgs p) {
    typedef fo_elem<Tag> E;
    typedef fo_mfma256<Tag> X;
    constexpr int MT = 256, BK = 64, F = 8, ROWS = 16, AHEAD = 7, ARING = AHEAD + 1;
    constexpr int FREE = ROWS - AHEAD;  // row behind whose MFMAs the step's slot is given up
    constexpr int PUB = 12;             // row behind whose MFMAs the next step's slot is published
    constexpr unsigned SLOT_B = 65536, BPART_B = 32768, BLOCK_B = 2048, KSTEP_X = 64, CHUNK_B = 4096;
    constexpr int PITCH = 128 + 8, CPR = 16, RPP = 4;
    constexpr unsigned STRIP_B = 2 * SLOT_B;
    constexpr int NST = 32;                                      // stores per wavefront and tile
    constexpr int YOUNG = loads_before_row256(PUB - FREE);       // loads of a step already requested at its PUB meeting
    static_assert(loads_before_row256(kLoadSpan256) == 16, "a stage is sixteen loads per wavefront");
    static_assert(FREE + kLoadSpan256 - ROWS < FREE && PUB > FREE && PUB <= 13, "load rows lie between two FREE meetings");
    // YOUNG is exact: between a FREE meeting (row 9) and the PUB meeting of the same step (row 12) rows 10-12 issue
    // loads_in_row256(0..2) loads and nothing else that counts in vmcnt; a tile's stores and the loads of rows 0-5 of
    // its successor's first step are older than those.  Further vector-memory instructions in that stretch would
    // only make the PUB wait stricter.  The wait relies on vmcnt retiring loads and stores in issue order (one
    // counter for both on this part); a part with a counter of its own for stores needs a wait on that one as well.
    static_assert(YOUNG == loads_in_row256(0) + loads_in_row256(1) + loads_in_row256(2), "loads of rows 10-12");
    static_assert(NST + 16 + YOUNG < 64, "vmcnt range: a tile's stores and a stage's loads in flight together");
    static_assert(FREE + kLoadSpan256 >= ROWS, "the rest of a stage's loads leaves in the rows of the next step");

    extern __shared__ fo_u32x4 smem[];
    const unsigned smem_lds = (unsigned)(uintptr_t)FO_LDS_PTR(smem);
    typedef const __attribute__((address_space(3))) fo_u32x4 *lds16_t;

    // A consumer wavefront may share the SIMD (it fits beside this kernel's registers); this wavefront's
    // instructions go first, the consumer's take the issue cycles that are left.
    __builtin_amdgcn_s_setprio(3);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int ntiles = p.count;
    const int KT = (p.K + BK - 1) / BK;
    const bool ktail = (p.K % BK) != 0;

    // Fragment addressing as in fo_gemm_kernel.h: lane l supplies row l & 15, k-chunk l >> 4 of a 16x32 block.
    const int frow = lane & 15, fk = lane >> 4;
    const int fkey = (frow >> 1) & 7;
    const unsigned la0 = smem_lds + (unsigned)((wm * 128 + frow) * 8 + (fk ^ fkey)) * 16;
    const unsigned lb0 = smem_lds + BPART_B + (unsigned)((wn * 128 + frow) * 8 + (fk ^ fkey)) * 16;
    const unsigned wa0 = smem_lds + (unsigned)(wave * 1024);  // wave-uniform; load c of a stage: + c * CHUNK_B (lane l: + 16 l by the hardware)

    // Loader: load c < 8 of a stage brings A rows (4c + wave) * 8 + lane / 8, load c >= 8 the same rows of B;
    // LDS slot `lane` of the 1 KiB block is (row lane / 8, physical chunk lane % 8), which receives logical chunk
    // phys ^ key(row).
    const int lrow = lane >> 3;
    const int lchunk = (lane & 7) ^ (((wave * 8 + lrow) >> 1) & 7);
    const unsigned a_off = (unsigned)((wave * 8 + lrow) * p.lda * 2 + lchunk * 16);
    const bool tail_out = (KT - 1) * BK + lchunk * 8 >= p.K;  // this lane's chunk of the last K step lies beyond K
    const unsigned a_off_t = tail_out ? 0x80000000u : a_off;  // beyond every descriptor's range
    // The descriptors point at the stage's first column of the tile's first row and cover exactly the
    // tile's rows from there (the host checks that this fits 31 bits).
    const unsigned a_span = (unsigned)((255 * p.lda + p.K) * 2);
    // A and B have one leading dimension (the launcher checks it), so the lane offsets, the span and the
    // row-block offsets of the eight loads per operand serve both.
    unsigned soff_a[8];
#pragma unroll
    for (int c = 0; c < 8; c++) {
        soff_a[c] = __builtin_amdgcn_readfirstlane((unsigned)(c * 32 * p.lda * 2));
    }

    // Loader state: the stage being requested (it runs two K steps ahead of the MFMAs, across tiles).
    int ld_tile = blockIdx.x, ld_kt = 0;
    unsigned a_cur = (ktail && KT == 1) ? a_off_t : a_off;  // this stage's lane offsets, A and B alike
    fo_srd_t ra, rb;
    auto make_srd = [&](const void *base, unsigned records) {
        const uint64_t b = (uint64_t)(uintptr_t)base;
        fo_srd_t r;
        r.x = __builtin_amdgcn_readfirstlane((unsigned)b);
        r.y = __builtin_amdgcn_readfirstlane((unsigned)(b >> 32) & 0xFFFF);  // stride 0: raw buffer
        r.z = __builtin_amdgcn_readfirstlane(records);
        r.w = 0x00020000u;  // 32-bit data format, no swizzle
        return r;
    };
    auto set_loader_tile = [&]() {
        if (ld_tile < ntiles) {
            int pm_, pn_;
            fo_unit_to_tile(ld_tile, p.first, p.sub_m, p.sub_n, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm_, &pn_);
            pm_ = __builtin_amdgcn_readfirstlane(pm_);
            pn_ = __builtin_amdgcn_readfirstlane(pn_);
            ra = make_srd(p.A + (size_t)pm_ * MT * p.lda, a_span);
            rb = make_srd(p.B + (size_t)pn_ * MT * p.lda, a_span);
        } else {
            ra = make_srd(p.A, 0);  // behind the last tile: every load is out of range, nothing is fetched
            rb = make_srd(p.B, 0);
        }
    };
    auto advance_loader = [&]() {
        ld_kt++;
        if (ld_kt == KT) {
            ld_kt = 0;
            ld_tile += gridDim.x;
            set_loader_tile();
        } else {
            // the next K step of the same tile: 128 bytes further along the rows
            const uint64_t ab = ((uint64_t)ra.y << 32 | ra.x) + BK * 2, bb = ((uint64_t)rb.y << 32 | rb.x) + BK * 2;
            ra.x = __builtin_amdgcn_readfirstlane((unsigned)ab);
            ra.y = __builtin_amdgcn_readfirstlane((unsigned)(ab >> 32));
            rb.x = __builtin_amdgcn_readfirstlane((unsigned)bb);
            rb.y = __builtin_amdgcn_readfirstlane((unsigned)(bb >> 32));
            ra.z = __builtin_amdgcn_readfirstlane(ra.z >= BK * 2 ? ra.z - BK * 2 : 0);
            rb.z = __builtin_amdgcn_readfirstlane(rb.z >= BK * 2 ? rb.z - BK * 2 : 0);
        }
        if (ktail) {
            const bool t = ld_kt == KT - 1;
            a_cur = t ? a_off_t : a_off;
        }
    };
    // load c of the loader's stage into the slot at byte offset `slot` (pipeline fill)
    auto load_chunk = [&](int c, unsigned slot) {
        if (c < 8)
            dma_buf16(ra, a_cur, soff_a[c & 7], (wa0 ^ slot) + c * CHUNK_B);
        else
            dma_buf16(rb, a_cur, soff_a[c & 7], (wa0 ^ slot) + c * CHUNK_B);
    };
    // the same riding on an MFMA (K loop)
    auto mfma_load_chunk = [&](fo_u32x4 x, fo_u32x4 y, fo_float4v &cc, int c, unsigned lds_base) {
        switch (c) {
#define FO_CASE(C_)                                                                                           \
    case C_:                                                                                                  \
        X::template go_load<C_ * CHUNK_B>(x, y, cc, lds_base, C_ < 8 ? ra : rb, a_cur, soff_a[C_ & 7]);       \
        break;
            FO_CASE(0) FO_CASE(1) FO_CASE(2) FO_CASE(3) FO_CASE(4) FO_CASE(5) FO_CASE(6) FO_CASE(7)
            FO_CASE(8) FO_CASE(9) FO_CASE(10) FO_CASE(11) FO_CASE(12) FO_CASE(13) FO_CASE(14) FO_CASE(15)
#undef FO_CASE
        }
    };

    // ---- signalling state (signal and scatter epilogues), as in fo_gemm_kernel.h
    const int sub_n = MT / p.BN, nsub = (MT / p.BM) * sub_n;  // reorder tiles per macro tile
    typedef const __attribute__((address_space(4))) int32_t *cptr_t;
    const cptr_t RAc = (cptr_t)(uintptr_t)p.RA;
    constexpr int NPRE = kPrefixRegs / 64;
    int pre[NPRE];
#pragma unroll
    for (int q = 0; q < NPRE; q++) pre[q] = 0;
    const bool reg_search = p.G <= kPrefixRegs;
    const bool signalling = MODE != MODE_PLAIN && !p.quiet;
    // The group sizes are requested in front of the pipeline fill and summed behind it (a round trip to memory and
    // some two dozen dependent cross-lane steps otherwise stand between the kernel's start and its first operand
    // load).  The requests are assembly: their registers are read only behind the fill's wait for loads that were
    // requested after them, and the compiler, which knows nothing of the fill's loads, would otherwise wait for
    // every one of those as well.  Lanes beyond G ask for element 0.
    int cs_raw[NPRE];
    if (signalling && reg_search) {
#pragma unroll
        for (int q = 0; q < NPRE; q++) {
            const int32_t *src = p.cseg + (q * 64 + lane < p.G ? q * 64 + lane : 0);
            asm volatile("global_load_dword %0, %1, off" : "=v"(cs_raw[q]) : "v"(src) : "memory");
        }
    }
    auto sum_groups = [&]() {
        if (signalling && reg_search) {
            int base = 0;
#pragma unroll
            for (int q = 0; q < NPRE; q++) {
                if (q * 64 < p.G) {  // wave-uniform
                    int v = q * 64 + lane < p.G ? cs_raw[q] : 0;
#pragma unroll
                    for (int d = 1; d < 64; d <<= 1) {
                        int o = __shfl_up(v, d, 64);
                        if (lane >= d) v += o;
                    }
                    pre[q] = v + base;
                    base = __shfl(pre[q], 63, 64);
                }
            }
        }
    };
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
    // Wavefront 0 announces a macro tile's reorder tiles: lane s < nsub holds the storage slot r and the group g of
    // reorder tile s (one register each; as scalars, slots and groups of this tile and of the one whose signal is
    // still owed took twenty scalar registers through the K loop and the kernel spilled 145 of them).  Callers
    // guarantee that every wavefront's write-through stores of those tiles are acknowledged (vmcnt) and that a
    // workgroup barrier lies between that wait and this call, so the atomic itself is relaxed.
    // Reorder tiles of one group are counted with one atomic: all resident workgroups finish a tile at about the
    // same time and bump the same few counters, and atomics on one address complete one after the other, some 25 ns
    // apart (512 tiles of 256x256 in 128x128 reorder tiles, 8 groups: 7 us per launch with one atomic per tile).
    auto announce = [&](int r, int g) {
        int count = 0;      // tiles of this lane's group from this lane on
        bool first = true;  // no earlier tile of this group
#pragma unroll
        for (int q = 0; q < kMaxSub; q++) {
            const int gq = __builtin_amdgcn_readlane(g, q);
            if (q < nsub && gq == g) {
                if (q < lane) first = false;
                if (q >= lane) count++;
            }
        }
        if (lane < nsub) {
            if (first) __hip_atomic_fetch_add(p.MM + g, count, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (p.monitor) {
                int o = __hip_atomic_fetch_add(p.MM + (p.TN - 1), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(p.MM + p.TN + r, o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    };
    // Storage slots of a macro tile's reorder tiles (scalar loads).  They are requested one tile ahead (in front of
    // the pipeline fill for the first tile, in front of the previous tile's epilogue otherwise) and awaited at the
    // tile's start: the round trip to memory then costs nothing, and no scalar load is pending at the K loop's head,
    // where it would turn every wait for LDS data into a wait for everything (scalar loads return out of order).
    int rs_next[kMaxSub] = {0, 0, 0, 0};
    auto request_slots = [&](int t) {
        if (MODE != MODE_PLAIN) {
            int tm_, tn_;
            fo_unit_to_tile(t, p.first, p.sub_m, p.sub_n, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &tm_, &tn_);
            tm_ = __builtin_amdgcn_readfirstlane(tm_);
            tn_ = __builtin_amdgcn_readfirstlane(tn_);
#pragma unroll
            for (int s = 0; s < kMaxSub; s++)
                if (s < nsub) rs_next[s] = RAc[(tm_ * (MT / p.BM) + s / sub_n) * p.TN + tn_ * sub_n + s % sub_n];
        }
    };
    // The slots that request_slots brought, as the rest of the kernel uses them: this wavefront's own reorder tile as a
    // scalar, all of them in lanes 0 .. nsub-1 of one register.
    const int my_sub = __builtin_amdgcn_readfirstlane(((wm * 128) / p.BM) * sub_n + (wn * 128) / p.BN);
    int r_mine = 0, v_rs = 0;
    auto take_slots = [&]() {
        if (MODE != MODE_PLAIN) {
#pragma unroll
            for (int s = 0; s < kMaxSub; s++) {
                int rr = rs_next[s];
                asm volatile("" : "+s"(rr));  // the scalar loads complete here
                if (s == my_sub) r_mine = rr;
                v_rs = lane == s ? rr : v_rs;
            }
        }
    };
    int v_prev_r = 0, v_prev_g = 0;  // slots and groups (per lane) of the tile whose signal is still owed
    int owed = 0;                    // PUB meetings until that signal may be sent

    fo_float4v acc[F][F];
    fo_u32x4 af[ARING], bf[2][F];
    auto load_a = [&](int slot, unsigned base, int kk, int i) {
        af[slot] = *reinterpret_cast<lds16_t>((base ^ (kk * KSTEP_X)) + i * BLOCK_B);
    };
    auto load_b = [&](int buf, unsigned base, int kk, int j) {
        bf[buf][j] = *reinterpret_cast<lds16_t>((base ^ (kk * KSTEP_X)) + j * BLOCK_B);
    };

    // ---- pipeline fill: stage 0 -> slot 0, stage 1 -> slot 1; the loader then stands at stage 1
    request_slots(blockIdx.x);
    set_loader_tile();
#pragma unroll
    for (int c = 0; c < 16; c++) load_chunk(c, 0);
    advance_loader();
#pragma unroll
    for (int c = 0; c < 16; c++) load_chunk(c, SLOT_B);
    wait_vmcnt<16>();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int j = 0; j < F; j++) load_b(0, lb0, 0, j);
#pragma unroll
    for (int i = 0; i < AHEAD; i++) load_a(i, la0, 0, i);
    sum_groups();  // the group sizes arrived before stage 0 did (requested earlier, vmcnt retires in issue order)

    int tile = blockIdx.x;
    unsigned slot_b = 0;  // byte offset of the slot the next K step reads
    for (;;) {
        int pm, pn;
        fo_unit_to_tile(tile, p.first, p.sub_m, p.sub_n, p.grid_m, p.grid_n, p.panel, p.xcd_remap, &pm, &pn);
        pm = __builtin_amdgcn_readfirstlane(pm);
        pn = __builtin_amdgcn_readfirstlane(pn);
        if (tile == (int)blockIdx.x) take_slots();  // later tiles: taken inside the previous tile's epilogue
        // Scatter: the row map entries of the wavefront's 128 rows, two per lane (lane l: rows l and 64 + l), are
        // requested here and rest in two registers through the K loop; the epilogue hands them to the lanes that
        // store each row.  Requested in the epilogue they cost every tile a round trip to memory with nothing to hide it.
        int32_t re_lo = 0, re_hi = 0;
        if (MODE == MODE_SCATTER) {
            const long trow = (long)(r_mine / p.rLDN) * p.BM + (wm * 128) % p.BM;
            re_lo = p.RE[trow + lane];
            re_hi = p.RE[trow + 64 + lane];
        }
#pragma unroll
        for (int i = 0; i < F; i++)
#pragma unroll
            for (int j = 0; j < F; j++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[i][j][v] = 0.f;
        fo_mfma_fence();

        // A tile whose predecessor's signal is still owed leaves the K loop after its first step, sends the signal and
        // re-enters: that step's PUB meeting has waited for the predecessor's stores in every wavefront (part of the
        // stage's loads was requested behind them, rows 0-5, and vmcnt retires in issue order), with the meeting's
        // barrier behind the wait.  The test inside the step (one scalar compare and branch per K step, after the PUB
        // meeting) cost the large square 4 us.
        int kt = 0;
        int kt_stop = (MODE != MODE_PLAIN && owed > 0) ? 1 : KT;
        for (;;) {
        do {
            unsigned la_ = la0 ^ slot_b, lb_ = lb0 ^ slot_b;
            asm volatile("" : "+v"(la_), "+v"(lb_));
            const unsigned lan = la_ ^ SLOT_B, lbn = lb_ ^ SLOT_B;
            // load targets: this step's slot, the previous step's (wave-uniform by construction; said so for the assembly's scalar operands)
            const unsigned lds_cur = __builtin_amdgcn_readfirstlane(wa0 ^ slot_b), lds_prev = lds_cur ^ SLOT_B;
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                const int kk = r / F, i = r % F;
                // The row's LDS fetches in issue order; executes number t (none for t < 0), returns how many there are.
                //   up to FREE: the A fragment of row r + AHEAD and, in rows 0-3, the second k-step's B fragments;
                //   behind PUB: the next step's first fragments (the A rows whose ring entry has fallen free: all
                //   of them so far in row PUB + 1, then one per row; its first k-step's B fragments, four per row).
                auto fetches = [&](int t) {
                    int n = 0;
                    const int q = r + AHEAD;  // A row the ring takes in behind row r, counted from this step's row 0
                    if (q < ROWS) {
                        if (t == n) load_a(q % ARING, la_, q / F, q % F);
                        n++;
                    } else if (r > PUB) {
#pragma unroll
                        for (int qq = ROWS; qq < ROWS + ARING; qq++) {
                            if (qq <= q && (r == PUB + 1 || qq == q)) {
                                if (t == n) load_a(qq % ARING, lan, 0, qq - ROWS);
                                n++;
                            }
                        }
                    }
                    if (r < 4) {
                        if (t == n) load_b(1, lb_, 1, 2 * r);
                        if (t == n + 1) load_b(1, lb_, 1, 2 * r + 1);
                        n += 2;
                    }
                    if (r > PUB && r - PUB <= 2) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            if (t == n) load_b(0, lbn, 0, (r - PUB - 1) * 4 + j);
                            n++;
                        }
                    }
                    return n;
                };
                const int nops = fetches(-1);
                // The row's direct-to-LDS loads ride on MFMA 1 and, if there are two, MFMA 5.
                const int d = r > FREE ? r - FREE - 1 : r + ROWS - FREE - 1;  // rows since the one behind FREE
                const int dfirst = loads_before_row256(d);
#pragma unroll
                for (int j = 0; j < F; j++) {
                    int dc = -1;
#pragma unroll
                    for (int c = 0; c < 2; c++)
                        if (c < loads_in_row256(d) && j == 1 + 4 * c) dc = c;
                    if (dc >= 0)
                        mfma_load_chunk(bf[kk][j], af[r % ARING], acc[i][j], dfirst + dc, r > FREE ? lds_cur : lds_prev);
                    else
                        X::go(bf[kk][j], af[r % ARING], acc[i][j]);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < 16; t++)
                        if (t >= j * nops / F && t < (j + 1) * nops / F) fetches(t);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (r == FREE) {
                    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's fetches from the step's slot have returned
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    advance_loader();
                }
                if (r == PUB) {
                    // The stage the next step reads has landed; younger and allowed in flight: this step's YOUNG loads.
                    // In a tile's first step the wait also covers the previous tile's stores: part of the stage's
                    // loads was requested behind them (rows 0-5), and vmcnt retires in issue order.
                    wait_vmcnt<YOUNG>();
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            slot_b ^= SLOT_B;
        } while (++kt < kt_stop);
            if (MODE == MODE_PLAIN || owed == 0) break;
            owed = 0;
            if (wave == 0) announce(v_prev_r, v_prev_g);
            // Nothing scalar stays in flight behind this rare path: with a scalar load possibly pending, the K
            // loop's waits for LDS data would all have to be waits for everything.
            __builtin_amdgcn_s_waitcnt(0xC07F);
            if (kt >= KT) break;
            kt_stop = KT;
        }

        fo_mfma_fence();
        const int next = tile + gridDim.x;
        const bool has_next = next < ntiles;
        if (has_next) request_slots(next);

        int v_done = 0;  // the slots of the tile that this epilogue stores (per lane)
        // ---- epilogue.  A wavefront's 128x128 block lies inside one reorder tile (BM and BN are multiples of
        // 128), so slot and base address are scalars.  The lane id is laundered so that this addressing is
        // recomputed per tile instead of living in registers across the K loop.
        {
            int el = lane;
            asm volatile("" : "+v"(el));
            const int erow = el & 15, ek = el >> 4;  // accumulator block: row erow, columns 4*ek .. 4*ek+3
            uint16_t *strip = reinterpret_cast<uint16_t *>(reinterpret_cast<char *>(smem) + STRIP_B) + wave * (16 * PITCH);
            const int srow = el / CPR, scol = el % CPR;
            const int ldp = MODE == MODE_PLAIN ? p.N : p.rLDN * p.BN;  // leading dimension of the output view
            const int row0 = (wm * 128) % p.BM, col0 = (wn * 128) % p.BN;
            const int r = r_mine;
            const int v_cur = v_rs;  // this tile's slots: the next tile's replace them inside the loop below
            const long trow = MODE == MODE_PLAIN ? (long)pm * MT + wm * 128 : (long)(r / p.rLDN) * p.BM + row0;
            const long tcol = MODE == MODE_PLAIN ? (long)pn * MT + wn * 128 : (long)(r % p.rLDN) * p.BN + col0;
            char *cbase = reinterpret_cast<char *>(p.C) + (trow * ldp + tcol) * 2;  // wave-uniform
            const unsigned lane_off = (unsigned)(srow * ldp + scol * 8) * 2;
            const bool stream_out = p.stream_out != 0;  // wave-uniform
#pragma unroll
            for (int i = 0; i < F; i++) {  // 16 output rows = one row of accumulator blocks
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < F; j++) {
                    fo_float4v a4 = acc[i][j];
                    asm volatile("" : "+a"(a4));  // leaves the accumulation registers here, not in one sweep in front of the epilogue
                    uint16_t h0 = E::from_f32(a4[0]);
                    uint16_t h1 = E::from_f32(a4[1]);
                    uint16_t h2 = E::from_f32(a4[2]);
                    uint16_t h3 = E::from_f32(a4[3]);
                    fo_u32x2 v;
                    v.x = (uint32_t)h0 | ((uint32_t)h1 << 16);
                    v.y = (uint32_t)h2 | ((uint32_t)h3 << 16);
                    *reinterpret_cast<fo_u32x2 *>(strip + erow * PITCH + j * 16 + ek * 4) = v;
                }
                // the strip is private to this wavefront: order its LDS writes before its reads
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int ps = 0; ps < 16 / RPP; ps++) {
                    const int row = ps * RPP + srow;
                    fo_u32x4 v = *reinterpret_cast<const fo_u32x4 *>(strip + row * PITCH + scol * 8);
                    if (MODE == MODE_SCATTER) {
                        // row i * 16 + ps * RPP + srow of the block: its entry sits in that lane of re_lo / re_hi
                        const long prow = __builtin_amdgcn_ds_bpermute(((i * 16 + ps * RPP) % 64 + srow) * 4,
                                                                       i * 16 + ps * RPP < 64 ? re_lo : re_hi);
                        if (stream_out)
                            store16_write_through_nt(p.C + (size_t)prow * ldp + tcol + scol * 8, v);
                        else
                            store16_write_through(p.C + (size_t)prow * ldp + tcol + scol * 8, v);
                    } else {
                        char *sb = cbase + (size_t)(i * 16 + ps * RPP) * ldp * 2;
                        if (MODE == MODE_PLAIN) {
                            if (stream_out)
                                store16_nt(sb, lane_off, v);
                            else
                                store16(sb, lane_off, v);
                        } else {
                            if (stream_out)
                                store16_write_through_nt(sb, lane_off, v);
                            else
                                store16_write_through(sb, lane_off, v);
                        }
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xC07F);  // strip reads done before the next pass overwrites it
                __builtin_amdgcn_wave_barrier();
                // The next tile's slots, requested in front of this epilogue, have arrived with the pass's waits: they
                // leave their four scalar registers here.
                if (i == 0 && has_next) take_slots();
            }
            v_done = v_cur;
        }

        if (signalling) {
            int v_g = 0;  // lane s: group of reorder tile s
            if (wave == 0) {
#pragma unroll
                for (int s = 0; s < kMaxSub; s++) {
                    if (s < nsub) {
                        const int g = group_of(__builtin_amdgcn_readlane(v_done, s));
                        v_g = lane == s ? g : v_g;
                    }
                }
            }
            if (has_next) {
                owed = 1;  // PUB meetings until this tile's stores have been waited for in every wavefront
                v_prev_r = v_done;
                v_prev_g = v_g;
            } else {
                // Last tile: every lane waits until its own write-through stores are acknowledged, the barrier
                // collects the workgroup, then one lane bumps the counters (the reference has no fence here,
                // src/overlap/gemm_with_signal.h:337-351).
                __builtin_amdgcn_s_waitcnt(0);
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                if (wave == 0) {
                    if (owed > 0) announce(v_prev_r, v_prev_g);
                    announce(v_done, v_g);
                }
            }
        }
        if (!has_next) break;
        tile = next;
    }
    __builtin_amdgcn_s_waitcnt(0);  // nothing of this wavefront is in flight when it ends
}

}  // namespace fo_gemm_dev
