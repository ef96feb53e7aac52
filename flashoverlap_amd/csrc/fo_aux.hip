// Bandwidth-bound side kernels of the overlap path: counting/wait, the
// consumer that stands in for the collective, and (reorder+)RMSNorm.
#include <stdlib.h>

#include <type_traits>

#include "fo_common.h"

namespace {

// ------------------------------------------------------------------ wait
// Replaces kernel_wait_flag (src/wait.cuh:5-9).  One lane polls with relaxed
// agent-scope loads (an acquire per poll would invalidate the XCD's L2 under the
// running GEMM every time) and sleeps between polls; on equality an acquiring
// CAS resets the counter to zero exactly as atomicCAS(addr, that, 0) does.
__global__ void fo_wait_kernel(int expect, int32_t *counter, long max_polls, int32_t *status) {
    long polls = 0;
    for (;;) {
        int v = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (v == expect) {
            int e = expect;
            if (__hip_atomic_compare_exchange_strong(counter, &e, 0, __ATOMIC_ACQ_REL,
                                                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
                return;
        }
        if (max_polls > 0 && ++polls >= max_polls) {
            if (status) __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
        __builtin_amdgcn_s_sleep(8);
    }
}

// Sets one word: the other half of a join through memory (see fo_set below).
__global__ void fo_set_kernel(int32_t *word, int value) {
    __hip_atomic_store(word, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The same for `count` consecutive groups: up to four wavefronts, lane l takes
// groups l, l + 256, ...  (a single lane walking 256 counters one after the
// other measured 130 us on counters that were all complete already; one
// wavefront with an acquiring CAS per group 4.5 us).  The resets are relaxed and
// one acquire fence per lane follows them.  A lane whose bounded poll runs out
// sets *status (if given) and leaves; its remaining groups keep their counts.
constexpr int WAIT_GROUPS_THREADS = 256;
__global__ __launch_bounds__(WAIT_GROUPS_THREADS) void fo_wait_groups_kernel(int count, const int32_t *expect,
                                                                             int32_t *counters, long max_polls,
                                                                             int32_t *status) {
    for (int g = threadIdx.x; g < count; g += blockDim.x) {
        const int want = expect[g];
        long polls = 0;
        for (;;) {
            int v = __hip_atomic_load(counters + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (v == want) {
                int e = want;
                if (__hip_atomic_compare_exchange_strong(counters + g, &e, 0, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT))
                    break;
            }
            if (max_polls > 0 && ++polls >= max_polls) {  // give up: flag it, leave the counter as it is
                if (status) __hip_atomic_store(status, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return;
            }
            __builtin_amdgcn_s_sleep(8);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// ------------------------------------------------------------------ consumer
template <typename Tag>
__device__ __forceinline__ fo_u32x4 add8(fo_u32x4 a, fo_u32x4 b) {
    typedef fo_elem<Tag> E;
    uint32_t x[4] = {a.x, a.y, a.z, a.w}, y[4] = {b.x, b.y, b.z, b.w}, o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float lo = E::to_f32((uint16_t)(x[i] & 0xffff)) + E::to_f32((uint16_t)(y[i] & 0xffff));
        float hi = E::to_f32((uint16_t)(x[i] >> 16)) + E::to_f32((uint16_t)(y[i] >> 16));
        o[i] = (uint32_t)E::from_f32(lo) | ((uint32_t)E::from_f32(hi) << 16);
    }
    return fo_u32x4{o[0], o[1], o[2], o[3]};
}

// The consumer runs beside the GEMM, whose workgroups each need most of a CU's
// LDS and registers.  It therefore uses few, thin workgroups (256 lanes, no LDS,
// a register budget that fits next to two GEMM wavefronts per SIMD) and gets
// its bandwidth from depth instead: every lane keeps UNROLL 16-byte pieces of
// both operands in flight.
constexpr int CONSUMER_THREADS = 256;
constexpr int CONSUMER_UNROLL = 4;
constexpr int CONSUMER_MAX_BLOCKS = 256;  // a spinning grid of this size cannot occupy every CU three-deep
// __launch_bounds__(256, 8) below caps the kernels at 64 VGPRs: the signalling GEMM holds two
// wavefronts of up to 224 registers on each SIMD, which leaves 64 of the 512 for one consumer
// wavefront.

// 16-byte load that bypasses the non-coherent caches (system-scope cache
// policy).  The fused consumer reads tiles that workgroups on other XCDs wrote
// through to memory moments ago; reading them this way needs no acquire fence,
// whose L2 invalidation would throw the running GEMM's operand panels out of
// this XCD's L2.  `base` is wave-uniform, `off` a per-lane byte offset.
__device__ __forceinline__ fo_u32x4 load16_coherent(const fo_u32x4 *base, unsigned off) {
    __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, 0x7fffffff, 0x00027000);
    return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, /*sc0 | sc1*/ 17);
}

// dst[i] += src[i] for i in [lo, hi) (16-byte units), the workgroup's lanes striding together.
// RS: piece i belongs to chunk q = i / chunk16 and lands at dst + q*seg_stride16 + (i - q*chunk16).
// With `own` set, the pieces of chunk `rank` are also copied to own + (i - rank*chunk16): this
// rank's share of the group, the output of a reduce-scatter with one rank present.
// COHERENT: src is read past the caches (see load16_coherent).
// STREAM: dst is read and written with non-temporal accesses.  An accumulator that is touched
// once per step and does not fit into the 256 MB memory-side cache beside everything else
// only evicts what will be used again (the GEMM's operands, the tiles the RMSNorm reads next):
// measured inside the overlapped step, 8192x8192 outputs, -2 % (K = 8192) and -9 % (K = 3584)
// of the whole step; on a 67 MB accumulator that is read again right away it costs 2 %.
template <typename Tag, bool RS, bool COHERENT, bool STREAM>
__device__ __forceinline__ void reduce_range(const fo_u32x4 *src, fo_u32x4 *dst, long lo, long hi,
                                             long chunk16, long seg_stride16, int tid, int nthreads,
                                             fo_u32x4 *own = nullptr, int rank = 0) {
    auto where = [&](long k) -> fo_u32x4 * {
        if (!RS) return dst + k;
        const long q = k / chunk16;
        return dst + q * seg_stride16 + (k - q * chunk16);
    };
    auto keep = [&](long k, fo_u32x4 v) {
        if (RS && own) {
            const long r = k - (long)rank * chunk16;
            if (r >= 0 && r < chunk16) own[r] = v;
        }
    };
    auto fetch = [&](long first, int u) -> fo_u32x4 {  // src[first + tid + u * nthreads], first wave-uniform
        if (COHERENT) return load16_coherent(src + first, (unsigned)(tid + u * nthreads) * 16u);
        return src[first + tid + (long)u * nthreads];
    };
    constexpr int U = RS ? CONSUMER_UNROLL / 2 : CONSUMER_UNROLL;
    long first = lo;
    const long step = (long)nthreads * U;
    for (; first + step <= hi; first += step) {
        const long i = first + tid;
        fo_u32x4 a[U], b[U];
#pragma unroll
        for (int u = 0; u < U; u++) a[u] = fetch(first, u);
#pragma unroll
        for (int u = 0; u < U; u++) {
            fo_u32x4 *d = where(i + (long)u * nthreads);
            b[u] = STREAM ? __builtin_nontemporal_load(d) : *d;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            fo_u32x4 *d = where(i + (long)u * nthreads);
            const fo_u32x4 v = add8<Tag>(b[u], a[u]);
            if (STREAM)
                __builtin_nontemporal_store(v, d);
            else
                *d = v;
        }
#pragma unroll
        for (int u = 0; u < U; u++) keep(i + (long)u * nthreads, a[u]);
    }
    for (; first < hi; first += nthreads) {
        if (first + tid < hi) {
            fo_u32x4 *d = where(first + tid);
            const fo_u32x4 a = fetch(first, 0);
            const fo_u32x4 v = add8<Tag>(STREAM ? __builtin_nontemporal_load(d) : *d, a);
            if (STREAM)
                __builtin_nontemporal_store(v, d);
            else
                *d = v;
            keep(first + tid, a);
        }
    }
}

// acc[q*seg_stride + i] += src[q*chunk + i] for q < W, i < chunk (16-byte units).
template <typename Tag>
__global__ __launch_bounds__(CONSUMER_THREADS, 8) void fo_consumer_kernel(const fo_u32x4 *src, fo_u32x4 *acc,
                                                                       long chunk16, int W,
                                                                       long seg_stride16, fo_u32x4 *own,
                                                                       int rank, int stream_acc) {
    const long total = chunk16 * W;
    const long per = (total + gridDim.x - 1) / gridDim.x;
    const long lo = per * blockIdx.x;
    const long hi = lo + per < total ? lo + per : total;
    if (lo >= hi) return;
    if (W <= 1) {
        if (stream_acc)
            reduce_range<Tag, false, false, true>(src, acc, lo, hi, 0, 0, threadIdx.x, blockDim.x);
        else
            reduce_range<Tag, false, false, false>(src, acc, lo, hi, 0, 0, threadIdx.x, blockDim.x);
    } else if (stream_acc) {
        reduce_range<Tag, true, false, true>(src, acc, lo, hi, chunk16, seg_stride16, threadIdx.x, blockDim.x, own,
                                             rank);
    } else {
        reduce_range<Tag, true, false, false>(src, acc, lo, hi, chunk16, seg_stride16, threadIdx.x, blockDim.x, own,
                                              rank);
    }
}

// The same for `ngroups` consecutive groups in one launch (blockIdx.y = group):
// group k holds cseg[k] tiles of tile16 16-byte units and starts where group
// k-1 ends; each group is cut into its own W chunks.  src, acc and own point at
// the first group's range (acc and own at offset/W of it).
template <typename Tag>
__global__ __launch_bounds__(CONSUMER_THREADS, 8) void fo_consumer_groups_kernel(
    const fo_u32x4 *src, fo_u32x4 *acc, const int32_t *cseg, long tile16, int W, long seg_stride16,
    fo_u32x4 *own, int rank, int stream_acc) {
    long off = 0;
    for (int k = 0; k < (int)blockIdx.y; k++) off += cseg[k];
    off *= tile16;
    const long total = (long)cseg[blockIdx.y] * tile16;
    const long per = (total + gridDim.x - 1) / gridDim.x;
    const long lo = per * blockIdx.x;
    const long hi = lo + per < total ? lo + per : total;
    if (lo >= hi) return;
    if (stream_acc)
        reduce_range<Tag, true, false, true>(src + off, acc + off / W, lo, hi, total / W, seg_stride16, threadIdx.x,
                                             blockDim.x, own ? own + off / W : nullptr, rank);
    else
        reduce_range<Tag, true, false, false>(src + off, acc + off / W, lo, hi, total / W, seg_stride16,
                                              threadIdx.x, blockDim.x, own ? own + off / W : nullptr, rank);
}

// One launch for all groups.  The work is cut into items (group g, slice s of
// that group's contiguous range); workgroup b owns items b, b+nb, b+2nb, ...
// in ascending order.  With as many slices as workgroups every workgroup takes
// its slice of every group in turn (large groups: the whole grid works on the
// group that just completed); with fewer, different workgroups wait on
// different groups at the same time (many small groups are consumed in
// parallel).  For its item a workgroup has one lane poll MM[g] == cseg[g]
// (relaxed agent-scope loads) and then all lanes reduce the slice, reading C
// past the caches.  There is no acquire fence and no kernel boundary between
// the groups: either would invalidate the L2 under the running GEMM.
//
// A poll is not free for the GEMM running beside the pollers: measured on
// MI355X, every agent-scope poll costs the 8192^3 GEMM about a nanosecond,
// wherever the polled word lives (one shared counter or one word per
// workgroup), so 256 workgroups polling every half microsecond make it 1.7x
// slower.  The host therefore passes the pause between a lane's polls
// (sleep_ticks, in s_sleep 16 units of 1024 clocks) so that the launch as a
// whole stays near ten million polls per second.
//
// No workgroup waits for another one; the last workgroup to leave resets every
// group counter (the CAS-to-zero of src/wait.cuh:5-9, deferred to the end of the
// launch, before which nothing can signal again) and clears workspace word 0.
// Word 1 is set if a bounded poll gave up.
template <typename Tag>
__global__ __launch_bounds__(CONSUMER_THREADS, 8) void fo_wait_reduce_kernel(
    const fo_u32x4 *C, fo_u32x4 *ACC, int32_t *MM, const int32_t *cseg, int G, long tile16, int W,
    long seg_stride16, int slices, int32_t *ws, long max_polls, int sleep_ticks, fo_u32x4 *OWN, int rank,
    int stream_acc) {
    __shared__ int first_tile_s, last;
    const int nb = gridDim.x;
    const long items = (long)G * slices;
    int scanned_g = -1, scanned_first = 0;  // incremental exclusive prefix sum of cseg (items ascend)
    for (long item = blockIdx.x; item < items; item += nb) {
        const int g = (int)(item / slices), sl = (int)(item - (long)g * slices);
        const int cnt = cseg[g];
        if (threadIdx.x == 0) {
            for (int j = scanned_g < 0 ? 0 : scanned_g; j < g; j++) scanned_first += cseg[j];
            scanned_g = g;
            first_tile_s = scanned_first;
            long polls = 0;
            while (__hip_atomic_load(MM + g, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != cnt) {
                if (max_polls > 0 && ++polls >= max_polls) {  // debugging bound: flag and go on
                    __hip_atomic_store(ws + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
                for (int k = 0; k < sleep_ticks; k++) __builtin_amdgcn_s_sleep(16);
            }
        }
        __syncthreads();
        // The poll's value has returned before any lane issues a load of the
        // group's data (barrier above), and those loads do not hit in a cache.
        if (ACC) {
            const long base16 = (long)first_tile_s * tile16;
            const long n16 = (long)cnt * tile16;
            const long lo = n16 * sl / slices, hi = n16 * (sl + 1) / slices;
            fo_u32x4 *own = OWN ? OWN + base16 / W : nullptr;
            if (W <= 1) {
                if (stream_acc)
                    reduce_range<Tag, false, true, true>(C + base16, ACC + base16, lo, hi, 0, 0, threadIdx.x,
                                                         blockDim.x);
                else
                    reduce_range<Tag, false, true, false>(C + base16, ACC + base16, lo, hi, 0, 0, threadIdx.x,
                                                          blockDim.x);
            } else if (stream_acc) {
                reduce_range<Tag, true, true, true>(C + base16, ACC + base16 / W, lo, hi, n16 / W, seg_stride16,
                                                    threadIdx.x, blockDim.x, own, rank);
            } else {
                reduce_range<Tag, true, true, false>(C + base16, ACC + base16 / W, lo, hi, n16 / W, seg_stride16,
                                                     threadIdx.x, blockDim.x, own, rank);
            }
        }
        __syncthreads();  // first_tile_s is rewritten for the next item
    }
    if (threadIdx.x == 0) {
        int left = __hip_atomic_fetch_add(ws, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last = (left == nb - 1);
    }
    __syncthreads();
    if (last) {
        for (int g = threadIdx.x; g < G; g += blockDim.x)
            __hip_atomic_store(MM + g, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) __hip_atomic_store(ws, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ------------------------------------------------------------------ RMSNorm
// Per-dtype arithmetic on one 16-byte chunk (8 elements).
//   sumsq: acc + sum of squares, fp32 (v_dot2c_f32_{f16,bf16}: two elements per instruction).
//   scale: y = round16(round16(x*s) * w), the two roundings of src/rmsnorm/rmsnorm.cuh:109-113.
//          The second product is a 16-bit multiply in the reference; the exact product of two
//          16-bit values rounded once is the same number, so fp16 uses the packed 16-bit
//          multiply and bf16 (no packed arithmetic on this part) an fp32 multiply and one rounding.
template <typename Tag> struct norm_math;
template <> struct norm_math<fo_f16_tag> {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ float sumsq(fo_u32x4 v, float acc) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t u = v[k];  // a copy: the cast must see this element, not the vector's first
            const h2 p = __builtin_bit_cast(h2, u);
            acc = __builtin_amdgcn_fdot2(p, p, acc, false);
        }
        return acc;
    }
    static __device__ __forceinline__ fo_u32x4 scale(fo_u32x4 v, float s, fo_u32x4 w) {
        fo_u32x4 o;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t u = v[k], uw = w[k];
            const h2 p = __builtin_bit_cast(h2, u);
            h2 q;
            q.x = (_Float16)((float)p.x * s);
            q.y = (_Float16)((float)p.y * s);
            const h2 y = q * __builtin_bit_cast(h2, uw);
            o[k] = __builtin_bit_cast(uint32_t, y);
        }
        return o;
    }
};
template <> struct norm_math<fo_bf16_tag> {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    typedef fo_elem<fo_bf16_tag> E;
    static __device__ __forceinline__ float sumsq(fo_u32x4 v, float acc) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t u = v[k];
            const b2 p = __builtin_bit_cast(b2, u);
            acc = __builtin_amdgcn_fdot2_f32_bf16(p, p, acc, false);
        }
        return acc;
    }
    static __device__ __forceinline__ fo_u32x4 scale(fo_u32x4 v, float s, fo_u32x4 w) {
        fo_u32x4 o;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t u = v[k], uw = w[k];
            const float lo = E::to_f32(E::from_f32(E::to_f32((uint16_t)(u & 0xffff)) * s));
            const float hi = E::to_f32(E::from_f32(E::to_f32((uint16_t)(u >> 16)) * s));
            const uint16_t ylo = E::from_f32(lo * E::to_f32((uint16_t)(uw & 0xffff)));
            const uint16_t yhi = E::from_f32(hi * E::to_f32((uint16_t)(uw >> 16)));
            o[k] = (uint32_t)ylo | ((uint32_t)yhi << 16);
        }
        return o;
    }
};

// One wavefront per output row, four rows per workgroup; each lane keeps its
// 16-byte chunks of the row in registers between the sum of squares and the
// scaling, so the row is read once.  How a chunk's source address is found:
//   NORM_PLAIN    the row itself (no reorder table);
//   NORM_SLOTS    gathered from the tile-reordered buffer with rldn == 1, BN a power of
//                 two and at most 128 tiles per row (every tile of the Algo table up to
//                 16384 columns): tile r is the contiguous block of BM rows of BN columns
//                 that starts at row r * BM, the index math is shifts and masks, and the
//                 storage slots of the row's tiles are fetched once per wavefront (lane l
//                 holds the slots of tiles l and l + 64) and handed out by shuffles: a
//                 table load per chunk would put a second memory round trip in front of
//                 every load of the row;
//   NORM_GENERAL  the index math of src/rmsnorm/rmsnorm.cuh:80-86 as written (divisions,
//                 a table load per chunk, batched in front of the row's loads).
// The path is a template parameter so that the loop that requests the row holds no
// branch: all of a row's loads are in flight before the first is waited for (with the
// paths as run-time branches inside that loop every chunk waited for its own load,
// sixteen round trips per row of 8192).  Lanes beyond the row's end request the row's
// last chunk again and are masked out of the sum and the stores.
// The second launch bound caps the registers (128 up to 16 chunks per lane, 256 above) so that
// enough wavefronts stay resident to cover the memory latency.
// STREAM: rows are read and written with non-temporal accesses (matrices that do not fit
// into the memory-side cache beside the GEMM's operands: inside the overlapped step the
// 8192x8192 RMSNorm then takes 55 instead of 64 us, and the GEMM that follows it 3 % less).
enum { NORM_PLAIN = 0, NORM_SLOTS = 1, NORM_GENERAL = 2 };

template <typename Tag, int MAXCH, bool STREAM, int PATH>
__global__ __launch_bounds__(256, MAXCH <= 16 ? 4 : 2) void fo_rmsnorm_kernel(const fo_u32x4 *X, fo_u32x4 *Y, const fo_u32x4 *Wt,
                                                         int bs, int dim, int BM, int BN, int rldn,
                                                         const int32_t *RA, float eps) {
    typedef norm_math<Tag> MATH;
    // The weight goes through LDS, fetched once per workgroup ahead of the rows: a weight
    // load from memory between two stores of the output row would make its wait (vmcnt
    // retires in order) a wait for the store before it, one round trip per chunk.
    __shared__ fo_u32x4 wlds[64 * MAXCH];
    const int lane = threadIdx.x & 63;
    const int nch = dim >> 3;  // 16-byte chunks per row
    constexpr int WPT = MAXCH / 4;  // weight chunks per lane of the workgroup
    fo_u32x4 wreg[WPT];
#pragma unroll
    for (int q = 0; q < WPT; q++) {
        const int c = threadIdx.x + q * 256;
        wreg[q] = Wt[c < nch ? c : nch - 1];
    }
    const int b = blockIdx.x * 4 + (threadIdx.x >> 6);
    const bool live = b < bs;  // a workgroup's rows beyond the matrix: the wavefront only helps with the weight
    const bool full = nch == 64 * MAXCH;  // every lane owns MAXCH chunks of the row
    const int ldn = PATH == NORM_PLAIN ? 0 : dim / BN;
    const int row_b = live ? b : bs - 1;  // such a wavefront requests the last row again and discards it
    const int tile_row = PATH == NORM_PLAIN ? 0 : row_b / BM, in_row = PATH == NORM_PLAIN ? 0 : row_b % BM;
    auto chunk_of = [&](int i) {  // this lane's i-th chunk, clamped into the row
        const int c = lane + i * 64;
        return c < nch ? c : nch - 1;
    };
    auto fetch = [&](long src) -> fo_u32x4 { return STREAM ? __builtin_nontemporal_load(&X[src]) : X[src]; };

    fo_u32x4 x[MAXCH];
    if (PATH == NORM_PLAIN) {
#pragma unroll
        for (int i = 0; i < MAXCH; i++) x[i] = fetch((long)row_b * nch + chunk_of(i));
    } else if (PATH == NORM_SLOTS) {
        const int bn_shift = __builtin_ctz(BN);
        const int32_t *row = RA + (long)tile_row * ldn;
        const int slot_lo = lane < ldn ? row[lane] : 0;
        auto request = [&](auto two_regs) {
            int slot_hi = 0;
            if (decltype(two_regs)::value) slot_hi = lane + 64 < ldn ? row[lane + 64] : 0;
#pragma unroll
            for (int i = 0; i < MAXCH; i++) {
                const int j = chunk_of(i) << 3;
                const int t = j >> bn_shift;
                int r = __shfl(slot_lo, t & 63, 64);
                if (decltype(two_regs)::value) {
                    const int hi = __shfl(slot_hi, t & 63, 64);
                    r = t < 64 ? r : hi;
                }
                x[i] = fetch((((long)r * BM + in_row) << (bn_shift - 3)) + ((j & (BN - 1)) >> 3));
            }
        };
        if (ldn <= 64)
            request(std::false_type{});
        else
            request(std::true_type{});
    } else {
        const long ldp16 = ((long)rldn * BN) >> 3;
        int r[MAXCH];
#pragma unroll
        for (int i = 0; i < MAXCH; i++) r[i] = RA[tile_row * ldn + (chunk_of(i) << 3) / BN];
#pragma unroll
        for (int i = 0; i < MAXCH; i++) {
            const int j = chunk_of(i) << 3;
            const long nr = (long)(r[i] / rldn) * BM + in_row;
            const int nc = (r[i] % rldn) * BN + j % BN;
            x[i] = fetch(nr * ldp16 + (nc >> 3));
        }
    }

    // the weight chunks were requested before the row: they are in registers when the row's
    // first chunk is (in-order return)
#pragma unroll
    for (int q = 0; q < WPT; q++) wlds[threadIdx.x + q * 256] = wreg[q];

    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAXCH; i++) {
        const float with = MATH::sumsq(x[i], ss);
        ss = (full || lane + i * 64 < nch) ? with : ss;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) ss += __shfl_xor(ss, d, 64);
    const float s = rsqrtf(ss / (float)dim + eps);
    __syncthreads();  // the weight is in LDS
    if (!live) return;

    fo_u32x4 *out = Y + (long)b * nch;
    auto emit = [&](auto whole_row) {
#pragma unroll
        for (int i = 0; i < MAXCH; i++) {
            const int c = lane + i * 64;
            if (decltype(whole_row)::value || c < nch) {
                const fo_u32x4 y = MATH::scale(x[i], s, wlds[c]);
                if (STREAM)
                    __builtin_nontemporal_store(y, &out[c]);
                else
                    out[c] = y;
            }
        }
    };
    if (full)
        emit(std::true_type{});
    else
        emit(std::false_type{});
}

template <typename Tag, bool STREAM, int PATH>
int launch_rmsnorm_on(const void *X, void *Y, const void *Wt, int bs, int dim, int BM, int BN,
                      int rldn, const int32_t *RA, float eps, hipStream_t stream) {
    const int nch = dim / 8;
    dim3 grid((bs + 3) / 4), block(256);
    const fo_u32x4 *x = static_cast<const fo_u32x4 *>(X);
    fo_u32x4 *y = static_cast<fo_u32x4 *>(Y);
    const fo_u32x4 *w = static_cast<const fo_u32x4 *>(Wt);
    if (nch <= 64 * 4)
        hipLaunchKernelGGL((fo_rmsnorm_kernel<Tag, 4, STREAM, PATH>), grid, block, 0, stream, x, y, w, bs, dim, BM, BN, rldn, RA, eps);
    else if (nch <= 64 * 8)
        hipLaunchKernelGGL((fo_rmsnorm_kernel<Tag, 8, STREAM, PATH>), grid, block, 0, stream, x, y, w, bs, dim, BM, BN, rldn, RA, eps);
    else if (nch <= 64 * 16)
        hipLaunchKernelGGL((fo_rmsnorm_kernel<Tag, 16, STREAM, PATH>), grid, block, 0, stream, x, y, w, bs, dim, BM, BN, rldn, RA, eps);
    else if (nch <= 64 * 32)
        hipLaunchKernelGGL((fo_rmsnorm_kernel<Tag, 32, STREAM, PATH>), grid, block, 0, stream, x, y, w, bs, dim, BM, BN, rldn, RA, eps);
    else
        return FO_ERR_SHAPE;  // rows above 16384 elements (the reference's limit too)
    FO_LAUNCH_CHECK();
    return FO_OK;
}

template <typename Tag, bool STREAM>
int launch_rmsnorm_as(const void *X, void *Y, const void *Wt, int bs, int dim, int BM, int BN,
                      int rldn, const int32_t *RA, float eps, hipStream_t stream) {
    if (!RA) return launch_rmsnorm_on<Tag, STREAM, NORM_PLAIN>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, stream);
    if (rldn == 1 && (BN & (BN - 1)) == 0 && dim / BN <= 128)
        return launch_rmsnorm_on<Tag, STREAM, NORM_SLOTS>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, stream);
    return launch_rmsnorm_on<Tag, STREAM, NORM_GENERAL>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, stream);
}

template <typename Tag>
int launch_rmsnorm(const void *X, void *Y, const void *Wt, int bs, int dim, int BM, int BN,
                   int rldn, const int32_t *RA, float eps, hipStream_t stream) {
    // Rows of exactly 8192 elements fill the row kernel's workgroup (four wavefronts per row, four chunks per
    // lane), and there it is the faster of the two: 8192 x 8192, nothing cached, 45.5-46.7 us against 47-50
    // (fp16 and bf16, reorder or not).  Narrower rows leave its lanes idle (16384 x 1024: 15.5 against 11.8 us)
    // and longer ones cost it its look-ahead.
    if (dim == 8192 && (int64_t)bs * dim * 2 <= 0xFFFFFFFFLL)
        return fo_norm_rows_with(std::is_same<Tag, fo_bf16_tag>::value ? FO_BF16 : FO_F16, X, Y, Wt, 0, bs, bs, dim, BM,
                                 BN, rldn, RA, eps, fo_streams((int64_t)bs * dim * 4), false, 0, stream);
    // input and output together against the cache that would have to hold them
    if (fo_streams((int64_t)bs * dim * 4))
        return launch_rmsnorm_as<Tag, true>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, stream);
    return launch_rmsnorm_as<Tag, false>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, stream);
}

// The same arithmetic for a range of rows, built to run beside a GEMM that holds every CU: one
// workgroup of four wavefronts works on one row at a time (lane t of the workgroup owns chunks t,
// t + 256, ...), so a row costs a lane CH x 4 registers instead of MAXCH x 4, the weight chunks stay
// in registers for all of the workgroup's rows, and the only LDS is eight partial sums.  One such
// workgroup fits into what a 256x256 GEMM workgroup leaves of a CU (the kernel above needs 16 KiB of
// LDS and about 100 registers for rows of 8192, and would wait for the GEMM to end).  A workgroup
// takes consecutive rows; the next row's chunks are requested before the current row is reduced,
// scaled and stored.  Addresses are buffer-relative: a chunk's byte offset inside its tile row's
// stretch of the reordered matrix is computed (and its tile's storage slot fetched) only when the
// rows move on to the next tile row, the row inside the tile is a scalar offset, and the output
// row's base is a scalar too, so a row costs a lane CH loads, CH stores and no address arithmetic.
// The matrix must lie within 4 GiB (32-bit byte offsets).
// Registers: up to 96 per lane, which is what the signalling GEMM's wavefront leaves of its SIMD's
// 512 (at most 408 with the accumulators); rows above 8192 elements (CH = 8) do without the look-ahead
// and may take 128, which fits beside the plain GEMM's wavefront only.
template <typename Tag, int CH, bool STREAM, int PATH>
__global__ __launch_bounds__(256, (CH <= 4 && !(CH == 4 && std::is_same<Tag, fo_bf16_tag>::value)) ? 5 : 4) void fo_norm_rows_kernel(const fo_u32x4 *X, fo_u32x4 *Y, const fo_u32x4 *Wt,
                                                              int row0, int nrows, int rows_per_wg, int dim, int BM,
                                                              int BN, int rldn, const int32_t *RA, float eps,
                                                              unsigned x_bytes) {
    typedef norm_math<Tag> MATH;
    __shared__ float part[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nch = dim >> 3;
    const bool full = nch == 256 * CH;
    const int first = row0 + blockIdx.x * rows_per_wg;
    const int last = first + rows_per_wg < row0 + nrows ? first + rows_per_wg : row0 + nrows;
    if (first >= last) return;
    constexpr int NT = STREAM ? 2 : 0;  // cache policy bits of the buffer instructions: non-temporal
    auto chunk_of = [&](int i) {  // this lane's i-th chunk, clamped into the row
        const int c = tid + i * 256;
        return c < nch ? c : nch - 1;
    };
    fo_u32x4 w[CH];
#pragma unroll
    for (int i = 0; i < CH; i++) w[i] = Wt[chunk_of(i)];
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc((void *)X, 0, x_bytes, 0x00027000);
    const int ldn = PATH == NORM_PLAIN ? 0 : dim / BN;
    const int bn_shift = PATH == NORM_SLOTS ? __builtin_ctz(BN) : 0;
    const unsigned ldp_bytes = (unsigned)rldn * BN * 2;  // row pitch of the reordered view
    unsigned off[CH];  // byte offset of this lane's chunks in row 0 of their tiles (PLAIN: in the row)
#pragma unroll
    for (int i = 0; i < CH; i++) off[i] = (unsigned)chunk_of(i) * 16u;
    int slot_row = -1;
    auto request = [&](int b, fo_u32x4(&x)[CH]) {
        unsigned row_off;  // wave-uniform
        if (PATH == NORM_PLAIN) {
            row_off = (unsigned)b * (unsigned)dim * 2u;
        } else {
            const int tile_row = b / BM, in_row = b - tile_row * BM;
            if (tile_row != slot_row) {  // the same for every lane of the workgroup
#pragma unroll
                for (int i = 0; i < CH; i++) {
                    const int j = chunk_of(i) << 3;
                    const int r = RA[(long)tile_row * ldn + (PATH == NORM_SLOTS ? j >> bn_shift : j / BN)];
                    if (PATH == NORM_SLOTS)
                        off[i] = ((unsigned)r * BM << (bn_shift + 1)) + (unsigned)(j & (BN - 1)) * 2u;
                    else
                        off[i] = (unsigned)(r / rldn) * BM * ldp_bytes + (unsigned)((r % rldn) * BN + j % BN) * 2u;
                }
                slot_row = tile_row;
            }
            row_off = (unsigned)in_row * ldp_bytes;
        }
        row_off = __builtin_amdgcn_readfirstlane(row_off);
#pragma unroll
        for (int i = 0; i < CH; i++)
            x[i] = __builtin_bit_cast(fo_u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, off[i], row_off, NT));
    };

    // One row: reduce, meet, scale, store.
    int buf = 0;
    auto finish = [&](int b, fo_u32x4(&x)[CH]) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const float with = MATH::sumsq(x[i], ss);
            ss = (full || tid + i * 256 < nch) ? with : ss;
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) ss += __shfl_xor(ss, d, 64);
        if (lane == 0) part[buf][wave] = ss;
        __syncthreads();
        // Two sets of partial sums: a wavefront that runs ahead writes the next row's into the other
        // set, and cannot reach the row after that before every wavefront has passed the next barrier.
        const float total = (part[buf][0] + part[buf][1]) + (part[buf][2] + part[buf][3]);
        buf ^= 1;
        const float s = rsqrtf(total / (float)dim + eps);
        // The output row as a buffer of its own: scalar base, the lane's chunks at tid * 16 + i * 4096; chunks beyond
        // the row's end are out of the buffer's range and the hardware drops their stores.  The stores are
        // assembly for two reasons.  The compiler counts loads and stores in one counter and, with both kinds in
        // flight, waits for everything before it touches a loaded register: the next row would never be on its
        // way during this one.  And a 16-byte store's data registers are read for some cycles after it issues, so
        // a vector instruction that writes one of them right behind it must keep two wait states; the compiler
        // leaves them out for the buffer form with a scalar offset register, and lanes 12-63 of a stored chunk
        // then carried the next chunk's intermediate values whenever the CU was busy.
        const uint64_t yb = (uint64_t)(uintptr_t)(Y + (long)b * nch);
        fo_u32x4 yr;
        yr.x = __builtin_amdgcn_readfirstlane((unsigned)yb);
        yr.y = __builtin_amdgcn_readfirstlane((unsigned)(yb >> 32) & 0xFFFF);
        yr.z = __builtin_amdgcn_readfirstlane((unsigned)nch * 16u);
        yr.w = 0x00027000u;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const fo_u32x4 y = MATH::scale(x[i], s, w[i]);
            if (STREAM)
                asm volatile("buffer_store_dwordx4 %0, %1, %2, %3 offen nt\n\ts_nop 1"
                             :
                             : "v"(y), "v"((unsigned)tid * 16u), "s"(yr), "s"(i * 4096)
                             : "memory");
            else
                asm volatile("buffer_store_dwordx4 %0, %1, %2, %3 offen\n\ts_nop 1"
                             :
                             : "v"(y), "v"((unsigned)tid * 16u), "s"(yr), "s"(i * 4096)
                             : "memory");
        }
    };

    // Rows take turns in two register sets, so the row after the one being finished is already on its way.
    constexpr bool AHEAD = CH <= 4;
    fo_u32x4 xa[CH], xb[AHEAD ? CH : 1];
    if (!AHEAD) {
        for (int b = first; b < last; b++) {
            request(b, xa);
            finish(b, xa);
        }
        return;
    }
    // The loop body holds no branch around a request: where paths with and without a request in flight
    // meet, the compiler waits as if there were none, i.e. for everything.  The last one or two rows follow it.
    fo_u32x4(&xb_)[CH] = reinterpret_cast<fo_u32x4(&)[CH]>(xb);
    request(first, xa);
    int b = first;
    for (; b + 2 < last; b += 2) {
        request(b + 1, xb_);
        finish(b, xa);
        request(b + 2, xa);
        finish(b + 1, xb_);
    }
    if (b + 1 < last) {
        request(b + 1, xb_);
        finish(b, xa);
        finish(b + 1, xb_);
    } else {
        finish(b, xa);
    }
}

// grid <= 0: one workgroup per 2 rows, at most 4096 (8192 x 8192 fp16 alone: 45.5 us from 4096 workgroups, 47.3 from 2048).  beside_gemm: at most 256 workgroups, each asking for
// kBesideGemmLds bytes of LDS it never touches (one workgroup per CU beside the GEMM's, as for the consumer).
template <typename Tag, bool STREAM, int PATH>
int launch_norm_rows_on(const void *X, void *Y, const void *Wt, int row0, int nrows, int dim, int BM, int BN, int rldn,
                        const int32_t *RA, float eps, bool beside_gemm, int grid, unsigned x_bytes, hipStream_t stream,
                        int32_t *info) {
    const int nch = dim / 8;
    if (nrows < 1) nrows = 1;  // the query for the kernel's resources comes with no rows
    if (grid <= 0) grid = (nrows + 1) / 2;
    const int most = beside_gemm ? 256 : 4096;
    if (grid > most) grid = most;
    const int rows_per_wg = (nrows + grid - 1) / grid;
    grid = (nrows + rows_per_wg - 1) / rows_per_wg;
    const int lds = beside_gemm ? kBesideGemmLds : 0;
    const fo_u32x4 *x = static_cast<const fo_u32x4 *>(X);
    fo_u32x4 *y = static_cast<fo_u32x4 *>(Y);
    const fo_u32x4 *w = static_cast<const fo_u32x4 *>(Wt);
    // info != null: nothing is launched; info = {registers per lane, LDS bytes per workgroup} of the kernel that would run
#define FO_NORM_ROWS(CH_)                                                                                               \
    if (info) {                                                                                                         \
        hipFuncAttributes attr;                                                                                         \
        FO_HIP_CHECK(hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(&fo_norm_rows_kernel<Tag, CH_, STREAM, PATH>))); \
        info[0] = attr.numRegs;                                                                                         \
        info[1] = (int)attr.sharedSizeBytes + lds;                                                                      \
        return FO_OK;                                                                                                   \
    }                                                                                                                   \
    hipLaunchKernelGGL((fo_norm_rows_kernel<Tag, CH_, STREAM, PATH>), dim3(grid), dim3(256), lds, stream, x, y, w, row0, \
                       nrows, rows_per_wg, dim, BM, BN, rldn, RA, eps, x_bytes)
    if (nch <= 256) {
        FO_NORM_ROWS(1);
    } else if (nch <= 512) {
        FO_NORM_ROWS(2);
    } else if (nch <= 1024) {
        FO_NORM_ROWS(4);
    } else if (nch <= 2048) {
        FO_NORM_ROWS(8);
    } else {
        return FO_ERR_SHAPE;
    }
#undef FO_NORM_ROWS
    FO_LAUNCH_CHECK();
    return FO_OK;
}

template <typename Tag, bool STREAM>
int launch_norm_rows_as(const void *X, void *Y, const void *Wt, int row0, int nrows, int dim, int BM, int BN, int rldn,
                        const int32_t *RA, float eps, bool beside_gemm, int grid, unsigned x_bytes, hipStream_t stream,
                        int32_t *info) {
    if (!RA)
        return launch_norm_rows_on<Tag, STREAM, NORM_PLAIN>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm,
                                                            grid, x_bytes, stream, info);
    if (rldn == 1 && (BN & (BN - 1)) == 0)
        return launch_norm_rows_on<Tag, STREAM, NORM_SLOTS>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm,
                                                            grid, x_bytes, stream, info);
    return launch_norm_rows_on<Tag, STREAM, NORM_GENERAL>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm,
                                                          grid, x_bytes, stream, info);
}

// FO_WAIT_MAX_POLLS (environment, read once): bound for the otherwise unbounded
// waits, so that a missing signal ends in a flagged exit instead of a hung GPU.
long default_max_polls() {
    static long v = [] {
        const char *e = getenv("FO_WAIT_MAX_POLLS");
        return e ? atol(e) : 0L;
    }();
    return v;
}

int consumer_grid(long n16, bool stream_acc) {
    long blocks = (n16 + CONSUMER_THREADS * CONSUMER_UNROLL - 1) / (CONSUMER_THREADS * CONSUMER_UNROLL);
    if (blocks < 1) blocks = 1;
    // Non-temporal accumulator traffic streams best from many short workgroups (8192^2 elements:
    // 6.8 TB/s from 1024 or 2048 workgroups, 6.2 from 256, 5.5 from 128).
    if (stream_acc) return (int)(blocks > 2048 ? 2048 : blocks);
    // Cacheable ranges far beyond the last-level cache stream best from 128 workgroups, each on one
    // long contiguous piece (measured on 8192^2: 7.0 TB/s against 6.7 TB/s for 256 or more).
    if (n16 >= (4L << 20)) return 128;
    if (blocks > 2 * CONSUMER_MAX_BLOCKS) blocks = 2 * CONSUMER_MAX_BLOCKS;  // it does not spin: two per CU are fine
    return (int)blocks;
}

}  // namespace

// max_polls < 0: the bound from the environment (none when unset); 0: unbounded.
int fo_wait_with(int expect, int32_t *counter, long max_polls, int32_t *status, fo_stream_t stream) {
    if (!counter) return FO_ERR_ARG;
    hipLaunchKernelGGL(fo_wait_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), expect,
                       counter, max_polls < 0 ? default_max_polls() : max_polls, status);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

extern "C" int fo_wait(int expect, int32_t *counter, fo_stream_t stream) {
    return fo_wait_with(expect, counter, -1, nullptr, stream);
}

extern "C" int fo_set(int32_t *word, int value, fo_stream_t stream) {
    if (!word) return FO_ERR_ARG;
    hipLaunchKernelGGL(fo_set_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), word, value);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

int fo_wait_groups_with(int count, const int32_t *expect_dev, int32_t *counters, long max_polls, int32_t *status,
                        fo_stream_t stream) {
    if (count <= 0 || !expect_dev || !counters) return FO_ERR_ARG;
    hipLaunchKernelGGL(fo_wait_groups_kernel, dim3(1), dim3(count < WAIT_GROUPS_THREADS ? count : WAIT_GROUPS_THREADS), 0,
                       static_cast<hipStream_t>(stream), count, expect_dev, counters,
                       max_polls < 0 ? default_max_polls() : max_polls, status);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

extern "C" int fo_wait_groups(int count, const int32_t *expect_dev, int32_t *counters, fo_stream_t stream) {
    return fo_wait_groups_with(count, expect_dev, counters, -1, nullptr, stream);
}

extern "C" int fo_wait_bounded(int expect, int32_t *counter, int64_t max_polls, int32_t *status,
                               fo_stream_t stream) {
    if (max_polls < 0) return FO_ERR_ARG;
    return fo_wait_with(expect, counter, (long)max_polls, status, stream);
}

// Holds a stream for a stretch of time: the link time of a collective in the link-rate model of the
// overlap handle (fo_overlap_set_link_rate).  One lane reads the constant-rate clock and sleeps between
// reads; it touches no memory and always ends (the clock advances, the host caps the stretch).
namespace {
__global__ void fo_pace_kernel(long long ticks) {
    const long long t0 = wall_clock64();
    while ((long long)wall_clock64() - t0 < ticks) __builtin_amdgcn_s_sleep(32);
}
}  // namespace

int fo_pace_with(double seconds, fo_stream_t stream) {
    if (!(seconds >= 0)) return FO_ERR_ARG;
    if (seconds > kMaxPaceSeconds) return FO_ERR_LIMIT;
    static int khz[64];  // ticks of wall_clock64 per millisecond, per device
    int dev = 0;
    FO_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return FO_ERR_STATE;
    if (!khz[dev]) {
        int rate = 0;
        FO_HIP_CHECK(hipDeviceGetAttribute(&rate, hipDeviceAttributeWallClockRate, dev));
        if (rate <= 0) return FO_ERR_STATE;
        khz[dev] = rate;
    }
    const long long ticks = (long long)(seconds * 1e3 * khz[dev]);
    if (ticks <= 0) return FO_OK;
    hipLaunchKernelGGL(fo_pace_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), ticks);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

extern "C" int fo_pace(int64_t nanoseconds, fo_stream_t stream) {
    if (nanoseconds < 0) return FO_ERR_ARG;
    return fo_pace_with(nanoseconds * 1e-9, stream);
}

// Fills n words; the clearing step of callers that may be under stream capture,
// where a memset node is avoided.
namespace {
__global__ void fo_fill_kernel(int32_t *words, int n, int value, int skip) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        if (i != skip) words[i] = value;
}
}  // namespace

int fo_fill_words(int32_t *words, int n, int value, fo_stream_t stream, int skip) {
    if (!words || n <= 0) return FO_ERR_ARG;
    const int blocks = (n + 255) / 256;
    hipLaunchKernelGGL(fo_fill_kernel, dim3(blocks < 64 ? blocks : 64), dim3(256), 0, static_cast<hipStream_t>(stream),
                       words, n, value, skip);
    FO_LAUNCH_CHECK();
    return FO_OK;
}

int fo_consumer_reduce_with(int dtype, const void *src, void *acc, int64_t nelem, int W, int64_t seg_stride,
                            void *own, int rank, bool stream_acc, fo_stream_t stream, bool beside_gemm) {
    if (!src || !acc || nelem < 0 || W <= 0) return FO_ERR_ARG;
    if (own && (rank < 0 || rank >= W)) return FO_ERR_ARG;
    if (nelem == 0) return FO_OK;
    if (nelem % W || (nelem / W) % 8 || (W > 1 && seg_stride % 8)) return FO_ERR_SHAPE;
    if (((uintptr_t)src | (uintptr_t)acc | (uintptr_t)own) & 15) return FO_ERR_SHAPE;
    const long chunk16 = nelem / W / 8;
    if (own && W == 1) {  // the whole range is this rank's: a plain copy beside the reduce
        FO_HIP_CHECK(hipMemcpyAsync(own, src, (size_t)nelem * 2, hipMemcpyDeviceToDevice,
                                    static_cast<hipStream_t>(stream)));
        own = nullptr;
    }
    dim3 grid(consumer_grid(chunk16 * W, stream_acc));
    dim3 block(beside_gemm && stream_acc && W == 1 ? kBesideGemmThreads : CONSUMER_THREADS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int lds = beside_gemm ? kBesideGemmLds : 0;
    if (dtype == FO_F16)
        hipLaunchKernelGGL(fo_consumer_kernel<fo_f16_tag>, grid, block, lds, s, (const fo_u32x4 *)src,
                           (fo_u32x4 *)acc, chunk16, W, (long)(seg_stride / 8), (fo_u32x4 *)own, rank,
                           (int)stream_acc);
    else if (dtype == FO_BF16)
        hipLaunchKernelGGL(fo_consumer_kernel<fo_bf16_tag>, grid, block, lds, s, (const fo_u32x4 *)src,
                           (fo_u32x4 *)acc, chunk16, W, (long)(seg_stride / 8), (fo_u32x4 *)own, rank,
                           (int)stream_acc);
    else
        return FO_ERR_DTYPE;
    FO_LAUNCH_CHECK();
    return FO_OK;
}

// The entry points below know only their own range: source and accumulator
// together decide.  The overlapped calls, which know the whole matrix, use the
// *_with forms.
extern "C" int fo_consumer_reduce_rs_own(int dtype, const void *src, void *acc, int64_t nelem, int W,
                                         int64_t seg_stride, void *own, int rank, fo_stream_t stream) {
    return fo_consumer_reduce_with(dtype, src, acc, nelem, W, seg_stride, own, rank, fo_streams(nelem * 4), stream);
}

int fo_consumer_reduce_groups_with(int dtype, const void *src, void *acc, const int32_t *cseg_dev, int ngroups,
                                   int64_t max_group_tiles, int64_t tile_elems, int W, int64_t seg_stride,
                                   void *own, int rank, bool stream_acc, fo_stream_t stream, bool beside_gemm) {
    if (!src || !acc || !cseg_dev || ngroups <= 0 || max_group_tiles <= 0 || tile_elems <= 0 || W < 2)
        return FO_ERR_ARG;
    if (own && (rank < 0 || rank >= W)) return FO_ERR_ARG;
    if (tile_elems % (8 * W) || seg_stride % 8) return FO_ERR_SHAPE;
    if (((uintptr_t)src | (uintptr_t)acc | (uintptr_t)own) & 15) return FO_ERR_SHAPE;
    const long tile16 = tile_elems / 8;
    int per_group = consumer_grid(max_group_tiles * tile16, stream_acc);
    const int most = stream_acc ? 2048 : 2 * CONSUMER_MAX_BLOCKS;
    if ((long)per_group * ngroups > most) per_group = most / ngroups;
    if (per_group < 1) per_group = 1;
    dim3 grid(per_group, ngroups), block(CONSUMER_THREADS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int lds = beside_gemm ? kBesideGemmLds : 0;
    if (dtype == FO_F16)
        hipLaunchKernelGGL(fo_consumer_groups_kernel<fo_f16_tag>, grid, block, lds, s, (const fo_u32x4 *)src,
                           (fo_u32x4 *)acc, cseg_dev, tile16, W, (long)(seg_stride / 8), (fo_u32x4 *)own, rank,
                           (int)stream_acc);
    else if (dtype == FO_BF16)
        hipLaunchKernelGGL(fo_consumer_groups_kernel<fo_bf16_tag>, grid, block, lds, s, (const fo_u32x4 *)src,
                           (fo_u32x4 *)acc, cseg_dev, tile16, W, (long)(seg_stride / 8), (fo_u32x4 *)own, rank,
                           (int)stream_acc);
    else
        return FO_ERR_DTYPE;
    FO_LAUNCH_CHECK();
    return FO_OK;
}

extern "C" int fo_consumer_reduce_rs_groups(int dtype, const void *src, void *acc, const int32_t *cseg_dev,
                                            int ngroups, int64_t max_group_tiles, int64_t tile_elems, int W,
                                            int64_t seg_stride, void *own, int rank, fo_stream_t stream) {
    return fo_consumer_reduce_groups_with(dtype, src, acc, cseg_dev, ngroups, max_group_tiles, tile_elems, W,
                                          seg_stride, own, rank,
                                          fo_streams(max_group_tiles * tile_elems * ngroups * 4), stream);
}

extern "C" int fo_consumer_reduce_rs(int dtype, const void *src, void *acc, int64_t nelem, int W,
                                     int64_t seg_stride, fo_stream_t stream) {
    return fo_consumer_reduce_rs_own(dtype, src, acc, nelem, W, seg_stride, nullptr, 0, stream);
}

extern "C" int fo_consumer_reduce(int dtype, const void *src, void *acc, int64_t nelem,
                                  fo_stream_t stream) {
    return fo_consumer_reduce_rs(dtype, src, acc, nelem, 1, 0, stream);
}

int fo_wait_reduce_groups_with(int dtype, const void *C, void *ACC, int32_t *MM, const int32_t *cseg_dev, int G,
                               int64_t tile_elems, int W, int64_t seg_stride, void *own, int rank,
                               int32_t *workspace, int nblocks, int slices, int poll_gap_ns, bool stream_acc,
                               long max_polls, fo_stream_t stream) {
    if (max_polls < 0) max_polls = default_max_polls();
    if (!MM || !cseg_dev || !workspace || G <= 0 || tile_elems <= 0 || W <= 0) return FO_ERR_ARG;
    if (ACC && !C) return FO_ERR_ARG;
    if (own && (!ACC || W < 2 || rank < 0 || rank >= W)) return FO_ERR_ARG;
    if (tile_elems % (8 * W) || (W > 1 && seg_stride % 8)) return FO_ERR_SHAPE;
    // The grid spins until the GEMM signals, so it must never be able to crowd the
    // GEMM's workgroups out of every CU: at most one thin workgroup per CU.
    if (nblocks <= 0 || nblocks > CONSUMER_MAX_BLOCKS) nblocks = CONSUMER_MAX_BLOCKS;
    if (slices <= 0) slices = (nblocks + G - 1) / G;
    if (slices > nblocks) slices = nblocks;
    // pause between one lane's polls: at least what keeps the launch near ten
    // million polls per second (0.1 us per workgroup), in ticks of about half a microsecond
    if (poll_gap_ns <= 0) poll_gap_ns = nblocks * 100;
    int sleep_ticks = (poll_gap_ns + 499) / 500;
    if (sleep_ticks < 1) sleep_ticks = 1;
    dim3 grid(nblocks), block(CONSUMER_THREADS);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == FO_F16)
        hipLaunchKernelGGL(fo_wait_reduce_kernel<fo_f16_tag>, grid, block, 0, s, (const fo_u32x4 *)C,
                           (fo_u32x4 *)ACC, MM, cseg_dev, G, (long)(tile_elems / 8), W,
                           (long)(seg_stride / 8), slices, workspace, max_polls, sleep_ticks,
                           (fo_u32x4 *)own, rank, (int)stream_acc);
    else if (dtype == FO_BF16)
        hipLaunchKernelGGL(fo_wait_reduce_kernel<fo_bf16_tag>, grid, block, 0, s, (const fo_u32x4 *)C,
                           (fo_u32x4 *)ACC, MM, cseg_dev, G, (long)(tile_elems / 8), W,
                           (long)(seg_stride / 8), slices, workspace, max_polls, sleep_ticks,
                           (fo_u32x4 *)own, rank, (int)stream_acc);
    else
        return FO_ERR_DTYPE;
    FO_LAUNCH_CHECK();
    return FO_OK;
}

// The group sizes live on the device: without the whole matrix's size the
// accumulator is treated as cacheable.
extern "C" int fo_wait_reduce_groups(int dtype, const void *C, void *ACC, int32_t *MM,
                                     const int32_t *cseg_dev, int G, int64_t tile_elems, int W,
                                     int64_t seg_stride, void *own, int rank, int32_t *workspace,
                                     int nblocks, int slices, int poll_gap_ns, fo_stream_t stream) {
    return fo_wait_reduce_groups_with(dtype, C, ACC, MM, cseg_dev, G, tile_elems, W, seg_stride, own, rank,
                                      workspace, nblocks, slices, poll_gap_ns, false, -1, stream);
}

extern "C" int fo_reorder_rmsnorm(int dtype, const void *X, void *Y, const void *Wt, int bs, int dim,
                                  int BM, int BN, int rldn, const int32_t *RA, float eps,
                                  fo_stream_t stream) {
    if (!X || !Y || !Wt || !RA || bs <= 0 || dim <= 0 || BM <= 0 || BN <= 0 || rldn <= 0)
        return FO_ERR_ARG;
    if (dim % 8 || BN % 8 || dim % BN || bs % BM) return FO_ERR_SHAPE;
    if (((long)(bs / BM) * (dim / BN)) % rldn) return FO_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == FO_F16) return launch_rmsnorm<fo_f16_tag>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, s);
    if (dtype == FO_BF16) return launch_rmsnorm<fo_bf16_tag>(X, Y, Wt, bs, dim, BM, BN, rldn, RA, eps, s);
    return FO_ERR_DTYPE;
}

int fo_norm_rows_with(int dtype, const void *X, void *Y, const void *Wt, int row0, int nrows, int bs, int dim, int BM,
                      int BN, int rldn, const int32_t *RA, float eps, bool stream_rows, bool beside_gemm, int grid,
                      fo_stream_t stream, int32_t *info) {
    if (((!X || !Y || !Wt) && !info) || bs <= 0 || dim <= 0 || BM <= 0 || BN <= 0 || rldn <= 0) return FO_ERR_ARG;
    if (row0 < 0 || nrows < 0 || row0 + nrows > bs) return FO_ERR_ARG;
    if (dim % 8 || dim > 16384) return FO_ERR_SHAPE;
    if (RA) {
        if (BN % 8 || dim % BN || bs % BM) return FO_ERR_SHAPE;
        if (((long)(bs / BM) * (dim / BN)) % rldn) return FO_ERR_SHAPE;
    }
    if ((int64_t)bs * dim * 2 > 0xFFFFFFFFLL) return FO_ERR_SHAPE;  // 32-bit byte offsets into X
    if (nrows == 0 && !info) return FO_OK;
    const unsigned x_bytes = (unsigned)((int64_t)bs * dim * 2);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == FO_F16)
        return stream_rows ? launch_norm_rows_as<fo_f16_tag, true>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm, grid, x_bytes, s, info)
                           : launch_norm_rows_as<fo_f16_tag, false>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm, grid, x_bytes, s, info);
    if (dtype == FO_BF16)
        return stream_rows ? launch_norm_rows_as<fo_bf16_tag, true>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm, grid, x_bytes, s, info)
                           : launch_norm_rows_as<fo_bf16_tag, false>(X, Y, Wt, row0, nrows, dim, BM, BN, rldn, RA, eps, beside_gemm, grid, x_bytes, s, info);
    return FO_ERR_DTYPE;
}

extern "C" int fo_norm_rows_kernel_info(int dtype, int dim, int reorder, int BN, int rldn, int beside_gemm,
                                        int32_t info[2]) {
    if (!info || dim <= 0 || dim % 8 || dim > 16384) return FO_ERR_ARG;
    static const int32_t one = 0;
    return fo_norm_rows_with(dtype, nullptr, nullptr, nullptr, 0, 0, reorder ? BN : 1, dim, reorder ? BN : 1,
                             reorder ? BN : 8, reorder ? rldn : 1, reorder ? &one : nullptr, 0.f, true, beside_gemm != 0, 0,
                             nullptr, info);
}

extern "C" int fo_reorder_rmsnorm_rows(int dtype, const void *X, void *Y, const void *Wt, int row0, int nrows, int bs,
                                       int dim, int BM, int BN, int rldn, const int32_t *RA, float eps,
                                       fo_stream_t stream) {
    return fo_norm_rows_with(dtype, X, Y, Wt, row0, nrows, bs, dim, BM, BN, rldn, RA, eps, fo_streams((int64_t)bs * dim * 4),
                             false, 0, stream);
}

extern "C" int fo_rmsnorm(int dtype, const void *X, void *Y, const void *Wt, int bs, int dim,
                          float eps, fo_stream_t stream) {
    if (!X || !Y || !Wt || bs <= 0 || dim <= 0) return FO_ERR_ARG;
    if (dim % 8) return FO_ERR_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == FO_F16) return launch_rmsnorm<fo_f16_tag>(X, Y, Wt, bs, dim, 1, 8, 1, nullptr, eps, s);
    if (dtype == FO_BF16) return launch_rmsnorm<fo_bf16_tag>(X, Y, Wt, bs, dim, 1, 8, 1, nullptr, eps, s);
    return FO_ERR_DTYPE;
}
