/*
 * flashoverlap.h -- C ABI of the MI355X (gfx950) FlashOverlap hot path.
 *
 * libfo_kernels.so exports exactly these symbols.  Plain pointers and sizes
 * only; every pointer named "device" must be HIP device memory on the current
 * device, every fo_stream_t is a hipStream_t (NULL = the null stream).  All
 * work is enqueued asynchronously; nothing here allocates device memory
 * except fo_overlap_create/fo_overlap_init (one stream) and the optional
 * workspace noted below.
 *
 * Return value: 0 = ok, <0 = argument error (FO_ERR_*), >0 = hipError_t.
 *
 * Each declaration cites the interface of infinigence/FlashOverlap that it
 * replaces (path:line in that tree).
 */
#ifndef FLASHOVERLAP_H
#define FLASHOVERLAP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *fo_stream_t; /* hipStream_t */

enum { FO_F16 = 0, FO_BF16 = 1 };

enum {
    FO_OK = 0,
    FO_ERR_ARG = -1,      /* null pointer / non-positive size */
    FO_ERR_SHAPE = -2,    /* M % BM, N % BN, K % 8, dim % 8 ... violated */
    FO_ERR_ALGO = -3,     /* Algo outside [0, fo_algo_count()) */
    FO_ERR_DTYPE = -4,    /* dtype not FO_F16 / FO_BF16 */
    FO_ERR_SEGMENTS = -5, /* sum(cSeg) != tile count, G <= 0, monitor with G > TN-1 */
    FO_ERR_STATE = -6,    /* fo_overlap_* called before the matching init; a launch that does not fit the device */
    FO_ERR_LIMIT = -7     /* more groups than the static scratch of the allocation-free call holds */
};

const char *fo_error_string(int code);
int fo_version(void);

/* ---- Algo index space -------------------------------------------------
 * Same 102-entry index space as the generated function-pointer tables
 * src/tiling/gemm_tiling.cuh:3-106 / signal_tiling.cuh / scatter_tiling.cuh
 * (generator tool/generate_instances.py:5-37).  info[12] =
 * {TbM,TbN,TbK,WarpM,WarpN,WarpK,InstM,InstN,InstK,Stages,Swizzle,SplitK}.
 * On gfx950 (TbM,TbN) are the reorder/signal tile BM x BN and Swizzle is the
 * raster panel height; the other fields are advisory. */
int fo_algo_count(void);
int fo_algo_info(int algo, int32_t info[12]);

/* Tile issue order of the GEMM kernels: order[s] = id (tm*TN + tn) of the
 * s-th BM x BN tile in workgroup dispatch order.  It is the analytic
 * counterpart of the hint that tune/search.py:83-157 measures in monitor
 * mode; order must hold (M/BM)*(N/BN) ints (host memory).  Where the last
 * wave of 256x256 workgroup tiles is at most half full, those tiles are
 * computed by a second launch in BM x BN tiles; the order lists them last. */
int fo_schedule_order(int algo, int M, int N, int32_t *order);

/* How the GEMM kernels cover the problem: reorder tiles per workgroup (the
 * workgroup tile may span several BM x BN tiles) and the number of workgroups.
 * One wave of the 256-CU chip completes 256 * tiles_per_workgroup tiles; the
 * reference's tuner uses sm_count - 2 tiles per wave (tune/search.py:404).
 * Both numbers describe the main launch's tiling of the whole problem. */
int fo_workgroup_tiles(int algo, int M, int N, int32_t *tiles_per_workgroup, int32_t *workgroups);
/* Reorder tiles that complete together: the workgroups the persistent GEMM
 * keeps resident on the current device times the reorder tiles per workgroup
 * (needs a GPU: the count comes from the occupancy of the compiled kernel).
 * The counterpart of sm_count - 2 in tune/search.py:404. */
int fo_gemm_wave_tiles(int dtype, int algo, int M, int N, int32_t *tiles);
/* What the main launch of a problem occupies on the device (needs a GPU; no
 * counterpart in the reference): info = {resident workgroups, vector
 * registers per lane (architectural + accumulation), LDS bytes per workgroup,
 * threads per workgroup} of the kernel with the given epilogue (0 plain,
 * 1 signal, 2 scatter).  The consumer kernels are built for one 64-register
 * wavefront per SIMD beside the GEMM's wavefronts (threads / 256 per SIMD and
 * workgroup): that holds while GEMM wavefronts per SIMD x registers stays at or
 * below 448. */
int fo_gemm_kernel_info(int dtype, int algo, int M, int N, int epilogue, int32_t info[4]);
/* The GEMM launches count on n CUs from this call on (n <= 0: on all of the
 * device's; 0 < n < 8 is FO_ERR_ARG): the persistent launches hold
 * n x workgroups-per-CU workgroups (rounded down to a multiple of 8), and
 * fo_schedule_order, fo_gemm_wave_tiles and fo_gemm_kernel_info answer for that
 * number.  For a caller that keeps CUs for other kernels, e.g. by putting the
 * consumer on a CU-masked stream and the GEMM on a stream masked to the rest.
 * Process-wide; take the schedule order (and the RA built from it) again after
 * changing it.  The reference assumes sm_count - 2 SMs for the GEMM in the same
 * places (tune/search.py:404-407, :459-464, test/test.py:330). */
int fo_gemm_set_cu_limit(int n);
/* Raster of the 256x256 launches (no counterpart in the reference, whose tile
 * order is the hardware scheduler's).  on != 0 (the default): where the tiles are
 * whole waves of the persistent launch and a wave is whole tile rows that split
 * into eight power-of-two blocks (one per XCD), wave k computes the tile rows
 * that follow those of wave k - 1, so that a consumer of whole output rows
 * (fo_overlap_gemm_allreduce_norm) can follow the GEMM wave by wave; elsewhere,
 * and with on == 0 everywhere, each XCD walks a panel of the Algo's swizzle
 * height across all columns.  Process-wide; take fo_schedule_order (and the RA
 * built from it) again after changing it. */
int fo_gemm_set_row_waves(int on);

/* ---- GEMM -------------------------------------------------------------
 * C[M,N] = A[M,K] . B[N,K]^T, 16-bit in/out, fp32 accumulate.
 * Replaces gemm_func_table[Algo](M,N,K,A,B,C,stream), src/gemm/gemm.cu:23-110,
 * typedef src/tiling/gemm_dispatcher.h:7-26. Requires M % TbM == 0,
 * N % TbN == 0 (the reference has no boundary handling either, README.md:73)
 * and K % 8 == 0 (rows are fetched in 16-byte pieces; a last K step that is not
 * full is zero-filled on chip). */
int fo_gemm(int dtype, int M, int N, int K, const void *A, const void *B, void *C, int algo,
            fo_stream_t stream);

/* GEMM + reordered tile store + per-group signal.
 * Replaces signal_func_table[Algo](M,N,K,rLDN,cSeg,A,B,C,MM,RA,if_monitor,stream),
 * src/overlap/gemm_signal.cu:15-97 (epilogue src/overlap/gemm_with_signal.h:236-256,
 * :291-361).  RA[TM*TN], cseg_dev[G], MM[>= G; monitor: (TM+1)*TN] are device
 * int32.  Tile t is stored at slot r = RA[t] of C viewed as
 * [(M*N)/(rLDN*BN), rLDN*BN]; once the tile's write-through stores have been
 * acknowledged to every wavefront of its workgroup, MM[group(r)] += 1;
 * monitor: o = MM[TN-1]++, MM[TN+r] = o.
 * G is an extra argument (the reference reads cSeg until the prefix sum passes
 * r); it lets the library validate on the host when cseg_host != NULL. */
int fo_gemm_signal(int dtype, int M, int N, int K, int rLDN, const int32_t *cseg_dev, int G,
                   const void *A, const void *B, void *C, int32_t *MM, const int32_t *RA,
                   int monitor, int algo, fo_stream_t stream);

/* As fo_gemm_signal, and row rho of the reshaped C goes to row RE[rho].
 * Replaces scatter_func_table[Algo](...,RE,...), src/overlap/gemm_scatter.cu:15-98
 * (src/overlap/gemm_with_scatter.h:229, :448-473). RE[(M*N)/(rLDN*BN)] device int32. */
int fo_gemm_scatter(int dtype, int M, int N, int K, int rLDN, const int32_t *cseg_dev, int G,
                    const void *A, const void *B, void *C, int32_t *MM, const int32_t *RA,
                    const int32_t *RE, int monitor, int algo, fo_stream_t stream);

/* ---- counting / wait kernel -------------------------------------------
 * Replaces kernel_wait_flag<<<1,1,0,stream>>>(expect, counter), src/wait.cuh:5-9:
 * spins (s_sleep between relaxed agent-scope polls) until *counter == expect,
 * then resets it to 0 with an acquiring compare-and-swap.  If the environment
 * variable FO_WAIT_MAX_POLLS is set to a positive number when the library is
 * first used, this wait, fo_wait_groups and the one inside
 * fo_wait_reduce_groups give up after that many polls -- a guard against a
 * hung GPU; unset, the wait is unbounded like the reference's.  These
 * stand-alone entry points have nowhere to report a give-up (use
 * fo_wait_bounded for that); the waits enqueued by the fo_overlap_* calls
 * report it through fo_overlap_status. */
int fo_wait(int expect, int32_t *counter, fo_stream_t stream);

/* fo_wait for `count` consecutive groups in one launch: for every g in
 * 0..count-1 (a lane per group, side by side), spin until counters[g] ==
 * expect_dev[g] (device array, e.g. cSEG_GPU + i), then reset counters[g]; the
 * kernel ends when all have been reset.  Used for groups that complete in the same wave of the
 * GEMM, where one launch per group would only add launch latency. */
int fo_wait_groups(int count, const int32_t *expect_dev, int32_t *counters, fo_stream_t stream);
/* One-lane kernel that stores value into *word.  With fo_wait(value, word, other_stream)
 * it joins two streams through memory: stream order makes everything enqueued before
 * fo_set complete (and visible) before the word changes, and the waiting stream continues
 * a few microseconds later -- an event wait across queues measured about 12 us here. */
int fo_set(int32_t *word, int value, fo_stream_t stream);
/* fo_wait that gives up after max_polls polls (0 = unbounded) and then writes 1
 * to *status (device int32, may be NULL) without touching the counter; on
 * success *status is left unchanged.  No counterpart in the reference (its
 * waiter spins forever); exists so that failure handling can be tested
 * without hanging a GPU. */
int fo_wait_bounded(int expect, int32_t *counter, int64_t max_polls, int32_t *status,
                    fo_stream_t stream);

/* ---- consumer (1-GPU stand-in for the collective) ------------------------
 * Stands in for ncclAllReduce(C+acc, C+acc, n, half, sum) at
 * src/overlap_impl.cu:256: acc[i] = round(float(acc[i]) + float(src[i])),
 * i < nelem; nelem % 8 == 0, 16-byte aligned pointers.
 * Cache policy (no effect on results): when source and accumulator together
 * exceed 192 MB the accumulator is read and written with non-temporal
 * accesses, so that it does not evict reusable data from the 256 MB
 * memory-side cache; the overlapped calls decide this from M*N instead of
 * the single range.  fo_reorder_rmsnorm / fo_rmsnorm do the same with their
 * rows (input + output above 192 MB). */
int fo_consumer_reduce(int dtype, const void *src, void *acc, int64_t nelem, fo_stream_t stream);

/* Stands in for ncclReduceScatter(C+acc, D+acc/W, n/W) at
 * src/overlap_impl.cu:312-313 with all W ranks emulated on one GPU: the group
 * src[0:nelem] holds W equal chunks; chunk q is accumulated into
 * acc + q*seg_stride (elements).  (nelem/W) % 8 == 0. */
int fo_consumer_reduce_rs(int dtype, const void *src, void *acc, int64_t nelem, int W,
                          int64_t seg_stride, fo_stream_t stream);
/* The same, and chunk `rank` of src is also copied to own[0 : nelem/W]: what
 * ncclReduceScatter(C + acc, D + acc/W, n/W, ...) leaves in D with one rank
 * present (src/overlap_impl.cu:312-313).  own == NULL: no copy. */
int fo_consumer_reduce_rs_own(int dtype, const void *src, void *acc, int64_t nelem, int W,
                              int64_t seg_stride, void *own, int rank, fo_stream_t stream);
/* The same for ngroups consecutive groups in one launch (W >= 2): group k has
 * cseg_dev[k] tiles of tile_elems elements and its own W chunks; src, acc and own
 * point at the first group's range (acc and own at offset/W).  max_group_tiles
 * (the largest cseg of the run, known on the host) sizes the grid. */
int fo_consumer_reduce_rs_groups(int dtype, const void *src, void *acc, const int32_t *cseg_dev,
                                 int ngroups, int64_t max_group_tiles, int64_t tile_elems, int W,
                                 int64_t seg_stride, void *own, int rank, fo_stream_t stream);

/* One launch that does, for every group i in order, what the host loop of
 * src/overlap_impl.cu:250-258 enqueues as 2*G launches: wait until
 * MM[i] == cseg[i], reset MM[i] to 0, then accumulate the group's contiguous
 * range of C into ACC (W == 1) or its W chunks into ACC + q*seg_stride at
 * offset acc/W (W > 1).  ACC == NULL: wait/reset only.  tile_elems = BM*BN.
 * own != NULL (needs ACC and W > 1): chunk `rank` of every group is also copied
 * to own + (group offset)/W, the reduce-scatter output with one rank present.
 * The counters are reset by the last workgroup to leave instead of per group.
 * workspace: device int32[2], zero before the first use; the kernel leaves
 * word 0 zero and sets word 1 only if a bounded poll gave up (see
 * FO_WAIT_MAX_POLLS below).  nblocks <= 0 picks a default grid.  slices = into
 * how many pieces a group's range is cut (one piece per workgroup at a time):
 * nblocks for large groups, so that the whole grid consumes the group that
 * just completed; fewer for small groups, so that different workgroups serve
 * different groups; <= 0 picks ceil(nblocks / G).  poll_gap_ns = pause between
 * one workgroup's polls of its group counter; every poll slows a GEMM running
 * beside the kernel a little, so <= 0 picks 100 ns per workgroup (about ten
 * million polls per second in total); pass less for problems that are over
 * in tens of microseconds.  C is read past the caches and the kernel contains
 * no acquire fence, so it does not disturb the L2 of a GEMM running beside it. */
int fo_wait_reduce_groups(int dtype, const void *C, void *ACC, int32_t *MM,
                          const int32_t *cseg_dev, int G, int64_t tile_elems, int W,
                          int64_t seg_stride, void *own, int rank, int32_t *workspace, int nblocks,
                          int slices, int poll_gap_ns, fo_stream_t stream);

/* ---- RMSNorm ----------------------------------------------------------
 * Replaces reorder_rmsnorm(X, RX, RW, BM, BN, rldn, RA), src/rmsnorm/rmsnorm.h:6-8,
 * src/rmsnorm/rmsnorm.cu:14-30, kernel src/rmsnorm/rmsnorm.cuh:64-117.
 * X is the tile-reordered [bs,dim] buffer, Y[bs,dim] row-major output,
 * Wt[dim].  eps is explicit (the reference hard-codes 1e-5, rmsnorm.cuh:102)
 * and so is the stream (the reference uses the legacy default stream).
 * dim % 8 == 0, BN % 8 == 0, bs % BM == 0, dim % BN == 0. */
int fo_reorder_rmsnorm(int dtype, const void *X, void *Y, const void *Wt, int bs, int dim, int BM,
                       int BN, int rldn, const int32_t *RA, float eps, fo_stream_t stream);

/* Rows [row0, row0 + nrows) of fo_reorder_rmsnorm (RA == NULL: of fo_rmsnorm): the
 * same arithmetic, src/rmsnorm/rmsnorm.cuh:64-117, for a range of output rows
 * whose tiles are complete while others are still being computed.  The kernel
 * is thin enough (registers, LDS) to run beside a GEMM that holds every CU;
 * fo_overlap_gemm_allreduce_norm enqueues it wave by wave.  bs * dim * 2 bytes
 * must stay below 4 GiB and dim <= 16384. */
int fo_reorder_rmsnorm_rows(int dtype, const void *X, void *Y, const void *Wt, int row0, int nrows, int bs,
                            int dim, int BM, int BN, int rldn, const int32_t *RA, float eps,
                            fo_stream_t stream);

/* What the kernel behind fo_reorder_rmsnorm_rows occupies (needs a GPU; no counterpart
 * in the reference): info = {vector registers per lane, LDS bytes per workgroup} of
 * the variant for rows of dim elements, with a reorder table of BN-wide tiles
 * (reorder != 0) or without, as launched beside a GEMM (beside_gemm != 0) or alone.
 * One workgroup of four wavefronts, one per SIMD: it runs beside the signalling
 * GEMM only while these registers (in eights) and fo_gemm_kernel_info's fit a SIMD's
 * 512 together, and this LDS fits beside the GEMM workgroup's in the CU's 160 KB. */
int fo_norm_rows_kernel_info(int dtype, int dim, int reorder, int BN, int rldn, int beside_gemm,
                             int32_t info[2]);

/* Replaces rmsnorm(X, RX, RW), src/rmsnorm/rmsnorm.cu:32-46, kernel rmsnorm.cuh:14-59. */
int fo_rmsnorm(int dtype, const void *X, void *Y, const void *Wt, int bs, int dim, float eps,
               fo_stream_t stream);

/* ---- host orchestration -------------------------------------------------
 * fo_overlap_t mirrors class OverlapImpl, src/overlap_impl.h:12-43. */
typedef struct fo_overlap fo_overlap_t;

int fo_overlap_create(fo_overlap_t **out);  /* OverlapImpl(), src/overlap_impl.cu:23-25 */
int fo_overlap_destroy(fo_overlap_t *h);    /* the reference never releases its streams */
/* CutlassInit(), src/overlap_impl.cu:31-33: the stream GEMMs are enqueued on. */
int fo_overlap_set_gemm_stream(fo_overlap_t *h, fo_stream_t gemm_stream);
/* OverlapInit(), src/overlap_impl.cu:139-141: creates the second (consumer)
 * stream, non-blocking, default priority. */
int fo_overlap_init(fo_overlap_t *h);
/* NcclInit(rank, world, id), src/overlap_impl.cu:50-63: records rank/world; no
 * communicator is created on one GPU (the reference also keeps comm == NULL
 * for world == 1). */
int fo_overlap_set_world(fo_overlap_t *h, int rank, int world);
/* Accumulation buffer of the stand-in consumer (no counterpart: the reference
 * reduces across ranks in place).  acc == NULL detaches it.  For W > 1 it is
 * [W, M/W, N] (seg_stride = M/W*N elements). */
int fo_overlap_set_accumulator(fo_overlap_t *h, void *acc, int64_t nelem);
/* How the per-group consumer path batches its launches (host-only, no GPU
 * needed): groups whose last tiles fall into the same stretch of wave_tiles
 * consecutive storage slots complete together and share one wait and one
 * consumer launch.  first[0..n] receives the first group of each batch and G
 * at the end (room for G + 1 entries); returns n, or a negative error.
 * wave_tiles <= 0: no batching. */
int fo_overlap_plan_batches(const int32_t *cseg_host, int G, int wave_tiles, int32_t *first);
/* The schedule of fo_overlap_gemm_allreduce_norm's normalisation (no counterpart in
 * the reference): runs[3k .. 3k+2] = {batch, first tile row, end tile row} says that
 * tile rows [first, end) of the output are normalised behind batch `batch` of
 * fo_overlap_plan_batches(cseg_host, G, wave_tiles, ...), i.e. as soon as the groups
 * holding all their tiles have been consumed.  At most four runs follow a batch that
 * is not the last (what a scattered reorder table leaves over goes behind the last
 * one).  RA_host: the reorder table [TM, TN] on the host.  Returns the number of
 * runs, FO_ERR_LIMIT if there are more than max_runs, or a negative error. */
int fo_overlap_plan_norm_rows(const int32_t *RA_host, int TM, int TN, const int32_t *cseg_host, int G,
                              int wave_tiles, int32_t *runs, int max_runs);
/* fused < 0 (default): chosen per call.  A GEMM below 6.4e10 flop (about 50 us)
 * keeps the whole call on the GEMM stream (the GEMM with its reordered store,
 * then one consumer launch: nothing that short can hide a fork and a join, and
 * the stream orders the two, so MM is not touched and stays zero; with the
 * monitor on, the signalling GEMM and one wait over all groups as elsewhere);
 * otherwise one launch when there are more than 16 groups, else per-wave
 * launches.  0: always the second stream with wait + consumer launches per
 * group (per GEMM wave) as the reference's host loop
 * (src/overlap_impl.cu:250-258); 1: always one fo_wait_reduce_groups launch
 * with the default grid; n > 1: the same with n workgroups. */
int fo_overlap_set_fused_consumer(fo_overlap_t *h, int fused);
/* The two thresholds of the automatic choice above (no counterpart in the
 * reference): GEMMs below in_stream_below_flop stay on the GEMM stream, more
 * than fused_from_groups groups get the one-launch consumer.  The defaults
 * (6.4e10, 16) were measured on one MI355X; a negative value restores one. */
int fo_overlap_set_schedule(fo_overlap_t *h, double in_stream_below_flop, int fused_from_groups);
/* Link-rate model (no counterpart in the reference, where the collective is
 * NCCL's and takes what the links give it: src/overlap_impl.cu:256, :312-313;
 * the tuner measures that rate into its bandwidth curve, tune/bandwidth.py:77-111).
 * On one GPU the consumer that stands in for the collective runs at HBM speed,
 * twenty to fifty times faster than a collective over the links, and there is
 * little for the schedule to hide.  With gigabytes_per_second > 0 every consumer
 * launch of the handle's calls (overlapped and serial ones alike) is followed, on
 * the same stream, by a one-lane kernel that holds the stream for
 * bytes of C in the launch / rate: the time the collective would spend on the links
 * at that algorithm bandwidth.  Results do not change.  The automatic choices then
 * go to per-wave launches on the second stream.  0 (default) switches it off.
 * A single stretch above one second returns FO_ERR_LIMIT from the call. */
int fo_overlap_set_link_rate(fo_overlap_t *h, double gigabytes_per_second);
/* The kernel of that model alone: holds `stream` for the given time (at most one
 * second; it reads the device's constant-rate clock, touches no memory and
 * always ends). */
int fo_pace(int64_t nanoseconds, fo_stream_t stream);
/* Bound, in polls, of every device-side wait the handle's calls enqueue
 * (group waits, the one-launch consumer's polls, fork and join): -1 (default)
 * takes FO_WAIT_MAX_POLLS from the environment, 0 waits without bound like
 * src/wait.cuh:5-9. */
int fo_overlap_set_wait_limit(fo_overlap_t *h, int64_t max_polls);
/* Failure detection (the reference's waiter spins forever on a lost signal):
 * synchronises both streams of the handle and stores into *gave_up whether
 * any bounded wait enqueued since the last query ran out of polls; the kernels
 * behind such a wait ran on incomplete data.  A non-zero answer also clears
 * the handle's flag words, so the handle can be used again once the caller
 * has zeroed MM. */
int fo_overlap_status(fo_overlap_t *h, int32_t *gave_up);
fo_stream_t fo_overlap_comm_stream(fo_overlap_t *h);

/* Gemm(A,B,C,Algo), src/overlap_impl.cu:35-48. */
int fo_overlap_gemm(fo_overlap_t *h, int dtype, int M, int N, int K, const void *A, const void *B,
                    void *C, int algo);
/* GemmAllReduceOverlap(...), src/overlap_impl.cu:214-264: signal GEMM on the
 * GEMM stream; per group {wait, consume} on the consumer stream (groups of one
 * GEMM wave share a launch, see fo_overlap_plan_batches); then the GEMM stream
 * is made to wait for the consumer stream, through memory (fo_set / fo_wait)
 * where the reference uses an event pair.  cseg_host[G] is host memory. */
int fo_overlap_gemm_allreduce(fo_overlap_t *h, int dtype, int M, int N, int K, const void *A,
                              const void *B, void *C, int32_t *MM, const int32_t *RA, int TM,
                              int TN, int rLDN, const int32_t *cseg_host,
                              const int32_t *cseg_dev, int G, int algo, int monitor);
/* fo_overlap_gemm_allreduce followed by fo_reorder_rmsnorm(C -> Y, Wt, eps) over the
 * same tiles (BM, BN of the Algo, RA, rLDN), as the reference's layers chain them
 * (example/RowParallelLinear.py:50-66 then example/RMSNorm.py:20-34, kernel
 * src/rmsnorm/rmsnorm.cuh:64-117), with the normalisation enqueued by the overlapped
 * call itself; no counterpart in the reference, where it is a separate call that
 * starts after the join.  A tile row of the output is normalised as soon as the group
 * holding its last tile has been consumed: behind each wait + consumer batch the
 * consumer stream gets the rows that batch completed (runs of consecutive tile
 * rows, at most four launches per batch; what a scattered reorder table leaves over
 * goes behind the last batch), so with a reorder table built from fo_schedule_order
 * and whole-row waves (fo_gemm_set_row_waves) only the last wave's consumer and rows
 * remain behind the GEMM.  RA_host: a host copy of RA (the call plans from it; it is
 * not kept).  Y[M,N] row-major, Wt[N]; N <= 16384, M*N*2 bytes below 4 GiB.  The GEMM
 * stream continues when Y is complete.  Results: C, MM and the accumulator exactly as
 * fo_overlap_gemm_allreduce leaves them; Y as fo_reorder_rmsnorm_rows computes it
 * (same arithmetic as fo_reorder_rmsnorm, partial sums in another order). */
int fo_overlap_gemm_allreduce_norm(fo_overlap_t *h, int dtype, int M, int N, int K, const void *A,
                                   const void *B, void *C, int32_t *MM, const int32_t *RA,
                                   const int32_t *RA_host, int TM, int TN, int rLDN,
                                   const int32_t *cseg_host, const int32_t *cseg_dev, int G, int algo,
                                   int monitor, void *Y, const void *Wt, float eps);
/* GemmReduceScatterOverlap(...), src/overlap_impl.cu:266-321.  D[M/W, N]
 * receives this rank's chunk of every group at offset acc/W (sum over the one
 * rank present); with an accumulator attached all W chunks are accumulated. */
int fo_overlap_gemm_reducescatter(fo_overlap_t *h, int dtype, int M, int N, int K, const void *A,
                                  const void *B, void *C, void *D, int32_t *MM, const int32_t *RA,
                                  const int32_t *RE, int TM, int TN, int rLDN,
                                  const int32_t *cseg_host, const int32_t *cseg_dev, int G,
                                  int algo, int monitor);
/* GemmAllReduce(A,B,C,Algo), src/overlap_impl.cu:65-81: plain GEMM then the
 * whole-C consumer on the same stream (the non-overlapped comparator). */
int fo_overlap_gemm_allreduce_serial(fo_overlap_t *h, int dtype, int M, int N, int K,
                                     const void *A, const void *B, void *C, int algo);
/* SegAllReduce(C, cSEG_CPU, SegNum), src/overlap_impl.cu:153-167: consumer over
 * SegNum consecutive segments of M*N/SegNum*cSeg[s] elements, on the GEMM
 * stream.  G = length of cseg_host (>= seg_num). */
int fo_overlap_seg_allreduce(fo_overlap_t *h, int dtype, void *C, int64_t MN,
                             const int32_t *cseg_host, int G, int seg_num);

/* ---- allocation-free call ------------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device
 * memory or create a handle: code running under a harness that forbids
 * hipMalloc, tight serving loops, code inside a stream capture.  It is
 * fo_overlap_gemm_allreduce without the handle and without MM: the group
 * counters and the flag words of fork, join and the one-launch consumer live
 * in a static device array inside the library (16 + 4096 int32 per device,
 * held until the process ends), the streams and the accumulator come as
 * arguments, and nothing is allocated, freed or created -- no hipMalloc, no
 * stream, no event.  acc may be NULL (no consumer), comm_stream == gemm_stream
 * keeps the whole call on one stream (the only form that can be captured into
 * a graph: two streams under capture return FO_ERR_STATE).  fused as in
 * fo_overlap_set_fused_consumer.  G > 4096 returns FO_ERR_LIMIT; the monitor is
 * not available (its stamps are an output that needs a caller's buffer).
 * The array is cleared by a small kernel at the start of every call.  All
 * calls on one device share it: two calls that overlap in time on one device
 * (different stream pairs, different host threads) race on the counters;
 * calls on the same stream pair are ordered by the join and do not. */
int fo_gemm_allreduce_overlap_static(int dtype, int M, int N, int K, const void *A, const void *B, void *C,
                                     void *acc, const int32_t *RA, int TM, int TN, int rLDN,
                                     const int32_t *cseg_host, const int32_t *cseg_dev, int G, int algo,
                                     int fused, fo_stream_t gemm_stream, fo_stream_t comm_stream);
/* Status of the allocation-free calls on the current device: synchronises both
 * streams, then *gave_up = 1 if a bounded device-side wait (FO_WAIT_MAX_POLLS)
 * of any such call ran out of polls since the last query (the consumer then
 * ran on incomplete tiles), else 0; reading clears the flag.  Allocates
 * nothing.  The counterpart of fo_overlap_status for calls without a handle. */
int fo_static_status(fo_stream_t gemm_stream, fo_stream_t comm_stream, int32_t *gave_up);

#ifdef __cplusplus
}
#endif
#endif /* FLASHOVERLAP_H */
