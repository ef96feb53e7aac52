// Host orchestration of the overlap path: the counterpart of class OverlapImpl
// (src/overlap_impl.h:12-43, src/overlap_impl.cu) behind a C handle.  Two HIP
// streams; every call only enqueues work and returns.  May be captured into a HIP graph.
#include <mutex>
#include <new>
#include <vector>

#include "fo_common.h"

namespace {

// Words of the workspace (device int32[kWorkspaceWords], zero between calls).
enum {
    kWsLeft = 0,    // workgroups of the one-launch consumer that have left
    kWsGaveUp = 1,  // set by any bounded wait of a call that ran out of polls
    kWsJoin = 4,    // consumer stream -> GEMM stream
    kWsFork = 5,    // GEMM stream -> consumer stream
    kWorkspaceWords = 16,
};

// Defaults of the scheduling choices below; a handle can override them
// (fo_overlap_set_schedule), they are measurements on one MI355X, not laws.
//
// Two launches per group cost a few microseconds each; beyond kFusedFromGroups
// groups the single wait+reduce launch is the faster consumer.  With few, large
// groups the per-group launches win: a kernel that starts when its group is
// complete needs no polling workgroups resident beside the GEMM.
//
// In automatic mode a GEMM shorter than kInStreamBelowFlop (about 50 us of this
// GPU) keeps the whole call on the GEMM stream: the GEMM with its reordered
// store and one consumer launch (with the monitor on: the signalling GEMM and
// one wait that resets every counter between them).  Fork, join and pollers beside the
// GEMM cost more than such a GEMM can hide (4096x4096x512 with 256 groups:
// 71 us overlapped, 48 us in stream).
//
// kGemmFlopPerNs: what a GEMM is expected to sustain, for sizing the pause
// between polls only.
constexpr int kFusedFromGroups = 16;
constexpr double kInStreamBelowFlop = 6.4e10;
constexpr double kGemmFlopPerNs = 1.2e6;

}  // namespace

struct fo_overlap {
    hipStream_t gemm_stream = nullptr;
    hipStream_t comm_stream = nullptr;  // null: every call stays on the GEMM stream
    hipEvent_t forked = nullptr, joined = nullptr;  // used only while the GEMM stream is being captured
    int32_t *workspace = nullptr;
    bool gemm_ready = false;
    bool overlap_ready = false;
    int rank = 0, world = 1;
    void *acc = nullptr;
    int64_t acc_nelem = 0;
    int fused = -1;        // -1: choose per call (one launch when there are many groups)
    long max_polls = -1;   // bound of every device-side wait; -1: FO_WAIT_MAX_POLLS, 0: none
    int fused_from_groups = kFusedFromGroups;
    double in_stream_below_flop = kInStreamBelowFlop;
    int token = 1;         // value the fork and join words carry from one stream to the other
    bool always_fork = false;  // the consumer stream must not start before this call's first kernel on the GEMM stream
    // Link-rate model (fo_overlap_set_link_rate): bytes per second a collective over the group's bytes would
    // sustain; 0: none.  With a rate every consumer launch is followed on its stream by a kernel that holds the
    // stream for the bytes' link time, so that the schedule can be timed against a link-bound collective on
    // one GPU.
    double link_bytes_per_s = 0;
};

namespace {

// With a link rate the automatic choices go to per-wave launches on the second stream: the link time
// follows each consumer launch, and it is what the second stream is there to hide.
bool in_stream(const fo_overlap *h, int M, int N, int K) {
    if (!h->comm_stream) return true;
    return h->fused < 0 && h->link_bytes_per_s <= 0 && 2.0 * M * N * K < h->in_stream_below_flop;
}

int fused_grid(const fo_overlap *h, int G) {  // 0: per-group launches, otherwise workgroups of the one launch
    if (h->fused < 0) return G > h->fused_from_groups && h->link_bytes_per_s <= 0 ? 256 : 0;
    if (h->fused == 1) return 256;
    return h->fused;
}

// Pause between a workgroup's polls in the one-launch consumer: 100 ns per
// workgroup keeps the GEMM's slowdown near one percent, but no more than about
// a sixtieth of the GEMM's expected duration, so that a short problem is not
// left waiting for a sleeping poller.
int fused_poll_gap_ns(int M, int N, int K, int grid) {
    const double gemm_ns = 2.0 * M * N * K / kGemmFlopPerNs;
    double gap = grid * 100.0;
    if (gap > gemm_ns / 60) gap = gemm_ns / 60;
    if (gap < 500) gap = 500;
    return (int)gap;
}

// Pieces per group for the one-launch consumer: about 32 KiB each, at most one per workgroup.
int fused_slices(int64_t total_elems, int G, int grid) {
    const int64_t per_group = total_elems / G;
    int64_t s = per_group / 16384;
    if (s < 1) s = 1;
    if (s > grid) s = grid;
    return (int)s;
}

// Groups [i, j) that complete in the same wave of the persistent GEMM (their last
// tiles fall into the same stretch of `wave` consecutive storage slots, which
// is the order the hint assigns) are waited for by one launch: they become
// ready within microseconds of each other, and a launch per group would only
// add its latency to the tail.  done = tiles of the groups before i.
int batch_end(const int32_t *cseg_host, int G, int i, long done, int wave) {
    if (wave <= 0) return i + 1;
    const long w = (done + cseg_host[i] - 1) / wave;
    int j = i + 1;
    long d = done + cseg_host[i];
    while (j < G && (d + cseg_host[j] - 1) / wave == w) d += cseg_host[j++];
    return j;
}

// Link time of `bytes` on `stream` (nothing without a rate).
int link_time(const fo_overlap *h, int64_t bytes, fo_stream_t stream) {
    if (h->link_bytes_per_s <= 0 || bytes <= 0) return FO_OK;
    return fo_pace_with((double)bytes / h->link_bytes_per_s, stream);
}

// Asked before a call enqueues anything: the largest stretch it could ask for (all of C) must be one that
// fo_pace_with accepts, so that a refusal cannot come between the fork and the join.
int link_fits(const fo_overlap *h, int64_t bytes) {
    if (h->link_bytes_per_s <= 0) return FO_OK;
    return (double)bytes / h->link_bytes_per_s > kMaxPaceSeconds ? FO_ERR_LIMIT : FO_OK;
}

int check_segments(const int32_t *cseg_host, int G, long tiles) {
    if (!cseg_host || G <= 0) return FO_ERR_SEGMENTS;
    long sum = 0;
    for (int i = 0; i < G; i++) {
        if (cseg_host[i] <= 0) return FO_ERR_SEGMENTS;
        sum += cseg_host[i];
    }
    return sum == tiles ? FO_OK : FO_ERR_SEGMENTS;
}

// While the GEMM stream is being captured into a HIP graph the two streams are tied
// together with events, as in the reference (src/overlap_impl.cu:246, :260-263): the
// event wait pulls the consumer stream into the capture, and in the graph the dependency
// is an edge, not a wait at run time.
bool capturing(const fo_overlap *h) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(h->gemm_stream, &st) != hipSuccess) return false;
    return st == hipStreamCaptureStatusActive;
}

// GEMM stream -> consumer stream, right before the GEMM is enqueued.  Outside a capture it
// goes through memory (a one-lane set on the GEMM stream, a one-lane wait on the other) and
// only the one-launch consumer needs it: its workgroups poll from the moment they start,
// and polls slow down whatever shares the memory system with them, so they must not start
// while the GEMM stream is still busy with the work that precedes the GEMM (the
// reference's wait kernels may start early: a single sleeping lane disturbs nobody).
int fork(fo_overlap *h, bool captured, bool polling_consumer) {
    if (captured) {
        if (!h->forked || !h->joined) return FO_ERR_STATE;  // a handle-free call has no events to capture with
        FO_HIP_CHECK(hipEventRecord(h->forked, h->gemm_stream));
        FO_HIP_CHECK(hipStreamWaitEvent(h->comm_stream, h->forked, 0));
        return FO_OK;
    }
    if (!polling_consumer && !h->always_fork) return FO_OK;
    int rc = fo_set(h->workspace + kWsFork, h->token, h->gemm_stream);
    if (rc) return rc;
    return fo_wait_with(h->token, h->workspace + kWsFork, h->max_polls, h->workspace + kWsGaveUp, h->comm_stream);
}

// consumer stream -> GEMM stream.  The reference records an event on the consumer stream
// and makes the GEMM stream wait for it (src/overlap_impl.cu:260-263); an event wait across
// queues measured about 12 us here, so outside a capture the join goes through memory: a
// one-lane kernel at the end of the consumer stream sets the workspace's join word (stream order
// makes all earlier work there complete and visible first), a one-lane wait behind the
// GEMM on the GEMM's stream consumes it.  The wait cannot start before the GEMM has ended
// and everything it waits for was enqueued before it; the GEMM stream continues about 4 us
// after the consumer's end.
int join(fo_overlap *h, bool captured) {
    if (captured) {
        FO_HIP_CHECK(hipEventRecord(h->joined, h->comm_stream));
        FO_HIP_CHECK(hipStreamWaitEvent(h->gemm_stream, h->joined, 0));
        return FO_OK;
    }
    int rc = fo_set(h->workspace + kWsJoin, h->token, h->comm_stream);
    if (rc) return rc;
    return fo_wait_with(h->token, h->workspace + kWsJoin, h->max_polls, h->workspace + kWsGaveUp, h->gemm_stream);
}

}  // namespace

extern "C" int fo_overlap_plan_batches(const int32_t *cseg_host, int G, int wave_tiles, int32_t *first) {
    if (!cseg_host || !first || G <= 0) return FO_ERR_ARG;
    for (int i = 0; i < G; i++)
        if (cseg_host[i] <= 0) return FO_ERR_SEGMENTS;
    int n = 0;
    long done = 0;
    for (int i = 0; i < G;) {
        const int j = batch_end(cseg_host, G, i, done, wave_tiles);
        first[n++] = i;
        for (int g = i; g < j; g++) done += cseg_host[g];
        i = j;
    }
    first[n] = G;
    return n;
}

extern "C" int fo_overlap_create(fo_overlap_t **out) {
    if (!out) return FO_ERR_ARG;
    *out = new (std::nothrow) fo_overlap();
    return *out ? FO_OK : FO_ERR_ARG;
}

extern "C" int fo_overlap_destroy(fo_overlap_t *h) {
    if (!h) return FO_ERR_ARG;
    // release everything even if one step fails; report the first failure
    hipError_t first = hipSuccess;
    auto note = [&](hipError_t e) {
        if (first == hipSuccess) first = e;
    };
    if (h->comm_stream) {
        note(hipStreamSynchronize(h->comm_stream));
        note(hipStreamDestroy(h->comm_stream));
    }
    if (h->forked) note(hipEventDestroy(h->forked));
    if (h->joined) note(hipEventDestroy(h->joined));
    if (h->workspace) note(hipFree(h->workspace));
    delete h;
    return (int)first;
}

extern "C" int fo_overlap_set_gemm_stream(fo_overlap_t *h, fo_stream_t gemm_stream) {
    if (!h) return FO_ERR_ARG;
    h->gemm_stream = static_cast<hipStream_t>(gemm_stream);
    h->gemm_ready = true;
    return FO_OK;
}

extern "C" int fo_overlap_init(fo_overlap_t *h) {
    if (!h) return FO_ERR_ARG;
    if (h->overlap_ready) return FO_OK;
    // Default priority on purpose (the reference asks for priority -5,
    // src/overlap_impl.cu:140): mixed-priority streams are avoided on this platform.
    FO_HIP_CHECK(hipStreamCreateWithFlags(&h->comm_stream, hipStreamNonBlocking));
    FO_HIP_CHECK(hipEventCreateWithFlags(&h->forked, hipEventDisableTiming));
    FO_HIP_CHECK(hipEventCreateWithFlags(&h->joined, hipEventDisableTiming));
    FO_HIP_CHECK(hipMalloc(&h->workspace, kWorkspaceWords * sizeof(int32_t)));
    FO_HIP_CHECK(hipMemset(h->workspace, 0, kWorkspaceWords * sizeof(int32_t)));
    h->overlap_ready = true;
    return FO_OK;
}

extern "C" int fo_overlap_set_world(fo_overlap_t *h, int rank, int world) {
    if (!h || world <= 0 || rank < 0 || rank >= world) return FO_ERR_ARG;
    h->rank = rank;
    h->world = world;
    return FO_OK;
}

extern "C" int fo_overlap_set_accumulator(fo_overlap_t *h, void *acc, int64_t nelem) {
    if (!h || nelem < 0) return FO_ERR_ARG;
    h->acc = acc;
    h->acc_nelem = acc ? nelem : 0;
    return FO_OK;
}

extern "C" int fo_overlap_set_fused_consumer(fo_overlap_t *h, int fused) {
    if (!h) return FO_ERR_ARG;
    h->fused = fused < 0 ? -1 : fused;
    return FO_OK;
}

extern "C" int fo_overlap_set_wait_limit(fo_overlap_t *h, int64_t max_polls) {
    if (!h || max_polls < -1) return FO_ERR_ARG;
    h->max_polls = (long)max_polls;
    return FO_OK;
}

extern "C" int fo_overlap_set_schedule(fo_overlap_t *h, double in_stream_below_flop, int fused_from_groups) {
    if (!h) return FO_ERR_ARG;
    h->in_stream_below_flop = in_stream_below_flop < 0 ? kInStreamBelowFlop : in_stream_below_flop;
    h->fused_from_groups = fused_from_groups < 0 ? kFusedFromGroups : fused_from_groups;
    return FO_OK;
}

extern "C" int fo_overlap_set_link_rate(fo_overlap_t *h, double gigabytes_per_second) {
    if (!h || !(gigabytes_per_second >= 0)) return FO_ERR_ARG;
    h->link_bytes_per_s = gigabytes_per_second * 1e9;
    return FO_OK;
}

extern "C" int fo_overlap_status(fo_overlap_t *h, int32_t *gave_up) {
    if (!h || !gave_up) return FO_ERR_ARG;
    *gave_up = 0;
    if (!h->overlap_ready) return FO_OK;
    FO_HIP_CHECK(hipStreamSynchronize(h->comm_stream));
    if (h->gemm_ready) FO_HIP_CHECK(hipStreamSynchronize(h->gemm_stream));
    FO_HIP_CHECK(hipMemcpy(gave_up, h->workspace + kWsGaveUp, sizeof(int32_t), hipMemcpyDeviceToHost));
    // A wait that gave up may have left the fork or join word set; both streams are idle now.
    if (*gave_up) FO_HIP_CHECK(hipMemset(h->workspace, 0, kWorkspaceWords * sizeof(int32_t)));
    return FO_OK;
}

extern "C" fo_stream_t fo_overlap_comm_stream(fo_overlap_t *h) {
    return h ? static_cast<fo_stream_t>(h->comm_stream) : nullptr;
}

extern "C" int fo_overlap_gemm(fo_overlap_t *h, int dtype, int M, int N, int K, const void *A,
                               const void *B, void *C, int algo) {
    if (!h) return FO_ERR_ARG;
    if (!h->gemm_ready) return FO_ERR_STATE;
    return fo_gemm(dtype, M, N, K, A, B, C, algo, h->gemm_stream);
}

namespace {

// The reorder+RMSNorm that follows the overlapped GEMM in the reference's layers (example/RMSNorm.py:20-34
// behind example/RowParallelLinear.py:50-66), enqueued by the overlapped call itself: a tile row of the output
// can be normalised as soon as the group that holds its last tile has been consumed, so the rows follow the
// consumer batch by batch on the consumer stream and only the last batch's rows remain behind the GEMM.
struct norm_plan {
    void *Y = nullptr;
    const void *Wt = nullptr;
    float eps = 0.f;
    const int32_t *RA_host = nullptr;
};

// Rows of tile rows [first, end) of Y, on `stream`.
int norm_tile_rows(const norm_plan &np, int dtype, const void *C, int M, int N, int BM, int BN, int rLDN,
                   const int32_t *RA, int first, int end, bool beside_gemm, fo_stream_t stream) {
    return fo_norm_rows_with(dtype, C, np.Y, np.Wt, first * BM, (end - first) * BM, M, N, BM, BN, rLDN, RA, np.eps,
                             fo_streams((int64_t)M * N * 4), beside_gemm, 0, stream);
}

// Tile rows whose tiles all lie in storage slots below `done` and that have not been normalised yet, as
// runs of consecutive tile rows [first, end); at most kMaxRuns runs per batch (a reorder table that scatters the
// rows of a wave leaves the rest to the last batch, which takes everything that is left).
// last_slot[tm] = largest slot of tile row tm; -1 once handed out.  Appends to `runs`.
constexpr int kMaxRuns = 4;
void ready_tile_rows(long *last_slot, int TM, long done, bool final_batch, std::vector<int> &runs) {
    int n = 0;
    for (int tm = 0; tm < TM;) {
        if (last_slot[tm] < 0 || last_slot[tm] >= done) {
            tm++;
            continue;
        }
        int end = tm;
        while (end < TM && last_slot[end] >= 0 && last_slot[end] < done) end++;
        if (!final_batch && n == kMaxRuns) break;
        runs.push_back(tm);
        runs.push_back(end);
        for (int t = tm; t < end; t++) last_slot[t] = -1;
        n++;
        tm = end;
    }
}

// Largest storage slot of every tile row of the reorder table; FO_ERR_ARG for an entry outside [0, TM*TN).
int last_slots(const int32_t *RA_host, int TM, int TN, std::vector<long> &last_slot) {
    last_slot.assign(TM, 0);
    for (int tm = 0; tm < TM; tm++)
        for (int tn = 0; tn < TN; tn++) {
            const long r = RA_host[(long)tm * TN + tn];
            if (r < 0 || r >= (long)TM * TN) return FO_ERR_ARG;
            if (r > last_slot[tm]) last_slot[tm] = r;
        }
    return FO_OK;
}

int norm_ready_rows(const norm_plan &np, long *last_slot, int TM, long done, bool final_batch, int dtype, const void *C,
                    int M, int N, int BM, int BN, int rLDN, const int32_t *RA, bool beside_gemm, fo_stream_t stream) {
    std::vector<int> runs;
    ready_tile_rows(last_slot, TM, done, final_batch, runs);
    for (size_t k = 0; k + 1 < runs.size(); k += 2) {
        int rc = norm_tile_rows(np, dtype, C, M, N, BM, BN, rLDN, RA, runs[k], runs[k + 1], beside_gemm, stream);
        if (rc) return rc;
    }
    return FO_OK;
}

// GemmAllReduceOverlap on whatever `h` describes: a caller's handle, or the
// streams and static workspace of a handle-free call.  np: the normalisation to enqueue behind the consumer
// (null: none).
int allreduce_overlap(fo_overlap *h, int dtype, int M, int N, int K, const void *A, const void *B, void *C,
                      int32_t *MM, const int32_t *RA, int TM, int TN, int rLDN, const int32_t *cseg_host,
                      const int32_t *cseg_dev, int G, int algo, int monitor, const norm_plan *np = nullptr) {
    int32_t info[12];
    int rc = fo_algo_info(algo, info);
    if (rc) return rc;
    if (M <= 0 || N <= 0 || M % info[0] || N % info[1]) return FO_ERR_SHAPE;
    if (TM != M / info[0] || TN != N / info[1]) return FO_ERR_SHAPE;  // RA.shape must match the Algo's tile
    rc = check_segments(cseg_host, G, (long)TM * TN);
    if (rc) return rc;
    const int64_t tile_elems = (int64_t)info[0] * info[1];
    if (h->acc && h->acc_nelem < (int64_t)M * N) return FO_ERR_ARG;
    rc = link_fits(h, (int64_t)M * N * 2);
    if (rc) return rc;
    std::vector<long> last_slot;  // per tile row: its largest storage slot
    if (np) {
        if (!np->Y || !np->Wt || !np->RA_host) return FO_ERR_ARG;
        if (N % 8 || N > 16384 || (int64_t)M * N * 2 > 0xFFFFFFFFLL) return FO_ERR_SHAPE;
        rc = last_slots(np->RA_host, TM, TN, last_slot);
        if (rc) return rc;
    }

    const bool same_stream = in_stream(h, M, N, K);
    const int fused = same_stream ? 0 : fused_grid(h, G);
    fo_stream_t cstream = same_stream ? h->gemm_stream : h->comm_stream;
    int32_t wave = 0;
    if (same_stream) {
        wave = TM * TN;  // every group in one batch
    } else if (!fused) {
        rc = fo_gemm_wave_tiles(dtype, algo, M, N, &wave);
        if (rc) return rc;
    }
    const bool captured = capturing(h);
    if (!same_stream) {
        rc = fork(h, captured, fused != 0);
        if (rc) return rc;
    }
    // On one stream the order of the launches is all the synchronisation there is
    // to do: unless the caller wants the monitor's stamps, the GEMM then leaves
    // the counters alone (they stay zero, as the waits would have left them).
    const bool quiet = same_stream && !monitor;
    rc = quiet ? fo_gemm_reordered_quiet(dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, RA, nullptr, algo,
                                         h->gemm_stream)
               : fo_gemm_signal(dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, MM, RA, monitor, algo,
                                h->gemm_stream);
    if (rc) return rc;  // the GEMM was refused: nothing of this call follows on either stream

    // C' and the accumulator together against the memory-side cache
    const bool stream_acc = fo_streams((int64_t)M * N * 4);
    if (fused) {
        rc = fo_wait_reduce_groups_with(dtype, C, h->acc, MM, cseg_dev, G, tile_elems, 1, 0, nullptr, 0,
                                        h->workspace, fused, fused_slices((int64_t)M * N, G, fused),
                                        fused_poll_gap_ns(M, N, K, fused), stream_acc, h->max_polls, h->comm_stream);
        if (rc) return rc;
        rc = link_time(h, (int64_t)M * N * 2, h->comm_stream);
        if (rc) return rc;
        if (np) {  // that launch ends when the last group has been consumed: every row at once
            rc = norm_tile_rows(*np, dtype, C, M, N, info[0], info[1], rLDN, RA, 0, TM, false, h->comm_stream);
            if (rc) return rc;
        }
    } else {
        int64_t off = 0;
        long done = 0;
        uint16_t *c = static_cast<uint16_t *>(C);
        uint16_t *acc = static_cast<uint16_t *>(h->acc);
        for (int i = 0; i < G;) {
            const int j = batch_end(cseg_host, G, i, done, wave);
            long tiles = 0;
            for (int g = i; g < j; g++) tiles += cseg_host[g];
            const int64_t n = tiles * tile_elems;
            if (!quiet) {
                int32_t *gave_up = h->workspace ? h->workspace + kWsGaveUp : nullptr;
                rc = j - i == 1 ? fo_wait_with(cseg_host[i], MM + i, h->max_polls, gave_up, cstream)  // resets the counter
                                : fo_wait_groups_with(j - i, cseg_dev + i, MM + i, h->max_polls, gave_up, cstream);
                if (rc) return rc;
            }
            if (acc) {  // the groups of a batch are one contiguous range
                rc = fo_consumer_reduce_with(dtype, c + off, acc + off, n, 1, 0, nullptr, 0, stream_acc, cstream,
                                             j < G && !same_stream);  // every batch but the last runs beside the GEMM
                if (rc) return rc;
            }
            rc = link_time(h, n * 2, cstream);
            if (rc) return rc;
            off += n;
            done += tiles;
            if (np) {
                rc = norm_ready_rows(*np, last_slot.data(), TM, done, j == G, dtype, C, M, N, info[0], info[1], rLDN, RA,
                                     j < G && !same_stream, cstream);
                if (rc) return rc;
            }
            i = j;
        }
    }
    return same_stream ? FO_OK : join(h, captured);
}

}  // namespace

// Which tile rows fo_overlap_gemm_allreduce_norm normalises behind which batch of groups, for a caller that wants
// to know (and for tests on a machine without a GPU): the same planner the call uses.
extern "C" int fo_overlap_plan_norm_rows(const int32_t *RA_host, int TM, int TN, const int32_t *cseg_host, int G,
                                         int wave_tiles, int32_t *runs, int max_runs) {
    if (!RA_host || !runs || TM <= 0 || TN <= 0 || max_runs <= 0) return FO_ERR_ARG;
    int rc = check_segments(cseg_host, G, (long)TM * TN);
    if (rc) return rc;
    std::vector<long> last_slot;
    rc = last_slots(RA_host, TM, TN, last_slot);
    if (rc) return rc;
    int n = 0, batch = 0;
    long done = 0;
    for (int i = 0; i < G; batch++) {
        const int j = batch_end(cseg_host, G, i, done, wave_tiles);
        for (int g = i; g < j; g++) done += cseg_host[g];
        std::vector<int> ready;
        ready_tile_rows(last_slot.data(), TM, done, j == G, ready);
        for (size_t k = 0; k + 1 < ready.size(); k += 2) {
            if (n == max_runs) return FO_ERR_LIMIT;
            runs[3 * n] = batch;
            runs[3 * n + 1] = ready[k];
            runs[3 * n + 2] = ready[k + 1];
            n++;
        }
        i = j;
    }
    return n;
}

extern "C" int fo_overlap_gemm_allreduce(fo_overlap_t *h, int dtype, int M, int N, int K,
                                         const void *A, const void *B, void *C, int32_t *MM,
                                         const int32_t *RA, int TM, int TN, int rLDN,
                                         const int32_t *cseg_host, const int32_t *cseg_dev, int G,
                                         int algo, int monitor) {
    if (!h || !MM) return FO_ERR_ARG;
    if (!h->gemm_ready || !h->overlap_ready) return FO_ERR_STATE;
    return allreduce_overlap(h, dtype, M, N, K, A, B, C, MM, RA, TM, TN, rLDN, cseg_host, cseg_dev, G, algo,
                             monitor);
}

extern "C" int fo_overlap_gemm_allreduce_norm(fo_overlap_t *h, int dtype, int M, int N, int K, const void *A,
                                              const void *B, void *C, int32_t *MM, const int32_t *RA,
                                              const int32_t *RA_host, int TM, int TN, int rLDN,
                                              const int32_t *cseg_host, const int32_t *cseg_dev, int G, int algo,
                                              int monitor, void *Y, const void *Wt, float eps) {
    if (!h || !MM) return FO_ERR_ARG;
    if (!h->gemm_ready || !h->overlap_ready) return FO_ERR_STATE;
    norm_plan np;
    np.Y = Y;
    np.Wt = Wt;
    np.eps = eps;
    np.RA_host = RA_host;
    return allreduce_overlap(h, dtype, M, N, K, A, B, C, MM, RA, TM, TN, rLDN, cseg_host, cseg_dev, G, algo, monitor,
                             &np);
}

extern "C" int fo_overlap_gemm_reducescatter(fo_overlap_t *h, int dtype, int M, int N, int K,
                                             const void *A, const void *B, void *C, void *D,
                                             int32_t *MM, const int32_t *RA, const int32_t *RE,
                                             int TM, int TN, int rLDN, const int32_t *cseg_host,
                                             const int32_t *cseg_dev, int G, int algo, int monitor) {
    if (!h || !MM || !RE) return FO_ERR_ARG;
    if (!h->gemm_ready || !h->overlap_ready) return FO_ERR_STATE;
    int32_t info[12];
    int rc = fo_algo_info(algo, info);
    if (rc) return rc;
    if (M <= 0 || N <= 0 || M % info[0] || N % info[1]) return FO_ERR_SHAPE;
    if (TM != M / info[0] || TN != N / info[1]) return FO_ERR_SHAPE;
    rc = check_segments(cseg_host, G, (long)TM * TN);
    if (rc) return rc;
    const int W = h->world;
    const int64_t tile_elems = (int64_t)info[0] * info[1];
    if (tile_elems % (8 * W) || ((int64_t)M * N) % W) return FO_ERR_SHAPE;
    const int64_t seg_stride = (int64_t)M * N / W;
    if (h->acc && h->acc_nelem < (int64_t)M * N) return FO_ERR_ARG;
    rc = link_fits(h, (int64_t)M * N * 2);
    if (rc) return rc;

    const bool same_stream = in_stream(h, M, N, K);
    const int fused = same_stream ? 0 : fused_grid(h, G);
    fo_stream_t cstream = same_stream ? h->gemm_stream : h->comm_stream;
    int32_t wave = 0;
    if (same_stream) {
        wave = TM * TN;  // every group in one batch
    } else if (!fused) {
        rc = fo_gemm_wave_tiles(dtype, algo, M, N, &wave);
        if (rc) return rc;
    }
    const bool captured = capturing(h);
    if (!same_stream) {
        rc = fork(h, captured, fused != 0);
        if (rc) return rc;
    }
    const bool quiet = same_stream && !monitor;  // as in fo_overlap_gemm_allreduce
    rc = quiet ? fo_gemm_reordered_quiet(dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, RA, RE, algo,
                                         h->gemm_stream)
               : fo_gemm_scatter(dtype, M, N, K, rLDN, cseg_dev, G, A, B, C, MM, RA, RE, monitor, algo,
                                 h->gemm_stream);
    if (rc) return rc;

    uint16_t *c = static_cast<uint16_t *>(C);
    uint16_t *d = static_cast<uint16_t *>(D);
    uint16_t *acc = static_cast<uint16_t *>(h->acc);
    // With an accumulator and W > 1 the consumer also writes this rank's chunk of
    // every group to D (ncclReduceScatter(C+acc -> D+acc/W, n/W) with one rank
    // present, src/overlap_impl.cu:312-313); otherwise a copy per group does.
    const bool own_in_consumer = d && acc && W > 1;
    const bool stream_acc = fo_streams((int64_t)M * N * 4);
    if (fused) {
        rc = fo_wait_reduce_groups_with(dtype, C, h->acc, MM, cseg_dev, G, tile_elems, W, seg_stride,
                                        own_in_consumer ? D : nullptr, h->rank, h->workspace, fused,
                                        fused_slices((int64_t)M * N, G, fused), fused_poll_gap_ns(M, N, K, fused),
                                        stream_acc, h->max_polls, cstream);
        if (rc) return rc;
        rc = link_time(h, (int64_t)M * N * 2, cstream);
        if (rc) return rc;
    }
    int64_t off = 0;
    long done = 0;
    for (int i = 0; i < G;) {
        const int j = fused ? i + 1 : batch_end(cseg_host, G, i, done, wave);
        const int64_t off_batch = off;
        if (!fused && !quiet) {
            int32_t *gave_up = h->workspace ? h->workspace + kWsGaveUp : nullptr;
            rc = j - i == 1 ? fo_wait_with(cseg_host[i], MM + i, h->max_polls, gave_up, cstream)
                            : fo_wait_groups_with(j - i, cseg_dev + i, MM + i, h->max_polls, gave_up, cstream);
            if (rc) return rc;
        }
        if (!fused && acc && W > 1 && j - i > 1) {
            // the groups of one wave in one launch; each keeps its own W chunks
            long most = 0;
            for (int g = i; g < j; g++) most = cseg_host[g] > most ? cseg_host[g] : most;
            rc = fo_consumer_reduce_groups_with(dtype, c + off, acc + off / W, cseg_dev + i, j - i, most,
                                                tile_elems, W, seg_stride, own_in_consumer ? d + off / W : nullptr,
                                                h->rank, stream_acc, cstream, j < G && !same_stream);
            if (rc) return rc;
        }
        for (int g = i; g < j; g++) {
            const int64_t n = cseg_host[g] * tile_elems;
            if (!fused && acc && !(W > 1 && j - i > 1)) {
                rc = fo_consumer_reduce_with(dtype, c + off, acc + off / W, n, W, seg_stride,
                                             own_in_consumer ? d + off / W : nullptr, h->rank, stream_acc, cstream,
                                             j < G && !same_stream);
                if (rc) return rc;
            }
            if (d && !own_in_consumer)
                FO_HIP_CHECK(hipMemcpyAsync(d + off / W, c + off + (int64_t)h->rank * (n / W),
                                            (size_t)(n / W) * 2, hipMemcpyDeviceToDevice,
                                            static_cast<hipStream_t>(cstream)));
            off += n;
            done += cseg_host[g];
        }
        if (!fused) {
            rc = link_time(h, (off - off_batch) * 2, cstream);
            if (rc) return rc;
        }
        i = j;
    }
    return same_stream ? FO_OK : join(h, captured);
}

extern "C" int fo_overlap_gemm_allreduce_serial(fo_overlap_t *h, int dtype, int M, int N, int K,
                                                const void *A, const void *B, void *C, int algo) {
    if (!h) return FO_ERR_ARG;
    if (!h->gemm_ready) return FO_ERR_STATE;
    if (h->acc && h->acc_nelem < (int64_t)M * N) return FO_ERR_ARG;
    int rc = fo_gemm(dtype, M, N, K, A, B, C, algo, h->gemm_stream);
    if (rc) return rc;
    if (h->acc) {
        rc = fo_consumer_reduce(dtype, C, h->acc, (int64_t)M * N, h->gemm_stream);
        if (rc) return rc;
    }
    return link_time(h, (int64_t)M * N * 2, h->gemm_stream);
}

extern "C" int fo_overlap_seg_allreduce(fo_overlap_t *h, int dtype, void *C, int64_t MN,
                                        const int32_t *cseg_host, int G, int seg_num) {
    if (!h || !C || !cseg_host || G <= 0 || seg_num <= 0 || MN <= 0) return FO_ERR_ARG;
    if (!h->gemm_ready) return FO_ERR_STATE;
    if (MN % seg_num || G < seg_num) return FO_ERR_SHAPE;
    if (h->acc && h->acc_nelem < MN) return FO_ERR_ARG;
    const int64_t unit = MN / seg_num;
    int64_t off = 0;
    uint16_t *c = static_cast<uint16_t *>(C);
    uint16_t *acc = static_cast<uint16_t *>(h->acc);
    for (int s = 0; s < seg_num; s++) {  // the reference iterates SegNum times over cSEG_CPU
        const int64_t n = unit * cseg_host[s];
        if (off + n > MN) return FO_ERR_SEGMENTS;
        if (acc) {
            int rc = fo_consumer_reduce(dtype, c + off, acc + off, n, h->gemm_stream);
            if (rc) return rc;
        }
        int rc = link_time(h, n * 2, h->gemm_stream);
        if (rc) return rc;
        off += n;
    }
    return FO_OK;
}

// ---------------------------------------------------------------- handle-free call that allocates nothing
// Callers that cannot allocate (code under a harness that forbids it, serving
// loops) have no handle: a handle owns a hipMalloc'ed workspace and, in the
// reference's interface, the caller brings the counters MM in a tensor of its own.
// Here both live in this file-scope array: kWorkspaceWords flag words, then one
// counter per group.  Each device the library runs on holds its own copy until the
// process ends; its address is asked for once per device.
constexpr int kStaticMaxGroups = 4096;
static __device__ __align__(256) int32_t scratch[kWorkspaceWords + kStaticMaxGroups];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
int32_t *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device (the array's name is not one)
int g_scratch_token[kMaxDevices];     // last fork/join token handed out on each device

int scratch_of_current_device(int32_t **ptr, int *token) {
    int dev = 0;
    FO_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return FO_ERR_STATE;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        FO_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return FO_ERR_STATE;
        g_scratch_ptr[dev] = static_cast<int32_t *>(p);
    }
    *ptr = g_scratch_ptr[dev];
    // never 0 (the words' resting value) and never the previous call's, so a word
    // that an abandoned wait left behind cannot pass for this call's
    g_scratch_token[dev] = g_scratch_token[dev] >= (1 << 30) ? 1 : g_scratch_token[dev] + 1;
    *token = g_scratch_token[dev];
    return FO_OK;
}

}  // namespace

extern "C" int fo_gemm_allreduce_overlap_static(int dtype, int M, int N, int K, const void *A, const void *B,
                                                void *C, void *acc, const int32_t *RA, int TM, int TN, int rLDN,
                                                const int32_t *cseg_host, const int32_t *cseg_dev, int G, int algo,
                                                int fused, fo_stream_t gemm_stream, fo_stream_t comm_stream) {
    if (G > kStaticMaxGroups) return FO_ERR_LIMIT;
    if (G <= 0 || !cseg_host || !cseg_dev) return FO_ERR_SEGMENTS;
    int32_t *ws = nullptr;
    int token = 0;
    int rc = scratch_of_current_device(&ws, &token);
    if (rc) return rc;
    fo_overlap ctx;
    ctx.gemm_stream = static_cast<hipStream_t>(gemm_stream);
    ctx.comm_stream = comm_stream == gemm_stream ? nullptr : static_cast<hipStream_t>(comm_stream);
    ctx.workspace = ws;
    ctx.gemm_ready = ctx.overlap_ready = true;
    ctx.acc = acc;
    ctx.acc_nelem = acc ? (int64_t)M * N : 0;
    ctx.fused = fused < 0 ? -1 : fused;
    ctx.token = token;
    ctx.always_fork = true;
    // Validate before the first launch, so that a refused call leaves nothing enqueued.
    int32_t info[12];
    rc = fo_algo_info(algo, info);
    if (rc) return rc;
    if (M <= 0 || N <= 0 || M % info[0] || N % info[1] || TM != M / info[0] || TN != N / info[1]) return FO_ERR_SHAPE;
    rc = check_segments(cseg_host, G, (long)TM * TN);
    if (rc) return rc;
    if (!A || !B || !C || !RA || K <= 0 || K % 8) return !A || !B || !C || !RA || K <= 0 ? FO_ERR_ARG : FO_ERR_SHAPE;
    if (ctx.comm_stream && capturing(&ctx)) return FO_ERR_STATE;  // two streams under capture need the handle's events
    // The array keeps what the last call on this device left: counters of a call whose
    // bounded wait gave up would still be standing.  Cleared by a kernel, not a memset
    // node, in case the GEMM stream is being captured.
    // The give-up word is left standing: fo_static_status reads and clears it.
    rc = fo_fill_words(ws, kWorkspaceWords + G, 0, ctx.gemm_stream, kWsGaveUp);
    if (rc) return rc;
    return allreduce_overlap(&ctx, dtype, M, N, K, A, B, C, ws + kWorkspaceWords, RA, TM, TN, rLDN, cseg_host,
                             cseg_dev, G, algo, 0);
}

// Whether a bounded device-side wait of an allocation-free call gave up since the
// last query on this device.  The calls have no handle to ask; the flag word of the
// static array is sticky across calls until it is read here.
extern "C" int fo_static_status(fo_stream_t gemm_stream, fo_stream_t comm_stream, int32_t *gave_up) {
    if (!gave_up) return FO_ERR_ARG;
    *gave_up = 0;
    int32_t *ws = nullptr;
    int token = 0;
    int rc = scratch_of_current_device(&ws, &token);
    if (rc) return rc;
    FO_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(gemm_stream)));
    if (comm_stream != gemm_stream) FO_HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(comm_stream)));
    FO_HIP_CHECK(hipMemcpy(gave_up, ws + kWsGaveUp, sizeof(int32_t), hipMemcpyDeviceToHost));
    // A wait that gave up may have left the fork or join word set; both streams are idle now.
    if (*gave_up) FO_HIP_CHECK(hipMemset(ws, 0, kWorkspaceWords * sizeof(int32_t)));
    return FO_OK;
}
