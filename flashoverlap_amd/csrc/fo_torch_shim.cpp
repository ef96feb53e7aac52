// TORCH_LIBRARY shim: the drop-in boundary of the reference (src/pybind.cpp:114-150)
// on top of the C ABI in include/flashoverlap.h.  It registers
//   torch.classes.flashoverlap_class.{OverlapImpl, BaselineImpl}
//   torch.ops.flashoverlap_op.{generate_nccl_id, reorder_rmsnorm}
// with the reference's method names and argument order, plus a few additions
// (marked "addition") that one GPU needs: the consumer's accumulation buffer,
// the fused consumer switch, bf16, explicit eps.
//
// Tensors are only unpacked to pointers here; no kernel code, no allocation.
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <torch/custom_class.h>
#include <torch/library.h>

#include <algorithm>
#include <vector>

#include "flashoverlap.h"

namespace {

void check(int rc, const char *what) {
    TORCH_CHECK(rc == 0, "flashoverlap: ", what, " failed: ", fo_error_string(rc), " (code ", rc, ")");
}

// The reference accepts fp16 only (data_ptr<at::Half>() throws otherwise); bf16 is an addition.
int dtype_of(const at::Tensor &t) {
    if (t.scalar_type() == at::kHalf) return FO_F16;
    if (t.scalar_type() == at::kBFloat16) return FO_BF16;
    TORCH_CHECK(false, "flashoverlap: expected a Half or BFloat16 tensor, got ", t.scalar_type());
}

void *dev_ptr(const at::Tensor &t, const char *name) {
    TORCH_CHECK(t.is_cuda(), "flashoverlap: ", name, " must be a GPU tensor");
    TORCH_CHECK(t.is_contiguous(), "flashoverlap: ", name, " must be contiguous");
    return t.data_ptr();
}

int32_t *dev_i32(const at::Tensor &t, const char *name) {
    TORCH_CHECK(t.scalar_type() == at::kInt, "flashoverlap: ", name, " must be int32");
    return static_cast<int32_t *>(dev_ptr(t, name));
}

const int32_t *host_i32(const at::Tensor &t, const char *name) {
    TORCH_CHECK(t.scalar_type() == at::kInt && !t.is_cuda() && t.is_contiguous(), "flashoverlap: ",
                name, " must be a contiguous int32 CPU tensor");
    return t.data_ptr<int32_t>();
}

fo_stream_t current_stream() { return c10::hip::getCurrentHIPStream().stream(); }

struct Shape {
    int M, N, K;
};
Shape gemm_shape(const at::Tensor &A, const at::Tensor &B, const at::Tensor &C) {
    TORCH_CHECK(A.dim() == 2 && B.dim() == 2, "flashoverlap: A[M,K] and B[N,K] must be 2-D");
    TORCH_CHECK(A.size(1) == B.size(1), "flashoverlap: A and B disagree on K");
    TORCH_CHECK(A.scalar_type() == B.scalar_type() && A.scalar_type() == C.scalar_type(),
                "flashoverlap: A, B and C must share one dtype");
    TORCH_CHECK(C.numel() == A.size(0) * B.size(0), "flashoverlap: C must hold M*N elements");
    return {(int)A.size(0), (int)B.size(0), (int)A.size(1)};
}

// The kernels index MM, RA, RE and D through raw pointers; the reference checks none of
// their sizes and overruns MM when there are more groups than tile columns
// (test/test.py:94 allocates TN ints).  Refuse before anything is launched.
void check_buffers(const Shape &s, int64_t Algo, const at::Tensor &MM, const at::Tensor &RA, int64_t rLDN,
                   const at::Tensor &cSEG_CPU, const at::Tensor &cSEG_GPU, bool monitor, const at::Tensor *RE,
                   const at::Tensor *D, int64_t world) {
    int32_t info[12];
    check(fo_algo_info((int)Algo, info), "Algo lookup");
    TORCH_CHECK(s.M % info[0] == 0 && s.N % info[1] == 0, "flashoverlap: M x N = ", s.M, " x ", s.N,
                " is not a multiple of the Algo's tile ", info[0], " x ", info[1]);
    const int64_t TM = s.M / info[0], TN = s.N / info[1], G = cSEG_GPU.numel();
    TORCH_CHECK(RA.dim() == 2 && RA.size(0) == TM && RA.size(1) == TN, "flashoverlap: RA must be [", TM, ", ", TN,
                "] for this Algo");
    TORCH_CHECK(cSEG_CPU.numel() == G, "flashoverlap: cSEG_CPU/cSEG_GPU differ");
    const int64_t need = monitor ? (TM + 1) * TN : std::max(G, TN);
    TORCH_CHECK(MM.numel() >= need, "flashoverlap: MM holds ", MM.numel(), " counters, ", need, " are needed (", G,
                " groups, ", TM, " x ", TN, " tiles", monitor ? ", monitor)" : ")");
    TORCH_CHECK(rLDN > 0 && (TM * TN) % rLDN == 0, "flashoverlap: rLDN = ", rLDN, " does not divide the tiles");
    if (RE) {
        const int64_t rows = (int64_t)s.M * s.N / (rLDN * info[1]);
        TORCH_CHECK(RE->numel() >= rows, "flashoverlap: RE holds ", RE->numel(), " rows, the reshaped output has ",
                    rows);
    }
    if (D) {
        TORCH_CHECK(world > 0 && D->numel() >= (int64_t)s.M * s.N / world, "flashoverlap: D holds ", D->numel(),
                    " elements, M*N/W = ", (int64_t)s.M * s.N / world, " are needed");
    }
}

// class OverlapImpl, src/overlap_impl.h:12-43.
struct OverlapImpl : torch::CustomClassHolder {
    fo_overlap_t *h = nullptr;
    at::Tensor acc;  // keeps the accumulation buffer alive
    int64_t rank_ = 0, world_ = 1;

    OverlapImpl() { check(fo_overlap_create(&h), "fo_overlap_create"); }
    ~OverlapImpl() override { fo_overlap_destroy(h); }

    void nccl_init(int64_t rank, int64_t world, std::vector<int64_t> /*id*/) {
        check(fo_overlap_set_world(h, (int)rank, (int)world), "nccl_init");
        rank_ = rank;
        world_ = world;
    }
    void cutlass_init() { check(fo_overlap_set_gemm_stream(h, current_stream()), "cutlass_init"); }
    void overlap_init() { check(fo_overlap_init(h), "overlap_init"); }

    void cutlass_gemm(at::Tensor A, at::Tensor B, at::Tensor C, int64_t Algo) {
        Shape s = gemm_shape(A, B, C);
        check(fo_overlap_gemm(h, dtype_of(A), s.M, s.N, s.K, dev_ptr(A, "A"), dev_ptr(B, "B"),
                              dev_ptr(C, "C"), (int)Algo),
              "cutlass_gemm");
    }

    void gemm_allreduce_overlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor MM, at::Tensor RA,
                                int64_t rLDN, at::Tensor cSEG_CPU, at::Tensor cSEG_GPU, int64_t Algo,
                                bool if_monitor) {
        Shape s = gemm_shape(A, B, C);
        check_buffers(s, Algo, MM, RA, rLDN, cSEG_CPU, cSEG_GPU, if_monitor, nullptr, nullptr, 1);
        TORCH_CHECK(!acc.defined() || acc.numel() >= (int64_t)s.M * s.N, "flashoverlap: the accumulator is smaller than M*N");
        check(fo_overlap_gemm_allreduce(h, dtype_of(A), s.M, s.N, s.K, dev_ptr(A, "A"), dev_ptr(B, "B"),
                                        dev_ptr(C, "C"), dev_i32(MM, "MM"), dev_i32(RA, "RA"),
                                        (int)RA.size(0), (int)RA.size(1), (int)rLDN,
                                        host_i32(cSEG_CPU, "cSEG_CPU"), dev_i32(cSEG_GPU, "cSEG_GPU"),
                                        (int)cSEG_GPU.size(0), (int)Algo, if_monitor ? 1 : 0),
              "gemm_allreduce_overlap");
    }

    // Addition: gemm_allreduce_overlap followed by reorder_rmsnorm(C -> Y) with the rows normalised on the consumer
    // stream as the groups that complete them are consumed (fo_overlap_gemm_allreduce_norm); RA_CPU is a host copy of RA.
    void gemm_allreduce_rmsnorm_overlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor MM, at::Tensor RA,
                                        at::Tensor RA_CPU, int64_t rLDN, at::Tensor cSEG_CPU, at::Tensor cSEG_GPU,
                                        int64_t Algo, bool if_monitor, at::Tensor Y, at::Tensor RW, double eps) {
        Shape s = gemm_shape(A, B, C);
        check_buffers(s, Algo, MM, RA, rLDN, cSEG_CPU, cSEG_GPU, if_monitor, nullptr, nullptr, 1);
        TORCH_CHECK(!acc.defined() || acc.numel() >= (int64_t)s.M * s.N, "flashoverlap: the accumulator is smaller than M*N");
        TORCH_CHECK(RA_CPU.numel() == RA.numel(), "flashoverlap: RA_CPU must be a host copy of RA");
        TORCH_CHECK(Y.scalar_type() == C.scalar_type() && RW.scalar_type() == C.scalar_type(),
                    "flashoverlap: C, Y and RW must share one dtype");
        TORCH_CHECK(Y.numel() == (int64_t)s.M * s.N && RW.numel() >= s.N, "flashoverlap: need Y[M,N] and RW[N]");
        check(fo_overlap_gemm_allreduce_norm(h, dtype_of(A), s.M, s.N, s.K, dev_ptr(A, "A"), dev_ptr(B, "B"),
                                             dev_ptr(C, "C"), dev_i32(MM, "MM"), dev_i32(RA, "RA"),
                                             host_i32(RA_CPU, "RA_CPU"), (int)RA.size(0), (int)RA.size(1), (int)rLDN,
                                             host_i32(cSEG_CPU, "cSEG_CPU"), dev_i32(cSEG_GPU, "cSEG_GPU"),
                                             (int)cSEG_GPU.size(0), (int)Algo, if_monitor ? 1 : 0, dev_ptr(Y, "Y"),
                                             dev_ptr(RW, "RW"), (float)eps),
              "gemm_allreduce_rmsnorm_overlap");
    }

    void gemm_reducescatter_overlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D,
                                    at::Tensor MM, at::Tensor RA, at::Tensor RE, int64_t rLDN,
                                    at::Tensor cSEG_CPU, at::Tensor cSEG_GPU, int64_t Algo,
                                    bool if_monitor) {
        Shape s = gemm_shape(A, B, C);
        TORCH_CHECK(D.scalar_type() == C.scalar_type(), "flashoverlap: C and D must share one dtype");
        check_buffers(s, Algo, MM, RA, rLDN, cSEG_CPU, cSEG_GPU, if_monitor, &RE, &D, world_);
        TORCH_CHECK(!acc.defined() || acc.numel() >= (int64_t)s.M * s.N, "flashoverlap: the accumulator is smaller than M*N");
        check(fo_overlap_gemm_reducescatter(
                  h, dtype_of(A), s.M, s.N, s.K, dev_ptr(A, "A"), dev_ptr(B, "B"), dev_ptr(C, "C"),
                  dev_ptr(D, "D"), dev_i32(MM, "MM"), dev_i32(RA, "RA"), dev_i32(RE, "RE"),
                  (int)RA.size(0), (int)RA.size(1), (int)rLDN, host_i32(cSEG_CPU, "cSEG_CPU"),
                  dev_i32(cSEG_GPU, "cSEG_GPU"), (int)cSEG_GPU.size(0), (int)Algo, if_monitor ? 1 : 0),
              "gemm_reducescatter_overlap");
    }

    // GemmAllReduce, src/overlap_impl.cu:65-81.
    void gemm_allreduce(at::Tensor A, at::Tensor B, at::Tensor C, int64_t Algo) {
        Shape s = gemm_shape(A, B, C);
        check(fo_overlap_gemm_allreduce_serial(h, dtype_of(A), s.M, s.N, s.K, dev_ptr(A, "A"),
                                               dev_ptr(B, "B"), dev_ptr(C, "C"), (int)Algo),
              "gemm_allreduce");
    }
    // GemmReduceScatter, src/overlap_impl.cu:83-101: plain GEMM, then the whole-C
    // reduce-scatter; with one rank present D receives this rank's 1/W of C.
    void gemm_reducescatter(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, int64_t Algo) {
        cutlass_gemm(A, B, C, Algo);
        scatter_whole(C, D);
    }
    // GemmAll2All, src/overlap_impl.cu:103-137: with one rank there is no peer to
    // exchange rows with; the GEMM and the trailing whole-C reduction remain.
    void gemm_all2all(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor /*D*/, int64_t Algo,
                      at::Tensor /*mLen_CPU*/) {
        gemm_allreduce(A, B, C, Algo);
    }
    // NcclAllReduce, src/overlap_impl.cu:143-151.
    void nccl_allreduce(at::Tensor C) {
        if (!acc.defined()) return;  // a one-rank sum is the identity
        TORCH_CHECK(acc.numel() >= C.numel() && acc.scalar_type() == C.scalar_type(),
                    "flashoverlap: the accumulator must hold C.numel() elements of C's dtype");
        check(fo_consumer_reduce(dtype_of(C), dev_ptr(C, "C"), acc.data_ptr(), C.numel(),
                                 current_stream()),
              "nccl_allreduce");
    }
    // NcclReduceScatter, src/overlap_impl.cu:168-178: in place, rank's chunk stays where it is.
    void nccl_reducescatter(at::Tensor /*C*/) {}
    void nccl_all2all(at::Tensor /*C*/, at::Tensor /*D*/, at::Tensor /*mLen_CPU*/) {}
    // SegAllReduce, src/overlap_impl.cu:153-167.
    void seg_allreduce(at::Tensor C, at::Tensor cSEG_CPU, int64_t SegNum) {
        check(fo_overlap_seg_allreduce(h, dtype_of(C), dev_ptr(C, "C"), C.numel(),
                                       host_i32(cSEG_CPU, "cSEG_CPU"), (int)cSEG_CPU.numel(),
                                       (int)SegNum),
              "seg_allreduce");
    }

    // addition: accumulation buffer of the stand-in consumer ([M,N], or [W,M/W,N] for reduce-scatter).
    void set_accumulator(at::Tensor ACC) {
        acc = ACC;
        check(fo_overlap_set_accumulator(h, dev_ptr(ACC, "ACC"), ACC.numel()), "set_accumulator");
    }
    void clear_accumulator() {
        acc = at::Tensor();
        check(fo_overlap_set_accumulator(h, nullptr, 0), "clear_accumulator");
    }
    // addition: -1 chosen per call (default), 0 two launches per group as the reference's host loop,
    // 1 one wait+reduce launch for all groups, n > 1 the same with n workgroups.
    void set_fused_consumer(int64_t fused) {
        check(fo_overlap_set_fused_consumer(h, (int)fused), "set_fused_consumer");
    }
    // addition: link-rate model, gigabytes per second of the collective the consumer stands in for (0: off).
    void set_link_rate(double gigabytes_per_second) {
        check(fo_overlap_set_link_rate(h, gigabytes_per_second), "set_link_rate");
    }
    // addition: whether a bounded device-side wait gave up since the last query (synchronises).
    int64_t status() {
        int32_t gave_up = 0;
        check(fo_overlap_status(h, &gave_up), "status");
        return gave_up;
    }

   private:
    void scatter_whole(const at::Tensor &C, at::Tensor &D) {
        // D = the rank-th 1/W of C_flat (recvcount = M*N/W, src/overlap_impl.cu:98-100).
        const int64_t W = C.numel() / D.numel();
        TORCH_CHECK(W >= 1 && D.numel() * W == C.numel(), "flashoverlap: D must hold M*N/W elements");
        D.view({-1}).copy_(C.view({-1}).narrow(0, rank_ * D.numel(), D.numel()), /*non_blocking=*/true);
    }
};

// class BaselineImpl, src/baseline_impl.h:10-34: vendor GEMM (here: torch's
// hipBLASLt-backed mm) followed by the collective stand-in on one stream.  It is
// the comparator of the speed test, not part of the product path.
struct BaselineImpl : torch::CustomClassHolder {
    at::Tensor acc;
    int64_t rank = 0, world = 1;

    void nccl_init(int64_t r, int64_t w, std::vector<int64_t> /*id*/) {
        rank = r;
        world = w;
    }
    void cublas_init() {}
    void cublas_gemm(at::Tensor A, at::Tensor B, at::Tensor C) { at::mm_out(C, A, B.t()); }
    void gemm_allreduce(at::Tensor A, at::Tensor B, at::Tensor C) {
        cublas_gemm(A, B, C);
        nccl_allreduce(C);
    }
    void gemm_reducescatter(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D) {
        cublas_gemm(A, B, C);
        D.view({-1}).copy_(C.view({-1}).narrow(0, rank * D.numel(), D.numel()), true);
    }
    void gemm_all2all(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor /*D*/,
                      at::Tensor /*mLen_CPU*/) {
        gemm_allreduce(A, B, C);
    }
    void nccl_allreduce(at::Tensor C) {
        if (acc.defined()) {
            TORCH_CHECK(acc.numel() >= C.numel() && acc.scalar_type() == C.scalar_type(),
                        "flashoverlap: the accumulator must hold C.numel() elements of C's dtype");
            check(fo_consumer_reduce(dtype_of(C), dev_ptr(C, "C"), acc.data_ptr(), C.numel(),
                                     current_stream()),
                  "nccl_allreduce");
        }
        if (link_gb_per_s > 0)  // the same link time the overlapped calls model (OverlapImpl.set_link_rate)
            check(fo_pace((int64_t)(C.numel() * C.element_size() / link_gb_per_s), current_stream()), "nccl_allreduce");
    }
    void nccl_reducescatter(at::Tensor /*C*/) {}
    void nccl_all2all(at::Tensor /*C*/, at::Tensor /*D*/, at::Tensor /*mLen_CPU*/) {}
    void set_accumulator(at::Tensor ACC) { acc = ACC; }  // addition
    double link_gb_per_s = 0;
    void set_link_rate(double gigabytes_per_second) {  // addition
        TORCH_CHECK(gigabytes_per_second >= 0, "flashoverlap: the link rate must not be negative");
        link_gb_per_s = gigabytes_per_second;
    }
};

// generate_nccl_id, src/nccl_utils.cu:7-14: 128 opaque bytes as 16 int64.  No
// communicator exists on one GPU, so the id is a constant tag.
std::vector<int64_t> generate_nccl_id() {
    std::vector<int64_t> id(16, 0);
    id[0] = 0x464c4153484f564cLL;  // "FLASHOVL"
    return id;
}

void reorder_rmsnorm_eps(at::Tensor X, at::Tensor RX, at::Tensor RW, int64_t BM, int64_t BN,
                         int64_t rldn, at::Tensor RA, double eps) {
    TORCH_CHECK(X.dim() == 2 && RX.sizes() == X.sizes(), "flashoverlap: X and RX must be [bs, dim]");
    TORCH_CHECK(X.scalar_type() == RX.scalar_type() && X.scalar_type() == RW.scalar_type(),
                "flashoverlap: X, RX and RW must share one dtype");
    TORCH_CHECK(RW.numel() >= X.size(1), "flashoverlap: RW must hold dim elements");
    TORCH_CHECK(BM > 0 && BN > 0 && X.size(0) % BM == 0 && X.size(1) % BN == 0,
                "flashoverlap: [bs, dim] must be a multiple of the tile");
    TORCH_CHECK(RA.numel() >= (X.size(0) / BM) * (X.size(1) / BN), "flashoverlap: RA holds ", RA.numel(),
                " entries, the matrix has ", (X.size(0) / BM) * (X.size(1) / BN), " tiles");
    check(fo_reorder_rmsnorm(dtype_of(X), dev_ptr(X, "X"), dev_ptr(RX, "RX"), dev_ptr(RW, "RW"),
                             (int)X.size(0), (int)X.size(1), (int)BM, (int)BN, (int)rldn,
                             dev_i32(RA, "RA"), (float)eps, current_stream()),
          "reorder_rmsnorm");
}

// reorder_rmsnorm, src/rmsnorm/rmsnorm.cu:14-30; eps fixed at 1e-5 as in rmsnorm.cuh:102.
void reorder_rmsnorm(at::Tensor X, at::Tensor RX, at::Tensor RW, int64_t BM, int64_t BN,
                     int64_t rldn, at::Tensor RA) {
    reorder_rmsnorm_eps(X, RX, RW, BM, BN, rldn, RA, 1e-5);
}

// rmsnorm, src/rmsnorm/rmsnorm.cu:32-46 (the reference compiles but does not register it).
void rmsnorm_eps(at::Tensor X, at::Tensor O, at::Tensor RW, double eps) {
    TORCH_CHECK(X.dim() == 2 && O.sizes() == X.sizes(), "flashoverlap: X and O must be [bs, dim]");
    TORCH_CHECK(X.scalar_type() == O.scalar_type() && X.scalar_type() == RW.scalar_type() && RW.numel() >= X.size(1),
                "flashoverlap: X, O and RW must share one dtype and RW must hold dim elements");
    check(fo_rmsnorm(dtype_of(X), dev_ptr(X, "X"), dev_ptr(O, "O"), dev_ptr(RW, "RW"), (int)X.size(0),
                     (int)X.size(1), (float)eps, current_stream()),
          "rmsnorm");
}

}  // namespace

TORCH_LIBRARY(flashoverlap_class, m) {
    m.class_<BaselineImpl>("BaselineImpl")
        .def(torch::init())
        .def("nccl_init", &BaselineImpl::nccl_init)
        .def("cublas_init", &BaselineImpl::cublas_init)
        .def("gemm_allreduce", &BaselineImpl::gemm_allreduce)
        .def("gemm_reducescatter", &BaselineImpl::gemm_reducescatter)
        .def("gemm_all2all", &BaselineImpl::gemm_all2all)
        .def("cublas_gemm", &BaselineImpl::cublas_gemm)
        .def("set_link_rate", &BaselineImpl::set_link_rate)
        .def("nccl_allreduce", &BaselineImpl::nccl_allreduce)
        .def("nccl_reducescatter", &BaselineImpl::nccl_reducescatter)
        .def("nccl_all2all", &BaselineImpl::nccl_all2all)
        .def("set_accumulator", &BaselineImpl::set_accumulator);
    m.class_<OverlapImpl>("OverlapImpl")
        .def(torch::init())
        .def("cutlass_init", &OverlapImpl::cutlass_init)
        .def("cutlass_gemm", &OverlapImpl::cutlass_gemm)
        .def("gemm_allreduce_overlap", &OverlapImpl::gemm_allreduce_overlap)
        .def("gemm_reducescatter_overlap", &OverlapImpl::gemm_reducescatter_overlap)
        .def("gemm_allreduce_rmsnorm_overlap", &OverlapImpl::gemm_allreduce_rmsnorm_overlap)  // addition
        .def("nccl_init", &OverlapImpl::nccl_init)
        .def("gemm_allreduce", &OverlapImpl::gemm_allreduce)
        .def("gemm_reducescatter", &OverlapImpl::gemm_reducescatter)
        .def("gemm_all2all", &OverlapImpl::gemm_all2all)
        .def("overlap_init", &OverlapImpl::overlap_init)
        .def("nccl_allreduce", &OverlapImpl::nccl_allreduce)
        .def("nccl_reducescatter", &OverlapImpl::nccl_reducescatter)
        .def("nccl_all2all", &OverlapImpl::nccl_all2all)
        .def("seg_allreduce", &OverlapImpl::seg_allreduce)
        .def("set_accumulator", &OverlapImpl::set_accumulator)
        .def("clear_accumulator", &OverlapImpl::clear_accumulator)
        .def("set_fused_consumer", &OverlapImpl::set_fused_consumer)
        .def("set_link_rate", &OverlapImpl::set_link_rate)
        .def("status", &OverlapImpl::status);
}

TORCH_LIBRARY(flashoverlap_op, m) {
    m.def("generate_nccl_id", &generate_nccl_id);
    m.def("reorder_rmsnorm", &reorder_rmsnorm);
    m.def("reorder_rmsnorm_eps", &reorder_rmsnorm_eps);  // addition
    m.def("rmsnorm", &rmsnorm_eps);                      // addition
}
