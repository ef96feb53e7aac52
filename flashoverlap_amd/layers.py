"""Layer wrappers over the drop-in boundary (torch.classes / torch.ops registered
by libst_pybinding.so).  Same constructor and forward signatures as the
reference's example/RMSNorm.py:7-34 and example/RowParallelLinear.py:8-82; the
differences are stated per class."""
import torch
import torch.nn as nn

from . import _capi
from .layout import div_up, generate_row_mapping, reorder_indices, counter_size

_loaded = False


def load_library():
    """torch.ops.load_library of the shim (the reference does this at import of
    every script, example/RMSNorm.py:5); raises if it has not been built."""
    global _loaded
    if not _loaded:
        import os
        if not os.path.exists(_capi.SHIM_LIB):
            raise ImportError(f"{_capi.SHIM_LIB} is missing: run `python -m flashoverlap_amd.build`")
        torch.ops.load_library(_capi.SHIM_LIB)
        _loaded = True


class RMSNorm(nn.Module):
    """Torch reference RMSNorm: fp32 normalise -> cast -> multiply by the 16-bit
    weight (example/RMSNorm.py:7-18)."""

    def __init__(self, dim, eps=1e-5, dtype=torch.float16, device="cuda"):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.empty(dim, dtype=dtype, device=device).normal_(mean=0., std=0.5))

    def _norm(self, x):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps)

    def forward(self, x):
        return self._norm(x.float()).type_as(x) * self.weight


class ReorderRMSNorm(nn.Module):
    """Fused un-permute + RMSNorm (example/RMSNorm.py:20-34).  Unlike the
    reference, whose kernel ignores the stored eps and uses 1e-5
    (src/rmsnorm/rmsnorm.cuh:102), eps is passed to the kernel; the default
    keeps the kernel's 1e-5."""

    def __init__(self, dim, M, BM, BN, hint, eps=1e-5, dtype=torch.float16, device="cuda"):
        super().__init__()
        load_library()
        self.eps = eps
        self.weight = nn.Parameter(torch.empty(dim, dtype=dtype, device=device).normal_(mean=0., std=0.5))
        self.bm, self.bn = BM, BN
        tm, tn = div_up(M, BM), div_up(dim, BN)
        self.reorder_array = reorder_indices(tm * tn, hint, device=device).reshape((tm, tn))

    def forward(self, x):
        out = torch.empty_like(x)
        torch.ops.flashoverlap_op.reorder_rmsnorm_eps(x, out, self.weight, self.bm, self.bn, 1,
                                                      self.reorder_array, self.eps)
        return out


class RowParallelLayer(nn.Module):
    """Serial comparator: x @ W^T for this rank's K-slice
    (example/RowParallelLinear.py:8-30).  With one GPU the collective is the
    identity (all_reduce) or the selection of this rank's row chunk after the
    row shuffle (reduce_scatter); no process group is needed."""

    def __init__(self, in_features, out_features, comm_op, rank=0, world_size=1,
                 dtype=torch.float16, device="cuda"):
        super().__init__()
        assert comm_op in ["all_reduce", "reduce_scatter"], \
            f"comm_op must be 'all_reduce' or 'reduce_scatter', but got '{comm_op}'"
        self.comm_op, self.rank, self.world_size = comm_op, rank, world_size
        self.weight = nn.Parameter(torch.randn(out_features, in_features, dtype=dtype, device=device))

    def forward(self, x):
        out = torch.matmul(x, self.weight.t())
        if self.comm_op == "reduce_scatter":
            rows = out.size(0) // self.world_size
            return out[self.rank * rows:(self.rank + 1) * rows].contiguous()
        return out


class OverlapRowParallelLayer(nn.Module):
    """Signal GEMM + per-group consumer through torch.classes.flashoverlap_class.OverlapImpl
    (example/RowParallelLinear.py:32-82).  The counter buffer is sized by
    max(len(cSeg), TN) instead of TN (the reference overruns it when there are
    more groups than tile columns)."""

    def __init__(self, rank, world_size, in_features, out_features, M, config, comm_op, nccl_id,
                 dtype=torch.float16, device="cuda"):
        super().__init__()
        assert comm_op in ["all_reduce", "reduce_scatter"], \
            f"comm_op must be 'all_reduce' or 'reduce_scatter', but got '{comm_op}'"
        load_library()
        self.weight = nn.Parameter(torch.randn(out_features, in_features, dtype=dtype, device=device))
        self.world_size, self.comm_op, self.rank = world_size, comm_op, rank

        self.overlap_class = torch.classes.flashoverlap_class.OverlapImpl()
        self.overlap_class.nccl_init(rank, world_size, nccl_id)
        self.overlap_class.cutlass_init()
        self.overlap_class.overlap_init()

        BM, BN = config["BM"], config["BN"]
        hint, cseg = config["hint"], config["cSeg"]
        tm, tn = div_up(M, BM), div_up(out_features, BN)
        self.algo = config["Algo"]
        self.counter = torch.zeros((1, counter_size(len(cseg), tm, tn)), dtype=torch.int, device=device)
        self.reorder_array = reorder_indices(tm * tn, hint, device=device).reshape((tm, tn))
        self.cseg_cpu = torch.tensor(cseg, dtype=torch.int32)
        self.cseg_gpu = self.cseg_cpu.to(device)
        if comm_op == "reduce_scatter":
            self.row_array = generate_row_mapping(M, out_features, BM, BN, cseg, world_size, device=device)
        else:
            self.row_array = None

    def forward(self, x):
        n = self.weight.size(0)
        if self.comm_op == "all_reduce":
            out = torch.empty((x.size(0), n), dtype=x.dtype, device=x.device)
            self.overlap_class.gemm_allreduce_overlap(
                x, self.weight, out, self.counter, self.reorder_array, 1, self.cseg_cpu,
                self.cseg_gpu, self.algo, False)
        else:
            tmp = torch.empty((x.size(0), n), dtype=x.dtype, device=x.device)
            out = torch.empty((x.size(0) // self.world_size, n), dtype=x.dtype, device=x.device)
            self.overlap_class.gemm_reducescatter_overlap(
                x, self.weight, tmp, out, self.counter, self.reorder_array, self.row_array, 1,
                self.cseg_cpu, self.cseg_gpu, self.algo, False)
        return out
