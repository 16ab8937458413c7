"""Single-rank nn.Module wrappers with the shape of the reference's examples
(example/RowParallelLinear.py:10-85, example/RMSNorm.py:10-37): what a model
would instantiate in place of its row-parallel linear and the norm behind it.
"""
from __future__ import annotations

import torch
import torch.nn as nn

import flashoverlap_amd
from . import tiling


class RMSNorm(nn.Module):
    """Plain torch RMSNorm, the comparison layer of example/RMSNorm.py:10-21."""

    def __init__(self, dim: int, eps: float = 1e-5, dtype=torch.float16, device="cuda"):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.empty(dim, dtype=dtype, device=device).normal_(mean=0.0, std=0.5))

    def _norm(self, x):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps)

    def forward(self, x):
        return self._norm(x.float()).type_as(x) * self.weight


class ReorderRMSNorm(nn.Module):
    """Un-permutes the overlapped GEMM's output while normalising
    (example/RMSNorm.py:23-37).  Unlike the reference, eps is honoured."""

    def __init__(self, dim: int, M: int, BM: int, BN: int, hint, eps: float = 1e-5, dtype=torch.float16,
                 device="cuda"):
        super().__init__()
        flashoverlap_amd.load()
        self.eps = eps
        self.weight = nn.Parameter(torch.empty(dim, dtype=dtype, device=device).normal_(mean=0.0, std=0.5))
        self.bm, self.bn = BM, BN
        tm, tn = tiling.div_up(M, BM), tiling.div_up(dim, BN)
        self.reorder_array = tiling.reorder_indices(tm * tn, hint, device).reshape(tm, tn)

    def forward(self, x):
        out = torch.empty((x.size(0), x.size(1)), dtype=x.dtype, device=x.device)
        torch.ops.flashoverlap_op.reorder_rmsnorm_eps(x, out, self.weight, self.bm, self.bn, 1, self.reorder_array,
                                                      self.eps)
        return out


class RowParallelLayer(nn.Module):
    """torch matmul followed by the collective of a one-rank group, i.e. the
    identity (example/RowParallelLinear.py:10-33)."""

    def __init__(self, in_features: int, out_features: int, dtype=torch.float16, device="cuda"):
        super().__init__()
        self.weight = nn.Parameter(torch.randn(out_features, in_features, dtype=dtype, device=device))

    def forward(self, x):
        return torch.matmul(x, self.weight.t())


class OverlapRowParallelLayer(nn.Module):
    """The overlapped linear of example/RowParallelLinear.py:35-85 on one GPU.

    config: dict with BM, BN, Algo, hint, cSeg (flashoverlap_amd.config).
    all_reduce returns a fresh tile-permuted tensor (feed it to
    ReorderRMSNorm) that the caller owns, like `out` in the reference;
    reduce_scatter returns this rank's receive buffer [M/world_size, N]
    (normalise it with BM // world_size).
    """

    def __init__(self, rank: int, world_size: int, in_features: int, out_features: int, M: int, config: dict,
                 comm_op: str, mccl_id=None, dtype=torch.float16, device="cuda"):
        super().__init__()
        assert comm_op in ["all_reduce", "reduce_scatter"], \
            f"comm_op must be 'all_reduce' or 'reduce_scatter', but got '{comm_op}'"
        flashoverlap_amd.load()
        self.weight = nn.Parameter(torch.randn(out_features, in_features, dtype=dtype, device=device))
        self.world_size, self.comm_op = world_size, comm_op
        self.overlap_class = torch.classes.flashoverlap_class.OverlapImpl()
        self.overlap_class.mccl_init(rank, world_size, mccl_id or torch.ops.flashoverlap_op.generate_mccl_id())
        self.overlap_class.mutlass_init()
        self.overlap_class.overlap_init()
        BM, BN, cseg = config["BM"], config["BN"], config["cSeg"]
        tm, tn = tiling.div_up(M, BM), tiling.div_up(out_features, BN)
        self.algo = config["Algo"]
        self.counter = torch.zeros((1, max(tn, len(cseg))), dtype=torch.int, device=device)
        self.reorder_array = tiling.reorder_indices(tm * tn, config["hint"], device).reshape(tm, tn)
        self.cseg_cpu = torch.tensor(cseg, dtype=torch.int32)
        self.cseg_gpu = self.cseg_cpu.to(device)
        self.row_array = (tiling.generate_row_mapping(M, out_features, BM, BN, cseg, world_size, device)
                          if comm_op == "reduce_scatter" else None)

    def forward(self, x):
        n = self.weight.size(0)
        if self.comm_op == "all_reduce":
            # tmp receives the GEMM's tiles; the per-group copies (the collective's stand-in) land in out
            tmp = torch.empty((x.size(0), n), dtype=x.dtype, device=x.device)
            out = torch.empty((x.size(0), n), dtype=x.dtype, device=x.device)
            self.overlap_class.set_staging(out)
            self.overlap_class.gemm_allreduce_overlap(x, self.weight, tmp, self.counter, self.reorder_array, 1,
                                                      self.cseg_cpu, self.cseg_gpu, self.algo, False)
            return out
        tmp = torch.empty((x.size(0), n), dtype=x.dtype, device=x.device)
        out = torch.empty((x.size(0) // self.world_size, n), dtype=x.dtype, device=x.device)
        self.overlap_class.gemm_reducescatter_overlap(x, self.weight, tmp, out, self.counter, self.reorder_array,
                                                      self.row_array, 1, self.cseg_cpu, self.cseg_gpu, self.algo,
                                                      False)
        return out
