"""The reference's two correctness examples on one MI355X
(example/correctness_ar.py:77-127, example/correctness_rs.py:78-142).

  python -m flashoverlap_amd.correctness --comm_op all_reduce     --m_dim 4096 --n_dim 4096 --k_dim 8192
  python -m flashoverlap_amd.correctness --comm_op reduce_scatter --m_dim 4096 --n_dim 4096 --k_dim 8192 --world_size 8

Builds the plain row-parallel linear + RMSNorm and the overlapped linear +
ReorderRMSNorm from the shape's tuning file (configs/m{M}n{N}k{K}_{gpu}.json, or
a default record if there is none), runs both on the same input and prints the
reference's result lines: all-ones operands and allclose(1e-2, 1e-2) for
all_reduce, N(0, 0.5) operands, the element of largest difference and
allclose(5e-2, 5e-2) for reduce_scatter.  With one GPU the collective of the
plain layer is the identity and --world_size only selects the ReduceScatter
slicing one rank of that world would see (--rank picks which).
"""
from __future__ import annotations

import argparse
import os
import sys

import torch
import torch.nn as nn

from . import config, layers, load, speed_test, tiling


def build_config(M, N, K, dtype, root="configs"):
    path = config.find_config(M, N, K, config.current_gpu_tags(), root)
    if os.path.exists(path):
        return config.load_config(path, M, N)
    return speed_test.default_config(M, N, K, 1, dtype, "cuda", warm_up=2, rep=5)


def run(comm_op: str, M: int, N: int, K: int, cfg: dict, world_size: int = 1, rank: int = 0, dtype=torch.float16,
        out=print) -> bool:
    """Returns the reference's `all_close`."""
    load()
    dev = "cuda"
    W = torch.ones((N,), dtype=dtype, device=dev).normal_(mean=0.0, std=0.5)
    norm = layers.RMSNorm(N, dtype=dtype, device=dev)
    norm.weight = nn.Parameter(W)
    lin = layers.RowParallelLayer(K, N, dtype=dtype, device=dev)
    olin = layers.OverlapRowParallelLayer(rank, world_size, K, N, M, cfg, comm_op, dtype=dtype, device=dev)
    if comm_op == "all_reduce":
        A = torch.ones((M, K), dtype=dtype, device=dev)
        B = torch.ones((N, K), dtype=dtype, device=dev)
        rnorm = layers.ReorderRMSNorm(N, M, cfg["BM"], cfg["BN"], cfg["hint"], dtype=dtype, device=dev)
    else:
        if M % world_size or cfg["BM"] % world_size:
            raise ValueError(f"reduce_scatter: M={M} and BM={cfg['BM']} must be multiples of world_size={world_size}")
        A = torch.ones((M, K), dtype=dtype, device=dev).normal_(mean=0.0, std=0.5)
        B = torch.ones((N, K), dtype=dtype, device=dev).normal_(mean=0.0, std=0.5)
        rnorm = layers.ReorderRMSNorm(N, M // world_size, cfg["BM"] // world_size, cfg["BN"], cfg["hint"], dtype=dtype,
                                      device=dev)
    rnorm.weight = nn.Parameter(W)
    lin.weight = nn.Parameter(B)
    olin.weight = nn.Parameter(B)
    torch.cuda.synchronize()
    with torch.no_grad():
        if comm_op == "all_reduce":
            x1 = lin(A)
        else:   # the rows a rank receives are those with row % world_size == rank, in order
            x1 = lin(tiling.reorder_rows_by_world_size(A, world_size)).view(world_size, M // world_size, N)[rank]
        x2 = olin(A)
        y1, y2 = norm(x1), rnorm(x2)
    torch.cuda.synchronize()
    expired = olin.overlap_class.wait_timeouts(True)
    if expired:
        out(f"{expired} bounded wait(s) expired: cSeg does not match the tiles, or the wait timeout is too short")
    if comm_op == "all_reduce":
        ok = torch.allclose(y1, y2, atol=1e-2, rtol=1e-2) and expired == 0
        out(f"[GEMM+AllReduce+RMSNorm] all close :  {ok}")
        return ok
    diff = torch.abs(y1 - y2)
    at = torch.unravel_index(torch.argmax(diff), diff.shape)
    out(f"Index of max absolute difference: {tuple(int(i) for i in at)}")
    out(f"Value in y1 at that index: {y1[at].item()}")
    out(f"Value in y2 at that index: {y2[at].item()}")
    out(f"Absolute difference: {diff[at].item()}")
    ok = torch.allclose(y1, y2, atol=5e-2, rtol=5e-2) and expired == 0
    out(f"[GEMM+ReduceScatter+RMSNorm] all close :  {ok}")
    return ok


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--m_dim", type=int, default=4096)
    ap.add_argument("--k_dim", type=int, default=8192)
    ap.add_argument("--n_dim", type=int, default=4096)
    ap.add_argument("--comm_op", default="all_reduce", choices=["all_reduce", "reduce_scatter"])
    ap.add_argument("--world_size", type=int, default=1)
    ap.add_argument("--rank", type=int, default=0)
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    ap.add_argument("--configs", default="configs", help="directory of the tuning files")
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("correctness: no GPU visible", file=sys.stderr)
        return 2
    if not 0 <= a.rank < a.world_size:
        ap.error(f"--rank {a.rank} outside 0..{a.world_size - 1}")
    load()
    dtype = getattr(torch, a.dtype)
    cfg = build_config(a.m_dim, a.n_dim, a.k_dim, dtype, a.configs)
    return 0 if run(a.comm_op, a.m_dim, a.n_dim, a.k_dim, cfg, a.world_size, a.rank, dtype) else 1


if __name__ == "__main__":
    sys.exit(main())
