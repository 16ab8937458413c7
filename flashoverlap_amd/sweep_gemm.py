"""M/N/K sweep of this library's plain GEMM against the vendor library, the table of the
reference's test/sweep_gemm.py, through the torch API only.

For every (M, N, K): BaselineImpl.mublas_gemm once, OverlapImpl.mutlass_gemm under every Algo,
the fastest Algo kept (the plain GEMM takes any M and N, so no Algo drops out for its tile); columns `M N K Algo muBLAS(ms)
MUTlass(ms) ratio note` with the reference's notes (ratio <= 1.1 "<== CLOSE", <= 1.3 "<= OK")
and its closing list of the ten closest shapes (test/sweep_gemm.py:93-140).  Same protocol as
the speed table: 20 warm-up and 200 timed launches with an event pair each.

  python -m flashoverlap_amd.sweep_gemm
  python -m flashoverlap_amd.sweep_gemm --k_dim 8192
  python -m flashoverlap_amd.sweep_gemm --m_list 1024 2048 4096 8192 --n_list 1024 2048 4096 8192
"""
from __future__ import annotations

import argparse
import sys

import torch

from . import capi, load, speed_test


def note_for(ratio: float) -> str:
    """test/sweep_gemm.py:121-125."""
    if ratio <= 1.1:
        return "<== CLOSE"
    if ratio <= 1.3:
        return "<= OK"
    return ""


def format_row(M, N, K, algo, vendor_ms, ours_ms) -> str:
    if ours_ms is None:
        return f"{M:>6} {N:>6} {K:>6} {'FAIL':>4}  {vendor_ms:>10.4f} {'N/A':>11} {'N/A':>6}  {'':>10}"
    ratio = ours_ms / vendor_ms
    return f"{M:>6} {N:>6} {K:>6} {algo:>4}  {vendor_ms:>10.4f} {ours_ms:>11.4f} {ratio:>6.2f}  {note_for(ratio):>10}"


HEADER = f"{'M':>6} {'N':>6} {'K':>6} {'Algo':>4}  {'muBLAS(ms)':>10} {'MUTlass(ms)':>11} {'ratio':>6}  {'note':>10}"


def bench_shape(M, N, K, dtype=torch.float16, algos=None, **kw):
    """(vendor ms, best ms or None, best Algo or -1)."""
    vendor = speed_test.perf_mublas_gemm(M, N, K, dtype, "cuda", **kw)
    best, best_algo = None, -1
    for algo in (range(capi.lib().fo_algo_count()) if algos is None else algos):
        try:
            t = speed_test.perf_mutlass_gemm(M, N, K, algo, dtype, "cuda", **kw)
        except RuntimeError:    # a shape the GEMM refuses (K not a multiple of 8) is a failed row, test/sweep_gemm.py:65-66
            continue
        if best is None or t < best:
            best, best_algo = t, algo
    return vendor, best, best_algo


def sweep(m_list, n_list, k_list, dtype=torch.float16, algos=None, out=print, **kw):
    load()
    out(HEADER)
    out("-" * 78)
    results = []
    for K in k_list:
        for M in m_list:
            for N in n_list:
                vendor, ours, algo = bench_shape(M, N, K, dtype, algos, **kw)
                out(format_row(M, N, K, algo, vendor, ours))
                if ours is not None:
                    results.append((M, N, K, algo, vendor, ours, ours / vendor))
    if results:
        out("\n--- Top 10 closest (MUTlass/muBLAS ratio) ---")
        out(f"{'M':>6} {'N':>6} {'K':>6} {'Algo':>4}  {'muBLAS(ms)':>10} {'MUTlass(ms)':>11} {'ratio':>6}")
        for M, N, K, algo, vendor, ours, ratio in sorted(results, key=lambda r: r[6])[:10]:
            out(f"{M:>6} {N:>6} {K:>6} {algo:>4}  {vendor:>10.4f} {ours:>11.4f} {ratio:>6.2f}")
    return results


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--m_list", type=int, nargs="+", default=[1024, 2048, 4096, 8192, 16384])
    ap.add_argument("--n_list", type=int, nargs="+", default=[1024, 2048, 4096, 8192, 16384])
    ap.add_argument("--k_dim", type=int, default=None, help="fixed K; if not set, K sweeps the M list")
    ap.add_argument("--k_list", type=int, nargs="+", default=None, help="explicit K list to sweep")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    ap.add_argument("--algos", type=int, nargs="+", default=None,
                    help="Algos to try (default all; they share one compute kernel and differ in the layout tile)")
    ap.add_argument("--rep", type=int, default=speed_test.REP)
    ap.add_argument("--warm_up", type=int, default=speed_test.WARM_UP)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("sweep_gemm: no GPU visible", file=sys.stderr)
        return 2
    k_list = a.k_list if a.k_list else [a.k_dim] if a.k_dim else a.m_list
    sweep(a.m_list, a.n_list, k_list, getattr(torch, a.dtype), a.algos,
          out=lambda s: print(s, flush=True), warm_up=a.warm_up, rep=a.rep)
    return 0


if __name__ == "__main__":
    sys.exit(main())
