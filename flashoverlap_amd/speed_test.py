"""Speed table of the reference's test/test.py on one MI355X, through the torch API only.

Same measurements, same protocol (test/test.py:26-27, 120-331): 20 warm-up and
200 timed iterations, one event pair per iteration, mean over the iterations,
for
  mublas_gemm   BaselineImpl.mublas_gemm                  (library GEMM, test.py:304-331)
  mccl_comm     OverlapImpl.mccl_allreduce / _reducescatter (bulk collective, :209-249)
  baseline      BaselineImpl.gemm_allreduce / gemm_reducescatter (:251-302)
  overlap       OverlapImpl.gemm_allreduce_overlap / gemm_reducescatter_overlap,
                or the non-overlapped gemm_allreduce when cSeg has one entry (:120-207)
and the table `mutlass_gemm | mublas_gemm | mccl_comm | baseline | overlap |
speedup` of test.py:374-389.  On one GPU the collective is the consumer copy, so
`mccl_comm` is a bulk device copy and `speedup` compares GEMM-then-copy with
GEMM-overlapped-with-per-group-copies.

The shape's tuning file is read like the reference does
(configs/m{M}n{N}k{K}_{gpu}.json, keys BM BN dur Algo hint cSeg rLDN); if there
is none, one is made from this library's known issue order (tiling.raster_hint),
one hardware wave per group, and a measured `dur`, and written with --save.

  python -m flashoverlap_amd.speed_test --m_dim 8192 --n_dim 4096 --k_dim 7168 --comm_op all_reduce
"""
from __future__ import annotations

import argparse
import os
import sys
import time

import torch

from . import capi, config, load, tiling

WARM_UP = 20
REP = 200
TILES_PER_WAVE_256 = 256   # workgroups resident at a time: one 256x256 macro tile per CU


WARM_UP_MS = 60.0   # the warm-up also lasts at least this long


def _timed(fn, warm_up=WARM_UP, rep=REP):
    """Mean milliseconds of fn() over `rep` iterations, one event pair each (test/test.py:157-164).
    The warm-up is the reference's 20 iterations and, beyond it, as many more as it takes to keep
    the GPU busy for WARM_UP_MS: a column measured right after a light one (the GEMM rows after the
    copy row) otherwise starts on a chip that has clocked down and reads 2-3 % slow."""
    for _ in range(warm_up):
        fn()
    if warm_up >= WARM_UP:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1000.0 < WARM_UP_MS:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
    start = [torch.cuda.Event(enable_timing=True) for _ in range(rep)]
    end = [torch.cuda.Event(enable_timing=True) for _ in range(rep)]
    for i in range(rep):
        start[i].record()
        fn()
        end[i].record()
    torch.cuda.synchronize()
    return sum(s.elapsed_time(e) for s, e in zip(start, end)) / rep


def _operands(M, N, K, dtype, device):
    A = torch.empty((M, K), dtype=dtype, device=device).normal_(mean=0.0, std=0.5)
    B = torch.empty((N, K), dtype=dtype, device=device).normal_(mean=0.0, std=0.5)
    C = torch.empty((M, N), dtype=dtype, device=device)
    return A, B, C


def _overlap_object(rank=0, world_size=1):
    o = torch.classes.flashoverlap_class.OverlapImpl()
    o.mccl_init(rank, world_size, torch.ops.flashoverlap_op.generate_mccl_id())
    o.mutlass_init()
    o.overlap_init()
    return o


def perf_mublas_gemm(M, N, K, dtype=torch.float16, device="cuda", **kw):
    """test/test.py:304-331."""
    A, B, C = _operands(M, N, K, dtype, device)
    b = torch.classes.flashoverlap_class.BaselineImpl()
    b.mublas_init()
    return _timed(lambda: b.mublas_gemm(A, B, C), **kw)


def perf_mutlass_gemm(M, N, K, Algo, dtype=torch.float16, device="cuda", **kw):
    """The `dur` the reference's GEMM profiler stores in the tuning file (tune/profile_config.py:59-74)."""
    A, B, C = _operands(M, N, K, dtype, device)
    o = _overlap_object()
    return _timed(lambda: o.mutlass_gemm(A, B, C, Algo), **kw)


def perf_comm(M, N, comm_type, world_size=1, dtype=torch.float16, device="cuda", **kw):
    """test/test.py:209-249."""
    o = _overlap_object(0, world_size)
    C = torch.empty((M, N), dtype=dtype, device=device)
    if comm_type == "all_reduce":
        return _timed(lambda: o.mccl_allreduce(C), **kw)
    if comm_type == "reduce_scatter":
        return _timed(lambda: o.mccl_reducescatter(C), **kw)
    return 0.0


def perf_baseline(M, N, K, comm_op, world_size=1, dtype=torch.float16, device="cuda", **kw):
    """test/test.py:251-302."""
    A, B, C = _operands(M, N, K, dtype, device)
    b = torch.classes.flashoverlap_class.BaselineImpl()
    b.mccl_init(0, world_size, torch.ops.flashoverlap_op.generate_mccl_id())
    b.mublas_init()
    if comm_op == "all_reduce":
        return _timed(lambda: b.gemm_allreduce(A, B, C), **kw)
    if comm_op == "reduce_scatter":
        D = torch.empty((M // world_size, N), dtype=dtype, device=device)
        return _timed(lambda: b.gemm_reducescatter(A, B, C, D), **kw)
    return 0.0


def perf_running(M, N, K, BM, BN, Algo, cSeg, hint, comm_op, world_size=1, dtype=torch.float16, device="cuda",
                 keep=None, **kw):
    """test/test.py:120-207.  `keep`, if a dict, receives the operands and outputs of the last
    iteration (for checking them)."""
    cSeg_CPU = torch.tensor(cSeg, dtype=torch.int32)
    cSeg_GPU = cSeg_CPU.to(device)
    TM, TN = tiling.div_up(M, BM), tiling.div_up(N, BN)
    tile_num = TM * TN
    o = _overlap_object(0, world_size)
    A, B, C = _operands(M, N, K, dtype, device)
    # one counter per group (the reference allocates TN, too few for many small groups)
    counters = torch.zeros(max(TN, len(cSeg)), dtype=torch.int32, device=device)
    RA = tiling.reorder_indices(tile_num, hint, device).reshape(TM, TN)
    D = RE = None
    if comm_op == "reduce_scatter":
        D = torch.empty((M // world_size, N), dtype=dtype, device=device)
        RE = tiling.generate_row_remap_array(M, N, BM, BN, cSeg, world_size, device)
    if len(cSeg) == 1:  # no overlapping
        if comm_op == "all_reduce":
            fn = lambda: o.gemm_allreduce(A, B, C, Algo)
        else:
            fn = lambda: o.gemm_reducescatter(A, B, C, D, Algo)
    elif comm_op == "all_reduce":
        fn = lambda: o.gemm_allreduce_overlap(A, B, C, counters, RA, 1, cSeg_CPU, cSeg_GPU, Algo, False)
    else:
        fn = lambda: o.gemm_reducescatter_overlap(A, B, C, D, counters, RA, RE, 1, cSeg_CPU, cSeg_GPU, Algo, False)
    dur = _timed(fn, **kw)
    if keep is not None:
        # host time to enqueue one call (nothing is waited for): what the torch-API path costs the CPU
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            fn()
        host_us = (time.perf_counter() - t0) / 20 * 1e6
        torch.cuda.synchronize()
        keep.update(A=A, B=B, C=C, D=D, RA=RA, RE=RE, counters=counters, overlap=o, host_us_per_call=host_us)
    return dur


def sustained_gemm(M, N, K, Algo=1, dtype=torch.float16, device="cuda", seconds=3.0, zeros=False):
    """Both GEMMs in a loop of `seconds` each (launches are queued 200 at a time), with the core clock
    sampled from rocm-smi while they run: what the chip sustains once its power management has
    settled, as opposed to the bursts of a few milliseconds that the table times.  zeros=True runs
    the same kernels on all-zero operands, which toggle nothing in the MFMA datapath.
    Returns {name: (us_per_launch, [sclk MHz samples])}."""
    import re
    import shutil
    import subprocess
    import threading
    import time
    A, B, C = _operands(M, N, K, dtype, device)
    if zeros:
        A.zero_()
        B.zero_()
    o = _overlap_object()
    b = torch.classes.flashoverlap_class.BaselineImpl()
    b.mublas_init()
    smi = shutil.which("rocm-smi")
    out = {}
    for name, fn in (("mutlass_gemm", lambda: o.mutlass_gemm(A, B, C, Algo)), ("mublas_gemm", lambda: b.mublas_gemm(A, B, C))):
        clocks, stop = [], threading.Event()

        def sample():
            while smi and not stop.is_set():
                try:
                    txt = subprocess.run([smi, "--showclocks"], capture_output=True, text=True, timeout=5).stdout
                    m = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", txt)
                    if m:
                        clocks.append(int(m.group(1)))
                except Exception:
                    pass
                stop.wait(0.25)
        th = threading.Thread(target=sample)
        th.start()
        t0, n = time.perf_counter(), 0
        while time.perf_counter() - t0 < seconds:
            for _ in range(200):
                fn()
            torch.cuda.synchronize()
            n += 200
        dt = time.perf_counter() - t0
        stop.set()
        th.join()
        out[name] = (dt / n * 1e6, clocks)
    return out


def default_config(M, N, K, Algo=1, dtype=torch.float16, device="cuda", **kw):
    """A tuning record for a shape that has no file: this library's issue order as the hint, one
    hardware wave (256 macro tiles) per group, the measured plain-GEMM time as `dur`."""
    BM, BN, _ = capi.algo_tile(Algo)
    tile_num = (M // BM) * (N // BN)
    per_wave = TILES_PER_WAVE_256 * (256 // BM) * (256 // BN)
    return {"BM": BM, "BN": BN, "Algo": Algo, "rLDN": 1, "hint": tiling.raster_hint(M, N, Algo),
            "cSeg": tiling.uniform_cseg(tile_num, per_wave),
            "dur": perf_mutlass_gemm(M, N, K, Algo, dtype, device, **kw)}


def speed_table(M, N, K, comm_op="all_reduce", cfg=None, world_size=1, dtype=torch.float16, device="cuda",
                single_seg=False, keep=None, **kw):
    """The rows of test/test.py:374-389 as a dict (milliseconds)."""
    load()
    if cfg is None:
        cfg = default_config(M, N, K, 1, dtype, device, **kw)
    data = dict(cfg)
    tile_num = (M // data["BM"]) * (N // data["BN"])
    if single_seg:
        data["cSeg"] = [tile_num]
        data["hint"] = list(range(tile_num))
    mublas = perf_mublas_gemm(M, N, K, dtype, device, **kw)
    comm = perf_comm(M, N, comm_op, world_size, dtype, device, **kw)
    keep = {} if keep is None else keep
    overlap = perf_running(M, N, K, data["BM"], data["BN"], data["Algo"], data["cSeg"], data["hint"], comm_op,
                           world_size, dtype, device, keep=keep, **kw)
    baseline = perf_baseline(M, N, K, comm_op, world_size, dtype, device, **kw)
    return {"m": M, "n": N, "k": K, "tile_num": tile_num, "cSeg": list(data["cSeg"]), "num_segs": len(data["cSeg"]),
            "mutlass_gemm": float(data["dur"]), "mublas_gemm": mublas, "mccl_comm": comm, "baseline": baseline,
            "overlap": overlap, "speedup": baseline / overlap, "overlap_host_us": keep["host_us_per_call"]}


def format_table(t) -> str:
    rows = [("m", t["m"]), ("n", t["n"]), ("k", t["k"]), ("tile_num", t["tile_num"]),
            ("cSeg", str(t["cSeg"]) if len(t["cSeg"]) <= 8 else f"{t['cSeg'][:3]}... x{len(t['cSeg'])}"),
            ("num_segs", t["num_segs"])]
    out = [f"{'Item':<25} {'Value':>15}", f"{'-----':<25} {'-----':>15}"]
    out += [f"{k:<25} {v!s:>15}" for k, v in rows]
    for key, label in (("mutlass_gemm", "mutlass_gemm (ms)"), ("mublas_gemm", "mublas_gemm (ms)"),
                       ("mccl_comm", "mccl_comm (ms)"), ("baseline", "baseline (mublas+mccl)"),
                       ("overlap", "overlap (mutlass+mccl)"), ("speedup", "speedup")):
        out.append(f"{label:<25} {t[key]:>15.4f}")
    out.append(f"{'overlap host enqueue (us)':<25} {t['overlap_host_us']:>15.1f}")
    return "\n".join(out)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--m_dim", type=int, default=4096)
    ap.add_argument("--k_dim", type=int, default=8192)
    ap.add_argument("--n_dim", type=int, default=8192)
    ap.add_argument("--comm_op", type=str, default="all_reduce", choices=["all_reduce", "reduce_scatter"])
    ap.add_argument("--single_seg", action="store_true", help="one segment: no overlap (GEMM, then the bulk copy)")
    ap.add_argument("--world_size", type=int, default=1, help="emulated world size of the ReduceScatter slicing")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    ap.add_argument("--configs", default="configs", help="directory of the per-shape tuning files")
    ap.add_argument("--save", action="store_true", help="write the tuning file if the shape has none")
    ap.add_argument("--sustained", type=float, default=0.0,
                    help="also loop each GEMM for this many seconds (random, then all-zero operands) and report "
                         "the sustained time per launch and the core clock")
    ap.add_argument("--rep", type=int, default=REP)
    ap.add_argument("--warm_up", type=int, default=WARM_UP)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("speed_test: no GPU visible", file=sys.stderr)
        return 2
    load()
    dtype = getattr(torch, a.dtype)
    m, n, k = a.m_dim, a.n_dim, a.k_dim
    path = config.find_config(m, n, k, config.current_gpu_tags(), a.configs)
    kw = {"warm_up": a.warm_up, "rep": a.rep}
    if os.path.exists(path):
        cfg = config.load_config(path, m, n)
    else:
        cfg = default_config(m, n, k, 1, dtype, "cuda", **kw)
        if a.save:
            config.save_solution(path, cfg["BM"], cfg["BN"], cfg["dur"], cfg["Algo"], cfg["hint"], cfg["cSeg"], 1)
    t = speed_table(m, n, k, a.comm_op, cfg, a.world_size, dtype, "cuda", a.single_seg, **kw)
    print(format_table(t))
    if a.sustained > 0:
        flops = 2.0 * m * n * k
        for zeros in (False, True):
            r = sustained_gemm(m, n, k, cfg["Algo"], dtype, "cuda", a.sustained, zeros)
            for name, (us, clocks) in r.items():
                print(f"sustained {a.sustained:.0f} s, {'zero' if zeros else 'random'} operands: {name:<13} {us:8.1f} us "
                      f"{flops / us / 1e6:7.1f} TFLOP/s  sclk MHz {clocks[2:] if len(clocks) > 4 else clocks}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
