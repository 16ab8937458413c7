#!/usr/bin/env python3
"""Benchmark of the single-GPU hot path on one MI355X.

A step is one pass of the path over one synthetic batch, inputs resident in HBM:
signalling GEMM on the caller's stream, on a second stream a wait kernel and a
consumer copy per group (or one persistent wait+consume kernel) releasing each
finished group into the staging buffer, an event join, then reorder+RMSNorm on
the staging buffer.

Prints ONE JSON line.  `value` is 2*M*N*K divided by the whole step time.  The
roofline object is for the dominant kernel (the signalling GEMM) as it ran
inside the timed steps, from HIP events around every launch on its own stream.
The same run also times, back to back and on their own, the signalling GEMM
and its plain twin (signal overhead), reorder+RMSNorm (HBM roofline) and the
consumer copy, the serial (non-overlapped) step, and a CPU baseline (the
oracle's fp32 matmul + RMSNorm on the host cores) on a bounded sample of the
same workload.  Launch order: W+K serial steps, W+K overlapped steps, then the
isolated kernels (5 warm-up + --kernel-iters + 10 launches each).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# The five benchmark configurations; (dtype, M, N, K, tiles per group, world size, eps, a_std, b_std).  A hardware
# wave of the GEMM kernel is 256 workgroups x 4 layout tiles = 1024 tiles of 128x128 (W); the tiles of
# one wave finish together, so groups are whole waves: c3 one wave per group, c4 two ("group size 2").
# c1 and c2 fit in one wave and keep the tile-count reading of their group sizes (4 and 256 tiles).
TILES_PER_WAVE = 1024
WORKLOADS = {
    "c1": ("fp16", 1024, 1024, 1024, 4, 1, 1e-6, None, None),
    "c2": ("fp16", 4096, 4096, 4096, 256, 1, 1e-5, None, None),
    "c3": ("bf16", 8192, 4096, 7168, TILES_PER_WAVE, 1, 1e-5, 1.0, 0.02),
    "c4": ("bf16", 16384, 8192, 1024, 2 * TILES_PER_WAVE, 1, 1e-5, None, None),
    "c5": ("bf16", 8192, 8192, 3584, TILES_PER_WAVE, 8, 1e-5, None, None),
}
NAMES = {
    "c1": "fp16 1024^3 plumbing shape",
    "c2": "fp16 4096^3 square GEMM",
    "c3": "Llama-3-8B down_proj share, bf16 8192x4096x7168",
    "c4": "Llama-3-70B o_proj share, bf16 16384x8192x1024",
    "c5": "Llama-3-70B down_proj share, ReduceScatter layout, bf16 8192x8192x3584",
}
PEAK_MFMA_TFLOPS = 2516.6   # MI355X dense fp16/bf16: 256 CU x 4096 FLOP/clk x 2.4 GHz
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E
# Bytes that cross the L2 -> memory interface per signalling-GEMM launch, from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of `bench.py --no-overlap` (profiles/gemm_signal_c3_counters.txt):
# FETCH_SIZE 344245 KiB x 1.999 (the 64 MiB consumer copy reads as 32786.5 KiB) + WRITE_SIZE 65600 KiB
# x 1.000.  None for workloads that have not been measured.
MEASURED_TRAFFIC_BYTES = {"c3": 771_800_000}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--group-tiles", type=int, default=0, help="tiles per signal group (0 = workload default)")
    ap.add_argument("--kernel-iters", type=int, default=100, help="timed launches per isolated kernel")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU-baseline work; 0 skips it")
    ap.add_argument("--consumer-blocks", type=int, default=64, help="workgroups of the persistent consumer")
    ap.add_argument("--consumer", default="auto", choices=["auto", "per_group", "persistent"])
    ap.add_argument("--no-overlap", action="store_true",
                    help="order the consumer behind the GEMM in the timed step (needed under counter collection, "
                         "which runs one kernel at a time)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build drives one GPU only; run with --gpus 1 "
              "(no collective, IPC or multi-rank code exists in this tree)", file=sys.stderr)
        return 2

    import torch
    from flashoverlap_amd import capi, tiling

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    L = capi.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    dts, M, N, K, w, ws, eps, a_std, b_std = WORKLOADS[a.workload]
    if a.group_tiles:
        w = a.group_tiles
    dt = torch.float16 if dts == "fp16" else torch.bfloat16
    code = capi.dtype_code(dt)
    algo = 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    cseg = tiling.uniform_cseg(T, w)
    G = len(cseg)

    # synthetic inputs: generated on the CPU with a fixed seed, cast, uploaded
    torch.manual_seed(0)
    sa = a_std if a_std is not None else 1.0 / K ** 0.5
    sb = b_std if b_std is not None else 1.0 / K ** 0.5
    A_h = (torch.randn(M, K) * sa).to(dt)
    B_h = (torch.randn(N, K) * sb).to(dt)
    g_h = (1 + 0.1 * torch.randn(N)).to(dt)
    A, B, gamma = A_h.to(dev), B_h.to(dev), g_h.to(dev)
    Cp = torch.empty(M * N, dtype=dt, device=dev)
    Cn = torch.empty(M, N, dtype=dt, device=dev)
    staging = torch.zeros(M * N, dtype=dt, device=dev)
    out = torch.empty(M, N, dtype=dt, device=dev)
    hint = tiling.raster_hint(M, N, algo)
    RA = tiling.reorder_indices(T, hint, dev).reshape(TM, TN)
    RE = tiling.generate_row_remap_array(M, N, BM, BN, cseg, ws, dev) if ws > 1 else None
    cseg_d = torch.tensor(cseg, dtype=torch.int32, device=dev)
    MM = torch.zeros(max(G, TN), dtype=torch.int32, device=dev)
    table = torch.empty(T, dtype=torch.int32, device=dev)
    capi.check(L.fo_build_group_table(cseg_d.data_ptr(), G, T, table.data_ptr(), None))
    comm = C.c_void_p()
    capi.check(L.fo_stream_create(C.byref(comm)))
    capi.check(L.fo_set_wait_timeout_ms(10000))
    main_stream = None  # the null stream; all launches of the main leg go there

    def gemm_signal():
        if ws > 1:
            capi.check(L.fo_gemm_scatter(code, algo, M, N, K, 1, cseg_d.data_ptr(), G, table.data_ptr(), A.data_ptr(),
                                         B.data_ptr(), Cp.data_ptr(), MM.data_ptr(), RA.data_ptr(), RE.data_ptr(), 0,
                                         main_stream))
        else:
            capi.check(L.fo_gemm_signal(code, algo, M, N, K, 1, cseg_d.data_ptr(), G, table.data_ptr(), A.data_ptr(),
                                        B.data_ptr(), Cp.data_ptr(), MM.data_ptr(), RA.data_ptr(), 0, main_stream))

    def gemm_plain():
        capi.check(L.fo_gemm(code, algo, M, N, K, A.data_ptr(), B.data_ptr(), Cn.data_ptr(), main_stream))

    # Same rule as OverlapImpl: up to 32 groups the reference's structure (one wait kernel and one
    # consumer launch per group, src/overlap_impl.cu:257-265), beyond that one persistent kernel.
    per_group = a.consumer == "per_group" or (a.consumer == "auto" and G <= 32)

    def wait_consume():
        if not per_group:
            capi.check(L.fo_wait_consume(cseg_d.data_ptr(), G, MM.data_ptr(), Cp.data_ptr(), staging.data_ptr(),
                                         BM * BN, ws, 0, ws, (M * N // ws) if ws > 1 else 0, None,
                                         a.consumer_blocks, comm))
            return
        acc = 0
        for g, n in enumerate(cseg):
            capi.check(L.fo_wait(n, MM.data_ptr() + 4 * g, comm))
            elems = n * BM * BN
            part = elems // ws
            for k in range(ws):  # ws > 1: slice k of the group goes to rank k's receive buffer
                capi.check(L.fo_consume(Cp.data_ptr() + 2 * (acc + k * part),
                                        staging.data_ptr() + 2 * (k * (M * N // ws) + acc // ws), 2 * part, comm))
            acc += elems

    def norm():
        if ws > 1:  # every rank slice is a layout with tile height BM/ws: ws problems, one launch
            capi.check(L.fo_reorder_rmsnorm_batched(code, staging.data_ptr(), gamma.data_ptr(), out.data_ptr(), ws,
                                                    M // ws, N, BM // ws, BN, 1, RA.data_ptr(), eps, main_stream))
        else:
            capi.check(L.fo_reorder_rmsnorm(code, staging.data_ptr(), gamma.data_ptr(), out.data_ptr(), M, N, BM, BN,
                                            1, RA.data_ptr(), eps, main_stream))

    def step(overlap=True, ev=None):
        if ev:
            capi.check(L.fo_event_record(ev[0], main_stream))
        gemm_signal()
        if ev:
            capi.check(L.fo_event_record(ev[1], main_stream))
        if not overlap:  # consumer ordered behind the GEMM: the serial reference for the overlap
            capi.check(L.fo_stream_join(main_stream, comm))
        wait_consume()
        capi.check(L.fo_stream_join(comm, main_stream))
        norm()

    def time_steps(overlap):
        """Wall time per step, and the signalling GEMM's own duration inside those same
        steps (one HIP event pair per step on the GEMM's stream)."""
        evs = []
        for _ in range(a.steps):
            e0, e1 = C.c_void_p(), C.c_void_p()
            capi.check(L.fo_event_create(C.byref(e0)))
            capi.check(L.fo_event_create(C.byref(e1)))
            evs.append((e0, e1))
        for _ in range(a.warmup):
            step(overlap)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for ev in evs:
            step(overlap, ev)
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / a.steps
        v, tot = C.c_float(), 0.0
        for e0, e1 in evs:
            capi.check(L.fo_event_elapsed_ms(e0, e1, C.byref(v)))
            tot += v.value
            capi.check(L.fo_event_destroy(e0))
            capi.check(L.fo_event_destroy(e1))
        return wall, tot / a.steps

    # ---- whole path: W warm-up steps, then exactly K timed steps -----------------
    serial_ms, serial_gemm_ms = time_steps(False)
    step_ms, step_gemm_ms = (serial_ms, serial_gemm_ms) if a.no_overlap else time_steps(True)
    timeouts = C.c_int()
    capi.check(L.fo_wait_timeouts(C.byref(timeouts), 1))
    if timeouts.value:
        print(f"bench.py: {timeouts.value} bounded waits expired; results invalid", file=sys.stderr)
        return 1

    # ---- isolated kernels, HIP events on the launch stream -----------------------
    def time_kernel(fn, iters):
        """Average launch duration: `iters` back-to-back launches between one HIP event pair on
        the launch stream (what a kernel trace reports as the kernel's average), and the
        shortest single launch out of 10 individually bracketed ones."""
        e0, e1 = C.c_void_p(), C.c_void_p()
        capi.check(L.fo_event_create(C.byref(e0)))
        capi.check(L.fo_event_create(C.byref(e1)))
        v = C.c_float()
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        capi.check(L.fo_event_record(e0, main_stream))
        for _ in range(iters):
            fn()
        capi.check(L.fo_event_record(e1, main_stream))
        torch.cuda.synchronize()
        capi.check(L.fo_event_elapsed_ms(e0, e1, C.byref(v)))
        avg = v.value / iters
        best = float("inf")
        for _ in range(10):
            capi.check(L.fo_event_record(e0, main_stream))
            fn()
            capi.check(L.fo_event_record(e1, main_stream))
            torch.cuda.synchronize()
            capi.check(L.fo_event_elapsed_ms(e0, e1, C.byref(v)))
            best = min(best, v.value)
        capi.check(L.fo_event_destroy(e0))
        capi.check(L.fo_event_destroy(e1))
        return avg, best

    it = a.kernel_iters
    # no waiter runs here: the group counters simply accumulate and are cleared afterwards
    sig_ms, sig_min = time_kernel(gemm_signal, it)
    MM.zero_()
    pl_ms, pl_min = time_kernel(gemm_plain, it)
    rms_ms, rms_min = time_kernel(norm, it)
    cons_ms, _ = time_kernel(
        lambda: capi.check(L.fo_consume(Cp.data_ptr(), staging.data_ptr(), 2 * M * N, main_stream)), it)

    flops = 2.0 * M * N * K
    rms_bytes = 2.0 * (M * N * 2) + N * 2
    cons_bytes = 2.0 * (M * N * 2)
    sig_tf = flops / sig_ms / 1e9
    pl_tf = flops / pl_ms / 1e9
    rms_gbps = rms_bytes / rms_ms / 1e6
    cu, khz, xcd = C.c_int(), C.c_int(), C.c_int()
    capi.check(L.fo_device_info(C.byref(cu), C.byref(khz), C.byref(xcd)))

    # ---- CPU baseline: the oracle on a bounded sample of the same workload -------
    cpu = None
    if a.cpu_seconds > 0:
        from oracle import fo_oracle as O
        torch.set_num_threads(os.cpu_count() or 1)
        probe = 128
        t = time.perf_counter()
        O.rmsnorm(O.gemm(A_h[:probe], B_h), g_h, eps)
        rate = probe / max(time.perf_counter() - t, 1e-6)              # rows per second, cold
        rows = int(min(M, max(probe, rate * a.cpu_seconds / 3)))
        rows -= rows % 64
        best = None
        for _ in range(3):
            t = time.perf_counter()
            c = O.gemm(A_h[:rows], B_h)
            t_mm = time.perf_counter() - t
            O.rmsnorm(c, g_h, eps)
            t_all = time.perf_counter() - t
            if best is None or t_all < best[0]:
                best = (t_all, t_mm)
        cpu = {"value": round(2.0 * rows * N * K / best[0] / 1e12, 4), "unit": "TFLOP/s",
               "cores": torch.get_num_threads(), "kind": "port",
               "sample": f"first {rows} of {M} rows of A: torch CPU fp32 matmul + RMSNorm, best of 3 "
                         f"({best[0]:.2f} s, matmul {best[1]:.2f} s)",
               "host_cpus": os.cpu_count()}

    line = {
        "metric": "signaling-GEMM TFLOP/s", "value": round(flops / step_ms / 1e9, 2), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(step_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dts, "data": "synthetic",
        "config": {"workload": f"{a.workload}: {NAMES[a.workload]}", "M": M, "N": N, "K": K,
                   "layout_tile": [BM, BN], "tiles": T, "tiles_per_wave": TILES_PER_WAVE, "tiles_per_group": w, "groups": G, "world_size": ws,
                   "eps": eps, "consumer": ("one wait kernel + one copy launch per group" if per_group else
                                f"persistent wait+consume, {a.consumer_blocks} workgroups"),
                   "step": ("signal GEMM -> wait+consume -> reorder+RMSNorm (serial)" if a.no_overlap else
                            "signal GEMM || wait+consume -> join -> reorder+RMSNorm")},
        "serial_step_ms": round(serial_ms, 5),
        # the dominant kernel as it ran inside the timed steps (consumer on the other stream, the
        # copy and the norm of the previous step in between launches)
        "roofline": {"bound": "mfma", "kernel": "gemm_kernel (signalling), inside the timed steps",
                     "achieved": round(flops / step_gemm_ms / 1e9, 2), "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / step_gemm_ms / 1e9 / PEAK_MFMA_TFLOPS, 4),
                     "traffic": MEASURED_TRAFFIC_BYTES.get(a.workload), "avg_us": round(step_gemm_ms * 1e3, 2),
                     "launches": a.steps},
        "gemm_signal_serial_step": {"achieved": round(flops / serial_gemm_ms / 1e9, 2), "unit": "TFLOP/s",
                                    "avg_us": round(serial_gemm_ms * 1e3, 2)},
        # the same kernel launched back to back on its own (A and B stay in the 256 MB Infinity Cache)
        "gemm_signal_isolated": {"achieved": round(sig_tf, 2), "unit": "TFLOP/s",
                                 "frac": round(sig_tf / PEAK_MFMA_TFLOPS, 4), "avg_us": round(sig_ms * 1e3, 2),
                                 "min_us": round(sig_min * 1e3, 2), "launches": it},
        "cpu_baseline": cpu,
        "gemm_plain": {"achieved": round(pl_tf, 2), "unit": "TFLOP/s", "frac": round(pl_tf / PEAK_MFMA_TFLOPS, 4),
                       "avg_us": round(pl_ms * 1e3, 2), "min_us": round(pl_min * 1e3, 2)},
        "signal_overhead_pct": round((sig_ms / pl_ms - 1.0) * 100.0, 2),
        "reorder_rmsnorm": {"bound": "hbm", "achieved": round(rms_gbps, 1), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                            "frac": round(rms_gbps / PEAK_HBM_GBPS, 4), "avg_us": round(rms_ms * 1e3, 2),
                            "min_us": round(rms_min * 1e3, 2), "bytes": rms_bytes},
        "consume_copy": {"achieved": round(cons_bytes / cons_ms / 1e6, 1), "unit": "GB/s",
                         "avg_us": round(cons_ms * 1e3, 2)},
        "device": {"cu": cu.value, "clock_khz": khz.value, "xcd": xcd.value},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
