#!/usr/bin/env python3
"""Benchmark of the single-GPU hot path on one MI355X.

A step is one pass of the path over one synthetic batch, inputs resident in HBM:
signalling GEMM on the caller's stream, on a second stream a wait kernel and a
consumer copy per group (or one persistent wait+consume kernel) releasing each
finished group into the staging buffer, an event join, then reorder+RMSNorm on
the staging buffer.

Prints ONE JSON line.  `value` is 2*M*N*K divided by the whole step time.  The
roofline object is for the dominant kernel (the signalling GEMM) as it ran
inside the timed steps, from a HIP event pair attached to every launch's own dispatch.
The same run also times, back to back and on their own, the signalling GEMM
and its plain twin (signal overhead), reorder+RMSNorm (HBM roofline; over a
rotation of buffer pairs larger than the 256 MB memory-side cache, and inside
the timed steps) and the consumer copy, the serial (non-overlapped) step, the
plain GEMM on all-zero operands (what the same instruction stream does when
the chip is not power-limited), and a CPU baseline (the oracle's fp32 matmul +
RMSNorm on the host cores) on a bounded sample of the same workload.  Launch
order: W+K serial steps, W+K overlapped steps, then the isolated kernels
(5 warm-up + --kernel-iters + 10 launches each).
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
# one wave finish together.  A "group size g" can be read as g tiles or as g waves (the reference's
# cSeg counts waves, tune/search.py:502-513).  c3 and c5: one wave per group.  c2 (sweep {1,2,4,8,16}) and
# c4 (size 2) default to the tile-count reading, which stresses the counters (c4: 4096 groups of 2
# tiles); `--reading waves` takes the other one (c4: 4 groups of 2048 tiles, c2: one group), and
# `--group-tiles` sets any size.  `--both-readings` puts the other reading's figures into the same record.
TILES_PER_WAVE = 1024
WORKLOADS = {
    "c1": ("fp16", 1024, 1024, 1024, 4, 1, 1e-6, None, None),
    "c2": ("fp16", 4096, 4096, 4096, 4, 1, 1e-5, None, None),
    "c3": ("bf16", 8192, 4096, 7168, TILES_PER_WAVE, 1, 1e-5, 1.0, 0.02),
    "c4": ("bf16", 16384, 8192, 1024, 2, 1, 1e-5, None, None),
    "c5": ("bf16", 8192, 8192, 3584, TILES_PER_WAVE, 8, 1e-5, None, None),
}
WAVE_READING = {"c2": TILES_PER_WAVE, "c4": 2 * TILES_PER_WAVE}   # tiles per group under the wave-count reading
NAMES = {
    "c1": "fp16 1024^3 plumbing shape",
    "c2": "fp16 4096^3 square GEMM",
    "c3": "Llama-3-8B down_proj share, bf16 8192x4096x7168",
    "c4": "Llama-3-70B o_proj share, bf16 16384x8192x1024",
    "c5": "Llama-3-70B down_proj share, ReduceScatter layout, bf16 8192x8192x3584",
}
PEAK_MFMA_TFLOPS = 2516.6   # MI355X dense fp16/bf16: 256 CU x 4096 FLOP/clk x 2.4 GHz
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E
MALL_BYTES = 256 << 20      # memory-side cache: a buffer rotation has to exceed it to measure HBM
# Bytes that cross the L2 -> memory interface per signalling-GEMM launch, from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of `bench.py --workload <wl> --no-overlap` (profiles/gemm_traffic_c2_c3_c4_c5.txt):
# FETCH_SIZE KiB x 2.000 (a 256 MiB consumer copy reads as 131094 KiB) + WRITE_SIZE KiB x 1.000.
# A workload without a tracked measurement has no entry, and its bench line then has no roofline.traffic.
MEASURED_TRAFFIC_BYTES = {"c2": 235_200_000, "c3": 772_100_000, "c4": 671_900_000, "c5": 841_500_000}


class Timer:
    """HIP-event timing through the C ABI, on the stream the kernels are launched on."""

    def __init__(self, L, capi, stream=None):
        self.L, self.capi, self.stream = L, capi, stream

    def event(self):
        e = C.c_void_p()
        self.capi.check(self.L.fo_event_create(C.byref(e)))
        return e

    def record(self, e):
        self.capi.check(self.L.fo_event_record(e, self.stream))

    def ms(self, e0, e1):
        v = C.c_float()
        self.capi.check(self.L.fo_event_elapsed_ms(e0, e1, C.byref(v)))
        return v.value

    def free(self, *evs):
        for e in evs:
            self.capi.check(self.L.fo_event_destroy(e))


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=500.0,
                    help="untimed steps run for this long before the first warm-up: a chip that comes from idle "
                         "needs tens of milliseconds of load before its clock has settled at the power limit")
    ap.add_argument("--workload", default="c3", choices=sorted(WORKLOADS))
    ap.add_argument("--group-tiles", type=int, default=0, help="tiles per signal group (0 = workload default)")
    ap.add_argument("--reading", default="default", choices=["default", "tiles", "waves"],
                    help="how a workload's group size is read (c2, c4): as tiles or as hardware waves")
    ap.add_argument("--both-readings", action="store_true",
                    help="c2/c4: also time the step under the other reading and put it into the record")
    ap.add_argument("--kernel-iters", type=int, default=100, help="timed launches per isolated kernel")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU-baseline work; 0 skips it")
    ap.add_argument("--mfma-loop-seconds", type=float, default=0.6,
                    help="how long to run the MFMA-only loop (fo_mfma_spin) on each operand set; 0 skips it")
    ap.add_argument("--consumer-blocks", type=int, default=0,
                    help="workgroups of the persistent consumer (0 = one per CU, which is also the maximum)")
    ap.add_argument("--consumer", default="auto", choices=["auto", "per_group", "persistent"])
    ap.add_argument("--last-group", default="settle_then_join", choices=["main", "comm", "settle", "settle_then_join"],
                    help="how the last group is released (per-group consumer): settle_then_join (default, what "
                         "OverlapImpl does): on the GEMM's own stream by one launch that settles the counter and copies, "
                         "the earlier groups joined behind it; settle: the same with the join in front; main: wait "
                         "kernel + copy on the GEMM's stream behind the join; comm: on the second stream like every "
                         "other group, as the reference does")
    ap.add_argument("--no-overlap", action="store_true",
                    help="order the consumer behind the GEMM in the timed step (needed under counter collection, "
                         "which runs one kernel at a time)")
    ap.add_argument("--fork", action="store_true",
                    help="order the second stream behind the main stream before the GEMM, which OverlapImpl does when "
                         "the call is being captured into a graph (costs 5-9 us of a step when done eagerly)")
    ap.add_argument("--tune", action="append", default=[], metavar="KNOB=VALUE",
                    help="library knob for this run (fo_tune: store_mode, release_mode, copy_streaming_stores)")
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
    for kv in a.tune:
        knob, _, val = kv.partition("=")
        capi.check(L.fo_tune(knob.encode(), int(val)))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    cu, khz, xcd = C.c_int(), C.c_int(), C.c_int()
    capi.check(L.fo_device_info(C.byref(cu), C.byref(khz), C.byref(xcd)))
    if a.consumer_blocks <= 0:
        a.consumer_blocks = cu.value

    dts, M, N, K, w_default, ws, eps, a_std, b_std = WORKLOADS[a.workload]
    w_tiles, w_waves = w_default, WAVE_READING.get(a.workload, w_default)
    w = w_waves if a.reading == "waves" else w_tiles
    if a.group_tiles:
        w = a.group_tiles
    dt = torch.float16 if dts == "fp16" else torch.bfloat16
    code = capi.dtype_code(dt)
    algo = 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN

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
    # reorder+RMSNorm reads `staging` and writes `out`; enough pairs that one pass over all of them
    # exceeds the memory-side cache, so a back-to-back rotation measures HBM and not that cache
    pair_bytes = 2 * M * N * 2
    npairs = max(1, -(-MALL_BYTES // pair_bytes) + 1)
    stagings = [torch.zeros(M * N, dtype=dt, device=dev) for _ in range(npairs)]
    outs = [torch.empty(M, N, dtype=dt, device=dev) for _ in range(npairs)]
    staging, out = stagings[0], outs[0]
    hint = tiling.raster_hint(M, N, algo)
    RA = tiling.reorder_indices(T, hint, dev).reshape(TM, TN)
    comm = C.c_void_p()
    capi.check(L.fo_stream_create(C.byref(comm)))
    capi.check(L.fo_set_wait_timeout_ms(10000))
    main_stream = None  # the null stream; all launches of the main leg go there
    tm = Timer(L, capi, main_stream)

    class Grouping:
        """Everything that depends on the group size: cSeg, counters, table, row remap."""

        def __init__(self, w):
            self.w = w
            self.cseg = tiling.uniform_cseg(T, w)
            self.G = len(self.cseg)
            self.cseg_d = torch.tensor(self.cseg, dtype=torch.int32, device=dev)
            self.MM = torch.zeros(max(self.G, TN), dtype=torch.int32, device=dev)
            self.table = torch.empty(T, dtype=torch.int32, device=dev)
            capi.check(L.fo_build_group_table(self.cseg_d.data_ptr(), self.G, T, self.table.data_ptr(), None))
            self.RE = tiling.generate_row_remap_array(M, N, BM, BN, self.cseg, ws, dev) if ws > 1 else None
            # Same rule as OverlapImpl: up to 32 groups the reference's structure (one wait kernel and one
            # consumer launch per group, src/overlap_impl.cu:257-265), beyond that one persistent kernel.
            self.per_group = a.consumer == "per_group" or (a.consumer == "auto" and self.G <= 32)

    def gemm_signal(g):
        if ws > 1:
            capi.check(L.fo_gemm_scatter(code, algo, M, N, K, 1, g.cseg_d.data_ptr(), g.G, g.table.data_ptr(),
                                         A.data_ptr(), B.data_ptr(), Cp.data_ptr(), g.MM.data_ptr(), RA.data_ptr(),
                                         g.RE.data_ptr(), 0, main_stream))
        else:
            capi.check(L.fo_gemm_signal(code, algo, M, N, K, 1, g.cseg_d.data_ptr(), g.G, g.table.data_ptr(),
                                        A.data_ptr(), B.data_ptr(), Cp.data_ptr(), g.MM.data_ptr(), RA.data_ptr(), 0,
                                        main_stream))

    def gemm_plain(a_t=None, b_t=None):
        a_t, b_t = (A, B) if a_t is None else (a_t, b_t)
        capi.check(L.fo_gemm(code, algo, M, N, K, a_t.data_ptr(), b_t.data_ptr(), Cn.data_ptr(), main_stream))

    def wait_consume(g):
        """The consumer of OverlapImpl::consume_groups; on return the main stream is ordered behind it."""
        if not g.per_group:
            capi.check(L.fo_wait_consume(g.cseg_d.data_ptr(), g.G, g.MM.data_ptr(), Cp.data_ptr(),
                                         staging.data_ptr(), BM * BN, ws, 0, ws, (M * N // ws) if ws > 1 else 0,
                                         None, a.consumer_blocks, None, comm))
            capi.check(L.fo_stream_join(comm, main_stream))
            return
        # like OverlapImpl: the groups before the last are copied beside the GEMM; if that is a lot of data,
        # with non-temporal stores (1), else with ordinary ones (2); the last group always with ordinary ones
        beside = 2 * BM * BN * sum(g.cseg[:-1])
        beside_policy = 1 if beside >= (64 << 20) else 2
        acc = 0
        for gi, n in enumerate(g.cseg):
            stream = comm
            last_on_main = gi == g.G - 1 and a.last_group != "comm"
            if last_on_main:
                # the last group completes with the GEMM: release it on the GEMM's stream
                if g.G > 1 and a.last_group != "settle_then_join":
                    capi.check(L.fo_stream_join(comm, main_stream))
                stream = main_stream
            settle = last_on_main and a.last_group != "main"
            if not settle:
                capi.check(L.fo_wait(n, g.MM.data_ptr() + 4 * gi, None, stream))
            elems = n * BM * BN
            part = elems // ws
            # one launch per group (ws > 1: slice k of the group goes to rank k's receive buffer)
            capi.check(L.fo_consume_slices(n, g.MM.data_ptr() + 4 * gi if settle else None, Cp.data_ptr() + 2 * acc,
                                           staging.data_ptr() + 2 * (acc // ws), 2 * part, ws, 2 * (M * N // ws),
                                           2 if gi == g.G - 1 else beside_policy, None, stream))
            acc += elems
        if a.last_group == "comm" or (a.last_group == "settle_then_join" and g.G > 1):
            capi.check(L.fo_stream_join(comm, main_stream))

    def norm(i=0):
        x, o = stagings[i], outs[i]
        if ws > 1:  # every rank slice is a layout with tile height BM/ws: ws problems, one launch
            capi.check(L.fo_reorder_rmsnorm_batched(code, x.data_ptr(), gamma.data_ptr(), o.data_ptr(), ws,
                                                    M // ws, N, BM // ws, BN, 1, RA.data_ptr(), eps, main_stream))
        else:
            capi.check(L.fo_reorder_rmsnorm(code, x.data_ptr(), gamma.data_ptr(), o.data_ptr(), M, N, BM, BN,
                                            1, RA.data_ptr(), eps, main_stream))

    def step(g, overlap=True, ev=None):
        if overlap and a.fork and (g.G > 1 or not g.per_group):
            capi.check(L.fo_stream_join(main_stream, comm))
        if ev:   # the GEMM's own dispatch carries the two events: its duration without launch gaps
            capi.check(L.fo_time_next_launch(ev[0], ev[1]))
        gemm_signal(g)
        if not overlap:  # consumer ordered behind the GEMM: the serial reference for the overlap
            capi.check(L.fo_stream_join(main_stream, comm))
        wait_consume(g)
        if ev and len(ev) > 2:
            capi.check(L.fo_time_next_launch(ev[2], ev[3]))
        norm()

    def time_steps(g, overlap, probes=0):
        """Wall time per step over exactly a.steps steps.  probes=2: every step's signalling GEMM also
        carries one HIP event pair, attached to the kernel's own dispatch (what a kernel trace reports:
        no launch gaps, no extra packets in the stream), and the mean duration is returned; probes=4:
        the same for reorder+RMSNorm as well.  The attached pairs can cost a few us of wall time per
        step, so the step time that is reported comes from a pass without them."""
        evs = [tuple(tm.event() for _ in range(probes)) for _ in range(a.steps)]
        for _ in range(a.warmup):
            step(g, overlap)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for ev in evs:
            step(g, overlap, ev)
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / a.steps
        gemm_ms = sum(tm.ms(e[0], e[1]) for e in evs) / a.steps if probes >= 2 else 0.0
        norm_ms = sum(tm.ms(e[2], e[3]) for e in evs) / a.steps if probes > 2 else 0.0
        for e in evs:
            tm.free(*e)
        return wall, gemm_ms, norm_ms

    def check_timeouts():
        n = C.c_int()
        capi.check(L.fo_wait_timeouts(C.byref(n), 1))
        if n.value:
            print(f"bench.py: {n.value} bounded waits expired; results invalid", file=sys.stderr)
        return n.value

    def consumer_name(g):
        return ("one wait kernel + one copy launch per group"
                + {"comm": "", "main": ", the last group on the GEMM's stream",
                   "settle": ", the last group settled and copied by one launch on the GEMM's stream",
                   "settle_then_join": ", the last group settled and copied by one launch on the GEMM's stream"}[
                       a.last_group]
                if g.per_group else
                f"persistent wait+consume, {a.consumer_blocks} workgroups")

    # ---- whole path: W warm-up steps, then exactly K timed steps -----------------
    grp = Grouping(w)
    # A process that has only allocated and copied finds the chip clocked down; the first tens of
    # milliseconds of load then run 3-6 % slow, which with a short --steps/--warmup is all that would
    # be measured.  Steps are therefore run, untimed, until the chip has been busy for --settle-ms;
    # the W warm-up steps and the K timed steps of every pass follow as the contract says.
    settled_ms, settle_steps, t_settle = 0.0, 0, time.perf_counter()
    while a.settle_ms > 0 and settled_ms < a.settle_ms:
        for _ in range(20):
            step(grp, not a.no_overlap)
        settle_steps += 20
        torch.cuda.synchronize()
        settled_ms = (time.perf_counter() - t_settle) * 1e3
    # the timed steps, then the same steps again with the kernels' event pairs attached
    serial_ms, _, _ = time_steps(grp, False)
    step_ms = serial_ms if a.no_overlap else time_steps(grp, True)[0]
    _, serial_gemm_ms, _ = time_steps(grp, False, probes=2)
    step_probed_ms, step_gemm_ms, _ = (serial_ms, serial_gemm_ms, 0.0) if a.no_overlap else time_steps(grp, True, probes=2)
    _, _, step_norm_ms = time_steps(grp, not a.no_overlap, probes=4)
    if check_timeouts():
        return 1

    # ---- isolated kernels, HIP events on the launch stream -----------------------
    def time_kernel(fn, iters):
        """Average launch duration: `iters` back-to-back launches between one HIP event pair on
        the launch stream (what a kernel trace reports as the kernel's average), and the
        shortest single launch out of 10 individually bracketed ones.  fn takes the launch index."""
        e0, e1 = tm.event(), tm.event()
        for i in range(5):
            fn(i)
        torch.cuda.synchronize()
        tm.record(e0)
        for i in range(iters):
            fn(i)
        tm.record(e1)
        torch.cuda.synchronize()
        avg = tm.ms(e0, e1) / iters
        best = float("inf")
        for i in range(10):
            tm.record(e0)
            fn(i)
            tm.record(e1)
            torch.cuda.synchronize()
            best = min(best, tm.ms(e0, e1))
        tm.free(e0, e1)
        return avg, best

    it = a.kernel_iters
    # no waiter runs here: the group counters simply accumulate and are cleared afterwards
    sig_ms, sig_min = time_kernel(lambda i: gemm_signal(grp), it)
    grp.MM.zero_()
    # the same launches with the signal in its release-ordered form (the atomic itself a release at
    # agent scope, which writes the L2's dirty lines back first) instead of the default (write-through
    # tile stores, acknowledged, a barrier, a relaxed atomic)
    default_release_mode = next((int(kv.partition("=")[2]) for kv in a.tune if kv.startswith("release_mode=")), 1)
    capi.check(L.fo_tune(b"release_mode", 0))
    sig_rel_ms, _ = time_kernel(lambda i: gemm_signal(grp), it)
    capi.check(L.fo_tune(b"release_mode", default_release_mode))
    grp.MM.zero_()
    pl_ms, pl_min = time_kernel(lambda i: gemm_plain(), it)
    # Every buffer of the rotation holds the step's real output: on an all-zero input the kernel runs
    # 9 % faster than on data (20.4 against 22.5 us on c3), which a rotation over one real and two
    # cleared buffers used to credit to it.
    for other_staging in stagings[1:]:
        other_staging.copy_(stagings[0])
    torch.cuda.synchronize()
    rms_rot_ms, _ = time_kernel(lambda i: norm(i % npairs), it)      # rotation larger than the memory-side cache
    rms_same_ms, rms_min = time_kernel(lambda i: norm(0), it)         # one pair over and over: served by that cache
    cons_ms, _ = time_kernel(
        lambda i: capi.check(L.fo_consume(Cp.data_ptr(), stagings[i % npairs].data_ptr(), 2 * M * N, main_stream)), it)
    # the yardstick for reorder+RMSNorm: the copy kernel over the same rotation, source and destination both
    # rotating (the consumer's copy above reads one source over and over, which the memory-side cache then holds)
    rot_copy_ms, _ = time_kernel(
        lambda i: capi.check(L.fo_consume(stagings[i % npairs].data_ptr(), outs[i % npairs].data_ptr(), 2 * M * N,
                                          main_stream)), it)
    # The same instruction stream on all-zero operands: the MFMAs toggle nothing, the chip stays
    # below its power limit and keeps its clock.  What separates this figure from gemm_plain is
    # the power limit, not the kernel's schedule.
    A0, B0 = torch.zeros_like(A), torch.zeros_like(B)
    z_ms, _ = time_kernel(lambda i: gemm_plain(A0, B0), max(10, it // 4))

    other = None
    if a.both_readings and a.workload in WAVE_READING and not a.group_tiles:
        w2 = w_tiles if w == w_waves else w_waves
        g2 = Grouping(w2)
        s2_serial, _, _ = time_steps(g2, False)
        s2_ms = s2_serial if a.no_overlap else time_steps(g2, True)[0]
        s2_gemm = 0.0 if a.no_overlap else time_steps(g2, True, probes=2)[1]
        if check_timeouts():
            return 1
        sig2_ms, _ = time_kernel(lambda i: gemm_signal(g2), it)
        g2.MM.zero_()
        other = {"reading": "waves" if w2 == w_waves else "tiles", "tiles_per_group": w2, "groups": g2.G,
                 "consumer": consumer_name(g2), "ms_per_step": round(s2_ms, 5), "serial_step_ms": round(s2_serial, 5),
                 "gemm_signal_in_step_us": round(s2_gemm * 1e3, 2), "gemm_signal_isolated_us": round(sig2_ms * 1e3, 2),
                 "signal_overhead_pct": round((sig2_ms / pl_ms - 1.0) * 100.0, 2)}

    # What the power limit leaves to the MFMAs alone: the GEMM's own MFMA instruction in a loop on
    # register operands taken from A (and from zeros), no memory, LDS or address work beside it.
    # The GEMM's rate can be read against the first figure: no kernel on these operands gets past it.
    mfma_loop = None
    if a.mfma_loop_seconds > 0:
        LB = capi.bench_lib()   # the probes live in a library of their own, outside the product's ABI
        sink = torch.zeros(1, dtype=torch.float32, device=dev)
        spin_flop = C.c_longlong()

        def spin_rate(buf, wide=0, traffic=0):
            def launch(i):      # 1024 rounds of 128 MFMAs per wavefront: about 1 ms
                capi.bench_check(LB.fo_mfma_spin(code, wide, traffic, buf.data_ptr(), buf.numel() * buf.element_size(),
                                                 1024, sink.data_ptr(), C.byref(spin_flop), main_stream))
            n = max(8, int(a.mfma_loop_seconds / 2 / 1e-3))
            for i in range(n):  # first half untimed: the clock settles to what the power limit allows
                launch(i)
            ms, _ = time_kernel(launch, n)
            tf = spin_flop.value / ms / 1e9
            return {"achieved": round(tf, 1), "frac": round(tf / PEAK_MFMA_TFLOPS, 4), "avg_us": round(ms * 1e3, 2)}

        mfma_loop = {"unit": "TFLOP/s", "instruction": f"v_mfma_f32_16x16x32_{'f16' if dts == 'fp16' else 'bf16'}",
                     "operands_of_A": spin_rate(A), "zero_operands": spin_rate(A0),
                     "operands_of_A_32x32x16": spin_rate(A, 1),
                     # the same loop with the fragment reads and the copies of a 256x256 tile beside the MFMAs,
                     # nothing waiting for them: this tile's operand traffic under a perfect schedule
                     "operands_of_A_with_fragment_reads": spin_rate(A, 0, 1),
                     "operands_of_A_with_tile_traffic": spin_rate(A, 0, 3),
                     "note": "one wavefront per SIMD issuing nothing but MFMAs on register operands, in the order of the GEMM's k-step, sustained "
                             f"{a.mfma_loop_seconds / 2:.1f} s before the timed half"}
    del A0, B0

    flops = 2.0 * M * N * K
    traffic_algorithmic = 2 * (M * K + N * K + M * N)   # A and B read once, C written once
    rms_bytes = 2.0 * (M * N * 2) + N * 2
    cons_bytes = 2.0 * (M * N * 2)
    sig_tf = flops / sig_ms / 1e9
    pl_tf = flops / pl_ms / 1e9
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

    def hbm(ms):
        gbps = rms_bytes / ms / 1e6
        return {"achieved": round(gbps, 1), "frac": round(gbps / PEAK_HBM_GBPS, 4), "avg_us": round(ms * 1e3, 2)}

    reading = ("tiles" if w == w_tiles else "waves" if w == w_waves else "custom") if a.workload in WAVE_READING else "waves"
    line = {
        "metric": "signaling-GEMM path step TFLOP/s", "value": round(flops / step_ms / 1e9, 2), "unit": "TFLOP/s",
        "value_is": "2*M*N*K / whole step time (signalling GEMM || consumer, then reorder+RMSNorm); "
                    "the signalling GEMM kernel's own rate is gemm_kernel_tflops = roofline.achieved",
        "gemm_kernel_tflops": round(flops / step_gemm_ms / 1e9, 2),
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "clock_settle_ms": round(settled_ms, 1), "clock_settle_steps": settle_steps,
        "ms_per_step": round(step_ms, 5),
        "ms_per_step_with_kernel_events": round(step_probed_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dts, "data": "synthetic",
        "config": {"workload": f"{a.workload}: {NAMES[a.workload]}", "M": M, "N": N, "K": K,
                   "layout_tile": [BM, BN], "tiles": T, "tiles_per_wave": TILES_PER_WAVE, "group_size_reading": reading,
                   "tiles_per_group": w, "groups": grp.G, "world_size": ws, "eps": eps, "consumer": consumer_name(grp),
                   "step": ("signal GEMM -> wait+consume -> reorder+RMSNorm (serial)" if a.no_overlap else
                            "signal GEMM || wait+consume -> join -> reorder+RMSNorm")},
        "serial_step_ms": round(serial_ms, 5),
        # the dominant kernel as it ran inside the timed steps (consumer on the other stream, the
        # copy and the norm of the previous step in between launches)
        "roofline": {"bound": "mfma", "kernel": "gemm_kernel (signalling), inside the same steps run again with an event pair on its dispatch",
                     "achieved": round(flops / step_gemm_ms / 1e9, 2), "peak": PEAK_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / step_gemm_ms / 1e9 / PEAK_MFMA_TFLOPS, 4),
                     "avg_us": round(step_gemm_ms * 1e3, 2), "launches": a.steps,
                     # HBM-side bytes per launch from the tracked counter summary of this workload
                     # (profiles/); the key is left out for a workload that has none
                     **({"traffic": MEASURED_TRAFFIC_BYTES[a.workload], "traffic_algorithmic": traffic_algorithmic}
                        if a.workload in MEASURED_TRAFFIC_BYTES else {})},
        "gemm_signal_serial_step": {"achieved": round(flops / serial_gemm_ms / 1e9, 2), "unit": "TFLOP/s",
                                    "avg_us": round(serial_gemm_ms * 1e3, 2)},
        # the same kernel launched back to back on its own (A and B stay in the 256 MB memory-side cache)
        "gemm_signal_isolated": {"achieved": round(sig_tf, 2), "unit": "TFLOP/s",
                                 "frac": round(sig_tf / PEAK_MFMA_TFLOPS, 4), "avg_us": round(sig_ms * 1e3, 2),
                                 "min_single_launch_us": round(sig_min * 1e3, 2), "launches": it},
        "cpu_baseline": cpu,
        "gemm_plain": {"achieved": round(pl_tf, 2), "unit": "TFLOP/s", "frac": round(pl_tf / PEAK_MFMA_TFLOPS, 4),
                       "avg_us": round(pl_ms * 1e3, 2), "min_single_launch_us": round(pl_min * 1e3, 2)},
        "gemm_plain_zero_operands": {"achieved": round(flops / z_ms / 1e9, 2), "unit": "TFLOP/s",
                                     "frac": round(flops / z_ms / 1e9 / PEAK_MFMA_TFLOPS, 4),
                                     "avg_us": round(z_ms * 1e3, 2),
                                     "note": "same kernel and shape, A = B = 0: not power-limited"},
        "mfma_only_loop": mfma_loop,
        # both back to back against the plain twin of the same run; "release" is the release-ordered atomic
        "signal_overhead_pct": round((sig_ms / pl_ms - 1.0) * 100.0, 2),
        "signal_overhead_pct_release": round((sig_rel_ms / pl_ms - 1.0) * 100.0, 2),
        "signal_form": {"default": "write-through tile stores, acknowledged (vmcnt 0), workgroup barrier, relaxed agent-scope atomic",
                        "release": "release-ordered agent-scope atomic (L2 write-back first), fo_tune release_mode=0",
                        "gemm_signal_release_isolated_us": round(sig_rel_ms * 1e3, 2)},
        # headline: back to back over a rotation of buffer pairs that exceeds the memory-side cache
        "reorder_rmsnorm": {"bound": "hbm", "peak": PEAK_HBM_GBPS, "unit": "GB/s", "bytes": rms_bytes,
                            **hbm(rms_rot_ms), "buffer_pairs": npairs,
                            "in_step": hbm(step_norm_ms),
                            "same_pair_back_to_back": {**hbm(rms_same_ms), "min_single_launch_us": round(rms_min * 1e3, 2)},
                            # the yardstick of the same run: a plain copy kernel moving the same bytes over the same rotation
                            "copy_kernel_same_run": {"achieved": round(cons_bytes / rot_copy_ms / 1e6, 1),
                                                     "frac": round(cons_bytes / rot_copy_ms / 1e6 / PEAK_HBM_GBPS, 4),
                                                     "avg_us": round(rot_copy_ms * 1e3, 2)}},
        "consume_copy": {"achieved": round(cons_bytes / cons_ms / 1e6, 1), "unit": "GB/s",
                         "avg_us": round(cons_ms * 1e3, 2)},
        "other_reading": other,
        "device": {"cu": cu.value, "clock_khz": khz.value, "xcd_assumed": xcd.value},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
