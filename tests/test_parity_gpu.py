"""GPU parity tests: the HIP path, called through the C ABI, against the CPU
oracle on the same seeded inputs.

Bars: integer artefacts (counters, tickets, group table, placement, staging,
row remap) bit-exact; GEMM on small-integer inputs bit-exact (every partial sum
is exact in fp32, so accumulation order cannot matter and any indexing mistake
shows); GEMM + RMSNorm on random inputs within rel-L2 1e-3 and max-abs 2e-2 of
the fp32 oracle cast through the same storage points (C -> dtype, out ->
dtype); the distance to the unquantised fp32 result is printed as information.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from flashoverlap_amd import capi, tiling
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-3
MAX_ABS_TOL = 2e-2


def _say(*a):
    print(*a, flush=True)


def _max_abs_ok(got, ref):
    """max-abs 2e-2, except where that is less than two units in the last place of the storage
    type.  The kernel's only freedom is the order of the fp32 accumulation, which can move an
    element of C by one storage ulp; downstream that element is rounded twice more (scaled value,
    then times gamma), so the final value can land two ulps from the oracle's.  A bf16 value of
    magnitude 2..4 has ulp 2^-6: two of them are 0.031 > 2e-2, so from that magnitude on the bound
    is two ulps."""
    mant = 7 if ref.dtype == torch.bfloat16 else 10
    r = ref.float().abs().clamp_min(2.0 ** -20)
    ulp = torch.exp2(torch.floor(torch.log2(r)) - mant)
    tol = torch.maximum(torch.full_like(ulp, MAX_ABS_TOL), 2 * ulp)
    return bool(((got.float() - ref.float()).abs() <= tol).all())


class Path:
    """One problem instance with its device buffers, driven through the C ABI."""

    def __init__(self, L, dev, dt, M, N, K, algo, cseg=None, hint=None, ws=1, monitor=False, seed=0,
                 integer_inputs=False, a_std=None, b_std=None):
        self.L, self.dev, self.dt = L, dev, dt
        self.M, self.N, self.K, self.algo, self.ws, self.monitor = M, N, K, algo, ws, monitor
        self.BM, self.BN, _ = capi.algo_tile(algo)
        self.TM, self.TN = M // self.BM, N // self.BN
        self.T = self.TM * self.TN
        g = torch.Generator().manual_seed(seed)
        if integer_inputs:
            self.A = torch.randint(-2, 3, (M, K), generator=g).to(dt)
            self.B = torch.randint(-2, 3, (N, K), generator=g).to(dt)
        else:
            sa = a_std if a_std is not None else 1.0 / K ** 0.5
            sb = b_std if b_std is not None else 1.0 / K ** 0.5
            self.A = (torch.randn(M, K, generator=g) * sa).to(dt)
            self.B = (torch.randn(N, K, generator=g) * sb).to(dt)
        self.gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(dt)
        self.hint = list(hint) if hint is not None else tiling.raster_hint(M, N, algo)
        self.cseg = list(cseg) if cseg is not None else [self.T]
        self.G = len(self.cseg)
        self.ra_host = tiling.reorder_indices(self.T, self.hint)
        self.dA, self.dB, self.dgamma = self.A.to(dev), self.B.to(dev), self.gamma.to(dev)
        self.dRA = self.ra_host.to(dev).reshape(self.TM, self.TN)
        self.dcseg = torch.tensor(self.cseg, dtype=torch.int32, device=dev)
        mm_len = (self.TN + self.T) if monitor else max(self.G, self.TN)
        self.dMM = torch.zeros(mm_len, dtype=torch.int32, device=dev)
        self.dtable = torch.full((self.T,), -1, dtype=torch.int32, device=dev)
        self.dC = torch.zeros(M * N, dtype=dt, device=dev)
        self.re_host = None
        self.dRE = None
        if ws > 1:
            self.re_host = tiling.generate_row_remap_array(M, N, self.BM, self.BN, self.cseg, ws)
            self.dRE = self.re_host.to(dev)
        self.code = capi.dtype_code(dt)

    def build_table(self, stream=None):
        capi.check(self.L.fo_build_group_table(self.dcseg.data_ptr(), self.G, self.T, self.dtable.data_ptr(), stream))

    def gemm_plain(self, out=None, stream=None):
        out = out if out is not None else torch.zeros(self.M, self.N, dtype=self.dt, device=self.dev)
        capi.check(self.L.fo_gemm(self.code, self.algo, self.M, self.N, self.K, self.dA.data_ptr(),
                                  self.dB.data_ptr(), out.data_ptr(), stream))
        return out

    def gemm_signal(self, use_table=True, stream=None, rldn=1):
        table = self.dtable.data_ptr() if use_table else None
        if self.dRE is not None:
            capi.check(self.L.fo_gemm_scatter(self.code, self.algo, self.M, self.N, self.K, rldn, self.dcseg.data_ptr(),
                                              self.G, table, self.dA.data_ptr(), self.dB.data_ptr(),
                                              self.dC.data_ptr(), self.dMM.data_ptr(), self.dRA.data_ptr(),
                                              self.dRE.data_ptr(), int(self.monitor), stream))
        else:
            capi.check(self.L.fo_gemm_signal(self.code, self.algo, self.M, self.N, self.K, rldn, self.dcseg.data_ptr(),
                                             self.G, table, self.dA.data_ptr(), self.dB.data_ptr(),
                                             self.dC.data_ptr(), self.dMM.data_ptr(), self.dRA.data_ptr(),
                                             int(self.monitor), stream))

    def reorder_rmsnorm(self, x, eps, bs=None, BM=None, stream=None):
        bs = bs if bs is not None else self.M
        BM = BM if BM is not None else self.BM
        out = torch.empty(bs, self.N, dtype=self.dt, device=self.dev)
        capi.check(self.L.fo_reorder_rmsnorm(self.code, x.data_ptr(), self.dgamma.data_ptr(), out.data_ptr(), bs,
                                             self.N, BM, self.BN, 1, self.dRA.data_ptr(), eps, stream))
        return out


@pytest.fixture(scope="module")
def L(fo_lib, dev):
    capi.check(fo_lib.fo_set_wait_timeout_ms(5000))
    return fo_lib


@pytest.fixture()
def comm_stream(L):
    s = C.c_void_p()
    capi.check(L.fo_stream_create(C.byref(s)))
    yield s
    capi.check(L.fo_stream_sync(s))
    capi.check(L.fo_stream_destroy(s))


def _timeouts(L):
    n = C.c_int()
    capi.check(L.fo_wait_timeouts(C.byref(n), 1))
    return n.value


# ---- GEMM --------------------------------------------------------------------

@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,algo", [(128, 128, 64, 1), (256, 256, 64, 0), (256, 512, 192, 3), (512, 256, 128, 5),
                                        (384, 640, 320, 1), (1024, 1024, 1024, 1), (2048, 4096, 256, 1),
                                        # K that is not a multiple of the 64-deep panel: a zero-padded last panel
                                        (128, 128, 8, 1), (256, 256, 72, 0), (256, 512, 200, 3), (512, 256, 120, 5),
                                        (384, 640, 328, 1), (1024, 1024, 1000, 1)])
def test_gemm_bit_exact_on_integer_inputs(L, dev, dt, M, N, K, algo):
    _say("gemm integer", dt, M, N, K, algo)
    p = Path(L, dev, dt, M, N, K, algo, integer_inputs=True)
    got = p.gemm_plain()
    torch.cuda.synchronize()
    want = O.gemm(p.A, p.B)
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("K", [2048, 2040])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_gemm_random_within_tolerance(L, dev, dt, K):
    M, N = 1024, 768
    _say("gemm random", dt, M, N, K)
    p = Path(L, dev, dt, M, N, K, 1, seed=3)
    got = p.gemm_plain().cpu()
    ref32 = O.gemm_fp32(p.A, p.B)
    gated = ref32.to(dt)
    _say("  vs unquantised fp32: rel-L2 %.2e max-abs %.2e" % (O.rel_l2(got, ref32), O.max_abs(got, ref32)))
    assert O.rel_l2(got, gated) < REL_L2_TOL and O.max_abs(got, gated) < MAX_ABS_TOL
    # fp32 accumulation order is the only freedom: at most one storage ulp apart
    ulp = 2 ** -10 if dt == torch.float16 else 2 ** -7
    assert ((got.float() - gated.float()).abs() <= ulp * gated.float().abs() + 1e-6).all()


def test_time_next_launch_gives_the_kernel_duration(L, dev):
    """Events attached to the dispatch bracket the kernel alone: a positive time, no longer than
    what an event pair recorded around the call measures; the pair is used up by one launch."""
    p = Path(L, dev, torch.bfloat16, 2048, 2048, 2048, 1, seed=1)
    out = torch.zeros(2048, 2048, dtype=p.dt, device=dev)
    p.gemm_plain(out=out)
    torch.cuda.synchronize()
    evs = [C.c_void_p() for _ in range(4)]
    for e in evs:
        capi.check(L.fo_event_create(C.byref(e)))
    inner0, inner1, outer0, outer1 = evs
    capi.check(L.fo_event_record(outer0, None))
    capi.check(L.fo_time_next_launch(inner0, inner1))
    p.gemm_plain(out=out)
    capi.check(L.fo_event_record(outer1, None))
    p.gemm_plain(out=out)                      # not timed: the pair was taken by the launch before
    torch.cuda.synchronize()
    t_in, t_out = C.c_float(), C.c_float()
    capi.check(L.fo_event_elapsed_ms(inner0, inner1, C.byref(t_in)))
    capi.check(L.fo_event_elapsed_ms(outer0, outer1, C.byref(t_out)))
    _say("  kernel %.1f us inside a bracket of %.1f us" % (t_in.value * 1e3, t_out.value * 1e3))
    flops = 2.0 * 2048 ** 3
    assert 0 < t_in.value <= t_out.value
    assert flops / (t_in.value * 1e-3) < 2.6e15          # not faster than the chip
    assert L.fo_time_next_launch(inner0, None) == capi.FO_ERR_ARG
    # a call that is rejected uses the pair up too: it must not stay armed for a later, unrelated launch
    capi.check(L.fo_event_record(inner0, None))
    capi.check(L.fo_event_record(inner1, None))
    torch.cuda.synchronize()
    capi.check(L.fo_time_next_launch(inner0, inner1))
    assert L.fo_gemm(p.code, 1, 2048, 2048, 12, p.dA.data_ptr(), p.dB.data_ptr(), out.data_ptr(), None) == capi.FO_ERR_SHAPE
    p.gemm_plain(out=out)                      # 30 us of kernel that the pair must not see
    torch.cuda.synchronize()
    capi.check(L.fo_event_elapsed_ms(inner0, inner1, C.byref(t_in)))
    assert t_in.value < 0.01, "the pair of a rejected call was attached to the next launch"
    for e in evs:
        capi.check(L.fo_event_destroy(e))


@pytest.mark.parametrize("wide,traffic", [(0, 0), (1, 0), (0, 1), (0, 2), (0, 3)])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_mfma_spin_runs_counts_its_work_and_leaves_the_sink_alone(L, dev, dt, wide, traffic):
    """(The probe lives in libfo_bench.so, outside the product library; the events are the product's.)
    The MFMA-only loop used as the power-limit yardstick, bare and with a GEMM tile's fragment
    reads and copies beside it: reads its operands inside the buffer it is given (an odd number
    of 16-byte chunks where it makes no copies, 4 MiB + 16 bytes where it does), reports 128 MFMAs
    x 16384 flop (or 64 x 32768) x 4 wavefronts x CUs per round, writes nothing outside its own
    LDS, and is not faster than the chip."""
    LB = capi.bench_lib()
    cu = C.c_int()
    capi.check(L.fo_device_info(C.byref(cu), None, None))
    nelem = (4 << 20) // 2 + 8 if traffic & 2 else 7 * 8
    buf = torch.randn(nelem + 64, device=dev).to(dt)
    tail = buf[nelem:].clone()                               # what lies behind the bytes handed over
    guard = torch.full((64,), 3.0, dtype=torch.float32, device=dev)
    flop = C.c_longlong()
    iters = 1024
    e0, e1 = C.c_void_p(), C.c_void_p()
    capi.check(L.fo_event_create(C.byref(e0)))
    capi.check(L.fo_event_create(C.byref(e1)))
    args = (capi.dtype_code(dt), wide, traffic, buf.data_ptr(), nelem * 2, iters, guard[32:].data_ptr(), C.byref(flop), None)
    capi.bench_check(LB.fo_mfma_spin(*args))
    capi.check(L.fo_event_record(e0, None))
    capi.bench_check(LB.fo_mfma_spin(*args))
    capi.check(L.fo_event_record(e1, None))
    torch.cuda.synchronize()
    ms = C.c_float()
    capi.check(L.fo_event_elapsed_ms(e0, e1, C.byref(ms)))
    assert flop.value == cu.value * 4 * iters * 128 * 2 * 16 * 16 * 32
    assert torch.equal(guard.cpu(), torch.full((64,), 3.0))
    assert torch.equal(buf[nelem:], tail)
    rate = flop.value / (ms.value * 1e-3)
    _say("  MFMA loop, wide %d traffic %d: %.0f TFLOP/s" % (wide, traffic, rate / 1e12))
    assert 0.3e15 < rate < 2.6e15
    assert LB.fo_mfma_spin(7, *args[1:]) == capi.FO_ERR_ARG
    assert LB.fo_mfma_spin(args[0], wide, 4, *args[3:]) == capi.FO_ERR_ARG
    assert LB.fo_mfma_spin(args[0], 1, 1, *args[3:]) == capi.FO_ERR_ARG
    assert LB.fo_mfma_spin(args[0], 0, 2, buf.data_ptr(), 1 << 20, 1, guard.data_ptr(), None, None) == capi.FO_ERR_ARG
    assert LB.fo_mfma_spin(args[0], wide, 0, None, 16, 1, guard.data_ptr(), None, None) == capi.FO_ERR_ARG
    assert LB.fo_mfma_spin(args[0], wide, 0, buf.data_ptr(), 8, 1, guard.data_ptr(), None, None) == capi.FO_ERR_ARG
    assert LB.fo_mfma_spin(args[0], wide, 0, buf.data_ptr(), 112, 0, guard.data_ptr(), None, None) == capi.FO_ERR_ARG
    capi.check(L.fo_event_destroy(e0))
    capi.check(L.fo_event_destroy(e1))


def test_gemm_rejects_unsupported_shapes(L, dev):
    a = torch.zeros(384, 384, dtype=torch.float16, device=dev)  # large enough for every call below
    assert L.fo_gemm(capi.FO_F16, 1, 256, 256, 44, a.data_ptr(), a.data_ptr(), a.data_ptr(), None) == capi.FO_ERR_SHAPE
    # the signalling modes place whole layout tiles (128x256 here); the plain GEMM takes the shape
    i = torch.zeros(64, dtype=torch.int32, device=dev)
    assert L.fo_gemm_signal(capi.FO_F16, 3, 384, 384, 64, 1, i.data_ptr(), 1, None, a.data_ptr(), a.data_ptr(),
                            a.data_ptr(), i.data_ptr(), i.data_ptr(), 0, None) == capi.FO_ERR_SHAPE
    capi.check(L.fo_gemm(capi.FO_F16, 3, 384, 384, 64, a.data_ptr(), a.data_ptr(), a.data_ptr(), None))
    torch.cuda.synchronize()


# ---- signalling epilogue -------------------------------------------------------

@pytest.mark.parametrize("dt,M,N,K,algo,w", [
    (torch.float16, 1024, 1024, 1024, 1, 4),      # benchmark configuration 1: 64 tiles, 16 groups of 4 (> TN = 8 counters)
    (torch.bfloat16, 512, 768, 128, 1, 5),        # ragged last group
    (torch.bfloat16, 512, 768, 136, 1, 5),        # the same with a partial last k panel
    (torch.float16, 1024, 2048, 64, 3, 3),        # 128x256 layout tile
    (torch.bfloat16, 2048, 1024, 64, 5, 7),       # 256x128 layout tile
    (torch.float16, 2048, 2048, 64, 1, 1),        # one tile per group: 256 counters
])
def test_signal_placement_counters_and_table(L, dev, dt, M, N, K, algo, w):
    _say("signal", dt, M, N, K, algo, w)
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    rng = np.random.default_rng(5)
    hint = rng.permutation(T).tolist()  # any permutation is legal, not only the raster order
    p = Path(L, dev, dt, M, N, K, algo, cseg=O.uniform_cseg(T, w), hint=hint, integer_inputs=True)
    p.build_table()
    torch.cuda.synchronize()
    assert p.dtable.cpu().tolist() == O.group_of_slots(p.cseg, range(T)).tolist()
    assert p.ra_host.tolist() == O.reorder_indices(T, hint).tolist()

    natural = p.gemm_plain()
    p.gemm_signal()
    torch.cuda.synchronize()
    # counters: every group has seen exactly its tiles
    assert p.dMM.cpu()[:p.G].tolist() == p.cseg
    assert p.dMM.cpu()[p.G:].sum() == 0
    # placement: bit-exact against the oracle's epilogue applied to the natural GEMM, and to the oracle GEMM
    assert torch.equal(p.dC.cpu(), O.place_tiles(natural.cpu(), p.ra_host.numpy(), BM, BN, 1))
    assert torch.equal(p.dC.cpu(), O.place_tiles(O.gemm(p.A, p.B), p.ra_host.numpy(), BM, BN, 1))
    # same result with the reference's in-kernel linear scan instead of the table
    p.dMM.zero_()
    p.dC.zero_()
    p.gemm_signal(use_table=False)
    torch.cuda.synchronize()
    assert p.dMM.cpu()[:p.G].tolist() == p.cseg
    assert torch.equal(p.dC.cpu(), O.place_tiles(natural.cpu(), p.ra_host.numpy(), BM, BN, 1))


@pytest.mark.parametrize("dt,M,N,K,algo", [(torch.float16, 512, 1024, 128, 1), (torch.bfloat16, 1024, 512, 64, 1),
                                           (torch.bfloat16, 512, 1024, 64, 3), (torch.float16, 2048, 4096, 64, 1)])
def test_signal_rldn_tn_identity_equals_plain_gemm(L, dev, dt, M, N, K, algo):
    """rLDN = TN with the identity RA makes the permuted view the natural row-major [M, N]
    (src/overlap/gemm_with_signal.h:149-165): the signalling kernel, and the scatter kernel with an
    identity RE, must then write exactly what the plain GEMM writes."""
    _say("signal rLDN=TN identity", dt, M, N, K, algo)
    BM, BN, _ = capi.algo_tile(algo)
    TN = N // BN
    T = (M // BM) * TN
    p = Path(L, dev, dt, M, N, K, algo, cseg=O.uniform_cseg(T, 3), hint=list(range(T)), seed=11)
    assert p.ra_host.tolist() == list(range(T))
    p.build_table()
    natural = p.gemm_plain()
    p.gemm_signal(rldn=TN)
    torch.cuda.synchronize()
    assert torch.equal(p.dC.view(M, N), natural)
    assert p.dMM.cpu()[:p.G].tolist() == p.cseg
    # scatter kernel, identity row map
    p.dRE = torch.arange(M * N // BN, dtype=torch.int32, device=dev)
    p.dC.zero_()
    p.dMM.zero_()
    p.gemm_signal(rldn=TN)
    torch.cuda.synchronize()
    assert torch.equal(p.dC.view(M, N), natural)
    assert p.dMM.cpu()[:p.G].tolist() == p.cseg


@pytest.mark.parametrize("dt,M,N,K,algo,rldn", [(torch.float16, 512, 1024, 128, 1, 2), (torch.bfloat16, 1024, 1024, 64, 1, 4),
                                                (torch.bfloat16, 1024, 2048, 64, 3, 2), (torch.float16, 2048, 2048, 64, 5, 8),
                                                (torch.bfloat16, 2048, 4096, 64, 1, 16)])
def test_signal_and_scatter_general_rldn(L, dev, dt, M, N, K, algo, rldn):
    """rLDN > 1 with a random RA (and, for the scatter kernel, a random row permutation RE of the
    [M*N/(rLDN*BN), rLDN*BN] view) against the oracle's epilogues, bit-exact."""
    _say("signal rLDN", dt, M, N, K, algo, rldn)
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    rng = np.random.default_rng(rldn * 31 + algo)
    p = Path(L, dev, dt, M, N, K, algo, cseg=O.uniform_cseg(T, 5), hint=rng.permutation(T).tolist(),
             integer_inputs=True, seed=rldn)
    p.build_table()
    p.gemm_signal(rldn=rldn)
    torch.cuda.synchronize()
    natural = O.gemm(p.A, p.B)
    assert torch.equal(p.dC.cpu(), O.place_tiles(natural, p.ra_host.numpy(), BM, BN, rldn))
    assert p.dMM.cpu()[:p.G].tolist() == p.cseg
    rows = M * N // (rldn * BN)                      # rows of the permuted view
    re = np.arange(M * N // BN, dtype=np.int32)
    re[:rows] = rng.permutation(rows).astype(np.int32)
    p.dRE = torch.from_numpy(re).to(dev)
    p.dC.zero_()
    p.dMM.zero_()
    p.gemm_signal(rldn=rldn)
    torch.cuda.synchronize()
    assert torch.equal(p.dC.cpu(), O.scatter_place(natural, p.ra_host.numpy(), re, BM, BN, rldn))
    assert p.dMM.cpu()[:p.G].tolist() == p.cseg


def test_group_table_edge_cases(L, dev):
    for cseg, T in (([5], 5), ([1] * 300, 300), ([0, 3, 0, 0, 2, 1], 6), ([2000, 48], 2048), ([3, 3], 8)):
        d = torch.tensor(cseg, dtype=torch.int32, device=dev)
        table = torch.full((T,), -7, dtype=torch.int32, device=dev)
        capi.check(L.fo_build_group_table(d.data_ptr(), len(cseg), T, table.data_ptr(), None))
        torch.cuda.synchronize()
        covered = min(T, sum(cseg))
        assert table.cpu()[:covered].tolist() == O.group_of_slots(cseg, range(covered)).tolist()
        assert (table.cpu()[covered:] == len(cseg) - 1).all()  # beyond sum(cSeg): clamped, stays in bounds


def test_monitor_mode_tickets(L, dev):
    # tune/search.py:164-187: identity RA, MM of (TM+1) x TN, tickets in MM[1:, :]
    M = N = 2048
    K = 64
    BM = BN = 128
    T = 256
    TN = N // BN
    cseg = O.uniform_cseg(T, 64)
    p = Path(L, dev, torch.float16, M, N, K, 1, cseg=cseg, hint=list(range(T)), monitor=True, integer_inputs=True)
    p.build_table()
    p.gemm_signal()
    torch.cuda.synchronize()
    mm = p.dMM.cpu()
    tickets = mm[TN:].tolist()
    assert sorted(tickets) == list(range(T))          # a permutation of 0..T-1
    assert mm[TN - 1] == T                            # the ticket counter
    assert mm[:len(cseg)].tolist() == cseg            # group counters untouched by the tickets


@pytest.mark.parametrize("ws,cseg_w", [(2, 3), (8, 4), (4, 16)])
def test_scatter_epilogue_and_reducescatter_slices(L, dev, comm_stream, ws, cseg_w):
    M, N, K, algo = 1024, 512, 128, 1
    _say("scatter", ws, cseg_w)
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    cseg = O.uniform_cseg(T, cseg_w)
    p = Path(L, dev, torch.bfloat16, M, N, K, algo, cseg=cseg, ws=ws, integer_inputs=True, seed=7)
    assert p.re_host.tolist() == O.row_remap(M, N, BM, BN, cseg, ws).tolist()
    p.build_table()
    p.gemm_signal()
    torch.cuda.synchronize()
    natural = O.gemm(p.A, p.B)
    want = O.scatter_place(natural, p.ra_host.numpy(), p.re_host.numpy(), BM, BN, 1)
    assert torch.equal(p.dC.cpu(), want)
    assert p.dMM.cpu()[:p.G].tolist() == cseg
    # consumer: all ws receive buffers side by side
    D = torch.zeros(ws, M * N // ws, dtype=p.dt, device=dev)
    torch.cuda.synchronize()         # the second stream is not ordered behind torch's: D must be cleared before it is written
    capi.check(L.fo_wait_consume(p.dcseg.data_ptr(), p.G, p.dMM.data_ptr(), p.dC.data_ptr(), D.data_ptr(), BM * BN,
                                 ws, 0, ws, M * N // ws, None, 4, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert _timeouts(L) == 0
    assert torch.equal(D.cpu(), O.consume_reducescatter(want, cseg, BM, BN, ws))
    assert p.dMM.cpu().sum() == 0
    # each slice is a permuted layout with tile height BM/ws of the rows m % ws == k;
    # reorder+RMSNorm with BM/ws on it equals RMSNorm of those rows
    for k in (0, ws - 1):
        out = p.reorder_rmsnorm(D[k], 1e-5, bs=M // ws, BM=BM // ws)
        torch.cuda.synchronize()
        ref = O.rmsnorm(natural[k::ws], p.gamma, 1e-5)
        assert O.rel_l2(out.cpu(), ref) < REL_L2_TOL and _max_abs_ok(out.cpu(), ref)
    # one rank's view: only slice 1
    one = torch.zeros(M * N // ws, dtype=p.dt, device=dev)
    torch.cuda.synchronize()
    p.gemm_signal()
    capi.check(L.fo_wait_consume(p.dcseg.data_ptr(), p.G, p.dMM.data_ptr(), p.dC.data_ptr(), one.data_ptr(), BM * BN,
                                 ws, 1, 1, 0, None, 2, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert torch.equal(one.cpu(), O.consume_reducescatter(want, cseg, BM, BN, ws)[1])


# ---- matrix edges that are odd multiples of 128 -----------------------------------

EDGE_SHAPES = [
    (1152, 512, 72, 3),     # 128x256 layout tile, M = 9 x 128: the last macro row is half inside
    (512, 640, 64, 5),      # 256x128 layout tile, N = 5 x 128: the last macro column is half inside
    (2944, 2944, 64, 1),    # 128x128, 23 x 23 tiles on 256x256 macro tiles: both edges and the corner
]


@pytest.mark.parametrize("M,N,K,algo", EDGE_SHAPES)
def test_half_macro_tiles_plain_signal_and_tickets(L, dev, M, N, K, algo):
    """M and N only have to be multiples of the layout tile, as in the reference
    (RA is [M/BM, N/BN], test/test.py:72-92); the 256x256 macro tile of this
    kernel then hangs over the edge and must store and signal only what is inside."""
    _say("edge", M, N, K, algo)
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    hint = tiling.raster_hint(M, N, algo)
    assert sorted(hint) == list(range(T))                    # every layout tile issued exactly once
    cseg = O.uniform_cseg(T, 7)
    p = Path(L, dev, torch.bfloat16, M, N, K, algo, cseg=cseg, hint=hint, integer_inputs=True, seed=13)
    p.build_table()
    guard = 4096                                             # nothing may be written past the outputs
    nat = torch.full((M * N + guard,), 7.0, dtype=p.dt, device=dev)
    p.gemm_plain(out=nat)
    p.dC = torch.full((M * N + guard,), 7.0, dtype=p.dt, device=dev)
    p.gemm_signal()
    torch.cuda.synchronize()
    want = O.gemm(p.A, p.B)
    assert torch.equal(nat[:M * N].cpu().view(M, N), want)
    assert (nat[M * N:] == 7.0).all() and (p.dC[M * N:] == 7.0).all()
    assert torch.equal(p.dC[:M * N].cpu(), O.place_tiles(want, p.ra_host.numpy(), BM, BN, 1))
    assert p.dMM.cpu()[:p.G].tolist() == cseg and p.dMM.cpu()[p.G:].sum() == 0
    # monitor mode: one ticket per layout tile, none for the parts outside
    TN = N // BN
    m = Path(L, dev, torch.bfloat16, M, N, K, algo, cseg=[T], hint=hint, monitor=True, integer_inputs=True, seed=13)
    m.gemm_signal(use_table=False)
    torch.cuda.synchronize()
    mm = m.dMM.cpu()
    assert sorted(mm[TN:].tolist()) == list(range(T)) and mm[TN - 1] == T and mm[0] == T


def test_half_macro_tiles_scatter(L, dev):
    M, N, K, algo, ws = 1152, 1024, 64, 3, 4     # 9 x 4 tiles of 128x256 -> 5 x 4 macro tiles, the last row half inside
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    _say("edge scatter", M, N, K)
    cseg = O.uniform_cseg(T, 20)
    p = Path(L, dev, torch.float16, M, N, K, algo, cseg=cseg, ws=ws, integer_inputs=True, seed=17)
    p.build_table()
    p.gemm_signal()
    torch.cuda.synchronize()
    want = O.scatter_place(O.gemm(p.A, p.B), p.ra_host.numpy(), p.re_host.numpy(), BM, BN, 1)
    assert torch.equal(p.dC.cpu(), want)
    assert p.dMM.cpu()[:p.G].tolist() == cseg


# ---- seeded random shapes ---------------------------------------------------------

def _random_problem(seed):
    """A shape the library accepts, drawn from a seed: any Algo, M and N multiples of its tile, K a
    multiple of 8, a ragged partition of the tiles into groups and a random slot permutation."""
    rng = np.random.default_rng(seed)
    algo = int(rng.integers(0, 6))
    BM, BN, _ = capi.algo_tile(algo)
    M = BM * int(rng.integers(1, 2560 // BM + 1))
    N = BN * int(rng.integers(1, 2560 // BN + 1))
    K = 8 * int(rng.integers(1, 41))
    T = (M // BM) * (N // BN)
    cuts = sorted(rng.choice(np.arange(1, T), size=min(T - 1, int(rng.integers(0, 6))), replace=False).tolist()) if T > 1 else []
    cseg = np.diff([0] + cuts + [T]).tolist()
    return algo, M, N, K, T, cseg, rng.permutation(T).tolist()


@pytest.mark.parametrize("seed", range(100, 116))
def test_random_shapes_plain_and_signal_bit_exact(L, dev, seed):
    algo, M, N, K, T, cseg, hint = _random_problem(seed)
    dt = torch.float16 if seed % 2 else torch.bfloat16
    _say("random shape", seed, dt, M, N, K, algo, cseg)
    BM, BN, _ = capi.algo_tile(algo)
    p = Path(L, dev, dt, M, N, K, algo, cseg=cseg, hint=hint, integer_inputs=True, seed=seed)
    p.build_table()
    want = O.gemm(p.A, p.B)
    assert torch.equal(p.gemm_plain().cpu(), want)
    p.gemm_signal(use_table=bool(seed & 2))
    torch.cuda.synchronize()
    assert torch.equal(p.dC.cpu(), O.place_tiles(want, p.ra_host.numpy(), BM, BN, 1))
    assert p.dMM.cpu()[:p.G].tolist() == cseg and p.dMM.cpu()[p.G:].sum() == 0


@pytest.mark.parametrize("seed", range(200, 208))
def test_random_shapes_scatter_bit_exact(L, dev, seed):
    algo, M, N, K, T, cseg, hint = _random_problem(seed)
    ws = (2, 4, 8)[seed % 3]
    _say("random scatter", seed, M, N, K, algo, ws, cseg)
    BM, BN, _ = capi.algo_tile(algo)
    p = Path(L, dev, torch.bfloat16, M, N, K, algo, cseg=cseg, hint=hint, ws=ws, integer_inputs=True, seed=seed)
    assert p.re_host.tolist() == O.row_remap(M, N, BM, BN, cseg, ws).tolist()
    p.build_table()
    p.gemm_signal()
    torch.cuda.synchronize()
    want = O.scatter_place(O.gemm(p.A, p.B), p.ra_host.numpy(), p.re_host.numpy(), BM, BN, 1)
    assert torch.equal(p.dC.cpu(), want)
    assert p.dMM.cpu()[:p.G].tolist() == cseg


# ---- wait / consume ------------------------------------------------------------

def test_wait_kernel_resets_counter_and_is_bounded(L, dev, comm_stream):
    mm = torch.tensor([3, 9], dtype=torch.int32, device=dev)
    capi.check(L.fo_wait(3, mm.data_ptr(), None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert mm.cpu().tolist() == [0, 9] and _timeouts(L) == 0
    # a count that is never reached: the waiter gives up after the limit, leaves
    # the counter alone and the stream carries on (the reference would spin forever)
    capi.check(L.fo_set_wait_timeout_ms(50))
    try:
        capi.check(L.fo_wait(5, mm.data_ptr() + 4, None, comm_stream))
        capi.check(L.fo_stream_sync(comm_stream))
        assert mm.cpu().tolist() == [0, 9] and _timeouts(L) == 1
        src = torch.arange(4096, dtype=torch.int16, device=dev)
        dst = torch.zeros_like(src)
        bad = torch.tensor([1, 1], dtype=torch.int32, device=dev)
        flags = torch.tensor([1, 0], dtype=torch.int32, device=dev)   # group 1 never completes
        torch.cuda.synchronize()     # src and dst are filled on torch's stream, the consumer runs on another
        capi.check(L.fo_wait_consume(bad.data_ptr(), 2, flags.data_ptr(), src.data_ptr(), dst.data_ptr(), 2048, 1, 0,
                                     1, 0, None, 3, None, comm_stream))
        capi.check(L.fo_stream_sync(comm_stream))
        assert _timeouts(L) == 1                      # the one workgroup that owns the small group reports it
        assert flags.cpu().tolist() == [0, 0]         # (the full counter was reset, the short one left as it was)
        # like the copy behind an expired wait kernel, the copy of the incomplete group is still made
        assert torch.equal(dst, src)
    finally:
        capi.check(L.fo_set_wait_timeout_ms(5000))


def test_settle_consume_clears_the_right_count_and_reports_a_wrong_one(L, dev, comm_stream):
    """The last group's launch: behind its producer on one stream the counter is final, so the
    launch checks it instead of waiting (same outcome as src/wait.cuh:5-9 on the right count)."""
    mm = torch.tensor([7, 9, 0], dtype=torch.int32, device=dev)
    src = torch.randint(-30000, 30000, (40000,), dtype=torch.int16, device=dev)
    dst = torch.zeros_like(src)
    torch.cuda.synchronize()         # filled on torch's stream, copied on another that is not ordered behind it
    capi.check(L.fo_settle_consume(7, mm.data_ptr(), src.data_ptr(), dst.data_ptr(), 2 * 40000, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert mm.cpu().tolist() == [0, 9, 0] and _timeouts(L) == 0 and torch.equal(dst, src)
    # a wrong count stays where it is and is counted, at once (no polling); the copy is still made
    dst.zero_()
    torch.cuda.synchronize()
    capi.check(L.fo_settle_consume(8, mm.data_ptr() + 4, src.data_ptr(), dst.data_ptr(), 2 * 40000, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert mm.cpu().tolist() == [0, 9, 0] and _timeouts(L) == 1 and torch.equal(dst, src)
    # an empty group still settles its counter
    capi.check(L.fo_settle_consume(0, mm.data_ptr() + 8, src.data_ptr(), dst.data_ptr(), 0, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert mm.cpu().tolist() == [0, 9, 0] and _timeouts(L) == 0
    assert L.fo_settle_consume(0, None, src.data_ptr(), dst.data_ptr(), 16, None, comm_stream) == capi.FO_ERR_ARG


def test_consume_slices_equals_one_copy_per_slice(L, dev, comm_stream):
    """One launch for all ranks' slices of a group (one collective call per group,
    src/overlap_impl.cu:319-320) against fo_consume slice by slice."""
    ws, part, stride = 8, 4096 * 5, 40000            # elements; stride > part: gaps between the receive buffers
    src = torch.randint(-30000, 30000, (ws * part + 64,), dtype=torch.int16, device=dev)
    want = torch.full((ws * stride,), -1, dtype=torch.int16, device=dev)
    got = want.clone()
    torch.cuda.synchronize()         # filled on torch's stream, copied on another that is not ordered behind it
    for k in range(ws):
        capi.check(L.fo_consume(src.data_ptr() + 2 * (64 + k * part), want.data_ptr() + 2 * k * stride, 2 * part,
                                comm_stream))
    capi.check(L.fo_consume_slices(0, None, src.data_ptr() + 2 * 64, got.data_ptr(), 2 * part, ws, 2 * stride,
                                   capi.FO_COPY_STREAM, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert torch.equal(got, want)
    assert (got.view(ws, stride)[:, part:] == -1).all()      # nothing written between the slices
    # with a counter: settled once, by the launch as a whole
    mm = torch.tensor([5], dtype=torch.int32, device=dev)
    got.fill_(-1)
    torch.cuda.synchronize()
    capi.check(L.fo_consume_slices(5, mm.data_ptr(), src.data_ptr() + 2 * 64, got.data_ptr(), 2 * part, ws, 2 * stride,
                                   capi.FO_COPY_CACHED, None, comm_stream))
    capi.check(L.fo_stream_sync(comm_stream))
    assert torch.equal(got, want) and mm.item() == 0 and _timeouts(L) == 0
    # slices that are not whole 16-byte units are refused
    assert L.fo_consume_slices(0, None, src.data_ptr(), got.data_ptr(), 2 * 4100, 2, 2 * stride, capi.FO_COPY_AUTO, None,
                               comm_stream) == capi.FO_ERR_SHAPE
    assert L.fo_consume_slices(0, None, src.data_ptr(), got.data_ptr(), 2 * 4096, 2, 2 * stride, 7, None,
                               comm_stream) == capi.FO_ERR_ARG


def test_consume_copies_exactly_the_bytes(L, dev):
    src = torch.randint(-30000, 30000, (100003,), dtype=torch.int16, device=dev)
    for off, n in ((0, 100003), (8, 77), (16, 8), (24, 4099)):
        dst = torch.full_like(src, -1)
        capi.check(L.fo_consume(src.data_ptr() + 2 * off, dst.data_ptr() + 2 * off, 2 * n, None))
        torch.cuda.synchronize()
        assert torch.equal(dst[off:off + n], src[off:off + n])
        assert (dst[:off] == -1).all() and (dst[off + n:] == -1).all()


@pytest.mark.parametrize("mode", ["per_group", "persistent"])
def test_overlapped_release_order_and_staging(L, dev, comm_stream, mode):
    """GEMM on one stream, waiter/consumer on another, started together; run
    twice with different A so that a stale cache line in the consumer would show."""
    M, N, K, algo = 2048, 2048, 512, 1
    BM, BN, _ = capi.algo_tile(algo)
    T = 256
    cseg = [40, 24, 64, 1, 127]
    _say("overlap", mode)
    p = Path(L, dev, torch.float16, M, N, K, algo, cseg=cseg, integer_inputs=True, seed=11)
    p.build_table()
    staging = torch.zeros(M * N, dtype=p.dt, device=dev)
    log = torch.full((p.G,), -1, dtype=torch.int32, device=dev)
    for rep in range(2):
        if rep == 1:
            p.A = -p.A
            p.dA = p.A.to(dev)
        staging.zero_()
        torch.cuda.synchronize()
        p.gemm_signal()
        if mode == "persistent":
            capi.check(L.fo_wait_consume(p.dcseg.data_ptr(), p.G, p.dMM.data_ptr(), p.dC.data_ptr(),
                                         staging.data_ptr(), BM * BN, 1, 0, 1, 0, log.data_ptr(), 6, None, comm_stream))
        else:
            acc = 0
            for g, n in enumerate(cseg):
                capi.check(L.fo_wait(n, p.dMM.data_ptr() + 4 * g, None, comm_stream))
                capi.check(L.fo_consume(p.dC.data_ptr() + 2 * acc, staging.data_ptr() + 2 * acc, 2 * n * BM * BN,
                                        comm_stream))
                acc += n * BM * BN
        capi.check(L.fo_stream_join(comm_stream, None))
        torch.cuda.synchronize()
        assert _timeouts(L) == 0
        want = O.place_tiles(O.gemm(p.A, p.B), p.ra_host.numpy(), BM, BN, 1)
        assert torch.equal(p.dC.cpu(), want)
        assert torch.equal(staging.cpu(), O.consume_allreduce(want, cseg, BM, BN))
        assert p.dMM.cpu().sum() == 0                     # every counter back to zero for the next call
        if mode == "persistent":
            assert log.cpu().tolist() == list(range(p.G))  # released in index order


# ---- RMSNorm -------------------------------------------------------------------

@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bs,dim", [(4, 8), (7, 520), (33, 1024), (16, 4096), (5, 8192), (3, 16384), (9, 4104)])
def test_plain_rmsnorm(L, dev, dt, bs, dim):
    g = torch.Generator().manual_seed(bs * dim)
    x = torch.randn(bs, dim, generator=g).to(dt)
    gamma = (1 + 0.1 * torch.randn(dim, generator=g)).to(dt)
    out = torch.empty(bs, dim, dtype=dt, device=dev)
    dx, dgamma = x.to(dev), gamma.to(dev)
    capi.check(L.fo_rmsnorm(capi.dtype_code(dt), dx.data_ptr(), dgamma.data_ptr(), out.data_ptr(), bs, dim, 1e-5, None))
    torch.cuda.synchronize()
    ref = O.rmsnorm(x, gamma, 1e-5)
    assert O.rel_l2(out.cpu(), ref) < REL_L2_TOL and O.max_abs(out.cpu(), ref) < MAX_ABS_TOL
    # same two-rounding order as the reference kernel: within two storage ulps of the oracle
    ulp = 2 ** -10 if dt == torch.float16 else 2 ** -7
    assert ((out.cpu().float() - ref.float()).abs() <= 2 * ulp * ref.float().abs() + 1e-6).all()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bs,dim,BM,BN,rldn", [(256, 512, 128, 128, 1), (256, 512, 128, 128, 2), (128, 1024, 64, 256, 1),
                                               (64, 384, 16, 8, 1), (96, 4096, 32, 128, 1)])
def test_reorder_rmsnorm(L, dev, dt, bs, dim, BM, BN, rldn):
    g = torch.Generator().manual_seed(dim + BM)
    Cn = torch.randn(bs, dim, generator=g).to(dt)
    gamma = (1 + 0.1 * torch.randn(dim, generator=g)).to(dt)
    T = (bs // BM) * (dim // BN)
    ra = O.reorder_indices(T, np.random.default_rng(T).permutation(T))
    x = O.place_tiles(Cn, ra, BM, BN, rldn)
    out = torch.empty(bs, dim, dtype=dt, device=dev)
    dx, dgamma, dra = x.to(dev), gamma.to(dev), torch.from_numpy(ra).to(dev)
    capi.check(L.fo_reorder_rmsnorm(capi.dtype_code(dt), dx.data_ptr(), dgamma.data_ptr(), out.data_ptr(), bs, dim,
                                    BM, BN, rldn, dra.data_ptr(), 1e-6, None))
    torch.cuda.synchronize()
    ref = O.reorder_rmsnorm(x, gamma, bs, dim, BM, BN, rldn, ra, 1e-6)
    assert torch.equal(ref, O.rmsnorm(Cn, gamma, 1e-6))
    assert O.rel_l2(out.cpu(), ref) < REL_L2_TOL and O.max_abs(out.cpu(), ref) < MAX_ABS_TOL
    # eps really is a parameter: a large one changes the result the way the formula says
    capi.check(L.fo_reorder_rmsnorm(capi.dtype_code(dt), dx.data_ptr(), dgamma.data_ptr(), out.data_ptr(), bs, dim,
                                    BM, BN, rldn, dra.data_ptr(), 3.0, None))
    torch.cuda.synchronize()
    ref3 = O.rmsnorm(Cn, gamma, 3.0)
    assert O.rel_l2(out.cpu(), ref3) < REL_L2_TOL


# ---- the five benchmark configurations, full size ------------------------------------------

def _full_path(L, dev, comm_stream, dt, M, N, K, w, eps, ws=1, a_std=None, b_std=None, check_rows=None):
    """Whole hot path on random inputs at full size: signalling GEMM overlapped
    with the persistent consumer, then reorder+RMSNorm, against the oracle."""
    algo = 1
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    cseg = O.uniform_cseg(T, w)
    p = Path(L, dev, dt, M, N, K, algo, cseg=cseg, ws=ws, a_std=a_std, b_std=b_std)
    p.build_table()
    dst = torch.zeros(M * N, dtype=dt, device=dev)
    p.gemm_signal()
    capi.check(L.fo_wait_consume(p.dcseg.data_ptr(), p.G, p.dMM.data_ptr(), p.dC.data_ptr(), dst.data_ptr(), BM * BN,
                                 ws, 0, ws, M * N // ws if ws > 1 else 0, None, 8, None, comm_stream))
    capi.check(L.fo_stream_join(comm_stream, None))
    torch.cuda.synchronize()
    assert _timeouts(L) == 0
    assert p.dMM.cpu().sum() == 0
    if ws == 1:
        if not torch.equal(dst, p.dC):                     # staging is the permuted C, bit for bit
            bad = (dst != p.dC).view(T, BM * BN)
            slots = bad.any(1).nonzero().flatten().tolist()
            first = bad[slots[0]].view(BM, BN)
            raise AssertionError(
                "staging differs from C in %d slots (first %s): rows %s of slot %d, %d of its bad elements are 0 in staging"
                % (len(slots), slots[:12], first.any(1).nonzero().flatten().tolist()[:16], slots[0],
                   int((dst.view(T, BM * BN)[slots[0]][bad[slots[0]]] == 0).sum())))
        out = p.reorder_rmsnorm(dst, eps)
        torch.cuda.synchronize()
        rows = torch.arange(M) if check_rows is None else check_rows
        got = out.cpu()[rows]
        src_rows = rows
    else:
        # every slice k holds the rows m % ws == k as a layout with tile height BM/ws
        outs = [p.reorder_rmsnorm(dst.view(ws, -1)[k], eps, bs=M // ws, BM=BM // ws) for k in range(ws)]
        torch.cuda.synchronize()
        full = torch.empty(M, N, dtype=dt)
        for k in range(ws):
            full[k::ws] = outs[k].cpu()
        rows = torch.arange(M) if check_rows is None else check_rows
        got = full[rows]
        src_rows = rows
    c32 = O.gemm_fp32(p.A[src_rows], p.B)
    gated = O.rmsnorm(c32.to(dt), p.gamma, eps)
    unq = O.rmsnorm_fp32(c32, p.gamma, eps)
    _say("  vs unquantised fp32: rel-L2 %.2e max-abs %.2e" % (O.rel_l2(got, unq), O.max_abs(got, unq)))
    _say("  vs storage-matched : rel-L2 %.2e max-abs %.2e" % (O.rel_l2(got, gated), O.max_abs(got, gated)))
    assert O.rel_l2(got, gated) < REL_L2_TOL and _max_abs_ok(got, gated)
    # permutation invariants at full size: un-permuting the signalled output gives the plain kernel's output
    natural = p.gemm_plain()
    torch.cuda.synchronize()
    if ws == 1:
        back = p.dC.view(T, BM, BN)[p.dRA.view(-1).long()].view(p.TM, p.TN, BM, BN).permute(0, 2, 1, 3).reshape(M, N)
        assert torch.equal(back, natural)
    return p


def test_config1_fp16_1024(L, dev, comm_stream):
    _say("config 1")
    _full_path(L, dev, comm_stream, torch.float16, 1024, 1024, 1024, 4, 1e-6)


@pytest.mark.parametrize("w", [1, 2, 4, 8, 16])
def test_config2_fp16_4096_group_sweep(L, dev, comm_stream, w):
    _say("config 2, group size", w)
    rows = torch.arange(0, 4096, 37)
    _full_path(L, dev, comm_stream, torch.float16, 4096, 4096, 4096, w, 1e-5, check_rows=rows)


def test_config3_bf16_llama8b_down_proj(L, dev, comm_stream):
    _say("config 3")
    rows = torch.arange(0, 8192, 61)
    _full_path(L, dev, comm_stream, torch.bfloat16, 8192, 4096, 7168, 256, 1e-5, a_std=1.0, b_std=0.02,
               check_rows=rows)


def test_config4_bf16_small_k_many_groups(L, dev, comm_stream):
    _say("config 4")
    rows = torch.arange(0, 16384, 251)
    _full_path(L, dev, comm_stream, torch.bfloat16, 16384, 8192, 1024, 2, 1e-5, check_rows=rows)


def test_config5_bf16_reducescatter_layout(L, dev, comm_stream):
    _say("config 5")
    rows = torch.arange(0, 8192, 127)
    _full_path(L, dev, comm_stream, torch.bfloat16, 8192, 8192, 3584, 256, 1e-5, ws=8, check_rows=rows)
