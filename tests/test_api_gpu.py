"""GPU tests of the torch-visible API, written the way the reference's own
scripts drive it (test/test.py:126-197, example/correctness_ar.py:99-127,
example/correctness_rs.py:100-142, example/RMSNorm.py:23-37), on one GPU."""
import numpy as np
import pytest
import torch

import flashoverlap_amd
from flashoverlap_amd import capi, tiling
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api(dev):
    flashoverlap_amd.load()
    capi.check(capi.lib().fo_set_wait_timeout_ms(5000))
    return torch.classes.flashoverlap_class


def _overlap(api, rank=0, size=1):
    o = api.OverlapImpl()
    o.mccl_init(rank, size, torch.ops.flashoverlap_op.generate_mccl_id())
    o.mutlass_init()
    o.overlap_init()
    return o


def _timeouts(*objects):
    """Expired waits: those counted in the words the given OverlapImpl objects own, plus those of
    callers that passed no word of their own (the per-device count of the C ABI)."""
    import ctypes
    n = ctypes.c_int()
    capi.check(capi.lib().fo_wait_timeouts(ctypes.byref(n), 1))
    return n.value + sum(o.wait_timeouts(True) for o in objects)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_mutlass_and_mublas_gemm(api, dev, dt):
    M, N, K = 512, 768, 256
    g = torch.Generator().manual_seed(0)
    A = torch.randint(-2, 3, (M, K), generator=g).to(dt).to(dev)
    B = torch.randint(-2, 3, (N, K), generator=g).to(dt).to(dev)
    want = O.gemm(A.cpu(), B.cpu())
    o = _overlap(api)
    C = torch.empty(M, N, dtype=dt, device=dev)
    o.mutlass_gemm(A, B, C, 1)
    torch.cuda.synchronize()
    assert torch.equal(C.cpu(), want)
    b = api.BaselineImpl()
    b.mccl_init(0, 1, torch.ops.flashoverlap_op.generate_mccl_id())
    b.mublas_init()
    C2 = torch.empty(M, N, dtype=dt, device=dev)
    b.mublas_gemm(A, B, C2)
    b.gemm_allreduce(A, B, C2)
    torch.cuda.synchronize()
    assert torch.equal(C2.cpu(), want)
    assert torch.equal(b.staging().cpu().view(M, N), want)


@pytest.mark.parametrize("mode", [1, 2])
def test_allreduce_overlap_like_correctness_ar(api, dev, mode):
    """All-ones A and B as in example/correctness_ar.py:104-106: every C element
    is K, so only the permutation and the norm are exercised; then seeded
    random inputs so the GEMM is exercised too."""
    M, N, K, algo = 1024, 1024, 1024, 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    hint = tiling.raster_hint(M, N, algo)
    cseg = tiling.uniform_cseg(T, 4)                       # 16 groups, more than TN = 8
    cSeg_CPU = torch.tensor(cseg, dtype=torch.int32)
    cSeg_GPU = cSeg_CPU.to(dev)
    counter = torch.zeros(len(cseg), dtype=torch.int32, device=dev)
    RA = tiling.reorder_indices(T, hint, dev).reshape(TM, TN)
    o = _overlap(api)
    o.set_consumer_mode(mode)
    g = torch.Generator().manual_seed(1)
    W = (torch.randn(N, generator=g) * 0.5).to(torch.float16).to(dev)
    cases = [(torch.ones(M, K, dtype=torch.float16), torch.ones(N, K, dtype=torch.float16)),
             ((torch.randn(M, K, generator=g) / K ** 0.5).half(), (torch.randn(N, K, generator=g) / K ** 0.5).half())]
    for A, B in cases:
        C = torch.empty(M, N, dtype=torch.float16, device=dev)
        o.gemm_allreduce_overlap(A.to(dev), B.to(dev), C, counter, RA, 1, cSeg_CPU, cSeg_GPU, algo, False)
        y = torch.empty(M, N, dtype=torch.float16, device=dev)
        torch.ops.flashoverlap_op.reorder_rmsnorm(o.staging().view(M, N), y, W, BM, BN, 1, RA)
        torch.cuda.synchronize()
        assert _timeouts(o) == 0
        assert counter.cpu().sum() == 0
        cref = O.gemm(A, B)
        # placement bit-exact: the staging buffer is the plain GEMM of the same kernel, permuted by the oracle
        nat = torch.empty(M, N, dtype=torch.float16, device=dev)
        o.mutlass_gemm(A.to(dev), B.to(dev), nat, algo)
        torch.cuda.synchronize()
        assert torch.equal(o.staging().cpu(), O.place_tiles(nat.cpu(), RA.cpu().numpy(), BM, BN, 1))
        # values: against the oracle's GEMM (accumulation order may differ by one storage ulp)
        assert O.rel_l2(nat.cpu(), cref) < 1e-3 and O.max_abs(nat.cpu(), cref) < 2e-2
        ref = O.rmsnorm(cref, W.cpu(), 1e-5)
        assert torch.allclose(y.cpu().float(), ref.float(), atol=1e-2, rtol=1e-2)      # the reference's own bar
        assert O.rel_l2(y.cpu(), ref) < 1e-3 and O.max_abs(y.cpu(), ref) < 2e-2


@pytest.mark.parametrize("stacked", [False, True])
def test_reducescatter_overlap_like_correctness_rs(api, dev, stacked):
    """example/correctness_rs.py:100-142 with an emulated world of 4: rank k's
    receive buffer, normalised with BM // world_size, equals RMSNorm of the
    rows k, k+ws, ... of the product."""
    M, N, K, algo, ws, rank = 1024, 512, 256, 1, 4, 2
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    hint = tiling.raster_hint(M, N, algo)
    cseg = [5, 11, 16]
    cSeg_CPU = torch.tensor(cseg, dtype=torch.int32)
    cSeg_GPU = cSeg_CPU.to(dev)
    counter = torch.zeros(TN, dtype=torch.int32, device=dev)
    RA = tiling.reorder_indices(T, hint, dev).reshape(TM, TN)
    RE = tiling.generate_row_remap_array(M, N, BM, BN, cseg, ws, dev)
    g = torch.Generator().manual_seed(2)
    A0 = (torch.randn(M, K, generator=g) * 0.5).to(torch.bfloat16)
    B = (torch.randn(N, K, generator=g) * 0.5).to(torch.bfloat16)
    W = (torch.randn(N, generator=g) * 0.5).to(torch.bfloat16)
    o = _overlap(api, rank, ws)
    tmp = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    out = torch.zeros((ws, M // ws, N) if stacked else (M // ws, N), dtype=torch.bfloat16, device=dev)
    o.gemm_reducescatter_overlap(A0.to(dev), B.to(dev), tmp, out, counter, RA, RE, 1, cSeg_CPU, cSeg_GPU, algo, False)
    torch.cuda.synchronize()
    assert _timeouts(o) == 0 and counter.cpu().sum() == 0
    cref = O.gemm(A0, B)
    slices = O.consume_reducescatter(O.scatter_place(cref, RA.cpu().numpy(), RE.cpu().numpy(), BM, BN, 1), cseg, BM,
                                     BN, ws)
    mine = out[rank] if stacked else out
    if stacked:
        assert O.rel_l2(out.cpu().view(ws, -1), slices) < 1e-3
    assert O.rel_l2(mine.cpu().view(-1), slices[rank]) < 1e-3
    y = torch.empty(M // ws, N, dtype=torch.bfloat16, device=dev)
    torch.ops.flashoverlap_op.reorder_rmsnorm(mine.contiguous(), y, W.to(dev), BM // ws, BN, 1, RA)
    torch.cuda.synchronize()
    x1 = O.reorder_rows_by_world_size(cref, ws).view(ws, M // ws, N)[rank]      # what the reference compares against
    ref = O.rmsnorm(x1, W, 1e-5)
    assert torch.allclose(y.cpu().float(), ref.float(), atol=5e-2, rtol=5e-2)     # the reference's own bar
    assert O.rel_l2(y.cpu(), ref) < 2.5e-3  # bf16 output rounding of a storage-matched oracle, C itself may differ by an ulp


def test_monitor_pass_like_the_tuner(api, dev):
    # tune/search.py:164-187
    M, N, K, algo = 2048, 2048, 128, 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    cseg = tiling.uniform_cseg(T, 100)
    cSeg_CPU = torch.tensor(cseg, dtype=torch.int32)
    MonitoredMatrix = torch.zeros((TM + 1, TN), dtype=torch.int32, device=dev)
    ReorderedArray = torch.arange(0, T, dtype=torch.int32, device=dev).reshape(TM, TN)
    A = torch.randn(M, K, dtype=torch.float16, device=dev)
    B = torch.randn(N, K, dtype=torch.float16, device=dev)
    C = torch.empty(M, N, dtype=torch.float16, device=dev)
    o = _overlap(api)
    samples = torch.empty((3, T), dtype=torch.int32, device=dev)
    for i in range(3):
        MonitoredMatrix[0] = 0
        o.gemm_allreduce_overlap(A, B, C, MonitoredMatrix, ReorderedArray, 1, cSeg_CPU, cSeg_CPU.to(dev), algo, True)
        samples[i, :] = MonitoredMatrix[1:, :].view(-1)
    torch.cuda.synchronize()
    assert _timeouts(o) == 0
    for i in range(3):
        assert sorted(samples[i].cpu().tolist()) == list(range(T))
    assert MonitoredMatrix[0, TN - 1].item() == T


def test_api_argument_checks(api, dev):
    o = _overlap(api)
    M = N = K = 256
    A = torch.zeros(M, K, dtype=torch.float16, device=dev)
    C = torch.zeros(M, N, dtype=torch.float16, device=dev)
    RA = torch.arange(4, dtype=torch.int32, device=dev).reshape(2, 2)
    mm = torch.zeros(4, dtype=torch.int32, device=dev)
    good = torch.tensor([4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="sum\\(cSeg\\)"):
        bad = torch.tensor([3], dtype=torch.int32)
        o.gemm_allreduce_overlap(A, A, C, mm, RA, 1, bad, bad.to(dev), 1, False)
    with pytest.raises(RuntimeError, match="counters"):
        many = torch.tensor([1, 1, 1, 1], dtype=torch.int32)
        o.gemm_allreduce_overlap(A, A, C, mm[:2], RA, 1, many, many.to(dev), 1, False)
    with pytest.raises(RuntimeError, match="RA is"):
        o.gemm_allreduce_overlap(A, A, C, mm, RA.reshape(1, 4), 1, good, good.to(dev), 1, False)
    with pytest.raises(RuntimeError, match="dtype"):
        o.gemm_allreduce_overlap(A, A.bfloat16(), C, mm, RA, 1, good, good.to(dev), 1, False)
    with pytest.raises(RuntimeError, match="Algo"):
        o.mutlass_gemm(A, A, C, 17)
    with pytest.raises(RuntimeError, match="more than one GPU"):
        _overlap(api, 0, 2).gemm_all2all(A, A, C, C, 1, torch.zeros(2, 2, dtype=torch.int32))
    torch.cuda.synchronize()
    assert _timeouts(o) == 0


def test_expired_wait_is_reported_through_the_torch_api(api, dev):
    """A wait bound far below the GEMM's run time (forced from the host; every kernel still exits
    normally): in checked mode the overlapped call raises, the counters come back zeroed, and the
    same object then runs a correct call."""
    M, N, K, algo = 8192, 8192, 32768, 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    # two groups: the first one (released on the second stream, where the wait starts with the GEMM)
    # holds tiles of the GEMM's last round, so it completes only when the GEMM ends: more than 2 ms
    # even on constant operands at full clock (4.4 PFLOP of work), twice the 1 ms bound
    cSeg_CPU = torch.tensor([T - 256, 256], dtype=torch.int32)
    cSeg_GPU = cSeg_CPU.to(dev)
    counter = torch.zeros(TN, dtype=torch.int32, device=dev)
    RA = tiling.reorder_indices(T, tiling.raster_hint(M, N, algo), dev).reshape(TM, TN)
    A = torch.ones(M, K, dtype=torch.bfloat16, device=dev)
    B = torch.ones(N, K, dtype=torch.bfloat16, device=dev)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    o = _overlap(api)
    o.set_check_timeouts(True)
    assert o.wait_timeouts(True) == 0
    o.set_wait_timeout_ms(1)
    try:
        with pytest.raises(RuntimeError, match="expired"):
            o.gemm_allreduce_overlap(A, B, C, counter, RA, 1, cSeg_CPU, cSeg_GPU, algo, False)
    finally:
        o.set_wait_timeout_ms(5000)
    assert counter.cpu().sum() == 0 and o.wait_timeouts(False) == 0
    o.gemm_allreduce_overlap(A, B, C, counter, RA, 1, cSeg_CPU, cSeg_GPU, algo, False)
    torch.cuda.synchronize()
    assert o.wait_timeouts(True) == 0 and counter.cpu().sum() == 0
    assert (o.staging() == K).all()


def test_an_expired_wait_belongs_to_the_object_that_made_it(api, dev):
    """Two OverlapImpl objects on one device.  The first runs, unchecked, a call whose wait is
    forced to expire from the host (1 ms bound, a GEMM of more than 2 ms); the second, in checked
    mode, then runs a small correct call.  The expiry is counted in the first object's own word:
    the second neither raises nor has its counters cleared, reports no expiry, and the per-device
    word of callers that pass no word of their own stays at zero."""
    M, N, K, algo = 8192, 8192, 32768, 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    cSeg_CPU = torch.tensor([T - 256, 256], dtype=torch.int32)
    counter = torch.zeros(TN, dtype=torch.int32, device=dev)
    RA = tiling.reorder_indices(T, tiling.raster_hint(M, N, algo), dev).reshape(TM, TN)
    A = torch.ones(M, K, dtype=torch.bfloat16, device=dev)
    B = torch.ones(N, K, dtype=torch.bfloat16, device=dev)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    m, n, k = 512, 512, 256
    tm, tn = m // BM, n // BN
    cseg2 = torch.tensor([3, tm * tn - 3], dtype=torch.int32)
    counter2 = torch.zeros(tn, dtype=torch.int32, device=dev)
    ra2 = tiling.reorder_indices(tm * tn, tiling.raster_hint(m, n, algo), dev).reshape(tm, tn)
    a2 = torch.ones(m, k, dtype=torch.bfloat16, device=dev)
    b2 = torch.ones(n, k, dtype=torch.bfloat16, device=dev)
    c2 = torch.empty(m, n, dtype=torch.bfloat16, device=dev)
    first, second = _overlap(api), _overlap(api)
    second.set_check_timeouts(True)
    assert _timeouts() == 0
    first.set_wait_timeout_ms(1)          # process-wide: the small call below stays far inside it
    try:
        first.gemm_allreduce_overlap(A, B, C, counter, RA, 1, cSeg_CPU, cSeg_CPU.to(dev), algo, False)
        torch.cuda.synchronize()
        second.gemm_allreduce_overlap(a2, b2, c2, counter2, ra2, 1, cseg2, cseg2.to(dev), algo, False)   # must not raise
    finally:
        first.set_wait_timeout_ms(5000)
    torch.cuda.synchronize()
    assert second.wait_timeouts(False) == 0 and counter2.cpu().sum() == 0
    assert (second.staging() == k).all()
    assert first.wait_timeouts(True) == 1 and first.wait_timeouts(False) == 0
    assert counter.cpu()[0] == T - 256    # the unchecked caller's counters are its own to clear
    assert _timeouts() == 0
    counter.zero_()
    first.gemm_allreduce_overlap(A, B, C, counter, RA, 1, cSeg_CPU, cSeg_CPU.to(dev), algo, False)
    torch.cuda.synchronize()
    assert first.wait_timeouts(True) == 0 and counter.cpu().sum() == 0 and (first.staging() == K).all()


def test_consumer_blocks_are_limited_to_the_cu_count(api, dev):
    o = _overlap(api)
    o.set_consumer_blocks(256)
    with pytest.raises(RuntimeError, match="one workgroup per CU"):
        o.set_consumer_blocks(100000)
