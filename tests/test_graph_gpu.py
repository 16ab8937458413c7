"""The overlapped call captured into a graph and replayed.

The reference's call (src/overlap_impl.cu:221-271) starts work on its second
stream without ordering it behind the caller's stream, so stream capture cannot
follow it there.  Here the call forks the second stream off the caller's before
the GEMM and joins it back at the end, which makes GEMM || wait+copy -> RMSNorm
one capturable unit of kernels (no memset nodes, no allocation after the first
call).  Every replay is checked bit for bit against the same call made eagerly,
with new operand values and eager work between the replays."""
import pytest
import torch

import flashoverlap_amd
from flashoverlap_amd import capi, tiling

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("w,mode", [(16, 1), (4, 2)])   # 4 groups released one by one; 16 groups, persistent consumer
def test_overlapped_call_replays_from_a_graph(dev, w, mode):
    flashoverlap_amd.load()
    # a wait that cannot be satisfied (graph branches run in the wrong order) must fail the test, not stall it
    capi.check(capi.lib().fo_set_wait_timeout_ms(2000))
    M, N, K, algo = 1024, 1024, 512, 1
    dt = torch.bfloat16
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    cseg = tiling.uniform_cseg(T, w)
    cSeg_CPU = torch.tensor(cseg, dtype=torch.int32)
    cSeg_GPU = cSeg_CPU.to(dev)
    RA = tiling.reorder_indices(T, tiling.raster_hint(M, N, algo), dev).reshape(TM, TN)
    gen = torch.Generator().manual_seed(11)

    def operands():
        return ((torch.randn(M, K, generator=gen) / K ** 0.5).to(dt).to(dev),
                (torch.randn(N, K, generator=gen) / K ** 0.5).to(dt).to(dev))

    side = torch.cuda.Stream()
    try:
        with torch.cuda.stream(side):
            o = torch.classes.flashoverlap_class.OverlapImpl()
            o.mccl_init(0, 1, torch.ops.flashoverlap_op.generate_mccl_id())
            o.mutlass_init()      # the GEMM stream is `side` from here on
            o.overlap_init()
            o.set_consumer_mode(mode)
            A, B = operands()
            W = (1 + 0.1 * torch.randn(N, generator=gen)).to(dt).to(dev)
            C = torch.empty(M, N, dtype=dt, device=dev)
            y = torch.empty(M, N, dtype=dt, device=dev)
            counter = torch.zeros(max(len(cseg), TN), dtype=torch.int32, device=dev)

            def call():
                o.gemm_allreduce_overlap(A, B, C, counter, RA, 1, cSeg_CPU, cSeg_GPU, algo, False)
                torch.ops.flashoverlap_op.reorder_rmsnorm(o.staging().view(M, N), y, W, BM, BN, 1, RA)

            for _ in range(3):    # first calls allocate the staging buffer and the group table
                call()
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                call()
            # checked mode waits for the call's completion, which a capture forbids: refused up front,
            # before anything is enqueued, with an error that says so (capture_error_mode: the failed
            # capture must not poison the streams of the rest of the process)
            o.set_check_timeouts(True)
            refused = torch.cuda.CUDAGraph()
            with pytest.raises(RuntimeError, match="set_check_timeouts"):
                with torch.cuda.graph(refused, stream=side, capture_error_mode="thread_local"):
                    call()
            o.set_check_timeouts(False)
            del refused
            for replay in range(4):
                print(f"graph replay {replay} w={w} mode={mode}", flush=True)
                a_new, b_new = operands()
                A.copy_(a_new)
                B.copy_(b_new)
                call()                                  # eager, same buffers
                side.synchronize()
                want_staging, want_y = o.staging().clone(), y.clone()
                assert want_y.float().abs().sum() > 0
                o.staging().zero_()
                y.zero_()
                C.zero_()
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                assert o.wait_timeouts(True) == 0
                assert counter.cpu().sum() == 0
                assert torch.equal(o.staging(), want_staging)
                assert torch.equal(y, want_y)
    finally:
        capi.check(capi.lib().fo_set_wait_timeout_ms(5000))
