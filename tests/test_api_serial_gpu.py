"""GPU tests of the non-overlapped entry points of OverlapImpl / BaselineImpl
(src/overlap_impl.cu:72-219, src/baseline_impl.cu:42-277) on one GPU, where
every collective is the consumer copy."""
import pytest
import torch

import flashoverlap_amd
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def api(dev):
    flashoverlap_amd.load()
    return torch.classes.flashoverlap_class


def _make(api, cls, rank=0, size=1):
    o = getattr(api, cls)()
    o.mccl_init(rank, size, torch.ops.flashoverlap_op.generate_mccl_id())
    if cls == "OverlapImpl":
        o.mutlass_init()
        o.overlap_init()
    else:
        o.mublas_init()
    return o


def _inputs(dev, dt, M=512, N=256, K=128, seed=0):
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-2, 3, (M, K), generator=g).to(dt)
    B = torch.randint(-2, 3, (N, K), generator=g).to(dt)
    return A, B, A.to(dev), B.to(dev), O.gemm(A, B)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_overlapimpl_serial_calls(api, dev, dt):
    A, B, dA, dB, want = _inputs(dev, dt)
    M, N = want.shape
    o = _make(api, "OverlapImpl")
    C = torch.zeros(M, N, dtype=dt, device=dev)
    o.gemm_allreduce(dA, dB, C, 1)
    torch.cuda.synchronize()
    assert torch.equal(C.cpu(), want) and torch.equal(o.staging().cpu().view(M, N), want)

    # a world of 4 seen from rank 3: this rank's quarter of C is what a ReduceScatter leaves with it
    o4 = _make(api, "OverlapImpl", 3, 4)
    C.zero_()
    D = torch.zeros(M // 4, N, dtype=dt, device=dev)
    o4.gemm_reducescatter(dA, dB, C, D, 1)
    torch.cuda.synchronize()
    assert torch.equal(D.cpu(), want.view(4, M // 4, N)[3])
    o4.mccl_reducescatter(C)
    torch.cuda.synchronize()
    assert torch.equal(o4.staging().cpu().view(4, M // 4, N)[3], want.view(4, M // 4, N)[3])

    # seg_allreduce: cSEG_CPU counts units of M*N/SegNum (src/overlap_impl.cu:160-173)
    o.mccl_allreduce(torch.zeros_like(C))          # clear the staging buffer
    seg = torch.tensor([1, 2, 1], dtype=torch.int32)
    o.seg_allreduce(C, seg, 4)
    torch.cuda.synchronize()
    assert torch.equal(o.staging().cpu().view(M, N), want)
    with pytest.raises(RuntimeError, match="exceed"):
        o.seg_allreduce(C, torch.tensor([3, 2], dtype=torch.int32), 4)

    o.gemm_all2all(dA, dB, C, D, 1, torch.zeros(1, 1, dtype=torch.int32))   # world of one: just the GEMM
    o.mccl_all2all(C, D, torch.zeros(1, 1, dtype=torch.int32))
    torch.cuda.synchronize()
    assert torch.equal(C.cpu(), want)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_baselineimpl_calls(api, dev, dt):
    A, B, dA, dB, want = _inputs(dev, dt, seed=1)
    M, N = want.shape
    b = _make(api, "BaselineImpl", 1, 2)
    C = torch.zeros(M, N, dtype=dt, device=dev)
    D = torch.zeros(M // 2, N, dtype=dt, device=dev)
    b.gemm_reducescatter(dA, dB, C, D)
    torch.cuda.synchronize()
    assert torch.equal(C.cpu(), want) and torch.equal(D.cpu(), want.view(2, M // 2, N)[1])
    b.mccl_allreduce(C)
    b.mccl_reducescatter(C)
    torch.cuda.synchronize()
    assert torch.equal(b.staging().cpu().view(M, N), want)
    with pytest.raises(RuntimeError, match="more than one GPU"):
        b.gemm_all2all(dA, dB, C, D, torch.zeros(2, 2, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="mublas_init"):
        api.BaselineImpl().mublas_gemm(dA, dB, C)
