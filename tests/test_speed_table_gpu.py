"""The speed table of test/test.py:374-389 through the torch API on one GPU: every column is
measured, and both paths it times (library GEMM + bulk copy, signalling GEMM overlapped with
per-group copies) produce the oracle's result on the operands they were timed on."""
import pytest
import torch

import flashoverlap_amd
from flashoverlap_amd import capi, speed_test, tiling
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("comm_op,ws", [("all_reduce", 1), ("reduce_scatter", 4)])
def test_speed_table_on_config1(dev, comm_op, ws):
    flashoverlap_amd.load()
    capi.check(capi.lib().fo_set_wait_timeout_ms(5000))
    M = N = K = 1024
    BM = BN = 128
    T = (M // BM) * (N // BN)
    # benchmark configuration 1: 64 tiles of 128x128 in 16 groups of 4, fp16
    cfg = {"BM": BM, "BN": BN, "Algo": 1, "rLDN": 1, "hint": tiling.raster_hint(M, N, 1),
           "cSeg": tiling.uniform_cseg(T, 4), "dur": speed_test.perf_mutlass_gemm(M, N, K, 1, warm_up=3, rep=10)}
    keep = {}
    t = speed_test.speed_table(M, N, K, comm_op, cfg, ws, torch.float16, "cuda", keep=keep, warm_up=3, rep=10)
    print("\n" + speed_test.format_table(t), flush=True)
    for col in ("mutlass_gemm", "mublas_gemm", "mccl_comm", "baseline", "overlap", "speedup"):
        assert t[col] > 0, col
    assert t["num_segs"] == 16 and t["tile_num"] == T and sum(t["cSeg"]) == T
    # one GPU: GEMM-then-copy can not be faster than the GEMM alone, nor the overlapped call
    assert t["baseline"] >= 0.9 * t["mublas_gemm"] and t["overlap"] >= 0.9 * t["mutlass_gemm"]
    n = keep["overlap"].wait_timeouts(True)
    assert n == 0 and keep["counters"].cpu().sum() == 0

    A, B = keep["A"].cpu(), keep["B"].cpu()
    cref = O.gemm(A, B)
    ra = keep["RA"].cpu().numpy()
    if comm_op == "all_reduce":
        got = keep["overlap"].staging().cpu()
        want = O.place_tiles(cref, ra, BM, BN, 1)
    else:   # rank 0's receive buffer of the per-group ReduceScatter
        got = keep["D"].cpu().reshape(-1)
        want = O.consume_reducescatter(O.scatter_place(cref, ra, keep["RE"].cpu().numpy(), BM, BN, 1), cfg["cSeg"],
                                       BM, BN, ws)[0]
    assert O.rel_l2(got, want) < 1e-3 and O.max_abs(got, want) < 2e-2 * max(1.0, want.abs().max().item())
    # the baseline path on the same operands: library GEMM, bulk copy
    b = torch.classes.flashoverlap_class.BaselineImpl()
    b.mccl_init(0, ws, torch.ops.flashoverlap_op.generate_mccl_id())
    b.mublas_init()
    C = torch.empty(M, N, dtype=torch.float16, device=dev)
    if comm_op == "all_reduce":
        b.gemm_allreduce(keep["A"], keep["B"], C)
        torch.cuda.synchronize()
        assert O.rel_l2(b.staging().cpu().view(M, N), cref) < 1e-3
    else:
        D = torch.empty(M // ws, N, dtype=torch.float16, device=dev)
        b.gemm_reducescatter(keep["A"], keep["B"], C, D)
        torch.cuda.synchronize()
        assert O.rel_l2(D.cpu(), cref[: M // ws]) < 1e-3
    assert O.rel_l2(C.cpu(), cref) < 1e-3


def test_gemm_sweep_table(dev):
    """test/sweep_gemm.py on two shapes, one of them no multiple of any tile: every row has a vendor time, the
    best Algo's time and their ratio; a shape the GEMM refuses is reported as failed, as the reference does,
    and left out of the summary."""
    from flashoverlap_amd import sweep_gemm
    lines = []
    results = sweep_gemm.sweep([1024, 1000], [1024], [512], torch.float16, out=lines.append, warm_up=2, rep=5)
    assert lines[0] == sweep_gemm.HEADER
    assert len(results) == 2 and [r[:3] for r in results] == [(1024, 1024, 512), (1000, 1024, 512)]
    for M, N, K, algo, vendor, ours, ratio in results:
        assert 0 <= algo < capi.lib().fo_algo_count() and vendor > 0 and ours > 0 and ratio == pytest.approx(ours / vendor)
    assert any("--- Top 10 closest" in l for l in lines)
    lines = []
    assert sweep_gemm.sweep([1024], [1024], [500], torch.float16, out=lines.append, warm_up=1, rep=2) == []
    assert "FAIL" in lines[2] and not any("--- Top 10" in l for l in lines)
