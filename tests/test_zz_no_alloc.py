"""fo_gemm_signal_static (the entry point that allocates nothing: its slot->group
table lives in a device array inside the library) against fo_gemm_signal with a
caller-owned table, through the C ABI.  Two calls in a row on one device, the
second with a smaller problem, so that anything left in the array by the first
call would show: D, the group counters and the monitor tickets must be
bit-identical to fo_gemm_signal's, and the counters must equal cSeg.
"""
import pytest
import torch

from flashoverlap_amd import capi, tiling

pytestmark = pytest.mark.gpu


def _run_pair(L, dev, dt, M, N, K, w, monitor, seed):
    algo = 1
    BM, BN, _ = capi.algo_tile(algo)
    TM, TN = M // BM, N // BN
    T = TM * TN
    cseg = tiling.uniform_cseg(T, w)
    G = len(cseg)
    g = torch.Generator().manual_seed(seed)
    A = torch.randint(-2, 3, (M, K), generator=g).to(dt).to(dev)
    B = torch.randint(-2, 3, (N, K), generator=g).to(dt).to(dev)
    perm = torch.randperm(T, generator=g).tolist()
    RA = tiling.reorder_indices(T, perm, dev).reshape(TM, TN)
    cs = torch.tensor(cseg, dtype=torch.int32, device=dev)
    mm_len = (TN + T) if monitor else max(G, TN)
    code = capi.dtype_code(dt)

    table = torch.empty(T, dtype=torch.int32, device=dev)
    capi.check(L.fo_build_group_table(cs.data_ptr(), G, T, table.data_ptr(), None))
    MM0 = torch.zeros(mm_len, dtype=torch.int32, device=dev)
    D0 = torch.zeros(M * N, dtype=dt, device=dev)
    capi.check(L.fo_gemm_signal(code, algo, M, N, K, 1, cs.data_ptr(), G, table.data_ptr(), A.data_ptr(),
                                B.data_ptr(), D0.data_ptr(), MM0.data_ptr(), RA.data_ptr(), int(monitor), None))
    MM1 = torch.zeros(mm_len, dtype=torch.int32, device=dev)
    D1 = torch.zeros(M * N, dtype=dt, device=dev)
    print(f"fo_gemm_signal_static {dt} {M}x{N}x{K} w={w} G={G} monitor={monitor}", flush=True)
    capi.check(L.fo_gemm_signal_static(code, algo, M, N, K, 1, cs.data_ptr(), G, A.data_ptr(), B.data_ptr(),
                                       D1.data_ptr(), MM1.data_ptr(), RA.data_ptr(), int(monitor), None))
    torch.cuda.synchronize()
    assert torch.equal(D1.view(torch.int16), D0.view(torch.int16))
    if monitor:
        # counters of the groups, the ticket count, and the set of tickets (their order is timing)
        assert torch.equal(MM1[:G], MM0[:G])
        assert MM1[TN - 1].item() == T
        assert torch.equal(MM1[TN:].sort().values, torch.arange(T, dtype=torch.int32, device=dev))
    else:
        assert torch.equal(MM1, MM0)
    assert MM1[:G].cpu().tolist() == cseg


def test_static_entry_matches_table_entry_twice(fo_lib, dev):
    L = fo_lib
    # first call: 512 tiles in 37 groups; second call, smaller: 32 tiles in 11 groups
    _run_pair(L, dev, torch.bfloat16, 2048, 4096, 256, 14, False, 1)
    _run_pair(L, dev, torch.float16, 512, 1024, 128, 3, False, 2)
    # and with monitor tickets (G <= TN - 1)
    _run_pair(L, dev, torch.bfloat16, 1024, 2048, 128, 16, True, 3)


def test_static_entry_rejects_too_many_tiles(fo_lib, dev):
    L = fo_lib
    # 65536 + 512 tiles of 128x128: beyond the static table; must fail before any launch
    M, N, K = 128 * 258, 128 * 256, 64
    one = torch.zeros(1, dtype=torch.int32, device=dev)
    rc = L.fo_gemm_signal_static(capi.FO_BF16, 1, M, N, K, 1, one.data_ptr(), 1, one.data_ptr(), one.data_ptr(),
                                 one.data_ptr(), one.data_ptr(), one.data_ptr(), 0, None)
    assert rc == capi.FO_ERR_LIMIT
    assert b"static table" in L.fo_last_error()
