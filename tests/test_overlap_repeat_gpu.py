"""Repeated overlapped runs with changing inputs: every iteration the staging
buffer must equal, bit for bit, the permuted product of that iteration's
inputs.  A consumer that released a group early, read a stale cache line of the
previous iteration's C, or left a counter behind would show here."""
import ctypes as C

import pytest
import torch

from flashoverlap_amd import capi, tiling

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("scatter", [False, True])
@pytest.mark.parametrize("mode,store,rel", [("per_group", 1, 0), ("persistent", 1, 0), ("persistent", 0, 0),
                                            ("per_group", 1, 1), ("persistent", 1, 1)])
def test_many_overlapped_iterations(fo_lib, dev, mode, store, rel, scatter):
    L = fo_lib
    capi.check(L.fo_set_wait_timeout_ms(5000))
    capi.check(L.fo_tune(b"store_mode", store))
    capi.check(L.fo_tune(b"release_mode", rel))
    try:
        dt, M, N, K, algo = torch.bfloat16, 4096, 2048, 512, 1
        BM = BN = 128
        TM, TN = M // BM, N // BN
        T = TM * TN
        cseg = tiling.uniform_cseg(T, 100)      # 6 groups, the last one short
        G = len(cseg)
        g = torch.Generator().manual_seed(5)
        sets = []
        RA = tiling.reorder_indices(T, tiling.raster_hint(M, N, algo), dev)
        # scatter kernel: rows of every group stably sorted by row % 4 (the ReduceScatter layout)
        RE = tiling.generate_row_remap_array(M, N, BM, BN, cseg, 4, dev) if scatter else None
        for _ in range(3):
            A = torch.randint(-2, 3, (M, K), generator=g).to(dt).to(dev)
            B = torch.randint(-2, 3, (N, K), generator=g).to(dt).to(dev)
            nat = torch.empty(M, N, dtype=dt, device=dev)
            capi.check(L.fo_gemm(capi.FO_BF16, algo, M, N, K, A.data_ptr(), B.data_ptr(), nat.data_ptr(), None))
            want = torch.empty(T, BM, BN, dtype=dt, device=dev)
            want[RA.long()] = nat.view(TM, BM, TN, BN).permute(0, 2, 1, 3).reshape(T, BM, BN)
            if scatter:
                rows = torch.empty(T * BM, BN, dtype=dt, device=dev)
                rows[RE.long()] = want.view(T * BM, BN)
                want = rows
            sets.append((A, B, want.reshape(-1)))
        cs = torch.tensor(cseg, dtype=torch.int32, device=dev)
        MM = torch.zeros(max(G, TN), dtype=torch.int32, device=dev)
        table = torch.empty(T, dtype=torch.int32, device=dev)
        capi.check(L.fo_build_group_table(cs.data_ptr(), G, T, table.data_ptr(), None))
        Cp = torch.zeros(M * N, dtype=dt, device=dev)
        staging = torch.zeros(M * N, dtype=dt, device=dev)
        comm = C.c_void_p()
        capi.check(L.fo_stream_create(C.byref(comm)))
        bad = torch.zeros(1, dtype=torch.int64, device=dev)
        iters = 150
        for it in range(iters):
            A, B, want = sets[it % 3]
            if scatter:
                capi.check(L.fo_gemm_scatter(capi.FO_BF16, algo, M, N, K, 1, cs.data_ptr(), G, table.data_ptr(),
                                             A.data_ptr(), B.data_ptr(), Cp.data_ptr(), MM.data_ptr(), RA.data_ptr(),
                                             RE.data_ptr(), 0, None))
            else:
                capi.check(L.fo_gemm_signal(capi.FO_BF16, algo, M, N, K, 1, cs.data_ptr(), G, table.data_ptr(),
                                            A.data_ptr(), B.data_ptr(), Cp.data_ptr(), MM.data_ptr(), RA.data_ptr(),
                                            0, None))
            if mode == "persistent":
                capi.check(L.fo_wait_consume(cs.data_ptr(), G, MM.data_ptr(), Cp.data_ptr(), staging.data_ptr(),
                                             BM * BN, 1, 0, 1, 0, None, 16, None, comm))
            else:
                acc = 0
                for gi, n in enumerate(cseg):
                    capi.check(L.fo_wait(n, MM.data_ptr() + 4 * gi, None, comm))
                    capi.check(L.fo_consume(Cp.data_ptr() + 2 * acc, staging.data_ptr() + 2 * acc, 2 * n * BM * BN,
                                            comm))
                    acc += n * BM * BN
            capi.check(L.fo_stream_join(comm, None))
            bad += (staging != want).sum()          # on the main stream, behind the join
            bad += MM.sum()
        torch.cuda.synchronize()
        n = C.c_int()
        capi.check(L.fo_wait_timeouts(C.byref(n), 1))
        capi.check(L.fo_stream_destroy(comm))
        assert n.value == 0
        assert bad.item() == 0
    finally:
        capi.check(L.fo_tune(b"store_mode", 1))
        capi.check(L.fo_tune(b"release_mode", 1))
