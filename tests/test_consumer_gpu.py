"""The persistent consumer on its own: ragged group sizes (zeros included) over
several 64-group passes, every counter preset to its group's size, for
different grid sizes and with the ReduceScatter slicing; checked against the
oracle's consume_allreduce / consume_reducescatter."""
import ctypes as C

import numpy as np
import pytest
import torch

from flashoverlap_amd import capi
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("nblocks", [1, 7, 64, 256])
@pytest.mark.parametrize("ws", [1, 4])
def test_ragged_groups(fo_lib, dev, nblocks, ws):
    L = fo_lib
    capi.check(L.fo_set_wait_timeout_ms(5000))
    rng = np.random.default_rng(nblocks * 10 + ws)
    BM, BN = 16, 64                      # small tiles keep the buffers small: 1024 elements each
    sizes = rng.integers(0, 5, size=1400).tolist() + [200, 0, 37, 1]   # a large group too: a team of many
    G, T = len(sizes), sum(sizes)
    src = torch.randint(-30000, 30000, (T * BM * BN,), dtype=torch.int16)
    d_src = src.to(dev)
    d_dst = torch.full_like(d_src, -1)
    cs = torch.tensor(sizes, dtype=torch.int32, device=dev)
    MM = cs.clone()
    log = torch.full((G,), -1, dtype=torch.int32, device=dev)
    stride = (T * BM * BN) // ws if ws > 1 else 0
    capi.check(L.fo_wait_consume(cs.data_ptr(), G, MM.data_ptr(), d_src.data_ptr(), d_dst.data_ptr(), BM * BN, ws, 0,
                                 ws, stride, log.data_ptr(), nblocks, None, None))
    torch.cuda.synchronize()
    n = C.c_int()
    capi.check(L.fo_wait_timeouts(C.byref(n), 1))
    assert n.value == 0
    assert MM.cpu().sum().item() == 0
    assert log.cpu().tolist() == list(range(G))
    if ws == 1:
        want = O.consume_allreduce(src, sizes, BM, BN)
    else:
        want = O.consume_reducescatter(src, sizes, BM, BN, ws).reshape(-1)
    assert torch.equal(d_dst.cpu(), want)


def test_more_workgroups_than_cus_is_refused(fo_lib, dev):
    """The consumer's workgroups wait while GEMM workgroups still have to be placed, so there may be
    at most one per CU; a larger grid is an error, not a silent clamp."""
    L = fo_lib
    cu = C.c_int()
    capi.check(L.fo_device_info(C.byref(cu), None, None))
    buf = torch.zeros(4096, dtype=torch.int32, device=dev)
    rc = L.fo_wait_consume(buf.data_ptr(), 1, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), 128, 1, 0, 1, 0, None,
                           cu.value + 1, None, None)
    assert rc == capi.FO_ERR_LIMIT
    assert b"one workgroup per CU" in L.fo_last_error()
