"""fo_reorder_rmsnorm_batched: several [bs, dim] problems that share RA in one
launch must equal the same problems launched one by one, and the oracle."""
import numpy as np
import pytest
import torch

from flashoverlap_amd import capi
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nbatch,bs,dim,BM,BN", [(8, 128, 1024, 16, 128), (3, 64, 384, 32, 8), (1, 256, 512, 128, 128)])
def test_batched_equals_single_launches(fo_lib, dev, dt, nbatch, bs, dim, BM, BN):
    L = fo_lib
    g = torch.Generator().manual_seed(nbatch * dim)
    T = (bs // BM) * (dim // BN)
    ra = O.reorder_indices(T, np.random.default_rng(T).permutation(T))
    natural = torch.randn(nbatch, bs, dim, generator=g).to(dt)
    gamma = (1 + 0.1 * torch.randn(dim, generator=g)).to(dt)
    x = torch.stack([O.place_tiles(natural[b], ra, BM, BN, 1) for b in range(nbatch)])
    dx, dgamma, dra = x.to(dev), gamma.to(dev), torch.from_numpy(ra).to(dev)
    code = capi.dtype_code(dt)
    batched = torch.empty(nbatch, bs, dim, dtype=dt, device=dev)
    capi.check(L.fo_reorder_rmsnorm_batched(code, dx.data_ptr(), dgamma.data_ptr(), batched.data_ptr(), nbatch, bs,
                                            dim, BM, BN, 1, dra.data_ptr(), 1e-5, None))
    single = torch.empty_like(batched)
    for b in range(nbatch):
        capi.check(L.fo_reorder_rmsnorm(code, dx[b].data_ptr(), dgamma.data_ptr(), single[b].data_ptr(), bs, dim, BM,
                                        BN, 1, dra.data_ptr(), 1e-5, None))
    torch.cuda.synchronize()
    assert torch.equal(batched, single)
    ref = torch.stack([O.rmsnorm(natural[b], gamma, 1e-5) for b in range(nbatch)])
    assert O.rel_l2(batched.cpu(), ref) < 1e-3 and O.max_abs(batched.cpu(), ref) < 2e-2


def test_batched_argument_checks(fo_lib, dev):
    a = torch.zeros(4096, dtype=torch.float16, device=dev)
    ra = torch.zeros(4, dtype=torch.int32, device=dev)
    args = (capi.FO_F16, a.data_ptr(), a.data_ptr(), a.data_ptr())
    assert fo_lib.fo_reorder_rmsnorm_batched(*args, 0, 8, 64, 4, 8, 1, ra.data_ptr(), 1e-5, None) == capi.FO_OK
    assert fo_lib.fo_reorder_rmsnorm_batched(*args, 70000, 8, 64, 4, 8, 1, ra.data_ptr(), 1e-5, None) == capi.FO_ERR_LIMIT
    assert fo_lib.fo_reorder_rmsnorm_batched(*args, 2, 8, 64, 4, 8, 1, None, 1e-5, None) == capi.FO_ERR_ARG
