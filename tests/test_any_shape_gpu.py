"""Shapes the reference's kernels do not take (README.md:75 of the reference: "the GEMM size
must be multiples of the tile"; src/rmsnorm/rmsnorm_launch.cu:11-21: rows of at most 1024 x 16
elements): the plain GEMM for any M and N, RMSNorm and reorder+RMSNorm for rows longer than a
wavefront keeps in registers.  All through the C ABI, against the oracle."""
import ctypes as C

import numpy as np
import pytest
import torch

from flashoverlap_amd import capi
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu

REL_L2_TOL, MAX_ABS_TOL = 1e-3, 2e-2     # the path's tolerance for floating-point results


@pytest.fixture(scope="module")
def L(fo_lib, dev):
    return fo_lib


GUARD = 4096   # elements in front of and behind D that no launch may touch


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [
    (1000, 1160, 264),     # ragged in M and N (N a multiple of 8), partial last k panel
    (1, 8, 8), (8, 1, 16), (3, 5, 24),           # smaller than any tile
    (127, 129, 72), (130, 7, 64), (257, 255, 136),   # N not a multiple of 8: rows of D are unaligned
    (300, 520, 1000), (129, 2048, 64), (2049, 136, 128),
    (4100, 2056, 512),     # 256x256 macro tiles with ragged last row and column of tiles
    (384, 640, 320),       # multiples of 128: the kernel without predicates
])
def test_plain_gemm_any_shape_bit_exact_on_integer_inputs(L, dev, dt, M, N, K):
    print(f"any-shape gemm {dt} {M}x{N}x{K}", flush=True)
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    A = torch.randint(-2, 3, (M, K), generator=g).to(dt)
    B = torch.randint(-2, 3, (N, K), generator=g).to(dt)
    # operands allocated exactly: a read beyond them would land in whatever the allocator put next
    dA, dB = A.to(dev), B.to(dev)
    buf = torch.full((GUARD + M * N + GUARD,), 7.0, dtype=dt, device=dev)
    D = buf[GUARD:GUARD + M * N]
    assert D.data_ptr() % 16 == 0
    for algo in (1, 3):    # the layout tile of `algo` places nothing in the plain GEMM
        D.fill_(7.0)
        capi.check(L.fo_gemm(capi.dtype_code(dt), algo, M, N, K, dA.data_ptr(), dB.data_ptr(), D.data_ptr(), None))
        torch.cuda.synchronize()
        assert torch.equal(D.cpu().view(M, N), O.gemm(A, B))
        assert (buf[:GUARD] == 7.0).all() and (buf[GUARD + M * N:] == 7.0).all()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
def test_plain_gemm_any_shape_random_within_tolerance(L, dev, dt):
    M, N, K = 1000, 1160, 2040
    g = torch.Generator().manual_seed(9)
    A = (torch.randn(M, K, generator=g) / K ** 0.5).to(dt)
    B = (torch.randn(N, K, generator=g) / K ** 0.5).to(dt)
    D = torch.empty(M, N, dtype=dt, device=dev)
    dA, dB = A.to(dev), B.to(dev)
    capi.check(L.fo_gemm(capi.dtype_code(dt), 1, M, N, K, dA.data_ptr(), dB.data_ptr(), D.data_ptr(), None))
    torch.cuda.synchronize()
    ref = O.gemm_fp32(A, B).to(dt)
    assert O.rel_l2(D.cpu(), ref) < REL_L2_TOL and O.max_abs(D.cpu(), ref) < MAX_ABS_TOL
    ulp = 2 ** -10 if dt == torch.float16 else 2 ** -7
    assert ((D.cpu().float() - ref.float()).abs() <= ulp * ref.float().abs() + 1e-6).all()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bs,dim", [(5, 16392), (3, 20480), (4, 32768), (2, 65544), (1, 131072)])
def test_plain_rmsnorm_long_rows(L, dev, dt, bs, dim):
    g = torch.Generator().manual_seed(dim)
    x = torch.randn(bs, dim, generator=g).to(dt)
    gamma = (1 + 0.1 * torch.randn(dim, generator=g)).to(dt)
    buf = torch.full((GUARD + bs * dim + GUARD,), 7.0, dtype=dt, device=dev)
    out = buf[GUARD:GUARD + bs * dim]
    dx, dgamma = x.to(dev), gamma.to(dev)
    capi.check(L.fo_rmsnorm(capi.dtype_code(dt), dx.data_ptr(), dgamma.data_ptr(), out.data_ptr(), bs, dim, 1e-5, None))
    torch.cuda.synchronize()
    ref = O.rmsnorm(x, gamma, 1e-5)
    got = out.cpu().view(bs, dim)
    assert O.rel_l2(got, ref) < REL_L2_TOL and O.max_abs(got, ref) < MAX_ABS_TOL
    # two roundings in the reference's order: within two storage ulps of the oracle
    ulp = 2 ** -10 if dt == torch.float16 else 2 ** -7
    assert ((got.float() - ref.float()).abs() <= 2 * ulp * ref.float().abs() + 1e-6).all()
    assert (buf[:GUARD] == 7.0).all() and (buf[GUARD + bs * dim:] == 7.0).all()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("bs,dim,BM,BN,rldn", [(256, 20480, 128, 128, 1), (128, 32768, 64, 256, 2), (32, 16640, 16, 128, 1)])
def test_reorder_rmsnorm_long_rows(L, dev, dt, bs, dim, BM, BN, rldn):
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
    ulp = 2 ** -10 if dt == torch.float16 else 2 ** -7
    assert ((out.cpu().float() - ref.float()).abs() <= 2 * ulp * ref.float().abs() + 1e-6).all()


def test_macro_tile_knob_changes_the_schedule_not_the_result(L, dev):
    """fo_tune "macro_tile": either workgroup tile gives the same bits, the issue order follows the
    setting, and a value the knob does not take is refused."""
    M, N, K = 2048, 4096, 264            # 128 tiles of 256x256: the shape at which the automatic choice changes over
    g = torch.Generator().manual_seed(5)
    A = torch.randint(-2, 3, (M, K), generator=g).to(torch.bfloat16)
    B = torch.randint(-2, 3, (N, K), generator=g).to(torch.bfloat16)
    dA, dB = A.to(dev), B.to(dev)
    want = O.gemm(A, B)
    hints = {}
    order_of_256x128 = capi.raster_hint(4, M, N)
    try:
        for mt in (128, 256, 0):
            capi.check(L.fo_tune(b"macro_tile", mt))
            D = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=dev)
            capi.check(L.fo_gemm(capi.FO_BF16, 1, M, N, K, dA.data_ptr(), dB.data_ptr(), D.data_ptr(), None))
            torch.cuda.synchronize()
            assert torch.equal(D.cpu(), want), mt
            hints[mt] = capi.raster_hint(1, M, N)
            assert sorted(hints[mt]) == list(range((M // 128) * (N // 128)))
            # a signalling launch under the same setting: counters full, placement by RA
            T = (M // 128) * (N // 128)
            ra = torch.tensor(hints[mt], dtype=torch.int64)
            RA = torch.empty(T, dtype=torch.int32)
            RA[ra] = torch.arange(T, dtype=torch.int32)
            cseg = torch.tensor([T // 2, T - T // 2], dtype=torch.int32, device=dev)
            MM = torch.zeros(64, dtype=torch.int32, device=dev)
            dRA = RA.to(dev)
            capi.check(L.fo_gemm_signal(capi.FO_BF16, 1, M, N, K, 1, cseg.data_ptr(), 2, None, dA.data_ptr(), dB.data_ptr(),
                                        D.data_ptr(), MM.data_ptr(), dRA.data_ptr(), 0, None))
            torch.cuda.synchronize()
            assert MM[:2].cpu().tolist() == [T // 2, T - T // 2]
            assert torch.equal(D.cpu().reshape(-1), O.place_tiles(want, RA.numpy().reshape(M // 128, N // 128), 128, 128, 1).reshape(-1))
        assert hints[128] != hints[256] and hints[0] == hints[128]      # up to 128 large tiles: the small one
        # the first workgroup of the large tile covers four layout tiles, that of the small tile one
        assert sorted(hints[256][:4]) == [0, 1, N // 128, N // 128 + 1] and hints[128][0] == 0
        assert L.fo_tune(b"macro_tile", 64) != 0
        # a 256x128 layout tile cannot be served by the small workgroup tile: the setting is ignored there
        capi.check(L.fo_tune(b"macro_tile", 128))
        assert capi.raster_hint(4, M, N) == order_of_256x128
    finally:
        capi.check(L.fo_tune(b"macro_tile", 0))



@pytest.mark.parametrize("M,N,K", [(8191, 4097, 7168), (8190, 4088, 7160)])
def test_plain_gemm_ragged_at_full_size(L, dev, M, N, K):
    """The c3 shape with one row and column missing / one added (N odd: element-wise stores; N a multiple of 8:
    16-byte stores with a ragged last tile): sampled rows against the oracle, and, for the whole output, two
    properties that hold at any size — integer-valued operands give the exact product, which is linear in A."""
    dt = torch.bfloat16
    print(f"ragged full size {M}x{N}x{K}", flush=True)
    g = torch.Generator().manual_seed(M + N)
    A = (torch.randn(M, K, generator=g)).to(dt)
    B = (0.02 * torch.randn(N, K, generator=g)).to(dt)
    dA, dB = A.to(dev), B.to(dev)
    buf = torch.full((GUARD + M * N + 8 + GUARD,), 7.0, dtype=dt, device=dev)
    start = GUARD + (-(buf.data_ptr() // 2 + GUARD) % 8)           # 16-byte aligned output
    D = buf[start:start + M * N]
    assert D.data_ptr() % 16 == 0
    capi.check(L.fo_gemm(capi.FO_BF16, 1, M, N, K, dA.data_ptr(), dB.data_ptr(), D.data_ptr(), None))
    torch.cuda.synchronize()
    assert (buf[:start] == 7.0).all() and (buf[start + M * N:] == 7.0).all()
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 4095, 4096, M - 257, M - 256, M - 2, M - 1])
    ref = O.gemm_fp32(A[rows], B).to(dt)
    got = D.view(M, N)[rows.to(dev)].cpu()
    assert O.rel_l2(got, ref) < REL_L2_TOL and O.max_abs(got, ref) < MAX_ABS_TOL
    # exact arithmetic: operands in {-1, 0, 1} (products and sums of up to K of them are exact in fp32 and,
    # for |sum| <= 256, in bf16); D(A1) + D(A2) == D(A1 + A2) where the supports of A1 and A2 do not overlap
    A1 = torch.zeros(M, K, dtype=dt)
    A2 = torch.zeros(M, K, dtype=dt)
    A1[:, 0:200:2] = torch.randint(-1, 2, (M, 100), generator=g).to(dt)
    A2[:, 1:201:2] = torch.randint(-1, 2, (M, 100), generator=g).to(dt)
    Bi = torch.zeros(N, K, dtype=dt)
    Bi[:, :200] = torch.randint(-1, 2, (N, 200), generator=g).to(dt)
    dBi = Bi.to(dev)
    outs = []
    for Ax in (A1, A2, A1 + A2):
        dAx = Ax.to(dev)
        Dx = torch.empty(M * N, dtype=dt, device=dev)
        capi.check(L.fo_gemm(capi.FO_BF16, 1, M, N, K, dAx.data_ptr(), dBi.data_ptr(), Dx.data_ptr(), None))
        torch.cuda.synchronize()
        outs.append(Dx.float())
    assert torch.equal(outs[0] + outs[1], outs[2])
    assert outs[2].abs().max() <= 200 and outs[2].abs().sum() > 0
    # and the corner block against the oracle, exactly
    corner = outs[2].view(M, N)[M - 300:, N - 300:].cpu()
    assert torch.equal(corner, O.gemm_fp32((A1 + A2)[M - 300:], Bi[N - 300:]))
