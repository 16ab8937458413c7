"""Pins the CPU oracle (oracle/fo_oracle.py) without any GPU: known answers,
closed forms, invariants and brute force, chosen so that a dropped term, a
swapped index or a transposed operand fails at least one check.  The reference
holds no golden vectors of its own (its tests are multi-GPU scripts that print
allclose); the known answers below are worked by hand from the reference's
statements."""
import itertools

import numpy as np
import pytest
import torch

from oracle import fo_oracle as O


# ---- reorder_indices -------------------------------------------------------

def test_reorder_indices_known_answers():
    # hint[i] = tile that takes slot i; tiles not named keep ascending order after them
    assert O.reorder_indices(8, [3, 1, 2]).tolist() == [3, 1, 2, 0, 4, 5, 6, 7]
    assert O.reorder_indices(6, [5, 4, 3, 2, 1, 0]).tolist() == [5, 4, 3, 2, 1, 0]
    assert O.reorder_indices(4, []).tolist() == [0, 1, 2, 3]
    assert O.reorder_indices(5, [4]).tolist() == [1, 2, 3, 4, 0]


def test_reorder_indices_inverse_permutation_law():
    rng = np.random.default_rng(0)
    for S in (1, 2, 7, 64, 513):
        hint = rng.permutation(S)
        ra = O.reorder_indices(S, hint)
        assert ra.dtype == np.int32
        # RA o hint = identity  <=>  RA is the inverse permutation of hint
        assert np.array_equal(ra[hint], np.arange(S))
        assert sorted(ra.tolist()) == list(range(S))


def test_reorder_indices_matches_literal_for_partial_hints():
    rng = np.random.default_rng(1)
    for S in (1, 5, 16, 40):
        for n in {0, 1, S // 2, S}:
            hint = rng.permutation(S)[:n].tolist()
            assert O.reorder_indices(S, hint).tolist() == O.reorder_indices_literal(S, hint)


# ---- cSeg builders ---------------------------------------------------------

def test_uniform_cseg():
    assert O.uniform_cseg(64, 4) == [4] * 16
    assert O.uniform_cseg(10, 4) == [4, 4, 2]
    assert O.uniform_cseg(3, 8) == [3]
    for T, w in itertools.product((1, 7, 64, 1024, 8192), (1, 2, 3, 106, 256)):
        c = O.uniform_cseg(T, w)
        assert sum(c) == T and len(c) == -(-T // w) and all(0 < x <= w for x in c)


def test_compositions():
    assert O.compositions(3) == [[1, 1, 1], [1, 2], [2, 1], [3]]
    assert O.compositions(1) == [[1]]
    for n in range(1, 11):
        cs = O.compositions(n)
        assert len(cs) == 2 ** (n - 1)
        assert all(sum(c) == n for c in cs)
        assert len({tuple(c) for c in cs}) == len(cs)


def test_cseg_from_composition():
    # 10 waves-worth of 106 tiles would be 1060; the output has 1024 tiles
    assert O.cseg_from_composition([1, 1, 2, 2, 4], 106, 1024) == [106, 106, 212, 212, 388]
    assert O.cseg_from_composition([3], 256, 512) == [512]
    for gp in O.compositions(5):
        assert sum(O.cseg_from_composition(list(gp), 30, 141)) == 141


# ---- slot -> group ---------------------------------------------------------

def test_group_of_slot_known_answer():
    cseg = [4, 4, 2]
    assert [O.group_of_slot_literal(cseg, s) for s in range(10)] == [0, 0, 0, 0, 1, 1, 1, 1, 2, 2]
    assert O.group_of_slots(cseg, range(10)).tolist() == [0, 0, 0, 0, 1, 1, 1, 1, 2, 2]


def test_group_of_slots_matches_literal_scan():
    rng = np.random.default_rng(2)
    for _ in range(20):
        cseg = rng.integers(0, 6, size=rng.integers(1, 12)).tolist()
        cseg[-1] += 1  # the scan needs a last non-empty group to stop in
        T = sum(cseg)
        lit = [O.group_of_slot_literal(cseg, s) for s in range(T)]
        assert O.group_of_slots(cseg, range(T)).tolist() == lit
        # every group g is hit exactly cseg[g] times
        assert np.bincount(lit, minlength=len(cseg)).tolist() == cseg


# ---- row remap -------------------------------------------------------------

def test_row_remap_known_answers():
    assert O.row_remap(8, 4, 4, 4, [1, 1], 2).tolist() == [0, 2, 1, 3, 4, 6, 5, 7]
    assert O.row_remap(8, 8, 4, 4, [3, 1], 4).tolist() == [0, 3, 6, 9, 1, 4, 7, 10, 2, 5, 8, 11, 12, 13, 14, 15]


@pytest.mark.parametrize("M,N,BM,BN,cseg,ws", [
    (8, 4, 4, 4, [1, 1], 2), (8, 8, 4, 4, [3, 1], 4), (16, 8, 4, 4, [2, 5, 1], 2),
    (12, 6, 6, 3, [1, 2, 1], 3), (12, 6, 6, 3, [4], 4), (10, 4, 5, 2, [1, 3], 2),
])
def test_row_remap_matches_literal_stable_sort(M, N, BM, BN, cseg, ws):
    got = O.row_remap(M, N, BM, BN, cseg, ws)
    assert got.tolist() == O.row_remap_literal(M, N, BM, BN, cseg, ws)
    assert sorted(got.tolist()) == list(range(M * N // BN))
    # rows never leave their group chunk
    c0 = 0
    for S in cseg:
        L = S * BM
        assert sorted(got[c0:c0 + L].tolist()) == list(range(c0, c0 + L))
        c0 += L


def test_row_remap_rank_slices_are_contiguous():
    M, N, BM, BN, ws = 16, 8, 8, 4, 4
    cseg = [1, 2, 1]
    re = O.row_remap(M, N, BM, BN, cseg, ws)
    c0 = 0
    for S in cseg:
        L = S * BM
        for k in range(ws):
            rows = [r for r in range(c0, c0 + L) if r % ws == k]
            assert re[rows].tolist() == list(range(c0 + k * (L // ws), c0 + (k + 1) * (L // ws)))
        c0 += L


def test_reorder_rows_by_world_size():
    x = torch.arange(8).reshape(8, 1)
    assert O.reorder_rows_by_world_size(x, 4).reshape(-1).tolist() == [0, 4, 1, 5, 2, 6, 3, 7]
    assert O.reorder_rows_by_world_size(x, 1).reshape(-1).tolist() == list(range(8))


# ---- placement -------------------------------------------------------------

def _rand_perm_ra(T, seed):
    return O.reorder_indices(T, np.random.default_rng(seed).permutation(T))


def test_place_tiles_rldn1_is_tile_major():
    M, N, BM, BN = 4, 6, 2, 3
    C = torch.arange(M * N, dtype=torch.float32).reshape(M, N)
    ident = np.arange(4, dtype=np.int32)
    got = O.place_tiles(C, ident, BM, BN, 1)
    want = C.reshape(2, BM, 2, BN).permute(0, 2, 1, 3).reshape(-1)
    assert torch.equal(got, want)


def test_place_tiles_rldn_tn_identity_is_natural_layout():
    M, N, BM, BN = 6, 8, 3, 2
    C = torch.randn(M, N)
    TN = N // BN
    ident = np.arange((M // BM) * TN, dtype=np.int32)
    assert torch.equal(O.place_tiles(C, ident, BM, BN, TN), C.reshape(-1))


@pytest.mark.parametrize("rldn", [1, 2])
def test_place_then_gather_round_trip(rldn):
    M, N, BM, BN = 8, 12, 2, 3
    T = (M // BM) * (N // BN)
    C = torch.randn(M, N)
    ra = _rand_perm_ra(T, 3)
    flat = O.place_tiles(C, ra, BM, BN, rldn)
    assert sorted(flat.tolist()) == sorted(C.reshape(-1).tolist())
    assert torch.equal(O.gather_tiles(flat, M, N, BM, BN, rldn, ra), C)


@pytest.mark.parametrize("rldn,with_re", [(1, False), (2, False), (1, True)])
def test_place_matches_literal_epilogue(rldn, with_re):
    M, N, BM, BN = 8, 6, 4, 3
    T = (M // BM) * (N // BN)
    C = torch.arange(M * N, dtype=torch.float32).reshape(M, N)
    ra = _rand_perm_ra(T, 4)
    re = O.row_remap(M, N, BM, BN, [1, 2, 1], 2) if with_re else None
    lit = O.place_tiles_literal(C.tolist(), ra, BM, BN, rldn, re)
    got = O.scatter_place(C, ra, re, BM, BN, rldn) if with_re else O.place_tiles(C, ra, BM, BN, rldn)
    assert got.tolist() == lit


def test_tile_of_slot_is_contiguous_range():
    # with rLDN=1, slot s occupies [s*BM*BN, (s+1)*BM*BN) with row stride BN
    M, N, BM, BN = 6, 6, 3, 2
    T = 6
    ra = _rand_perm_ra(T, 5)
    C = torch.arange(M * N, dtype=torch.float32).reshape(M, N)
    flat = O.place_tiles(C, ra, BM, BN, 1)
    for t in range(T):
        mt, nt = divmod(t, N // BN)
        tile = C[mt * BM:(mt + 1) * BM, nt * BN:(nt + 1) * BN].reshape(-1)
        s = int(ra[t])
        assert torch.equal(flat[s * BM * BN:(s + 1) * BM * BN], tile)


def test_reducescatter_slices_are_small_tile_layouts():
    # After the scatter epilogue and the per-group ReduceScatter, rank k holds an
    # ordinary permuted layout with tile height BM/ws of the rows m % ws == k
    # (why the reference builds ReorderRMSNorm with BM//world_size).
    M, N, BM, BN, ws = 16, 8, 8, 4, 4
    T = (M // BM) * (N // BN)
    cseg = [1, 2, 1]
    C = torch.randn(M, N)
    ra = _rand_perm_ra(T, 6)
    re = O.row_remap(M, N, BM, BN, cseg, ws)
    D = O.consume_reducescatter(O.scatter_place(C, ra, re, BM, BN, 1), cseg, BM, BN, ws)
    want = O.reorder_rows_by_world_size(C, ws).reshape(ws, M // ws, N)
    for k in range(ws):
        got = O.gather_tiles(D[k], M // ws, N, BM // ws, BN, 1, ra)
        assert torch.equal(got, want[k])
        assert torch.equal(got, C[k::ws])


# ---- counters --------------------------------------------------------------

def test_signal_counters_and_wait():
    T, TN = 12, 4
    cseg = [5, 4, 3]
    ra = _rand_perm_ra(T, 7)
    order = np.random.default_rng(8).permutation(T)
    mm = O.signal_counters(ra, cseg, order, TN)
    assert mm[:3].tolist() == cseg and mm.sum() == T
    released, after = O.wait_release(mm, cseg)
    assert released == [0, 1, 2] and not after.any()
    with pytest.raises(RuntimeError):
        O.wait_release(mm, [5, 5, 2])


def test_monitor_tickets_are_completion_ranks():
    T, TN = 12, 4
    cseg = [6, 6]  # monitor mode needs len(cSeg) <= TN-1
    ra = _rand_perm_ra(T, 9)
    order = np.random.default_rng(10).permutation(T)
    mm = O.signal_counters(ra, cseg, order, TN, monitor=True)
    assert mm[TN - 1] == T
    tickets = mm[TN:TN + T]
    assert sorted(tickets.tolist()) == list(range(T))
    for rank, t in enumerate(order):
        assert tickets[ra[t]] == rank


def test_consume_allreduce_is_identity_on_covered_range():
    BM, BN = 2, 2
    cseg = [1, 3, 2]
    x = torch.randn(6 * BM * BN)
    assert torch.equal(O.consume_allreduce(x, cseg, BM, BN), x)
    assert O.group_ranges(cseg, BM, BN) == [(0, 4), (4, 16), (16, 24)]


# ---- floating point --------------------------------------------------------

def test_gemm_exact_on_small_integers_and_not_transposed():
    g = torch.Generator().manual_seed(0)
    A = torch.randint(-3, 4, (5, 16), generator=g).to(torch.float16)
    B = torch.randint(-3, 4, (7, 16), generator=g).to(torch.float16)
    want = torch.tensor([[sum(int(a) * int(b) for a, b in zip(ra, rb)) for rb in B.tolist()] for ra in A.tolist()])
    got = O.gemm(A, B)
    assert got.shape == (5, 7) and got.dtype == torch.float16
    assert torch.equal(got.long(), want)


def test_gemm_fp32_close_to_fp64():
    g = torch.Generator().manual_seed(1)
    A = (torch.randn(64, 512, generator=g) / 512 ** 0.5).to(torch.bfloat16)
    B = (torch.randn(48, 512, generator=g) / 512 ** 0.5).to(torch.bfloat16)
    ref = A.double() @ B.double().t()
    assert O.rel_l2(O.gemm_fp32(A, B), ref) < 1e-6


def test_rmsnorm_closed_forms():
    # a constant row c normalises to c/sqrt(c^2+eps) ~ sign(c); gamma scales columnwise
    x = torch.full((2, 8), 3.0, dtype=torch.float16)
    gamma = torch.arange(1, 9, dtype=torch.float16)
    out = O.rmsnorm(x, gamma, 1e-6)
    assert torch.allclose(out.float(), gamma.float().expand(2, 8), atol=1e-3)
    # scale invariance: rmsnorm(a*x) == rmsnorm(x) for a > 0 when eps is negligible
    g = torch.Generator().manual_seed(2)
    y = torch.randn(4, 64, generator=g)
    a = O.rmsnorm_fp32(y, torch.ones(64), 0.0)
    b = O.rmsnorm_fp32(4.0 * y, torch.ones(64), 0.0)
    assert torch.allclose(a, b, atol=1e-6)
    # unit RMS of the output
    assert torch.allclose(a.pow(2).mean(-1), torch.ones(4), atol=1e-5)
    # eps enters under the square root, added to the mean square
    z = torch.zeros(1, 4)
    z[0, 0] = 2.0  # mean square = 1
    assert torch.allclose(O.rmsnorm_fp32(z, torch.ones(4), 3.0)[0, 0], torch.tensor(2.0 / 2.0))


def test_rmsnorm_two_roundings_stay_within_storage_ulp():
    g = torch.Generator().manual_seed(3)
    for dt, ulp in ((torch.float16, 2 ** -10), (torch.bfloat16, 2 ** -7)):
        x = torch.randn(8, 256, generator=g).to(dt)
        gamma = (1 + 0.1 * torch.randn(256, generator=g)).to(dt)
        exact = O.rmsnorm_fp32(x, gamma, 1e-5)
        got = O.rmsnorm(x, gamma, 1e-5).float()
        assert ((got - exact).abs() <= 1.5 * ulp * exact.abs() + 1e-6).all()


def test_reorder_rmsnorm_undoes_the_permutation():
    M, N, BM, BN = 8, 16, 4, 8
    T = (M // BM) * (N // BN)
    g = torch.Generator().manual_seed(4)
    C = torch.randn(M, N, generator=g).to(torch.float16)
    gamma = (1 + 0.1 * torch.randn(N, generator=g)).to(torch.float16)
    ra = _rand_perm_ra(T, 11)
    got = O.reorder_rmsnorm(O.place_tiles(C, ra, BM, BN, 1), gamma, M, N, BM, BN, 1, ra, 1e-6)
    assert torch.equal(got, O.rmsnorm(C, gamma, 1e-6))


def test_config1_plumbing_run_on_cpu():
    """Benchmark configuration 1 end to end on the CPU oracle: fp16 1024^3, 128x128
    tiles, groups of 4 tiles, reordered output + RMSNorm against fp32."""
    M = N = K = 1024
    BM = BN = 128
    torch.manual_seed(0)
    A = (torch.randn(M, K) / K ** 0.5).to(torch.float16)
    B = (torch.randn(N, K) / K ** 0.5).to(torch.float16)
    gamma = (1 + 0.1 * torch.randn(N)).to(torch.float16)
    T = (M // BM) * (N // BN)
    cseg = O.uniform_cseg(T, 4)
    assert len(cseg) == 16 > N // BN  # more groups than the reference's TN counters
    hint = np.random.default_rng(0).permutation(T)
    ra = O.reorder_indices(T, hint)
    C = O.gemm(A, B)
    cperm = O.place_tiles(C, ra, BM, BN, 1)
    mm = O.signal_counters(ra, cseg, hint, N // BN)
    released, after = O.wait_release(mm, cseg)
    assert released == list(range(16)) and not after.any()
    staging = O.consume_allreduce(cperm, cseg, BM, BN)
    out = O.reorder_rmsnorm(staging, gamma, M, N, BM, BN, 1, ra, 1e-6)
    ref = O.rmsnorm_fp32(O.gemm_fp32(A, B), gamma, 1e-6)
    assert O.rel_l2(out, ref) < 1e-3 and O.max_abs(out, ref) < 2e-2
