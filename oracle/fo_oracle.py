"""CPU oracle for the FlashOverlap single-GPU hot path.

THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke check
in __graft_entry__ and the cpu_baseline leg of bench.py may import it, and only
as the checker.  The product path (flashoverlap_amd + its HIP libraries) never
imports it and has no CPU fallback.

Every function restates, on the CPU, what one piece of the reference does and
cites the reference file:line it follows (paths relative to the reference
checkout).  Integer work is numpy (closed forms) with a *_literal twin written
as plain loops that follow the reference statement by statement; the literal
twins are for small inputs and exist so that the closed forms are pinned by
something other than themselves.  Floating-point work is torch on the CPU in
fp32 with the reference's storage roundings (fp16, or bf16 for the configs the
reference itself cannot run).

How each function is pinned (see tests/test_oracle.py):
  reorder_indices      known answers, inverse-permutation law, literal twin
  uniform_cseg         closed form ceil/min, sums to T
  compositions         count 2^(n-1), known answer n=3, each sums to n
  cseg_from_composition known answer, sums to T
  group_of_slots       known answer, literal while-loop twin
  row_remap            two known answers, literal stable-sort twin, permutation
  place_tiles          round trip with gather_tiles, rLDN=TN identity special
                       case equals the natural row-major matrix
  scatter_place        brute force per element on tiny shapes, rank slices
                       contiguous, A.6 identity with reorder_rmsnorm
  signal_counters      counts equal cSeg, tickets are a permutation
  wait_release         releases in index order, counters return to zero
  gemm / rmsnorm       textbook fp32 formulas (the arithmetic of the reference
                       GEMM lives in MUTlass, which is not in the reference
                       tree: parity unpinned by the reference itself, pinned
                       here by exact small-integer cases and fp64 comparison)
"""
from __future__ import annotations

import numpy as np
import torch

# --------------------------------------------------------------------------
# integer tiling logic
# --------------------------------------------------------------------------


def div_up(x: int, y: int) -> int:
    """test/test.py:69-70."""
    return (x + y - 1) // y


def reorder_indices(S: int, hint) -> np.ndarray:
    """RA = reorder_indices(S, hint): RA[hint[i]] = i, and the tiles that are
    not named by hint take the slots len(hint), len(hint)+1, ... in ascending
    tile order (test/test.py:72-88, example/utils.py:6-22)."""
    hint = np.asarray(hint, dtype=np.int64).reshape(-1)
    ra = np.full(S, -1, dtype=np.int64)
    ra[hint] = np.arange(hint.size)
    rest = np.flatnonzero(ra < 0)
    ra[rest] = hint.size + np.arange(rest.size)
    return ra.astype(np.int32)


def reorder_indices_literal(S: int, hint) -> list:
    """Statement-by-statement twin of test/test.py:72-88 (small S only)."""
    new_order = [-1] * S
    i = 0
    for element in hint:
        new_order[element] = i
        i += 1
    nxt = len(hint)
    for x in range(S):
        named = False
        for h in hint:
            if h == x:
                named = True
        if not named:
            new_order[x] = nxt
            nxt += 1
    return new_order


def uniform_cseg(T: int, w: int) -> list:
    """Groups of w tiles, the last one short: cSeg[i] = min(w, T - i*w) for
    i < ceil(T/w) (tune/search.py:137-144)."""
    return [min(w, T - i * w) for i in range(div_up(T, w))]


def compositions(n: int) -> list:
    """All ordered compositions of n in the order the reference's
    integer_partitions enumerates them (tune/search.py:462-471)."""
    out = []

    def rec(rem, path):
        if rem == 0:
            out.append(path)
            return
        for i in range(1, rem + 1):
            rec(rem - i, path + [i])

    rec(n, [])
    return out


def cseg_from_composition(gp, W: int, T: int) -> list:
    """cSeg[j] = gp[j]*W, the last entry clipped to the tiles that remain
    (tune/search.py:502-513)."""
    cseg, acc = [], 0
    for j, g in enumerate(gp):
        if j < len(gp) - 1:
            cseg.append(g * W)
            acc += g * W
        else:
            cseg.append(min(g * W, T - acc))
    return cseg


def group_of_slot_literal(cseg, s: int) -> int:
    """The epilogue's linear scan (src/overlap/gemm_with_signal.h:188-193)."""
    idx_bound = cseg[0]
    it = 0
    while idx_bound <= s:
        it += 1
        idx_bound += cseg[it]
    return it


def group_of_slots(cseg, slots) -> np.ndarray:
    """Closed form of the scan: number of inclusive prefix sums <= slot."""
    cum = np.cumsum(np.asarray(cseg, dtype=np.int64))
    return np.searchsorted(cum, np.asarray(slots, dtype=np.int64), side="right").astype(np.int32)


def row_remap(M: int, N: int, BM: int, BN: int, cseg, ws: int) -> np.ndarray:
    """RE: inside every group chunk of cSeg[g]*BM rows of the rLDN=1 view the
    rows are stably sorted by row % ws; RE[orig] = new position
    (test/test.py:90-118).  Closed form, valid for any chunk start/length."""
    R = M * N // BN
    assert sum(cseg) * BM == R, "sum(cSeg) must equal the number of tiles"
    re = np.empty(R, dtype=np.int64)
    c0 = 0
    for S in cseg:
        L = S * BM
        r = np.arange(c0, c0 + L)
        res = r % ws
        # rows with residue < k that live in this chunk precede residue k
        first = (-c0) % ws  # offset in the chunk of the first row with residue 0
        cnt = np.array([len(range((first + k) % ws, L, ws)) for k in range(ws)])
        base = np.concatenate([[0], np.cumsum(cnt)[:-1]])
        off0 = np.array([(first + k) % ws for k in range(ws)])
        re[r] = c0 + base[res] + ((r - c0) - off0[res]) // ws
        c0 += L
    return re.astype(np.int32)


def row_remap_literal(M: int, N: int, BM: int, BN: int, cseg, ws: int) -> list:
    """Statement-by-statement twin of test/test.py:90-118 (stable sort)."""
    R = M * N // BN
    reordered = [0] * R
    cur = 0
    for S in cseg:
        chunk = list(range(cur, cur + S * BM))
        keyed = sorted(chunk, key=lambda r: r % ws)  # Python's sort is stable
        for i, r in enumerate(keyed):
            reordered[cur + i] = r
        cur += S * BM
    remap = [0] * R
    for new, orig in enumerate(reordered):
        remap[orig] = new
    return remap


def reorder_rows_by_world_size(x: torch.Tensor, ws: int) -> torch.Tensor:
    """Rows stably sorted by row % ws (example/utils.py:54-65)."""
    M = x.shape[0]
    idx = sorted(range(M), key=lambda r: r % ws)
    return x[torch.tensor(idx, dtype=torch.long)]


# --------------------------------------------------------------------------
# placement of output tiles
# --------------------------------------------------------------------------


def _tile_dest_index(M, N, BM, BN, RA, rLDN, RE=None):
    """Flat destination index of every element (m, n) of the natural matrix.

    Tile t = (m/BM)*TN + n/BN goes to slot s = RA[t]; D is viewed as
    [M*N/(rLDN*BN), rLDN*BN]; the tile lands at block-row s/rLDN, block-col
    s%rLDN (src/overlap/gemm_with_signal.h:147-165).  With RE the row index of
    that view is mapped through RE (src/overlap/gemm_with_scatter.h:166-176).
    """
    TN = N // BN
    ra = np.asarray(RA, dtype=np.int64).reshape(-1)
    m = np.arange(M, dtype=np.int64)[:, None]
    n = np.arange(N, dtype=np.int64)[None, :]
    s = ra[(m // BM) * TN + (n // BN)]
    row = (s // rLDN) * BM + (m % BM)
    col = (s % rLDN) * BN + (n % BN)
    if RE is not None:
        row = np.asarray(RE, dtype=np.int64)[row]
    return row * (rLDN * BN) + col


def place_tiles(C: torch.Tensor, RA, BM: int, BN: int, rLDN: int = 1) -> torch.Tensor:
    """The flat M*N buffer the signalling epilogue writes
    (src/overlap/gemm_with_signal.h:145-181)."""
    M, N = C.shape
    dst = torch.from_numpy(_tile_dest_index(M, N, BM, BN, RA, rLDN)).reshape(-1)
    out = torch.empty(M * N, dtype=C.dtype)
    out[dst] = C.reshape(-1)
    return out


def scatter_place(C: torch.Tensor, RA, RE, BM: int, BN: int, rLDN: int = 1) -> torch.Tensor:
    """The flat buffer the scatter epilogue writes
    (src/overlap/gemm_with_scatter.h:146-177)."""
    M, N = C.shape
    dst = torch.from_numpy(_tile_dest_index(M, N, BM, BN, RA, rLDN, RE)).reshape(-1)
    out = torch.empty(M * N, dtype=C.dtype)
    out[dst] = C.reshape(-1)
    return out


def place_tiles_literal(C, RA, BM, BN, rLDN=1, RE=None):
    """Loop twin of the two epilogues, element by element (tiny shapes)."""
    M, N = len(C), len(C[0])
    TN = N // BN
    ra = [int(v) for v in np.asarray(RA).reshape(-1)]
    out = [None] * (M * N)
    ld = rLDN * BN
    for mt in range(M // BM):
        for nt in range(TN):
            slot = ra[mt * TN + nt]
            new_m, new_n = slot // rLDN, slot % rLDN
            for r in range(BM):
                for c in range(BN):
                    row = new_m * BM + r
                    if RE is not None:
                        row = int(RE[row])
                    out[row * ld + new_n * BN + c] = C[mt * BM + r][nt * BN + c]
    return out


def gather_tiles(x: torch.Tensor, bs: int, dim: int, BM: int, BN: int, rldn: int, RA) -> torch.Tensor:
    """The gather reorder_rmsnorm performs before normalising: out[b, j] =
    x[((s/rldn)*BM + b%BM)*(rldn*BN) + (s%rldn)*BN + j%BN], s = RA[(b/BM)*ldn +
    j/BN], ldn = dim/BN (src/rmsnorm/rmsnorm.cuh:78-84,
    src/rmsnorm/rmsnorm_launch.cu:18)."""
    ldn = dim // BN
    ra = np.asarray(RA, dtype=np.int64).reshape(-1)
    b = np.arange(bs, dtype=np.int64)[:, None]
    j = np.arange(dim, dtype=np.int64)[None, :]
    s = ra[(b // BM) * ldn + (j // BN)]
    src = ((s // rldn) * BM + b % BM) * (rldn * BN) + (s % rldn) * BN + (j % BN)
    return x.reshape(-1)[torch.from_numpy(src).reshape(-1)].reshape(bs, dim)


# --------------------------------------------------------------------------
# counter protocol
# --------------------------------------------------------------------------


def signal_counters(RA, cseg, completion_order, TN: int, monitor: bool = False, mm_len: int | None = None):
    """State of the counter buffer MM after every tile has signalled, tiles
    finishing in completion_order (a sequence of original tile ids).
    Normal mode: MM[group(slot)] += 1.  Monitor mode additionally takes a
    ticket from MM[TN-1] and stores it at MM[TN+slot]
    (src/overlap/gemm_with_signal.h:184-201)."""
    ra = np.asarray(RA, dtype=np.int64).reshape(-1)
    T = ra.size
    if mm_len is None:
        mm_len = (TN + T) if monitor else max(len(cseg), TN)
    mm = np.zeros(mm_len, dtype=np.int32)
    for t in completion_order:
        s = int(ra[t])
        g = group_of_slot_literal(cseg, s)
        mm[g] += 1
        if monitor:
            order = int(mm[TN - 1])
            mm[TN - 1] += 1
            mm[TN + s] = order
    return mm


def wait_release(mm: np.ndarray, cseg):
    """The host loop launches one waiter per group, in index order, on one
    stream (src/overlap_impl.cu:257-265); waiter g returns once MM[g] ==
    cSeg[g] and swaps it to 0 (src/wait.cuh:5-9).  Returns the release order
    and the counter state afterwards; raises if a waiter could never return."""
    mm = mm.copy()
    order = []
    for g, that in enumerate(cseg):
        if int(mm[g]) != int(that):
            raise RuntimeError(f"waiter {g} would spin forever: MM={int(mm[g])} cSeg={that}")
        mm[g] = 0
        order.append(g)
    return order, mm


def group_ranges(cseg, BM: int, BN: int):
    """Element range [lo, hi) of the permuted buffer that group g occupies
    (src/overlap_impl.cu:259,264): commSize = M*N/TileNum * cSeg[g]."""
    out, acc = [], 0
    for s in cseg:
        out.append((acc, acc + s * BM * BN))
        acc += s * BM * BN
    return out


def consume_allreduce(cperm: torch.Tensor, cseg, BM: int, BN: int) -> torch.Tensor:
    """One-GPU stand-in for the per-group in-place AllReduce
    (src/overlap_impl.cu:263): every released range is copied to the same
    offsets of a staging buffer."""
    staging = torch.zeros_like(cperm.reshape(-1))
    for lo, hi in group_ranges(cseg, BM, BN):
        staging[lo:hi] = cperm.reshape(-1)[lo:hi]
    return staging


def consume_reducescatter(cperm: torch.Tensor, cseg, BM: int, BN: int, ws: int) -> torch.Tensor:
    """One-GPU stand-in for the per-group ReduceScatter
    (src/overlap_impl.cu:319-320): rank k receives the k-th 1/ws of group g at
    D_k + start_g/ws.  Returns all ws receive buffers stacked, [ws, M*N/ws]."""
    flat = cperm.reshape(-1)
    total = flat.numel()
    D = torch.zeros(ws, total // ws, dtype=flat.dtype)
    for lo, hi in group_ranges(cseg, BM, BN):
        n = (hi - lo) // ws
        for k in range(ws):
            D[k, lo // ws: lo // ws + n] = flat[lo + k * n: lo + (k + 1) * n]
    return D


# --------------------------------------------------------------------------
# floating point
# --------------------------------------------------------------------------


def gemm_fp32(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """D = A . B^T with fp32 accumulation, alpha=1, beta=0
    (src/overlap/gemm_signal.cu:33-39, src/gemm/gemm.cu:33-39)."""
    return A.float() @ B.float().t()


def gemm(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """gemm_fp32 rounded once (RN) to the storage dtype of A
    (src/overlap/gemm_with_signal.h:179: ElementD(alpha * acc))."""
    return gemm_fp32(A, B).to(A.dtype)


def rmsnorm_fp32(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """Textbook RMSNorm in fp32, no storage rounding
    (example/RMSNorm.py:16-21)."""
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * gamma.float()


def rmsnorm(x: torch.Tensor, gamma: torch.Tensor, eps: float) -> torch.Tensor:
    """RMSNorm with the kernel's two storage roundings: the scaled value is
    rounded to the storage dtype, then multiplied by gamma in that dtype
    (src/rmsnorm/rmsnorm.cuh:104-110; the reference fixes eps=1e-5 at :100)."""
    xf = x.float()
    scale = torch.rsqrt(xf.pow(2).sum(-1, keepdim=True) / x.shape[-1] + eps)
    y = (xf * scale).to(x.dtype)
    return (y.float() * gamma.float()).to(x.dtype)


def reorder_rmsnorm(x: torch.Tensor, gamma: torch.Tensor, bs: int, dim: int, BM: int, BN: int,
                    rldn: int, RA, eps: float = 1e-5) -> torch.Tensor:
    """Gather from the tile-permuted buffer, then RMSNorm
    (src/rmsnorm/rmsnorm.cuh:62-115)."""
    return rmsnorm(gather_tiles(x, bs, dim, BM, BN, rldn, RA), gamma, eps)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.double() - b.double()).abs().max())


# --------------------------------------------------------------------------
# tuner
# --------------------------------------------------------------------------


def vote_hint_literal(samples, wSize: int):
    """Statement-by-statement twin of the majority vote in tune/search.py:218-263
    (plain loops; torch.mode's tie rule = smallest value)."""
    n = len(samples)
    TileNum = len(samples[0])
    WaveNum = div_up(TileNum, wSize)
    tile_wave = [[min(samples[i][t] // wSize, WaveNum - 1) for t in range(TileNum)] for i in range(n)]
    tile_modes, mode_counts = [], []
    for ti in range(TileNum):
        col = [tile_wave[i][ti] for i in range(n)]
        best = max(set(col), key=lambda v: (col.count(v), -v))
        tile_modes.append(best)
        mode_counts.append(col.count(best))
    wave_tiles = {w: [] for w in range(WaveNum)}
    for ti in range(TileNum):
        wave_tiles[tile_modes[ti]].append((mode_counts[ti], ti))
    for w in wave_tiles:
        wave_tiles[w].sort(reverse=True)
    unassigned = []
    assigned = {w: [] for w in range(WaveNum)}
    for w in range(WaveNum):
        target = wSize if w < WaveNum - 1 else TileNum - w * wSize
        tiles = wave_tiles[w]
        assigned[w] = [t[1] for t in tiles[:target]]
        unassigned.extend([t[1] for t in tiles[target:]])
    for w in range(WaveNum):
        target = wSize if w < WaveNum - 1 else TileNum - w * wSize
        while len(assigned[w]) < target and unassigned:
            assigned[w].append(unassigned.pop())
    hint = []
    for w in range(WaveNum):
        target = wSize if w < WaveNum - 1 else TileNum - w * wSize
        if len(assigned[w]) < target:
            return False, []
        hint.extend(assigned[w])
    return True, hint


def predict_latency_literal(gemm_dur, comm_ms, gp, wave_size, tile_num, tile_bytes):
    """Pipeline recurrence of tune/search.py:316-344 without the reference's
    rescaling for compute units set aside for the collective."""
    if len(gp) == 1:
        return comm_ms(gp[0] * tile_bytes) + gemm_dur
    wave_num = div_up(tile_num, wave_size)
    acc_comm = acc_comp = 0.0
    for i in range(len(gp)):
        comm = 0.0 if i == 0 else comm_ms(gp[i - 1] * tile_bytes)
        acc_comm = max(acc_comp, acc_comm) + comm
        acc_comp += gemm_dur / wave_num * div_up(gp[i], wave_size)
    return max(acc_comp, acc_comm) + comm_ms(gp[-1] * tile_bytes)
