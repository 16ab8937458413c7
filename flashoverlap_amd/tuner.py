"""Wave-group tuning helpers: the single-GPU slice of the reference tuner
(tune/search.py).

What is here: the monitor-mode sampling pass and its majority vote
(tune/search.py:164-263), the pipeline latency model and the predictive search
over wave compositions (tune/search.py:316-344, 462-471, 502-513), with the
consumer copy in the place of the collective.  The measuring steps around them
(GEMM profile, bandwidth curve, timed and predictive search, the tuning file)
are in tune.py.

The vote exists in the reference because its GEMM scheduler is opaque; this
library's issue order is a known function (tiling.raster_hint), so the sampled
hint is mainly a cross-check of that function against the hardware.
"""
from __future__ import annotations

import numpy as np
import torch

from . import tiling


def vote_hint(samples, wave_size: int):
    """Majority vote over sampled completion ranks (tune/search.py:218-263).

    samples: [n_samples, T] integer array, samples[i, t] = completion rank of
    tile t in sample i.  Every tile is assigned to the wave (rank // wave_size)
    it was seen in most often; a wave keeps its most confident tiles up to its
    size and the surplus fills waves that are short.  Returns (consistent,
    hint) with hint the tiles wave by wave.
    """
    s = np.asarray(samples, dtype=np.int64)
    if s.ndim != 2 or s.shape[0] == 0:
        raise ValueError("samples must be [n_samples, T]")
    n, T = s.shape
    waves = tiling.div_up(T, wave_size)
    tw = np.minimum(s // wave_size, waves - 1)
    # mode per tile, smallest value on ties (what torch.mode returns)
    counts = np.zeros((waves, T), dtype=np.int64)
    for w in range(waves):
        counts[w] = (tw == w).sum(axis=0)
    mode = counts.argmax(axis=0)
    conf = counts.max(axis=0)
    target = [wave_size if w < waves - 1 else T - w * wave_size for w in range(waves)]
    assigned, spare = [], []
    for w in range(waves):
        tiles = [t for t in range(T) if mode[t] == w]
        # most confident first; among equals the higher tile id first, as the reference's
        # reverse sort of (count, tile) pairs does
        tiles.sort(key=lambda t: (conf[t], t), reverse=True)
        assigned.append(tiles[:target[w]])
        spare.extend(tiles[target[w]:])
    for w in range(waves):
        while len(assigned[w]) < target[w] and spare:
            assigned[w].append(spare.pop())
    consistent = all(len(assigned[w]) == target[w] for w in range(waves))
    hint = [t for w in range(waves) for t in assigned[w]] if consistent else []
    return consistent, hint


def sample_completion_order(overlap, M: int, N: int, K: int, algo: int, BM: int, BN: int, wave_size: int,
                            dtype=torch.float16, samples: int = 20, warmup: int = 5, device="cuda"):
    """Monitor pass of tune/search.py:164-187 on one GPU: identity RA, MM of
    (TM+1) x TN, if_monitor=True; returns an int tensor [samples, T] of
    completion ranks.  `overlap` is an initialised OverlapImpl."""
    TM, TN = M // BM, N // BN
    T = TM * TN
    cseg = tiling.uniform_cseg(T, wave_size)
    if len(cseg) > TN - 1:
        raise ValueError(f"monitor mode keeps its ticket counter in MM[TN-1]: {len(cseg)} groups need TN > {len(cseg)}")
    cseg_cpu = torch.tensor(cseg, dtype=torch.int32)
    cseg_gpu = cseg_cpu.to(device)
    A = torch.empty((M, K), dtype=dtype, device=device).normal_(0.0, 0.5)
    B = torch.empty((N, K), dtype=dtype, device=device).normal_(0.0, 0.5)
    C = torch.empty((M, N), dtype=dtype, device=device)
    mm = torch.zeros((TM + 1, TN), dtype=torch.int32, device=device)
    ra = torch.arange(0, T, dtype=torch.int32, device=device).reshape(TM, TN)
    out = torch.empty((samples, T), dtype=torch.int32, device=device)
    for i in range(warmup + samples):
        mm[0] = 0
        overlap.gemm_allreduce_overlap(A, B, C, mm, ra, 1, cseg_cpu, cseg_gpu, algo, True)
        if i >= warmup:
            out[i - warmup, :] = mm[1:, :].reshape(-1)
    torch.cuda.synchronize()
    return out.cpu()


def predict_latency(gemm_ms: float, comm_ms, groups, wave_size: int, tile_num: int, tile_bytes: int) -> float:
    """Pipeline model of tune/search.py:316-344: group i's transfer starts when
    both its tiles and the previous transfer are done.  groups are tile counts
    per group (multiples of wave_size except the last); comm_ms(bytes) is the
    time of one transfer.  Unlike the reference no compute units are set aside
    for the transfer, so the GEMM time is not rescaled."""
    waves = tiling.div_up(tile_num, wave_size)
    if len(groups) == 1:
        return gemm_ms + comm_ms(groups[0] * tile_bytes)
    comp = comm = 0.0
    for i, g in enumerate(groups):
        dur = 0.0 if i == 0 else comm_ms(groups[i - 1] * tile_bytes)
        comm = max(comp, comm) + dur
        comp += gemm_ms / waves * tiling.div_up(g, wave_size)
    return max(comp, comm) + comm_ms(groups[-1] * tile_bytes)


def predictive_search(gemm_ms: float, comm_ms, wave_size: int, tile_num: int, tile_bytes: int, max_waves: int = 16):
    """Best wave composition under predict_latency (the predictive branch of
    tune/search.py:516-600).  Returns (cSeg, predicted_ms)."""
    waves = tiling.div_up(tile_num, wave_size)
    if waves > max_waves:
        raise ValueError(f"{waves} waves give 2^{waves - 1} compositions; raise max_waves to search them")
    best = None
    for gp in tiling.integer_partitions(waves):
        cseg = tiling.cseg_from_groups(gp, wave_size, tile_num)
        t = predict_latency(gemm_ms, comm_ms, cseg, wave_size, tile_num, tile_bytes)
        if best is None or t < best[1]:
            best = (cseg, t)
    return best
