"""The reference's three tuning steps on one MI355X, through the torch API only.

  python -m flashoverlap_amd.tune profile   --m_dim M --n_dim N --k_dim K      tune/profile_config.py
  python -m flashoverlap_amd.tune bandwidth --comm_op all_reduce               tune/bandwidth.py
  python -m flashoverlap_amd.tune search    --m_dim M --n_dim N --k_dim K      tune/search.py
  python -m flashoverlap_amd.tune all       --m_dim M --n_dim N --k_dim K      the three in a row

`profile` times the plain GEMM under every Algo and writes the ten fastest, best
first, as lists `BM BN dur Algo` into configs/m{M}n{N}k{K}_{gpu}.json
(tune/profile_config.py:78-111).  `bandwidth` times the bulk transfer over 36
message sizes from 2^20 to 2^28.75 elements and stores (elements, GiB/s) pairs in
configs/bandwidth_{comm_op}_tp{world_size}.pt (tune/bandwidth.py:108-152).
`search` samples the completion order in monitor mode, votes a `hint`, picks
`cSeg` either by timing every wave composition (tune/search.py:473-514) or by
the pipeline model over the bandwidth curve (tune/search.py:517-588), and adds
`hint cSeg rLDN` and the chosen scalars to the shape's file, which
speed_test.py and layers.py then read.

On one GPU the transfer is the consumer copy, so a curve point is message bytes
per second of that copy (the reference's bus-bandwidth factors 2(n-1)/n and
(n-1)/n vanish at n = 1 and are left out on both sides of the interpolation).
A wave is what the GPU holds at a time: one 256x256 macro tile per compute
unit, i.e. cu_count * (256/BM) * (256/BN) layout tiles; nothing is set aside for
the transfer, so the model does not rescale the GEMM time as the reference does
for its two reserved processors.  Beyond the reference: the predictive search
also times its few best candidates and keeps the one that measured best, and
both searches time the single-group call so that the file never holds a
partition that lost against not overlapping at all.
"""
from __future__ import annotations

import argparse
import json
import os
import sys

import numpy as np
import torch

from . import capi, config, load, speed_test, tiling, tuner

EXHAUSTIVE_UP_TO_ELEMENTS = 33554432   # tune/search.py:606: larger outputs take the predictive search
CURVE_POINTS = 36


# ------------------------------------------------------------------ host logic (no GPU)

def curve_sizes(points: int = CURVE_POINTS) -> list:
    """Message sizes in elements, a quarter octave apart, multiples of 1024 (tune/bandwidth.py:108)."""
    return [int(2 ** (20 + 0.25 * i)) // 1024 * 1024 for i in range(points)]


def interpolate_latency(samples, elements: float, element_bytes: int = 2) -> float:
    """Milliseconds of one transfer of `elements` elements: the bandwidth is interpolated linearly
    between the curve's points and held constant outside them (tune/search.py:294-313)."""
    s = np.asarray(samples, dtype=np.float64)
    if s.ndim != 2 or s.shape[1] != 2 or s.shape[0] == 0:
        raise ValueError("samples must be [n, 2] pairs of (elements, GiB/s)")
    if np.any(np.diff(s[:, 0]) <= 0) or np.any(s[:, 1] <= 0):
        raise ValueError("curve sizes must increase and bandwidths must be positive")
    bw = float(np.interp(float(elements), s[:, 0], s[:, 1]))
    return float(elements) * element_bytes / bw / (1024 ** 3) * 1000.0


def wave_tiles(BM: int, BN: int, cu_count: int = 256) -> int:
    """Layout tiles that finish together: one 256x256 macro tile per compute unit."""
    if 256 % BM or 256 % BN:
        raise ValueError(f"layout tile {BM}x{BN} does not divide the 256x256 macro tile")
    return cu_count * (256 // BM) * (256 // BN)


def candidate_csegs(tile_num: int, wave_size: int, min_group_waves: int = 1, prune: bool = False) -> list:
    """Every cSeg whose groups are whole multiples of `min_group_waves` waves, in the reference's
    enumeration order.  With `prune`, compositions of more than five groups whose first group is
    longer than two units are skipped, as the predictive search does (tune/search.py:561-562)."""
    waves = tiling.div_up(tile_num, wave_size)
    units = tiling.div_up(waves, min_group_waves)
    out = []
    for gp in tiling.integer_partitions(units):
        if prune and len(gp) > 5 and gp[0] > 2:
            continue
        out.append(tiling.cseg_from_groups(gp, wave_size * min_group_waves, tile_num))
    return out


def rank_by_model(gemm_ms: float, samples, csegs, wave_size: int, tile_num: int, tile_elements: int,
                  element_bytes: int = 2) -> list:
    """(predicted ms, cSeg) for every candidate, best first; ties keep the enumeration order."""
    comm = lambda nbytes: interpolate_latency(samples, nbytes / element_bytes, element_bytes)
    scored = [(tuner.predict_latency(gemm_ms, comm, c, wave_size, tile_num, tile_elements * element_bytes), i, c)
              for i, c in enumerate(csegs)]
    scored.sort(key=lambda t: (t[0], t[1]))
    return [(t, c) for t, _, c in scored]


def curve_path(comm_op: str, world_size: int, root: str = "configs") -> str:
    return os.path.join(root, f"bandwidth_{comm_op}_tp{world_size}.pt")


def load_profile(path: str):
    """The candidate lists a profile wrote; a file that already holds a search result gives its one choice."""
    with open(path, "r", encoding="utf-8") as f:
        data = json.load(f)
    for key in ("BM", "BN", "dur", "Algo"):
        if key not in data:
            raise ValueError(f"{path}: no '{key}'; run the profile step first")
    as_list = lambda v: list(v) if isinstance(v, list) else [v]
    BM, BN, dur, algo = (as_list(data[k]) for k in ("BM", "BN", "dur", "Algo"))
    if not (len(BM) == len(BN) == len(dur) == len(algo)) or not BM:
        raise ValueError(f"{path}: BM, BN, dur and Algo must be lists of one length")
    return BM, BN, dur, algo


# ------------------------------------------------------------------ measurements

def _gpu_tag() -> str:
    return config.current_gpu_tag()


def _cu_count() -> int:
    return torch.cuda.get_device_properties(0).multi_processor_count


def profile_config(M: int, N: int, K: int, dtype=torch.float16, root: str = "configs", top: int = 10, **kw) -> str:
    """tune/profile_config.py:78-111: the plain GEMM under every Algo whose tile divides the
    output, the `top` fastest kept, best first."""
    load()
    timed = []
    for algo in range(capi.lib().fo_algo_count()):
        BM, BN, _ = capi.algo_tile(algo)
        if M % BM or N % BN:
            continue
        timed.append((speed_test.perf_mutlass_gemm(M, N, K, algo, dtype, "cuda", **kw), BM, BN, algo))
    if not timed:
        raise ValueError(f"no Algo's tile divides {M}x{N}")
    timed.sort(key=lambda t: t[0])
    timed = timed[:top]
    path = config.config_path(M, N, K, _gpu_tag(), root)
    config.save_profile(path, [t[1] for t in timed], [t[2] for t in timed], [t[0] for t in timed], [t[3] for t in timed])
    return path


def bandwidth_curve(comm_op: str = "all_reduce", world_size: int = 1, dtype=torch.float16, root: str = "configs",
                    points: int = CURVE_POINTS, verbose: bool = True, **kw) -> str:
    """tune/bandwidth.py:108-152 with the consumer copy as the transfer."""
    load()
    sizes = curve_sizes(points)
    curve = torch.zeros((len(sizes), 2))
    for i, size in enumerate(sizes):
        ms = speed_test.perf_comm(1024, size // 1024, comm_op, world_size, dtype, "cuda", **kw)
        gibs = size * dtype.itemsize / (ms / 1000.0) / (1024 ** 3)
        curve[i, 0], curve[i, 1] = size, gibs
        if verbose:
            print(f"Size: {size / 2 ** 20:.1f} M elements, {ms * 1000:.1f} us, {gibs:.1f} GiB/s", flush=True)
    path = curve_path(comm_op, world_size, root)
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    torch.save(curve, path)
    return path


def compute_hint(M: int, N: int, K: int, BM: int, BN: int, Algo: int, wave_size: int, dtype=torch.float16,
                 samples: int = 20):
    """tune/search.py:155-291: sample the completion ranks in monitor mode, vote.  Returns
    (consistent, hint, agrees) with `agrees` saying whether every wave of the voted hint holds the
    tiles this library's own issue order puts there."""
    o = speed_test._overlap_object()
    ranks = tuner.sample_completion_order(o, M, N, K, Algo, BM, BN, wave_size, dtype, samples=samples)
    ok, hint = tuner.vote_hint(ranks.numpy(), wave_size)
    agrees = False
    if ok:
        issue = tiling.raster_hint(M, N, Algo)
        agrees = all(sorted(hint[w:w + wave_size]) == sorted(issue[w:w + wave_size])
                     for w in range(0, len(hint), wave_size))
    return ok, hint, agrees


def _pick_candidate(M, N, K, BM_list, BN_list, dur_list, Algo_list, wave_units, dtype, tries, say):
    """The first profiled candidate whose sampled order votes consistently (tune/search.py:483-498)."""
    for t in range(min(tries, len(BM_list))):
        BM, BN, dur, Algo = BM_list[t], BN_list[t], dur_list[t], Algo_list[t]
        tile_num = tiling.div_up(M, BM) * tiling.div_up(N, BN)
        wave = wave_tiles(BM, BN, _cu_count())
        wave_num = tiling.div_up(tile_num, wave)
        unit = wave_units(wave_num)
        groups = tiling.div_up(tile_num, wave * unit)
        if groups > N // BN - 1:
            # monitor mode keeps its ticket counter in MM[TN-1]; with that many groups the sampling
            # pass cannot run, and this library's issue order is known without it
            say(f"Algo {Algo}: {groups} groups leave no room for the monitor's ticket counter; using the issue order")
            return BM, BN, dur, Algo, tiling.raster_hint(M, N, Algo), tile_num, wave, wave_num, unit
        ok, hint, agrees = compute_hint(M, N, K, BM, BN, Algo, wave * unit, dtype)
        if ok:
            say(f"Algo {Algo} ({BM}x{BN}): consistent completion order"
                f"{', equal wave by wave to the issue order' if agrees else ', differs from the issue order'}")
            return BM, BN, dur, Algo, hint, tile_num, wave, wave_num, unit
        say(f"Algo {Algo} ({BM}x{BN}): completion order not consistent, trying the next candidate")
    raise RuntimeError("Tuning fails: no candidate gave a consistent completion order; raise the group size")


def _time(M, N, K, BM, BN, Algo, cseg, hint, comm_op, world_size, dtype, **kw) -> float:
    return speed_test.perf_running(M, N, K, BM, BN, Algo, cseg, hint, comm_op, world_size, dtype, "cuda", **kw)


def exhaustive_search(M: int, N: int, K: int, comm_op: str = "all_reduce", world_size: int = 1, dtype=torch.float16,
                      root: str = "configs", max_waves: int = 12, say=print, **kw) -> dict:
    """tune/search.py:473-514: every composition of the waves is timed."""
    load()
    path = config.config_path(M, N, K, _gpu_tag(), root)
    BM, BN, dur, Algo, hint, tile_num, wave, wave_num, _ = _pick_candidate(
        M, N, K, *load_profile(path), lambda w: 1, dtype, 5, say)
    if wave_num > max_waves:
        raise ValueError(f"{wave_num} waves give 2^{wave_num - 1} compositions to time; use the predictive search")
    say("Start exhaustive searching.")
    best = None
    for cseg in candidate_csegs(tile_num, wave):
        t = _time(M, N, K, BM, BN, Algo, cseg, hint, comm_op, world_size, dtype, **kw)
        say(f"{cseg} {t:.4f}")
        if best is None or t < best[0]:
            best = (t, cseg)
    say(f"Best solution:  {best[1]}")
    config.save_solution(path, BM, BN, dur, Algo, hint, best[1], 1)
    say("Solution saved.")
    return {"path": path, "cSeg": best[1], "ms": best[0], "BM": BM, "BN": BN, "Algo": Algo}


def fast_search(M: int, N: int, K: int, samples, comm_op: str = "all_reduce", world_size: int = 1, dtype=torch.float16,
                root: str = "configs", confirm: int = 4, say=print, **kw) -> dict:
    """tune/search.py:517-588: the pipeline model over the bandwidth curve ranks the compositions;
    the `confirm` best and the single group are timed and the fastest of those is kept."""
    load()
    path = config.config_path(M, N, K, _gpu_tag(), root)
    BM, BN, dur, Algo, hint, tile_num, wave, wave_num, unit = _pick_candidate(
        M, N, K, *load_profile(path), lambda w: tiling.div_up(w, 10), dtype, 10, say)
    say("Start predictive searching.")
    ranked = rank_by_model(dur, samples, candidate_csegs(tile_num, wave, unit, prune=True), wave * unit, tile_num,
                           BM * BN, dtype.itemsize)
    say("Search process finished.")
    tried = [c for _, c in ranked[:max(1, confirm)]]
    if [tile_num] not in tried:
        tried.append([tile_num])
    predicted = {tuple(c): t for t, c in ranked}
    best = None
    for cseg in tried:
        t = _time(M, N, K, BM, BN, Algo, cseg, hint, comm_op, world_size, dtype, **kw)
        say(f"{cseg} predicted {predicted.get(tuple(cseg), float('nan')):.4f} measured {t:.4f}")
        if best is None or t < best[0]:
            best = (t, cseg)
    say(f"Searched latency: {best[0]:.4f}")
    say(f"Best solution:  {best[1]}")
    config.save_solution(path, BM, BN, dur, Algo, hint, best[1], 1)
    say("Solution saved.")
    return {"path": path, "cSeg": best[1], "ms": best[0], "BM": BM, "BN": BN, "Algo": Algo,
            "predicted_ms": predicted.get(tuple(best[1]))}


def search(M: int, N: int, K: int, comm_op: str = "all_reduce", world_size: int = 1, dtype=torch.float16,
           root: str = "configs", predictive: bool = False, say=print, **kw) -> dict:
    """The choice of tune/search.py:599-612: outputs of more than 2^25 elements, or on request, take the
    predictive search, which needs the bandwidth curve of this transfer and world size."""
    if predictive or M * N > EXHAUSTIVE_UP_TO_ELEMENTS:
        cpath = curve_path(comm_op, world_size, root)
        if not os.path.exists(cpath):
            raise FileNotFoundError(f"{cpath}: run the bandwidth step first")
        samples = torch.load(cpath, weights_only=True)
        say("Bandwidth curve captured.")
        return fast_search(M, N, K, samples.numpy(), comm_op, world_size, dtype, root, say=say, **kw)
    return exhaustive_search(M, N, K, comm_op, world_size, dtype, root, say=say, **kw)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("step", choices=["profile", "bandwidth", "search", "all"])
    ap.add_argument("--m_dim", type=int, default=4096)
    ap.add_argument("--k_dim", type=int, default=8192)
    ap.add_argument("--n_dim", type=int, default=8192)
    ap.add_argument("--comm_op", default="all_reduce", choices=["all_reduce", "reduce_scatter"])
    ap.add_argument("--world_size", type=int, default=1, help="emulated world size of the ReduceScatter slicing")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    ap.add_argument("--predictive_search", action="store_true")
    ap.add_argument("--configs", default="configs", help="directory of the tuning files")
    ap.add_argument("--rep", type=int, default=speed_test.REP)
    ap.add_argument("--warm_up", type=int, default=speed_test.WARM_UP)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("tune: no GPU visible", file=sys.stderr)
        return 2
    dtype = getattr(torch, a.dtype)
    kw = {"warm_up": a.warm_up, "rep": a.rep}
    m, n, k = a.m_dim, a.n_dim, a.k_dim
    if a.step in ("profile", "all"):
        print("GEMM configs saved:", profile_config(m, n, k, dtype, a.configs, **kw))
    need_curve = a.predictive_search or m * n > EXHAUSTIVE_UP_TO_ELEMENTS
    if a.step == "bandwidth" or (a.step == "all" and need_curve
                                 and not os.path.exists(curve_path(a.comm_op, a.world_size, a.configs))):
        print("Bandwidth curve saved:", bandwidth_curve(a.comm_op, a.world_size, dtype, a.configs, **kw))
    if a.step in ("search", "all"):
        search(m, n, k, a.comm_op, a.world_size, dtype, a.configs, a.predictive_search, **kw)
    return 0


if __name__ == "__main__":
    sys.exit(main())
