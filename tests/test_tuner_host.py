"""CPU tests of the tuner slice and the config files: vote and latency model
against the oracle's literal twins and against closed forms; the JSON layout
against what the reference's scripts read and write."""
import json

import numpy as np
import pytest

from flashoverlap_amd import config, tiling, tuner
from oracle import fo_oracle as O


def _noisy_samples(T, w, n, swaps, seed):
    rng = np.random.default_rng(seed)
    base = rng.permutation(T)            # base[rank] = tile
    out = []
    for _ in range(n):
        order = base.copy()
        for _ in range(swaps):
            i, j = rng.integers(0, T, 2)
            order[i], order[j] = order[j], order[i]
        ranks = np.empty(T, dtype=np.int64)
        ranks[order] = np.arange(T)
        out.append(ranks)
    return np.array(out), base


def test_vote_recovers_a_clean_order():
    T, w = 24, 5
    samples, base = _noisy_samples(T, w, 7, 0, 0)
    ok, hint = tuner.vote_hint(samples, w)
    assert ok and sorted(hint) == list(range(T))
    for wave in range(tiling.div_up(T, w)):
        assert sorted(hint[wave * w:(wave + 1) * w]) == sorted(base[wave * w:(wave + 1) * w].tolist())


@pytest.mark.parametrize("T,w,n,swaps,seed", [(24, 5, 9, 3, 1), (64, 16, 20, 10, 2), (30, 30, 3, 5, 3), (17, 4, 5, 8, 4),
                                              (8, 1, 4, 2, 5)])
def test_vote_matches_literal_twin_and_keeps_invariants(T, w, n, swaps, seed):
    samples, _ = _noisy_samples(T, w, n, swaps, seed)
    ok, hint = tuner.vote_hint(samples, w)
    ok_l, hint_l = O.vote_hint_literal(samples.tolist(), w)
    assert (ok, hint) == (ok_l, hint_l)
    if ok:
        assert sorted(hint) == list(range(T))
        # a tile that every sample saw in the same wave stays in that wave if the wave is not oversubscribed
        waves = np.minimum(samples // w, tiling.div_up(T, w) - 1)
        unanimous = [t for t in range(T) if (waves[:, t] == waves[0, t]).all()]
        per_wave = {x: sum(1 for t in unanimous if waves[0, t] == x) for x in set(waves[0])}
        for t in unanimous:
            if per_wave[waves[0, t]] <= (w if waves[0, t] < tiling.div_up(T, w) - 1 else T - waves[0, t] * w):
                assert hint.index(t) // w == waves[0, t]


def test_vote_rejects_bad_input():
    with pytest.raises(ValueError):
        tuner.vote_hint(np.zeros((0, 4)), 2)


def test_predict_latency_closed_forms():
    comm = lambda b: b / 1000.0
    # one group: nothing overlaps
    assert tuner.predict_latency(2.0, comm, [8], 2, 8, 500) == pytest.approx(2.0 + 4.0)
    # free transfers: the GEMM time
    assert tuner.predict_latency(2.0, lambda b: 0.0, [2, 2, 4], 2, 8, 500) == pytest.approx(2.0)
    # transfers much slower than compute: first group's compute, then all transfers back to back
    slow = lambda b: b * 1.0
    assert tuner.predict_latency(4.0, slow, [2, 2, 4], 2, 8, 1) == pytest.approx(4.0 / 4 * 1 + 2 + 2 + 4)
    # against the oracle's recurrence on every composition
    for gp in tiling.integer_partitions(5):
        cseg = tiling.cseg_from_groups(gp, 3, 14)
        assert tuner.predict_latency(1.7, comm, cseg, 3, 14, 640) == pytest.approx(
            O.predict_latency_literal(1.7, comm, cseg, 3, 14, 640))


def test_predictive_search_prefers_overlap_when_transfers_are_cheap_and_one_group_when_latency_dominates():
    cheap = lambda b: b / 1e6
    cseg, t = tuner.predictive_search(1.0, cheap, 4, 16, 1000)
    assert sum(cseg) == 16 and len(cseg) > 1 and t < 1.0 + cheap(16 * 1000)
    fixed_cost = lambda b: 5.0 + b / 1e9
    cseg, t = tuner.predictive_search(1.0, fixed_cost, 4, 16, 1000)
    assert cseg == [16]
    with pytest.raises(ValueError):
        tuner.predictive_search(1.0, cheap, 1, 64, 10)


def test_config_files_use_the_reference_layout(tmp_path):
    path = config.config_path(4096, 4096, 4096, "mi355x", str(tmp_path))
    assert path.endswith("m4096n4096k4096_mi355x.json")
    config.save_profile(path, [128, 256], [128, 128], [0.12, 0.15], [1, 5])
    assert json.load(open(path)) == {"BM": [128, 256], "BN": [128, 128], "dur": [0.12, 0.15], "Algo": [1, 5]}
    with pytest.raises(ValueError, match="no search result"):
        config.load_config(path)
    T = 32 * 32
    hint = list(range(T))[::-1]
    cseg = tiling.uniform_cseg(T, 256)
    config.save_solution(path, 128, 128, 0.12, 1, hint, cseg)
    data = json.load(open(path))
    assert set(data) == {"BM", "BN", "dur", "Algo", "hint", "cSeg", "rLDN"} and data["rLDN"] == 1
    got = config.load_config(path, 4096, 4096)
    assert got["hint"] == hint and got["cSeg"] == cseg and got["BM"] == 128 and got["Algo"] == 1
    config.save_solution(path, 128, 128, 0.12, 1, hint, cseg[:-1])
    with pytest.raises(ValueError, match="sum\\(cSeg\\)"):
        config.load_config(path, 4096, 4096)
    config.save_solution(path, 128, 128, 0.12, 1, [0, 0], cseg)
    with pytest.raises(ValueError, match="hint"):
        config.load_config(path, 4096, 4096)
    assert config.gpu_tag("AMD Instinct MI355X") == "mi355x"
