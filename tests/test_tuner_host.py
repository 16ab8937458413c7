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
    assert config.gpu_tag("AMD Radeon Graphics", "gfx950:sramecc+:xnack-") == "gfx950"
    assert config.gpu_tag("AMD Instinct MI355X", "gfx950:sramecc+:xnack-") == "mi355x"
    # a file saved under the architecture is found by a driver that reports the product, and the other way round
    config.save_profile(config.config_path(8, 8, 8, "gfx950", str(tmp_path)), [128], [128], [0.1], [1])
    assert config.find_config(8, 8, 8, ["mi355x", "gfx950"], str(tmp_path)).endswith("m8n8k8_gfx950.json")
    assert config.find_config(8, 8, 16, ["mi355x", "gfx950"], str(tmp_path)).endswith("m8n8k16_mi355x.json")


# ---- the tuning driver's host logic (flashoverlap_amd/tune.py)

def test_curve_sizes_follow_the_reference_grid():
    from flashoverlap_amd import tune
    sizes = tune.curve_sizes()
    assert len(sizes) == 36 and sizes[0] == 1 << 20 and sizes[4] == 1 << 21 and sizes[32] == 1 << 28
    assert all(s % 1024 == 0 for s in sizes) and all(b > a for a, b in zip(sizes, sizes[1:]))
    assert sizes[1] == int(2 ** 20.25) // 1024 * 1024


def test_interpolated_latency_known_answers():
    from flashoverlap_amd import tune
    gib = 1024 ** 3
    curve = [(1 << 20, 100.0), (1 << 22, 300.0), (1 << 24, 300.0)]
    # on a point: bytes / bandwidth
    assert tune.interpolate_latency(curve, 1 << 20) == pytest.approx((1 << 21) / (100.0 * gib) * 1000)
    # half way between two points the bandwidth is their mean
    mid = ((1 << 20) + (1 << 22)) / 2
    assert tune.interpolate_latency(curve, mid) == pytest.approx(mid * 2 / (200.0 * gib) * 1000)
    # outside the curve the end values hold, so the time grows with the size
    assert tune.interpolate_latency(curve, 1 << 26) == pytest.approx((1 << 27) / (300.0 * gib) * 1000)
    assert tune.interpolate_latency(curve, 1 << 10) == pytest.approx((1 << 11) / (100.0 * gib) * 1000)
    # four-byte elements move twice the bytes
    assert tune.interpolate_latency(curve, 1 << 22, 4) == pytest.approx(2 * tune.interpolate_latency(curve, 1 << 22))
    for bad in ([], [(1, 2, 3)], [(2, 1.0), (1, 1.0)], [(1, 0.0), (2, 1.0)]):
        with pytest.raises(ValueError):
            tune.interpolate_latency(bad, 10)


def test_wave_tiles_and_candidates():
    from flashoverlap_amd import tune
    assert tune.wave_tiles(128, 128) == 1024 and tune.wave_tiles(256, 128) == 512 and tune.wave_tiles(256, 256, 304) == 304
    with pytest.raises(ValueError):
        tune.wave_tiles(96, 128)
    # c4: 8192 tiles of 128x128 are eight waves
    all_of_c4 = tune.candidate_csegs(8192, 1024)
    assert len(all_of_c4) == 2 ** 7 and all(sum(c) == 8192 for c in all_of_c4)
    assert all_of_c4[0] == [1024] * 8 and all_of_c4[-1] == [8192]
    assert len({tuple(c) for c in all_of_c4}) == len(all_of_c4)
    # a last wave that is not full is clipped, never dropped
    ragged = tune.candidate_csegs(2500, 1024)
    assert sorted(map(tuple, ragged)) == sorted([(1024, 1024, 452), (1024, 1476), (2048, 452), (2500,)])
    # groups of two waves at least: four units
    coarse = tune.candidate_csegs(8192, 1024, 2)
    assert len(coarse) == 2 ** 3 and all(g % 2048 == 0 for c in coarse for g in c)
    # the predictive search's pruning: more than five groups only with a first group of one or two units
    pruned = tune.candidate_csegs(8192, 1024, prune=True)
    dropped = [c for c in all_of_c4 if c not in pruned]
    assert dropped and all(len(c) > 5 and c[0] > 2048 for c in dropped)
    assert all(not (len(c) > 5 and c[0] > 2048) for c in pruned)


def test_model_ranking_orders_by_the_pipeline_model():
    from flashoverlap_amd import tune
    cands = tune.candidate_csegs(4096, 1024)
    tile_elems = 128 * 128
    # a transfer that costs next to nothing: every partition predicts the GEMM time, the order of enumeration stays
    fast = [(1 << 20, 1e9), (1 << 28, 1e9)]
    ranked = tune.rank_by_model(1.0, fast, cands, 1024, 4096, tile_elems)
    assert [c for _, c in ranked][0] == cands[0] and all(t == pytest.approx(1.0, abs=1e-3) for t, _ in ranked)
    # a slow link (1 GiB/s: the 32 MiB of a wave take 31 ms against 0.25 ms of compute): every prediction
    # must equal the oracle's recurrence, best first
    slow = [(1 << 20, 1.0), (1 << 28, 1.0)]
    ranked = tune.rank_by_model(1.0, slow, cands, 1024, 4096, tile_elems)
    comm = lambda nbytes: tune.interpolate_latency(slow, nbytes / 2)
    for t, c in ranked:
        assert t == pytest.approx(O.predict_latency_literal(1.0, comm, c, 1024, 4096, tile_elems * 2))
    assert [t for t, _ in ranked] == sorted(t for t, _ in ranked)
    assert ranked[-1][1] == [4096]          # nothing overlapped is the worst when the link is the bottleneck


def test_profile_lists_are_read_back(tmp_path):
    from flashoverlap_amd import tune
    path = str(tmp_path / "m1n1k1_x.json")
    config.save_profile(path, [128, 256], [128, 128], [0.2, 0.3], [1, 5])
    assert tune.load_profile(path) == ([128, 256], [128, 128], [0.2, 0.3], [1, 5])
    config.save_solution(path, 128, 128, 0.2, 1, [0], [1])
    assert tune.load_profile(path) == ([128], [128], [0.2], [1])
    json.dump({"BM": [128]}, open(path, "w"))
    with pytest.raises(ValueError, match="profile step"):
        tune.load_profile(path)
    assert tune.curve_path("all_reduce", 1, "cfg").endswith("cfg/bandwidth_all_reduce_tp1.pt")


def test_sweep_rows_follow_the_reference_table():
    from flashoverlap_amd import sweep_gemm
    assert sweep_gemm.note_for(1.0) == "<== CLOSE" and sweep_gemm.note_for(1.1) == "<== CLOSE"
    assert sweep_gemm.note_for(1.2) == "<= OK" and sweep_gemm.note_for(1.3) == "<= OK" and sweep_gemm.note_for(1.31) == ""
    row = sweep_gemm.format_row(1024, 2048, 4096, 3, 0.5, 0.6)
    assert row.split() == ["1024", "2048", "4096", "3", "0.5000", "0.6000", "1.20", "<=", "OK"]
    assert len(row) == len(sweep_gemm.HEADER)
    failed = sweep_gemm.format_row(1024, 2048, 4096, -1, 0.5, None)
    assert failed.split() == ["1024", "2048", "4096", "FAIL", "0.5000", "N/A", "N/A"]
