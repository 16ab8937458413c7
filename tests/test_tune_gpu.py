"""The tuning steps of tune/profile_config.py, tune/bandwidth.py and tune/search.py on one GPU, with the
consumer copy as the transfer: the files they write have the reference's layout, and the overlapped call
driven by the searched file gives the oracle's result."""
import json

import pytest
import torch

import flashoverlap_amd
from flashoverlap_amd import capi, config, speed_test, tiling, tune
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu

M, N, K = 8192, 4096, 512            # 2048 tiles of 128x128: two waves of 1024
FAST = {"warm_up": 2, "rep": 5}


def _check_overlapped_call(cfg, comm_op, ws):
    keep = {}
    speed_test.perf_running(M, N, K, cfg["BM"], cfg["BN"], cfg["Algo"], cfg["cSeg"], cfg["hint"], comm_op, ws,
                            torch.float16, "cuda", keep=keep, **FAST)
    torch.cuda.synchronize()
    assert keep["overlap"].wait_timeouts(True) == 0 and keep["counters"].cpu().sum() == 0
    cref = O.gemm(keep["A"].cpu(), keep["B"].cpu())
    ra = keep["RA"].cpu().numpy()
    if comm_op == "all_reduce":
        got = keep["C"].cpu().reshape(-1) if len(cfg["cSeg"]) == 1 else keep["overlap"].staging().cpu().reshape(-1)
        want = cref.reshape(-1) if len(cfg["cSeg"]) == 1 else O.place_tiles(cref, ra, cfg["BM"], cfg["BN"], 1).reshape(-1)
    else:
        got = keep["D"].cpu().reshape(-1)
        if len(cfg["cSeg"]) == 1:
            want = cref[: M // ws].reshape(-1)
        else:
            want = O.consume_reducescatter(O.scatter_place(cref, ra, keep["RE"].cpu().numpy(), cfg["BM"], cfg["BN"], 1),
                                           cfg["cSeg"], cfg["BM"], cfg["BN"], ws)[0].reshape(-1)
    assert O.rel_l2(got, want) < 1e-3


def test_profile_then_exhaustive_search(dev, tmp_path):
    flashoverlap_amd.load()
    capi.check(capi.lib().fo_set_wait_timeout_ms(5000))
    root = str(tmp_path)
    path = tune.profile_config(M, N, K, torch.float16, root, **FAST)
    assert path == config.config_path(M, N, K, config.current_gpu_tag(), root)
    prof = json.load(open(path))
    assert set(prof) == {"BM", "BN", "dur", "Algo"}
    n = len(prof["Algo"])
    assert n == capi.lib().fo_algo_count() and prof["dur"] == sorted(prof["dur"]) and all(d > 0 for d in prof["dur"])
    for bm, bn, algo in zip(prof["BM"], prof["BN"], prof["Algo"]):
        assert capi.algo_tile(algo)[:2] == (bm, bn)
    with pytest.raises(ValueError, match="no search result"):
        config.load_config(path)

    said = []
    got = tune.search(M, N, K, "all_reduce", 1, torch.float16, root, say=said.append, **FAST)
    cfg = config.load_config(path, M, N)
    tiles = (M // cfg["BM"]) * (N // cfg["BN"])
    wave = tune.wave_tiles(cfg["BM"], cfg["BN"], torch.cuda.get_device_properties(0).multi_processor_count)
    assert cfg["cSeg"] == got["cSeg"] and cfg["cSeg"] in tune.candidate_csegs(tiles, wave)
    assert sorted(cfg["hint"]) == list(range(tiles)) and cfg["rLDN"] == 1
    assert cfg["Algo"] in prof["Algo"] and isinstance(cfg["dur"], float)
    timed = [s for s in said if s.startswith("[")]
    assert len(timed) == len(tune.candidate_csegs(tiles, wave))      # every composition was timed
    assert any("consistent completion order" in s for s in said)
    _check_overlapped_call(cfg, "all_reduce", 1)


def test_bandwidth_curve_then_predictive_search(dev, tmp_path):
    flashoverlap_amd.load()
    capi.check(capi.lib().fo_set_wait_timeout_ms(5000))
    root = str(tmp_path)
    ws = 4
    with pytest.raises(FileNotFoundError):
        tune.load_profile(config.config_path(M, N, K, "mi355x", root))
    tune.profile_config(M, N, K, torch.float16, root, top=2, **FAST)
    with pytest.raises(FileNotFoundError, match="bandwidth step"):
        tune.search(M, N, K, "reduce_scatter", ws, torch.float16, root, predictive=True, say=lambda s: None, **FAST)
    cpath = tune.bandwidth_curve("reduce_scatter", ws, torch.float16, root, points=9, verbose=False, **FAST)
    assert cpath == tune.curve_path("reduce_scatter", ws, root)
    curve = torch.load(cpath, weights_only=True)
    assert curve.shape == (9, 2) and curve[:, 0].tolist() == [float(s) for s in tune.curve_sizes(9)]
    assert (curve[:, 1] > 1.0).all()               # GiB/s of a device copy
    # at these sizes (2 to 8 MiB, a quarter of it copied) a transfer is a kernel launch: microseconds, not milliseconds
    lat = [tune.interpolate_latency(curve.numpy(), s) for s in tune.curve_sizes(9)]
    assert all(0.001 < t < 1.0 for t in lat)
    said = []
    got = tune.search(M, N, K, "reduce_scatter", ws, torch.float16, root, predictive=True, say=said.append, **FAST)
    cfg = config.load_config(config.config_path(M, N, K, config.current_gpu_tag(), root), M, N)
    assert cfg["cSeg"] == got["cSeg"] and sum(cfg["cSeg"]) == (M // cfg["BM"]) * (N // cfg["BN"])
    assert "Bandwidth curve captured." in said and any("predicted" in s and "measured" in s for s in said)
    assert got["ms"] > 0
    _check_overlapped_call(cfg, "reduce_scatter", ws)
