"""GPU tests of the nn.Module wrappers and the tuner's monitor pass, following
example/correctness_ar.py:99-127, example/correctness_rs.py:100-142 and
tune/search.py:164-263 on one GPU."""
import ctypes

import numpy as np
import pytest
import torch

import flashoverlap_amd
from flashoverlap_amd import capi, config, layers, tiling, tuner
from oracle import fo_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ready(dev):
    flashoverlap_amd.load()
    capi.check(capi.lib().fo_set_wait_timeout_ms(5000))
    return dev


def _no_timeouts(*objects):
    """No wait expired: neither in the words the given OverlapImpl objects own nor in the per-device one."""
    n = ctypes.c_int()
    capi.check(capi.lib().fo_wait_timeouts(ctypes.byref(n), 1))
    return n.value == 0 and all(o.wait_timeouts(True) == 0 for o in objects)


def _config(M, N, algo, w, tmp_path):
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    path = config.config_path(M, N, 0, "mi355x", str(tmp_path))
    config.save_solution(path, BM, BN, 0.0, algo, tiling.raster_hint(M, N, algo), tiling.uniform_cseg(T, w))
    return config.load_config(path, M, N)


def test_allreduce_layers_like_correctness_ar(ready, tmp_path):
    dev = ready
    M, N, K = 1024, 2048, 512
    cfg = _config(M, N, 1, 24, tmp_path)
    torch.manual_seed(0)
    A = torch.empty((M, K), dtype=torch.float16, device=dev).normal_(0.0, 0.5)
    B = torch.empty((N, K), dtype=torch.float16, device=dev).normal_(0.0, 0.5)
    W = torch.empty((N,), dtype=torch.float16, device=dev).normal_(0.0, 0.5)
    norm = layers.RMSNorm(N, device=dev)
    norm.weight = torch.nn.Parameter(W)
    rnorm = layers.ReorderRMSNorm(N, M, cfg["BM"], cfg["BN"], cfg["hint"], device=dev)
    rnorm.weight = torch.nn.Parameter(W)
    lin = layers.RowParallelLayer(K, N, device=dev)
    lin.weight = torch.nn.Parameter(B)
    olin = layers.OverlapRowParallelLayer(0, 1, K, N, M, cfg, "all_reduce", device=dev)
    olin.weight = torch.nn.Parameter(B)
    with torch.no_grad():
        y1 = norm(lin(A))
        x2 = olin(A)
        y2 = rnorm(x2)
        # the layer's result belongs to the caller: a second forward must not overwrite it
        kept = x2.clone()
        x3 = olin(torch.zeros_like(A))
    torch.cuda.synchronize()
    assert x3.data_ptr() != x2.data_ptr() and torch.equal(x2, kept) and not x3.any()
    assert _no_timeouts(olin.overlap_class)
    assert torch.allclose(y1, y2, atol=1e-2, rtol=1e-2)                       # the reference's bar
    ref = O.rmsnorm(O.gemm(A.cpu(), B.cpu()), W.cpu(), 1e-5)
    assert O.rel_l2(y2.cpu(), ref) < 1e-3 and O.max_abs(y2.cpu(), ref) < 2e-2  # this build's bar


def test_reducescatter_layers_like_correctness_rs(ready, tmp_path):
    dev = ready
    M, N, K, ws, rank = 1024, 1024, 256, 4, 1
    cfg = _config(M, N, 1, 16, tmp_path)
    torch.manual_seed(1)
    A0 = torch.empty((M, K), dtype=torch.bfloat16, device=dev).normal_(0.0, 0.5)
    A1 = tiling.reorder_rows_by_world_size(A0, ws)
    B = torch.empty((N, K), dtype=torch.bfloat16, device=dev).normal_(0.0, 0.5)
    W = torch.empty((N,), dtype=torch.bfloat16, device=dev).normal_(0.0, 0.5)
    norm = layers.RMSNorm(N, dtype=torch.bfloat16, device=dev)
    norm.weight = torch.nn.Parameter(W)
    rnorm = layers.ReorderRMSNorm(N, M // ws, cfg["BM"] // ws, cfg["BN"], cfg["hint"], dtype=torch.bfloat16,
                                  device=dev)
    rnorm.weight = torch.nn.Parameter(W)
    lin = layers.RowParallelLayer(K, N, dtype=torch.bfloat16, device=dev)
    lin.weight = torch.nn.Parameter(B)
    olin = layers.OverlapRowParallelLayer(rank, ws, K, N, M, cfg, "reduce_scatter", dtype=torch.bfloat16, device=dev)
    olin.weight = torch.nn.Parameter(B)
    with torch.no_grad():
        x1 = lin(A1).view(ws, M // ws, N)[rank]       # what a one-rank reduce_scatter leaves with this rank
        y1 = norm(x1)
        y2 = rnorm(olin(A0))
    torch.cuda.synchronize()
    assert _no_timeouts(olin.overlap_class)
    assert torch.allclose(y1, y2, atol=5e-2, rtol=5e-2)                       # the reference's bar
    ref = O.rmsnorm(O.gemm(A0.cpu(), B.cpu())[rank::ws], W.cpu(), 1e-5)
    assert O.rel_l2(y2.cpu(), ref) < 2.5e-3


def test_monitor_sampling_and_vote_agree_with_the_raster(ready):
    """The sampled hint is a permutation whose waves are the waves of the known
    issue order: with 256-wide macro tiles and one workgroup per CU the first 256
    workgroups (1024 layout tiles) finish before any of the second round."""
    dev = ready
    M, N, K, algo = 8192, 4096, 256, 1
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    wave = 1024
    o = torch.classes.flashoverlap_class.OverlapImpl()
    o.mccl_init(0, 1, torch.ops.flashoverlap_op.generate_mccl_id())
    o.mutlass_init()
    o.overlap_init()
    samples = tuner.sample_completion_order(o, M, N, K, algo, BM, BN, wave, samples=6, warmup=2, device=dev)
    assert _no_timeouts(o)
    assert samples.shape == (6, T)
    for row in samples.tolist():
        assert sorted(row) == list(range(T))
    ok, hint = tuner.vote_hint(samples.numpy(), wave)
    assert ok and sorted(hint) == list(range(T))
    issued = tiling.raster_hint(M, N, algo)
    agree = len(set(hint[:wave]) & set(issued[:wave])) / wave
    print("first-wave agreement between sampled and analytic hint: %.3f" % agree, flush=True)
    assert agree > 0.9


@pytest.mark.parametrize("comm_op,ws,rank,dt", [("all_reduce", 1, 0, torch.float16), ("reduce_scatter", 8, 3, torch.bfloat16)])
def test_correctness_examples(ready, tmp_path, comm_op, ws, rank, dt):
    """The two example scripts of the reference as one command: its result lines, and True."""
    from flashoverlap_amd import correctness
    M, N, K = 2048, 1024, 512
    cfg = _config(M, N, 1, 32, tmp_path)
    said = []
    assert correctness.run(comm_op, M, N, K, cfg, ws, rank, dt, out=said.append)
    want = "[GEMM+AllReduce+RMSNorm] all close :  True" if comm_op == "all_reduce" else "[GEMM+ReduceScatter+RMSNorm] all close :  True"
    assert said[-1] == want
    if comm_op == "reduce_scatter":
        assert said[0].startswith("Index of max absolute difference") and len(said) == 5
    # a cSeg that does not add up to the tiles is refused: by the overlapped call, or already by the row map
    bad = dict(cfg, cSeg=cfg["cSeg"][:-1])
    with pytest.raises((RuntimeError, ValueError)):
        correctness.run(comm_op, M, N, K, bad, ws, rank, dt, out=lambda s: None)
    # the command line, on a shape without a tuning file
    assert correctness.main(["--m_dim", "1024", "--n_dim", "1024", "--k_dim", "256", "--comm_op", comm_op,
                             "--world_size", str(ws), "--rank", str(rank), "--dtype", str(dt).split(".")[1],
                             "--configs", str(tmp_path)]) == 0
