"""CPU-side checks of the product's host logic: the Python tiling helpers
against the oracle, the C-ABI library's exported symbols against the header,
the workgroup rasterisation, and the torch binding's argument checking.  No
device work is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from flashoverlap_amd import capi, tiling
from oracle import fo_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI ----------------------------------------------------------------

def _declared_symbols(header="flashoverlap_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fo_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(fo_lib):
    names = _declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(fo_lib, n), f"{n} is declared in the header but not exported"
    assert sorted(capi.SIGNATURES) == names, "capi.SIGNATURES and the header disagree"


def test_probe_library_is_separate_from_the_product(fo_lib):
    """The measurement probes are a library of their own: declared in their own header, exported
    by libfo_bench.so, and neither declared nor exported by the product library."""
    names = _declared_symbols("flashoverlap_bench.h")
    assert names == sorted(capi.BENCH_SIGNATURES) and "fo_mfma_spin" in names
    bench = capi.bench_lib()
    for n in names:
        assert hasattr(bench, n), f"{n} is declared in flashoverlap_bench.h but not exported"
        assert n not in capi.SIGNATURES and not hasattr(fo_lib, n), f"{n} leaked into the product library"


def test_algo_table_matches_reference_instances(fo_lib):
    # src/inc/signal_instances.inc:1-6
    want = [(128, 128, 32), (128, 128, 64), (128, 256, 32), (128, 256, 64), (256, 128, 32), (256, 128, 64)]
    assert fo_lib.fo_algo_count() == len(want)
    assert [capi.algo_tile(i) for i in range(len(want))] == want
    with pytest.raises(capi.FoError):
        capi.algo_tile(6)
    with pytest.raises(capi.FoError):
        capi.algo_tile(-1)


def test_argument_errors_return_codes_not_exits(fo_lib):
    # shape / argument validation happens before any device call
    # the plain GEMM takes any M and N; the signalling modes only multiples of the layout tile
    rc = fo_lib.fo_gemm_signal(capi.FO_F16, 1, 100, 128, 64, 1, 16, 1, None, 16, 16, 16, 16, 16, 0, None)
    assert rc == capi.FO_ERR_SHAPE and b"multiples" in fo_lib.fo_last_error()
    assert fo_lib.fo_gemm(capi.FO_F16, 1, 0, 128, 64, 16, 16, 16, None) == capi.FO_ERR_SHAPE
    assert fo_lib.fo_gemm(capi.FO_F16, 1, 128, 128, 36, 16, 16, 16, None) == capi.FO_ERR_SHAPE
    assert fo_lib.fo_gemm(7, 1, 128, 128, 64, 16, 16, 16, None) == capi.FO_ERR_ARG
    assert fo_lib.fo_gemm(capi.FO_F16, 9, 128, 128, 64, 16, 16, 16, None) == capi.FO_ERR_ARG
    assert fo_lib.fo_gemm(capi.FO_F16, 1, 128, 128, 64, None, 16, 16, None) == capi.FO_ERR_ARG
    assert fo_lib.fo_gemm(capi.FO_F16, 1, 128, 128, 64, 8, 16, 16, None) == capi.FO_ERR_ARG  # misaligned
    assert fo_lib.fo_gemm_signal(capi.FO_F16, 1, 128, 128, 64, 1, None, 1, None, 16, 16, 16, None, None, 0,
                                 None) == capi.FO_ERR_ARG
    assert fo_lib.fo_wait(1, None, None, None) == capi.FO_ERR_ARG
    assert fo_lib.fo_consume(16, 16, 3, None) == capi.FO_ERR_ARG
    assert fo_lib.fo_consume(None, None, 0, None) == capi.FO_OK  # empty copy is a no-op
    assert fo_lib.fo_reorder_rmsnorm(capi.FO_F16, 16, 16, 16, 8, 60, 4, 4, 1, 16, 1e-5, None) == capi.FO_ERR_SHAPE
    assert fo_lib.fo_reorder_rmsnorm(capi.FO_F16, 16, 16, 16, 8, 64, 4, 8, 1, None, 1e-5, None) == capi.FO_ERR_ARG
    assert fo_lib.fo_rmsnorm(capi.FO_F16, 16, 16, 16, 0, 64, 1e-5, None) == capi.FO_OK  # zero rows
    assert fo_lib.fo_rmsnorm(capi.FO_F16, 16, 16, 16, 4, 32764, 1e-5, None) == capi.FO_ERR_SHAPE   # dim % 8
    assert fo_lib.fo_set_wait_timeout_ms(0) == capi.FO_ERR_ARG
    assert fo_lib.fo_wait_consume(16, 2, 16, 16, 16, 100, 1, 0, 1, 0, None, 4, None, None) == capi.FO_ERR_SHAPE
    assert fo_lib.fo_wait_consume(16, 2, 16, 16, 16, 128, 2, 1, 2, 0, None, 4, None, None) == capi.FO_ERR_ARG


# ---- rasterisation ---------------------------------------------------------

@pytest.mark.parametrize("algo,M,N", [(1, 1024, 1024), (1, 4096, 4096), (0, 8192, 4096), (1, 16384, 8192),
                                      (1, 8192, 8192), (3, 1024, 2048), (5, 2048, 1024), (1, 384, 640),
                                      (1, 128, 128), (1, 2304, 256), (3, 1152, 256), (1, 4480, 4224), (5, 256, 8320)])
def test_raster_hint_is_a_permutation_grouped_by_workgroup(algo, M, N):
    BM, BN, _ = capi.algo_tile(algo)
    T = (M // BM) * (N // BN)
    hint = tiling.raster_hint(M, N, algo)
    assert sorted(hint) == list(range(T))
    # RA built from it maps the i-th issued tile to slot i
    ra = tiling.reorder_indices(T, hint)
    assert ra[torch.tensor(hint)].tolist() == list(range(T))


def test_raster_xcd_locality():
    # c3: 8192x4096 with 256x256 macro tiles = 32x16 workgroups.  Workgroup i
    # runs on XCD i % 8; the 32 workgroups of one XCD that run concurrently
    # (ids x, x+8, ..., x+248) must form a compact block so they share panels.
    hint = np.array(tiling.raster_hint(8192, 4096, 1)).reshape(512, 4)  # 4 layout tiles per workgroup
    TN = 4096 // 128
    first = hint[:, 0]
    gm, gn = (first // TN) // 2, (first % TN) // 2
    for x in range(8):
        ids = np.arange(x, 256, 8)
        rows, cols = np.unique(gm[ids]), np.unique(gn[ids])
        assert len(rows) * len(cols) == 32 and len(rows) <= 8


@pytest.mark.parametrize("M,N", [(8192, 4096), (16384, 8192), (8192, 8192), (4096, 4096)])
def test_raster_waves_finish_whole_rows(M, N):
    """A hardware wave is 256 workgroups; with N <= 8192 the workgroups of a wave cover whole
    bands of 8 macro-tile rows, all XCDs working on the same A rows at the same time."""
    hint = np.array(tiling.raster_hint(M, N, 1)).reshape(-1, 4)[:, 0]      # first layout tile of every workgroup
    TN = N // 128
    gm, gn = (hint // TN) // 2, (hint % TN) // 2
    GN = N // 256
    for w in range(len(hint) // 256):
        rows = np.unique(gm[256 * w:256 * (w + 1)])
        assert len(rows) * GN == 256 and rows.max() - rows.min() == len(rows) - 1
        for r in rows:
            assert sorted(gn[256 * w:256 * (w + 1)][gm[256 * w:256 * (w + 1)] == r]) == list(range(GN))


def test_raster_hint_rejects_bad_shapes():
    with pytest.raises(capi.FoError):
        tiling.raster_hint(1000, 1024, 1)
    with pytest.raises(capi.FoError):
        tiling.raster_hint(384, 384, 3)  # 128x256 tile needs multiples of 256


# ---- python tiling helpers vs oracle ----------------------------------------

def test_tiling_helpers_match_oracle():
    rng = np.random.default_rng(0)
    for S in (1, 8, 64, 1000):
        for n in (0, S // 2, S):
            hint = rng.permutation(S)[:n].tolist()
            assert tiling.reorder_indices(S, hint).tolist() == O.reorder_indices(S, hint).tolist()
    assert tiling.reorder_indices(8, [3, 1, 2]).dtype == torch.int32
    for T, w in ((64, 4), (10, 4), (8192, 2), (2048, 256)):
        assert tiling.uniform_cseg(T, w) == O.uniform_cseg(T, w)
    for n in range(1, 9):
        assert tiling.integer_partitions(n) == O.compositions(n)
    assert tiling.cseg_from_groups([1, 1, 2, 2, 4], 106, 1024) == O.cseg_from_composition([1, 1, 2, 2, 4], 106, 1024)
    for args in ((8, 4, 4, 4, [1, 1], 2), (8, 8, 4, 4, [3, 1], 4), (64, 32, 16, 8, [3, 5, 8], 8),
                 (12, 6, 6, 3, [1, 2, 1], 3)):
        assert tiling.generate_row_remap_array(*args).tolist() == O.row_remap(*args).tolist()
    x = torch.arange(24).reshape(12, 2)
    assert torch.equal(tiling.reorder_rows_by_world_size(x, 4), O.reorder_rows_by_world_size(x, 4))


def test_tiling_helpers_reject_bad_input():
    with pytest.raises(ValueError):
        tiling.reorder_indices(4, [0, 0])
    with pytest.raises(ValueError):
        tiling.reorder_indices(4, [4])
    with pytest.raises(ValueError):
        tiling.generate_row_remap_array(8, 4, 4, 4, [1], 2)
    with pytest.raises(ValueError):
        tiling.uniform_cseg(8, 0)


# ---- torch binding ----------------------------------------------------------

@pytest.fixture(scope="module")
def binding():
    import flashoverlap_amd
    flashoverlap_amd.load()
    return torch.classes.flashoverlap_class


def test_binding_registers_reference_api(binding):
    # src/pybind.cpp:114-150
    o, b = binding.OverlapImpl(), binding.BaselineImpl()
    for name in ("mutlass_init", "mutlass_gemm", "gemm_allreduce_overlap", "gemm_reducescatter_overlap", "mccl_init",
                 "gemm_allreduce", "gemm_reducescatter", "gemm_all2all", "overlap_init", "mccl_allreduce",
                 "mccl_reducescatter", "mccl_all2all", "seg_allreduce"):
        assert hasattr(o, name), name
    for name in ("mccl_init", "mublas_init", "gemm_allreduce", "gemm_reducescatter", "gemm_all2all", "mublas_gemm",
                 "mccl_allreduce", "mccl_reducescatter", "mccl_all2all"):
        assert hasattr(b, name), name
    ident = torch.ops.flashoverlap_op.generate_mccl_id()
    assert len(ident) == 16 and ident != torch.ops.flashoverlap_op.generate_mccl_id()
    assert hasattr(torch.ops.flashoverlap_op, "reorder_rmsnorm")


def test_binding_errors_are_python_exceptions(binding):
    o = binding.OverlapImpl()
    ident = torch.ops.flashoverlap_op.generate_mccl_id()
    o.mccl_init(0, 1, ident)
    with pytest.raises(RuntimeError, match="rank"):
        o.mccl_init(2, 2, ident)
    with pytest.raises(RuntimeError, match="16 entries"):
        o.mccl_init(0, 1, [1, 2, 3])
    z = torch.zeros(2, 2, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="mutlass_init"):
        o.mutlass_gemm(z, z, z, 1)
    with pytest.raises(RuntimeError, match="GPU"):
        torch.ops.flashoverlap_op.reorder_rmsnorm(z, z, z[0], 2, 2, 1, torch.zeros(1, 1, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="float16 or bfloat16"):
        torch.ops.flashoverlap_op.reorder_rmsnorm(z.float(), z, z[0], 2, 2, 1, torch.zeros(1, 1, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="0 \\(auto\\)"):
        o.set_consumer_mode(5)


def test_oracle_is_not_reachable_from_the_product():
    pkg = os.path.join(ROOT, "flashoverlap_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".h", ".hip")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src, f"{f} mentions the oracle"
