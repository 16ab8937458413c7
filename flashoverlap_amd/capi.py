"""ctypes view of libfo_hip.so's C ABI (include/flashoverlap_hip.h).

Used by the tests, the bench harness and the host-side tiling helpers.  There is
no fallback: if the library has not been built, loading raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfo_hip.so")

FO_F16, FO_BF16 = 0, 1
FO_OK, FO_ERR_ARG, FO_ERR_SHAPE, FO_ERR_HIP, FO_ERR_TIMEOUT, FO_ERR_LIMIT = range(6)
FO_COPY_AUTO, FO_COPY_STREAM, FO_COPY_CACHED = range(3)   # store policy of fo_consume_slices

_vp, _ip, _i, _ll, _sz, _f = C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_longlong, C.c_size_t, C.c_float

# name -> (restype, argtypes); one entry per declaration in the header.
SIGNATURES = {
    "fo_version": (_i, []),
    "fo_last_error": (C.c_char_p, []),
    "fo_algo_count": (_i, []),
    "fo_algo_tile": (_i, [_i, _ip, _ip, _ip]),
    "fo_device_info": (_i, [_ip, _ip, _ip]),
    "fo_gemm": (_i, [_i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "fo_gemm_signal": (_i, [_i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "fo_gemm_scatter": (_i, [_i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "fo_gemm_signal_static": (_i, [_i, _i, _i, _i, _i, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "fo_build_group_table": (_i, [_vp, _i, _i, _vp, _vp]),
    "fo_raster_hint": (_i, [_i, _i, _i, _ip]),
    "fo_tune": (_i, [C.c_char_p, _i]),
    "fo_wait": (_i, [_i, _vp, _vp, _vp]),
    "fo_wait_consume": (_i, [_vp, _i, _vp, _vp, _vp, _ll, _i, _i, _i, _ll, _vp, _i, _vp, _vp]),
    "fo_set_wait_timeout_ms": (_i, [_i]),
    "fo_wait_timeouts": (_i, [_ip, _i]),
    "fo_consume": (_i, [_vp, _vp, _sz, _vp]),
    "fo_settle_consume": (_i, [_i, _vp, _vp, _vp, _sz, _vp, _vp]),
    "fo_consume_slices": (_i, [_i, _vp, _vp, _vp, _sz, _i, _sz, _i, _vp, _vp]),
    "fo_reorder_rmsnorm": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _f, _vp]),
    "fo_reorder_rmsnorm_batched": (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _f, _vp]),
    "fo_rmsnorm": (_i, [_i, _vp, _vp, _vp, _i, _i, _f, _vp]),
    "fo_stream_create": (_i, [C.POINTER(_vp)]),
    "fo_stream_destroy": (_i, [_vp]),
    "fo_stream_sync": (_i, [_vp]),
    "fo_stream_join": (_i, [_vp, _vp]),
    "fo_stream_is_capturing": (_i, [_vp, C.POINTER(C.c_int)]),
    "fo_time_next_launch": (_i, [_vp, _vp]),
    "fo_event_create": (_i, [C.POINTER(_vp)]),
    "fo_event_destroy": (_i, [_vp]),
    "fo_event_record": (_i, [_vp, _vp]),
    "fo_event_sync": (_i, [_vp]),
    "fo_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(_f)]),
}

# libfo_bench.so (include/flashoverlap_bench.h): measurement probes, loaded by bench.py and its test only.
BENCH_LIB_PATH = os.path.join(_HERE, "lib", "libfo_bench.so")
BENCH_SIGNATURES = {
    "fo_bench_last_error": (C.c_char_p, []),
    "fo_mfma_spin": (_i, [_i, _i, _i, _vp, _sz, _i, _vp, C.POINTER(_ll), _vp]),
}

_lib = None
_bench_lib = None


class FoError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"libfo_hip error {code}: {msg}")
        self.code = code


def lib() -> C.CDLL:
    """The loaded library with argtypes set; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m flashoverlap_amd.build` (there is no CPU fallback)")
        try:  # share the HIP runtime that torch already loaded, when torch is in the process
            import torch  # noqa: F401
        except Exception:
            pass
        handle = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
        # FO_TUNE="knob=value,knob=value" applies fo_tune settings at load time
        for item in filter(None, os.environ.get("FO_TUNE", "").split(",")):
            key, _, value = item.partition("=")
            check(handle.fo_tune(key.strip().encode(), int(value)))
    return _lib


def bench_lib() -> C.CDLL:
    """The measurement-probe library with argtypes set; raises if it is not built."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise FileNotFoundError(f"{BENCH_LIB_PATH} is missing: build it with `python -m flashoverlap_amd.build`")
        try:
            import torch  # noqa: F401
        except Exception:
            pass
        handle = C.CDLL(BENCH_LIB_PATH, mode=C.RTLD_LOCAL)
        for name, (res, args) in BENCH_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _bench_lib = handle
    return _bench_lib


def bench_check(code: int) -> None:
    if code != FO_OK:
        raise FoError(code, bench_lib().fo_bench_last_error().decode())


def check(code: int) -> None:
    if code != FO_OK:
        raise FoError(code, lib().fo_last_error().decode())


def algo_tile(algo: int):
    bm, bn, bk = C.c_int(), C.c_int(), C.c_int()
    check(lib().fo_algo_tile(algo, C.byref(bm), C.byref(bn), C.byref(bk)))
    return bm.value, bn.value, bk.value


def raster_hint(algo: int, M: int, N: int) -> list:
    bm, bn, _ = algo_tile(algo)
    if M <= 0 or N <= 0 or M % bm or N % bn:
        raise FoError(FO_ERR_SHAPE, f"M={M} N={N} not multiples of the {bm}x{bn} tile")
    T = (M // bm) * (N // bn)
    buf = (C.c_int * T)()
    check(lib().fo_raster_hint(algo, M, N, buf))
    return list(buf)


def dtype_code(torch_dtype) -> int:
    import torch
    if torch_dtype == torch.float16:
        return FO_F16
    if torch_dtype == torch.bfloat16:
        return FO_BF16
    raise TypeError(f"unsupported dtype {torch_dtype}: the path computes in fp16 or bf16")


def ptr(t) -> int:
    """Device (or host) address of a torch tensor, 0 for None."""
    return 0 if t is None else t.data_ptr()
