"""MI355X-native implementation of FlashOverlap's single-GPU hot path.

`load()` registers torch.classes.flashoverlap_class.{OverlapImpl,BaselineImpl}
and torch.ops.flashoverlap_op.* from the in-tree libst_pybinding.so, which is
what a caller of the reference does with torch.ops.load_library.  The device
code lives in libfo_hip.so (C ABI in include/flashoverlap_hip.h; ctypes view
in flashoverlap_amd.capi).  There is no CPU fallback anywhere in this package.
"""
from __future__ import annotations

import os

_HERE = os.path.dirname(os.path.abspath(__file__))
BINDING_PATH = os.path.join(_HERE, "lib", "libst_pybinding.so")
_loaded = False


def load() -> str:
    """Load libst_pybinding.so into torch (idempotent); returns its path."""
    global _loaded
    if not _loaded:
        if not os.path.exists(BINDING_PATH):
            raise FileNotFoundError(
                f"{BINDING_PATH} is missing: build it with `python -m flashoverlap_amd.build`")
        import torch
        from . import capi
        capi.lib()  # libfo_hip.so first, so the binding resolves against the in-tree copy
        torch.ops.load_library(BINDING_PATH)
        _loaded = True
    return BINDING_PATH
