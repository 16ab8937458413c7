"""Host-side tiling helpers with the names and meaning of the reference's Python
helpers (test/test.py:69-118 = example/utils.py:3-65, tune/search.py:137-144,
462-471, 502-513), returning torch tensors on the caller's device.

The reference builds these per script; here they are one module.  Differences:
reorder_indices is O(S) instead of O(S*len(hint)); `device` must be passed
explicitly (the reference hard-codes its own accelerator).
"""
from __future__ import annotations

import numpy as np
import torch

from . import capi


def div_up(x: int, y: int) -> int:
    return (x + y - 1) // y


def reorder_indices(S: int, hint, device="cpu") -> torch.Tensor:
    """RA with RA[hint[i]] = i; tiles not in hint follow in ascending order
    (test/test.py:72-88).  int32, shape [S]."""
    hint = np.asarray(list(hint), dtype=np.int64)
    if hint.size and (hint.min() < 0 or hint.max() >= S):
        raise ValueError("hint entries must be tile ids in [0, S)")
    if np.unique(hint).size != hint.size:
        raise ValueError("hint must not repeat a tile")
    new_order = np.full(S, -1, dtype=np.int64)
    new_order[hint] = np.arange(hint.size)
    rest = np.flatnonzero(new_order < 0)
    new_order[rest] = hint.size + np.arange(rest.size)
    return torch.from_numpy(new_order.astype(np.int32)).to(device)


def generate_row_remap_array(M: int, N: int, BM: int, BN: int, S_list, world_size: int, device="cpu") -> torch.Tensor:
    """RE: rows of every group chunk stably sorted by row % world_size;
    RE[orig] = new (test/test.py:90-118).  int32, shape [M*N/BN]."""
    total_tiles = (M * N) // (BM * BN)
    if sum(S_list) != total_tiles:
        raise ValueError("sum(S_list) must equal total number of tiles")
    rows = np.arange(M * N // BN, dtype=np.int64)
    new_of = np.empty_like(rows)
    cur = 0
    for S in S_list:
        n = S * BM
        chunk = rows[cur:cur + n]
        order = np.argsort(chunk % world_size, kind="stable")
        new_of[chunk[order]] = cur + np.arange(n)
        cur += n
    return torch.from_numpy(new_of.astype(np.int32)).to(device)


generate_row_mapping = generate_row_remap_array  # name used in example/utils.py:24


def reorder_rows_by_world_size(tensor: torch.Tensor, world_size: int) -> torch.Tensor:
    """Rows stably sorted by row % world_size (example/utils.py:54-65)."""
    M = tensor.shape[0]
    mod = torch.arange(M, device=tensor.device) % world_size
    return tensor[torch.argsort(mod, stable=True)]


def uniform_cseg(tile_num: int, wave_size: int) -> list:
    """cSeg of ceil(T/w) groups of w tiles, the last one short
    (tune/search.py:137-144)."""
    if wave_size <= 0:
        raise ValueError("wave_size must be positive")
    return [min(wave_size, tile_num - i * wave_size) for i in range(div_up(tile_num, wave_size))]


def integer_partitions(n: int) -> list:
    """Ordered compositions of n, in the reference's enumeration order
    (tune/search.py:462-471)."""
    result = []
    stack = [(n, [])]
    # depth-first, smallest first part first, like the recursive original
    while stack:
        remaining, path = stack.pop()
        if remaining == 0:
            result.append(path)
            continue
        for i in range(remaining, 0, -1):
            stack.append((remaining - i, path + [i]))
    return result


def cseg_from_groups(gp, wave_size: int, tile_num: int) -> list:
    """Wave counts per group -> tile counts per group, last group clipped
    (tune/search.py:502-513)."""
    out, acc = [], 0
    for j, g in enumerate(gp):
        if j < len(gp) - 1:
            out.append(g * wave_size)
            acc += g * wave_size
        else:
            out.append(min(g * wave_size, tile_num - acc))
    return out


def raster_hint(M: int, N: int, algo: int) -> list:
    """Issue order of layout tiles in this library's GEMM kernels for the
    given shape and Algo; takes the place of the sampled `hint` of
    tune/search.py:164-263."""
    return capi.raster_hint(algo, M, N)
