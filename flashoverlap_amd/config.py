"""Per-shape tuning files in the reference's format.

The reference keeps one JSON per problem, `configs/m{M}n{N}k{K}_{gpu}.json`:
the GEMM profiler writes lists `BM`, `BN`, `dur`, `Algo` (best first,
tune/profile_config.py:59-74); the search replaces them by the chosen scalars
and adds `hint`, `cSeg`, `rLDN` (tune/search.py:83-101); the speed test and the
examples read those (test/test.py:347-367, example/correctness_ar.py:90-97).
Files written here can be read by the reference's scripts and vice versa.
"""
from __future__ import annotations

import json
import os

REQUIRED_AFTER_SEARCH = ("BM", "BN", "dur", "Algo", "hint", "cSeg", "rLDN")


def gpu_tag(device_name: str, arch: str = "") -> str:
    """The reference cuts characters 7..10 out of the device name
    (tune/search.py:72).  Here a product name that is recognised gives its tag;
    a driver that reports only a generic name ("AMD Radeon Graphics") gives the
    architecture instead ("gfx950" out of "gfx950:sramecc+:xnack-")."""
    name = device_name.lower()
    for tag in ("mi355x", "mi350x", "mi325x", "mi300x"):
        if tag in name:
            return tag
    if arch:
        return arch.split(":")[0].lower()
    return name.replace(" ", "")[-6:] or "gpu"


def current_gpu_tag(device: int = 0) -> str:
    """gpu_tag of a visible device."""
    import torch
    props = torch.cuda.get_device_properties(device)
    return gpu_tag(props.name, getattr(props, "gcnArchName", ""))


def current_gpu_tags(device: int = 0) -> list:
    """Tags under which a tuning file of the visible device may have been saved: the product tag
    if the driver reports one, then the architecture (the same silicon reports either, depending
    on the driver)."""
    import torch
    props = torch.cuda.get_device_properties(device)
    arch = getattr(props, "gcnArchName", "").split(":")[0].lower()
    tags = [gpu_tag(props.name, arch)]
    if arch and arch not in tags:
        tags.append(arch)
    return tags


def find_config(M: int, N: int, K: int, tags, root: str = "configs") -> str:
    """Path of the first existing tuning file among the tags, else the path under the first tag."""
    for tag in tags:
        path = config_path(M, N, K, tag, root)
        if os.path.exists(path):
            return path
    return config_path(M, N, K, tags[0], root)


def config_path(M: int, N: int, K: int, gpu: str, root: str = "configs") -> str:
    return os.path.join(root, f"m{M}n{N}k{K}_{gpu}.json")


def save_profile(path: str, BM, BN, dur, Algo) -> None:
    """Top candidates of a GEMM sweep, best first (lists of equal length)."""
    if not (len(BM) == len(BN) == len(dur) == len(Algo)):
        raise ValueError("BM, BN, dur and Algo must have the same length")
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    with open(path, "w", encoding="utf-8") as f:
        json.dump({"BM": list(BM), "BN": list(BN), "dur": list(dur), "Algo": list(Algo)}, f, indent=4)


def save_solution(path: str, BM: int, BN: int, gemm_dur: float, Algo: int, hint, cSeg, rLDN: int = 1) -> None:
    """Adds the search result to an existing file (or creates it)."""
    data = {}
    if os.path.exists(path):
        with open(path, "r", encoding="utf-8") as f:
            data = json.load(f)
    data.update({"hint": [int(h) for h in hint], "cSeg": [int(c) for c in cSeg], "rLDN": int(rLDN),
                 "BM": int(BM), "BN": int(BN), "dur": float(gemm_dur), "Algo": int(Algo)})
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    with open(path, "w", encoding="utf-8") as f:
        json.dump(data, f, indent=4)


def load_config(path: str, M: int | None = None, N: int | None = None) -> dict:
    """Reads a searched configuration and checks that it is usable: scalar
    BM/BN/Algo, cSeg summing to the tile count, hint without repeats."""
    with open(path, "r", encoding="utf-8") as f:
        data = json.load(f)
    missing = [k for k in REQUIRED_AFTER_SEARCH if k not in data]
    if missing:
        raise ValueError(f"{path}: no search result yet (missing {missing})")
    if isinstance(data["BM"], list):
        raise ValueError(f"{path}: BM/BN/Algo are still candidate lists; run the search first")
    if M is not None and N is not None:
        tiles = (M // data["BM"]) * (N // data["BN"])
        if sum(data["cSeg"]) != tiles:
            raise ValueError(f"{path}: sum(cSeg) = {sum(data['cSeg'])} but the output has {tiles} tiles")
        if len(set(data["hint"])) != len(data["hint"]) or any(h < 0 or h >= tiles for h in data["hint"]):
            raise ValueError(f"{path}: hint must name distinct tiles below {tiles}")
    return data
