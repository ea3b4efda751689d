"""Loader for tests/golden/cc1d_golden.npz (written by tests/golden/make_golden.py)."""
import os

import numpy as np
import torch

_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cc1d_golden.npz")
_cache = {}


def load_case(case: str) -> dict:
    """All tensors of one fixture case, e.g. load_case("fwd_c1")["x"]."""
    if "npz" not in _cache:
        _cache["npz"] = np.load(_PATH, allow_pickle=False)
    npz = _cache["npz"]
    out = {}
    for key in npz.files:
        if not key.startswith(case + "/") or key.endswith("__dtype"):
            continue
        name = key[len(case) + 1:]
        arr = npz[key]
        if key + "__dtype" in npz.files:
            dt = getattr(torch, str(npz[key + "__dtype"]))
            out[name] = torch.from_numpy(arr.view(np.int16).copy()).view(dt)
        else:
            out[name] = torch.from_numpy(arr.copy())
    return out
