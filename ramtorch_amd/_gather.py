"""Loader of the optional descriptor gatherer (``csrc/host_gather.cpp``).

``AdamW.step`` spends about 2 us of interpreter time per tensor collecting
addresses; for parameter sets with tens of thousands of tensors that is far more
than the update itself.  The gatherer does the same walk in C++.  It is a
convenience: when it has not been built, or does not load against the installed
torch, ``module()`` returns None and the Python loop does the work.
"""
from __future__ import annotations

import importlib.util
import os
import warnings

_mod = None
_tried = False


def module():
    global _mod, _tried
    if _tried:
        return _mod
    _tried = True
    if os.environ.get("RAMTORCH_AMD_NO_GATHER"):
        return None
    from . import build
    path = build.gather_path()
    if not os.path.exists(path):
        return None
    try:
        import torch
        spec = importlib.util.spec_from_file_location("_rt_gather", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        from . import functional as F
        if mod.DESC_SIZE != F.DESC_DTYPE.itemsize:
            raise ImportError("descriptor layout mismatch")
        mod.set_types(torch.Tensor, torch.nn.Parameter)
        _mod = mod
    except Exception as e:  # built against another torch, missing symbols ...
        warnings.warn(f"ramtorch_amd: descriptor gatherer not usable ({e}); using the Python loop")
        _mod = None
    return _mod
