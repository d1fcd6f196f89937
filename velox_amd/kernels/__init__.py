"""The HIP kernels of the step.  ``load_ops`` builds (if need be) and loads them, or raises."""
from __future__ import annotations

from typing import Dict

import torch

from .build import BuildError, build_all, ensure_attention, ensure_core  # noqa: F401
from .hip_ops import HipOps, KernelError  # noqa: F401

_LOADED: Dict[str, HipOps] = {}


def load_ops(device="cuda") -> HipOps:
    device = torch.device(device)
    if device.type != "cuda":
        raise KernelError(f"the engine runs on a GPU only (got device {device}); there is no CPU path")
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible to this process; the engine has no CPU path")
    if device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    key = str(device)
    if key not in _LOADED:
        _LOADED[key] = HipOps(device)
    return _LOADED[key]
