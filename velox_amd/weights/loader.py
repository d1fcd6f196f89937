"""Binding safetensors tensors to a model's parts by name.

The table of what goes where is not in this file: every part declares its tensors
(:class:`~velox_amd.parts.base.Param`), and this module only walks that table.  The
reference does the same job in ``src/weight_loader.py``: shard listing ``:31-55``,
q/k/v and gate/up fusion by concatenating rows ``:91-98``, tied head ``:100-104``, strict
shapes ``:123-126``.  Differences: tensors are read one at a time straight into device
memory (no whole-checkpoint copy on the host), and every problem (missing tensors,
unexpected tensors, wrong shapes) is collected and raised as ONE ``WeightsError``.

Dtypes: a ``matrix`` is held in the run dtype whatever the checkpoint stores (bfloat16 is
widened exactly in a float32 run; float32 is rounded once, to nearest even, in a bfloat16
run, as the reference's ``param.copy_(src.to(device, dtype))`` does, ``src/weight_loader.py:127``);
``vector`` tensors (norm weights, biases) are always held in float32; a part that needs a
tensor exactly as stored declares it with role ``stored`` (32-bit stays 32-bit); integer
tensors become int32.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Tuple

import torch
from safetensors import safe_open

from ..parts.base import Param, Part

_SINGLE_FILE = "model.safetensors"
_INDEX_FILE = "model.safetensors.index.json"


class WeightsError(RuntimeError):
    """Raised once per load, listing every missing, unexpected and mis-shaped tensor."""

    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[str]) -> None:
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = ["checkpoint does not match the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        super().__init__("\n".join(lines))


def list_weight_files(model_dir: str) -> List[str]:
    index_path = os.path.join(model_dir, _INDEX_FILE)
    if os.path.exists(index_path):
        with open(index_path, "r", encoding="utf-8") as handle:
            index = json.load(handle)
        names = sorted(set(index["weight_map"].values()))
        return [os.path.join(model_dir, name) for name in names]
    single_path = os.path.join(model_dir, _SINGLE_FILE)
    if os.path.exists(single_path):
        return [single_path]
    raise FileNotFoundError(f"no safetensors weights found in {model_dir}")


class _Checkpoint:
    """Lazy view of one or more safetensors files: names, shapes, and tensors on demand."""

    def __init__(self, files: List[str]) -> None:
        self._handles = [safe_open(path, framework="pt", device="cpu") for path in files]
        self._where: Dict[str, int] = {}
        for index, handle in enumerate(self._handles):
            for name in handle.keys():
                self._where[name] = index
        if not self._where:
            raise RuntimeError(f"checkpoint {files} contained no tensors")

    def names(self):
        return self._where.keys()

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self._handles[self._where[name]].get_slice(name).get_shape())

    def tensor(self, name: str) -> torch.Tensor:
        return self._handles[self._where[name]].get_tensor(name)


def held_dtype(role: str, stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    """The dtype a tensor is kept in, from its role, its stored dtype and the run dtype.  A ``matrix`` takes the run
    dtype whatever it is stored in (reference ``src/weight_loader.py:127`` converts while it copies); a ``vector`` is
    float32; a ``stored`` tensor that the checkpoint holds in 32-bit (or wider) stays float32 and otherwise takes the
    run dtype; integers become int32."""
    if not stored.is_floating_point:
        return torch.int32
    if role == "vector":
        return torch.float32
    if role == "stored" and stored in (torch.float32, torch.float64):
        return torch.float32
    return run_dtype


def expected_names(parts: List[Part]) -> List[Tuple[Part, str, Param, List[str]]]:
    rows = []
    for part in parts:
        for attr, param in part.params().items():
            rows.append((part, attr, param, [part.prefix + source for source in param.sources]))
    return rows


@torch.no_grad()
def bind_from_checkpoint(model, model_dir: str, run_dtype: torch.dtype, device) -> int:
    """Fills every declared tensor of ``model`` from the folder's safetensors; returns the parameter count."""
    checkpoint = _Checkpoint(list_weight_files(model_dir))
    device = torch.device(device)
    rows = expected_names(model.all_parts())

    missing: List[str] = []
    wrong: List[str] = []
    used = set()
    plan = []
    for part, attr, param, names in rows:
        absent = [name for name in names if name not in checkpoint]
        if absent:
            if param.alias_of is not None and len(absent) == len(names):
                plan.append((part, attr, param, None))
                continue
            missing.extend(absent)
            used.update(name for name in names if name in checkpoint)
            continue
        ok = True
        for name, want in zip(names, param.source_shapes):
            used.add(name)
            got = checkpoint.shape(name)
            if tuple(got) != tuple(want):
                wrong.append(f"{name}: checkpoint {tuple(got)} vs model {tuple(want)}")
                ok = False
        if ok:
            plan.append((part, attr, param, names))
    unexpected = sorted(name for name in checkpoint.names() if name not in used)
    # a tied checkpoint that also stores its head is tolerated: the tied table is used
    aliased = {part.prefix + s for part, _, param, names in plan if names is None for s in param.sources}
    tolerated = {n for n in unexpected if n in aliased}
    unexpected = [n for n in unexpected if n not in tolerated]
    if missing or unexpected or wrong:
        raise WeightsError(sorted(missing), unexpected, wrong)

    bound: Dict[str, torch.Tensor] = {}
    count = 0
    deferred = []
    for part, attr, param, names in plan:
        if names is None:
            deferred.append((part, attr, param))
            continue
        pieces = [checkpoint.tensor(name) for name in names]
        stored = pieces[0].dtype
        for piece in pieces[1:]:
            stored = torch.promote_types(stored, piece.dtype)
        dtype = held_dtype(param.role, stored, run_dtype)
        target = torch.empty(param.shape, dtype=dtype, device=device)
        row = 0
        for piece in pieces:
            n = piece.shape[0] if piece.dim() > 0 else 1
            target[row:row + n].copy_(piece.to(dtype))
            row += n
        setattr(part, attr, target)
        if len(names) == 1:
            bound[names[0]] = target
        count += target.numel()
    for part, attr, param in deferred:
        if param.alias_of not in bound:
            raise WeightsError([param.alias_of], [], [])
        setattr(part, attr, bound[param.alias_of])
    for part in model.all_parts():
        part.finalize(device, run_dtype)
    return count
