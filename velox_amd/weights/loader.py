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
            lines.append("    (tensors the model has no place for are refused, so that a misnamed weight cannot go unnoticed; an export that "
                         "carries buffers of no use loads with ignore_unexpected_weights=True, which prints their number and goes on)")
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(wrong_shape))
        super().__init__("\n".join(lines))


def list_weight_files(model_dir: str) -> List[str]:
    """The folder's safetensors files: the shards its index names, else the single file (reference
    ``src/weight_loader.py:31-47``)."""
    indexed = os.path.join(model_dir, _INDEX_FILE)
    if os.path.isfile(indexed):
        with open(indexed, "r", encoding="utf-8") as handle:
            shards = set(json.load(handle)["weight_map"].values())
        return [os.path.join(model_dir, shard) for shard in sorted(shards)]
    whole = os.path.join(model_dir, _SINGLE_FILE)
    if not os.path.isfile(whole):
        raise FileNotFoundError(f"{model_dir} holds neither {_SINGLE_FILE} nor {_INDEX_FILE}")
    return [whole]


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


def named_tensors(model):
    """The binder's inverse: every tensor a bound model holds, under its checkpoint name (fused rows cut apart again,
    a shared tensor named once), in the dtype it is held in."""
    seen = set()
    for part, attr, param, names in expected_names(model.all_parts()):
        held = getattr(part, attr)
        row = 0
        for name, shape in zip(names, param.source_shapes):
            n = shape[0] if len(shape) > 0 else 1
            piece = held[row:row + n].reshape(shape)
            row += n
            if name not in seen and param.alias_of is None:
                seen.add(name)
                yield name, piece


class TensorSource:
    """Where a binder takes tensors from, by checkpoint name.  ``names()``: every name it holds; ``shape(name)``;
    ``tensor(name)``: the tensor, on any device, in the dtype it is stored in.  The binder asks for tensors in the order
    the model's parts declare them."""

    def names(self):
        raise NotImplementedError

    def __contains__(self, name: str) -> bool:
        return name in self.names()

    def shape(self, name: str) -> Tuple[int, ...]:
        raise NotImplementedError

    def tensor(self, name: str) -> torch.Tensor:
        raise NotImplementedError


@torch.no_grad()
def bind(model, source, run_dtype: torch.dtype, device, ignore_unexpected: bool = False) -> int:
    """Fills every declared tensor of ``model`` from ``source`` (files of a folder, or tensors drawn at random: anything
    with ``names``, ``shape`` and ``tensor``); returns the parameter count.  The one place where rows are concatenated,
    a tied tensor is shared and held dtypes are decided."""
    checkpoint = source
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
    if unexpected and ignore_unexpected and not missing and not wrong:
        # (as the reference does, src/weight_loader.py:131-136)
        print(f"[weights] ignoring {len(unexpected)} tensors the model has no place for: {', '.join(unexpected[:8])}{' ...' if len(unexpected) > 8 else ''}")
        unexpected = []
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
        del pieces
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


def bind_from_checkpoint(model, model_dir: str, run_dtype: torch.dtype, device, ignore_unexpected: bool = False) -> int:
    """``bind`` from the folder's safetensors files."""
    return bind(model, _Checkpoint(list_weight_files(model_dir)), run_dtype, device, ignore_unexpected=ignore_unexpected)
