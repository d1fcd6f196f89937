"""Batched sampling with per-request options.

What the reference's sampler computes (``engine/sampler.py:131-232``): logits to float32;
repetition / presence / frequency penalties over the request's prompt and output tokens;
rows with temperature 0 take the argmax; other rows divide by ``max(T, 1e-5)``, keep the
``top_k`` largest and the shortest prefix of the sorted probabilities whose exclusive
cumulative sum stays below ``top_p``, renormalise, and draw with the exponential race
``argmax(p / e)``, ``e ~ Exp(1)`` clamped at 1e-10 (equal to a categorical draw).

Here all of that is one kernel call per step.  The noise comes from a counter-based
generator keyed by (the request's seed, how many tokens the request has produced), so a
seeded request draws the same tokens whatever else is in the batch and in whichever row it
sits; unseeded requests get a seed from the sampler's own generator when first seen.
"""
from __future__ import annotations

import random
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .params import SamplingParams


class _Upload:
    """Small int32 arrays from the host to the device without a wait: a ring of pinned buffers, each guarded by an event
    (a buffer is written again only when the copy that read it has run), copied with ``non_blocking``.  From pageable
    memory the same copy would make the host wait for everything queued on the stream before it."""

    def __init__(self, device: torch.device, ring: int = 4) -> None:
        self.device = device
        self.pinned = device.type == "cuda"
        self._host: List[Optional[torch.Tensor]] = [None] * ring
        self._device: List[Optional[torch.Tensor]] = [None] * ring
        self._events = [torch.cuda.Event() if self.pinned else None for _ in range(ring)]
        self._used = [False] * ring
        self._next = 0

    def send(self, values: np.ndarray) -> torch.Tensor:
        """``values``: int32, any shape -> a device tensor of that shape (valid until the ring comes round again)."""
        flat = np.ascontiguousarray(values, dtype=np.int32).reshape(-1)
        if not self.pinned:
            return torch.from_numpy(flat.copy()).to(self.device).view(values.shape)
        index = self._next
        self._next = (index + 1) % len(self._host)
        if self._used[index]:
            self._events[index].synchronize()
        if self._host[index] is None or self._host[index].numel() < flat.size:
            size = max(1024, 1 << int(flat.size - 1).bit_length())
            self._host[index] = torch.empty(size, dtype=torch.int32, pin_memory=True)
            self._device[index] = torch.empty(size, dtype=torch.int32, device=self.device)
        self._host[index].numpy()[:flat.size] = flat
        target = self._device[index][:flat.size]
        target.copy_(self._host[index][:flat.size], non_blocking=True)
        self._events[index].record()
        self._used[index] = True
        return target.view(values.shape)


class Sampler:
    def __init__(self, ops, device, seed: Optional[int] = None) -> None:
        self.ops = ops
        self.device = torch.device(device)
        self._rng = random.Random(seed)
        self._seeds: Dict[str, int] = {}
        self._upload = _Upload(self.device)

    def _seed_for(self, request_id: str, params: SamplingParams) -> int:
        seed = self._seeds.get(request_id)
        if seed is None:
            seed = params.seed if params.seed is not None else self._rng.getrandbits(62)
            self._seeds[request_id] = int(seed) & ((1 << 62) - 1)
            seed = self._seeds[request_id]
        return seed

    def release(self, request_id: str) -> None:
        self._seeds.pop(request_id, None)

    @torch.no_grad()
    def sample(
        self,
        logits: torch.Tensor,
        sampling_params: Sequence[SamplingParams],
        request_ids: Sequence[str],
        num_generated: Sequence[int],
        histories: Optional[Sequence[Sequence[int]]] = None,
    ) -> torch.Tensor:
        """``logits`` float32 [R, V] -> int32 tokens [R] on the device.

        ``num_generated[r]`` is how many tokens request ``r`` has produced before this one (the
        generator's counter); ``histories[r]`` is its prompt plus output, needed only by penalties.
        """
        rows, vocab = logits.shape
        if len(sampling_params) != rows:
            raise ValueError(f"got {len(sampling_params)} sampling params for a batch of {rows}")
        if logits.dtype != torch.float32:
            raise ValueError("the sampler takes float32 logits")

        if any(p.has_penalties for p in sampling_params):
            if histories is None:
                raise ValueError("penalties need the requests' token histories")
            logits = self._apply_penalties(logits, sampling_params, histories)

        if all(p.is_greedy for p in sampling_params):
            return self.ops.argmax(logits)

        packed = np.zeros((rows, 6), dtype=np.int32)
        as_float = packed.view(np.float32)
        for r, (p, rid, n) in enumerate(zip(sampling_params, request_ids, num_generated)):
            seed = self._seed_for(rid, p)
            as_float[r, 0] = p.temperature
            as_float[r, 1] = p.top_p
            packed[r, 2] = p.top_k if 0 < p.top_k < vocab else 0
            packed[r, 3] = seed & 0x7FFFFFFF
            packed[r, 4] = (seed >> 31) & 0x7FFFFFFF
            packed[r, 5] = int(n)
        with_filter = any((not p.is_greedy) and (0 < p.top_k < vocab or p.top_p < 1.0) for p in sampling_params)
        return self.ops.sample(logits, self._upload.send(packed), with_filter=with_filter)

    def _apply_penalties(self, logits, sampling_params, histories) -> torch.Tensor:
        """A penalised copy of ``logits``.  Histories, their lengths and the coefficients travel as one int32 array."""
        rows = logits.shape[0]
        width = max(1, max(len(h) for h in histories))
        packed = np.zeros(rows * (width + 4), dtype=np.int32)
        tokens = packed[: rows * width].reshape(rows, width)
        lengths = packed[rows * width: rows * (width + 1)]
        coeffs = packed[rows * (width + 1):].view(np.float32).reshape(rows, 3)
        for r, (p, h) in enumerate(zip(sampling_params, histories)):
            tokens[r, : len(h)] = np.asarray(h, dtype=np.int32)
            lengths[r] = len(h)
            coeffs[r] = (p.repetition_penalty, p.presence_penalty, p.frequency_penalty)
        sent = self._upload.send(packed)
        out = logits.clone()
        self.ops.apply_penalties(
            out,
            sent[: rows * width].view(rows, width),
            sent[rows * width: rows * (width + 1)],
            sent[rows * (width + 1):].view(torch.float32).view(rows, 3),
        )
        return out
