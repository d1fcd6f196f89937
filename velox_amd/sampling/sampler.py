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


class Sampler:
    def __init__(self, ops, device, seed: Optional[int] = None) -> None:
        self.ops = ops
        self.device = torch.device(device)
        self._rng = random.Random(seed)
        self._seeds: Dict[str, int] = {}

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
        options = torch.from_numpy(packed).to(self.device)
        return self.ops.sample(logits, options)

    def _apply_penalties(self, logits, sampling_params, histories) -> torch.Tensor:
        rows = logits.shape[0]
        width = max(1, max(len(h) for h in histories))
        tokens = np.zeros((rows, width), dtype=np.int32)
        lengths = np.zeros(rows, dtype=np.int32)
        coeffs = np.zeros((rows, 3), dtype=np.float32)
        for r, (p, h) in enumerate(zip(sampling_params, histories)):
            tokens[r, : len(h)] = np.asarray(h, dtype=np.int32)
            lengths[r] = len(h)
            coeffs[r] = (p.repetition_penalty, p.presence_penalty, p.frequency_penalty)
        out = logits.clone()
        self.ops.apply_penalties(
            out,
            torch.from_numpy(tokens).to(self.device),
            torch.from_numpy(lengths).to(self.device),
            torch.from_numpy(coeffs).to(self.device),
        )
        return out
