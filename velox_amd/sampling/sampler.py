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

    def __init__(self, device: torch.device, ring: int = 16) -> None:
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


class _SeenCounts:
    """How often each request with penalties has seen each token (prompt and output): an int32 table on the device, one row
    per such request.  A row is built once from the request's tokens and then kept up to date from the sampler's output on
    the device, so a step's penalties need neither the request's history on the host nor the value of a token that is
    still being sampled."""

    def __init__(self, ops, device: torch.device, upload: _Upload) -> None:
        self.ops = ops
        self.device = device
        self.upload = upload
        self.table: Optional[torch.Tensor] = None
        self.row_of_request: Dict[str, int] = {}
        self.free_rows: List[int] = []

    def row_for(self, request_id: str, vocab: int, history) -> int:
        """The request's row, built from ``history()`` (its tokens so far) when the request is new here."""
        row = self.row_of_request.get(request_id)
        if row is not None:
            return row
        tokens = np.asarray(history(), dtype=np.int32)
        if tokens.size and int(tokens.min()) < 0:
            raise ValueError(f"request {request_id}: its history holds a token that is still being sampled")
        if self.table is None or self.table.shape[1] != vocab:
            self.table = torch.zeros((8, vocab), dtype=torch.int32, device=self.device)
            self.row_of_request.clear()
            self.free_rows = list(range(7, -1, -1))
        if not self.free_rows:
            rows = self.table.shape[0]
            self.table = torch.cat([self.table, torch.zeros_like(self.table)])
            self.free_rows = list(range(2 * rows - 1, rows - 1, -1))
        row = self.free_rows.pop()
        self.row_of_request[request_id] = row
        self.table[row].zero_()
        if tokens.size:
            self.ops.count_tokens(self.table[row], self.upload.send(tokens))
        return row

    def release(self, request_id: str) -> None:
        row = self.row_of_request.pop(request_id, None)
        if row is not None:
            self.free_rows.append(row)


class Sampler:
    def __init__(self, ops, device, seed: Optional[int] = None) -> None:
        self.ops = ops
        self.device = torch.device(device)
        self._rng = random.Random(seed)
        self._seeds: Dict[str, int] = {}
        self._upload = _Upload(self.device)
        self._seen = _SeenCounts(ops, self.device, self._upload)

    def _seed_for(self, request_id: str, params: SamplingParams) -> int:
        seed = self._seeds.get(request_id)
        if seed is None:
            seed = params.seed if params.seed is not None else self._rng.getrandbits(62)
            self._seeds[request_id] = int(seed) & ((1 << 62) - 1)
            seed = self._seeds[request_id]
        return seed

    def release(self, request_id: str) -> None:
        self._seeds.pop(request_id, None)
        self._seen.release(request_id)

    @torch.no_grad()
    def sample(
        self,
        logits: torch.Tensor,
        sampling_params: Sequence[SamplingParams],
        request_ids: Sequence[str],
        num_generated: Sequence[int],
        histories: Optional[Sequence] = None,
    ) -> torch.Tensor:
        """``logits`` float32 [R, V] -> int32 tokens [R] on the device.

        ``num_generated[r]`` is how many tokens request ``r`` has produced before this one (the
        generator's counter).  ``histories[r]``, needed only by penalties and only the first time a
        request is seen (or the first time after ``release``): its prompt plus output so far, as a
        list or as a function that returns one.  From then on the sampler counts the request's
        tokens itself, from its own output."""
        rows, vocab = logits.shape
        if len(sampling_params) != rows or len(request_ids) != rows:
            raise ValueError(f"got {len(sampling_params)} sampling params and {len(request_ids)} ids for a batch of {rows}")
        if logits.dtype != torch.float32:
            raise ValueError("the sampler takes float32 logits")

        row_of = None
        if any(p.has_penalties for p in sampling_params):
            logits, row_of = self._apply_penalties(logits, sampling_params, request_ids, histories)

        if all(p.is_greedy for p in sampling_params):
            tokens = self.ops.argmax(logits)
        else:
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
            tokens = self.ops.sample(logits, self._upload.send(packed), with_filter=with_filter)
        if row_of is not None:
            self.ops.count_sampled(self._seen.table, row_of, tokens)  # the new tokens are seen from the next step on
        return tokens

    def _apply_penalties(self, logits, sampling_params, request_ids, histories):
        """A penalised copy of ``logits`` and the rows' places in the table of counts (-1: no penalties)."""
        rows, vocab = logits.shape
        packed = np.zeros(rows * 4, dtype=np.int32)
        row_of = packed[:rows]
        coeffs = packed[rows:].view(np.float32).reshape(rows, 3)
        for r, (p, rid) in enumerate(zip(sampling_params, request_ids)):
            coeffs[r] = (p.repetition_penalty, p.presence_penalty, p.frequency_penalty)
            if not p.has_penalties:
                row_of[r] = -1
                continue
            if rid not in self._seen.row_of_request and (histories is None or histories[r] is None):
                raise ValueError(f"penalties need the token history of request {rid} the first time it is sampled")
            history = histories[r] if histories is not None else None
            row_of[r] = self._seen.row_for(rid, vocab, history if callable(history) else (lambda h=history: h))
        sent = self._upload.send(packed)
        out = logits.clone()
        row_of_device = sent[:rows]
        self.ops.apply_penalties_from_counts(out, self._seen.table, row_of_device, sent[rows:].view(torch.float32).view(rows, 3))
        return out, row_of_device
