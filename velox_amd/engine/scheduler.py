"""Continuous batching with portions of prompts, decode priority and recompute preemption.

The decisions are the reference's (``engine/scheduler.py:161-291``):

0. requests that finished are dropped and their pages and slot given back;
1. decoding requests go first, in arrival order, one token each; when no page is free the
   NEWEST running request is preempted, again and again, until the token fits or the
   request itself was the victim (``:148-159,190-208``);
2. running prefills get ``min(outstanding, budget, max_prefill_chunk_size)`` tokens, cut down
   to what fits in their pages plus the free ones; only the oldest prefill may preempt
   newer requests to get room (``:221-255``);
3. waiting requests are admitted first come first served while budget and slots remain,
   keeping a watermark of pages free; the first that does not fit stops admission (``:257-291``).

Preemption frees every page, resets ``num_computed_tokens`` to zero and puts the request at the
FRONT of the waiting queue; its generated tokens stay, so the recomputation covers prompt
plus generated tokens and no token is sampled twice (``:136-146``).

What happens when pages run out is therefore: decode -> preempt the newest; prefill -> a
smaller portion, the oldest may evict; admission -> wait.  A request that could never fit
in the pool even alone is refused by ``add_request`` (the reference would spin on it).
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional

from ..cache.manager import CacheManager
from .request import FinishReason, Request, RequestStatus


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 32
    max_num_batched_tokens: int = 2048
    max_prefill_chunk_size: int = 512
    max_model_len: int = 4096
    watermark: float = 0.01


@dataclass
class SchedulerOutput:
    prefill_batch: List[Request] = field(default_factory=list)
    decode_batch: List[Request] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)
    num_batched_tokens: int = 0

    def is_empty(self) -> bool:
        return not self.prefill_batch and not self.decode_batch


class Scheduler:
    def __init__(self, cache: CacheManager, config: Optional[SchedulerConfig] = None, **overrides) -> None:
        self.config = config or SchedulerConfig(**overrides)
        self.cache = cache
        self.config.max_model_len = min(self.config.max_model_len, cache.max_model_len)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.requests: Dict[str, Request] = {}
        self._watermark_pages = max(1, int(cache.num_total_pages * self.config.watermark))
        self.num_preemptions = 0
        self.num_finished = 0

    # -- queue --------------------------------------------------------------------------
    def add_request(self, request: Request) -> None:
        limit = self.config.max_model_len
        if request.num_prompt_tokens >= limit:
            raise ValueError(
                f"prompt of {request.num_prompt_tokens} tokens does not fit in max_model_len={limit} "
                "(at least one token must remain for generation)"
            )
        if request.num_prompt_tokens + request.sampling_params.max_tokens > limit:
            raise ValueError(
                f"prompt of {request.num_prompt_tokens} tokens plus max_tokens={request.sampling_params.max_tokens} "
                f"exceeds max_model_len={limit}"
            )
        if request.request_id in self.requests:
            raise ValueError(f"request id {request.request_id!r} is already queued")
        self.requests[request.request_id] = request
        self.waiting.append(request)

    def abort_request(self, request_id: str) -> bool:
        request = self.requests.get(request_id)
        if request is None or request.finished:
            return False
        request.finish(FinishReason.ABORT)
        self._release(request)
        try:
            self.waiting.remove(request)
        except ValueError:
            pass
        if request in self.running:
            self.running.remove(request)
        self.requests.pop(request_id, None)
        return True

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    @property
    def num_waiting(self) -> int:
        return len(self.waiting)

    @property
    def num_running(self) -> int:
        return len(self.running)

    # -- cache bookkeeping --------------------------------------------------------------
    def _release(self, request: Request) -> None:
        if request.cache is not None:
            self.cache.free_sequence(request.cache)
            request.cache = None

    def _preempt(self, request: Request, output: Optional[SchedulerOutput] = None) -> None:
        if output is not None:
            # a victim may already have been given its token of this step (the reference leaves it in the
            # batch, engine/scheduler.py:241-247): it must not run without its pages
            if request in output.decode_batch:
                output.decode_batch.remove(request)
            if request in output.prefill_batch:
                output.prefill_batch.remove(request)
            output.preempted.append(request)
        self._release(request)
        request.num_computed_tokens = 0
        request.status = RequestStatus.PREEMPTED
        request.num_preemptions += 1
        self.num_preemptions += 1
        if request in self.running:
            self.running.remove(request)
        self.waiting.appendleft(request)

    def _make_room(self, request: Request, num_tokens: int, output: SchedulerOutput) -> bool:
        while not self.cache.can_append(request.cache, request.num_computed_tokens, num_tokens):
            if not self.running:
                return False
            victim = self.running[-1]  # always the newest, even when that is the caller
            self._preempt(victim, output)
            if victim is request:
                return False
        return True

    # -- one scheduling decision --------------------------------------------------------
    def schedule(self) -> SchedulerOutput:
        output = SchedulerOutput()
        self._reap_finished()
        budget = self.config.max_num_batched_tokens
        self._schedule_decodes(output, budget)
        budget -= len(output.decode_batch)
        budget = self._schedule_running_prefills(output, budget)
        self._admit(output, budget)
        output.num_batched_tokens = len(output.decode_batch) + sum(r.current_chunk_size for r in output.prefill_batch)
        return output

    def schedule_ahead(self, in_flight: List[Request]) -> Optional[List[Request]]:
        """The decode step after the one in flight, decided before that one's tokens are known (not in the reference,
        which waits for every step's tokens before it schedules the next).

        ``in_flight`` are the requests of a decode-only step that has been launched but whose tokens have not been
        appended yet: each will hold one token more than ``all_token_ids`` shows and one computed position more than
        ``num_computed_tokens``.  The next step can be fixed now only if nothing else could claim a place in it: no
        request waits, every running request is one of ``in_flight`` and keeps decoding whatever token it draws (its
        length limit is not reached by the token in flight), and every one finds its next page without preemption.
        Then the requests' tables are grown and the list comes back (order kept); otherwise None, and nothing has
        changed.  A request that stops on the token in flight has then been given a place it does not use: the caller
        drops its row, and its pages go back when it is reaped."""
        self._reap_finished()
        if self.waiting or not in_flight or len(self.running) != len(in_flight) or len(in_flight) > self.config.max_num_batched_tokens:
            return None
        chosen = set(id(r) for r in in_flight)
        needed = [0] * len(self.cache.groups)
        for request in self.running:
            if id(request) not in chosen or request.status is not RequestStatus.RUNNING_DECODE or request.finished or request.cache is None:
                return None
            if len(request.output_token_ids) + 1 >= request.sampling_params.max_tokens:
                return None  # finishes by length on the token in flight: a step of another shape follows
            after = request.num_computed_tokens + 1
            if after + 1 > self.config.max_model_len:
                return None
            for index, pages in enumerate(self.cache.pages_to_append(request.cache, after, 1)):
                needed[index] += pages
        reclaimable = self.cache.num_reclaimable_pages()
        if any(n > group.allocator.num_free + reclaimable for n, group in zip(needed, self.cache.groups)):
            return None
        for request in in_flight:
            if not self.cache.append(request.cache, request.num_computed_tokens + 1, 1):
                raise RuntimeError("pages counted as free could not be taken")  # single-threaded: cannot happen
            request.current_chunk_size = 1
        return list(in_flight)

    def _reap_finished(self) -> None:
        still = []
        for request in self.running:
            if request.finished:
                self._release(request)
                self.requests.pop(request.request_id, None)
                self.num_finished += 1
            else:
                still.append(request)
        self.running = still

    def _schedule_decodes(self, output: SchedulerOutput, budget: int) -> None:
        for request in list(self.running):
            if request.status is not RequestStatus.RUNNING_DECODE or request not in self.running:
                continue
            if budget - len(output.decode_batch) <= 0:
                break
            if not self._make_room(request, 1, output) or not self.cache.append(request.cache, request.num_computed_tokens, 1):
                if request in self.running:
                    self._preempt(request, output)
                continue
            request.current_chunk_size = 1
            output.decode_batch.append(request)

    def _schedule_running_prefills(self, output: SchedulerOutput, budget: int) -> int:
        oldest_seen = False
        for request in list(self.running):
            if request.status is not RequestStatus.RUNNING_PREFILL or request not in self.running:
                continue
            if budget <= 0:
                break
            oldest = not oldest_seen
            oldest_seen = True
            wanted = min(request.num_uncomputed_tokens, budget, self.config.max_prefill_chunk_size)
            chunk = min(wanted, self.cache.max_new_tokens(request.cache, request.num_computed_tokens))
            while chunk <= 0 and oldest and self.running and self.running[-1] is not request:
                victim = self.running[-1]
                self._preempt(victim, output)
                chunk = min(wanted, self.cache.max_new_tokens(request.cache, request.num_computed_tokens))
            if chunk <= 0 or not self.cache.append(request.cache, request.num_computed_tokens, chunk):
                continue
            request.current_chunk_size = chunk
            output.prefill_batch.append(request)
            budget -= chunk
        return budget

    def _admit(self, output: SchedulerOutput, budget: int) -> None:
        while self.waiting and budget > 0:
            if len(self.running) >= self.config.max_num_seqs:
                break
            request = self.waiting[0]
            sequence = self.cache.new_sequence()
            if sequence is None:
                break
            # pages of a prefix that an earlier request has published are taken over, not computed (reference :268-277)
            cached = self.cache.match_prefix(sequence, request.all_token_ids)
            wanted = min(len(request.all_token_ids) - cached, budget, self.config.max_prefill_chunk_size)
            headroom = self.cache.num_available_pages() - self._watermark_pages
            chunk = min(wanted, self.cache.max_new_tokens(sequence, cached, headroom_pages=headroom))
            if chunk <= 0 or not self.cache.append(sequence, cached, chunk):
                self.cache.free_sequence(sequence)
                break
            self.waiting.popleft()
            request.cache = sequence
            request.num_computed_tokens = cached
            request.num_cached_tokens = cached
            request.status = RequestStatus.RUNNING_PREFILL
            request.current_chunk_size = chunk
            self.running.append(request)
            output.prefill_batch.append(request)
            budget -= chunk

    # -- after the forward --------------------------------------------------------------
    def advance(self, request: Request, num_tokens: int) -> None:
        """``num_tokens`` more of the request are now in the cache; pages behind a window go back."""
        request.num_computed_tokens += num_tokens
        if request.cache is not None:
            self.cache.release_behind_window(request.cache, request.num_computed_tokens)
            self.cache.publish(request.cache, request.all_token_ids, request.num_computed_tokens)

    def stats(self) -> Dict[str, float]:
        total = self.cache.num_total_pages
        used = self.cache.num_used_pages()
        return {
            "num_running": float(len(self.running)),
            "num_waiting": float(len(self.waiting)),
            "num_preemptions": float(self.num_preemptions),
            "num_finished": float(self.num_finished),
            "total_blocks": float(total),
            "free_blocks": float(self.cache.num_free_pages()),
            "evictable_blocks": float(self.cache.num_reclaimable_pages()),
            "prefix_hit_rate": 0.0 if self.cache.prefix is None else self.cache.prefix.hit_rate,
            "used_blocks": float(used),
            "usage": 0.0 if total == 0 else used / total,
        }
