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
    """The reference's knobs under the reference's names (``engine/scheduler.py:16-23``)."""

    max_num_seqs: int = 32
    max_num_batched_tokens: int = 2048
    max_prefill_chunk_size: int = 512
    max_model_len: int = 4096
    watermark: float = 0.01


@dataclass(frozen=True)
class Portion:
    """``count`` tokens of ``request.all_token_ids`` from position ``start`` on: a piece of a prompt (or of a prompt plus
    what was generated before a preemption) that one step computes."""

    request: Request
    start: int
    count: int

    @property
    def completes(self) -> bool:
        """Whether the request's tokens are all in the cache after this portion, so that its last row is sampled."""
        return self.start + self.count >= len(self.request.all_token_ids)


@dataclass
class StepPlan:
    """What one step computes: a single token for each of ``decodes``, then ``portions``.  ``preempted`` lists who lost
    their pages while the plan was made; none of them is in the plan."""

    decodes: List[Request] = field(default_factory=list)
    portions: List[Portion] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return len(self.decodes) + sum(p.count for p in self.portions)

    def is_empty(self) -> bool:
        return not self.decodes and not self.portions

    def requests(self) -> List[Request]:
        return self.decodes + [p.request for p in self.portions]

    def count_of(self, request: Request) -> int:
        """Tokens of ``request`` in this step (0: it is not in it)."""
        if any(r is request for r in self.decodes):
            return 1
        return next((p.count for p in self.portions if p.request is request), 0)

    def withdraw(self, request: Request) -> None:
        self.decodes = [r for r in self.decodes if r is not request]
        self.portions = [p for p in self.portions if p.request is not request]


class Scheduler:
    def __init__(self, cache: CacheManager, config: Optional[SchedulerConfig] = None, **overrides) -> None:
        self.config = config or SchedulerConfig(**overrides)
        self.cache = cache
        self.config.max_model_len = min(self.config.max_model_len, cache.max_model_len)
        self.waiting: Deque[Request] = deque()  # first come first served; a preempted request goes to the front
        self.running: List[Request] = []  # in order of admission: the last one is the newest
        self.requests: Dict[str, Request] = {}
        # admission leaves this many pages free, so that running requests can grow for a while without preempting
        self._pages_held_back = max(1, int(cache.num_total_pages * self.config.watermark))
        self.num_preemptions = 0
        self.num_finished = 0

    # -- requests come and go -------------------------------------------------------------------
    def add_request(self, request: Request) -> None:
        """Queues a request; refuses one that could not run to its end even alone (reference ``engine/scheduler.py:67-82``
        checks the same two lengths; its pool capacity counts the reserved page, so a request of exactly that size would
        wait for ever there)."""
        limit = self.config.max_model_len
        prompt, generated = request.num_prompt_tokens, request.sampling_params.max_tokens
        if prompt >= limit:
            raise ValueError(f"request {request.request_id!r}: a prompt of {prompt} tokens leaves no room to generate under max_model_len={limit}")
        if prompt + generated > limit:
            raise ValueError(f"request {request.request_id!r}: {prompt} prompt tokens + max_tokens={generated} is more than max_model_len={limit}")
        if request.request_id in self.requests:
            raise ValueError(f"there is already a request with the id {request.request_id!r}")
        self.requests[request.request_id] = request
        self.waiting.append(request)

    def abort_request(self, request_id: str) -> bool:
        """Ends a queued or running request now and gives back what it holds; False if there is none to end."""
        request = self.requests.pop(request_id, None)
        if request is None or request.finished:
            return False
        request.finish(FinishReason.ABORT)
        self._give_back(request)
        self.running = [r for r in self.running if r is not request]
        self.waiting = deque(r for r in self.waiting if r is not request)
        return True

    def has_work(self) -> bool:
        return bool(self.waiting) or bool(self.running)

    @property
    def num_waiting(self) -> int:
        return len(self.waiting)

    @property
    def num_running(self) -> int:
        return len(self.running)

    def _give_back(self, request: Request) -> None:
        if request.cache is not None:
            self.cache.free_sequence(request.cache)
            request.cache = None

    def _drop_finished(self) -> None:
        """Requests that ended since the last decision leave ``running``; their pages and slot go back only now, so a step
        that was still in flight when they ended wrote into pages that were still theirs.  A request may also end while it
        WAITS: it was preempted with a token still in flight, and that token turned out to be its last.  It holds nothing,
        and must not be admitted again."""
        ended = [r for r in self.running if r.finished]
        ended_waiting = [r for r in self.waiting if r.finished]
        if not ended and not ended_waiting:
            return
        for request in ended + ended_waiting:
            self._give_back(request)
            self.requests.pop(request.request_id, None)
        self.num_finished += len(ended) + len(ended_waiting)
        if ended:
            self.running = [r for r in self.running if not r.finished]
        if ended_waiting:
            self.waiting = deque(r for r in self.waiting if not r.finished)

    def _preempt(self, victim: Request, plan: Optional[StepPlan] = None) -> None:
        """Recompute preemption: everything the victim holds goes back, it waits at the front of the queue and is later
        computed again from its first token, generated tokens included."""
        if plan is not None:
            # it may have been given a place in this very plan already (the reference leaves such a request in its
            # batch, engine/scheduler.py:241-247): it must not run without pages
            plan.withdraw(victim)
            plan.preempted.append(victim)
        self._give_back(victim)
        victim.evicted()
        self.running = [r for r in self.running if r is not victim]
        self.waiting.appendleft(victim)
        self.num_preemptions += 1

    # -- one decision ---------------------------------------------------------------------------
    def schedule(self) -> StepPlan:
        self._drop_finished()
        plan = StepPlan()
        budget = self.config.max_num_batched_tokens
        budget = self._place_decodes(plan, budget)
        budget = self._place_running_prompts(plan, budget)
        self._admit_waiting(plan, budget)
        return plan

    def _place_decodes(self, plan: StepPlan, budget: int) -> int:
        """One token for every decoding request, oldest first.  When the token's page cannot be had, the newest running
        request is preempted, as often as it takes; if that comes to be the request itself, it waits."""
        for request in [r for r in self.running if r.status is RequestStatus.RUNNING_DECODE]:
            if budget <= 0:
                break
            if request.cache is None:
                continue  # preempted for an older request earlier in this loop
            while request.cache is not None and not self.cache.can_append(request.cache, request.num_computed_tokens, 1):
                self._preempt(self.running[-1], plan)
            if request.cache is None:
                continue
            if not self.cache.append(request.cache, request.num_computed_tokens, 1):
                self._preempt(request, plan)  # (beyond max_model_len: cannot happen to a request that add_request let in)
                continue
            plan.decodes.append(request)
            budget -= 1
        return budget

    def _portion_that_fits(self, request: Request, sequence, computed: int, budget: int, headroom_pages: Optional[int] = None) -> int:
        wanted = min(len(request.all_token_ids) - computed, budget, self.config.max_prefill_chunk_size)
        return min(wanted, self.cache.max_new_tokens(sequence, computed, headroom_pages=headroom_pages))

    def _place_running_prompts(self, plan: StepPlan, budget: int) -> int:
        """The next portion of every request whose prompt is under way, cut to the budget, the portion limit and the pages
        that can be had.  Only the oldest of them may take pages from others, and only from requests newer than itself."""
        under_way = [r for r in self.running if r.status is RequestStatus.RUNNING_PREFILL]
        for index, request in enumerate(under_way):
            if budget <= 0:
                break
            if request.cache is None:
                continue  # preempted for the oldest one
            count = self._portion_that_fits(request, request.cache, request.num_computed_tokens, budget)
            while count <= 0 and index == 0 and self.running[-1] is not request:
                self._preempt(self.running[-1], plan)
                count = self._portion_that_fits(request, request.cache, request.num_computed_tokens, budget)
            if count <= 0 or not self.cache.append(request.cache, request.num_computed_tokens, count):
                continue
            plan.portions.append(Portion(request, request.num_computed_tokens, count))
            budget -= count
        return budget

    def _admit_waiting(self, plan: StepPlan, budget: int) -> None:
        """Waiting requests start in their order of arrival while tokens, slots and pages (less those held back) are left.
        The first one that does not fit ends admission for this step: nobody overtakes it."""
        while self.waiting and budget > 0 and len(self.running) < self.config.max_num_seqs:
            request = self.waiting[0]
            sequence = self.cache.new_sequence()
            if sequence is None:
                return
            # pages of a prefix that an earlier request has published are taken over, not computed (reference :268-277)
            cached = self.cache.match_prefix(sequence, request.all_token_ids)
            headroom = self.cache.num_available_pages() - self._pages_held_back
            count = self._portion_that_fits(request, sequence, cached, budget, headroom_pages=headroom)
            if count <= 0 or not self.cache.append(sequence, cached, count):
                self.cache.free_sequence(sequence)  # (the matched pages too)
                return
            self.waiting.popleft()
            request.admitted(sequence, cached)
            self.running.append(request)
            plan.portions.append(Portion(request, cached, count))
            budget -= count

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
