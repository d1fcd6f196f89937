"""The engine loop: scheduler -> one step of the model -> sampler -> request bookkeeping.

Entry points and their meaning follow the reference (``engine/engine.py``):
``Engine.from_pretrained(EngineConfig(model=folder))`` ``:105-172``, ``add_request`` ``:213``,
``step`` ``:275-369``, ``generate`` ``:398-410``, ``has_work`` ``:265``, ``abort_request`` ``:216``,
``snapshot`` ``:412-417``.  Where the reference runs a prefill forward and a decode forward on
two streams and concatenates their last rows, ``step`` here hands ONE mixed batch to the
step function.  The one host wait per step is the read of the sampled tokens
(reference ``:358-359``).
"""
from __future__ import annotations

import collections
import logging
import queue
import time
from dataclasses import dataclass
from typing import Deque, Dict, FrozenSet, Iterable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager, pages_that_fit
from ..config.engine_config import EngineConfig
from ..config.model_config import read_generation_eos
from ..config.registry import config_from_dict, get_architecture, load_config
from ..parts.model import DecoderModel
from ..sampling.sampler import Sampler
from ..weights import bind_from_checkpoint, bind_random
from .batch import StepEntry
from .request import PENDING_TOKEN, FinishReason, Request
from .runner import ModelRunner
from .scheduler import Portion, Scheduler, SchedulerConfig, StepPlan

@dataclass
class _Flight:
    """A step that has been queued on the device."""

    decode: List[Request]
    prefill: List[Portion]
    sampled: List[Request]  # the requests whose rows were sampled, in row order
    tokens: Optional[torch.Tensor]  # int32 [len(sampled)] on the device
    landing: Optional[tuple] = None  # (pinned host tensor the tokens are copied to, event recorded behind the copy)
    booked: bool = False  # positions advanced and room made for the sampled tokens (Engine._book)
    expected: Optional[List[Optional[int]]] = None  # per sampled row: the token's index in the request's output, None = nobody waits for it
    timer: Optional[tuple] = None  # (event before the step's first kernel, event behind its last): the device's time for it

    def requests(self) -> List[Request]:
        return self.decode + [portion.request for portion in self.prefill]


logger = logging.getLogger(__name__)

_STAGES = ("scheduler_ms", "prepare_ms", "forward_ms", "sampling_ms", "cpu_sync_wait_ms", "step_ms", "gpu_ms")


def model_position_limit(model_config) -> int:
    """The most positions the architecture itself allows: ``ModelSpec.max_position`` of the spec made without a limit of
    the caller's (every architecture's ``make_spec`` fills it from whatever its configuration calls it)."""
    return int(get_architecture(model_config.architecture).make_spec(model_config, None).max_position)


def build_model(model_config, dtype: torch.dtype, device, max_position: Optional[int] = None) -> DecoderModel:
    spec = get_architecture(model_config.architecture).make_spec(model_config, max_position)
    return DecoderModel(spec)


class Engine:
    def __init__(self, model: DecoderModel, cache: CacheManager, config: EngineConfig, ops, eos_token_ids: Optional[Iterable[int]] = None) -> None:
        config.validate()
        self.config = config
        self.device = torch.device(config.device)
        self.dtype = config.torch_dtype()
        self.model = model
        self.cache = cache
        self.ops = ops
        self.eos_token_ids: FrozenSet[int] = frozenset(eos_token_ids if eos_token_ids is not None else model.spec.eos_token_ids)
        self.scheduler = Scheduler(
            cache,
            SchedulerConfig(
                max_num_seqs=config.max_num_seqs,
                max_num_batched_tokens=config.max_num_batched_tokens,
                max_prefill_chunk_size=config.max_prefill_chunk_size,
                max_model_len=config.max_model_len,
                watermark=config.watermark,
            ),
        )
        self.max_model_len = self.scheduler.config.max_model_len
        self.runner = ModelRunner(
            model, cache, ops, self.dtype, self.device,
            max_num_tokens=config.max_num_batched_tokens,
            max_num_seqs=config.max_num_seqs,
            enable_graphs=config.enable_cuda_graphs,
        )
        self.sampler = Sampler(ops, self.device, seed=config.seed)
        # per-step times by stage, the most recent 65,536 steps (an engine that serves for days does not grow)
        self.stats: Dict[str, Deque[float]] = {name: collections.deque(maxlen=65536) for name in _STAGES}
        self.num_steps = 0
        self._ahead: Optional[_Flight] = None
        # requests and aborts handed over by other threads, taken in at the start of the next step
        self._pending_adds: "queue.Queue[Request]" = queue.Queue()
        self._pending_aborts: "queue.Queue[str]" = queue.Queue()
        self._landings = []
        self._next_landing = 0
        self._timers: List[tuple] = []  # event pairs of queued steps whose device time has not been read yet
        if self.device.type == "cuda":
            rows = max(config.max_num_seqs, 1)
            self._landings = [(torch.zeros(rows, dtype=torch.int32, pin_memory=True), torch.cuda.Event()) for _ in range(3)]

    # -- construction -------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, config: Optional[EngineConfig] = None, ops=None, **overrides) -> "Engine":
        config = config or EngineConfig(**overrides)
        config.validate()
        model_config = load_config(config.model)
        eos = read_generation_eos(config.model)
        return cls._assemble(config, model_config, ops, eos, lambda model, dtype, device: bind_from_checkpoint(model, config.model, dtype, device, ignore_unexpected=config.ignore_unexpected_weights))

    @classmethod
    def from_random(cls, model_config_dict: dict, seed: int, config: Optional[EngineConfig] = None, ops=None, generator_device: str = "cpu", **overrides) -> "Engine":
        """An engine over random weights drawn in memory (no folder), for shapes too large to write out."""
        config = config or EngineConfig(**overrides)
        config.validate()
        model_config = config_from_dict(model_config_dict)
        return cls._assemble(
            config, model_config, ops, None,
            lambda model, dtype, device: bind_random(model, seed, dtype, device, generator_device=generator_device),
        )

    @classmethod
    def _assemble(cls, config: EngineConfig, model_config, ops, eos, bind) -> "Engine":
        device = torch.device(config.device)
        dtype = config.torch_dtype()
        if ops is None:
            from ..kernels import load_ops

            ops = load_ops(device)
        max_model_len = min(config.max_model_len, model_position_limit(model_config))
        config.max_model_len = max_model_len
        model = build_model(model_config, dtype, device, max_position=max_model_len)
        bind(model, dtype, device)
        needs = model.cache_needs()
        if hasattr(ops, "pack_decode_weights"):
            ops.pack_decode_weights = config.pack_decode_weights
        ops.prepare(model, dtype)
        num_pages = config.num_gpu_blocks
        if num_pages is None:
            probe = CacheManager(needs, config.block_size, 2, config.max_num_seqs, dtype, device, allocate_tensors=False)
            free_bytes, _ = torch.cuda.mem_get_info(device)
            free_bytes += torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
            num_pages = pages_that_fit(probe.bytes_per_page(), free_bytes, config.gpu_memory_utilization, config.kv_cache_reserve_mb * 1024 * 1024)
            wanted = (config.max_num_seqs * max_model_len + config.block_size - 1) // config.block_size + 1
            num_pages = min(num_pages, max(2, wanted))
        cache = CacheManager(needs, config.block_size, num_pages, config.max_num_seqs, dtype, device, max_model_len=max_model_len,
                             prefix_caching=config.enable_prefix_caching, scatter_pages=config.scatter_pages)
        engine = cls(model, cache, config, ops, eos_token_ids=eos)
        engine.warmup()
        return engine

    def warmup(self) -> None:
        if self.device.type != "cuda":
            return
        self.runner.capture_decode_graphs()
        # one prompt portion of the usual size on the null page: the first request does not pay for the matrix library's
        # first use of a data type and of these shapes (about 50 ms for the first portion otherwise)
        for count in sorted({self.config.max_prefill_chunk_size, self.config.max_num_batched_tokens}):
            self.runner.warm_prefill(count)  # (a step's portions together may reach the token budget)
        torch.cuda.synchronize()

    def tune_matrix_products(self, token_counts: Sequence[int], progress=None) -> int:
        """Optional, bfloat16 only: has the matrix library time its candidate kernels for this model's weight shapes at
        the given numbers of tokens per step (typically the prefill chunk size and the larger decode batch sizes) and
        keep the fastest.  Takes seconds per shape.  A step of prompt portions with a few rows less than one of these
        counts is padded up to it from then on (``ModelRunner.tuned_row_counts``); other steps are unaffected.  Only products that
        the engine hands to the library are timed (``ops.library_serves``); captured decode steps are captured again
        if one of them holds such a product.  ``progress(text)``, if given, is told after every count (a ladder of
        counts takes minutes)."""
        if self.dtype != torch.bfloat16 or self.device.type != "cuda" or not hasattr(self.ops, "tune_library_products"):
            return 0
        shapes = set()
        for part in self.model.all_parts():
            for attr, param in part.params().items():
                tensor = getattr(part, attr, None)
                if param.role == "matrix" and param.product and tensor is not None and tensor.dim() == 2 and tensor.dtype == torch.bfloat16:
                    shapes.add(tuple(tensor.shape))
        done = 0
        recapture = False
        results_file = self.ops.tuning_file() if self.config.library_tuning_file == "auto" else self.config.library_tuning_file
        counts = sorted(set(int(m) for m in token_counts))
        for index, count in enumerate(counts):
            served = [shape for shape in shapes if self.ops.library_serves(count, *shape)]
            if served:
                done += self.ops.tune_library_products(served, [count], results_file=results_file)
                if progress is not None:
                    progress(f"timed the library's kernels for steps of {count} rows ({index + 1} of {len(counts)} counts, {len(served)} products)")
                recapture = recapture or count <= self.config.max_num_seqs
                if count > self.config.max_num_seqs and count not in self.runner.tuned_row_counts:
                    self.runner.tuned_row_counts = sorted(self.runner.tuned_row_counts + [count])  # steps a little shorter are padded up to it
        if recapture and self.runner.uses_graphs:
            self.runner.capture_decode_graphs()
            torch.cuda.synchronize()
        return done

    # -- requests -----------------------------------------------------------------------
    def add_request(self, request: Request) -> None:
        bad = [t for t in request.prompt_token_ids if not 0 <= t < self.model.spec.vocab_size]
        if bad:
            raise ValueError(f"token ids outside the vocabulary of {self.model.spec.vocab_size}: {bad[:8]}")
        self.scheduler.add_request(request)

    def abort_request(self, request_id: str) -> bool:
        self.sampler.release(request_id)
        return self.scheduler.abort_request(request_id)

    def abort_all(self) -> str:
        self._drain_control_queue()
        for request_id in list(self.scheduler.requests):
            self.abort_request(request_id)
        return "aborted"

    def check_limits(self, num_prompt_tokens: int, max_tokens: int) -> None:
        """Raises ValueError for a request that ``add_request`` would refuse for its length (reference ``:226-237``)."""
        limit = self.max_model_len
        if num_prompt_tokens >= limit:
            raise ValueError(f"prompt of {num_prompt_tokens} tokens does not fit in max_model_len={limit} "
                             "(at least one token must remain for generation)")
        if num_prompt_tokens + max_tokens > limit:
            raise ValueError(f"prompt of {num_prompt_tokens} tokens plus max_tokens={max_tokens} exceeds max_model_len={limit}")

    def submit(self, request: Request) -> None:
        """``add_request`` for other threads than the one that steps: the request is taken in when the next step begins
        (reference ``:239-263``).  Its length is checked here, in the caller's thread."""
        self.check_limits(request.num_prompt_tokens, request.sampling_params.max_tokens)
        self._pending_adds.put(request)

    def request_abort(self, request_id: str) -> None:
        """``abort_request`` for other threads: carried out when the next step begins."""
        self._pending_aborts.put(request_id)

    def _drain_control_queue(self) -> None:
        while True:
            try:
                request = self._pending_adds.get_nowait()
            except queue.Empty:
                break
            try:
                self.add_request(request)
            except ValueError:
                logger.exception("rejecting request %s", request.request_id)
                request.finish(FinishReason.ABORT)
        while True:
            try:
                request_id = self._pending_aborts.get_nowait()
            except queue.Empty:
                break
            self.abort_request(request_id)

    def has_work(self) -> bool:
        return self.scheduler.has_work() or not self._pending_adds.empty()

    # -- one step -----------------------------------------------------------------------
    @torch.no_grad()
    def step(self) -> None:
        """One step of every scheduled request.  When it returns, each of them holds its new token.

        With ``decode_lookahead`` the NEXT step is already running by then.  As soon as a step is queued, everything about
        it that does not depend on the values of the tokens it samples is booked: positions advance, and each sampled
        request gets a pending token in its lists (``Request.expect_token``; a request that reaches its length with it is
        closed).  On that state the scheduler decides the next step, of any kind (prompt portions, admissions,
        preemptions, decodes), and it is queued with the pending tokens' values taken on the device from this step's
        sampler output.  Only then does the host wait for this step's tokens.  The device so never waits for the host to
        schedule, lay out and launch, between decode steps (the reference's 1.5 ms gap per step) or between the steps of
        long prompts.  A request that stops on a token that was still in flight has a row in the successor that nobody
        reads; what it held goes back at the next scheduling decision (anything a later owner of those pages does
        comes, in stream order, behind that row's writes)."""
        step_start = time.perf_counter()
        self._drain_control_queue()
        flight, self._ahead = self._ahead, None
        if flight is not None and not any(self._alive(r) for r in flight.requests()):
            flight = None  # launched for requests that have all stopped or been aborted since
        if flight is None:
            scheduled = self.scheduler.schedule()
            self.stats["scheduler_ms"].append((time.perf_counter() - step_start) * 1000)
            if scheduled.is_empty():
                return
            flight = self._launch(scheduled)
        if self.config.decode_lookahead:
            self._book(flight)
            t0 = time.perf_counter()
            ahead = self.scheduler.schedule()
            self.stats["scheduler_ms"].append((time.perf_counter() - t0) * 1000)
            if not ahead.is_empty():
                self._ahead = self._launch(ahead, pending=flight)
        self._finish_step(flight)
        self.num_steps += 1
        self.stats["step_ms"].append((time.perf_counter() - step_start) * 1000)

    @staticmethod
    def _alive(request: Request) -> bool:
        return not request.finished and request.cache is not None

    def _launch(self, plan: StepPlan, pending: Optional["_Flight"] = None) -> "_Flight":
        """Queues one step on the device: the forward over the batch and the sampler.  ``pending``: the step before this
        one, booked but not finished: its sampled tokens are pending in the requests' lists, and their values are taken on
        the device from its sampler's output."""
        entries: List[StepEntry] = []
        sampled: List[Request] = []
        dest_rows: List[int] = []
        source_rows: List[int] = []
        source_of = {id(r): row for row, r in enumerate(pending.sampled)} if pending is not None else {}

        def source_row(request: Request) -> int:
            # a pending token belongs to the step just before this one: nothing else can still be in flight
            row = source_of.get(id(request))
            if row is None:
                raise RuntimeError(f"request {request.request_id!r} has a token in flight, but the step before this one did not sample it")
            return row

        at = 0  # rows of the step so far
        # decode rows first, then prompt portions; only rows that complete their tokens are sampled
        for request in plan.decodes:
            start = request.num_computed_tokens
            token = request.all_token_ids[start]
            if token == PENDING_TOKEN:
                dest_rows.append(at)
                source_rows.append(source_row(request))
            entries.append(StepEntry(request.cache, [token], start, [0]))
            sampled.append(request)
            at += 1
        for portion in plan.portions:
            request, start, count = portion.request, portion.start, portion.count
            tokens = request.all_token_ids[start:start + count]
            if tokens[-1] == PENDING_TOKEN:  # (only a request's newest token can be pending)
                dest_rows.append(at + count - 1)
                source_rows.append(source_row(request))
            entries.append(StepEntry(request.cache, tokens, start, [count - 1] if portion.completes else []))
            if portion.completes:
                sampled.append(request)
            at += count

        timer = None
        if self.device.type == "cuda":
            timer = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            timer[0].record()
        t0 = time.perf_counter()
        logits = self.runner.step(entries, device_ids=(pending.tokens, dest_rows, source_rows) if dest_rows else None)
        self.stats["prepare_ms"].append(self.runner.last_prepare_ms)
        self.stats["forward_ms"].append((time.perf_counter() - t0) * 1000 - self.runner.last_prepare_ms)

        tokens_gpu = None
        if sampled:
            t0 = time.perf_counter()
            # (penalties: the sampler counts a request's tokens itself once it has seen its history, which it asks for
            # the first time only; a request is new to it at the end of its prompt, when no token of it is pending)
            needs_history = any(r.sampling_params.has_penalties for r in sampled)
            tokens_gpu = self.sampler.sample(
                logits,
                [r.sampling_params for r in sampled],
                [r.request_id for r in sampled],
                [len(r.output_token_ids) for r in sampled],
                histories=[(lambda r=r: r.all_token_ids) for r in sampled] if needs_history else None,
            )
            self.stats["sampling_ms"].append((time.perf_counter() - t0) * 1000)
        # the copy of the tokens to the host is queued right behind the sampler, before a later step can be queued
        # behind it: waiting for it then waits for this step only
        landing = None
        if timer is not None:
            timer[1].record()
        if tokens_gpu is not None and self.device.type == "cuda":
            landing = self._landings[self._next_landing]
            self._next_landing = (self._next_landing + 1) % len(self._landings)
            landing[0][: len(sampled)].copy_(tokens_gpu, non_blocking=True)
            landing[1].record()
        return _Flight(list(plan.decodes), list(plan.portions), sampled, tokens_gpu, landing, timer=timer)

    def _book(self, flight: "_Flight") -> None:
        """What a queued step changes whatever tokens it draws: its positions are in the cache, and every sampled request
        has one more token (pending until the step's tokens arrive)."""
        if flight.booked:
            return
        flight.booked = True
        for request in flight.decode:
            if self._alive(request):
                self.scheduler.advance(request, 1)
        for portion in flight.prefill:
            if self._alive(portion.request):
                self.scheduler.advance(portion.request, portion.count)
        flight.expected = [request.expect_token() if self._alive(request) else None for request in flight.sampled]

    def _finish_step(self, flight: "_Flight") -> None:
        """Waits for the step's tokens and hands them to their requests; stops."""
        self._book(flight)
        if flight.timer is not None:
            self._timers.append(flight.timer)
        if flight.tokens is None:
            return
        sync_start = time.perf_counter()
        # the one place per step where the host waits for the device
        if flight.landing is not None:
            flight.landing[1].synchronize()
            tokens = flight.landing[0][: len(flight.sampled)].tolist()
        else:
            tokens = flight.tokens.tolist()
        self.stats["cpu_sync_wait_ms"].append((time.perf_counter() - sync_start) * 1000)
        # the device's time for the steps that have ended by now (this one has: its tokens are here)
        while self._timers and self._timers[0][1].query():
            begin, end = self._timers.pop(0)
            self.stats["gpu_ms"].append(begin.elapsed_time(end))
        for request, index, token in zip(flight.sampled, flight.expected, tokens):
            if index is None:
                continue  # it had stopped or been aborted before this step was booked
            aborted = request.finish_reason is FinishReason.ABORT
            request.deliver_token(index, int(token), announce=not aborted)
            if aborted:
                continue
            reason = request.stop_reason(int(token), self.eos_token_ids)
            if reason is not None:
                request.finish(reason)
                self.sampler.release(request.request_id)

    @torch.no_grad()
    def generate(self, requests: Sequence[Request], max_steps: Optional[int] = None) -> List[Request]:
        for request in requests:
            self.add_request(request)
        steps = 0
        while self.has_work():
            self.step()
            steps += 1
            if max_steps is not None and steps >= max_steps:
                break
        return list(requests)

    def snapshot(self) -> Dict[str, float]:
        stats = self.scheduler.stats()
        stats["num_steps"] = float(self.num_steps)
        stats["cuda_graphs"] = 1.0 if self.runner.uses_graphs else 0.0
        stats["kv_cache_bytes"] = float(self.cache.bytes_per_page() * (self.cache.num_total_pages + 1))
        return stats
