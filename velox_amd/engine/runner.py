"""The step function: one batch of (request, its next tokens) through the model, from the cache.

The reference runs a step as up to two forwards, a varlen prefill batch and a decode
batch (``engine/engine.py:303-316``, ``engine/model_runner.py:298-313``).  Here a step is ONE
forward over one flat batch: every entry brings ``q_len >= 1`` tokens that start at its own
position; portions of prompts sit beside single decoded tokens.  Only the tokens given
are run; everything earlier is read from the cache.  Logits come back for the wanted rows
only, in float32 (the reference likewise runs its head on chosen rows,
``engine/engine.py:307-309,339-341``).

A batch in which every entry has one token may be replayed from a captured HIP graph:
graphs are captured per batch-size bucket 1, 2, 4, ... (reference
``engine/model_runner.py:19-26,331-368``), rows beyond the batch are padded with one-token
rows that read and write the reserved null page, and the step's tensors live at fixed
addresses that the host refreshes before each replay.  A capture fixes how its kernels are
launched; a part whose kernels would be launched differently behind short contexts says so
(``Part.capture_key_bounds``) and gets further captures of the same bucket, each for steps whose
sequences all stay within a bound on their length; a step replays the tightest capture that
covers it.  The captured activations live in the pool of the framework's graph allocator
(``torch.cuda.graph_pool_handle``), shared by all captures; the step's inputs and the parts'
scratch are the runner's own buffers.
"""
from __future__ import annotations

import time
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheManager
from ..parts.model import DecoderModel
from .batch import BatchBuilder, StepContext, StepEntry, StepLimits, Workspace


def decode_buckets(max_num_seqs: int) -> List[int]:
    buckets: List[int] = []
    size = 1
    while size < max_num_seqs:
        buckets.append(size)
        size *= 2
    buckets.append(max_num_seqs)
    return buckets




class ModelRunner:
    def __init__(
        self,
        model: DecoderModel,
        cache: CacheManager,
        ops,
        dtype: torch.dtype,
        device,
        max_num_tokens: int,
        max_num_seqs: int,
        enable_graphs: bool = False,
    ) -> None:
        self.model = model
        self.cache = cache
        self.ops = ops
        self.dtype = dtype
        self.device = torch.device(device)
        self.max_num_tokens = max(int(max_num_tokens), int(max_num_seqs))
        self.max_num_seqs = int(max_num_seqs)
        self.builder = BatchBuilder(cache, self.device, self.max_num_tokens, self.max_num_seqs + 1)  # (+1: the rows that pad a step, see tuned_row_counts)
        # Numbers of rows for which the matrix library's kernels have been timed (``Engine.tune_matrix_products``).  The
        # library picks a kernel per exact shape, and an untimed number of rows gets its default choice, about a quarter
        # slower at these sizes: a step of portions that is a little short of a timed number of rows is padded up to it with
        # rows of a sequence on the null page.
        self.tuned_row_counts: List[int] = []
        self.max_padding = 0.12  # the most a step is made longer, as a share of its own rows
        self.num_padded_steps = 0
        self.last_prepare_ms = 0.0  # host time of the last step's batch layout (block tables, positions, ids)
        # every part's scratch at its largest, before anything runs: captured steps hold these addresses
        self.workspace = Workspace(self.device)
        limits = StepLimits(self.max_num_tokens, self.max_num_seqs, cache.max_model_len)
        for part in model.all_parts():
            for name, numel in part.workspace_needs(ops, limits).items():
                self.workspace.reserve(name, numel)
        self.workspace.fix()
        # a model with a part that reads the host while it runs (``Part.graph_safe`` False) is never captured
        self.enable_graphs = bool(enable_graphs) and self.device.type == "cuda" and model.allows_capture()
        self._graphs: Dict[int, Tuple[object, torch.Tensor, torch.Tensor]] = {}
        # the same buckets again for steps whose sequences are all short: bucket -> [(bound on keys, capture)], tightest first
        self._bounded_graphs: Dict[int, List[Tuple[int, Tuple[object, torch.Tensor, torch.Tensor]]]] = {}
        self._graph_buffers: Dict[int, torch.Tensor] = {}
        self._graph_pool = None
        self.num_graph_replays = 0
        self.num_short_graph_replays = 0  # those of them through the captures for short contexts

    # -- the step -----------------------------------------------------------------------
    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry], device_ids: Optional[tuple] = None) -> Optional[torch.Tensor]:
        """Runs the entries' tokens as one batch; returns float32 logits ``[wanted, vocab]``
        in the order of the entries and of their ``want`` (None when nothing is wanted).
        ``device_ids``: see ``BatchBuilder.build`` (token ids that are still being sampled by the step in flight)."""
        if self.enable_graphs and all(len(e.token_ids) == 1 for e in entries):
            if all(list(e.want) == [0] for e in entries):
                bucket = self._bucket_for(len(entries))
                if bucket is not None:
                    return self._replay(bucket, entries, device_ids)
        if self.tuned_row_counts:
            entries = self._padded_to_tuned_rows(entries)
        t0 = time.perf_counter()
        ctx = self.builder.build(entries, self.ops, self.dtype, self.workspace, device_ids=device_ids)
        self.last_prepare_ms = (time.perf_counter() - t0) * 1000
        return self._forward(ctx)

    def _padded_to_tuned_rows(self, entries: Sequence[StepEntry]) -> Sequence[StepEntry]:
        total = sum(len(e.token_ids) for e in entries)
        if total <= self.max_num_seqs:
            return entries  # decode-sized: the skinny kernels do not care, captured steps pad themselves
        target = next((n for n in self.tuned_row_counts if n >= total), None)
        if target is None or target == total or target > self.max_num_tokens or target - total > self.max_padding * total:
            return entries
        from ..cache.manager import SequenceCache

        extra = target - total
        pages = (extra + self.cache.page_size - 1) // self.cache.page_size
        null_seq = SequenceCache(slot=self.cache.state.pad_slot, tables=[[0] * pages for _ in self.cache.groups], released=[0 for _ in self.cache.groups])
        self.num_padded_steps += 1
        return list(entries) + [StepEntry(null_seq, [0] * extra, 0, [])]

    def _forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        residual, pending = self.model.forward(ctx.token_ids, ctx)
        if ctx.rows is None:
            return None
        return self.model.logits(residual, pending, ctx.rows, ctx)

    # -- captured decode ----------------------------------------------------------------
    def _bucket_for(self, batch: int) -> Optional[int]:
        for bucket in sorted(self._graphs):
            if bucket >= batch:
                return bucket
        return None

    def _padded_entries_context(self, bucket: int, entries: Sequence[StepEntry], device_ids: Optional[tuple] = None) -> StepContext:
        t0 = time.perf_counter()
        buffer = self._graph_buffers[bucket]
        padded = [StepEntry(e.seq, e.token_ids, e.start, [0]) for e in entries]
        ctx = self.builder.build(
            padded, self.ops, self.dtype, self.workspace,
            device_buffer=buffer, pad_to=bucket, width=self.builder.width, device_ids=device_ids,
        )
        self.last_prepare_ms = (time.perf_counter() - t0) * 1000
        return ctx

    @torch.no_grad()
    def capture_decode_graphs(self, buckets: Optional[Sequence[int]] = None, warmup_iters: int = 2) -> None:
        """Captures one graph per bucket over padded one-token rows (reference ``engine/model_runner.py:331-368``)."""
        if not self.enable_graphs:
            return
        buckets = list(buckets) if buckets is not None else decode_buckets(self.max_num_seqs)
        self._graph_pool = torch.cuda.graph_pool_handle()
        self._bounded_graphs.clear()
        parts = self.model.all_parts()
        longest = self.cache.max_model_len
        for bucket in buckets:
            capacity = self.builder.section_total(bucket, bucket, bucket, self.builder.width)
            self._graph_buffers[bucket] = torch.zeros(capacity, dtype=torch.int32, device=self.device)
            self._graphs[bucket] = self._capture(self._graph_context(bucket, longest), warmup_iters)
            bounds = sorted({int(b) for part in parts for b in part.capture_key_bounds(self.ops, bucket, longest) if 0 < int(b) < longest})
            if bounds:
                self._bounded_graphs[bucket] = [(bound, self._capture(self._graph_context(bucket, bound), warmup_iters)) for bound in bounds]
        torch.cuda.synchronize()

    def _capture(self, ctx: StepContext, warmup_iters: int):
        stream = torch.cuda.Stream(device=self.device)
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            for _ in range(warmup_iters):
                self._forward(ctx)
        torch.cuda.current_stream().wait_stream(stream)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            logits = self._forward(ctx)
        return graph, logits, ctx

    def _graph_context(self, bucket: int, max_kv_len: int) -> StepContext:
        """A context of ``bucket`` padded rows only (all on the null page), laid out in the bucket's buffer."""
        from ..cache.manager import SequenceCache

        null_seq = SequenceCache(slot=self.cache.state.pad_slot, tables=[[0] for _ in self.cache.groups], released=[0 for _ in self.cache.groups])
        entries = [StepEntry(null_seq, [0], 0, [0]) for _ in range(bucket)]
        ctx = self.builder.build(
            entries, self.ops, self.dtype, self.workspace,
            device_buffer=self._graph_buffers[bucket], pad_to=bucket, width=self.builder.width,
        )
        ctx.all_decode = True
        # lengths are read from device memory at replay; the capture must not specialise on them beyond their bound
        for group in ctx.groups:
            group.max_kv_len = max_kv_len
        ctx.rows = ctx.rows[:bucket]
        return ctx

    @torch.no_grad()
    def warm_prefill(self, num_tokens: int) -> None:
        """Runs one prompt portion of ``num_tokens`` tokens on the null page and drops the result, so that whatever a
        first portion pays once (the matrix library loads its kernels for a data type at first use, tens of
        milliseconds, and picks a kernel per shape) is paid before the first request."""
        from ..cache.manager import SequenceCache

        num_tokens = max(2, min(int(num_tokens), self.builder.max_num_tokens, self.cache.max_model_len))
        pages = (num_tokens + self.cache.page_size - 1) // self.cache.page_size
        null_seq = SequenceCache(slot=self.cache.state.pad_slot, tables=[[0] * pages for _ in self.cache.groups], released=[0 for _ in self.cache.groups])
        ctx = self.builder.build([StepEntry(null_seq, [0] * num_tokens, 0, [num_tokens - 1])], self.ops, self.dtype, self.workspace)
        self._forward(ctx)

    def _replay(self, bucket: int, entries: Sequence[StepEntry], device_ids: Optional[tuple] = None) -> torch.Tensor:
        graph, logits, _ = self._graphs[bucket]
        if bucket in self._bounded_graphs:
            keys = max(e.start for e in entries) + 1  # the longest sequence of the step, this token's key included
            for bound, capture in self._bounded_graphs[bucket]:
                if keys <= bound:
                    graph, logits, _ = capture
                    self.num_short_graph_replays += 1
                    break
        self._padded_entries_context(bucket, entries, device_ids)  # refreshes the bucket's buffer in place
        graph.replay()
        self.num_graph_replays += 1
        return logits[: len(entries)]

    @property
    def uses_graphs(self) -> bool:
        return bool(self._graphs)
