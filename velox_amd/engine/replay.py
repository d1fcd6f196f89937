"""Trace replay: given token ids fed step by step through the engine's own model, step function,
cache manager and kernels; logits written out; nothing sampled.

Input, one JSON object per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries`` are one batch: for each request its next tokens and the places among them whose
logits are wanted.  ``end`` names requests that are finished after the step; their pages and
slot are given back.  For a step in which something is wanted, ``<out>/<step>.f32`` holds the
logits ``[wanted, vocab]`` as little-endian float32, in the order of the entries and of ``want``.
After every step ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import json
import os
import sys
from typing import Dict, IO, List, Optional

import numpy as np
import torch

from ..cache.manager import CacheManager, SequenceCache
from ..config.engine_config import resolve_dtype
from ..config.registry import load_config
from ..weights import bind_from_checkpoint
from .batch import StepEntry
from .engine import build_model, model_position_limit
from .runner import ModelRunner


class TraceError(RuntimeError):
    pass


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, block_size: int = 16, max_live: int = 8, device: str = "cuda", ops=None,
                 enable_graphs: bool = False) -> None:
        """``max_live``: the most requests that are live at a time (and so in one step).  ``enable_graphs``: steps in which
        every entry brings one token and wants it are replayed from captured HIP graphs, as the engine decodes."""
        self.device = torch.device(device)
        self.dtype = resolve_dtype(dtype)
        if ops is None:
            from ..kernels import load_ops

            ops = load_ops(self.device)
        self.ops = ops
        self.config = load_config(model_dir)
        pages = (int(max_tokens) + block_size - 1) // block_size
        if pages < 1:
            raise TraceError("--max-tokens must be positive")
        capacity = pages * block_size
        self.max_model_len = min(capacity, model_position_limit(self.config))
        self.model = build_model(self.config, self.dtype, self.device, max_position=self.max_model_len)
        bind_from_checkpoint(self.model, model_dir, self.dtype, self.device)
        ops.prepare(self.model, self.dtype)
        self.cache = CacheManager(self.model.cache_needs(), block_size, pages + 1, max_live, self.dtype, self.device, max_model_len=self.max_model_len)
        self.runner = ModelRunner(self.model, self.cache, ops, self.dtype, self.device, max_num_tokens=max(capacity, 64), max_num_seqs=max_live, enable_graphs=enable_graphs)
        self.runner.capture_decode_graphs()
        self.vocab_size = self.model.spec.vocab_size
        self.live: Dict[str, List] = {}  # id -> [SequenceCache, tokens in the cache]

    def step(self, record: dict) -> Optional[np.ndarray]:
        entries: List[StepEntry] = []
        ids: List[str] = []
        for item in record.get("entries", []):
            rid = str(item["id"])
            tokens = [int(t) for t in item["tokens"]]
            want = [int(w) for w in item.get("want", [])]
            if not tokens:
                raise TraceError(f"step {record.get('step')}: request {rid!r} brings no tokens")
            if rid in ids:
                raise TraceError(f"step {record.get('step')}: request {rid!r} appears twice")
            bad = [t for t in tokens if not 0 <= t < self.vocab_size]
            if bad:
                raise TraceError(f"request {rid!r}: token ids outside the vocabulary of {self.vocab_size}: {bad[:8]}")
            if rid not in self.live:
                seq = self.cache.new_sequence()
                if seq is None:
                    raise TraceError(f"request {rid!r}: no free slot ({len(self.live)} requests are live)")
                self.live[rid] = [seq, 0]
            seq, computed = self.live[rid]
            if computed + len(tokens) > self.max_model_len:
                raise TraceError(f"request {rid!r} would reach {computed + len(tokens)} tokens; the limit is {self.max_model_len}")
            if not self.cache.append(seq, computed, len(tokens)):
                raise TraceError(f"request {rid!r}: out of cache pages ({self.cache.num_free_pages()} free) for {len(tokens)} more tokens")
            entries.append(StepEntry(seq, tokens, computed, want))
            ids.append(rid)
        logits = self.runner.step(entries) if entries else None
        for rid, entry in zip(ids, entries):
            self.live[rid][1] += len(entry.token_ids)
            self.cache.release_behind_window(self.live[rid][0], self.live[rid][1])
        for rid in record.get("end", []):
            state = self.live.pop(str(rid), None)
            if state is not None:
                self.cache.free_sequence(state[0])
        if logits is None:
            return None
        return logits.float().cpu().numpy().astype("<f4", copy=False)


def run(model_dir: str, dtype: str, out_dir: str, max_tokens: int, block_size: int = 16, stream: IO[str] = sys.stdin, device: str = "cuda") -> int:
    os.makedirs(out_dir, exist_ok=True)
    replayer = Replayer(model_dir, dtype, max_tokens, block_size=block_size, device=device)
    for line in stream:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        logits = replayer.step(record)
        if logits is not None:
            logits.tofile(os.path.join(out_dir, f"{step}.f32"))
        print(f"done {step}", flush=True)
    return 0
