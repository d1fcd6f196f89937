"""The tensors one step needs, built on the host and sent to the device in one copy.

The reference builds the same arrays per forward (``engine/model_runner.py:171-270``: input ids,
positions, slot mapping, sequence lengths, cumulative query lengths, block tables) through
pinned staging buffers with one copy each.  Here all of them are sections of ONE int32
staging buffer, so a step costs one host-to-device copy; a ring of staging buffers, each
guarded by an event, keeps the host from overwriting a buffer whose copy has not run yet
(the race the reference documents, ``engine/model_runner.py:67-77,124-131``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, SequenceCache


@dataclass
class StepEntry:
    """One request's share of a step: its next ``token_ids``, which start at position ``start``
    of the request; ``want`` lists the places among these tokens whose logits are asked for."""

    seq: SequenceCache
    token_ids: Sequence[int]
    start: int
    want: Sequence[int] = ()


@dataclass
class GroupBatch:
    block_tables: torch.Tensor  # int32 [B, W]
    slot_mapping: torch.Tensor  # int32 [T]: page * page_size + offset of every token's key
    kv_lens: torch.Tensor  # int32 [B]: keys in the cache once this step's are written
    max_kv_len: int
    max_kv_len_of_portions: int = 0  # the same over the sequences behind the leading one-token sequences (0: there are none)


class WorkspaceError(RuntimeError):
    pass


class Workspace:
    """Scratch tensors by name, kept across steps so their addresses are stable.

    A captured step holds the addresses of the buffers it was captured with, so a buffer must never be replaced once a
    capture may exist.  The runner therefore asks every part what it can need at most (``Part.workspace_needs``),
    reserves that before anything runs and calls :meth:`fix`; from then on a request for more than is there is an
    error, not a new allocation.  A workspace that was never fixed (a test's own) grows on demand.
    """

    def __init__(self, device) -> None:
        self.device = device
        self._buffers: Dict[str, torch.Tensor] = {}
        self.fixed = False

    def reserve(self, name: str, numel: int, dtype: torch.dtype = torch.float32) -> None:
        """Makes sure ``name`` holds at least ``numel`` elements."""
        buf = self._buffers.get(name)
        if buf is not None and buf.dtype == dtype and buf.numel() >= numel:
            return
        if self.fixed:
            have = "nothing" if buf is None else f"{buf.numel()} x {buf.dtype}"
            raise WorkspaceError(f"workspace buffer {name!r} holds {have} but {numel} x {dtype} are asked for; captured steps hold its "
                                 "address, so it cannot be replaced (the part that uses it must state this size in workspace_needs)")
        self._buffers[name] = torch.empty(max(int(numel), 1), dtype=dtype, device=self.device)

    def fix(self) -> None:
        self.fixed = True

    def get(self, name: str, numel: int, dtype: torch.dtype = torch.float32) -> torch.Tensor:
        self.reserve(name, numel, dtype)
        return self._buffers[name][:numel]

    def addresses(self) -> Dict[str, int]:
        return {name: buf.data_ptr() for name, buf in self._buffers.items()}


@dataclass(frozen=True)
class StepLimits:
    """The most a step can hold: what parts size their scratch for."""

    max_num_tokens: int
    max_num_seqs: int
    max_model_len: int


@dataclass
class StepContext:
    ops: object
    dtype: torch.dtype
    device: torch.device
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor  # int32 [T]
    positions: torch.Tensor  # int32 [T]
    cu_q: torch.Tensor  # int32 [B + 1]
    slots: torch.Tensor  # int32 [B]: state slot of every sequence
    rows: Optional[torch.Tensor]  # int32 [R]: token rows whose logits are wanted
    q_lens: List[int]
    starts: List[int]
    max_q_len: int
    all_decode: bool
    groups: List[GroupBatch]
    workspace: Workspace
    cache: CacheManager = field(repr=False, default=None)
    decode_prefix: int = 0  # how many of the first sequences bring exactly one token

    def cache_view(self, entry: int):
        return self.cache.view(entry, self.groups)


def _align(n: int, to: int = 4) -> int:
    return (n + to - 1) // to * to


class BatchBuilder:
    def __init__(self, cache: CacheManager, device, max_num_tokens: int, max_num_seqs: int, ring: int = 3) -> None:
        self.cache = cache
        self.device = torch.device(device)
        self.max_num_tokens = int(max_num_tokens)
        self.max_num_seqs = int(max_num_seqs)
        self.width = max(1, cache.max_pages_per_seq)
        self.capacity = self.section_total(self.max_num_tokens, self.max_num_seqs, self.max_num_tokens, self.width)
        pin = self.device.type == "cuda"
        self._host = [torch.zeros(self.capacity, dtype=torch.int32, pin_memory=pin) for _ in range(ring)]
        self._device = [torch.zeros(self.capacity, dtype=torch.int32, device=self.device) for _ in range(ring)]
        self._events = [torch.cuda.Event() if pin else None for _ in range(ring)]
        self._used = [False] * ring
        self._next = 0

    def section_total(self, t: int, b: int, r: int, w: int) -> int:
        n_groups = len(self.cache.groups)
        return _align(t) * 2 + _align(b + 1) + _align(b) * 3 + _align(r) + n_groups * (_align(b) + _align(t) + _align(b * w))

    def build(self, entries: Sequence[StepEntry], ops, dtype, workspace: Workspace, device_buffer: Optional[torch.Tensor] = None, pad_to: Optional[int] = None, width: Optional[int] = None,
              device_ids: Optional[tuple] = None) -> StepContext:
        """Lays the step out.  ``pad_to``/``width``/``device_buffer`` are for captured decode steps:
        the batch is padded to ``pad_to`` one-token rows that read and write the null page, the
        block table has the fixed ``width``, and the sections land in the caller's buffer.

        ``device_ids = (tokens int32 [R] on the device, dest_rows, source_rows)``: token ids that the host does not know
        yet (the step that samples them is still in flight): row ``dest_rows[k]`` of this step's tokens is
        ``tokens[source_rows[k]]``; the entries hold a placeholder there.  They are copied into place on the device, behind
        the staging copy, in stream order."""
        cache = self.cache
        page = cache.page_size
        b_real = len(entries)
        b = pad_to if pad_to is not None else b_real
        q_lens = [len(e.token_ids) for e in entries] + [1] * (b - b_real)
        starts = [int(e.start) for e in entries] + [0] * (b - b_real)
        t = sum(q_lens)
        if b_real == 0 or min(q_lens) < 1:
            raise ValueError("a step needs at least one entry and every entry at least one token")
        if t > self.max_num_tokens or b > self.max_num_seqs:
            raise ValueError(f"step of {t} tokens / {b} sequences exceeds the limits {self.max_num_tokens} / {self.max_num_seqs}")

        ids = np.zeros(t, dtype=np.int32)
        positions = np.zeros(t, dtype=np.int32)
        cu = np.zeros(b + 1, dtype=np.int32)
        cu[1:] = np.cumsum(q_lens)
        slots = np.full(b, cache.state.pad_slot, dtype=np.int32)
        rows: List[int] = []
        for i, e in enumerate(entries):
            lo, n = int(cu[i]), q_lens[i]
            if n == 1:  # a decoded token: plain integers are quicker than arrays of one
                ids[lo] = e.token_ids[0]
                positions[lo] = e.start
            else:
                ids[lo:lo + n] = np.asarray(e.token_ids, dtype=np.int32)
                positions[lo:lo + n] = np.arange(e.start, e.start + n, dtype=np.int32)
            slots[i] = e.seq.slot
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"want index {w} outside the entry's {n} tokens")
                rows.append(lo + int(w))
        if pad_to is not None:
            rows.extend(range(int(cu[b_real]), t))  # padded rows ask for their own logits: fixed layout
        r = len(rows)

        if width is None:
            width = 1
            for e in entries:
                for table in e.seq.tables:
                    width = max(width, len(table))
        total = self.section_total(t, b, r, width)
        if total > self.capacity:
            raise ValueError("step does not fit the staging buffer")

        index = self._next
        self._next = (self._next + 1) % len(self._host)
        if self._used[index] and self._events[index] is not None:
            self._events[index].synchronize()
        host = self._host[index].numpy()
        device = device_buffer if device_buffer is not None else self._device[index]

        offset = 0
        sections = {}

        def put(name: str, values: np.ndarray, length: int) -> None:
            nonlocal offset
            host[offset:offset + length] = values.reshape(-1)
            sections[name] = (offset, length)
            offset += _align(length)

        put("ids", ids, t)
        put("positions", positions, t)
        put("cu", cu, b + 1)
        put("slots", slots, b)
        put("rows", np.asarray(rows, dtype=np.int32), r)
        # always laid out: a captured step reads its sections at fixed places.  At most one token per entry is still to
        # come (its newest)
        source = np.zeros(b, dtype=np.int32)
        dest = np.zeros(b, dtype=np.int32)
        num_device_ids = 0
        if device_ids is not None:
            tokens_on_device, dest_rows, source_rows = device_ids
            num_device_ids = len(dest_rows)
            if num_device_ids != len(source_rows) or num_device_ids > b_real:
                raise ValueError("token ids on the device: one source row per destination row, at most one per entry")
            if num_device_ids and (min(dest_rows) < 0 or max(dest_rows) >= t or min(source_rows) < 0 or max(source_rows) >= tokens_on_device.shape[0]):
                raise ValueError("token ids on the device: a row outside the step or outside the sampled tokens")
            if tokens_on_device.dtype != torch.int32 or tokens_on_device.dim() != 1:
                raise ValueError("token ids on the device must be int32 [R]")
            source[:num_device_ids] = np.asarray(source_rows, dtype=np.int32)
            dest[:num_device_ids] = np.asarray(dest_rows, dtype=np.int32)
        put("source", source, b)
        put("dest", dest, b)
        max_kv: List[int] = []
        max_kv_portions: List[int] = []
        decode_prefix = next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens))
        for g, group in enumerate(cache.groups):
            kv = np.ones(b, dtype=np.int32)
            slot_map = np.zeros(t, dtype=np.int32)
            tables = np.zeros((b, width), dtype=np.int32)
            for i, e in enumerate(entries):
                table = e.seq.table_arrays()[g]
                n = q_lens[i]
                end = e.start + n
                if len(table) * page < end:
                    raise ValueError(f"entry {i}: its block table covers {len(table) * page} tokens but the step reaches {end}")
                tables[i, : len(table)] = table
                kv[i] = end
                if n == 1:
                    slot_map[cu[i]] = int(table[e.start // page]) * page + e.start % page
                else:
                    pos = np.arange(e.start, end, dtype=np.int64)
                    slot_map[cu[i]:cu[i + 1]] = table[pos // page].astype(np.int64) * page + pos % page
            put(f"kv{g}", kv, b)
            put(f"slot{g}", slot_map, t)
            put(f"bt{g}", tables, b * width)
            max_kv.append(int(kv.max()))
            max_kv_portions.append(int(kv[decode_prefix:].max()) if decode_prefix < b else 0)

        device[:offset].copy_(self._host[index][:offset], non_blocking=True)
        if self._events[index] is not None:
            self._events[index].record()
            self._used[index] = True

        def view(name: str) -> torch.Tensor:
            lo, n = sections[name]
            return device[lo:lo + n]

        if num_device_ids:
            ops.place_tokens(view("ids"), view("dest"), view("source"), device_ids[0], num_device_ids)

        groups = [
            GroupBatch(
                block_tables=view(f"bt{g}").view(b, width),
                slot_mapping=view(f"slot{g}"),
                kv_lens=view(f"kv{g}"),
                max_kv_len=max_kv[g],
                max_kv_len_of_portions=max_kv_portions[g],
            )
            for g in range(len(cache.groups))
        ]
        return StepContext(
            ops=ops, dtype=dtype, device=self.device, num_tokens=t, num_seqs=b,
            token_ids=view("ids"), positions=view("positions"), cu_q=view("cu"), slots=view("slots"),
            rows=view("rows") if r else None,
            q_lens=q_lens, starts=starts, max_q_len=max(q_lens), all_decode=max(q_lens) == 1,
            groups=groups, workspace=workspace, cache=cache,
            decode_prefix=decode_prefix,
        )
