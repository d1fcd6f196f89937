"""The cache manager: page pools per group of layers, block tables per request, state slots.

Every schedule entry of a model states what its mixer needs (``PagedNeed``, ``StateNeed``
or nothing).  Entries with equal paged needs form a *group*: one pool of pages, one
allocator, one block table per request; page ``p`` of a group addresses page ``p`` of
every entry in it (the reference has exactly one such group for all layers,
``src/paged_kv_cache.py:51-55``).  A group whose need has a window gives pages back as soon
as every key in them lies behind the window of all queries still to come.  Entries with
a ``StateNeed`` get one row per request in fixed-size tensors, indexed by the request's
*slot* (the reference's ``seq_index``, ``engine/scheduler.py:58,113-129``); slot rows are zeroed
when a request takes the slot.

What a page holds is the need's to say (``PagedNeed.tensors``: names, shapes per page and
dtypes): per entry of a group every named tensor is ``[pages, *shape of one page]``, with the
page size where the shape says ``PAGE``.  The manager knows nothing of keys or values.

Growth rule per group (reference ``src/block_manager.py:74-99``): a request that has
``num_computed`` tokens in the cache and is given ``n`` more needs
``ceil((num_computed + n) / page_size)`` table entries.  All groups grow together or
not at all.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import PAGE, PagedNeed, StateNeed
from .allocator import NULL_PAGE, PoolExhausted, PageAllocator
from .prefix import PrefixCache


@dataclass
class SequenceCache:
    """What one live request holds: a block table per group and (always) a slot."""

    slot: int
    tables: List[List[int]]
    released: List[int]  # per group: number of leading table entries already given back
    version: int = 0  # counts the changes of ``tables``: whoever changes a table in place adds one
    published: int = 0  # leading pages that are nodes of the prefix cache (matched at admission or published since)
    publishing: bool = True  # false once another request's page stood where this one's would have gone

    def table_arrays(self) -> List[np.ndarray]:
        """The block tables as int32 arrays, converted again only after a change (see ``version``)."""
        if self._arrays_version != self.version or self._arrays is None:
            self._arrays = [np.asarray(table, dtype=np.int32) for table in self.tables]
            self._arrays_version = self.version
        return self._arrays

    _arrays: Optional[List[np.ndarray]] = field(default=None, repr=False, compare=False)
    _arrays_version: int = field(default=-1, repr=False, compare=False)


class PageGroup:
    def __init__(self, need: PagedNeed, entries: List[int], num_pages: int, page_size: int, dtype: torch.dtype, device, allocate_tensors: bool,
                 scatter_pages: bool = False) -> None:
        self.need = need
        self.entries = list(entries)
        self.page_size = int(page_size)
        self.allocator = PageAllocator(num_pages, scatter=scatter_pages)
        self.dtype = dtype
        # name -> (shape of one page, the dimension of it that runs over the page's tokens, dtype)
        self.layout: Dict[str, Tuple[Tuple[int, ...], int, torch.dtype]] = {}
        for name, shape, tensor_dtype in need.tensors:
            shape = tuple(int(n) for n in shape)
            axis = shape.index(PAGE)
            self.layout[name] = (shape[:axis] + (self.page_size,) + shape[axis + 1:], axis, tensor_dtype or dtype)
        # name -> [entries of the group, pages, *shape of one page]
        self.tensors: Dict[str, torch.Tensor] = {}
        if allocate_tensors:
            for name, (shape, _, tensor_dtype) in self.layout.items():
                self.tensors[name] = torch.zeros((len(entries), num_pages, *shape), dtype=tensor_dtype, device=device)

    def bytes_per_page(self) -> int:
        per_entry = 0
        for shape, _, tensor_dtype in self.layout.values():
            numel = 1
            for n in shape:
                numel *= n
            per_entry += numel * torch.empty((), dtype=tensor_dtype).element_size()
        return per_entry * len(self.entries)

    def table_entries_for(self, num_tokens: int) -> int:
        return (num_tokens + self.page_size - 1) // self.page_size

    def first_needed_page(self, num_computed: int) -> int:
        """Index of the first table entry a query at position >= num_computed may still read."""
        if self.need.window is None:
            return 0
        first_key = max(0, num_computed - self.need.window + 1)
        return first_key // self.page_size


class StateSlots:
    """Rows of fixed-size state, one per live request, plus one spare row for padded batch rows."""

    def __init__(self, needs: Dict[int, StateNeed], max_num_seqs: int, dtype: torch.dtype, device, allocate_tensors: bool) -> None:
        self.max_num_seqs = int(max_num_seqs)
        self.pad_slot = self.max_num_seqs
        self._free: List[int] = list(range(self.max_num_seqs - 1, -1, -1))
        self._held = [False] * self.max_num_seqs
        self.tensors: Dict[int, Dict[str, torch.Tensor]] = {}
        if allocate_tensors:
            for entry, need in needs.items():
                self.tensors[entry] = {
                    name: torch.zeros((self.max_num_seqs + 1, *shape), dtype=dt or dtype, device=device)
                    for name, shape, dt in need.tensors
                }

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> Optional[int]:
        if not self._free:
            return None
        slot = self._free.pop()
        self._held[slot] = True
        for tensors in self.tensors.values():
            for tensor in tensors.values():
                tensor[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        if not 0 <= slot < self.max_num_seqs or not self._held[slot]:
            raise RuntimeError(f"slot {slot} is not held")
        self._held[slot] = False
        self._free.append(slot)

    def assert_consistent(self) -> None:
        if len(set(self._free)) != len(self._free):
            raise AssertionError("slot free list contains duplicates")
        for slot in range(self.max_num_seqs):
            if self._held[slot] == (slot in self._free):
                raise AssertionError(f"slot {slot}: held={self._held[slot]} but free={slot in self._free}")


@dataclass
class PagedView:
    """What a mixer with a ``PagedNeed`` is handed for one schedule entry and one step: its page tensors by the names its
    need gave them, each ``[pages, *shape of one page]``."""

    tensors: Dict[str, torch.Tensor]
    block_size: int
    batch: object  # engine.batch.GroupBatch of this step


@dataclass
class StateView:
    tensors: Dict[str, torch.Tensor]


class CacheManager:
    def __init__(
        self,
        needs: Sequence[object],
        page_size: int,
        num_pages: int,
        max_num_seqs: int,
        dtype: torch.dtype,
        device="cpu",
        max_model_len: Optional[int] = None,
        allocate_tensors: bool = True,
        prefix_caching: bool = False,
        scatter_pages: bool = False,
    ) -> None:
        if page_size <= 0 or (page_size & (page_size - 1)) != 0:
            raise ValueError(f"page_size must be a power of two, got {page_size}")
        self.page_size = int(page_size)
        self.dtype = dtype
        self.device = torch.device(device)
        self.groups: List[PageGroup] = []
        self.entry_group: Dict[int, Tuple[int, int]] = {}
        by_need: Dict[PagedNeed, List[int]] = {}
        state_needs: Dict[int, StateNeed] = {}
        for entry, need in enumerate(needs):
            if isinstance(need, PagedNeed):
                by_need.setdefault(need, []).append(entry)
            elif isinstance(need, StateNeed):
                state_needs[entry] = need
            elif need is not None:
                raise TypeError(f"schedule entry {entry}: unknown cache need {need!r}")
        for need, entries in by_need.items():
            index = len(self.groups)
            self.groups.append(PageGroup(need, entries, num_pages, page_size, dtype, self.device, allocate_tensors, scatter_pages))
            for position, entry in enumerate(entries):
                self.entry_group[entry] = (index, position)
        self.state = StateSlots(state_needs, max_num_seqs, dtype, self.device, allocate_tensors)
        self.state_entries = set(state_needs)
        capacity = (num_pages - 1) * page_size
        self.max_model_len = min(max_model_len, capacity) if max_model_len else capacity
        self.max_pages_per_seq = (self.max_model_len + page_size - 1) // page_size
        # Prefixes are shared only where a request holds every page of its past: no window gives pages back early,
        # and no state of fixed size stands for tokens that a sharer would skip.
        self.prefix: Optional[PrefixCache] = None
        if prefix_caching and self.supports_prefix_caching():
            self.prefix = PrefixCache([group.allocator for group in self.groups], page_size)

    def supports_prefix_caching(self) -> bool:
        return bool(self.groups) and not self.state_entries and all(group.need.window is None for group in self.groups)

    # -- sizes --------------------------------------------------------------------------
    def bytes_per_page(self) -> int:
        return sum(group.bytes_per_page() for group in self.groups)

    @property
    def num_total_pages(self) -> int:
        return min((g.allocator.num_total for g in self.groups), default=0)

    def num_free_pages(self) -> int:
        """Free pages of the tightest group."""
        return min((g.allocator.num_free for g in self.groups), default=1 << 30)

    def num_reclaimable_pages(self) -> int:
        """Pages (per group) that only the prefix cache holds: they are given back when a request needs them."""
        return self.prefix.num_reclaimable if self.prefix is not None else 0

    def num_available_pages(self) -> int:
        """Free plus reclaimable pages of the tightest group: what bounds growth (reference
        ``src/block_manager.py:34-35``)."""
        return self.num_free_pages() + self.num_reclaimable_pages()

    def num_used_pages(self) -> int:
        return max((g.allocator.num_used for g in self.groups), default=0)

    # -- sequences ----------------------------------------------------------------------
    def new_sequence(self) -> Optional[SequenceCache]:
        slot = self.state.acquire()
        if slot is None:
            return None
        return SequenceCache(slot=slot, tables=[[] for _ in self.groups], released=[0 for _ in self.groups])

    def pages_to_append(self, seq: SequenceCache, num_computed: int, num_new: int) -> List[int]:
        return [
            max(0, group.table_entries_for(num_computed + num_new) - len(table))
            for group, table in zip(self.groups, seq.tables)
        ]

    def can_append(self, seq: SequenceCache, num_computed: int, num_new: int) -> bool:
        if num_computed + num_new > self.max_model_len:
            return False
        extra = self.pages_to_append(seq, num_computed, num_new)
        reclaimable = self.num_reclaimable_pages()
        return all(n <= g.allocator.num_free + reclaimable for n, g in zip(extra, self.groups))

    def max_new_tokens(self, seq: Optional[SequenceCache], num_computed: int, headroom_pages: Optional[int] = None) -> int:
        """How many tokens past ``num_computed`` fit in the pages the request has plus the free ones
        (less ``headroom_pages`` held back), capped by ``max_model_len`` (reference ``engine/scheduler.py:210-219``)."""
        limit = self.max_model_len - num_computed
        reclaimable = self.num_reclaimable_pages()
        for index, group in enumerate(self.groups):
            have = len(seq.tables[index]) if seq is not None else 0
            free = group.allocator.num_free + reclaimable
            free = free if headroom_pages is None else min(free, headroom_pages)
            pages = min(have + max(0, free), self.max_pages_per_seq)
            limit = min(limit, pages * group.page_size - num_computed)
        return max(0, limit)

    def append(self, seq: SequenceCache, num_computed: int, num_new: int) -> bool:
        """Grows every group's table to cover ``num_computed + num_new`` tokens; all or nothing."""
        if num_computed + num_new > self.max_model_len:
            return False
        extra = self.pages_to_append(seq, num_computed, num_new)
        reclaimable = self.num_reclaimable_pages()
        for n, group, table in zip(extra, self.groups, seq.tables):
            if n > group.allocator.num_free + reclaimable or len(table) + n > self.max_pages_per_seq:
                return False
        short = max((n - group.allocator.num_free for n, group in zip(extra, self.groups)), default=0)
        if short > 0:
            self.prefix.evict(short)  # (an evicted node gives back one page in every group)
            if any(n > group.allocator.num_free for n, group in zip(extra, self.groups)):
                return False
        for n, group, table in zip(extra, self.groups, seq.tables):
            if n:
                table.extend(group.allocator.take_many(n))
                seq.version += 1
        return True

    # -- shared prefixes -----------------------------------------------------------------------
    def match_prefix(self, seq: SequenceCache, tokens: Sequence[int]) -> int:
        """For a request that holds nothing yet: puts the published pages of the longest known prefix of ``tokens``
        into its tables and returns how many tokens they cover.  At least one token is left to compute, so that there
        is a row to take logits from (reference ``src/block_manager.py:52-72``)."""
        if self.prefix is None or any(seq.tables):
            return 0
        nodes = self.prefix.match(tokens, max_pages=min((len(tokens) - 1) // self.page_size, self.max_pages_per_seq))
        for node in nodes:
            for index, (group, page) in enumerate(zip(self.groups, node.pages)):
                group.allocator.share(page)
                seq.tables[index].append(page)
            self.prefix.page_taken(node.pages[0])
        if nodes:
            seq.version += 1
        seq.published = len(nodes)
        seq.publishing = True
        return len(nodes) * self.page_size

    def publish(self, seq: SequenceCache, tokens: Sequence[int], num_computed: int) -> None:
        """Offers the pages that the request has filled since the last call to later requests (reference
        ``src/block_manager.py:101-112``).  ``tokens[:num_computed]`` are in the cache."""
        if self.prefix is None or not seq.publishing:
            return
        whole = min(num_computed // self.page_size, min(len(table) for table in seq.tables))
        if whole > seq.published:
            seq.published, seq.publishing = self.prefix.publish(tokens, seq.tables, seq.published, whole)

    def release_behind_window(self, seq: SequenceCache, num_computed: int) -> int:
        """Gives back pages no later query can read; their table entries become the null page."""
        given_back = 0
        for index, group in enumerate(self.groups):
            first = min(group.first_needed_page(num_computed), len(seq.tables[index]))
            table = seq.tables[index]
            for position in range(seq.released[index], first):
                if table[position] != NULL_PAGE:
                    group.allocator.drop(table[position])
                    table[position] = NULL_PAGE
                    seq.version += 1
                    given_back += 1
            seq.released[index] = max(seq.released[index], first)
        return given_back

    def free_pages(self, seq: SequenceCache) -> None:
        for index in range(len(self.groups) - 1, -1, -1):  # (group 0 last: its count tells the prefix cache who holds a node)
            group = self.groups[index]
            for page in seq.tables[index]:  # (in table order, so that the request's last page is the next one handed out)
                if page != NULL_PAGE:
                    group.allocator.drop(page)
                    if index == 0 and self.prefix is not None:
                        self.prefix.page_dropped(page)
            seq.tables[index] = []
            seq.released[index] = 0
        seq.published = 0
        seq.publishing = True
        seq.version += 1

    def free_sequence(self, seq: SequenceCache) -> None:
        self.free_pages(seq)
        if seq.slot is not None and seq.slot >= 0:
            self.state.release(seq.slot)
            seq.slot = -1

    def slot_for(self, seq: SequenceCache, group_index: int, token_index: int) -> int:
        page = seq.tables[group_index][token_index // self.page_size]
        return page * self.page_size + token_index % self.page_size

    # -- views handed to the mixers ----------------------------------------------------------
    def view(self, entry: int, group_batches: Sequence[object]):
        if entry in self.entry_group:
            g, position = self.entry_group[entry]
            group = self.groups[g]
            return PagedView({name: tensor[position] for name, tensor in group.tensors.items()}, group.page_size, group_batches[g])
        if entry in self.state_entries:
            return StateView(self.state.tensors[entry])
        return None

    def gather_sequence(self, entry: int, seq: SequenceCache, length: int) -> Dict[str, torch.Tensor]:
        """What the first ``length`` tokens of one request hold in the entry's page tensors, token by token: per tensor
        ``[length, *shape of one page without its token dimension]`` (a debugging aid, reference
        ``src/paged_kv_cache.py:125-150``)."""
        g, position = self.entry_group[entry]
        group = self.groups[g]
        index = torch.arange(length)
        pages = torch.tensor(seq.tables[g], dtype=torch.long)[index // group.page_size].to(self.device)
        offsets = (index % group.page_size).to(self.device)
        out = {}
        for name, tensor in group.tensors.items():
            axis = group.layout[name][1]
            per_page = tensor[position].movedim(1 + axis, 1)  # [pages, page_size, ...]
            out[name] = per_page[pages, offsets]
        return out

    # -- invariants ---------------------------------------------------------------------
    def assert_consistent(self, live: Sequence[SequenceCache] = ()) -> None:
        """Allocator invariants, and: every used page is held by the live requests that list it and, if published, once
        more by the prefix cache; no request lists a page twice; no page is lost."""
        self.state.assert_consistent()
        if self.prefix is not None:
            self.prefix.assert_consistent()
        for index, group in enumerate(self.groups):
            group.allocator.verify()
            holders: Dict[int, int] = {}
            for seq in live:
                pages = [p for p in seq.tables[index] if p != NULL_PAGE]
                if len(set(pages)) != len(pages):
                    raise AssertionError(f"group {index}: a request lists a page twice")
                for page in pages:
                    holders[page] = holders.get(page, 0) + 1
            published = set()
            if self.prefix is not None:
                published = {node.pages[index] for node in self.prefix._node_of.values()}
            if self.prefix is None and any(count != 1 for count in holders.values()):
                raise AssertionError(f"group {index}: a page is held twice")
            for page in set(holders) | published:
                expected = holders.get(page, 0) + (page in published)
                if group.allocator.holders(page) != expected:
                    raise AssertionError(f"group {index}: page {page} has refcount {group.allocator.holders(page)}, expected {expected}")
            if live is not None and len(set(holders) | published) != group.allocator.num_used:
                raise AssertionError(f"group {index}: {group.allocator.num_used} pages used but {len(set(holders) | published)} accounted for (a page was lost)")


def pages_that_fit(bytes_per_page: int, free_bytes: int, utilization: float, reserve_bytes: int) -> int:
    """Pool size from free memory (reference ``src/paged_kv_cache.py:183-194``)."""
    budget = int(free_bytes * utilization) - reserve_bytes
    if budget <= 0:
        raise RuntimeError("not enough free GPU memory for a cache pool")
    pages = budget // max(1, bytes_per_page)
    if pages < 2:
        raise RuntimeError("free GPU memory is too small to hold even one cache page")
    return int(pages)
