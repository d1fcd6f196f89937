"""Sharing of prompt prefixes between requests: a trie of FULL pages keyed by their tokens.

What it does is the reference's ``RadixCache`` plus the part of ``BlockSpaceManager`` that drives it
(``src/radix_cache.py:53-226``, ``src/block_manager.py:52-72,101-112``): when a request is admitted, the longest
run of whole pages at the start of its tokens that some earlier request has computed is found, those pages are put
into its block tables (reference counted, never written again) and only the rest is computed; after every step the
pages that a request has filled are published; a published page that no request holds stays until the pool runs
short and then goes, least recently used first.  Only full pages are shared, so nothing is ever copied.

Differences in construction.  A node holds one page per page group (groups grow together, so one trie serves all
of them).  Children are found by their tokens themselves, a tuple of ``page_size`` ints under the parent node, so
there is no hash to collide.  A request publishes a page only below a node whose page it holds itself: when another
request has published the same tokens first with a page of its own, this request stops publishing (its further
pages stay private).  Hence every holder of a node's page also holds the pages of all its ancestors, a node's
reference count is never below that of a descendant, and the pages that can be had back by eviction are exactly
those of the nodes that nobody but the trie holds: ``num_reclaimable`` is kept as a counter and is exact, where the
reference counts unheld leaves only (``src/radix_cache.py:85-90``).
"""
from __future__ import annotations

import heapq
from typing import Dict, List, Optional, Sequence, Tuple

from .allocator import PageAllocator


class PrefixNode:
    __slots__ = ("tokens", "pages", "parent", "children", "stamp", "alive")

    def __init__(self, tokens: Tuple[int, ...], pages: Tuple[int, ...], parent: Optional["PrefixNode"]) -> None:
        self.tokens = tokens
        self.pages = pages  # one page per group
        self.parent = parent
        self.children: Dict[Tuple[int, ...], "PrefixNode"] = {}
        self.stamp = 0
        self.alive = True


class PrefixCache:
    def __init__(self, allocators: Sequence[PageAllocator], page_size: int) -> None:
        if not allocators:
            raise ValueError("a prefix cache needs at least one page group")
        self.allocators = list(allocators)
        self.page_size = int(page_size)
        self.root = PrefixNode((), (), None)
        self._node_of: Dict[int, PrefixNode] = {}  # by the node's page in group 0
        self._clock = 0
        self._heap: List[Tuple[int, int, PrefixNode]] = []  # (stamp, tie-break, leaf nobody holds); entries go stale
        self._pushes = 0
        self.num_reclaimable = 0  # nodes whose pages only the trie holds
        self.num_queries = 0
        self.num_hits = 0
        self.num_queried_tokens = 0
        self.num_matched_tokens = 0

    # -- sizes --------------------------------------------------------------------------
    @property
    def num_nodes(self) -> int:
        return len(self._node_of)

    @property
    def hit_rate(self) -> float:
        return 0.0 if self.num_queried_tokens == 0 else self.num_matched_tokens / self.num_queried_tokens

    def holds(self, first_group_page: int) -> bool:
        return first_group_page in self._node_of

    # -- bookkeeping ----------------------------------------------------------------------
    def _held_by_requests(self, node: PrefixNode) -> bool:
        return self.allocators[0].holders(node.pages[0]) > 1

    def _touch(self, node: PrefixNode) -> None:
        self._clock += 1
        node.stamp = self._clock
        self._offer(node)

    def _offer(self, node: PrefixNode) -> None:
        """Queues the node for eviction if it is a leaf that no request holds."""
        if node.alive and node is not self.root and not node.children and not self._held_by_requests(node):
            self._pushes += 1
            heapq.heappush(self._heap, (node.stamp, self._pushes, node))

    def page_taken(self, first_group_page: int) -> None:
        """A request has just added its reference to a published page (called after the increment)."""
        node = self._node_of.get(first_group_page)
        if node is not None and self.allocators[0].holders(first_group_page) == 2:
            self.num_reclaimable -= 1

    def page_dropped(self, first_group_page: int) -> None:
        """A request has just given up its reference to a published page (called after the decrement)."""
        node = self._node_of.get(first_group_page)
        if node is not None and self.allocators[0].holders(first_group_page) == 1:
            self.num_reclaimable += 1
            self._offer(node)

    # -- the three operations -----------------------------------------------------------------
    def match(self, tokens: Sequence[int], max_pages: int) -> List[PrefixNode]:
        """The nodes of the longest published run of whole pages at the start of ``tokens``, at most ``max_pages``."""
        whole = min(len(tokens) // self.page_size, max_pages)
        if whole <= 0:
            return []
        self.num_queries += 1
        self.num_queried_tokens += whole * self.page_size
        found: List[PrefixNode] = []
        node = self.root
        for index in range(whole):
            child = node.children.get(tuple(tokens[index * self.page_size:(index + 1) * self.page_size]))
            if child is None:
                break
            found.append(child)
            node = child
        for child in found:
            self._touch(child)
        if found:
            self.num_hits += 1
            self.num_matched_tokens += len(found) * self.page_size
        return found

    def publish(self, tokens: Sequence[int], tables: Sequence[Sequence[int]], first: int, last: int) -> Tuple[int, bool]:
        """Publishes pages ``first .. last - 1`` of a request (whole pages of ``tokens``; ``tables[g]`` is its block table
        in group ``g``); pages before ``first`` are nodes already, with this request's pages.  Returns ``(pages that are
        nodes now, open)``: ``open`` turns false when another request's page stands where this one's would go, and the
        request then publishes no further."""
        node = self.root
        for index in range(first):
            node = node.children[tuple(tokens[index * self.page_size:(index + 1) * self.page_size])]
        for index in range(first, last):
            key = tuple(tokens[index * self.page_size:(index + 1) * self.page_size])
            if any(token < 0 for token in key):
                # a place holder for a token that a step in flight is still drawing: its value is not known, so the page
                # cannot be found by its tokens; it is offered once the value has arrived
                return index, True
            child = node.children.get(key)
            pages = tuple(table[index] for table in tables)
            if child is not None:
                if child.pages != pages:
                    return index, False
            else:
                child = PrefixNode(key, pages, node)
                for allocator, page in zip(self.allocators, pages):
                    allocator.share(page)
                node.children[key] = child
                self._node_of[pages[0]] = child
            self._touch(child)
            node = child
        return last, True

    def evict(self, count: int) -> int:
        """Gives back the pages of up to ``count`` nodes that no request holds, least recently used leaves first."""
        freed = 0
        while freed < count and self._heap:
            stamp, _, node = heapq.heappop(self._heap)
            if not node.alive or node.stamp != stamp or node.children or self._held_by_requests(node):
                continue  # stale: the node is offered again when it can go
            parent = node.parent
            del parent.children[node.tokens]
            del self._node_of[node.pages[0]]
            node.alive = False
            node.parent = None
            for allocator, page in zip(self.allocators, node.pages):
                allocator.drop(page)
            self.num_reclaimable -= 1
            freed += 1
            if parent is not self.root:
                self._offer(parent)
        return freed

    def clear(self) -> int:
        """Drops every node that no request holds; returns how many."""
        return self.evict(len(self._node_of))

    # -- invariants ---------------------------------------------------------------------
    def assert_consistent(self) -> None:
        seen = 0
        unheld = 0
        stack = [self.root]
        while stack:
            node = stack.pop()
            for key, child in node.children.items():
                if child.parent is not node or child.tokens != key or not child.alive:
                    raise AssertionError("prefix trie: a child does not point back at its parent")
                if len(key) != self.page_size or len(child.pages) != len(self.allocators):
                    raise AssertionError("prefix trie: a node of the wrong size")
                if self._node_of.get(child.pages[0]) is not child:
                    raise AssertionError("prefix trie: a reachable node is missing from the page index")
                counts = [allocator.holders(page) for allocator, page in zip(self.allocators, child.pages)]
                if min(counts) < 1 or len(set(counts)) != 1:
                    raise AssertionError(f"prefix trie: pages {child.pages} have reference counts {counts}")
                if node is not self.root and counts[0] > self.allocators[0].holders(node.pages[0]):
                    raise AssertionError("prefix trie: a page is held by more requests than its parent")
                seen += 1
                unheld += counts[0] == 1
                stack.append(child)
        if seen != len(self._node_of):
            raise AssertionError("prefix trie: the page index holds nodes that cannot be reached")
        if unheld != self.num_reclaimable:
            raise AssertionError(f"prefix trie: {unheld} nodes are held by nobody but the count says {self.num_reclaimable}")

    def stats(self) -> Dict[str, float]:
        return {
            "nodes": float(self.num_nodes),
            "reclaimable": float(self.num_reclaimable),
            "queries": float(self.num_queries),
            "hits": float(self.num_hits),
            "queried_tokens": float(self.num_queried_tokens),
            "matched_tokens": float(self.num_matched_tokens),
            "hit_rate": self.hit_rate,
        }
