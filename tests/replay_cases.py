"""Traces for the replay tests: the same requests whole, with the last 32 tokens one by one, in portions of
changing size, and mixed with other requests in a pool so small that pages are used again.  A trace is a
list of step records in the format ``bin/trace_run`` reads."""
from __future__ import annotations

import random
from typing import Dict, List, Tuple

import numpy as np
import torch

from helpers import random_tokens
from plain_qwen2 import qwen2_logits


def request_set(vocab: int, lengths, seed: int) -> Dict[str, List[int]]:
    return {f"r{i}": random_tokens(vocab, n, seed * 100 + i) for i, n in enumerate(lengths)}


def expected_logits(config, weights, requests) -> Dict[str, torch.Tensor]:
    return {rid: qwen2_logits(config, weights, tokens) for rid, tokens in requests.items()}


def whole(requests) -> List[dict]:
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def tail_one_by_one(requests, tail: int = 32) -> List[dict]:
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": [rid] if i == len(toks) - 1 else []})
    return steps


def changing_portions(requests, sizes=(7, 2, 5, 3, 11, 2, 16, 1, 2, 9)) -> List[dict]:
    steps = []
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}],
                          "end": [rid] if at + n == len(toks) else []})
            at += n
    return steps


def mixed(requests, seed: int, max_live: int = 4, preempt: Tuple[str, ...] = ()) -> List[dict]:
    """Up to ``max_live`` requests at a time; every step gives each live request (sometimes leaving one out) a
    portion of 1..16 tokens, so portions of some sit beside single tokens of others; a request that is done
    ends and the next one starts in its pages.  A request named in ``preempt`` is ended once when it is about half
    way (what it holds goes back), waits while the others go on in its pages, and is then fed again from its first
    token under the same id: what a scheduler does to a preempted request (reference ``engine/scheduler.py:136-146``)."""
    rng = random.Random(seed)
    waiting = list(requests)
    live: Dict[str, int] = {}
    to_preempt = set(preempt)
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.15:
                continue  # left out of this step; it goes on later
            at = live[rid]
            left = len(requests[rid]) - at
            n = min(left, rng.choice([1, 1, 1, 2, 2, 3, 5, 8, 16]))
            entries.append({"id": rid, "tokens": requests[rid][at:at + n], "want": list(range(n))})
            live[rid] = at + n
            if at + n == len(requests[rid]):
                end.append(rid)
            elif rid in to_preempt and 2 * (at + n) >= len(requests[rid]):
                to_preempt.discard(rid)
                end.append(rid)
                waiting.insert(min(1, len(waiting)), rid)  # behind the next newcomer, which takes over its pages first
        if not entries:
            continue
        for rid in end:
            del live[rid]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    assert not to_preempt, "a request to preempt never got half way"
    return steps


def tokens_needed(trace: List[dict], round_to: int) -> int:
    """The most tokens live requests hold at any time, each request's count rounded up to ``round_to``."""
    held: Dict[str, int] = {}
    most = 0
    for record in trace:
        for entry in record["entries"]:
            held[entry["id"]] = held.get(entry["id"], 0) + len(entry["tokens"])
        most = max(most, sum((n + round_to - 1) // round_to * round_to for n in held.values()))
        for rid in record["end"]:
            held.pop(rid, None)
    return most


def collect(trace: List[dict], outputs: Dict[int, np.ndarray], requests) -> Dict[str, torch.Tensor]:
    """Puts the logits of every step back in order per request: {id: [len, vocab]}."""
    rows: Dict[str, Dict[int, np.ndarray]] = {rid: {} for rid in requests}
    at: Dict[str, int] = {rid: 0 for rid in requests}
    for record in trace:
        out = outputs.get(record["step"])
        row = 0
        for entry in record["entries"]:
            for w in entry["want"]:
                rows[entry["id"]][at[entry["id"]] + w] = out[row]  # (a request that starts over overwrites its first run)
                row += 1
            at[entry["id"]] += len(entry["tokens"])
        assert out is None or row == out.shape[0]
        for rid in record["end"]:
            at[rid] = 0  # ended: if it comes again it starts from its first token
    result = {}
    for rid, found in rows.items():
        assert sorted(found) == list(range(len(requests[rid]))), f"{rid}: positions {sorted(found)[:5]}..."
        result[rid] = torch.from_numpy(np.stack([found[p] for p in range(len(requests[rid]))]))
    return result


def first_runs(trace: List[dict], outputs: Dict[int, np.ndarray], requests) -> Dict[str, Dict[int, np.ndarray]]:
    """For requests that a trace ends half way and feeds again: the logits of the first run, {id: {position: row}}."""
    rows: Dict[str, Dict[int, np.ndarray]] = {}
    at: Dict[str, int] = {rid: 0 for rid in requests}
    for record in trace:
        out = outputs.get(record["step"])
        row = 0
        for entry in record["entries"]:
            for w in entry["want"]:
                rows.setdefault(entry["id"], {}).setdefault(at[entry["id"]] + w, out[row])
                row += 1
            at[entry["id"]] += len(entry["tokens"])
        for rid in record["end"]:
            at[rid] = 0
    return rows


def run_trace(replayer, trace: List[dict]) -> Dict[int, np.ndarray]:
    outputs = {}
    for record in trace:
        out = replayer.step(record)
        if out is not None:
            outputs[record["step"]] = out
    assert not replayer.live, "a trace must end every request it starts"
    replayer.cache.assert_consistent([])
    assert replayer.cache.num_used_pages() == 0
    return outputs
