"""The scheduler's decisions, driven without a model: what a step would compute is simulated."""
import pytest
import torch

from velox_amd.cache import CacheManager
from velox_amd.engine.request import FinishReason, Request, RequestStatus
from velox_amd.engine.scheduler import Scheduler, SchedulerConfig
from velox_amd.parts import kv_pages
from velox_amd.sampling import SamplingParams


def make(pages=33, page=4, seqs=4, budget=16, chunk=8, max_len=128, watermark=0.01):
    cache = CacheManager([kv_pages(1, 16)], page, pages, seqs, torch.float32, "cpu", max_model_len=max_len, allocate_tensors=False)
    return Scheduler(cache, SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=budget, max_prefill_chunk_size=chunk, max_model_len=max_len, watermark=watermark))


def request(rid, prompt_len, max_tokens=4):
    return Request(rid, list(range(1, prompt_len + 1)), SamplingParams(temperature=0.0, max_tokens=max_tokens, ignore_eos=True))


def run_step(s, out):
    """What the engine does after a forward: advance, append a token to rows that completed their tokens."""
    scheduled = out.requests()
    assert len({id(r) for r in scheduled}) == len(scheduled), "a request is in a step twice"
    assert all(r.cache is not None and r in s.running for r in scheduled), "a scheduled request has no pages"
    assert not any(r in scheduled for r in out.preempted if r.cache is None)
    sampled = list(out.decodes)
    for r in out.decodes:
        s.advance(r, 1)
    for portion in out.portions:
        assert portion.start == portion.request.num_computed_tokens
        s.advance(portion.request, portion.count)
        if portion.completes:
            sampled.append(portion.request)
    for r in sampled:
        r.record_token(1000 + len(r.output_token_ids))
        reason = r.stop_reason(r.output_token_ids[-1], frozenset())
        if reason:
            r.finish(reason)


def portions(out):
    return [(p.request.request_id, p.count) for p in out.portions]


def test_prompt_is_cut_under_budget_and_chunk_then_decodes_first():
    s = make(budget=16, chunk=8)
    a, b = request("a", 19), request("b", 5)
    s.add_request(a)
    s.add_request(b)
    out = s.schedule()
    assert portions(out) == [("a", 8), ("b", 5)] and (out.count_of(a), out.count_of(b)) == (8, 5)
    assert out.num_tokens == 13 and not out.decodes
    run_step(s, out)
    assert a.status is RequestStatus.RUNNING_PREFILL and b.status is RequestStatus.RUNNING_DECODE and b.output_token_ids == [1000]
    out = s.schedule()
    assert [r.request_id for r in out.decodes] == ["b"] and portions(out) == [("a", 8)] and out.count_of(b) == 1
    run_step(s, out)
    out = s.schedule()
    assert out.count_of(a) == 3 and a.num_computed_tokens == 16 and out.portions[0].start == 16 and out.portions[0].completes
    run_step(s, out)
    assert a.status is RequestStatus.RUNNING_DECODE and a.output_token_ids == [1000]


def test_budget_counts_decodes_before_prompts():
    s = make(budget=6, chunk=6, seqs=4)
    for i in range(3):
        s.add_request(request(f"d{i}", 2, max_tokens=20))
    run_step(s, s.schedule())
    s.add_request(request("p", 30))
    out = s.schedule()
    assert len(out.decodes) == 3 and portions(out) == [("p", 3)]  # 6 - 3 decodes


def test_finish_frees_pages_at_the_next_schedule_and_reasons():
    s = make()
    a = request("a", 6, max_tokens=2)
    s.add_request(a)
    run_step(s, s.schedule())
    run_step(s, s.schedule())
    assert a.finished and a.finish_reason is FinishReason.LENGTH and len(a.output_token_ids) == 2
    assert s.cache.num_used_pages() > 0 and s.has_work()
    out = s.schedule()
    assert out.is_empty() and s.cache.num_used_pages() == 0 and not s.has_work() and s.num_finished == 1
    s.cache.assert_consistent([])
    stop = Request("s", [1, 2, 3], SamplingParams(max_tokens=9, stop_token_ids=[77]))
    assert stop.stop_reason(77, frozenset()) is FinishReason.STOP and stop.stop_reason(5, frozenset({5})) is FinishReason.STOP
    assert stop.stop_reason(6, frozenset({5})) is None
    assert Request("i", [1], SamplingParams(max_tokens=9, ignore_eos=True)).stop_reason(5, frozenset({5})) is None


def test_limits_are_refused_at_add():
    s = make(max_len=32)
    with pytest.raises(ValueError):
        s.add_request(request("long", 32))
    with pytest.raises(ValueError):
        s.add_request(request("long2", 30, max_tokens=3))
    s.add_request(request("fits", 30, max_tokens=2))
    with pytest.raises(ValueError):
        s.add_request(request("fits", 3))
    with pytest.raises(ValueError):
        Request("empty", [], SamplingParams())
    # the pool bounds the length too: 8 usable pages of 4
    small = make(pages=9, max_len=4096)
    assert small.config.max_model_len == 32


def test_admission_waits_for_slots_and_keeps_a_watermark_first_come_first_served():
    s = make(pages=11, seqs=2, budget=64, chunk=64, watermark=0.2)  # 10 usable pages, watermark 2
    for rid, n in (("a", 12), ("b", 20), ("c", 4)):
        s.add_request(request(rid, n, max_tokens=2))
    out = s.schedule()
    # a takes 3 pages; b wants 5 of the 7 left, headroom 7 - 2 = 5: fits; c finds no slot
    assert portions(out) == [("a", 12), ("b", 20)] and s.num_waiting == 1
    run_step(s, out)
    s2 = make(pages=11, seqs=4, budget=64, chunk=64, watermark=0.2)
    for rid, n in (("a", 12), ("b", 28), ("c", 4)):
        s2.add_request(request(rid, n, max_tokens=2))
    out = s2.schedule()
    # b needs 7 pages, headroom is 5: it gets a 20-token portion (5 pages); c then sees headroom 0 and waits behind it
    assert portions(out) == [("a", 12), ("b", 20)]
    assert [r.request_id for r in s2.waiting] == ["c"]


def test_decode_out_of_pages_preempts_the_newest_and_recomputes_it():
    s = make(pages=7, page=4, seqs=3, budget=32, chunk=32, watermark=0.01)  # 6 usable pages
    a, b = request("a", 8, max_tokens=12), request("b", 8, max_tokens=12)
    s.add_request(a)
    s.add_request(b)
    run_step(s, s.schedule())  # 2 pages each, one token sampled each
    assert s.cache.num_free_pages() == 2
    run_step(s, s.schedule())  # both decode: position 8 needs a third page each
    assert s.cache.num_free_pages() == 0 and not s.num_preemptions
    for _ in range(3):
        run_step(s, s.schedule())  # positions 9, 10, 11 fit
    out = s.schedule()  # position 12: a needs a 4th page, none free: b (the newest) is preempted
    assert [r.request_id for r in out.preempted] == ["b"] and [r.request_id for r in out.decodes] == ["a"]
    assert b.num_preemptions == 1 and s.num_preemptions == 1 and len(b.output_token_ids) == 5  # its tokens are kept
    # the same scheduling decision admits it again from the front of the queue, from position 0, with what fits
    assert b.status is RequestStatus.RUNNING_PREFILL and b.num_computed_tokens == 0
    assert portions(out) == [("b", 4)] and out.portions[0].start == 0  # 2 pages free, 1 held back
    run_step(s, out)
    s.cache.assert_consistent([a.cache, b.cache])
    # its recomputation covers prompt and generated tokens (13), then it decodes on: no token is lost or sampled twice
    guard = 0
    while b.status is not RequestStatus.RUNNING_DECODE:
        run_step(s, s.schedule())
        guard += 1
        assert guard < 50
    assert len(b.output_token_ids) == 6 and b.num_computed_tokens == 13
    while s.has_work():
        run_step(s, s.schedule())
    assert len(a.output_token_ids) == 12 and len(b.output_token_ids) == 12 and s.cache.num_used_pages() == 0
    assert a.output_token_ids == b.output_token_ids == [1000 + i for i in range(12)]
    s.cache.assert_consistent([])


def test_oldest_prefill_may_evict_newer_requests_but_a_newer_prefill_waits():
    s = make(pages=6, page=4, seqs=3, budget=12, chunk=8, watermark=0.01)  # 5 usable pages
    a, b = request("a", 18, max_tokens=2), request("b", 12, max_tokens=2)
    s.add_request(a)
    s.add_request(b)
    out = s.schedule()  # a: 8 tokens, 2 pages; b: the 4 tokens the budget leaves, 1 page
    assert portions(out) == [("a", 8), ("b", 4)]
    run_step(s, out)
    out = s.schedule()  # a takes the last 2 free pages; b finds none and, not being the oldest, just waits
    assert portions(out) == [("a", 8)] and not out.preempted
    run_step(s, out)
    out = s.schedule()  # a needs one more page: as the oldest prefill it evicts b, the newest request
    assert [r.request_id for r in out.preempted] == ["b"] and portions(out) == [("a", 2)]
    assert b.num_preemptions == 1 and b.num_computed_tokens == 0 and b.status is RequestStatus.PREEMPTED and s.waiting[0] is b
    run_step(s, out)
    while s.has_work():
        run_step(s, s.schedule())
    assert len(a.output_token_ids) == 2 and len(b.output_token_ids) == 2 and s.cache.num_used_pages() == 0


def test_two_requests_that_cannot_both_fit_still_finish():
    s = make(pages=5, page=4, seqs=2, budget=32, chunk=32, watermark=0.01)  # 4 usable pages; a alone needs all of them
    a, b = request("a", 8, max_tokens=8), request("b", 7, max_tokens=8)
    s.add_request(a)
    s.add_request(b)
    guard = 0
    while s.has_work():
        out = s.schedule()
        for victim in out.preempted:
            assert victim is b  # the older request never yields to the newer one
        run_step(s, out)
        s.cache.assert_consistent([r.cache for r in s.running if r.cache is not None])
        guard += 1
        assert guard < 200
    assert s.num_preemptions >= 1 and b.num_preemptions >= 1 and a.num_preemptions == 0
    assert a.output_token_ids == b.output_token_ids == [1000 + i for i in range(8)]
    s.cache.assert_consistent([])


def test_abort_gives_everything_back_at_once():
    s = make()
    a = request("a", 9)
    s.add_request(a)
    run_step(s, s.schedule())
    assert s.abort_request("a") and a.finish_reason is FinishReason.ABORT and a.status is RequestStatus.ABORTED
    assert s.cache.num_used_pages() == 0 and not s.has_work() and not s.abort_request("a")
    s.cache.assert_consistent([])


def test_a_victim_leaves_the_step_it_was_already_given_a_token_in():
    # a decodes and b (newer) decodes too; then ... the oldest prefill evicts the newest request, which already sits in the decode batch
    s = make(pages=7, page=4, seqs=3, budget=16, chunk=8, watermark=0.01)  # 6 usable pages
    a = request("a", 20, max_tokens=2)
    b = request("b", 3, max_tokens=9)
    s.add_request(a)
    s.add_request(b)
    run_step(s, s.schedule())  # a: 8 tokens (2 pages); b: whole prompt (1 page), decoding from now on
    run_step(s, s.schedule())  # b decodes; a: 8 more (4 pages)
    assert s.cache.num_free_pages() == 1
    out = s.schedule()  # b decodes (position 4: takes the last page); a then needs a 5th page and evicts b
    assert [r.request_id for r in out.preempted] == ["b"] and b not in out.decodes and out.count_of(b) == 0
    run_step(s, out)
    while s.has_work():
        run_step(s, s.schedule())
    assert len(a.output_token_ids) == 2 and len(b.output_token_ids) == 9


def test_a_step_can_be_decided_while_the_tokens_of_the_one_before_are_pending():
    """What the engine does with a step in flight: positions advance and each sampled request gets a pending token at once;
    on that state the next step is decided.  A request that reaches its length with the pending token is closed: it is
    dropped at the next decision, and its token still arrives."""
    from velox_amd.engine.request import PENDING_TOKEN

    s = make(pages=33, page=4, budget=16, chunk=8)
    a, b = request("a", 6, max_tokens=2), request("b", 11, max_tokens=5)
    s.add_request(a)
    s.add_request(b)
    first = s.schedule()  # a whole (6), b's first 8
    assert portions(first) == [("a", 6), ("b", 8)]
    # booked before its tokens are known
    for p in first.portions:
        s.advance(p.request, p.count)
    slot = a.expect_token()
    assert a.output_token_ids == [PENDING_TOKEN] and a.status is RequestStatus.RUNNING_DECODE and not a.finished
    second = s.schedule()  # decided with a's token pending: a decodes, b goes on
    assert second.decodes == [a] and portions(second) == [("b", 3)] and a.all_token_ids[a.num_computed_tokens] == PENDING_TOKEN
    a.deliver_token(slot, 41)
    assert a.output_token_ids == [41] and a.all_token_ids[-1] == 41
    # the second step in flight: a's second token is its last
    s.advance(a, 1)
    s.advance(b, 3)
    slot_a, slot_b = a.expect_token(), b.expect_token()
    assert a.closing and a.finished and a.finish_reason is None and a.status is RequestStatus.FINISHED and not b.closing
    third = s.schedule()
    assert third.decodes == [b] and a not in s.running and a.cache is None and s.num_finished == 1
    a.deliver_token(slot_a, 42)
    a.finish(a.stop_reason(42, frozenset()))
    b.deliver_token(slot_b, 7)
    assert a.finish_reason is FinishReason.LENGTH and a.output_token_ids == [41, 42] and b.output_token_ids == [7]
    s.cache.assert_consistent([b.cache])


def test_listeners_hear_tokens_and_the_end_and_may_fail():
    r = request("r", 3, max_tokens=2)
    heard = []
    r.subscribe(on_token=lambda req, token: heard.append((req.request_id, "token", token)),
                on_finish=lambda req, reason: heard.append((req.request_id, "finish", reason)))
    r.subscribe(on_token=lambda req, token: 1 / 0, on_finish=lambda req, reason: 1 / 0)  # a failing listener is logged, the request goes on
    r.record_token(7)
    r.record_token(8)
    assert r.num_output_tokens == 2 and r.all_token_ids == [1, 2, 3, 7, 8] and r.first_token_time is not None
    r.finish(r.stop_reason(8, frozenset()))
    r.finish(FinishReason.ABORT)  # the second end is not heard
    assert heard == [("r", "token", 7), ("r", "token", 8), ("r", "finish", FinishReason.LENGTH)]
    assert r.finished and r.status is RequestStatus.FINISHED and r.time_to_first_token >= 0


def test_status_follows_from_what_the_request_holds():
    s = make(pages=33, page=4, budget=8, chunk=8)
    r = request("r", 11, max_tokens=3)
    assert r.status is RequestStatus.WAITING
    s.add_request(r)
    run_step(s, s.schedule())
    assert r.status is RequestStatus.RUNNING_PREFILL and r.num_uncomputed_tokens == 3
    run_step(s, s.schedule())
    assert r.status is RequestStatus.RUNNING_DECODE and r.num_uncomputed_tokens == 1 and r.output_token_ids == [1000]
    s._preempt(r)
    assert r.status is RequestStatus.PREEMPTED and r.cache is None and r.num_computed_tokens == 0 and r.num_uncomputed_tokens == 12
    run_step(s, s.schedule())
    assert r.status is RequestStatus.RUNNING_PREFILL and r.num_preemptions == 1
    while s.has_work():
        run_step(s, s.schedule())
    assert r.status is RequestStatus.FINISHED and r.output_token_ids == [1000, 1001, 1002]
