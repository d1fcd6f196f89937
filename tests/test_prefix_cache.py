"""Sharing of prompt prefixes: the trie alone, the cache manager with it, the scheduler's admissions, and generation
through the engine on the CPU (reference behaviour: ``src/radix_cache.py``, ``src/block_manager.py:52-72,101-112``,
``engine/scheduler.py:136-146,257-291``)."""
import random

import pytest
import torch

from helpers import PAGE_SIZE, make_folder, random_tokens
from plain_qwen2 import qwen2_logits, read_model_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.cache import CacheManager
from velox_amd.cache.allocator import PageAllocator
from velox_amd.cache.prefix import PrefixCache
from velox_amd.engine.request import RequestStatus
from velox_amd.engine.scheduler import Scheduler, SchedulerConfig
from velox_amd.parts import StateNeed, kv_pages


# -- the trie alone ------------------------------------------------------------------------------------------------------
def test_publish_match_and_eviction_order():
    allocator = PageAllocator(12)
    trie = PrefixCache([allocator], page_size=2)
    tokens_a = [1, 2, 3, 4, 5, 6, 7]
    pages_a = allocator.take_many(4)  # the fourth page is not full
    assert trie.publish(tokens_a, [pages_a], 0, 3) == (3, True) and trie.num_nodes == 3 and trie.num_reclaimable == 0
    assert [allocator.holders(p) for p in pages_a] == [2, 2, 2, 1]
    # a second request with the same first two pages and another third
    tokens_b = [1, 2, 3, 4, 9, 9, 9]
    found = trie.match(tokens_b, max_pages=3)
    assert [n.pages for n in found] == [(pages_a[0],), (pages_a[1],)]
    for node in found:
        allocator.share(node.pages[0])
        trie.page_taken(node.pages[0])
    own = allocator.take()
    assert trie.publish(tokens_b, [[pages_a[0], pages_a[1], own]], 2, 3) == (3, True) and trie.num_nodes == 4
    trie.assert_consistent()
    # the first request ends: its third page is held by nobody any more, the first two still by the second request
    for page in pages_a:
        allocator.drop(page)
        trie.page_dropped(page)
    assert trie.num_reclaimable == 1 and allocator.holders(pages_a[2]) == 1 and allocator.holders(pages_a[3]) == 0
    trie.assert_consistent()
    assert trie.evict(5) == 1 and allocator.holders(pages_a[2]) == 0 and trie.num_nodes == 3
    # the second ends too: leaves go before their parents, the least recently used leaf first
    for page in (pages_a[0], pages_a[1], own):
        allocator.drop(page)
        trie.page_dropped(page)
    assert trie.num_reclaimable == 3
    assert trie.evict(1) == 1 and allocator.holders(own) == 0 and allocator.holders(pages_a[1]) == 1
    assert trie.match([1, 2, 3, 4, 9, 9], max_pages=3)[-1].pages == (pages_a[1],)
    assert trie.evict(10) == 2 and trie.num_nodes == 0 and allocator.num_used == 0 and trie.num_reclaimable == 0
    trie.assert_consistent()
    allocator.verify()
    assert trie.hit_rate == pytest.approx((4 + 4) / (6 + 6))


def test_a_page_with_a_token_still_in_flight_is_not_published():
    """A request's newest token may be a place holder while the step that draws it runs: a page that holds it is offered
    only once the value is there, and the request goes on publishing then."""
    from velox_amd.engine.request import PENDING_TOKEN

    allocator = PageAllocator(8)
    trie = PrefixCache([allocator], page_size=2)
    pages = allocator.take_many(3)
    tokens = [1, 2, 3, PENDING_TOKEN, 5, 6]
    assert trie.publish(tokens, [pages], 0, 3) == (1, True) and trie.num_nodes == 1
    assert trie.match([1, 2, 3, PENDING_TOKEN, 5], max_pages=2)[-1].pages == (pages[0],)
    tokens[3] = 4
    assert trie.publish(tokens, [pages], 1, 3) == (3, True) and trie.num_nodes == 3
    trie.assert_consistent()


def test_least_recently_used_leaf_goes_first_and_a_held_leaf_stays():
    allocator = PageAllocator(10)
    trie = PrefixCache([allocator], page_size=1)
    pages = {}
    for token in (10, 20, 30):
        pages[token] = allocator.take()
        trie.publish([token], [[pages[token]]], 0, 1)
        allocator.drop(pages[token])
        trie.page_dropped(pages[token])
    assert trie.num_reclaimable == 3
    trie.match([10], max_pages=1)  # 10 is the most recently used now, 20 the least
    holder = trie.match([20], max_pages=1)[0]  # ... but 20 is taken by a request
    allocator.share(holder.pages[0])
    trie.page_taken(holder.pages[0])
    assert trie.num_reclaimable == 2
    assert trie.evict(1) == 1 and not trie.holds(pages[30]) and trie.holds(pages[10]) and trie.holds(pages[20])
    assert trie.evict(5) == 1 and trie.holds(pages[20]) and trie.num_nodes == 1  # the held one cannot go
    allocator.drop(pages[20])
    trie.page_dropped(pages[20])
    assert trie.evict(5) == 1 and trie.num_nodes == 0
    trie.assert_consistent()


def test_a_request_stops_publishing_where_another_request_page_stands():
    allocator = PageAllocator(10)
    trie = PrefixCache([allocator], page_size=2)
    first = allocator.take_many(2)
    second = allocator.take_many(3)
    assert trie.publish([1, 2, 3, 4], [first], 0, 2) == (2, True)
    # the same tokens computed by another request at the same time, with pages of its own: nothing of it is published,
    # not even its third page, which would hang below a node whose page it does not hold
    assert trie.publish([1, 2, 3, 4, 5, 6], [second], 0, 3) == (0, False)
    assert trie.num_nodes == 2 and [allocator.holders(p) for p in second] == [1, 1, 1]
    trie.assert_consistent()


def test_nodes_hold_one_page_per_group():
    a, b = PageAllocator(6), PageAllocator(6)
    trie = PrefixCache([a, b], page_size=2)
    pa, pb = a.take_many(2), b.take_many(2)
    pb.reverse()
    assert trie.publish([7, 7, 8, 8], [pa, pb], 0, 2) == (2, True)
    for page in pa:
        a.drop(page)
    for page in pb:
        b.drop(page)
    for page in pa:
        trie.page_dropped(page)
    assert trie.num_reclaimable == 2 and a.num_used == 2 and b.num_used == 2
    assert [n.pages for n in trie.match([7, 7, 8, 8, 1], max_pages=2)] == [(pa[0], pb[0]), (pa[1], pb[1])]
    assert trie.evict(2) == 2 and a.num_used == 0 and b.num_used == 0


# -- the cache manager with it ---------------------------------------------------------------------------------------------
def manager(pages=9, page=4, seqs=4, needs=None, **kwargs):
    return CacheManager(needs or [kv_pages(1, 16)], page, pages, seqs, torch.float32, "cpu", allocate_tensors=False, prefix_caching=True, **kwargs)


def test_only_models_whose_requests_hold_their_whole_past_share_prefixes():
    assert manager().prefix is not None
    assert manager(needs=[kv_pages(1, 16), kv_pages(2, 32)]).prefix is not None
    assert manager(needs=[kv_pages(1, 16), kv_pages(1, 16, window=8)]).prefix is None
    assert manager(needs=[kv_pages(1, 16), StateNeed((("s", (4,), None),))]).prefix is None
    assert CacheManager([kv_pages(1, 16)], 4, 9, 4, torch.float32, "cpu", allocate_tensors=False).prefix is None


def test_matched_pages_enter_the_table_and_one_token_is_left_to_compute():
    m = manager(pages=12)
    tokens = list(range(100, 112))  # three full pages
    a = m.new_sequence()
    assert m.match_prefix(a, tokens) == 0
    assert m.append(a, 0, 12)
    m.publish(a, tokens, 7)
    assert a.published == 1 and m.prefix.num_nodes == 1  # only pages that are full of computed tokens
    m.publish(a, tokens, 12)
    assert a.published == 3
    b = m.new_sequence()
    assert m.match_prefix(b, tokens) == 8 and b.tables[0] == a.tables[0][:2]  # the whole prompt is known, but a row must be computed
    c = m.new_sequence()
    assert m.match_prefix(c, tokens + [5]) == 12 and c.tables[0] == a.tables[0]
    d = m.new_sequence()
    assert m.match_prefix(d, tokens[:4] + [0] + tokens[5:]) == 4
    m.assert_consistent([a, b, c, d])
    assert [m.groups[0].allocator.holders(p) for p in a.tables[0]] == [5, 4, 3]
    for seq in (a, b, c, d):
        m.free_sequence(seq)
    m.assert_consistent([])
    assert m.num_used_pages() == 3 and m.num_reclaimable_pages() == 3 and m.num_available_pages() == 11 and m.num_free_pages() == 8


def test_published_pages_are_given_back_when_a_request_needs_them():
    m = manager(pages=9, page=4)  # 8 usable pages
    first = m.new_sequence()
    tokens = list(range(24))
    assert m.append(first, 0, 24)
    m.publish(first, tokens, 24)
    m.free_sequence(first)
    assert m.num_free_pages() == 2 and m.num_reclaimable_pages() == 6 and m.num_available_pages() == 8
    other = m.new_sequence()
    assert m.max_new_tokens(other, 0) == 32 and m.can_append(other, 0, 20) and not m.can_append(other, 0, 33)
    assert m.append(other, 0, 20)  # 5 pages: 2 free ones and 3 from the trie, the deepest (least useful) first
    assert m.prefix.num_nodes == 3 and m.num_reclaimable_pages() == 3
    again = m.new_sequence()
    assert m.match_prefix(again, tokens) == 12  # the first three pages survived
    m.assert_consistent([other, again])
    assert m.num_available_pages() == 0 and not m.append(again, 12, 1)  # pages that a request holds cannot be had back
    m.free_sequence(other)
    assert m.append(again, 12, 4 * 5) and m.num_free_pages() == 0
    m.assert_consistent([again])


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_of_requests_with_common_prefixes(seed):
    """Requests that share prefixes come, grow, publish, are preempted and go in random order in a small pool: after every
    action no page is lost or held by the wrong number of owners, and what the trie can give back is what it says."""
    rng = random.Random(seed)
    page = rng.choice([1, 2, 4])
    m = manager(pages=rng.randrange(12, 30), page=page, seqs=5)
    stems = [[rng.randrange(3) for _ in range(rng.randrange(1, 6) * page)] for _ in range(3)]
    live = {}  # seq id -> [seq, tokens, computed]
    for action in range(400):
        choice = rng.random()
        if choice < 0.3 and len(live) < 5:
            seq = m.new_sequence()
            tokens = list(rng.choice(stems)) + [rng.randrange(3) for _ in range(rng.randrange(1, 3 * page + 2))]
            computed = m.match_prefix(seq, tokens)
            assert computed < len(tokens) and computed % page == 0 and len(seq.tables[0]) == computed // page
            live[action] = [seq, tokens, computed]
        elif choice < 0.75 and live:
            key = rng.choice(list(live))
            seq, tokens, computed = live[key]
            step = min(rng.randrange(1, 2 * page + 1), len(tokens) - computed) or 1
            if computed + step > len(tokens):
                tokens.append(rng.randrange(3))  # a decoded token
            available = m.num_available_pages()
            needed = m.pages_to_append(seq, computed, step)[0]
            assert m.can_append(seq, computed, step) == (needed <= available and computed + step <= m.max_model_len)
            if m.append(seq, computed, step):
                live[key][2] = computed + step
                m.publish(seq, tokens, computed + step)
            else:
                m.free_sequence(seq)  # preempted
                del live[key]
        elif live:
            key = rng.choice(list(live))
            m.free_sequence(live.pop(key)[0])
        m.assert_consistent([entry[0] for entry in live.values()])
        held = {p for entry in live.values() for p in entry[0].tables[0]}
        assert m.num_reclaimable_pages() == sum(1 for p in m.prefix._node_of if p not in held)
    for entry in live.values():
        m.free_sequence(entry[0])
    m.assert_consistent([])
    assert m.prefix.clear() == m.prefix.num_reclaimable + m.num_used_pages() or m.num_used_pages() == 0
    assert m.num_used_pages() == 0 and m.prefix.num_nodes == 0


# -- the scheduler's admissions ----------------------------------------------------------------------------------------------
def scheduler(pages=33, page=4, seqs=4, budget=16, chunk=8, max_len=128, watermark=0.01):
    cache = CacheManager([kv_pages(1, 16)], page, pages, seqs, torch.float32, "cpu", max_model_len=max_len, allocate_tensors=False, prefix_caching=True)
    return Scheduler(cache, SchedulerConfig(max_num_seqs=seqs, max_num_batched_tokens=budget, max_prefill_chunk_size=chunk, max_model_len=max_len, watermark=watermark))


def run_step(s, out):
    sampled = list(out.decodes)
    for r in out.decodes:
        s.advance(r, 1)
    for portion in out.portions:
        s.advance(portion.request, portion.count)
        if portion.completes:
            sampled.append(portion.request)
    for r in sampled:
        r.record_token(1000 + len(r.output_token_ids))
        reason = r.stop_reason(r.output_token_ids[-1], frozenset())
        if reason:
            r.finish(reason)


def run_to_end(s, limit=200):
    for _ in range(limit):
        if not s.has_work():
            return
        run_step(s, s.schedule())
    raise AssertionError("the scheduler did not finish")


def test_admission_takes_over_a_published_prefix():
    s = scheduler(budget=16, chunk=8)
    prompt = list(range(1, 23))  # 22 tokens: five full pages of 4
    first = Request("first", prompt, SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))
    s.add_request(first)
    run_to_end(s)
    assert first.num_cached_tokens == 0 and s.cache.prefix.num_nodes == 5  # 22 prompt + 1 generated token computed: 5 full pages
    second = Request("second", prompt + [77, 78], SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True))
    s.add_request(second)
    out = s.schedule()
    assert [p.request for p in out.portions] == [second] and second.num_cached_tokens == 20 and second.num_computed_tokens == 20
    assert out.count_of(second) == 4 and out.portions[0].start == 20 and out.num_tokens == 4
    run_to_end(s)
    # the same prompt again: all of it is known, but its last page is computed again so that there is a row to sample from
    third = Request("third", prompt[:20], SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
    s.add_request(third)
    out = s.schedule()
    assert third.num_cached_tokens == 16 and out.count_of(third) == 4
    run_to_end(s)
    s.cache.assert_consistent([])
    assert s.stats()["prefix_hit_rate"] > 0 and s.stats()["evictable_blocks"] == s.cache.prefix.num_nodes


def test_a_preempted_request_finds_its_own_pages_again():
    s = scheduler(pages=13, page=4, budget=32, chunk=16, max_len=48, watermark=0.0)  # 12 usable pages
    a = Request("a", list(range(1, 17)), SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True))
    b = Request("b", list(range(101, 117)), SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True))
    s.add_request(a)
    s.add_request(b)
    for _ in range(60):
        if not s.has_work():
            break
        run_step(s, s.schedule())
        s.cache.assert_consistent([r.cache for r in s.running if r.cache is not None])
    assert a.finished and b.finished and len(a.output_token_ids) == 20 and len(b.output_token_ids) == 20
    assert b.num_preemptions >= 1 and b.num_cached_tokens >= 4  # its recomputation began behind pages it had published itself
    assert a.output_token_ids == [1000 + i for i in range(20)] and b.output_token_ids == [1000 + i for i in range(20)]


def test_pages_that_only_the_trie_holds_count_as_room_for_admission():
    s = scheduler(pages=9, page=4, budget=32, chunk=32, max_len=32, watermark=0.0)
    first = Request("first", list(range(1, 25)), SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
    s.add_request(first)
    run_to_end(s)
    assert s.cache.num_free_pages() == 2 and s.cache.num_reclaimable_pages() == 6
    other = Request("other", list(range(201, 225)), SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
    s.add_request(other)
    out = s.schedule()
    assert [p.request for p in out.portions] == [other] and out.count_of(other) == 24 and other.status is RequestStatus.RUNNING_PREFILL
    assert s.cache.prefix.num_nodes == 2  # four of the first request's pages had to go
    run_to_end(s)
    s.cache.assert_consistent([])


# -- through the engine ------------------------------------------------------------------------------------------------------
def engine_for(folder, name, **overrides):
    options = dict(model=folder, dtype="float32", device="cpu", max_model_len=128, max_num_seqs=4, max_num_batched_tokens=32,
                   max_prefill_chunk_size=7, block_size=PAGE_SIZE[name], num_gpu_blocks=64, enable_cuda_graphs=False, seed=0)
    options.update(overrides)
    return Engine.from_pretrained(EngineConfig(**options), ops=TorchOps())


def greedy(prompts, n, prefix="r"):
    return [Request(f"{prefix}{i}", p, SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)) for i, p in enumerate(prompts)]


@pytest.mark.parametrize("name", ["A", "B"])
def test_generation_with_shared_prefixes_equals_generation_without(tmp_path, name):
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    stem = random_tokens(config["vocab_size"], 3 * PAGE_SIZE[name] + 1, seed=5)
    prompts = [stem + random_tokens(config["vocab_size"], n, seed=n) for n in (2, 9, 1, 14)] + [stem[:2 * PAGE_SIZE[name]]]
    plain = engine_for(folder, name, enable_prefix_caching=False)
    assert plain.cache.prefix is None
    expected = [r.output_token_ids for r in plain.generate(greedy(prompts, 6))]
    engine = engine_for(folder, name)  # on by default
    assert engine.cache.prefix is not None
    first = engine.generate(greedy(prompts[:1], 6, prefix="first"))[0]
    assert first.output_token_ids == expected[0] and first.num_cached_tokens == 0
    rest = engine.generate(greedy(prompts[1:], 6, prefix="rest"))
    assert [r.output_token_ids for r in rest] == expected[1:]
    assert [r.num_cached_tokens for r in rest[:3]] == [3 * PAGE_SIZE[name]] * 3
    assert rest[3].num_cached_tokens == PAGE_SIZE[name]  # a prompt that is known in full: its last page is computed again
    # the logits behind a taken-over prefix are those of the whole sequence
    tokens = prompts[2] + rest[1].output_token_ids
    logits = qwen2_logits(config, weights, tokens[:-1])
    for step, token in enumerate(rest[1].output_token_ids):
        assert int(logits[len(prompts[2]) - 1 + step].argmax()) == token
    engine.cache.assert_consistent([])
    assert engine.cache.num_used_pages() == engine.cache.prefix.num_nodes == engine.cache.num_reclaimable_pages() > 0
    assert engine.snapshot()["prefix_hit_rate"] > 0.3
    engine.cache.prefix.clear()
    assert engine.cache.num_used_pages() == 0


def test_a_small_pool_evicts_published_pages_and_preempts_without_changing_tokens(tmp_path):
    folder = make_folder(tmp_path, "B")
    config, _ = read_model_folder(folder)
    page = PAGE_SIZE["B"]
    stem = random_tokens(config["vocab_size"], 2 * page, seed=9)
    prompts = [stem + random_tokens(config["vocab_size"], 5 + 3 * i, seed=20 + i) for i in range(6)]
    roomy = engine_for(folder, "B", enable_prefix_caching=False)
    expected = [r.output_token_ids for r in roomy.generate(greedy(prompts, 12))]
    needed = max((len(p) + 12 + page - 1) // page for p in prompts)
    tight = engine_for(folder, "B", num_gpu_blocks=2 * needed + 2, max_model_len=needed * page)
    done = tight.generate(greedy(prompts, 12))
    assert [r.output_token_ids for r in done] == expected
    assert tight.scheduler.num_preemptions > 0 and tight.cache.prefix.num_hits > 0
    assert tight.cache.prefix.num_nodes < sum(len(r.all_token_ids) // page for r in done)  # some published pages had to go
    tight.cache.assert_consistent([])
