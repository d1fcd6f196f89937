"""Generation through the Python entry point on a CPU (plain references as kernels): scheduler, step
function, sampler and request bookkeeping together."""
import pytest
import torch

from helpers import PAGE_SIZE, make_folder, random_tokens
from plain_qwen2 import qwen2_logits, read_model_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.engine.request import FinishReason


def engine_for(folder, name, **overrides):
    options = dict(model=folder, dtype="float32", device="cpu", max_model_len=128, max_num_seqs=4, max_num_batched_tokens=32,
                   max_prefill_chunk_size=7, block_size=PAGE_SIZE[name], num_gpu_blocks=64, enable_cuda_graphs=False, seed=0,
                   enable_prefix_caching=False)  # (as in the reference's numerics tests; the prefix cache has tests of its own)
    options.update(overrides)
    return Engine.from_pretrained(EngineConfig(**options), ops=TorchOps())


def plain_greedy(config, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(qwen2_logits(config, weights, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def greedy(prompts, n, prefix="r"):
    return [Request(f"{prefix}{i}", p, SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)) for i, p in enumerate(prompts)]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain_and_batched_equals_alone(tmp_path, name):
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=n) for n in (5, 9, 13, 22)]
    engine = engine_for(folder, name)
    together = engine.generate(greedy(prompts, 8))
    for request, prompt in zip(together, prompts):
        assert request.output_token_ids == plain_greedy(config, weights, prompt, 8)
        assert request.finish_reason is FinishReason.LENGTH and len(request.output_token_ids) == 8
    for i, prompt in enumerate(prompts):
        alone = engine.generate(greedy([prompt], 8, prefix=f"alone{i}-"))[0]
        assert alone.output_token_ids == together[i].output_token_ids
    assert engine.cache.num_used_pages() == 0
    engine.cache.assert_consistent([])
    assert engine.snapshot()["num_finished"] == 8.0


def test_preemption_does_not_change_the_tokens(tmp_path):
    folder = make_folder(tmp_path, "B")
    config, _ = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=40 + n) for n in (20, 31, 12, 25)]
    roomy = engine_for(folder, "B", num_gpu_blocks=64).generate(greedy(prompts, 24))
    tight_engine = engine_for(folder, "B", num_gpu_blocks=13, watermark=0.01)  # 12 pages of 8 for 4 x (up to 55) tokens
    tight = tight_engine.generate(greedy(prompts, 24))
    assert tight_engine.scheduler.num_preemptions > 0
    for a, b in zip(roomy, tight):
        assert a.output_token_ids == b.output_token_ids and len(b.output_token_ids) == 24
    assert tight_engine.cache.num_used_pages() == 0
    tight_engine.cache.assert_consistent([])


def test_stop_tokens_and_limits(tmp_path):
    folder = make_folder(tmp_path, "A")
    config, weights = read_model_folder(folder)
    prompt = random_tokens(256, 6, 2)
    expected = plain_greedy(config, weights, prompt, 6)
    engine = engine_for(folder, "A")
    stop_at = expected[2]
    request = Request("stop", prompt, SamplingParams(temperature=0.0, max_tokens=6, stop_token_ids=[stop_at]))
    engine.generate([request])
    cut = expected.index(stop_at) + 1
    assert request.output_token_ids == expected[:cut] and request.finish_reason is FinishReason.STOP  # the stop token stays
    with pytest.raises(ValueError):
        engine.add_request(Request("big", [1] * 200, SamplingParams(max_tokens=1)))
    with pytest.raises(ValueError):
        engine.add_request(Request("oov", [1, 256], SamplingParams(max_tokens=1)))


def test_seeded_sampling_is_independent_of_the_batch(tmp_path):
    folder = make_folder(tmp_path, "B")
    config, _ = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=70 + n) for n in (1, 17, 40, 8)]

    def sampled(i, prompt):
        return Request(f"s{i}", prompt, SamplingParams(temperature=0.8, max_tokens=6, seed=100 + i, ignore_eos=True))

    engine = engine_for(folder, "B")
    together = engine.generate([sampled(i, p) for i, p in enumerate(prompts)])
    again = engine_for(folder, "B").generate([sampled(i, p) for i, p in enumerate(prompts)])
    assert [r.output_token_ids for r in together] == [r.output_token_ids for r in again]
    alone = engine.generate([sampled(2, prompts[2])])[0]
    assert alone.output_token_ids == together[2].output_token_ids
    # a greedy request keeps its tokens next to sampled ones
    greedy_alone = engine.generate(greedy([prompts[1]], 6, prefix="g-alone"))[0]
    mixed = engine.generate([sampled(7, prompts[0]), greedy([prompts[1]], 6, prefix="g-mixed")[0], sampled(8, prompts[3])])
    assert mixed[1].output_token_ids == greedy_alone.output_token_ids
    assert len({tuple(r.output_token_ids) for r in together}) > 1


@pytest.mark.parametrize("name", ["A", "B"])
def test_launching_the_next_step_early_changes_no_token(tmp_path, name):
    """decode_lookahead launches a decode step before the tokens of the step before it have been read: same tokens,
    same finish reasons, also when a request stops on a token that was still in flight, and every page comes back."""
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=90 + n) for n in (4, 11, 19)]
    expected = [plain_greedy(config, weights, p, 10) for p in prompts]
    stop_at = expected[1][4]  # request 1 stops in the middle of the others' decoding

    def requests(prefix):
        out = greedy(prompts, 10, prefix=prefix)
        out[1] = Request(f"{prefix}stop", prompts[1], SamplingParams(temperature=0.0, max_tokens=10, stop_token_ids=[stop_at]))
        out[2] = Request(f"{prefix}short", prompts[2], SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True))
        return out

    results = {}
    for lookahead in (True, False):
        engine = engine_for(folder, name, decode_lookahead=lookahead)
        launches = []
        inner = engine.runner.step
        engine.runner.step = lambda entries, device_ids=None: (launches.append(device_ids is not None), inner(entries, device_ids=device_ids))[1]
        done = engine.generate(requests("on-" if lookahead else "off-"))
        results[lookahead] = [(r.output_token_ids, r.finish_reason) for r in done]
        assert any(launches) == lookahead
        assert engine.cache.num_used_pages() == 0
        engine.cache.assert_consistent([])
        assert engine._ahead is None or not any(engine._alive(r) for r in engine._ahead.sampled)
    assert results[True] == results[False]
    cut = expected[1].index(stop_at) + 1
    assert results[True][0] == (expected[0], FinishReason.LENGTH)
    assert results[True][1] == (expected[1][:cut], FinishReason.STOP)
    assert results[True][2] == (expected[2][:3], FinishReason.LENGTH)


def test_abort_while_a_step_is_in_flight(tmp_path):
    folder = make_folder(tmp_path, "A")
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=95 + n) for n in (6, 9)]
    engine = engine_for(folder, "A")
    keep, drop = greedy(prompts, 12)
    engine.add_request(keep)
    engine.add_request(drop)
    while len(keep.output_token_ids) < 4:
        engine.step()
    assert engine._ahead is not None  # a decode step is in flight
    engine.abort_request(drop.request_id)
    while engine.has_work():
        engine.step()
    assert keep.output_token_ids == plain_greedy(config, weights, prompts[0], 12)
    assert drop.finish_reason is FinishReason.ABORT and len(drop.output_token_ids) < 12
    assert engine.cache.num_used_pages() == 0
    engine.cache.assert_consistent([])


def test_requests_and_aborts_from_another_thread(tmp_path):
    """``submit`` and ``request_abort`` may be called from any thread; the stepping thread takes them in at the start of
    its next step (reference ``engine/engine.py:239-263``)."""
    import threading

    folder = make_folder(tmp_path, "A")
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=120 + n) for n in (5, 8, 11)]
    engine = engine_for(folder, "A")
    first, second, dropped = greedy(prompts, 10)
    engine.add_request(first)
    for _ in range(3):
        engine.step()

    def client():
        engine.submit(second)
        engine.submit(dropped)
        with pytest.raises(ValueError):
            engine.submit(Request("too-long", [1] * engine.max_model_len, SamplingParams(max_tokens=1)))

    thread = threading.Thread(target=client)
    thread.start()
    thread.join()
    assert engine.has_work() and second.request_id not in engine.scheduler.requests  # not taken in before a step begins
    engine.step()
    assert second.request_id in engine.scheduler.requests and dropped.request_id in engine.scheduler.requests
    aborter = threading.Thread(target=lambda: engine.request_abort(dropped.request_id))
    aborter.start()
    aborter.join()
    while engine.has_work():
        engine.step()
    assert first.output_token_ids == plain_greedy(config, weights, prompts[0], 10)
    assert second.output_token_ids == plain_greedy(config, weights, prompts[1], 10)
    assert dropped.finish_reason is FinishReason.ABORT and len(dropped.output_token_ids) < 10
    # a request id that is queued twice is refused when it is taken in, not in the submitting thread
    again = greedy(prompts[:1], 2)[0]
    twin = greedy(prompts[:1], 2)[0]
    engine.submit(again)
    engine.submit(twin)
    engine.step()
    assert twin.finish_reason is FinishReason.ABORT and not again.finished
    assert engine.abort_all() == "aborted" and not engine.has_work()
    assert engine.cache.num_used_pages() == 0


@pytest.mark.parametrize("prefix_caching", [False, True])
def test_every_kind_of_step_is_launched_early_also_with_preemption_and_late_arrivals(tmp_path, prefix_caching):
    """A pool so small that requests are preempted and recomputed, prompts that take several portions, a request that
    arrives while others decode, one that stops on a token in flight: with the next step always launched before this one's
    tokens are read, every request ends with the plain model's tokens, as with one step at a time."""
    folder = make_folder(tmp_path, "B")
    config, weights = read_model_folder(folder)
    page = PAGE_SIZE["B"]
    stem = random_tokens(config["vocab_size"], 2 * page + 1, seed=70)
    prompts = [stem + random_tokens(config["vocab_size"], n, seed=71 + n) for n in (3, 14, 1, 9, 22)]
    steps = 12
    expected = [plain_greedy(config, weights, p, steps) for p in prompts]
    stop_at = expected[3][6]
    needed = max((len(p) + steps + page - 1) // page for p in prompts)

    def run(lookahead):
        engine = engine_for(folder, "B", decode_lookahead=lookahead, num_gpu_blocks=2 * needed + 2, max_model_len=needed * page,
                            enable_prefix_caching=prefix_caching, max_num_batched_tokens=16, max_prefill_chunk_size=6)
        requests = greedy(prompts, steps, prefix=f"{lookahead}-")
        requests[3] = Request(f"{lookahead}-stop", prompts[3], SamplingParams(temperature=0.0, max_tokens=steps, stop_token_ids=[stop_at]))
        early = {"portions": 0, "pending": 0}
        inner = engine._launch

        def launch(plan, pending=None):
            if pending is not None:
                early["portions"] += len(plan.portions)
                early["pending"] += 1
            return inner(plan, pending=pending)

        engine._launch = launch
        for request in requests[:3]:
            engine.add_request(request)
        for _ in range(4):
            engine.step()
        for request in requests[3:]:
            engine.add_request(request)  # arrive while the others run
        while engine.has_work():
            engine.step()
            engine.cache.assert_consistent([r.cache for r in engine.scheduler.running if r.cache is not None])
        assert engine.cache.num_used_pages() == (engine.cache.prefix.num_nodes if prefix_caching else 0)
        assert (early["pending"] > 0) == lookahead and (early["portions"] > 0) == lookahead
        return requests, (engine.scheduler.num_preemptions, engine.cache.prefix.num_hits if prefix_caching else 0)

    ahead, (preemptions, hits) = run(True)
    plain, _ = run(False)
    assert hits > 0 if prefix_caching else preemptions > 0  # (with the stem shared the pool is large enough)
    cut = expected[3].index(stop_at) + 1
    for index, (a, b) in enumerate(zip(ahead, plain)):
        want = expected[index][:cut] if index == 3 else expected[index]
        assert a.output_token_ids == want and b.output_token_ids == want, (index, a.output_token_ids, b.output_token_ids, want)
        assert a.finish_reason is (FinishReason.STOP if index == 3 else FinishReason.LENGTH) and a.finish_reason is b.finish_reason
        assert -1 not in a.all_token_ids


def test_penalties_keep_their_counts_through_early_launches_and_preemption(tmp_path):
    """Penalties over prompt and output with every step launched before the tokens of the one before are read: the
    sampler counts a request's tokens on the device from its own output, so the penalised tokens are those of the plain
    model under the reference's formula, also for requests that are preempted and recomputed in a small pool, beside a
    request without penalties; at the end the sampler holds nothing of any request."""
    folder = make_folder(tmp_path, "B")
    config, weights = read_model_folder(folder)
    page = PAGE_SIZE["B"]
    vocab = config["vocab_size"]
    prompts = [[5, 9, 5, 9, 5, 9, 5, 9, 12, 5, 9], random_tokens(vocab, 19, seed=91), [7] * 13 + random_tokens(vocab, 4, seed=92), random_tokens(vocab, 9, seed=93)]
    coefficients = [dict(repetition_penalty=1.6, frequency_penalty=0.05, presence_penalty=0.02), dict(repetition_penalty=1.3, presence_penalty=0.03),
                    dict(frequency_penalty=0.4), {}]
    steps = 14

    def plain_penalised(prompt, repetition_penalty=1.0, presence_penalty=0.0, frequency_penalty=0.0):
        tokens = list(prompt)
        for _ in range(steps):
            logits = qwen2_logits(config, weights, tokens)[-1:].clone()
            TorchOps().apply_penalties(logits, torch.tensor([tokens]), torch.tensor([len(tokens)]),
                                       torch.tensor([[repetition_penalty, presence_penalty, frequency_penalty]]))
            tokens.append(int(logits[0].argmax()))
        return tokens[len(prompt):]

    expected = [plain_penalised(p, **c) for p, c in zip(prompts, coefficients)]
    assert expected[0] != plain_greedy(config, weights, prompts[0], steps)  # the penalties decide
    needed = max((len(p) + steps + page - 1) // page for p in prompts)
    for lookahead in (True, False):
        engine = engine_for(folder, "B", decode_lookahead=lookahead, num_gpu_blocks=2 * needed + 2, max_model_len=needed * page,
                            max_num_batched_tokens=16, max_prefill_chunk_size=6)
        requests = [Request(f"{lookahead}-{i}", p, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True, **c))
                    for i, (p, c) in enumerate(zip(prompts, coefficients))]
        done = engine.generate(requests)
        assert engine.scheduler.num_preemptions > 0
        for index, request in enumerate(done):
            assert request.output_token_ids == expected[index], (lookahead, index, request.output_token_ids, expected[index])
        assert engine.sampler._seen.row_of_request == {} and engine.sampler._seeds == {}


def test_a_request_that_stops_on_the_token_pending_at_its_preemption_is_not_admitted_again(tmp_path):
    """With the next step decided before this one's tokens are read, a request can lose its pages while its newest token
    is still in flight, and wait.  If that token ends it (a stop token), it ends while it waits: it must leave the queue,
    never take pages or a slot again, and the sampler must hold nothing of it."""
    from velox_amd.engine.request import PENDING_TOKEN

    folder = make_folder(tmp_path, "B")
    config, weights = read_model_folder(folder)
    steps = 20
    found = 0
    for lengths, pages in (((20, 31, 12, 25), 9), ((8, 50, 40, 12), 13), ((8, 50, 40, 12), 18)):
        prompts = [random_tokens(config["vocab_size"], n, seed=42 + n) for n in lengths]

        def build(stops):
            engine = engine_for(folder, "B", num_gpu_blocks=pages, watermark=0.01)
            requests = [Request(f"q{i}", p, SamplingParams(temperature=0.8, top_k=20, seed=7 + i, max_tokens=steps, stop_token_ids=stops.get(i, [])))
                        for i, p in enumerate(prompts)]
            return engine, requests

        # first run: who waits, after a scheduling decision, with its newest token still pending, and what that token is
        engine, requests = build({})
        events = []
        inner = engine.scheduler.schedule

        def schedule():
            plan = inner()
            events.extend((requests.index(r), len(r.output_token_ids) - 1) for r in engine.scheduler.waiting if r.all_token_ids[-1] == PENDING_TOKEN)
            return plan

        engine.scheduler.schedule = schedule
        engine.generate(requests)
        usable = [(who, at) for who, at in events if requests[who].output_token_ids[at] not in requests[who].output_token_ids[:at]]
        if not usable:
            continue
        who, at = usable[0]
        stop_token = requests[who].output_token_ids[at]
        reference = [list(r.output_token_ids) for r in requests]

        # second run: that token is a stop token of that request
        engine, again = build({who: [stop_token]})
        admissions_after_end = []
        for request in again:
            inner_admitted = request.admitted
            request.admitted = lambda cache, cached, request=request, inner_admitted=inner_admitted: (
                admissions_after_end.append(request.request_id) if request.finished else None, inner_admitted(cache, cached))[1]
        engine.generate(again)
        assert again[who].finish_reason is FinishReason.STOP and again[who].output_token_ids == reference[who][:at + 1]
        assert admissions_after_end == []
        assert engine.sampler._seen.row_of_request == {} and engine.sampler._seeds == {}
        assert engine.cache.num_used_pages() == 0 and not engine.scheduler.requests
        engine.cache.assert_consistent([])
        assert engine.snapshot()["num_finished"] == 4.0
        found += 1
    assert found > 0  # the case did occur
