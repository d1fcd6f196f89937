"""Generation through the Python entry point on the GPU: greedy tokens against the plain model, batched equals
alone, preemption, HIP-graph decode equals eager decode, sampling, and the command line."""
import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import PAGE_SIZE, make_folder, random_tokens
from plain_qwen2 import qwen2_logits, read_model_folder
from velox_amd import Engine, EngineConfig, Request, SamplingParams

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def engine_for(folder, name, dtype="float32", **overrides):
    options = dict(model=folder, dtype=dtype, device="cuda", max_model_len=160, max_num_seqs=4, max_num_batched_tokens=32,
                   max_prefill_chunk_size=7, block_size=PAGE_SIZE[name], num_gpu_blocks=96, enable_cuda_graphs=False, seed=0,
                   enable_prefix_caching=False)  # (as in the reference's numerics tests; the prefix cache has tests of its own)
    options.update(overrides)
    return Engine.from_pretrained(EngineConfig(**options))


def plain_greedy(config, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(qwen2_logits(config, weights, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def greedy(prompts, n, prefix="r"):
    return [Request(f"{prefix}{i}", p, SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True)) for i, p in enumerate(prompts)]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain(tmp_path, name):
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=n) for n in (5, 9, 13, 40)]
    engine = engine_for(folder, name)
    together = engine.generate(greedy(prompts, 8))
    for request, prompt in zip(together, prompts):
        assert request.output_token_ids == plain_greedy(config, weights, prompt, 8)
    for i, prompt in enumerate(prompts):
        assert engine.generate(greedy([prompt], 8, prefix=f"alone{i}-"))[0].output_token_ids == together[i].output_token_ids
    assert engine.cache.num_used_pages() == 0
    engine.cache.assert_consistent([])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_an_engine_over_weights_drawn_on_the_device_computes_the_plain_models_logits(name, dtype):
    """``Engine.from_random(generator_device="cuda")`` is what every measurement runs on: its tensors, read back under
    their checkpoint names, give the plain model the engine's logits and tokens (fused rows, the tied head, held dtypes
    and the kernels' copies of the weights are all behind them)."""
    from helpers import CONFIGS
    from velox_amd.weights import named_tensors

    config = CONFIGS[name]
    engine = Engine.from_random(config, seed=21, config=EngineConfig(
        dtype=dtype, device="cuda", max_model_len=160, max_num_seqs=4, max_num_batched_tokens=64, max_prefill_chunk_size=7,
        block_size=PAGE_SIZE[name], num_gpu_blocks=96, enable_cuda_graphs=False, seed=0, enable_prefix_caching=False), generator_device="cuda")
    weights = {key: value.float().cpu() for key, value in named_tensors(engine.model)}
    assert ("lm_head.weight" in weights) != bool(config["tie_word_embeddings"])
    assert abs(float(weights["model.norm.weight"].mean()) - 1.0) < 0.05 and abs(float(weights["model.embed_tokens.weight"].std()) - 0.02) < 0.003
    prompts = [random_tokens(config["vocab_size"], n, seed=n) for n in (5, 9, 13, 40)]
    done = engine.generate(greedy(prompts, 6))
    from velox_amd.engine.batch import StepEntry
    for request, prompt in zip(done, prompts):
        if dtype == "float32":
            assert request.output_token_ids == plain_greedy(config, weights, prompt, 6)
        # the logits of the whole sequence in one step
        tokens = prompt + request.output_token_ids
        sequence = engine.cache.new_sequence()
        assert engine.cache.append(sequence, 0, len(tokens))
        got = engine.runner.step([StepEntry(sequence, tokens, 0, list(range(len(tokens))))]).float().cpu()
        engine.cache.free_sequence(sequence)
        want = qwen2_logits(config, weights, tokens)
        tolerance = dict(rtol=2e-4, atol=2e-5) if dtype == "float32" else dict(rtol=5e-2, atol=3e-2)  # (those of the whole-prompt tests)
        torch.testing.assert_close(got, want, **tolerance)


def test_graph_decode_equals_eager_decode_and_preemption_keeps_tokens(tmp_path):
    """float32: every kernel is this repository's own and sums in a fixed order, so the tokens must be identical."""
    dtype = "float32"
    folder = make_folder(tmp_path, "B", "float32")
    config, _ = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=40 + n) for n in (20, 31, 12, 25)]
    eager = engine_for(folder, "B", dtype).generate(greedy(prompts, 30))
    graph_engine = engine_for(folder, "B", dtype, enable_cuda_graphs=True)
    assert graph_engine.runner.uses_graphs
    graphed = graph_engine.generate(greedy(prompts, 30))
    assert graph_engine.runner.num_graph_replays > 20
    assert [r.output_token_ids for r in graphed] == [r.output_token_ids for r in eager]
    # a second round through the same graphs, with other requests in the same slots and pages
    again = graph_engine.generate(greedy(list(reversed(prompts)), 30, prefix="again"))
    assert [r.output_token_ids for r in again] == [r.output_token_ids for r in reversed(eager)]
    tight_engine = engine_for(folder, "B", dtype, num_gpu_blocks=14, enable_cuda_graphs=True)
    tight = tight_engine.generate(greedy(prompts, 30))
    assert tight_engine.scheduler.num_preemptions > 0
    assert [r.output_token_ids for r in tight] == [r.output_token_ids for r in eager]
    assert tight_engine.cache.num_used_pages() == 0


def test_captured_steps_behind_few_keys_and_behind_many(tmp_path):
    """With a long context allowed, a bucket has two captures: one whose attention splits the keys as the longest context
    needs, one for steps whose sequences all hold few keys (one workgroup per sequence and KV head).  A request that grows
    past the bound moves from the one to the other; tokens as without graphs (float32: bit for bit)."""
    from velox_amd.parts.attention import SHORT_CONTEXT_KEYS

    folder = make_folder(tmp_path, "B", "float32")
    config, _ = read_model_folder(folder)
    assert config["max_position_embeddings"] >= 1024
    prompts = [random_tokens(config["vocab_size"], n, seed=70 + n) for n in (SHORT_CONTEXT_KEYS - 14, 40)]
    options = dict(max_model_len=1024, max_num_batched_tokens=512, max_prefill_chunk_size=256, num_gpu_blocks=400)
    eager = engine_for(folder, "B", "float32", **options).generate(greedy(prompts, 30))
    engine = engine_for(folder, "B", "float32", enable_cuda_graphs=True, **options)
    assert sorted(engine.runner._bounded_graphs) == [1, 2, 4] and all([b for b, _ in v] == [SHORT_CONTEXT_KEYS] for v in engine.runner._bounded_graphs.values())
    graphed = engine.generate(greedy(prompts, 30))
    assert [r.output_token_ids for r in graphed] == [r.output_token_ids for r in eager]
    assert 10 <= engine.runner.num_short_graph_replays <= 20 and engine.runner.num_graph_replays >= 29
    # the short request alone stays behind few keys to its end
    before = engine.runner.num_short_graph_replays
    alone = engine.generate(greedy(prompts[1:], 30, prefix="alone"))
    assert alone[0].output_token_ids == eager[1].output_token_ids
    assert engine.runner.num_short_graph_replays - before >= 29


@pytest.mark.parametrize("graphs", [False, True])
def test_launching_the_next_step_early_changes_no_token(tmp_path, graphs):
    """decode_lookahead on the GPU, eager and through graphs: the next decode step is queued, with its token ids taken
    on the device from the sampler's output, before the host reads the tokens.  Same tokens and finish reasons as with
    one step at a time, also for a request that stops on a token that was still in flight."""
    folder = make_folder(tmp_path, "B", "float32")
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=60 + n) for n in (7, 15, 22, 3)]
    expected = [plain_greedy(config, weights, p, 14) for p in prompts]
    stop_at = expected[1][5]

    def requests(prefix):
        out = greedy(prompts, 14, prefix=prefix)
        out[1] = Request(f"{prefix}stop", prompts[1], SamplingParams(temperature=0.0, max_tokens=14, stop_token_ids=[stop_at]))
        out[2] = Request(f"{prefix}short", prompts[2], SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True))
        out[3] = Request(f"{prefix}drawn", prompts[3], SamplingParams(temperature=0.9, max_tokens=14, seed=5, ignore_eos=True))
        return out

    results = {}
    for lookahead in (True, False):
        engine = engine_for(folder, "B", "float32", enable_cuda_graphs=graphs, decode_lookahead=lookahead)
        launches = []
        inner = engine.runner.step
        engine.runner.step = lambda entries, device_ids=None: (launches.append(device_ids is not None), inner(entries, device_ids=device_ids))[1]
        done = engine.generate(requests("on-" if lookahead else "off-"))
        results[lookahead] = [(r.output_token_ids, r.finish_reason) for r in done]
        assert any(launches) == lookahead
        assert engine.cache.num_used_pages() == 0
        engine.cache.assert_consistent([])
    assert results[True] == results[False]
    cut = expected[1].index(stop_at) + 1
    assert results[True][0][0] == expected[0]
    assert results[True][1][0] == expected[1][:cut]
    assert results[True][2][0] == expected[2][:4]
    assert len(results[True][3][0]) == 14


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["A", "B"])
def test_graph_replay_gives_the_eager_logits(tmp_path, name, dtype):
    """The same decode batch through the eager step and through the captured graph, on the same cache state, for
    several steps with eager work between the replays.  (In bfloat16 the matrix library may pick another kernel under
    capture, so the comparison allows rounding.)"""
    from helpers import Harness
    from velox_amd.engine.batch import StepEntry
    from velox_amd.kernels import load_ops

    folder = make_folder(tmp_path, name, "float32" if dtype == torch.float32 else "bfloat16")
    config, weights = read_model_folder(folder)
    h = Harness(folder, load_ops("cuda"), dtype, "cuda", PAGE_SIZE[name], num_pages=64, max_num_seqs=4, enable_graphs=True)
    h.runner.capture_decode_graphs()
    assert sorted(h.runner._graphs) == [1, 2, 4]
    sequences = {rid: random_tokens(config["vocab_size"], n, seed=n) for rid, n in (("a", 30), ("b", 9), ("c", 17))}
    for rid, tokens in sequences.items():
        h.feed([(rid, tokens[:-6], [])])
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=3e-2, atol=2e-2)
    for step in range(6):
        live = ["a", "b", "c"] if step % 2 == 0 else ["c", "a"]  # 3 rows pad to the bucket of 4; 2 rows fill theirs
        entries = []
        for rid in live:
            seq, computed = h.live[rid]
            assert h.cache.append(seq, computed, 1)
            entries.append(StepEntry(seq, [sequences[rid][computed]], computed, [0]))
        eager = h.runner._forward(h.runner.builder.build(entries, h.runner.ops, dtype, h.runner.workspace)).float().cpu()
        replays = h.runner.num_graph_replays
        graphed = h.runner.step(entries).float().cpu()
        assert h.runner.num_graph_replays == replays + 1
        torch.testing.assert_close(graphed, eager, **tol)
        plain_tol = dict(rtol=2e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=5e-2, atol=3e-2)
        for row, rid in enumerate(live):
            computed = h.live[rid][1]
            torch.testing.assert_close(graphed[row], qwen2_logits(config, weights, sequences[rid][:computed + 1])[-1], **plain_tol)
            h.live[rid][1] += 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_a_little_short_of_a_timed_row_count_are_padded_onto_the_null_page(tmp_path, dtype):
    """Once the library's kernels have been timed for a number of rows, a step of prompt portions with a few rows less runs
    with that many: the extra rows belong to a sequence on the null page, and nobody's logits change."""
    folder = make_folder(tmp_path, "B", dtype)
    config, weights = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=90 + n) for n in (29, 30, 3)]  # 62 rows in the first step, 3 in the next ones
    plain = engine_for(folder, "B", dtype, max_num_batched_tokens=64, max_prefill_chunk_size=32).generate(greedy(prompts, 5))
    engine = engine_for(folder, "B", dtype, max_num_batched_tokens=64, max_prefill_chunk_size=32)
    engine.runner.tuned_row_counts = [16, 64]  # (as tune_matrix_products leaves them)
    padded = engine.generate(greedy(prompts, 5, prefix="padded"))
    assert engine.runner.num_padded_steps == 1  # 62 -> 64; decode-sized steps and steps far from a timed count stay as they are
    assert [r.output_token_ids for r in padded] == [r.output_token_ids for r in plain]
    if dtype == "float32":
        for request, prompt in zip(padded, prompts):
            assert request.output_token_ids == plain_greedy(config, weights, prompt, 5)
    assert engine.cache.num_used_pages() == 0
    engine.cache.assert_consistent([])


def test_library_tuning_recaptures_the_decode_graphs_and_keeps_the_logits(tmp_path):
    """bfloat16: after the matrix library has picked kernels for a decode batch size, the captured steps are captured
    again (they hold the library's kernels) and generation still agrees with the plain model to rounding."""
    folder = make_folder(tmp_path, "A", "bfloat16")
    config, weights = read_model_folder(folder)
    engine = engine_for(folder, "A", "bfloat16", enable_cuda_graphs=True, max_num_seqs=32, max_num_batched_tokens=64)
    assert engine.ops.library_serves(128, 64, 64) and not engine.ops.library_serves(8, 1 << 16, 1 << 12)
    assert not engine.ops.library_serves(32, 256, 64)  # too small for the library's timing to mean anything
    before = dict(engine.runner._graphs)
    assert engine.tune_matrix_products([128]) > 0
    assert engine.runner.tuned_row_counts == [128]
    assert all(engine.runner._graphs[b] is before[b] for b in before)  # no captured step has 128 rows
    engine.ops.library_serves = lambda m, n, k: m > 16  # (tiny weights: pretend they are worth timing)
    assert engine.tune_matrix_products([32]) > 0
    assert sorted(engine.runner._graphs) == sorted(before) and all(engine.runner._graphs[b] is not before[b] for b in before)
    prompts = [random_tokens(config["vocab_size"], 6 + i, seed=70 + i) for i in range(20)]
    replays = engine.runner.num_graph_replays
    done = engine.generate(greedy(prompts, 3))
    assert engine.runner.num_graph_replays > replays
    for request, prompt in zip(done[:4], prompts):
        logits = qwen2_logits(config, weights, prompt + request.output_token_ids[:-1])[len(prompt) - 1:]
        for step, token in enumerate(request.output_token_ids):
            assert logits[step][token] >= logits[step].max() - 0.05  # the chosen token is the best one up to rounding


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_requests_that_take_over_a_published_prefix(tmp_path, dtype):
    """Prefix caching on the GPU, with captured decode steps: a request whose prompt begins like an earlier one computes
    only what follows the shared pages, and its tokens are those of the whole sequence through the plain model."""
    folder = make_folder(tmp_path, "A", dtype)
    config, weights = read_model_folder(folder)
    page = PAGE_SIZE["A"]
    stem = random_tokens(config["vocab_size"], 4 * page + 3, seed=31)
    prompts = [stem + random_tokens(config["vocab_size"], n, seed=60 + n) for n in (3, 1, 11, 6)]
    engine = engine_for(folder, "A", dtype, enable_prefix_caching=True, enable_cuda_graphs=True)
    assert engine.cache.prefix is not None
    first = engine.generate(greedy(prompts[:1], 10, prefix="first"))[0]
    rest = engine.generate(greedy(prompts[1:], 10, prefix="rest"))
    assert first.num_cached_tokens == 0 and [r.num_cached_tokens for r in rest] == [4 * page] * 3
    assert engine.runner.num_graph_replays > 0
    for request, prompt in zip([first] + rest, prompts):
        logits = qwen2_logits(config, weights, prompt + request.output_token_ids[:-1])[len(prompt) - 1:]
        for step, token in enumerate(request.output_token_ids):
            if dtype == "float32":
                assert int(logits[step].argmax()) == token
            else:
                assert logits[step][token] >= logits[step].max() - 0.05  # the best token up to rounding
    engine.cache.assert_consistent([])
    assert engine.cache.num_used_pages() == engine.cache.prefix.num_nodes > 0


def test_batches_of_every_size_class_with_layers_of_the_real_size(tmp_path):
    """bfloat16, two layers with the sizes of Qwen2.5-7B, captured decode steps: 40 requests decode together (the 64-row
    bucket: split-K products and the library), then 12 (the 16-row bucket: the fused decode kernels), then one.  Every
    chosen token has to be the plain model's best one up to rounding (see the replay test of the same sizes: the
    logits' error is about 1% of their spread of 1.2, eight times that for the worst of them)."""
    from test_replay_gpu import QWEN25_7B_TWO_LAYERS
    from velox_amd.weights import write_random_model

    folder = write_random_model(QWEN25_7B_TWO_LAYERS, str(tmp_path / "real_size"), 4, dtype="bfloat16")
    config, weights = read_model_folder(folder)
    engine = Engine.from_pretrained(EngineConfig(model=folder, dtype="bfloat16", device="cuda", max_model_len=64, max_num_seqs=64,
                                                 max_num_batched_tokens=256, max_prefill_chunk_size=128, num_gpu_blocks=300, seed=0))
    assert sorted(engine.runner._graphs) == [1, 2, 4, 8, 16, 32, 64]
    for count, seed in ((40, 200), (12, 300), (1, 400)):
        prompts = [random_tokens(config["vocab_size"], 3 + (i % 7), seed=seed + i) for i in range(count)]
        replays = engine.runner.num_graph_replays
        done = engine.generate(greedy(prompts, 5, prefix=f"n{count}-"))
        assert engine.runner.num_graph_replays >= replays + 4
        for request, prompt in list(zip(done, prompts))[::max(1, count // 6)]:
            logits = qwen2_logits(config, weights, prompt + request.output_token_ids[:-1])[len(prompt) - 1:]
            # a bfloat16 run's logits differ from the plain model's by at most 1.75% of their spread in the root mean square
            # (the bound the replayed logits at these widths are held to).  The engine's best token can then stand below
            # the plain best by the errors of two logits: six such deviations are allowed, far out for two chosen logits
            margin = 6 * 0.0175 * float(logits.std())
            for step, token in enumerate(request.output_token_ids):
                assert logits[step][token] >= logits[step].max() - margin, (count, request.request_id, step, margin)
    engine.cache.assert_consistent([])


def test_a_small_pool_with_shared_prefixes_captured_steps_and_early_launches(tmp_path):
    """float32 on the GPU with everything on at once: prefix caching, captured decode steps, the next step launched
    early, and a pool so small that requests are preempted and published pages evicted.  The tokens are the plain
    model's, request by request."""
    folder = make_folder(tmp_path, "B", "float32")
    config, weights = read_model_folder(folder)
    page = PAGE_SIZE["B"]
    stem = random_tokens(config["vocab_size"], 2 * page + 3, seed=9)
    prompts = [stem + random_tokens(config["vocab_size"], 4 + 3 * i, seed=20 + i) for i in range(7)]
    needed = max((len(p) + 14 + page - 1) // page for p in prompts)
    engine = engine_for(folder, "B", "float32", enable_prefix_caching=True, enable_cuda_graphs=True,
                        num_gpu_blocks=2 * needed + 3, max_model_len=needed * page)
    done = engine.generate(greedy(prompts, 14))
    for request, prompt in zip(done, prompts):
        assert request.output_token_ids == plain_greedy(config, weights, prompt, 14), request.request_id
    assert engine.scheduler.num_preemptions > 0 and engine.cache.prefix.num_hits > 0 and engine.runner.num_graph_replays > 0
    engine.cache.assert_consistent([])


def test_sampling_through_the_engine(tmp_path):
    folder = make_folder(tmp_path, "B")
    config, _ = read_model_folder(folder)
    prompts = [random_tokens(config["vocab_size"], n, seed=70 + n) for n in (1, 17, 40, 8)]

    def sampled(i, prompt, **kw):
        return Request(f"s{i}", prompt, SamplingParams(temperature=0.8, max_tokens=6, seed=100 + i, ignore_eos=True, **kw))

    engine = engine_for(folder, "B")
    together = engine.generate([sampled(i, p) for i, p in enumerate(prompts)])
    again = engine_for(folder, "B").generate([sampled(i, p) for i, p in enumerate(prompts)])
    assert [r.output_token_ids for r in together] == [r.output_token_ids for r in again]
    assert engine.generate([sampled(2, prompts[2])])[0].output_token_ids == together[2].output_token_ids
    greedy_alone = engine.generate(greedy([prompts[1]], 6, prefix="g-alone"))[0]
    mixed = engine.generate([sampled(7, prompts[0]), greedy([prompts[1]], 6, prefix="g-mixed")[0], sampled(8, prompts[3], top_k=5, top_p=0.9)])
    assert mixed[1].output_token_ids == greedy_alone.output_token_ids
    top1 = engine.generate([Request("k1", prompts[1], SamplingParams(temperature=1.5, top_k=1, max_tokens=6, ignore_eos=True))])[0]
    assert top1.output_token_ids == greedy_alone.output_token_ids
    # penalties over prompt plus output: the tokens that the plain model's logits give under the reference's formula; a
    # prompt that repeats few tokens makes the penalties decide (without them the tokens differ), beside a neighbour
    # with another history and other coefficients
    from torch_ops import TorchOps

    config, weights = read_model_folder(folder)
    histories = [[5, 9, 5, 9, 5, 9, 5, 9, 12, 5, 9], prompts[2]]
    coefficients = [dict(repetition_penalty=1.6, frequency_penalty=0.05, presence_penalty=0.02), dict(repetition_penalty=1.2, presence_penalty=0.03)]

    def plain_penalised(prompt, steps, repetition_penalty=1.0, presence_penalty=0.0, frequency_penalty=0.0):
        tokens = list(prompt)
        for _ in range(steps):
            logits = qwen2_logits(config, weights, tokens)[-1:].clone()
            TorchOps().apply_penalties(logits, torch.tensor([tokens]), torch.tensor([len(tokens)]),
                                       torch.tensor([[repetition_penalty, presence_penalty, frequency_penalty]]))
            tokens.append(int(logits[0].argmax()))
        return tokens[len(prompt):]

    penalised = engine.generate([Request(f"pen{i}", h, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True, **c))
                                 for i, (h, c) in enumerate(zip(histories, coefficients))])
    for request, history, c in zip(penalised, histories, coefficients):
        assert request.output_token_ids == plain_penalised(history, 10, **c), request.request_id
    assert penalised[0].output_token_ids != plain_penalised(histories[0], 10)  # the penalties changed what is chosen


def test_many_penalised_requests_admitted_in_one_step_with_captured_steps(tmp_path):
    """Forty short prompts with penalties finish their prompts in a handful of steps: each brings its history to the
    sampler's table of counts through the ring of pinned buffers (more uploads in one step than the ring has places),
    the table grows twice, decode steps are captured and launched ahead; every request gets the plain model's penalised
    tokens, and when all are done the sampler holds nothing."""
    from torch_ops import TorchOps

    folder = make_folder(tmp_path, "A")
    config, weights = read_model_folder(folder)
    vocab = config["vocab_size"]
    prompts = [[3 + i % 5, 9, 3 + i % 5, 9, 17] + random_tokens(vocab, 1 + i % 4, seed=300 + i) for i in range(40)]
    steps = 6

    def plain_penalised(prompt, repetition, presence, frequency):
        tokens = list(prompt)
        for _ in range(steps):
            logits = qwen2_logits(config, weights, tokens)[-1:].clone()
            TorchOps().apply_penalties(logits, torch.tensor([tokens]), torch.tensor([len(tokens)]), torch.tensor([[repetition, presence, frequency]]))
            tokens.append(int(logits[0].argmax()))
        return tokens[len(prompt):]

    engine = engine_for(folder, "A", max_num_seqs=40, max_num_batched_tokens=512, max_prefill_chunk_size=64, num_gpu_blocks=400, enable_cuda_graphs=True)
    coefficients = [(1.0 + 0.1 * (i % 7), 0.02 * (i % 3), 0.05 * (i % 4)) for i in range(40)]
    requests = [Request(f"many{i}", p, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True, repetition_penalty=c[0], presence_penalty=c[1],
                                                      frequency_penalty=c[2])) for i, (p, c) in enumerate(zip(prompts, coefficients))]
    done = engine.generate(requests)
    assert engine.runner.num_graph_replays > 0
    differs = 0
    for request, prompt, c in zip(done, prompts, coefficients):
        want = plain_penalised(prompt, *c)
        assert request.output_token_ids == want, (request.request_id, request.output_token_ids, want)
        differs += want != plain_greedy(config, weights, prompt, steps)
    assert differs > 10  # the penalties decide for many of them
    assert engine.sampler._seen.row_of_request == {} and engine.sampler._seen.table.shape[0] >= 40


def test_two_hundred_requests_of_every_kind_in_a_small_pool_and_in_a_roomy_one(tmp_path):
    """Greedy, penalised, sampled and sampled-with-penalties requests, some with stop tokens, some behind a shared stem,
    arriving in bursts: once with a pool so small that requests are preempted hundreds of times, captured decode steps,
    every step launched ahead and shared prefixes; once with room for all, one step at a time, nothing captured or
    shared.  float32, so both give every request the same tokens.  Then the same with requests aborted at random: the
    cache, the slots and the sampler's tables are left clean."""
    import random

    folder = make_folder(tmp_path, "B")
    config, _ = read_model_folder(folder)
    vocab = config["vocab_size"]

    def make_requests(tag, count, seed):
        rng = random.Random(seed)
        stem = [rng.randrange(vocab) for _ in range(40)]
        made = []
        for i in range(count):
            kind = rng.random()
            prompt = (stem[:rng.choice([0, 16, 32, 40])] if rng.random() < 0.5 else []) + [rng.randrange(vocab) for _ in range(rng.randint(1, 70))]
            options = dict(max_tokens=rng.randint(1, 40), ignore_eos=rng.random() < 0.7)
            if kind < 0.4:
                options.update(temperature=0.0)
            elif kind < 0.6:
                options.update(temperature=0.0, repetition_penalty=1.3, frequency_penalty=0.1)
            elif kind < 0.8:
                options.update(temperature=0.8, top_p=0.9, seed=i)
            else:
                options.update(temperature=0.7, top_k=20, top_p=0.8, repetition_penalty=1.05, seed=1000 + i)
            if rng.random() < 0.2:
                options["stop_token_ids"] = [rng.randrange(vocab) for _ in range(20)]
            made.append(Request(f"{tag}{i}", prompt, SamplingParams(**options)))
        return made

    def run(tag, count, seed, aborts, **options):
        engine = engine_for(folder, "B", max_num_seqs=8, max_num_batched_tokens=64, max_prefill_chunk_size=24, **options)
        requests = make_requests(tag, count, seed)
        rng = random.Random(seed + 1)
        waiting, steps = list(requests), 0
        while waiting or engine.has_work():
            if steps % 25 == 0:
                for _ in range(rng.randint(4, 14)):
                    if waiting:
                        engine.add_request(waiting.pop(0))
            if aborts and rng.random() < 0.05 and engine.scheduler.running:
                engine.abort_request(rng.choice(engine.scheduler.running).request_id)
            engine.step()
            steps += 1
            if steps % 100 == 0:
                engine.cache.assert_consistent([r.cache for r in engine.scheduler.running if r.cache is not None])
        engine.cache.assert_consistent([])
        assert engine.cache.num_used_pages() == (engine.cache.prefix.num_nodes if engine.cache.prefix is not None else 0)
        assert engine.sampler._seen.row_of_request == {} and engine.sampler._seeds == {}
        assert all(r.finished and -1 not in r.all_token_ids for r in requests)
        return requests, engine

    tight, engine = run("t", 200, 5, False, num_gpu_blocks=40, enable_cuda_graphs=True, decode_lookahead=True, enable_prefix_caching=True)
    assert engine.scheduler.num_preemptions > 50 and engine.runner.num_graph_replays > 100 and engine.cache.prefix.num_hits > 0
    roomy, _ = run("t", 200, 5, False, num_gpu_blocks=400, enable_cuda_graphs=False, decode_lookahead=False, enable_prefix_caching=False)
    for a, b in zip(tight, roomy):
        assert a.output_token_ids == b.output_token_ids and a.finish_reason is b.finish_reason, (a.request_id, a.sampling_params, a.output_token_ids, b.output_token_ids)
    aborted, _ = run("x", 200, 9, True, num_gpu_blocks=40, enable_cuda_graphs=True, decode_lookahead=True, enable_prefix_caching=True)
    assert sum(r.finish_reason.name == "ABORT" for r in aborted) > 10


def test_pool_sized_from_free_memory_when_no_page_count_is_given(tmp_path):
    """``num_gpu_blocks=None``: the pool takes what the free memory allows (reference ``src/paged_kv_cache.py:159-194``), capped at
    what ``max_num_seqs`` requests of ``max_model_len`` tokens can ever hold; a utilisation that leaves nothing is an error."""
    folder = make_folder(tmp_path, "A", "bfloat16")
    engine = engine_for(folder, "A", "bfloat16", num_gpu_blocks=None, gpu_memory_utilization=0.5, max_model_len=160, max_num_seqs=4)
    page = PAGE_SIZE["A"]
    assert engine.cache.num_total_pages == 4 * 160 // page  # the cap: far less than half of the card
    config, weights = read_model_folder(folder)
    prompt = random_tokens(config["vocab_size"], 30, seed=3)
    assert len(engine.generate(greedy([prompt], 6))[0].output_token_ids) == 6
    free_bytes, _ = torch.cuda.mem_get_info()
    from velox_amd.cache.manager import pages_that_fit

    with pytest.raises(RuntimeError, match="not enough free GPU memory"):
        pages_that_fit(engine.cache.bytes_per_page(), free_bytes, 0.5, free_bytes)
    # uncapped: a long context and many requests want more pages than fit in a sliver of the free memory
    small = engine_for(folder, "A", "bfloat16", num_gpu_blocks=None, gpu_memory_utilization=0.9, kv_cache_reserve_mb=0, max_model_len=512, max_num_seqs=32,
                       max_num_batched_tokens=64)
    wanted = 32 * 512 // page
    assert small.cache.num_total_pages == wanted  # still the cap on this card; the arithmetic below is what a small card would get
    assert pages_that_fit(small.cache.bytes_per_page(), 3 * small.cache.bytes_per_page() + 5, 1.0, 0) == 3


def test_command_line(tmp_path):
    folder = make_folder(tmp_path, "A", "bfloat16")
    out = tmp_path / "result.json"
    process = subprocess.run(
        [sys.executable, os.path.join(ROOT, "benchmark.py"), "--model", folder, "--num-requests", "5", "--max-tokens", "6", "--prompt-len", "11",
         "--max-model-len", "64", "--max-num-seqs", "4", "--max-num-batched-tokens", "32", "--max-prefill-chunk-size", "8", "--block-size", "4",
         "--num-gpu-blocks", "64", "--output-json", str(out), "--seed", "3"],
        capture_output=True, text=True, timeout=600)
    assert process.returncode == 0, process.stderr[-2000:]
    result = json.loads(out.read_text())[0]
    assert result["num_requests"] == 5 and result["generated_tokens"] == 30 and result["prompt_tokens"] == 55
    assert "Decode throughput" in process.stdout and "TTFT" in process.stdout
    records = result["requests"]  # one per request, as in the reference's JSON
    assert len(records) == 5 and all(r["prompt_tokens"] == 11 and r["generated_tokens"] == 6 for r in records)
    assert all(0 < r["ttft"] <= r["end_to_end"] <= result["wall_seconds"] for r in records) and "outputs" not in result
    assert sorted(records[0]) == ["cached_prompt_tokens", "end_to_end", "generated_tokens", "id", "prompt_tokens", "ttft"]
