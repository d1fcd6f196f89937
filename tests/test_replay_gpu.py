"""Replay on the GPU, float32 and bfloat16: each request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size down to two tokens; mixed, up to four live requests in a pool so
small that pages are used again; long decoding; the first tokens of a sequence; sharpened attention; the program
itself as a user starts it."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import replay_cases as rc
from helpers import CONFIGS, PAGE_SIZE, make_folder, random_tokens
from plain_qwen2 import qwen2_logits, read_model_folder
from velox_amd.engine.replay import Replayer

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# float32: summation order is the only difference.  bfloat16: activations are rounded to 8 bits of mantissa
# between kernels; logits of these models are of order one.
TOL = {"float32": dict(rtol=2e-4, atol=2e-5), "bfloat16": dict(rtol=5e-2, atol=3e-2)}


def storage_for(dtype):
    return "float32" if dtype == "float32" else "bfloat16"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_four_ways_of_cutting(tmp_path, name, dtype):
    folder = make_folder(tmp_path, name, storage_for(dtype))
    config, weights = read_model_folder(folder)
    requests = rc.request_set(config["vocab_size"], [141, 37, 98, 64, 75, 33, 120], seed=11)
    expected = rc.expected_logits(config, weights, requests)
    page = PAGE_SIZE[name]
    results = {}
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)),
                         ("portions", rc.changing_portions(requests)), ("mixed", rc.mixed(requests, seed=5)),
                         ("recompute", rc.mixed(requests, seed=8, preempt=("r0", "r2", "r6")))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page)
        outputs = rc.run_trace(replayer, trace)
        results[label] = rc.collect(trace, outputs, requests)
        for rid in requests:
            torch.testing.assert_close(results[label][rid], expected[rid], msg=lambda m: f"{name} {dtype} {label} {rid}: {m}", **TOL[dtype])
        if label in ("mixed", "recompute"):
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
        if label == "recompute":
            # requests ended half way, their pages taken by others, then fed again from their first token under the same
            # id (what preemption does): the first run's logits were right too, and the second run's match them
            first = rc.first_runs(trace, outputs, requests)
            for rid in ("r0", "r2", "r6"):
                assert sum(1 for r in trace if rid in r["end"]) == 2 and len(first[rid]) >= len(requests[rid]) // 2
                for position, row in first[rid].items():
                    torch.testing.assert_close(torch.from_numpy(row.copy()), expected[rid][position], **TOL[dtype])
    if dtype == "float32":
        # the ways of cutting agree with each other much closer than any of them must with the plain model
        for label in ("tail", "portions", "mixed", "recompute"):
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], rtol=5e-5, atol=5e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", [21, 22, 23, 24, 25, 26])
def test_mixed_traces_in_more_random_orders(tmp_path, seed, dtype):
    """Other orders of arrival, other cuts and other requests that are ended half way and fed again, one configuration
    per seed: up to four live requests, portions beside single tokens, a pool smaller than the requests' sum."""
    name = "ABC"[seed % 3]
    folder = make_folder(tmp_path, name, storage_for(dtype))
    config, weights = read_model_folder(folder)
    lengths = [33 + (seed * 7 + 29 * i) % 110 for i in range(8)]
    requests = rc.request_set(config["vocab_size"], lengths, seed=seed)
    expected = rc.expected_logits(config, weights, requests)
    page = PAGE_SIZE[name]
    again = tuple(f"r{i}" for i in range(8) if (seed + i) % 3 == 0)
    trace = rc.mixed(requests, seed=seed, preempt=again)
    replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page)
    got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
    for rid in requests:
        torch.testing.assert_close(got[rid], expected[rid], msg=lambda m: f"{name} {dtype} seed {seed} {rid}: {m}", **TOL[dtype])
    assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
    replayer.cache.assert_consistent([])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_first_tokens(tmp_path, dtype):
    folder = make_folder(tmp_path, "B", storage_for(dtype))
    config, weights = read_model_folder(folder)
    requests = {"long": random_tokens(320, 300, 1), "one": [7], "two": [9, 3], "three": [1, 2, 3]}
    expected = rc.expected_logits(config, weights, requests)
    trace = []
    for rid, toks in requests.items():  # everything one token at a time
        for i, t in enumerate(toks):
            trace.append({"step": len(trace), "entries": [{"id": rid, "tokens": [t], "want": [0]}], "end": [rid] if i == len(toks) - 1 else []})
    replayer = Replayer(folder, dtype, rc.tokens_needed(trace, 8), block_size=8)
    got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
    for rid in requests:
        torch.testing.assert_close(got[rid], expected[rid], msg=lambda m: f"{rid}: {m}", **TOL[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharpened_attention_shows_far_keys_and_page_edges(tmp_path, dtype):
    """Queries and keys of every layer scaled up so that single scores stand out: a key read from the wrong
    page, a wrong position or a stale page then changes the logits by far more than rounding."""
    folder = make_folder(tmp_path, "A", storage_for(dtype))
    path = os.path.join(folder, "model.safetensors")
    raw = load_file(path)
    for layer in range(2):
        for proj in ("q_proj", "k_proj"):
            for kind in ("weight", "bias"):
                key = f"model.layers.{layer}.self_attn.{proj}.{kind}"
                raw[key] = (raw[key].float() * 6.0).to(raw[key].dtype)
    save_file(raw, path)
    config, weights = read_model_folder(folder)
    requests = rc.request_set(256, [333, 47, 200, 129], seed=23)
    expected = rc.expected_logits(config, weights, requests)
    probs = torch.softmax(expected["r0"], -1)
    for label, trace in (("portions", rc.changing_portions(requests)), ("mixed", rc.mixed(requests, seed=9)), ("tail", rc.tail_one_by_one(requests))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, 4), block_size=4)
        got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
        for rid in requests:
            torch.testing.assert_close(got[rid], expected[rid], msg=lambda m: f"{dtype} {label} {rid}: {m}", **TOL[dtype])


def test_trace_run_program(tmp_path):
    folder = make_folder(tmp_path, "B", "bfloat16")
    config, weights = read_model_folder(folder)
    requests = rc.request_set(320, [70, 45, 90], seed=31)
    expected = rc.expected_logits(config, weights, requests)
    trace = rc.mixed(requests, seed=2)
    trace[3]["entries"][0]["want"] = []  # a step may want nothing of an entry
    wanted_steps = [r["step"] for r in trace if any(e["want"] for e in r["entries"])]
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / f"out_{dtype}"
        process = subprocess.run(
            [os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out_dir), "--max-tokens", str(rc.tokens_needed(trace, 64))],
            input="".join(json.dumps(r) + "\n" for r in trace), capture_output=True, text=True, timeout=600,
        )
        assert process.returncode == 0, process.stderr[-2000:]
        assert [line for line in process.stdout.splitlines() if line.startswith("done")] == [f"done {r['step']}" for r in trace]
        vocab = config["vocab_size"]
        outputs = {s: np.fromfile(out_dir / f"{s}.f32", dtype="<f4").reshape(-1, vocab) for s in wanted_steps}
        assert sorted(int(p.stem) for p in out_dir.iterdir()) == wanted_steps
        # positions that were asked for agree with the plain model
        at = {rid: 0 for rid in requests}
        for record in trace:
            row = 0
            for entry in record["entries"]:
                for w in entry["want"]:
                    torch.testing.assert_close(torch.from_numpy(outputs[record["step"]][row]), expected[entry["id"]][at[entry["id"]] + w], **TOL[dtype])
                    row += 1
                at[entry["id"]] += len(entry["tokens"])


QWEN25_7B_TWO_LAYERS = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "use_sliding_window": False, "max_position_embeddings": 32768,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_the_real_size_in_four_ways_of_cutting(tmp_path, dtype):
    """Two layers with the sizes of Qwen2.5-7B (width 3584, 28 heads over 4 groups of size 128, 18944 inner columns, a
    vocabulary of 152064): the sizes at which the decode kernels, the library's products and the wide attention kernel
    take other paths than with the tiny models.  One engine serves all four traces, so pages are used again between
    them as well."""
    from velox_amd.weights import write_random_model

    folder = write_random_model(QWEN25_7B_TWO_LAYERS, str(tmp_path / "real_size"), 3, dtype=storage_for(dtype))
    config, weights = read_model_folder(folder)
    requests = rc.request_set(config["vocab_size"], [97, 33, 150, 64], seed=41)
    expected = rc.expected_logits(config, weights, requests)
    traces = {"whole": rc.whole(requests), "tail": rc.tail_one_by_one(requests), "portions": rc.changing_portions(requests),
              "mixed": rc.mixed(requests, seed=6)}
    replayer = Replayer(folder, dtype, max(rc.tokens_needed(t, 16) for t in traces.values()), block_size=16)
    if dtype == "float32":
        # Sums of 3584 and 18944 float32 terms round differently in every order of adding, more than the tiny models'
        # sums of a hundred terms do.  The yardstick is the plain model's own float32 rounding, measured against the same
        # model in float64: the engine has to be as close to the exact logits as the plain float32 implementation is.
        exact = {rid: qwen2_logits(config, weights, tokens, dtype=torch.float64) for rid, tokens in requests.items()}
        rounding = max(float((expected[rid].double() - exact[rid]).abs().max()) for rid in requests)
        assert 1e-6 < rounding < 2e-4, rounding
        tol = dict(rtol=0.0, atol=3 * rounding)
        expected = {rid: exact[rid].float() for rid in requests}
    results = {}
    for label, trace in traces.items():
        results[label] = rc.collect(trace, rc.run_trace(replayer, trace), requests)
        for rid in requests:
            if dtype == "float32":
                torch.testing.assert_close(results[label][rid], expected[rid], msg=lambda m: f"{dtype} {label} {rid}: {m}", **tol)
                continue
            # bfloat16: about twenty tensors on the way to a logit are rounded to 8 bits (relative error up to 2^-9 each,
            # independent): the logits' error is then about 2^-9 * sqrt(20) = 0.9% of their spread in the root mean
            # square, whatever the width.  Twice that is allowed, and eight such deviations for the worst of the 15
            # million logits; a key read from a wrong place or a wrong position changes logits by their whole spread.
            spread = float(expected[rid].std())
            error = results[label][rid] - expected[rid]
            assert float(error.pow(2).mean().sqrt()) < 0.0175 * spread, (label, rid, float(error.pow(2).mean().sqrt()), spread)
            assert float(error.abs().max()) < 8 * 0.0175 * spread, (label, rid, float(error.abs().max()), spread)
    if dtype == "float32":
        for label in ("tail", "portions", "mixed"):
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], **tol)


OTHER_REAL_WIDTHS = {
    # two layers each; the vocabulary is cut down (and made odd), it does not touch the layers' kernels
    "qwen2.5-1.5b": dict(num_hidden_layers=2, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                         vocab_size=32003, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True),
    "qwen2.5-32b": dict(num_hidden_layers=2, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=27648,
                        vocab_size=32003, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False),
}


def test_a_prompt_of_2048_tokens_in_true_32_bit_at_the_real_width(tmp_path):
    """float32 at the widths of Qwen2.5-7B and at the prompt length the measurements use: ONE portion of 2,048 tokens (the
    exact product with 2,048 rows and inner sizes of 3584 and 18944, the 32-bit attention kernel with a head size of 128
    over a 2,048-row portion), then eight single tokens.  Two layers; the vocabulary is cut down and made odd.  The
    yardstick is the plain model in float64: the engine has to be as close to it as three times the plain float32
    model's own rounding."""
    from velox_amd.weights import write_random_model

    config = dict(QWEN25_7B_TWO_LAYERS, vocab_size=32003)
    folder = write_random_model(config, str(tmp_path / "real_width"), 5, dtype="float32")
    config, weights = read_model_folder(folder)
    tokens = random_tokens(config["vocab_size"], 2056, seed=15)
    places = [0, 1, 15, 16, 17, 511, 1023, 1024, 2031, 2032, 2046, 2047]  # of the portion: page edges, tile edges, the ends
    exact = qwen2_logits(config, weights, tokens, dtype=torch.float64)
    plain = qwen2_logits(config, weights, tokens)
    rounding = float((plain.double() - exact).abs().max())
    assert 1e-6 < rounding < 2e-4, rounding
    replayer = Replayer(folder, "float32", 2112, block_size=16)
    first = replayer.step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:2048], "want": places}], "end": []})
    rest = [replayer.step({"step": 1 + i, "entries": [{"id": "a", "tokens": [tokens[2048 + i]], "want": [0]}], "end": []}) for i in range(8)]
    got = torch.from_numpy(np.concatenate([first] + rest)).double()
    want = torch.cat([exact[places], exact[2048:]])
    assert float((got - want).abs().max()) < 3 * rounding, (float((got - want).abs().max()), rounding)
    assert float(want.std()) > 100 * rounding  # (the logits' spread: the bound is a small share of it)


@pytest.mark.parametrize("shape", sorted(OTHER_REAL_WIDTHS))
def test_layers_of_the_other_real_sizes(tmp_path, shape):
    """bfloat16, two layers with the widths of Qwen2.5-1.5B and of Qwen2.5-32B: the products' kernels are picked by width and
    by the number of rows (up to 16, up to 32, up to 64, more), and these are the widths the picking was measured at.  Whole
    prompts, portions of changing size, single tokens, and 20 requests decoding together through a captured step, against
    the plain model, to the bound that the 7B widths are held to."""
    from velox_amd.weights import write_random_model

    config = dict(OTHER_REAL_WIDTHS[shape], architectures=["Qwen2ForCausalLM"], model_type="qwen2", use_sliding_window=False, max_position_embeddings=4096)
    folder = write_random_model(config, str(tmp_path / shape), 9, dtype="bfloat16")
    config, weights = read_model_folder(folder)
    requests = rc.request_set(config["vocab_size"], [70, 33, 121] + [18 + (5 * i) % 13 for i in range(20)], seed=81)
    expected = rc.expected_logits(config, weights, requests)
    names = list(requests)
    few = {rid: requests[rid] for rid in names[:3]}
    crowd = names[3:]
    together = []  # the crowd: prompts eight at a time without their last five tokens, then five steps of 20 single tokens
    for lo in range(0, len(crowd), 8):
        together.append({"step": len(together), "end": [], "entries": [{"id": rid, "tokens": requests[rid][:-5], "want": list(range(len(requests[rid]) - 5))} for rid in crowd[lo:lo + 8]]})
    for i in range(5):
        together.append({"step": len(together), "end": crowd if i == 4 else [],
                         "entries": [{"id": rid, "tokens": [requests[rid][len(requests[rid]) - 5 + i]], "want": [0]} for rid in crowd]})
    traces = {"tail": rc.tail_one_by_one(few), "portions": rc.changing_portions(few, sizes=(40, 2, 17, 33, 1, 64)), "mixed": rc.mixed(few, seed=3),
              "together": together}
    replayer = Replayer(folder, "bfloat16", max(rc.tokens_needed(t, 16) for t in traces.values()), block_size=16, max_live=32, enable_graphs=True)
    for label, trace in traces.items():
        subset = {rid: requests[rid] for rid in (crowd if label == "together" else few)}
        got = rc.collect(trace, rc.run_trace(replayer, trace), subset)
        for rid in subset:
            spread = float(expected[rid].std())
            error = got[rid] - expected[rid]
            assert float(error.pow(2).mean().sqrt()) < 0.0175 * spread, (shape, label, rid, float(error.pow(2).mean().sqrt()), spread)
            assert float(error.abs().max()) < 8 * 0.0175 * spread, (shape, label, rid, float(error.abs().max()), spread)
    assert replayer.runner.num_graph_replays >= 5


@pytest.mark.parametrize("live", [40, 12])
def test_captured_decode_steps_of_many_requests_at_the_real_size(tmp_path, live):
    """40 and 12 requests decode together through the captured steps of 64 and 16 rows, at the widths of Qwen2.5-7B:
    the products of 17 to 64 rows (split sums, the library's kernels), the decode attention with many sequences and rows
    padded onto the null page.  Logits of every decoded position against the plain model, to the bound of the test above."""
    from velox_amd.weights import write_random_model

    folder = write_random_model(QWEN25_7B_TWO_LAYERS, str(tmp_path / "real_size"), 3, dtype="bfloat16")
    config, weights = read_model_folder(folder)
    decoded = 6
    lengths = [20 + (7 * i) % 23 for i in range(live)]
    requests = rc.request_set(config["vocab_size"], lengths, seed=61)
    trace = []
    names = list(requests)
    for lo in range(0, live, 8):  # prompts, eight requests a step, all but the last `decoded` tokens
        trace.append({"step": len(trace), "end": [],
                      "entries": [{"id": rid, "tokens": requests[rid][:len(requests[rid]) - decoded], "want": []} for rid in names[lo:lo + 8]]})
    for i in range(decoded):
        trace.append({"step": len(trace), "end": names if i == decoded - 1 else [],
                      "entries": [{"id": rid, "tokens": [requests[rid][len(requests[rid]) - decoded + i]], "want": [0]} for rid in names]})
    replayer = Replayer(folder, "bfloat16", rc.tokens_needed(trace, 16), block_size=16, max_live=64, enable_graphs=True)
    assert replayer.runner.uses_graphs
    outputs = rc.run_trace(replayer, trace)
    assert replayer.runner.num_graph_replays == decoded
    eager = Replayer(folder, "bfloat16", rc.tokens_needed(trace, 16), block_size=16, max_live=64, enable_graphs=False, ops=replayer.ops)
    eager_outputs = rc.run_trace(eager, trace)
    for index, rid in enumerate(names):
        expected = qwen2_logits(config, weights, requests[rid])[-decoded:]
        got = torch.stack([torch.from_numpy(outputs[len(trace) - decoded + i][index].copy()) for i in range(decoded)])
        spread = float(expected.std())
        error = got - expected
        assert float(error.pow(2).mean().sqrt()) < 0.0175 * spread, (rid, float(error.pow(2).mean().sqrt()), spread)
        assert float(error.abs().max()) < 8 * 0.0175 * spread, (rid, float(error.abs().max()), spread)
        # a captured step pads to 16 or 64 rows and may take other kernels than the same step uncaptured (the rows decide):
        # the two agree as two bfloat16 runs do
        same = torch.stack([torch.from_numpy(eager_outputs[len(trace) - decoded + i][index].copy()) for i in range(decoded)])
        assert float((got - same).pow(2).mean().sqrt()) < 0.0175 * spread


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_context_in_large_portions_then_token_by_token(tmp_path, dtype):
    """6,000 tokens: portions of 2,048 behind thousands of cached keys (the wide attention kernel and the one with two
    sets of waves), then single tokens over a key range that is split many ways, beside a short request that decodes
    in the same steps.  Queries and keys are sharpened so that a far key read wrongly shows."""
    from velox_amd.weights import write_random_model

    config = dict(CONFIGS["A"], max_position_embeddings=8192)
    folder = write_random_model(config, str(tmp_path / "long"), 7, dtype=storage_for(dtype))
    path = os.path.join(folder, "model.safetensors")
    raw = load_file(path)
    for layer in range(2):
        for proj in ("q_proj", "k_proj"):
            key = f"model.layers.{layer}.self_attn.{proj}.weight"
            raw[key] = (raw[key].float() * 4.0).to(raw[key].dtype)
    save_file(raw, path)
    config, weights = read_model_folder(folder)
    long_tokens = random_tokens(256, 6000, seed=77)
    short_tokens = random_tokens(256, 40, seed=78)
    expected = {"long": qwen2_logits(config, weights, long_tokens), "short": qwen2_logits(config, weights, short_tokens)}
    trace, at = [], 0
    for size in (2048, 2048, 1872):
        trace.append({"step": len(trace), "entries": [{"id": "long", "tokens": long_tokens[at:at + size], "want": [0, size // 2, size - 1]}], "end": []})
        at += size
    trace.append({"step": len(trace), "entries": [{"id": "short", "tokens": short_tokens[:8], "want": [7]}], "end": []})
    for i in range(32):
        trace.append({"step": len(trace), "entries": [{"id": "long", "tokens": [long_tokens[at + i]], "want": [0]},
                                                      {"id": "short", "tokens": [short_tokens[8 + i]], "want": [0]}],
                      "end": ["long", "short"] if i == 31 else []})
    assert at + 32 == 6000
    replayer = Replayer(folder, dtype, rc.tokens_needed(trace, 4), block_size=4)
    outputs = rc.run_trace(replayer, trace)
    held = {"long": 0, "short": 0}
    for record in trace:
        row = 0
        for entry in record["entries"]:
            for w in entry["want"]:
                got = torch.from_numpy(outputs[record["step"]][row].copy())
                torch.testing.assert_close(got, expected[entry["id"]][held[entry["id"]] + w],
                                           msg=lambda m: f"{dtype} step {record['step']} {entry['id']} position {held[entry['id']] + w}: {m}", **TOL[dtype])
                row += 1
            held[entry["id"]] += len(entry["tokens"])


ODD_CONFIGS = {
    # one KV head of size 256 for two query heads, pages of 64 tokens
    "wide_heads": dict(num_hidden_layers=2, hidden_size=512, num_attention_heads=2, num_key_value_heads=1, intermediate_size=384,
                       vocab_size=777, rope_theta=20000.0, rms_norm_eps=1e-5, tie_word_embeddings=True, page=64),
    # 18 query heads on one KV head (more rows than one tile of 16), inner width and vocabulary that no tile divides, pages of 2
    "large_group": dict(num_hidden_layers=2, hidden_size=288, num_attention_heads=18, num_key_value_heads=1, intermediate_size=100,
                        vocab_size=1001, rope_theta=1e5, rms_norm_eps=1e-3, tie_word_embeddings=False, page=2),
    # heads whose sizes add up to more than the width, every head with keys of its own
    "own_head_size": dict(num_hidden_layers=3, hidden_size=104, num_attention_heads=5, num_key_value_heads=5, head_dim=64,
                          intermediate_size=72, vocab_size=90, rope_theta=300.0, rms_norm_eps=1e-6, tie_word_embeddings=False, page=32),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD_CONFIGS))
def test_sizes_at_the_edges_of_what_the_kernels_take(tmp_path, name, dtype):
    from velox_amd.weights import write_random_model

    config = dict(ODD_CONFIGS[name], architectures=["Qwen2ForCausalLM"], model_type="qwen2", use_sliding_window=False, max_position_embeddings=512)
    page = config.pop("page")
    folder = write_random_model(config, str(tmp_path / name), 5, dtype=storage_for(dtype))
    config, weights = read_model_folder(folder)
    requests = rc.request_set(config["vocab_size"], [83, 40, 130], seed=51)
    expected = rc.expected_logits(config, weights, requests)
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)), ("mixed", rc.mixed(requests, seed=4, max_live=2))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, max(page, 64)), block_size=page)
        got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
        for rid in requests:
            torch.testing.assert_close(got[rid], expected[rid], msg=lambda m: f"{name} {dtype} {label} {rid}: {m}", **TOL[dtype])
