"""Replay on the GPU, float32 and bfloat16: each request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size down to two tokens; mixed, up to four live requests in a pool so
small that pages are used again; long decoding; the first tokens of a sequence; sharpened attention; the program
itself as a user starts it."""
import json
import os
import subprocess
import sys

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
                         ("portions", rc.changing_portions(requests)), ("mixed", rc.mixed(requests, seed=5))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page)
        results[label] = rc.collect(trace, rc.run_trace(replayer, trace), requests)
        for rid in requests:
            torch.testing.assert_close(results[label][rid], expected[rid], msg=lambda m: f"{name} {dtype} {label} {rid}: {m}", **TOL[dtype])
        if label == "mixed":
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
    if dtype == "float32":
        # the ways of cutting agree with each other much closer than any of them must with the plain model
        for label in ("tail", "portions", "mixed"):
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], rtol=5e-5, atol=5e-6)


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
