#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, as one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

A "step" is one decode step of the whole engine loop (scheduler, one forward over the batch,
sampling, the host's read of the sampled tokens).  The default run has the layer sizes of
Qwen2.5-7B with random weights N(0, 0.02), a batch of 8 and a context of 4096 tokens: the
requests are prefilled through the engine so that they reach the context length at the last
timed step.  ``value`` is decoded tokens per second.  The same line carries the prefill of one
2,048-token prompt (mean of the repeats), the decode step's share of the HBM roofline, and under
``points``: decode at batch 1 and 64 at the same context, a sampled decode step (temperature 0.8,
top-p 0.9) at batch 64, and the reference's own decode workload, batches of 1, 8 and 64 requests
with 512-token prompts that generate 256 tokens each (``decode_b<B>_p512_g256``: batch / mean step
over the steps in which all of them decode, ``..._frac``: that step's share of the HBM roofline,
``e2e_b<B>_p512_g256``: generated tokens / wall time with the prompts' time included, which is how
the reference's ``benchmark.py:204`` counts).
"""
from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM_GBS = 8000.0
SLACK = 512  # requests whose prompt is done first decode on while the others' prompts are still being read
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN25_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "use_sliding_window": False, "max_position_embeddings": 32768,
}
# the other two shapes the reference is quoted on (--shape): the headline stays the 7B shape
SHAPES = {
    "7b": ("Qwen2.5-7B shape", QWEN25_7B),
    "1.5b": ("Qwen2.5-1.5B shape", dict(QWEN25_7B, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                                          vocab_size=151936, tie_word_embeddings=True)),
    "32b": ("Qwen2.5-32B shape", dict(QWEN25_7B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8,
                                        intermediate_size=27648, rms_norm_eps=1e-6)),
}


def linear_params_per_layer(c):
    h, nh, nkv, inter = c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"], c["intermediate_size"]
    d = c.get("head_dim") or h // nh
    return h * (nh + 2 * nkv) * d + nh * d * h + 3 * h * inter


def decode_bytes(c, layers, batch, context, elem):
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    h, nh, nkv = c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"]
    d = c.get("head_dim") or h // nh
    per_layer = linear_params_per_layer(c) * elem + (nh + 2 * nkv) * d * 4 + 2 * h * 4
    weights = layers * per_layer + c["vocab_size"] * h * elem + h * 4 + batch * h * elem
    cache = batch * context * layers * 2 * nkv * d * elem
    return weights + cache


def prefill_flops(c, layers, tokens):
    h, nh = c["hidden_size"], c["num_attention_heads"]
    d = c.get("head_dim") or h // nh
    linear = 2 * tokens * layers * linear_params_per_layer(c)
    attention = layers * 2 * tokens * tokens * nh * d  # QK^T and PV over the causal half
    head = 2 * h * c["vocab_size"]
    return linear + attention + head


def make_engine(model_config, dtype, batch, context, chunk, graphs, seed=0):
    from velox_amd import Engine, EngineConfig

    max_len = context + SLACK
    pages = batch * ((max_len + 15) // 16 + 1) + (chunk + 15) // 16 + 64
    return Engine.from_random(
        model_config, seed,
        EngineConfig(dtype=dtype, device="cuda:0", max_model_len=max_len, max_num_seqs=batch,
                     max_num_batched_tokens=max(chunk, batch), max_prefill_chunk_size=chunk, block_size=16,
                     num_gpu_blocks=pages, enable_cuda_graphs=graphs, enable_prefix_caching=False, seed=seed),
        generator_device="cuda",
    )


def time_decode(engine, vocab, batch, context, steps, warmup, seed=0, sampling=None):
    """Reads ``batch`` prompts in through the engine, then times ``steps`` steps in which every request decodes.
    Every request holds at least ``context`` tokens at the last timed step (those admitted first a few more).
    Returns (seconds per step, mean tokens in the cache per request over the timed steps)."""
    import random

    import torch

    from velox_amd import Request, SamplingParams
    from velox_amd.engine.request import RequestStatus

    rng = random.Random(seed)
    prompt_len = max(1, context - steps - warmup)
    requests = [
        Request(f"decode-{batch}-{i}-{bool(sampling)}", [rng.randrange(vocab) for _ in range(prompt_len)],
                SamplingParams(max_tokens=steps + warmup + SLACK - 1, ignore_eos=True, **(sampling or {"temperature": 0.0})))
        for i in range(batch)
    ]
    for request in requests:
        engine.add_request(request)
    while any(r.status is not RequestStatus.RUNNING_DECODE for r in requests):
        engine.step()
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    before = [len(r.output_token_ids) for r in requests]
    held = sum(r.num_computed_tokens for r in requests)
    start = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    assert all(len(r.output_token_ids) == n + steps for r, n in zip(requests, before)), "a timed step did not decode one token per request"
    mean_context = (held / batch) + (steps + 1) / 2
    for request in requests:
        engine.abort_request(request.request_id)
    return elapsed / steps, mean_context


def time_workload(engine, vocab, batch, prompt_len, generated, seed=2):
    """The reference's decode benchmark: ``batch`` requests with prompts of ``prompt_len`` random tokens generate
    ``generated`` tokens each.  Returns (seconds per step over the steps in which all of them decode, mean tokens in the
    cache per request over those steps, generated tokens per second of wall time from the first add to the last token)."""
    import random

    import torch

    from velox_amd import Request, SamplingParams
    from velox_amd.engine.request import RequestStatus

    rng = random.Random(seed)
    requests = [Request(f"work-{batch}-{i}", [rng.randrange(vocab) for _ in range(prompt_len)],
                        SamplingParams(temperature=0.0, max_tokens=generated, ignore_eos=True)) for i in range(batch)]
    torch.cuda.synchronize()
    wall_start = time.perf_counter()
    for request in requests:
        engine.add_request(request)
    while any(r.status is not RequestStatus.RUNNING_DECODE for r in requests):
        engine.step()
    torch.cuda.synchronize()
    held = sum(r.num_computed_tokens for r in requests)
    steps = 0
    start = time.perf_counter()
    while not any(len(r.output_token_ids) >= generated - 1 for r in requests):  # (a step ahead may be in flight: stop one short)
        engine.step()
        steps += 1
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    while engine.has_work():
        engine.step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - wall_start
    assert all(len(r.output_token_ids) == generated for r in requests)
    return elapsed / steps, held / batch + (steps + 1) / 2, batch * generated / wall


def time_prefill(engine, vocab, tokens, repeats=3, seed=1):
    import random

    import torch

    from velox_amd import Request, SamplingParams

    rng = random.Random(seed)
    times = []
    for attempt in range(repeats + 1):
        request = Request(f"prefill-{attempt}", [rng.randrange(vocab) for _ in range(tokens)],
                          SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True))
        engine.add_request(request)
        torch.cuda.synchronize()
        start = time.perf_counter()
        engine.step()  # the whole prompt in one step, logits of the last row, one sampled token
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        assert len(request.output_token_ids) == 1, "the prompt did not prefill in one step"
        engine.step()  # reaps the finished request
        if attempt > 0:
            times.append(elapsed)
    return sum(times) / len(times), min(times)


def far_points(model_config, layers, args) -> dict:
    """Sizes beyond the headline's, each with its share of the roofline: decode behind a long context, a long prefill,
    and the true 32-bit path's decode step.  Engines are built one after the other (the first is given up)."""
    import gc

    import torch

    out = {}
    vocab = model_config["vocab_size"]
    elem = 2 if args.dtype == "bf16" else 4
    gc.collect()
    torch.cuda.empty_cache()
    long_context = 32256
    far = make_engine(model_config, args.dtype, 8, long_context, 8192, not args.no_graphs)
    for batch in (1, 8):
        each_s, mean_context = time_decode(far, vocab, batch, long_context, 16, 4)
        out[f"decode_b{batch}_ctx{long_context}"] = round(batch / each_s, 2)
        out[f"decode_b{batch}_ctx{long_context}_frac"] = round(decode_bytes(model_config, layers, batch, mean_context, elem) / each_s / 1e9 / PEAK_HBM_GBS, 4)
    long_s, _ = time_prefill(far, vocab, 8192, repeats=2)
    out["prefill_8192_tok_s"] = round(8192 / long_s, 1)
    out["prefill_8192_frac"] = round(prefill_flops(model_config, layers, 8192) / long_s / PEAK_FLOPS[args.dtype], 4)
    far.abort_all()
    del far
    gc.collect()
    torch.cuda.empty_cache()
    if args.dtype == "bf16":
        exact = make_engine(model_config, "fp32", 8, args.context, 512, not args.no_graphs)
        each_s, mean_context = time_decode(exact, vocab, 8, args.context, 16, 4)
        out["decode_b8_fp32"] = round(8 / each_s, 2)
        out["decode_b8_fp32_frac"] = round(decode_bytes(model_config, layers, 8, mean_context, 4) / each_s / 1e9 / PEAK_HBM_GBS, 4)
        exact.abort_all()
    return out


def main() -> int:
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (both numbers are reported)")
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096)
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--no-graphs", action="store_true")
    parser.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    parser.add_argument("--no-tune", action="store_true", help="do not let the matrix library pick its kernels for the prefill shapes")
    parser.add_argument("--no-probes", action="store_true", help="skip the probes of what the card delivers (streaming read, bfloat16 matrix instructions)")
    parser.add_argument("--shape", default="7b", choices=sorted(SHAPES), help="layer sizes: the headline is 7b; 1.5b and 32b are the reference's other two")
    parser.add_argument("--far", action="store_true",
                        help="further sizes under `points`: decode at batch 1 and 8 behind 32,256 tokens, a prefill of 8,192 tokens, and a decode step of a true float32 run (batch 8)")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine (single-GPU tier)")
        return 2

    import torch

    shape_name, shape = SHAPES[args.shape]
    model_config = dict(shape)
    full_layers = model_config["num_hidden_layers"]
    layers = args.layers or full_layers
    model_config["num_hidden_layers"] = layers
    elem = 2 if args.dtype == "bf16" else 4
    vocab = model_config["vocab_size"]
    graphs = not args.no_graphs
    batches = [args.batch] if args.no_points else sorted({1, args.batch, 64})

    engine = make_engine(model_config, args.dtype, max(batches), args.context, args.prefill_tokens, graphs)
    from velox_amd.engine.runner import decode_buckets

    # the library picks its kernels for the prefill's rows and for the decode batches it serves (graph buckets above 16 rows)
    tuned = 0 if args.no_tune else engine.tune_matrix_products([args.prefill_tokens] + [b for b in decode_buckets(max(batches)) if b > 16])
    step_s, contexts = {}, {}
    for batch in batches:
        steps = args.steps if batch == args.batch else max(8, args.steps // 2)
        step_s[batch], contexts[batch] = time_decode(engine, vocab, batch, args.context, steps, args.warmup)
    points = {f"decode_b{b}": round(b / t, 2) for b, t in step_s.items() if b != args.batch}
    if not args.no_points:
        sampled_s, _ = time_decode(engine, vocab, 64, args.context, max(8, args.steps // 2), args.warmup, sampling={"temperature": 0.8, "top_p": 0.9, "seed": 7})
        points["decode_b64_sampled"] = round(64 / sampled_s, 2)
        # the sampling options that Qwen2.5's own generation settings name: a filter of both kinds and a repetition penalty
        penalised_s, _ = time_decode(engine, vocab, 64, args.context, max(8, args.steps // 2), args.warmup,
                                     sampling={"temperature": 0.7, "top_p": 0.8, "top_k": 20, "repetition_penalty": 1.05, "seed": 7})
        points["decode_b64_sampled_penalised"] = round(64 / penalised_s, 2)
        for batch in (1, 8, 64):
            each_s, mean_context, wall_rate = time_workload(engine, vocab, batch, 512, 256)
            points[f"decode_b{batch}_p512_g256"] = round(batch / each_s, 2)
            points[f"decode_b{batch}_p512_g256_frac"] = round(decode_bytes(model_config, layers, batch, mean_context, elem) / each_s / 1e9 / PEAK_HBM_GBS, 4)
            points[f"e2e_b{batch}_p512_g256"] = round(wall_rate, 2)
    prefill_s, prefill_best_s = time_prefill(engine, vocab, args.prefill_tokens)

    main_step = step_s[args.batch]
    bytes_read = decode_bytes(model_config, layers, args.batch, contexts[args.batch], elem)
    achieved = bytes_read / main_step / 1e9
    flops = prefill_flops(model_config, layers, args.prefill_tokens)
    result = {
        "metric": "decode_tokens_per_second",
        "value": round(args.batch / main_step, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(main_step * 1000, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: random weights N(0,0.02), uniform random token ids",
        "config": {
            "model": shape_name, "layers": layers, "layers_full": full_layers,
            "hidden": model_config["hidden_size"], "heads": model_config["num_attention_heads"],
            "kv_heads": model_config["num_key_value_heads"], "head_dim": model_config["hidden_size"] // model_config["num_attention_heads"],
            "intermediate": model_config["intermediate_size"], "vocab": vocab,
            "global_batch": args.batch, "seq_len": args.context, "mean_context": round(contexts[args.batch], 1), "page_size": 16,
            "prefill_tokens": args.prefill_tokens, "hip_graphs": graphs, "library_gemm_tuned": tuned > 0, "parallelism": "single-gpu",
        },
        "prefill": {
            "value": round(args.prefill_tokens / prefill_s, 1), "tokens": args.prefill_tokens,
            "ms": round(prefill_s * 1000, 3), "frac": round(flops / prefill_s / PEAK_FLOPS[args.dtype], 4), "ms_best": round(prefill_best_s * 1000, 3),
        },
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(achieved / PEAK_HBM_GBS, 4),
        },
        "points": points,
    }
    if not args.no_probes:
        # what this card delivers to a kernel that only reads, and to one that only issues matrix instructions: the
        # fractions above are of the published peaks, these say how much of the gap is the card's own
        read_gbs, mfma_tflops = engine.ops.probe_read_bandwidth(), engine.ops.probe_mfma_rate()
        result["probes"] = {
            "hbm_read_gbs": round(read_gbs, 1), "mfma_bf16_tflops": round(mfma_tflops, 1),
            "decode_frac_of_read": round(achieved / read_gbs, 4),
        }
        if args.dtype == "bf16":
            result["probes"]["prefill_frac_of_mfma"] = round(flops / prefill_s / 1e12 / mfma_tflops, 4)
    if args.far:
        engine.abort_all()
        engine = None  # (its weights and cache are given up before the next engines are built)
        points.update(far_points(model_config, layers, args))
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
