#!/usr/bin/env python3
"""End-to-end benchmark of the engine from the command line, in the manner of the reference's
``benchmark.py``: its options (``:349-388``), the quantities it reports and the keys of its JSON
(``:184-223,232-276``).

The engine is token-in / token-out, so where the reference tokenises hand-written chat prompts
(``:17-47,149-153``) this program draws seeded random token ids of the workload's lengths.
``--model`` is a model folder (config.json + model.safetensors); ``--random-weights SEED`` with
``--shape`` runs a named shape on random weights instead.
"""
from __future__ import annotations

import argparse
import json
import os
import random
import statistics
import sys
import time
from typing import Dict, List, Optional

SHAPES = {
    "tinyA": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, intermediate_size=128,
                  vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=4096),
    "tinyB": dict(num_hidden_layers=3, hidden_size=96, num_attention_heads=3, num_key_value_heads=1, intermediate_size=224,
                  vocab_size=320, rope_theta=1e6, rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=4096),
    "1.5b": dict(num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, num_key_value_heads=2, intermediate_size=8960,
                 vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=True, max_position_embeddings=32768),
    "7b": dict(num_hidden_layers=28, hidden_size=3584, num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944,
               vocab_size=152064, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768),
    "32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=40, num_key_value_heads=8, intermediate_size=27648,
                vocab_size=152064, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768),
}
WORKLOAD_LENGTHS = {"short": (16, 64), "long": (256, 1024)}


def summarise(values: List[float]) -> Dict[str, float]:
    """Count, mean and nearest-rank percentiles of a list of numbers (zeros for an empty list)."""
    ordered = sorted(values)
    count = len(ordered)
    out = {"n": count, "mean": statistics.fmean(ordered) if count else 0.0}
    for name, share in (("p50", 0.5), ("p90", 0.9), ("p99", 0.99), ("max", 1.0)):
        out[name] = ordered[min(count - 1, int(share * count))] if count else 0.0
    return out


def heading(title: str) -> None:
    bar = "=" * 78
    print(f"\n{bar}\n  {title}\n{bar}")


def print_table(columns, rows, indent: str = "  ") -> None:
    """``columns``: (title, width, format) per column, the first left-aligned; ``rows``: one tuple of values per line."""
    print(indent + "".join(f"{title:<{width}}" if index == 0 else f"{title:>{width}}" for index, (title, width, _) in enumerate(columns)))
    for row in rows:
        cells = [format(value, fmt) for value, (_, _, fmt) in zip(row, columns)]
        print(indent + "".join(f"{cell:<{width}}" if index == 0 else f"{cell:>{width}}" for index, (cell, (_, width, _)) in enumerate(zip(cells, columns))))


SHARED_PREFIX_TOKENS = 96  # stands in for the reference's shared system prompt (``benchmark.py:42-47``, about 90 tokens)


def build_prompts(workload: str, count: int, vocab: int, limit: int, fixed_len: Optional[int], seed: int, shared_prefix: bool = False,
                  length_range: Optional[tuple] = None) -> List[List[int]]:
    rng = random.Random(seed)
    prefix = [rng.randrange(vocab) for _ in range(min(SHARED_PREFIX_TOKENS, max(0, limit - 1)))] if shared_prefix else []
    prompts = []
    for index in range(count):
        if fixed_len:
            length = fixed_len
        elif length_range:
            length = rng.randint(*length_range)
        else:
            kind = workload if workload != "mixed" else ("short", "long")[index % 2]
            lo, hi = WORKLOAD_LENGTHS[kind]
            length = rng.randint(lo, hi)
        length = max(1, min(length, limit - len(prefix)))
        prompts.append(prefix + [rng.randrange(vocab) for _ in range(length)])
    return prompts


class Measurement:
    """Times of one workload, taken where the engine announces them: every request's token and finish listeners note the
    clock (``Request.subscribe``), so a token counts when the engine hands it over, not when a poll notices it."""

    def __init__(self, requests) -> None:
        self.begin = time.perf_counter()
        self.token_times: Dict[str, List[float]] = {r.request_id: [] for r in requests}
        self.finished_at: Dict[str, float] = {}
        self.peak_running = self.peak_pages = 0
        for request in requests:
            request.subscribe(on_token=self._token, on_finish=self._finish)

    def _token(self, request, _token_id) -> None:
        self.token_times[request.request_id].append(time.perf_counter())

    def _finish(self, request, _reason) -> None:
        self.finished_at[request.request_id] = time.perf_counter()

    def after_step(self, engine) -> None:
        self.peak_running = max(self.peak_running, engine.scheduler.num_running)
        self.peak_pages = max(self.peak_pages, engine.cache.num_used_pages())

    def first_token_delays(self) -> List[float]:
        return [times[0] - self.begin for times in self.token_times.values() if times]

    def gaps_between_tokens_ms(self) -> List[float]:
        return [(later - earlier) * 1000 for times in self.token_times.values() for earlier, later in zip(times, times[1:])]

    def per_request(self, requests) -> List[Dict]:
        """One record per request, as the reference's JSON holds them (``benchmark.py:208-218``)."""
        records = []
        for request in requests:
            times = self.token_times[request.request_id]
            done = self.finished_at.get(request.request_id)
            records.append({
                "id": request.request_id, "prompt_tokens": request.num_prompt_tokens, "generated_tokens": len(request.output_token_ids),
                "ttft": times[0] - self.begin if times else None, "end_to_end": done - self.begin if done is not None else None,
                "cached_prompt_tokens": request.num_cached_tokens,  # (of a preempted request: at its last admission)
            })
        return records


def run_workload(engine, prompts, sampling, label: str) -> Dict:
    """Queues every prompt at once and steps the engine until nothing is left.  The result's keys are the reference's
    (``benchmark.py:184-223``): scripts that read its JSON read this one."""
    import torch

    from velox_amd import Request

    requests = [Request(f"{label}-{index}", prompt, sampling(index)) for index, prompt in enumerate(prompts)]
    measured = Measurement(requests)
    for request in requests:
        engine.add_request(request)
    while engine.has_work():
        engine.step()
        measured.after_step(engine)
    torch.cuda.synchronize()
    wall = time.perf_counter() - measured.begin
    records = measured.per_request(requests)
    prompt_tokens = sum(r["prompt_tokens"] for r in records)
    generated = sum(r["generated_tokens"] for r in records)
    per_second = (lambda tokens: tokens / wall) if wall > 0 else (lambda tokens: 0.0)
    return {
        "label": label, "wall_seconds": wall, "num_requests": len(requests),
        "prompt_tokens": prompt_tokens, "generated_tokens": generated, "cached_prompt_tokens": sum(r["cached_prompt_tokens"] for r in records),
        "decode_throughput": per_second(generated), "total_throughput": per_second(prompt_tokens + generated),
        "ttft": summarise(measured.first_token_delays()), "itl_ms": summarise(measured.gaps_between_tokens_ms()),
        "steps": engine.num_steps, "preemptions": engine.scheduler.num_preemptions,
        "max_running": measured.peak_running, "max_blocks_used": measured.peak_pages,
        "requests": records,
        "outputs": {r.request_id: r.output_token_ids for r in requests},
    }


_PERCENTILES = (("mean", "mean"), ("p50", "p50"), ("p90", "p90"), ("p99", "p99"), ("max", "max"))


def report(result: Dict, engine, show_outputs: bool) -> None:
    import torch

    heading(f"RESULTS: {result['label']}")
    cached_share = result["cached_prompt_tokens"] / max(1, result["prompt_tokens"])
    facts = [
        ("Requests", f"{result['num_requests']}"),
        ("Wall time", f"{result['wall_seconds']:.3f} s"),
        ("Engine steps", f"{result['steps']}"),
        ("Prompt tokens", f"{result['prompt_tokens']}"),
        ("Generated tokens", f"{result['generated_tokens']}"),
        ("Decode throughput", f"{result['decode_throughput']:.2f} tok/s"),
        ("End-to-end throughput", f"{result['total_throughput']:.2f} tok/s"),
        ("Peak running requests", f"{result['max_running']}"),
        ("Peak KV blocks in use", f"{result['max_blocks_used']}"),
        ("Preemptions", f"{result['preemptions']}"),
        ("Prompt tokens cached", f"{result['cached_prompt_tokens']} ({cached_share:.1%}, prefix caching {'on' if engine.cache.prefix is not None else 'off'})"),
    ]
    for name, value in facts:
        print(f"  {name:<22}: {value}")
    print()
    for title, key, digits in (("TTFT (s)", "ttft", 3), ("ITL (ms)", "itl_ms", 2)):
        print(f"  {title:<10} " + "  ".join(f"{name}={result[key][field]:.{digits}f}" for name, field in _PERCENTILES))
    print("-" * 78)
    print("  Per-step breakdown (ms)")
    stage_rows = []
    for stage, values in engine.stats.items():
        numbers = summarise(values)
        stage_rows.append((stage, numbers["n"], numbers["mean"], numbers["p50"], numbers["p90"], numbers["p99"], sum(values) / 1000))
    print_table((("stage", 20, ""), ("n", 7, "d"), ("mean", 10, ".3f"), ("p50", 10, ".3f"), ("p90", 10, ".3f"), ("p99", 10, ".3f"), ("total(s)", 11, ".3f")), stage_rows)
    device_seconds = sum(engine.stats.get("gpu_ms", [])) / 1000
    busy_share = device_seconds / result["wall_seconds"] if result["wall_seconds"] else 0.0
    print(f"\n  GPU busy      : {device_seconds:.3f} s  ({busy_share:.1%} of wall time)")
    print(f"  HIP graphs    : {'on' if engine.runner.uses_graphs else 'off'}")
    print(f"  Peak GPU alloc: {torch.cuda.max_memory_allocated() / 1e9:.3f} GB")
    if show_outputs:
        heading("SAMPLE OUTPUTS (token ids)")
        for request_id, tokens in list(result["outputs"].items())[:4]:
            print(f"  [{request_id}] {tokens[:32]}")


def parse_args(argv=None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description="End-to-end benchmark for the engine.")
    parser.add_argument("--model", default=None, help="model folder (config.json + model.safetensors)")
    parser.add_argument("--random-weights", type=int, default=None, metavar="SEED", help="run --shape on random weights drawn with this seed")
    parser.add_argument("--shape", default="7b", choices=sorted(SHAPES))
    parser.add_argument("--dtype", default="auto")
    parser.add_argument("--workload", default="mixed", choices=["short", "long", "mixed"])
    parser.add_argument("--prompt-len", type=int, default=None, help="every prompt has this many tokens (overrides --workload)")
    parser.add_argument("--prompt-len-range", default=None, metavar="LO,HI", help="prompt lengths uniform in [LO, HI] (overrides --workload)")
    parser.add_argument("--num-requests", type=int, default=16)
    parser.add_argument("--max-tokens", type=int, default=128)
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top-p", type=float, default=1.0)
    parser.add_argument("--max-model-len", type=int, default=2048)
    parser.add_argument("--max-num-seqs", type=int, default=32)
    parser.add_argument("--max-num-batched-tokens", type=int, default=2048)
    parser.add_argument("--max-prefill-chunk-size", type=int, default=512)
    parser.add_argument("--block-size", type=int, default=16)
    parser.add_argument("--num-gpu-blocks", type=int, default=None)
    parser.add_argument("--gpu-memory-utilization", type=float, default=0.85)
    parser.add_argument("--kv-cache-dtype", default="auto", help="only 'auto' (the run dtype): quantized caches are not built")
    parser.add_argument("--quantization", default=None, help="not built: anything but none is refused")
    parser.add_argument("--no-prefix-caching", action="store_true", help="compute every prompt in full (no sharing of prompt prefixes between requests)")
    parser.add_argument("--no-cuda-graphs", "--no-hip-graphs", dest="no_graphs", action="store_true")
    parser.add_argument("--shared-system-prompt", action="store_true", help="every prompt starts with the same %d tokens" % SHARED_PREFIX_TOKENS)
    parser.add_argument("--tune-library", action="store_true",
                        help="let the matrix library time its kernels for the prefill chunk size and the larger decode batches first (bfloat16; takes seconds per shape)")
    parser.add_argument("--sweep-batch-size", default=None, help="comma-separated max_num_seqs values to sweep")
    parser.add_argument("--rounds", type=int, default=1, help="replay the workload N times")
    parser.add_argument("--show-outputs", action="store_true")
    parser.add_argument("--output-json", default=None)
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--compare-hf", action="store_true", help="not built (the reference compares with another library's model; this engine's yardstick is the plain model under tests/)")
    args = parser.parse_args(argv)
    if args.compare_hf:
        parser.error("--compare-hf is not built: no library model is part of this engine; tests/plain_qwen2.py is the yardstick")
    return args


def main(argv=None) -> int:
    args = parse_args(argv)
    import torch

    if not torch.cuda.is_available():
        raise SystemExit("this benchmark requires a GPU")
    from velox_amd import Engine, EngineConfig, SamplingParams

    if (args.model is None) == (args.random_weights is None):
        raise SystemExit("give either --model FOLDER or --random-weights SEED (with --shape)")

    def make_engine(max_num_seqs: int):
        config = EngineConfig(
            model=args.model or "", dtype=args.dtype, max_model_len=args.max_model_len, max_num_seqs=max_num_seqs,
            max_num_batched_tokens=max(args.max_num_batched_tokens, max_num_seqs), max_prefill_chunk_size=args.max_prefill_chunk_size,
            block_size=args.block_size, num_gpu_blocks=args.num_gpu_blocks, gpu_memory_utilization=args.gpu_memory_utilization,
            kv_cache_dtype=args.kv_cache_dtype, quantization=args.quantization,
            enable_prefix_caching=not args.no_prefix_caching, enable_cuda_graphs=not args.no_graphs, seed=args.seed)
        if args.model:
            return Engine.from_pretrained(config)
        model_config = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", **SHAPES[args.shape]}
        return Engine.from_random(model_config, args.random_weights, config, generator_device="cuda")

    def sampling(index: int):
        return SamplingParams(temperature=args.temperature, top_p=args.top_p, max_tokens=args.max_tokens, ignore_eos=True,
                              seed=None if args.temperature == 0.0 else args.seed * 1000 + index)

    sizes = [int(v) for v in args.sweep_batch_size.split(",")] if args.sweep_batch_size else [args.max_num_seqs]
    results = []
    for max_num_seqs in sizes:
        engine = make_engine(max_num_seqs)
        if args.tune_library:
            from velox_amd.engine.runner import decode_buckets

            # a ladder of step sizes up to the token budget: a step is padded up to the next one when that is close
            budget = max(args.max_num_batched_tokens, max_num_seqs)
            ladder = sorted({args.max_prefill_chunk_size, budget} | {n for n in range(128, budget + 1, 128) if n * 8 >= budget})
            engine.tune_matrix_products(ladder + [b for b in decode_buckets(max_num_seqs) if b > 16], progress=lambda text: print(f"  [tune] {text}", flush=True))
        vocab = engine.model.spec.vocab_size
        limit = engine.max_model_len - args.max_tokens - 1
        if limit < 1:
            raise SystemExit("--max-tokens leaves no room for a prompt under --max-model-len")
        length_range = tuple(int(v) for v in args.prompt_len_range.split(",")) if args.prompt_len_range else None
        prompts = build_prompts(args.workload, args.num_requests, vocab, limit, args.prompt_len, args.seed, args.shared_system_prompt, length_range)
        heading("ENGINE BENCHMARK")
        print(f"  Model            : {args.model or args.shape + ' (random weights)'}")
        print(f"  PyTorch / HIP    : {torch.__version__} / {torch.version.hip}")
        print(f"  GPU              : {torch.cuda.get_device_name(0)}")
        print(f"  KV blocks        : {engine.cache.num_total_pages} x {engine.cache.page_size} tokens")
        for round_index in range(args.rounds):
            for values in engine.stats.values():
                values.clear()
            torch.cuda.reset_peak_memory_stats()
            result = run_workload(engine, prompts, sampling, f"engine(max_num_seqs={max_num_seqs})" + (f" round={round_index + 1}" if args.rounds > 1 else ""))
            result["kv_blocks"] = engine.cache.num_total_pages
            result["max_num_seqs"] = max_num_seqs
            report(result, engine, args.show_outputs and round_index == 0)
            results.append(result)
        del engine
        torch.cuda.empty_cache()
    if len(sizes) > 1:
        heading("BATCH SIZE SWEEP")
        columns = (("max_num_seqs", 14, "d"), ("kv_blocks", 11, "d"), ("peak_used", 11, "d"), ("wall(s)", 10, ".2f"), ("tok/s", 10, ".2f"),
                   ("TTFT p50", 11, ".3f"), ("ITL p50", 10, ".2f"), ("preempt", 9, "d"))
        print_table(columns, [(r["max_num_seqs"], r["kv_blocks"], r["max_blocks_used"], r["wall_seconds"], r["decode_throughput"], r["ttft"]["p50"],
                               r["itl_ms"]["p50"], r["preemptions"]) for r in results])
    if args.output_json:
        folder = os.path.dirname(os.path.abspath(args.output_json))
        os.makedirs(folder, exist_ok=True)
        with open(args.output_json, "w", encoding="utf-8") as handle:
            json.dump([{key: value for key, value in r.items() if key != "outputs"} for r in results], handle, indent=2)
        print(f"\nWrote {args.output_json}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
