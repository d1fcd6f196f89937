#!/usr/bin/env python3
"""End-to-end benchmark of the engine from the command line, in the manner of the reference's
``benchmark.py`` (its options ``:349-388``, its step loop ``:160-182``, its report ``:232-276``).

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
    if not values:
        return {"n": 0, "mean": 0.0, "p50": 0.0, "p90": 0.0, "p99": 0.0, "max": 0.0}
    ordered = sorted(values)

    def pct(q: float) -> float:
        return ordered[min(len(ordered) - 1, int(q * len(ordered)))]

    return {"n": len(values), "mean": statistics.fmean(values), "p50": pct(0.5), "p90": pct(0.9), "p99": pct(0.99), "max": ordered[-1]}


def rule(title: str = "") -> None:
    print("\n" + "=" * 78 + f"\n  {title}\n" + "=" * 78 if title else "-" * 78)


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


def run_workload(engine, prompts, sampling, label: str) -> Dict:
    import torch

    from velox_amd import Request

    requests = [Request(f"{label}-{i}", p, sampling(i)) for i, p in enumerate(prompts)]
    token_times: Dict[str, List[float]] = {r.request_id: [] for r in requests}
    seen = {r.request_id: 0 for r in requests}
    start = time.perf_counter()
    for request in requests:
        engine.add_request(request)
    log = []
    while engine.has_work():
        engine.step()
        now = time.perf_counter()
        log.append((engine.scheduler.num_running, engine.scheduler.num_waiting, engine.cache.num_used_pages()))
        for request in requests:
            produced = len(request.output_token_ids)
            if produced > seen[request.request_id]:
                token_times[request.request_id].extend([now] * (produced - seen[request.request_id]))
                seen[request.request_id] = produced
    torch.cuda.synchronize()
    wall = time.perf_counter() - start
    ttft = [times[0] - start for times in token_times.values() if times]
    itl = [(b - a) * 1000 for times in token_times.values() for a, b in zip(times, times[1:])]
    generated = sum(len(r.output_token_ids) for r in requests)
    prompt_tokens = sum(len(p) for p in prompts)
    cached_tokens = sum(r.num_cached_tokens for r in requests)  # (of a preempted request: at its last admission)
    return {
        "label": label, "wall_seconds": wall, "num_requests": len(requests), "prompt_tokens": prompt_tokens,
        "generated_tokens": generated, "decode_throughput": generated / wall if wall else 0.0,
        "total_throughput": (prompt_tokens + generated) / wall if wall else 0.0,
        "ttft": summarise(ttft), "itl_ms": summarise(itl), "steps": engine.num_steps,
        "preemptions": engine.scheduler.num_preemptions, "cached_prompt_tokens": cached_tokens,
        "max_running": max((entry[0] for entry in log), default=0), "max_blocks_used": max((entry[2] for entry in log), default=0),
        "outputs": {r.request_id: r.output_token_ids for r in requests},
    }


def report(result: Dict, engine, show_outputs: bool) -> None:
    import torch

    rule(f"RESULTS: {result['label']}")
    print(f"  Requests              : {result['num_requests']}")
    print(f"  Wall time             : {result['wall_seconds']:.3f} s")
    print(f"  Engine steps          : {result['steps']}")
    print(f"  Prompt tokens         : {result['prompt_tokens']}")
    print(f"  Generated tokens      : {result['generated_tokens']}")
    print(f"  Decode throughput     : {result['decode_throughput']:.2f} tok/s")
    print(f"  End-to-end throughput : {result['total_throughput']:.2f} tok/s")
    print(f"  Peak running requests : {result['max_running']}")
    print(f"  Peak KV blocks in use : {result['max_blocks_used']}")
    print(f"  Preemptions           : {result['preemptions']}")
    share = 100.0 * result['cached_prompt_tokens'] / max(1, result['prompt_tokens'])
    print(f"  Prompt tokens cached  : {result['cached_prompt_tokens']} ({share:.1f}%, prefix caching {'on' if engine.cache.prefix is not None else 'off'})")
    ttft, itl = result["ttft"], result["itl_ms"]
    print(f"\n  TTFT (s)   mean={ttft['mean']:.3f}  p50={ttft['p50']:.3f}  p90={ttft['p90']:.3f}  p99={ttft['p99']:.3f}  max={ttft['max']:.3f}")
    print(f"  ITL (ms)   mean={itl['mean']:.2f}  p50={itl['p50']:.2f}  p90={itl['p90']:.2f}  p99={itl['p99']:.2f}  max={itl['max']:.2f}")
    rule()
    print("  Per-step breakdown (ms)")
    print(f"  {'stage':<20}{'n':>7}{'mean':>10}{'p50':>10}{'p90':>10}{'p99':>10}{'total(s)':>11}")
    for stage, values in engine.stats.items():
        s = summarise(values)
        print(f"  {stage:<20}{s['n']:>7}{s['mean']:>10.3f}{s['p50']:>10.3f}{s['p90']:>10.3f}{s['p99']:>10.3f}{sum(values) / 1000:>11.3f}")
    gpu_ms = sum(engine.stats.get("gpu_ms", []))
    busy = gpu_ms / 1000 / result["wall_seconds"] if result["wall_seconds"] else 0.0
    print(f"\n  GPU busy      : {gpu_ms / 1000:.3f} s  ({busy:.1%} of wall time)")
    print(f"  HIP graphs    : {'on' if engine.runner.uses_graphs else 'off'}")
    print(f"  Peak GPU alloc: {torch.cuda.max_memory_allocated() / 1e9:.3f} GB")
    if show_outputs:
        rule("SAMPLE OUTPUTS (token ids)")
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
        rule("ENGINE BENCHMARK")
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
            report(result, engine, args.show_outputs and round_index == 0)
            results.append(result)
        del engine
        torch.cuda.empty_cache()
    if len(sizes) > 1:
        rule("BATCH SIZE SWEEP")
        print(f"  {'max_num_seqs':>14}{'kv_blocks':>11}{'peak_used':>11}{'wall(s)':>10}{'tok/s':>10}{'TTFT p50':>11}{'ITL p50':>10}{'preempt':>9}")
        for size, result in zip(sizes, results):
            print(f"  {size:>14}{result['kv_blocks']:>11}{result['max_blocks_used']:>11}{result['wall_seconds']:>10.2f}"
                  f"{result['decode_throughput']:>10.2f}{result['ttft']['p50']:>11.3f}{result['itl_ms']['p50']:>10.2f}{result['preemptions']:>9}")
    if args.output_json:
        for result in results:
            result.pop("outputs", None)
        os.makedirs(os.path.dirname(os.path.abspath(args.output_json)), exist_ok=True)
        with open(args.output_json, "w", encoding="utf-8") as handle:
            json.dump(results, handle, indent=2)
        print(f"\nWrote {args.output_json}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
