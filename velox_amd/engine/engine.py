"""The engine loop: scheduler -> one step of the model -> sampler -> request bookkeeping.

Entry points and their meaning follow the reference (``engine/engine.py``):
``Engine.from_pretrained(EngineConfig(model=folder))`` ``:105-172``, ``add_request`` ``:213``,
``step`` ``:275-369``, ``generate`` ``:398-410``, ``has_work`` ``:265``, ``abort_request`` ``:216``,
``snapshot`` ``:412-417``.  Where the reference runs a prefill forward and a decode forward on
two streams and concatenates their last rows, ``step`` here hands ONE mixed batch to the
step function.  The one host wait per step is the read of the sampled tokens
(reference ``:358-359``).
"""
from __future__ import annotations

import time
from typing import Dict, FrozenSet, Iterable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager, pages_that_fit
from ..config.engine_config import EngineConfig
from ..config.model_config import read_generation_eos
from ..config.registry import config_from_dict, get_architecture, load_config
from ..parts.model import DecoderModel
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from ..weights import bind_from_checkpoint, bind_random
from .batch import StepEntry
from .request import FinishReason, Request
from .runner import ModelRunner
from .scheduler import Scheduler, SchedulerConfig

_STAGES = ("scheduler_ms", "prepare_ms", "forward_ms", "sampling_ms", "cpu_sync_wait_ms", "step_ms")


def build_model(model_config, dtype: torch.dtype, device, max_position: Optional[int] = None) -> DecoderModel:
    spec = get_architecture(model_config.architecture).make_spec(model_config, max_position)
    return DecoderModel(spec)


class Engine:
    def __init__(self, model: DecoderModel, cache: CacheManager, config: EngineConfig, ops, eos_token_ids: Optional[Iterable[int]] = None) -> None:
        config.validate()
        self.config = config
        self.device = torch.device(config.device)
        self.dtype = config.torch_dtype()
        self.model = model
        self.cache = cache
        self.ops = ops
        self.eos_token_ids: FrozenSet[int] = frozenset(eos_token_ids if eos_token_ids is not None else model.spec.eos_token_ids)
        self.scheduler = Scheduler(
            cache,
            SchedulerConfig(
                max_num_seqs=config.max_num_seqs,
                max_num_batched_tokens=config.max_num_batched_tokens,
                max_prefill_chunk_size=config.max_prefill_chunk_size,
                max_model_len=config.max_model_len,
                watermark=config.watermark,
            ),
        )
        self.max_model_len = self.scheduler.config.max_model_len
        self.runner = ModelRunner(
            model, cache, ops, self.dtype, self.device,
            max_num_tokens=config.max_num_batched_tokens,
            max_num_seqs=config.max_num_seqs,
            enable_graphs=config.enable_cuda_graphs,
        )
        self.sampler = Sampler(ops, self.device, seed=config.seed)
        self.stats: Dict[str, List[float]] = {name: [] for name in _STAGES}
        self.num_steps = 0

    # -- construction -------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, config: Optional[EngineConfig] = None, ops=None, **overrides) -> "Engine":
        config = config or EngineConfig(**overrides)
        config.validate()
        model_config = load_config(config.model)
        eos = read_generation_eos(config.model)
        return cls._assemble(config, model_config, ops, eos, lambda model, dtype, device: bind_from_checkpoint(model, config.model, dtype, device))

    @classmethod
    def from_random(cls, model_config_dict: dict, seed: int, config: Optional[EngineConfig] = None, ops=None, generator_device: str = "cpu", **overrides) -> "Engine":
        """An engine over random weights drawn in memory (no folder), for shapes too large to write out."""
        config = config or EngineConfig(**overrides)
        config.validate()
        model_config = config_from_dict(model_config_dict)
        return cls._assemble(
            config, model_config, ops, None,
            lambda model, dtype, device: bind_random(model, seed, dtype, device, generator_device=generator_device),
        )

    @classmethod
    def _assemble(cls, config: EngineConfig, model_config, ops, eos, bind) -> "Engine":
        device = torch.device(config.device)
        dtype = config.torch_dtype()
        if ops is None:
            from ..kernels import load_ops

            ops = load_ops(device)
        max_position = getattr(model_config, "max_position_embeddings", None)
        max_model_len = min(config.max_model_len, max_position) if max_position else config.max_model_len
        config.max_model_len = max_model_len
        model = build_model(model_config, dtype, device, max_position=max_model_len)
        bind(model, dtype, device)
        needs = model.cache_needs()
        if hasattr(ops, "pack_decode_weights"):
            ops.pack_decode_weights = config.pack_decode_weights
        ops.prepare(model, dtype)
        num_pages = config.num_gpu_blocks
        if num_pages is None:
            probe = CacheManager(needs, config.block_size, 2, config.max_num_seqs, dtype, device, allocate_tensors=False)
            free_bytes, _ = torch.cuda.mem_get_info(device)
            free_bytes += torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
            num_pages = pages_that_fit(probe.bytes_per_page(), free_bytes, config.gpu_memory_utilization, config.kv_cache_reserve_mb * 1024 * 1024)
            wanted = (config.max_num_seqs * max_model_len + config.block_size - 1) // config.block_size + 1
            num_pages = min(num_pages, max(2, wanted))
        cache = CacheManager(needs, config.block_size, num_pages, config.max_num_seqs, dtype, device, max_model_len=max_model_len)
        engine = cls(model, cache, config, ops, eos_token_ids=eos)
        engine.warmup()
        return engine

    def warmup(self) -> None:
        if self.device.type != "cuda":
            return
        self.runner.capture_decode_graphs()
        torch.cuda.synchronize()

    def tune_matrix_products(self, token_counts: Sequence[int]) -> int:
        """Optional, bfloat16 only: has the matrix library time its candidate kernels for this model's weight shapes at
        the given numbers of tokens per step (typically the prefill chunk size) and keep the fastest.  Takes seconds
        per shape; steps with other token counts are unaffected."""
        if self.dtype != torch.bfloat16 or self.device.type != "cuda":
            return 0
        shapes = set()
        for part in self.model.all_parts():
            for attr, param in part.params().items():
                tensor = getattr(part, attr, None)
                if param.role == "matrix" and tensor is not None and tensor.dim() == 2 and tensor.dtype == torch.bfloat16 and attr != "table":
                    shapes.add(tuple(tensor.shape))
        counts = [m for m in token_counts if m > 64]  # smaller steps run on the engine's own kernels
        return self.ops.tune_library_products(shapes, counts) if counts else 0

    # -- requests -----------------------------------------------------------------------
    def add_request(self, request: Request) -> None:
        bad = [t for t in request.prompt_token_ids if not 0 <= t < self.model.spec.vocab_size]
        if bad:
            raise ValueError(f"token ids outside the vocabulary of {self.model.spec.vocab_size}: {bad[:8]}")
        self.scheduler.add_request(request)

    def abort_request(self, request_id: str) -> bool:
        self.sampler.release(request_id)
        return self.scheduler.abort_request(request_id)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    # -- one step -----------------------------------------------------------------------
    @torch.no_grad()
    def step(self) -> None:
        step_start = time.perf_counter()
        scheduled = self.scheduler.schedule()
        self.stats["scheduler_ms"].append((time.perf_counter() - step_start) * 1000)
        if scheduled.is_empty():
            return

        entries: List[StepEntry] = []
        sampled: List[Request] = []
        # decode rows first, then prompt portions; only rows that complete their tokens are sampled
        for request in scheduled.decode_batch:
            token = request.all_token_ids[request.num_computed_tokens]
            entries.append(StepEntry(request.cache, [token], request.num_computed_tokens, [0]))
            sampled.append(request)
        for request in scheduled.prefill_batch:
            start = request.num_computed_tokens
            chunk = request.current_chunk_size
            tokens = request.all_token_ids[start:start + chunk]
            completes = start + chunk >= len(request.all_token_ids)
            entries.append(StepEntry(request.cache, tokens, start, [chunk - 1] if completes else []))
            if completes:
                sampled.append(request)

        t0 = time.perf_counter()
        logits = self.runner.step(entries)
        self.stats["forward_ms"].append((time.perf_counter() - t0) * 1000)

        tokens: List[int] = []
        if sampled:
            t0 = time.perf_counter()
            needs_history = any(r.sampling_params.has_penalties for r in sampled)
            tokens_gpu = self.sampler.sample(
                logits,
                [r.sampling_params for r in sampled],
                [r.request_id for r in sampled],
                [len(r.output_token_ids) for r in sampled],
                histories=[r.all_token_ids for r in sampled] if needs_history else None,
            )
            sync_start = time.perf_counter()
            tokens = tokens_gpu.tolist()  # the one place per step where the host waits for the device
            self.stats["cpu_sync_wait_ms"].append((time.perf_counter() - sync_start) * 1000)
            self.stats["sampling_ms"].append((time.perf_counter() - t0) * 1000)

        for request in scheduled.decode_batch:
            self.scheduler.advance(request, 1)
        for request in scheduled.prefill_batch:
            self.scheduler.advance(request, request.current_chunk_size)
            request.refresh_status()
        for request, token in zip(sampled, tokens):
            request.append_token(int(token))
            request.refresh_status()
            reason = request.should_stop(int(token), self.eos_token_ids)
            if reason is not None:
                request.finish(reason)
                self.sampler.release(request.request_id)

        self.num_steps += 1
        self.stats["step_ms"].append((time.perf_counter() - step_start) * 1000)

    @torch.no_grad()
    def generate(self, requests: Sequence[Request], max_steps: Optional[int] = None) -> List[Request]:
        for request in requests:
            self.add_request(request)
        steps = 0
        while self.has_work():
            self.step()
            steps += 1
            if max_steps is not None and steps >= max_steps:
                break
        return list(requests)

    def snapshot(self) -> Dict[str, float]:
        stats = self.scheduler.stats()
        stats["num_steps"] = float(self.num_steps)
        stats["cuda_graphs"] = 1.0 if self.runner.uses_graphs else 0.0
        stats["kv_cache_bytes"] = float(self.cache.bytes_per_page() * (self.cache.num_total_pages + 1))
        return stats
