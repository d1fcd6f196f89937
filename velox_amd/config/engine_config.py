"""Engine options, with the reference's names and meanings (``engine/config.py:34-75``).

``download_dir``, ``kv_cache_dtype`` and ``quantization`` are accepted at their reference
defaults only, so that the reference's call sites keep working: there is no hub to
download from, and the cache and the weights hold the run dtype (anything else is refused).
Added: ``watermark`` (the reference keeps it in its scheduler configuration,
``engine/scheduler.py:23``).  ``enable_cuda_graphs`` keeps the reference's
name; what it switches here is HIP-graph capture of the all-decode step.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

# reference engine/config.py:8-17
_DTYPES = {
    "auto": None,
    "bfloat16": torch.bfloat16,
    "bf16": torch.bfloat16,
    "float32": torch.float32,
    "fp32": torch.float32,
}


def resolve_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"run dtype must be bfloat16 or float32, got {name}")
        return name
    key = (name or "auto").lower()
    if key in ("float16", "fp16", "half"):
        raise ValueError("float16 is not a run dtype of this engine; use bfloat16 or float32")
    if key not in _DTYPES:
        raise ValueError(f"unknown dtype {name!r}; expected one of {sorted(_DTYPES)}")
    return _DTYPES[key] or torch.bfloat16


@dataclass
class EngineConfig:
    model: str = ""
    dtype: str = "auto"
    device: str = "cuda"

    download_dir: Optional[str] = None

    max_model_len: int = 4096
    max_num_seqs: int = 32
    max_num_batched_tokens: int = 2048
    max_prefill_chunk_size: int = 512

    block_size: int = 16
    num_gpu_blocks: Optional[int] = None
    gpu_memory_utilization: float = 0.90
    kv_cache_reserve_mb: int = 512

    # pages of a prompt prefix that an earlier request has computed are taken over instead of computed again (on by
    # default as in the reference; models whose layers keep a window or a state of fixed size run without it)
    enable_prefix_caching: bool = True
    kv_cache_dtype: str = "auto"
    quantization: Optional[str] = None
    enable_cuda_graphs: bool = True
    # a second copy of every bfloat16 weight in the order the decode kernels read it: faster decoding for the
    # weights' size again in memory (not a reference option)
    pack_decode_weights: bool = True
    # fresh pages are handed out all over the pool instead of 1, 2, 3, ...: sequences decoded together then do not read
    # the same memory channels at the same moment (not a reference option)
    scatter_pages: bool = True
    # launch a decode step's successor before reading the step's tokens (not a reference option)
    decode_lookahead: bool = True
    # where ``Engine.tune_matrix_products`` keeps what the matrix library's timings found, so that a later start does not
    # time the same shapes again: "auto" = beside the built kernel libraries, None = nowhere (not a reference option)
    library_tuning_file: Optional[str] = "auto"
    watermark: float = 0.01
    # tensors of the model folder that the model has no place for: False = an error that lists them, True = their number
    # is printed and they are ignored (what the reference always does, ``src/weight_loader.py:131-136``)
    ignore_unexpected_weights: bool = False

    seed: Optional[int] = None

    def torch_dtype(self) -> torch.dtype:
        return resolve_dtype(self.dtype)

    def validate(self) -> None:
        """Refuses option values that cannot work together (the limits are the reference's, ``engine/config.py:61-75``)."""
        def power_of_two(n: int) -> bool:
            return n > 0 and n & (n - 1) == 0

        checks = (
            (self.max_num_seqs >= 1, f"max_num_seqs={self.max_num_seqs}: at least one request runs at a time"),
            (self.max_prefill_chunk_size >= 1, f"max_prefill_chunk_size={self.max_prefill_chunk_size}: a portion has at least one token"),
            (self.max_model_len >= 2, f"max_model_len={self.max_model_len}: a prompt token and a generated one need two positions"),
            (self.max_num_batched_tokens >= self.max_prefill_chunk_size,
             f"max_num_batched_tokens={self.max_num_batched_tokens} is less than one portion of a prompt (max_prefill_chunk_size={self.max_prefill_chunk_size})"),
            (self.max_num_batched_tokens >= self.max_num_seqs,
             f"max_num_batched_tokens={self.max_num_batched_tokens} is less than a decode step of max_num_seqs={self.max_num_seqs} requests"),
            (0.0 < self.gpu_memory_utilization <= 1.0, f"gpu_memory_utilization={self.gpu_memory_utilization}: a share of the memory, above 0 and at most 1"),
            (power_of_two(self.block_size), f"block_size={self.block_size}: pages hold a power of two of tokens"),
            ((self.kv_cache_dtype or "auto").lower() in ("auto", str(self.dtype).lower()),
             f"kv_cache_dtype={self.kv_cache_dtype!r}: the cache holds the run dtype; quantized caches are not built"),
            (self.quantization in (None, "", "none"), f"quantization={self.quantization!r}: weight quantization is not built"),
        )
        failed = [message for ok, message in checks if not ok]
        if failed:
            raise ValueError("engine options: " + "; ".join(failed))
