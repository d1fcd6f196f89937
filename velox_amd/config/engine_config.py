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

    seed: Optional[int] = None

    def torch_dtype(self) -> torch.dtype:
        return resolve_dtype(self.dtype)

    def validate(self) -> None:
        # reference engine/config.py:61-75
        if self.max_num_seqs < 1:
            raise ValueError("max_num_seqs must be at least 1")
        if self.max_num_batched_tokens < self.max_prefill_chunk_size:
            raise ValueError("max_num_batched_tokens must be at least max_prefill_chunk_size")
        if self.max_num_batched_tokens < self.max_num_seqs:
            raise ValueError("max_num_batched_tokens must leave room for one token per running sequence")
        if not 0.0 < self.gpu_memory_utilization <= 1.0:
            raise ValueError("gpu_memory_utilization must be in (0, 1]")
        if self.block_size <= 0 or (self.block_size & (self.block_size - 1)) != 0:
            raise ValueError("block_size must be a power of two")
        if self.max_prefill_chunk_size < 1 or self.max_model_len < 2:
            raise ValueError("max_prefill_chunk_size must be at least 1 and max_model_len at least 2")
        if (self.kv_cache_dtype or "auto").lower() not in ("auto", str(self.dtype).lower()):
            raise ValueError(f"kv_cache_dtype={self.kv_cache_dtype!r}: the cache holds the run dtype; quantized caches are not built")
        if self.quantization not in (None, "", "none"):
            raise ValueError(f"quantization={self.quantization!r}: weight quantization is not built")
