"""Tiny configurations and small utilities shared by the tests."""
from __future__ import annotations

import random
from typing import List

import torch

from velox_amd.cache.manager import CacheManager
from velox_amd.config.registry import load_config
from velox_amd.engine.batch import StepEntry
from velox_amd.engine.engine import build_model
from velox_amd.engine.runner import ModelRunner
from velox_amd.weights import bind_from_checkpoint, write_random_model

# Two configurations that differ in every size and option, plus a third with a head size that
# does not divide the width, a width and a vocabulary that are no power of two, and scaled positions.
TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": True, "use_sliding_window": False, "max_position_embeddings": 512,
}
TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "intermediate_size": 224, "vocab_size": 320, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": False, "use_sliding_window": False, "max_position_embeddings": 1024,
}
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 80, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 48,
    "intermediate_size": 150, "vocab_size": 263, "rope_theta": 50000.0, "rms_norm_eps": 3e-6,
    "rope_scaling": {"type": "linear", "factor": 2.0},
    "tie_word_embeddings": False, "use_sliding_window": False, "max_position_embeddings": 2048,
}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
SEEDS = {"A": 0, "B": 1, "C": 2}


def make_folder(tmp_path, name: str, storage: str = "float32") -> str:
    path = str(tmp_path / f"tiny_{name}_{storage}")
    return write_random_model(CONFIGS[name], path, SEEDS[name], dtype=storage)


def random_tokens(vocab: int, length: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(length)]


class Harness:
    """Model + cache manager + step function, driven by hand (no scheduler)."""

    def __init__(self, model_dir: str, ops, dtype, device, page_size: int, num_pages: int, max_num_seqs: int = 4, max_num_tokens: int = 1024, enable_graphs: bool = False):
        self.config = load_config(model_dir)
        self.device = torch.device(device)
        self.dtype = dtype
        self.model = build_model(self.config, dtype, self.device)
        bind_from_checkpoint(self.model, model_dir, dtype, self.device)
        ops.prepare(self.model, dtype)
        self.cache = CacheManager(self.model.cache_needs(), page_size, num_pages, max_num_seqs, dtype, self.device)
        self.runner = ModelRunner(self.model, self.cache, ops, dtype, self.device, max_num_tokens, max_num_seqs, enable_graphs=enable_graphs)
        self.live = {}

    def feed(self, batch, end=()):
        """``batch``: list of (request id, tokens, want indices).  Returns float32 logits on the CPU or None."""
        entries = []
        for rid, tokens, want in batch:
            if rid not in self.live:
                seq = self.cache.new_sequence()
                assert seq is not None, "no free slot"
                self.live[rid] = [seq, 0]
            seq, computed = self.live[rid]
            assert self.cache.append(seq, computed, len(tokens)), f"out of pages for {rid}"
            entries.append(StepEntry(seq, list(tokens), computed, list(want)))
        logits = self.runner.step(entries)
        for rid, tokens, _ in batch:
            self.live[rid][1] += len(tokens)
            self.cache.release_behind_window(self.live[rid][0], self.live[rid][1])
        for rid in end:
            seq, _ = self.live.pop(rid)
            self.cache.free_sequence(seq)
        return None if logits is None else logits.float().cpu()
