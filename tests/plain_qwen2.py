"""A plain, slow Qwen2.5 forward written from the reference's formulas.

Whole sequences, no cache, no batching, one function per part, float32 (or float64) on
the CPU, sharing no code with ``velox_amd``.  Every function cites the lines of the
reference's files (paths from the reference's root) it was written from.  The reference
was read, not run.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import torch
from safetensors.torch import load_file


def read_model_folder(model_dir: str, dtype: torch.dtype = torch.float32):
    """config.json as a dict and every tensor of model.safetensors widened to ``dtype``."""
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: t.to(dtype) for name, t in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return config, weights


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """src/rmsnorm.py:20-28: var = sum(x^2)/N; out = x * rsqrt(var + eps) * w (eps inside the root, no offset on w)."""
    var = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x * torch.rsqrt(var + eps) * weight


def rope_tables(head_dim: int, theta: float, num_positions: int, factor: float = 1.0, dtype=torch.float32):
    """src/rope.py:45-56: inv_freq = 1 / theta^(arange(0, d, 2) / d); positions / factor (linear scaling only,
    src/rope.py:11-18); cos and sin of the outer product.  The reference builds them in float32."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    positions = torch.arange(num_positions, dtype=torch.float32)
    if factor != 1.0:
        positions = positions / factor
    freqs = torch.outer(positions, inv_freq)
    return freqs.cos().to(dtype), freqs.sin().to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """src/rope.py:73-85 and src/rope_inplace.py:25-47: halves (i, i + d/2) are a pair;
    new_lo = lo*cos - hi*sin, new_hi = lo*sin + hi*cos, with the table row of the token's position.
    ``x`` is [T, heads, d]."""
    c = cos[positions.long()].unsqueeze(1)
    s = sin[positions.long()].unsqueeze(1)
    lo, hi = x.chunk(2, dim=-1)
    return torch.cat([lo * c - hi * s, lo * s + hi * c], dim=-1)


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int] = None) -> torch.Tensor:
    """src/attention_prefill.py:36,101,115-117,119-139 for a whole sequence (no earlier context):
    query head h reads kv head h // G; score = (q . k) * scale; key n is kept iff n <= query position;
    softmax over the kept keys; out = p @ v.  ``window`` (not in the reference) keeps keys > position - window.
    q [T, nh, d]; k, v [T, nkv, d] -> [T, nh, d]."""
    t, nh, d = q.shape
    group = nh // k.shape[1]
    out = torch.empty_like(q)
    pos = torch.arange(t)
    keep = pos[:, None] >= pos[None, :]
    if window is not None:
        keep &= pos[None, :] > pos[:, None] - window
    for h in range(nh):
        kv = h // group
        scores = (q[:, h, :] @ k[:, kv, :].T) * scale
        scores = scores.masked_fill(~keep, float("-inf"))
        m = scores.max(dim=-1, keepdim=True).values
        p = torch.exp(scores - m)
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, kv, :]
    return out


def gated_mlp(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """src/mlp.py:13-15: down(silu(gate(x)) * up(x)), silu(z) = z * sigmoid(z), no biases."""
    gate = x @ w_gate.T
    up = x @ w_up.T
    return (gate * torch.sigmoid(gate) * up) @ w_down.T


def attention_layer(x, weights: Dict[str, torch.Tensor], prefix: str, nh: int, nkv: int, d: int, cos, sin, positions, window=None):
    """src/self_attention.py:48-56,90: q/k/v = x W^T + b (the fused matrix is rows [Wq; Wk; Wv],
    src/weight_loader.py:91-98), heads split, rotate q and k, attend, o_proj without bias; scale = d^-0.5 (:35)."""
    t = x.shape[0]
    q = x @ weights[prefix + "q_proj.weight"].T + weights[prefix + "q_proj.bias"]
    k = x @ weights[prefix + "k_proj.weight"].T + weights[prefix + "k_proj.bias"]
    v = x @ weights[prefix + "v_proj.weight"].T + weights[prefix + "v_proj.bias"]
    q = apply_rope(q.view(t, nh, d), cos, sin, positions)
    k = apply_rope(k.view(t, nkv, d), cos, sin, positions)
    v = v.view(t, nkv, d)
    out = causal_attention(q, k, v, 1.0 / math.sqrt(d), window)
    return out.reshape(t, nh * d) @ weights[prefix + "o_proj.weight"].T


def qwen2_logits(config: dict, weights: Dict[str, torch.Tensor], token_ids, dtype: torch.dtype = torch.float32, first_position: int = 0) -> torch.Tensor:
    """Logits at every position of one whole sequence, [T, vocab].

    src/transformer.py:43-52 (embed, layers, final norm), src/decoder_layer.py:41-54 (pre-norm residual block),
    src/transformer.py:60-62,67-68 (head, tied to the embedding table when tie_word_embeddings),
    defaults of absent keys from src/config.py:34-41.  ``first_position`` shifts every position (for the
    invariance test: only distances between positions count)."""
    hidden_size = int(config["hidden_size"])
    nh = int(config["num_attention_heads"])
    nkv = int(config.get("num_key_value_heads", nh))
    d = int(config.get("head_dim") or hidden_size // nh)
    eps = float(config.get("rms_norm_eps", config.get("layer_norm_eps", 1e-6)))
    theta = float(config.get("rope_theta", 10000.0))
    scaling = config.get("rope_scaling") or {}
    kind = scaling.get("type") or scaling.get("rope_type")
    factor = float(scaling.get("factor", 1.0)) if kind == "linear" else 1.0

    w = {name: t.to(dtype) for name, t in weights.items()}
    ids = torch.as_tensor(list(token_ids), dtype=torch.long)
    t = ids.shape[0]
    positions = torch.arange(first_position, first_position + t)
    cos, sin = rope_tables(d, theta, first_position + t, factor, dtype)

    h = w["model.embed_tokens.weight"][ids]
    for layer in range(int(config["num_hidden_layers"])):
        p = f"model.layers.{layer}."
        a = rms_norm(h, w[p + "input_layernorm.weight"], eps)
        h = h + attention_layer(a, w, p + "self_attn.", nh, nkv, d, cos, sin, positions)
        m = rms_norm(h, w[p + "post_attention_layernorm.weight"], eps)
        h = h + gated_mlp(m, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    h = rms_norm(h, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if config.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return h @ head.T
