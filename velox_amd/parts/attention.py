"""Grouped-query attention over the paged cache.

Order of operations follows the reference's ``SelfAttention.forward``
(``src/self_attention.py:46-90``): one fused QKV product (rows ``[Wq; Wk; Wv]``, bias
``[bq; bk; bv]``), split into heads, rotate Q and K, write K and V into the cache,
attend over the cache (so a portion reads its own keys from the cache), output
product.  ``scale = head_dim ** -0.5`` is applied to the float32 scores after the dot
(``src/self_attention.py:35``, ``src/attention_prefill.py:101``).  Query head ``h`` reads
KV head ``h // (heads / kv_heads)`` (``src/attention_prefill.py:36``).

Every size is a constructor argument; ``window`` (None = all keys) and ``bias`` are
options of the part, chosen by the architecture per layer.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import PAGE, Mixer, PagedNeed, Param, PositionEncoding, fused_rows, register_part, single

# Behind this many keys a decode step's attention runs without splitting a sequence's keys over workgroups (splits and
# their merge cost about as much as one workgroup's walk over that many keys): captured steps exist a second time for
# steps whose sequences are all that short, when the two would be launched differently.
SHORT_CONTEXT_KEYS = 384


def kv_pages(num_kv_heads: int, head_dim: int, window: Optional[int] = None) -> PagedNeed:
    """What attention keeps per page: keys ``[kv_heads, page, head_dim]`` and values transposed, ``[kv_heads, head_dim,
    page]`` (a run of consecutive keys for one channel is then one contiguous access for the kernels' second product)."""
    return PagedNeed((("k", (int(num_kv_heads), PAGE, int(head_dim)), None), ("v", (int(num_kv_heads), int(head_dim), PAGE), None)), window)


class AttentionMixer(Mixer):
    def __init__(
        self,
        prefix: str,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: Optional[PositionEncoding] = None,
        qkv_bias: bool = True,
        window: Optional[int] = None,
        scale: Optional[float] = None,
    ) -> None:
        super().__init__(prefix)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads={num_heads} must be a multiple of num_kv_heads={num_kv_heads}")
        if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
            raise ValueError(f"head_dim={head_dim}: the attention kernels take multiples of 16 from 16 to 256")
        if window is not None and window < 1:
            raise ValueError(f"window={window} must be at least 1")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.position = position
        self.qkv_bias = bool(qkv_bias)
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / (self.head_dim ** 0.5)
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.qkv_weight: Optional[torch.Tensor] = None
        self.qkv_bias_vec: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, q, kv = self.hidden_size, self.q_size, self.kv_size
        out = {
            "qkv_weight": fused_rows(
                ("q_proj.weight", "k_proj.weight", "v_proj.weight"), ((q, h), (kv, h), (kv, h))
            ),
            "o_weight": single("o_proj.weight", (h, q)),
        }
        if self.qkv_bias:
            out["qkv_bias_vec"] = fused_rows(
                ("q_proj.bias", "k_proj.bias", "v_proj.bias"), ((q,), (kv,), (kv,)), role="vector"
            )
        return out

    def cache_need(self):
        return kv_pages(self.num_kv_heads, self.head_dim, self.window)

    def _rotary_tables(self):
        tables = self.position.rotary_tables() if self.position is not None else None
        return tables if tables is not None else (None, None)

    def prepare_kernels(self, ops) -> None:
        load = getattr(ops, "attention_library", None)
        if load is not None:
            load(self.head_dim)  # built at first use for this head size; a missing compiler fails here, not in a step
        cos, _ = self._rotary_tables()
        whole_heads = cos is not None and 2 * cos.shape[1] == self.head_dim
        self.prepare_weight(ops, "qkv_weight", rotary_heads=(self.num_heads, self.num_kv_heads, self.head_dim) if whole_heads else None)
        self.prepare_weight(ops, "o_weight")

    def capture_key_bounds(self, ops, batch: int, max_model_len: int):
        choose = getattr(ops, "choose_splits", None)
        if choose is None or max_model_len <= SHORT_CONTEXT_KEYS:
            return ()
        differs = choose(batch, self.num_kv_heads, 1, max_model_len, True) != choose(batch, self.num_kv_heads, 1, SHORT_CONTEXT_KEYS, True)
        return (SHORT_CONTEXT_KEYS,) if differs else ()

    def workspace_needs(self, ops, limits):
        sizes = getattr(ops, "attention_scratch_elems", None)
        if sizes is None:
            return {}
        partial_out, partial_lse = sizes(self.num_heads, self.num_kv_heads, self.head_dim, limits.max_num_tokens, limits.max_num_seqs, limits.max_model_len)
        return {"attention_partial_out": partial_out, "attention_partial_lse": partial_lse}

    accepts_sink = True  # its last product may add itself to the residual (ResidualSink)
    accepts_deferred = True  # its first product can read a DeferredNorm

    def forward(self, x, ctx, cache, owns_cache: bool = True, sink=None):
        ops = ctx.ops
        cos, sin = self._rotary_tables()
        meta = cache.batch
        # product, bias (added in float32), rotation and the write into the cache: one kernel for decode-sized batches
        q = ops.qkv_rope_write(
            x, self.operand("qkv_weight"), self.qkv_bias_vec if self.qkv_bias else None,
            self.num_heads, self.num_kv_heads, self.head_dim,
            ctx.positions, cos, sin,
            meta.slot_mapping, cache.tensors["k"], cache.tensors["v"], cache.block_size,
            write_kv=owns_cache,
        )
        attn = ops.paged_attention(
            q, self.num_heads, self.num_kv_heads, self.head_dim,
            cache.tensors["k"], cache.tensors["v"], cache.block_size,
            meta.block_tables, ctx.cu_q, meta.kv_lens,
            ctx.max_q_len, meta.max_kv_len, self.scale, self.window,
            ctx.all_decode, ctx.workspace,
            decode_prefix=getattr(ctx, "decode_prefix", 0), portions_max_kv_len=getattr(meta, "max_kv_len_of_portions", 0) or None,
        )
        return ops.linear(attn, self.operand("o_weight"), None, ctx.dtype, partials_ok=True, residual_norm=sink)


register_part("mixer", "attention", AttentionMixer)
