"""Plain PyTorch references of every kernel the engine calls, one function per kernel.

They take the same arguments as the HIP wrappers in ``velox_amd.kernels`` and work on the
same memory layouts (paged keys ``[pages, kv_heads, page, d]``, paged values
``[pages, kv_heads, d, page]``), so that (1) each HIP kernel is compared with its reference
alone, at sizes of the test's choosing, and (2) the host side of the engine (batching,
cache manager, scheduler) can be exercised on a CPU by handing ``TorchOps`` to it.  The
product never loads this file.
"""
from __future__ import annotations

import numpy as np
import torch


# ----------------------------------------------------------------------------------------
# counter-based generator (Philox 4x32, 10 rounds), as the sampling kernel uses it
# ----------------------------------------------------------------------------------------
_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = np.uint32(0x9E3779B9), np.uint32(0xBB67AE85)


def philox4x32(counter: np.ndarray, key: np.ndarray) -> np.ndarray:
    """``counter`` uint32 [..., 4], ``key`` uint32 [..., 2] -> uint32 [..., 4]."""
    c = [counter[..., i].astype(np.uint32) for i in range(4)]
    k0 = key[..., 0].astype(np.uint32)
    k1 = key[..., 1].astype(np.uint32)
    for _ in range(10):
        p0 = _M0 * c[0].astype(np.uint64)
        p1 = _M1 * c[2].astype(np.uint64)
        hi0, lo0 = (p0 >> np.uint64(32)).astype(np.uint32), p0.astype(np.uint32)
        hi1, lo1 = (p1 >> np.uint64(32)).astype(np.uint32), p1.astype(np.uint32)
        c = [hi1 ^ c[1] ^ k0, lo1, hi0 ^ c[3] ^ k1, lo0]
        k0 = (k0 + _W0).astype(np.uint32)
        k1 = (k1 + _W1).astype(np.uint32)
    return np.stack(c, axis=-1)


def exponential_noise(vocab: int, seed_lo: int, seed_hi: int, counter: int) -> np.ndarray:
    """Exp(1) noise of one row: element i uses lane i % 4 of block i // 4; u = (bits >> 8 + 0.5) / 2^24."""
    blocks = (vocab + 3) // 4
    ctr = np.zeros((blocks, 4), dtype=np.uint32)
    ctr[:, 0] = np.arange(blocks, dtype=np.uint32)
    ctr[:, 1] = np.uint32(counter)
    key = np.zeros((blocks, 2), dtype=np.uint32)
    key[:, 0] = np.uint32(seed_lo)
    key[:, 1] = np.uint32(seed_hi)
    bits = philox4x32(ctr, key).reshape(-1)[:vocab]
    u = ((bits >> np.uint32(8)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 16777216.0)
    return np.maximum(-np.log(u), np.float32(1e-10)).astype(np.float32)


class TorchOps:
    """The kernels' arithmetic in plain PyTorch, on whatever device the tensors live."""

    name = "torch-reference"

    def prepare(self, model, dtype) -> None:
        pass

    def materialize(self, x):
        return x

    def qkv_rope_write(self, x, weight, bias, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=True):
        qkv = self.linear(x, weight, None, x.dtype)
        self.rope_kv_write(qkv, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=write_kv, bias=bias)
        return qkv

    # -- embedding and norms ------------------------------------------------------------
    def place_tokens(self, ids, dest, source, tokens, count):
        ids[dest[:count].long()] = tokens[source[:count].long()]

    def embed(self, token_ids, table):
        return table[token_ids.long()].float()

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype):
        if delta is not None and delta.dim() == 3:
            delta = delta.float().sum(0)
        if delta is not None:
            residual += delta.float()
        var = (residual * residual).sum(-1, keepdim=True) / residual.shape[-1]
        return (residual * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)

    def add_rmsnorm_rows(self, residual, delta, rows, weight, eps, out_dtype):
        if delta is not None and delta.dim() == 3:
            delta = delta.float().sum(0)
        x = residual[rows.long()]
        if delta is not None:
            x = x + delta[rows.long()].float()
        var = (x * x).sum(-1, keepdim=True) / x.shape[-1]
        return (x * torch.rsqrt(var + eps) * weight.float()).to(out_dtype)

    # -- matrix products ----------------------------------------------------------------
    def linear(self, x, weight, bias, out_dtype, partials_ok=False, residual_norm=None):
        out = x.float() @ weight.float().T
        if bias is not None:
            out = out + bias.float()
        return out.to(out_dtype)

    def linear_silu_mul(self, x, gate_up_weight, out_dtype, **_):
        return self.silu_mul(self.linear(x, gate_up_weight, None, out_dtype))

    def silu_mul(self, gate_up):
        inter = gate_up.shape[-1] // 2
        gate = gate_up[:, :inter].float()
        up = gate_up[:, inter:].float()
        return (gate * torch.sigmoid(gate) * up).to(gate_up.dtype)

    # -- rotary + cache write -----------------------------------------------------------
    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, positions, cos, sin, slot_mapping, k_cache, v_cache, block_size, write_kv=True, bias=None):
        t = qkv.shape[0]
        q_size, kv_size = num_heads * head_dim, num_kv_heads * head_dim
        wide = qkv.float()
        if bias is not None:
            wide = wide + bias
        q = wide[:, :q_size].reshape(t, num_heads, head_dim).clone()
        k = wide[:, q_size:q_size + kv_size].reshape(t, num_kv_heads, head_dim).clone()
        v = wide[:, q_size + kv_size:].reshape(t, num_kv_heads, head_dim)
        if cos is not None:
            half = cos.shape[1]
            c = cos[positions.long()].unsqueeze(1)
            s = sin[positions.long()].unsqueeze(1)
            for x in (q, k):
                lo = x[..., :half].clone()
                hi = x[..., half:2 * half].clone()
                x[..., :half] = lo * c - hi * s
                x[..., half:2 * half] = lo * s + hi * c
        # one rounding, at the store; only the rotated queries go back into qkv
        qkv[:, :q_size] = q.reshape(t, q_size).to(qkv.dtype)
        if write_kv:
            pages = (slot_mapping.long() // block_size)
            offsets = (slot_mapping.long() % block_size)
            k_cache[pages, :, offsets, :] = k.to(k_cache.dtype)
            v_cache[pages, :, :, offsets] = v.to(v_cache.dtype)

    # -- attention over the paged cache -------------------------------------------------
    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_size, block_tables, cu_q, kv_lens, max_q_len, max_kv_len, scale, window, all_decode, workspace, splits=None, decode_prefix=0, portions_max_kv_len=None):
        t = qkv.shape[0]
        group = num_heads // num_kv_heads
        q_all = qkv[:, : num_heads * head_dim].view(t, num_heads, head_dim)
        out = torch.zeros((t, num_heads, head_dim), dtype=torch.float32, device=qkv.device)
        cu = cu_q.tolist()
        lens = kv_lens.tolist()
        for b in range(len(lens)):
            lo, hi = cu[b], cu[b + 1]
            q_len, kv_len = hi - lo, lens[b]
            ctx = kv_len - q_len
            index = torch.arange(kv_len, device=qkv.device)
            pages = block_tables[b].long()[index // block_size]
            offsets = index % block_size
            keys = k_cache[pages, :, offsets, :].float()  # [kv_len, nkv, d]
            values = v_cache[pages, :, :, offsets].float()  # [kv_len, nkv, d]
            q_pos = ctx + torch.arange(q_len, device=qkv.device)
            keep = q_pos[:, None] >= index[None, :]
            if window is not None:
                keep &= index[None, :] > q_pos[:, None] - window
            for h in range(num_heads):
                kv = h // group
                scores = (q_all[lo:hi, h].float() @ keys[:, kv].T) * scale
                scores = scores.masked_fill(~keep, float("-inf"))
                m = scores.max(-1, keepdim=True).values
                p = torch.exp(scores - m)
                denom = p.sum(-1, keepdim=True)
                p = p.to(qkv.dtype).float()  # the kernel rounds p to the value dtype for the second product
                out[lo:hi, h] = (p @ values[:, kv]) / denom
        return out.to(qkv.dtype).view(t, num_heads * head_dim)

    # -- sampling -----------------------------------------------------------------------
    def argmax(self, logits):
        return logits.argmax(dim=-1).to(torch.int32)

    def sample(self, logits, options, with_filter=True, chunks=None):
        return torch.tensor(
            [self.sample_row(logits[r].cpu().numpy(), options[r].cpu().numpy())[0] for r in range(logits.shape[0])],
            dtype=torch.int32, device=logits.device,
        )

    @staticmethod
    def sample_row(row: np.ndarray, option: np.ndarray):
        """One row of the sampling kernel; returns (token, scores) with -inf for dropped tokens."""
        as_float = option.view(np.float32)
        temperature, top_p = float(as_float[0]), float(as_float[1])
        top_k, seed_lo, seed_hi, counter = int(option[2]), int(option[3]), int(option[4]), int(option[5])
        row = row.astype(np.float32)
        if temperature == 0.0:
            return int(row.argmax()), row
        x = row / np.float32(max(temperature, 1e-5))
        x = x - x.max()
        p = np.exp(x.astype(np.float64))
        p = p / p.sum()
        order = np.argsort(-x, kind="stable")
        keep = np.ones_like(x, dtype=bool)
        sorted_x = x[order]
        sorted_p = p[order]
        exclusive = np.cumsum(sorted_p) - sorted_p
        # tokens of equal value share rank and mass: the first of a run decides for all of it
        first_of_run = np.concatenate([[0], np.flatnonzero(np.diff(sorted_x) != 0) + 1])
        run_id = np.zeros(len(x), dtype=np.int64)
        run_id[first_of_run] = 1
        run_id = np.cumsum(run_id) - 1
        rank = first_of_run[run_id]
        mass = exclusive[first_of_run][run_id]
        keep_sorted = mass < top_p
        if top_k > 0:
            keep_sorted &= rank < top_k
        keep[order] = keep_sorted
        noise = exponential_noise(len(x), seed_lo, seed_hi, counter)
        scores = np.where(keep, x - np.log(noise), -np.inf).astype(np.float32)
        return int(scores.argmax()), scores

    def count_tokens(self, counts_row, tokens):
        ok = (tokens >= 0) & (tokens < counts_row.numel())
        counts_row += torch.bincount(tokens[ok].long(), minlength=counts_row.numel()).to(counts_row.dtype)

    def count_sampled(self, counts, row_of, tokens):
        for r in range(tokens.numel()):
            if int(row_of[r]) >= 0 and 0 <= int(tokens[r]) < counts.shape[1]:
                counts[int(row_of[r]), int(tokens[r])] += 1

    def apply_penalties_from_counts(self, logits, counts, row_of, coeffs):
        for r in range(logits.shape[0]):
            if int(row_of[r]) < 0:
                continue
            repetition, presence, frequency = (float(c) for c in coeffs[r])
            seen = counts[int(row_of[r])]
            ids = torch.nonzero(seen).flatten()
            vals = logits[r, ids] - frequency * seen[ids].float()
            vals = torch.where(vals > 0, vals / repetition, vals * repetition) - presence
            logits[r, ids] = vals

    def apply_penalties(self, logits, tokens, lengths, coeffs):
        """engine/sampler.py:169-189 of the reference: frequency first (times the count), then repetition
        (positive / r, negative * r) and presence, each once per distinct seen token."""
        for r in range(logits.shape[0]):
            seen = tokens[r, : int(lengths[r])].long()
            if seen.numel() == 0:
                continue
            repetition, presence, frequency = (float(c) for c in coeffs[r])
            ids, counts = torch.unique(seen, return_counts=True)
            vals = logits[r, ids] - frequency * counts.float()
            vals = torch.where(vals > 0, vals / repetition, vals * repetition) - presence
            logits[r, ids] = vals
