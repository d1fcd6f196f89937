"""Times single kernels on the GPU, alone: the measurements that the launch rules in ``csrc/`` and ``hip_ops.py`` quote.

    python -m velox_amd.kernels.measure attention [--heads 28 --kv-heads 4 --head-dim 128 --page 16]

``barrier``: what a barrier across the workgroups of one resident kernel costs, against the boundary between two kernels
of a captured step (a chain of empty kernels in a HIP graph).

``attention``: portions of prompts through ``paged_attention`` for a list of (sequences, tokens each, keys each), once
with the kernel the launcher picks by shape and once with each kernel forced (``velox_attention_portion_kernel``):
1 = the kernels that stage tiles through registers, 2 = tiles loaded straight into LDS, 3 = the same with two sets of
waves.  A kernel is timed inside a HIP graph of several launches, so that the host's launch time does not count.
"""
from __future__ import annotations

import argparse
import math

import torch

ATTENTION_SHAPES = ((1, 512, 512), (1, 1024, 1024), (1, 2048, 2048), (2, 2048, 2048), (4, 2048, 2048), (1, 4096, 4096), (4, 512, 512), (4, 512, 1024),
                    (4, 512, 2048), (4, 512, 4096), (1, 2048, 4096), (2, 1024, 3072), (1, 512, 4096), (4, 512, 8192), (1, 512, 30000), (1, 8192, 8192),
                    (8, 256, 1024), (16, 128, 2048))


def time_in_graph(fn, launches: int = 5, rounds: int = 3) -> float:
    """Microseconds per call of ``fn``: the best of ``rounds`` timed replays of a graph that holds ``launches`` calls,
    after replays that keep the GPU busy for some milliseconds (a first replay after a pause runs at a lower clock)."""
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(launches):
            fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def timed(replays: int) -> float:
        start.record()
        for _ in range(replays):
            graph.replay()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / replays

    once = max(timed(1), 1e-3)
    timed(max(2, min(50, int(8.0 / once))))
    return min(timed(3) for _ in range(rounds)) / launches * 1e3


def attention_case(sequences: int, tokens: int, keys: int, heads: int, kv_heads: int, head_dim: int, page: int):
    pages_each = (keys + page - 1) // page
    total = sequences * pages_each + 1
    k = torch.randn(total, kv_heads, page, head_dim, device="cuda", dtype=torch.bfloat16)
    v = torch.randn(total, kv_heads, head_dim, page, device="cuda", dtype=torch.bfloat16)
    tables = (torch.randperm(total - 1, device="cuda") + 1).view(sequences, pages_each).to(torch.int32)  # pages in no order
    qkv = torch.randn(sequences * tokens, (heads + 2 * kv_heads) * head_dim, device="cuda", dtype=torch.bfloat16)
    cu_q = torch.arange(0, sequences * tokens + 1, tokens, device="cuda", dtype=torch.int32)
    kv_lens = torch.full((sequences,), keys, device="cuda", dtype=torch.int32)
    return qkv, k, v, tables, cu_q, kv_lens


def measure_attention(args) -> None:
    from ..engine.batch import Workspace
    from . import load_ops

    ops = load_ops("cuda")
    library = ops.attention_library(args.head_dim)
    workspace = Workspace(torch.device("cuda"))
    heads, kv_heads, d, page = args.heads, args.kv_heads, args.head_dim, args.page
    print(f"{heads} heads over {kv_heads} KV heads of {d} channels, pages of {page}; us per call and PFLOP/s of the causal arithmetic")
    print(f"{'sequences x tokens behind keys':>32}  {'staged':>16}  {'direct':>16}  {'direct, two sets':>16}  {'by shape':>16}  splits")
    try:
        for sequences, tokens, keys in ATTENTION_SHAPES:
            qkv, k, v, tables, cu_q, kv_lens = attention_case(sequences, tokens, keys, heads, kv_heads, d, page)
            flops = sequences * 4 * (tokens * (keys - tokens) + tokens * tokens / 2) * heads * d
            splits = ops.choose_portion_splits(sequences * tokens, heads // kv_heads, kv_heads, keys)
            cells = []
            for choice in (1, 2, 3, 0):
                library.velox_attention_portion_kernel(choice)
                each = time_in_graph(lambda: ops.paged_attention(qkv, heads, kv_heads, d, k, v, page, tables, cu_q, kv_lens, tokens, keys, 1 / math.sqrt(d),
                                                                 None, False, workspace))
                cells.append(f"{each:8.1f} {flops / each / 1e9:6.3f}")
            print(f"{sequences:>8} x {tokens:>5} behind {keys - tokens:>6}  " + "  ".join(f"{c:>16}" for c in cells) + f"  {splits:>6}",
                  flush=True)
    finally:
        library.velox_attention_portion_kernel(0)


def measure_barrier(args) -> None:
    from . import load_ops

    ops = load_ops("cuda")
    print(f"barrier across {ops.num_cus} workgroups of 256 threads inside one kernel, us each:")
    print(f"  relaxed agent-scope counters, no cache maintenance   {ops.probe_grid_barrier(False):7.2f}")
    print(f"  release on arrival, acquire behind the barrier       {ops.probe_grid_barrier(True):7.2f}")
    token = torch.zeros(64, dtype=torch.int32, device="cuda")
    each = time_in_graph(lambda: token.add_(1), launches=200)
    print(f"boundary between two kernels of a captured chain (200 launches of a 64-element add), us each   {each:7.2f}")


def main() -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("what", choices=["attention", "barrier"])
    parser.add_argument("--heads", type=int, default=28)
    parser.add_argument("--kv-heads", type=int, default=4)
    parser.add_argument("--head-dim", type=int, default=128)
    parser.add_argument("--page", type=int, default=16)
    args = parser.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("these measurements need a GPU")
    {"attention": measure_attention, "barrier": measure_barrier}[args.what](args)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
