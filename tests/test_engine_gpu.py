"""The engine on the GPU with its HIP kernels against the plain whole-sequence model."""
import pytest
import torch

from helpers import CONFIGS, PAGE_SIZE, Harness, make_folder, random_tokens
from plain_qwen2 import qwen2_logits, read_model_folder

pytestmark = pytest.mark.gpu

TOL = {torch.float32: dict(rtol=2e-4, atol=2e-5), torch.bfloat16: dict(rtol=5e-2, atol=3e-2)}


@pytest.fixture(scope="module")
def ops():
    from velox_amd.kernels import load_ops

    return load_ops("cuda")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_then_decode_matches_plain(tmp_path, ops, name, dtype):
    folder = make_folder(tmp_path, name, "float32" if dtype == torch.float32 else "bfloat16")
    config, weights = read_model_folder(folder)
    tokens = random_tokens(config["vocab_size"], 100, seed=7)
    expected = qwen2_logits(config, weights, tokens)
    h = Harness(folder, ops, dtype, "cuda", PAGE_SIZE[name], num_pages=64)
    split = len(tokens) - 32
    got = [h.feed([("a", tokens[:split], list(range(split)))])]
    for i in range(split, len(tokens)):
        got.append(h.feed([("a", [tokens[i]], [0])]))
    got = torch.cat(got)
    torch.testing.assert_close(got, expected, **TOL[dtype])


def test_workspace_addresses_never_change_once_the_runner_exists(tmp_path, ops):
    """Captured steps hold the addresses of the attention's partial buffers: they are sized once, for the largest step the
    limits allow, and capture, a warm-up portion, a mixed step and a portion whose keys are split all find them in place."""
    from velox_amd.weights import write_random_model

    config = dict(CONFIGS["A"], max_position_embeddings=8192)
    folder = write_random_model(config, str(tmp_path / "long"), seed=3, dtype="bfloat16")
    h = Harness(folder, ops, torch.bfloat16, "cuda", page_size=16, num_pages=600, max_num_seqs=8, max_num_tokens=512, enable_graphs=True)
    before = h.runner.workspace.addresses()
    assert before and h.runner.workspace.fixed
    h.runner.capture_decode_graphs()
    h.runner.warm_prefill(512)
    tokens = random_tokens(config["vocab_size"], 4400, seed=1)
    for lo in range(0, 4096, 512):
        h.feed([("long", tokens[lo:lo + 512], [])])
    h.feed([("short", tokens[:40], [39])])
    calls = []
    original = ops.choose_portion_splits
    ops.choose_portion_splits = lambda *args: calls.append(original(*args)) or calls[-1]
    try:
        h.feed([("short", [5], [0]), ("long", tokens[4096:4200], [103])])  # a decoded token beside a portion behind 4,096 keys
    finally:
        ops.choose_portion_splits = original
    assert max(calls) > 1  # the portion's keys were split: the partial buffers were used
    for _ in range(3):
        h.feed([("short", [7], [0]), ("long", [9], [0])])  # captured steps
    assert h.runner.num_graph_replays == 3
    torch.cuda.synchronize()
    assert h.runner.workspace.addresses() == before
    with pytest.raises(RuntimeError, match="cannot be replaced"):
        h.runner.workspace.get("attention_partial_out", 1 << 30)
