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


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_the_cache_holds_the_first_layers_rotated_keys_and_values(tmp_path, ops, name):
    """What the pages hold, read back in sequence order (``CacheManager.gather_sequence``): layer 0's keys with bias and
    rotation and its values with bias, as the plain formulas give them from the embeddings, for a prompt fed in portions
    that end inside pages, then single tokens, beside another request whose pages lie between this one's."""
    from plain_qwen2 import apply_rope, rms_norm, rope_tables

    folder = make_folder(tmp_path, name, "float32")
    config, weights = read_model_folder(folder)
    tokens = random_tokens(config["vocab_size"], 61, seed=17)
    other = random_tokens(config["vocab_size"], 30, seed=18)
    h = Harness(folder, ops, torch.float32, "cuda", PAGE_SIZE[name], num_pages=64)
    h.feed([("a", tokens[:7], [])])
    h.feed([("b", other[:11], []), ("a", tokens[7:30], [])])
    h.feed([("a", tokens[30:55], []), ("b", other[11:], [])])
    for i in range(55, 61):
        h.feed([("a", [tokens[i]], [0])])

    nh = int(config["num_attention_heads"])
    nkv = int(config.get("num_key_value_heads", nh))
    d = int(config.get("head_dim") or config["hidden_size"] // nh)
    scaling = config.get("rope_scaling") or {}
    factor = float(scaling.get("factor", 1.0)) if (scaling.get("type") or scaling.get("rope_type")) == "linear" else 1.0
    cos, sin = rope_tables(d, float(config.get("rope_theta", 10000.0)), len(tokens), factor)
    x = rms_norm(weights["model.embed_tokens.weight"][torch.tensor(tokens)], weights["model.layers.0.input_layernorm.weight"],
                 float(config.get("rms_norm_eps", 1e-6)))
    p = "model.layers.0.self_attn."
    keys = apply_rope((x @ weights[p + "k_proj.weight"].T + weights[p + "k_proj.bias"]).view(-1, nkv, d), cos, sin, torch.arange(len(tokens)))
    values = (x @ weights[p + "v_proj.weight"].T + weights[p + "v_proj.bias"]).view(-1, nkv, d)
    held = h.cache.gather_sequence(0, h.live["a"][0], len(tokens))
    got_keys, got_values = held["k"], held["v"]  # [tokens, kv_heads, head_dim] both: the token dimension comes first
    torch.testing.assert_close(got_keys.float().cpu(), keys, rtol=2e-5, atol=2e-6)
    torch.testing.assert_close(got_values.float().cpu(), values, rtol=2e-5, atol=2e-6)
    assert len(set(h.live["a"][0].tables[0]) & set(h.live["b"][0].tables[0])) == 0


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
