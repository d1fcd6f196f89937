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
