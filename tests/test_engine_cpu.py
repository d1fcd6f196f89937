"""Host side of the engine (batching, cache manager, step function) on a CPU, with the kernels'
plain PyTorch references standing in for the kernels, against the plain whole-sequence model."""
import pytest
import torch

from helpers import PAGE_SIZE, Harness, make_folder, random_tokens
from plain_qwen2 import qwen2_logits, read_model_folder
from torch_ops import TorchOps


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_then_decode_matches_plain(tmp_path, name):
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    tokens = random_tokens(config["vocab_size"], 45, seed=7)
    expected = qwen2_logits(config, weights, tokens)
    h = Harness(folder, TorchOps(), torch.float32, "cpu", PAGE_SIZE[name], num_pages=32)
    split = 30
    got = [h.feed([("a", tokens[:split], list(range(split)))])]
    for i in range(split, len(tokens)):
        got.append(h.feed([("a", [tokens[i]], [0])]))
    got = torch.cat(got)
    torch.testing.assert_close(got, expected, rtol=1e-4, atol=1e-5)
    h.feed([], end=["a"]) if False else h.cache.free_sequence(h.live.pop("a")[0])
    h.cache.assert_consistent([])


def test_mixed_batch_with_page_reuse(tmp_path):
    name = "B"
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    prompts = {rid: random_tokens(config["vocab_size"], n, seed=i) for i, (rid, n) in enumerate([("a", 23), ("b", 17), ("c", 9), ("d", 31)])}
    expected = {rid: qwen2_logits(config, weights, toks) for rid, toks in prompts.items()}
    h = Harness(folder, TorchOps(), torch.float32, "cpu", PAGE_SIZE[name], num_pages=9)  # 8 usable pages of 8
    got = {rid: [] for rid in prompts}
    # a and b start; a finishes, its pages go to c; then d takes what b and c give back
    def run(batch, end=()):
        out = h.feed([(rid, prompts[rid][lo:hi], list(range(hi - lo))) for rid, lo, hi in batch], end=end)
        row = 0
        for rid, lo, hi in batch:
            got[rid].append(out[row:row + hi - lo])
            row += hi - lo
    run([("a", 0, 7), ("b", 0, 2)])
    run([("a", 7, 8), ("b", 2, 11)])
    run([("a", 8, 23), ("b", 11, 12)], end=["a"])
    run([("b", 12, 13), ("c", 0, 9)], end=["c"])
    run([("b", 13, 17), ("d", 0, 5)], end=["b"])
    run([("d", 5, 31)], end=["d"])
    for rid in prompts:
        torch.testing.assert_close(torch.cat(got[rid]), expected[rid], rtol=1e-4, atol=1e-5)
    h.cache.assert_consistent([])
    assert h.cache.num_used_pages() == 0


def test_a_step_padded_up_to_a_timed_number_of_rows_keeps_its_logits(tmp_path):
    """A step of portions a little short of a row count the matrix library was timed for gets rows of a sequence on the
    null page: with every slot but one decoding beside the portions (the padding is then one sequence more than
    ``max_num_seqs``), the logits are those of the same step unpadded, and the null page is all the padding wrote to."""
    name = "B"
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    prompts = {rid: random_tokens(config["vocab_size"], n, seed=50 + i) for i, (rid, n) in enumerate([("a", 12), ("b", 9), ("c", 15), ("d", 40)])}

    def run(tuned):
        h = Harness(folder, TorchOps(), torch.float32, "cpu", PAGE_SIZE[name], num_pages=32, max_num_seqs=4, max_num_tokens=64)
        h.runner.tuned_row_counts = tuned
        for rid in "abc":  # three of the four slots decode
            h.feed([(rid, prompts[rid][:-1], [])])
        batch = [(rid, prompts[rid][-1:], [0]) for rid in "abc"] + [("d", prompts["d"], [0, 39])]
        out = h.feed(batch)
        return h, out

    plain, want = run([])
    padded, got = run([48])  # 43 rows -> 48: five rows more, within the 12% that a step may grow by
    assert padded.runner.num_padded_steps == 1 and plain.runner.num_padded_steps == 0
    torch.testing.assert_close(got, want, rtol=0, atol=0)
    torch.testing.assert_close(got[-1], qwen2_logits(config, weights, prompts["d"])[-1], rtol=1e-4, atol=1e-5)
    for mine, theirs in zip(padded.cache.groups, plain.cache.groups):
        for name in mine.tensors:
            assert torch.equal(mine.tensors[name][:, 1:], theirs.tensors[name][:, 1:])  # everything but the null page


def test_a_fixed_workspace_refuses_to_replace_a_buffer():
    import pytest
    import torch

    from velox_amd.engine.batch import Workspace, WorkspaceError

    workspace = Workspace(torch.device("cpu"))
    first = workspace.get("a", 10)
    assert workspace.get("a", 4).data_ptr() == first.data_ptr()
    grown = workspace.get("a", 100)  # not fixed: grows on demand
    assert grown.numel() == 100
    workspace.reserve("b", 50)
    workspace.fix()
    assert workspace.get("a", 100).data_ptr() == grown.data_ptr()
    assert workspace.get("b", 50).numel() == 50
    with pytest.raises(WorkspaceError, match="'a'"):
        workspace.get("a", 101)
    with pytest.raises(WorkspaceError, match="nothing"):
        workspace.get("c", 1)


def test_without_a_gpu_the_engine_refuses_loudly(tmp_path, monkeypatch):
    """No CPU path stands behind the kernels: asking for the product's operations without a GPU, or on the CPU, is one
    clear error, also through the Python entry point; so is a box without the compiler and without built libraries."""
    from velox_amd import Engine, EngineConfig
    from velox_amd.kernels import KernelError, build, load_ops

    with pytest.raises(KernelError, match="no CPU path"):
        load_ops("cpu")
    if not torch.cuda.is_available():
        with pytest.raises(KernelError, match="no GPU is visible"):
            load_ops("cuda")
        folder = make_folder(tmp_path, "A")
        with pytest.raises(KernelError, match="no GPU is visible"):
            Engine.from_pretrained(EngineConfig(model=folder, dtype="bfloat16"))
    monkeypatch.setenv("HIPCC", str(tmp_path / "no_such_compiler"))
    monkeypatch.setenv("PATH", str(tmp_path))
    real_isfile = build.os.path.isfile
    monkeypatch.setattr(build.os.path, "isfile", lambda path: False if str(path).endswith("hipcc") else real_isfile(path))
    with pytest.raises(build.BuildError, match="hipcc not found"):
        build.find_hipcc()
