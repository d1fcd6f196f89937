"""The replay program's logic on a CPU: the kernels' plain references stand in for the kernels, everything
else (model, step function, cache manager, the trace format) is the product's."""
import pytest
import torch

import replay_cases as rc
from helpers import PAGE_SIZE, make_folder
from plain_qwen2 import read_model_folder
from torch_ops import TorchOps
from velox_amd.engine.replay import Replayer, TraceError

TOL = dict(rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("name", ["A", "B"])
def test_all_ways_of_cutting_agree_with_the_plain_model(tmp_path, name):
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder)
    requests = rc.request_set(config["vocab_size"], [41, 17, 58, 9, 33, 26], seed=3)
    expected = rc.expected_logits(config, weights, requests)
    page = PAGE_SIZE[name]
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)),
                         ("portions", rc.changing_portions(requests)), ("mixed", rc.mixed(requests, seed=5)),
                         ("recompute", rc.mixed(requests, seed=6, preempt=("r0", "r2", "r4")))):
        pool = rc.tokens_needed(trace, page)
        replayer = Replayer(folder, "float32", pool, block_size=page, device="cpu", ops=TorchOps())
        outputs = rc.run_trace(replayer, trace)
        got = rc.collect(trace, outputs, requests)
        for rid in requests:
            torch.testing.assert_close(got[rid], expected[rid], msg=lambda m: f"{name} {label} {rid}: {m}", **TOL)
        if label == "recompute":
            # the requests that were ended half way and fed again from their first token: both runs gave the plain logits
            first = rc.first_runs(trace, outputs, requests)
            for rid in ("r0", "r2", "r4"):
                assert sum(1 for r in trace if rid in r["end"]) == 2
                for position, row in first[rid].items():
                    torch.testing.assert_close(torch.from_numpy(row), expected[rid][position], **TOL)
        if label in ("mixed", "recompute"):
            # the pool is so small that pages were handed out more than once
            total_pages = sum((len(t) + page - 1) // page for t in requests.values())
            assert total_pages > replayer.cache.num_total_pages


def test_trace_errors_are_reported(tmp_path):
    folder = make_folder(tmp_path, "A")
    replayer = Replayer(folder, "float32", 16, block_size=4, device="cpu", ops=TorchOps(), max_live=2)
    with pytest.raises(TraceError, match="vocabulary"):
        replayer.step({"step": 0, "entries": [{"id": "a", "tokens": [1, 999], "want": []}], "end": []})
    assert replayer.step({"step": 1, "entries": [{"id": "b", "tokens": [1, 2, 3], "want": []}], "end": []}) is None
    with pytest.raises(TraceError, match="out of cache pages|limit"):
        replayer.step({"step": 2, "entries": [{"id": "c", "tokens": list(range(14)), "want": []}], "end": []})
    with pytest.raises(TraceError, match="twice"):
        replayer.step({"step": 3, "entries": [{"id": "b", "tokens": [1], "want": []}, {"id": "b", "tokens": [1], "want": []}], "end": []})
    with pytest.raises(ValueError, match="want"):
        replayer.step({"step": 4, "entries": [{"id": "b", "tokens": [1], "want": [3]}], "end": []})
