"""Weights by name from safetensors: one error for everything wrong, dtypes, the random-weights folder."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY_A, TINY_B, make_folder
from velox_amd.config import load_config
from velox_amd.engine.engine import build_model
from velox_amd.weights import WeightsError, bind_from_checkpoint, bind_random, held_dtype, write_random_model


def _load(folder, dtype=torch.float32):
    model = build_model(load_config(folder), dtype, "cpu")
    bind_from_checkpoint(model, folder, dtype, "cpu")
    return model


def test_random_folder_round_trip_and_fusion(tmp_path):
    folder = make_folder(tmp_path, "B")
    raw = load_file(os.path.join(folder, "model.safetensors"))
    assert "lm_head.weight" in raw and raw["model.layers.2.self_attn.k_proj.bias"].shape == (32,)
    model = _load(folder)
    mixer = model.blocks[1].mixer
    p = "model.layers.1.self_attn."
    want = torch.cat([raw[p + "q_proj.weight"], raw[p + "k_proj.weight"], raw[p + "v_proj.weight"]])
    assert torch.equal(mixer.qkv_weight, want)
    assert torch.equal(mixer.qkv_bias_vec, torch.cat([raw[p + "q_proj.bias"], raw[p + "k_proj.bias"], raw[p + "v_proj.bias"]]))
    ff = model.blocks[1].feed_forward
    assert torch.equal(ff.gate_up_weight, torch.cat([raw["model.layers.1.mlp.gate_proj.weight"], raw["model.layers.1.mlp.up_proj.weight"]]))
    assert torch.equal(model.head.weight, raw["lm_head.weight"]) and model.head.weight.data_ptr() != model.embedding.table.data_ptr()
    # norm weights are around one, everything else around zero
    assert abs(float(raw["model.norm.weight"].mean()) - 1.0) < 0.05 and abs(float(raw["model.embed_tokens.weight"].mean())) < 0.01
    assert abs(float(raw["model.embed_tokens.weight"].std()) - 0.02) < 0.002


def test_same_seed_same_weights_other_seed_other_weights(tmp_path):
    a = load_file(os.path.join(write_random_model(TINY_A, str(tmp_path / "a"), 5, "float32"), "model.safetensors"))
    b = load_file(os.path.join(write_random_model(TINY_A, str(tmp_path / "b"), 5, "float32"), "model.safetensors"))
    c = load_file(os.path.join(write_random_model(TINY_A, str(tmp_path / "c"), 6, "float32"), "model.safetensors"))
    assert all(torch.equal(a[k], b[k]) for k in a) and not torch.equal(a["model.norm.weight"], c["model.norm.weight"])
    # in-memory binding with the host generator gives the folder's values
    model = build_model(load_config(str(tmp_path / "a")), torch.float32, "cpu")
    bind_random(model, 5, torch.float32, "cpu", storage_dtype=torch.float32)
    assert torch.equal(model.embedding.table, a["model.embed_tokens.weight"])
    assert torch.equal(model.final_norm.weight, a["model.norm.weight"])


def test_tied_head_shares_the_table(tmp_path):
    folder = make_folder(tmp_path, "A")
    assert "lm_head.weight" not in load_file(os.path.join(folder, "model.safetensors"))
    model = _load(folder)
    assert model.head.weight.data_ptr() == model.embedding.table.data_ptr()


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_folder(tmp_path, "B")
    path = os.path.join(folder, "model.safetensors")
    raw = load_file(path)
    del raw["model.layers.0.self_attn.q_proj.bias"]
    del raw["model.norm.weight"]
    raw["model.layers.7.mlp.up_proj.weight"] = torch.zeros(3, 3)
    raw["extra.tensor"] = torch.zeros(1)
    raw["model.layers.1.mlp.down_proj.weight"] = torch.zeros(96, 100)
    raw["lm_head.weight"] = torch.zeros(320, 95)
    save_file(raw, path)
    with pytest.raises(WeightsError) as err:
        _load(folder)
    e = err.value
    assert e.missing == ["model.layers.0.self_attn.q_proj.bias", "model.norm.weight"]
    assert e.unexpected == ["extra.tensor", "model.layers.7.mlp.up_proj.weight"]
    assert len(e.wrong_shape) == 2 and any("down_proj" in w and "(96, 100)" in w and "(96, 224)" in w for w in e.wrong_shape)
    text = str(e)
    for fragment in ("missing tensors (2)", "unexpected tensors (2)", "wrong shapes (2)", "extra.tensor", "lm_head.weight"):
        assert fragment in text


def test_missing_files(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(FileNotFoundError):
        _load(str(tmp_path))


def test_dtypes_kept(tmp_path):
    # stored bfloat16: stays bfloat16 in a bfloat16 run, widened exactly in a float32 run; vectors always float32
    folder = make_folder(tmp_path, "B", "bfloat16")
    raw = load_file(os.path.join(folder, "model.safetensors"))
    bf = _load(folder, torch.bfloat16)
    assert bf.embedding.table.dtype == torch.bfloat16 and bf.blocks[0].mixer.qkv_weight.dtype == torch.bfloat16
    assert bf.final_norm.weight.dtype == torch.float32 and bf.blocks[0].mixer.qkv_bias_vec.dtype == torch.float32
    assert torch.equal(bf.final_norm.weight, raw["model.norm.weight"].float())
    wide = _load(folder, torch.float32)
    assert wide.embedding.table.dtype == torch.float32 and torch.equal(wide.embedding.table, raw["model.embed_tokens.weight"].float())
    # stored float32 takes the run dtype too (reference src/weight_loader.py:127): rounded once, to nearest even, so the
    # tensors are those of a folder that stores the same values in bfloat16
    folder32 = make_folder(tmp_path, "B", "float32")
    raw32 = load_file(os.path.join(folder32, "model.safetensors"))
    narrowed = _load(folder32, torch.bfloat16)
    assert narrowed.blocks[0].mixer.qkv_weight.dtype == torch.bfloat16 and narrowed.embedding.table.dtype == torch.bfloat16
    assert narrowed.head.weight.dtype == torch.bfloat16 and narrowed.blocks[2].feed_forward.down_weight.dtype == torch.bfloat16
    assert torch.equal(narrowed.blocks[0].mixer.qkv_weight, bf.blocks[0].mixer.qkv_weight)
    assert torch.equal(narrowed.head.weight, raw32["lm_head.weight"].to(torch.bfloat16))
    assert narrowed.final_norm.weight.dtype == torch.float32 and torch.equal(narrowed.final_norm.weight, raw32["model.norm.weight"])
    assert held_dtype("matrix", torch.float32, torch.bfloat16) == torch.bfloat16
    assert held_dtype("matrix", torch.int64, torch.bfloat16) == torch.int32
    assert held_dtype("matrix", torch.float16, torch.bfloat16) == torch.bfloat16
    # a part may ask for a tensor as stored: 32-bit stays 32-bit
    assert held_dtype("stored", torch.float32, torch.bfloat16) == torch.float32
    assert held_dtype("stored", torch.bfloat16, torch.float32) == torch.float32
    assert held_dtype("stored", torch.bfloat16, torch.bfloat16) == torch.bfloat16


def test_a_bfloat16_run_on_a_float32_folder_gives_the_logits_of_the_bfloat16_folder(tmp_path):
    from helpers import PAGE_SIZE, Harness, random_tokens
    from torch_ops import TorchOps

    tokens = random_tokens(TINY_B["vocab_size"], 20, seed=3)
    logits = []
    for storage in ("float32", "bfloat16"):
        folder = make_folder(tmp_path, "B", storage)
        if storage == "float32":
            # vectors (biases, norm weights) are held in float32 as stored: give them the values the other folder holds,
            # so that the matrices' conversion is the only difference left
            path = os.path.join(folder, "model.safetensors")
            raw = load_file(path)
            save_file({name: t.to(torch.bfloat16).float() if t.dim() == 1 else t for name, t in raw.items()}, path)
        h = Harness(folder, TorchOps(), torch.bfloat16, "cpu", PAGE_SIZE["B"], num_pages=16)
        assert h.model.blocks[1].feed_forward.gate_up_weight.dtype == torch.bfloat16
        logits.append(h.feed([("a", tokens, list(range(len(tokens))))]))
    assert torch.equal(logits[0], logits[1])


def _shard(folder, pieces=2, drop=None):
    """Splits the folder's model.safetensors into ``pieces`` shards with an index file (the layout of every larger
    checkpoint, reference ``src/weight_loader.py:31-55``); ``drop`` names a tensor left out of its shard."""
    path = os.path.join(folder, "model.safetensors")
    raw = load_file(path)
    os.unlink(path)
    names = sorted(raw)
    weight_map = {}
    for index in range(pieces):
        shard = f"model-{index + 1:05d}-of-{pieces:05d}.safetensors"
        mine = names[index::pieces]  # interleaved: the q, k and v rows of one fused tensor come from different files
        save_file({name: raw[name] for name in mine if name != drop}, os.path.join(folder, shard))
        weight_map.update({name: shard for name in mine})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w", encoding="utf-8") as handle:
        json.dump({"metadata": {"total_size": sum(t.numel() * t.element_size() for t in raw.values())}, "weight_map": weight_map}, handle)
    return raw


def test_sharded_checkpoint_with_an_index_file(tmp_path):
    folder = make_folder(tmp_path, "B")
    whole = _load(folder)
    raw = _shard(folder, pieces=3)
    assert not os.path.exists(os.path.join(folder, "model.safetensors"))
    sharded = _load(folder)
    for a, b in zip(whole.all_parts(), sharded.all_parts()):
        for attr in a.params():
            assert torch.equal(getattr(a, attr), getattr(b, attr)), (a.prefix, attr)
    p = "model.layers.2.self_attn."
    assert torch.equal(sharded.blocks[2].mixer.qkv_weight, torch.cat([raw[p + "q_proj.weight"], raw[p + "k_proj.weight"], raw[p + "v_proj.weight"]]))


def test_sharded_checkpoint_with_a_tensor_missing_from_its_shard(tmp_path):
    folder = make_folder(tmp_path, "A")
    _shard(folder, pieces=2, drop="model.layers.1.mlp.up_proj.weight")
    with pytest.raises(WeightsError) as err:
        _load(folder)
    assert err.value.missing == ["model.layers.1.mlp.up_proj.weight"] and not err.value.unexpected and not err.value.wrong_shape


def test_index_file_that_names_a_shard_that_is_not_there(tmp_path):
    folder = make_folder(tmp_path, "A")
    _shard(folder, pieces=2)
    os.unlink(os.path.join(folder, "model-00002-of-00002.safetensors"))
    with pytest.raises(FileNotFoundError, match="model-00002-of-00002.safetensors"):
        _load(folder)


def test_random_weights_in_memory_go_through_the_binder_of_folders(tmp_path):
    """``bind_random`` is the folder's binder fed from a stream of random tensors: fused rows, the tied head, held dtypes
    and the values themselves are the folder's, and reading a bound model back by checkpoint name gives the folder's file."""
    import velox_amd.weights.random_init as random_init
    from velox_amd.weights import RandomSource, named_tensors

    assert "setattr" not in open(random_init.__file__).read()
    for name, config in (("A", TINY_A), ("B", TINY_B)):
        folder = write_random_model(config, str(tmp_path / name), 11, "bfloat16")
        raw = load_file(os.path.join(folder, "model.safetensors"))
        for run_dtype in (torch.float32, torch.bfloat16):
            from_folder = _load(folder, run_dtype)
            in_memory = build_model(load_config(folder), run_dtype, "cpu")
            bind_random(in_memory, 11, run_dtype, "cpu", storage_dtype=torch.bfloat16)
            back = dict(named_tensors(in_memory))
            assert sorted(back) == sorted(raw)
            for key, stored in raw.items():
                assert torch.equal(back[key].float(), stored.float()), key
            for (_, a), (_, b) in zip(named_tensors(from_folder), named_tensors(in_memory)):
                assert a.dtype == b.dtype and torch.equal(a, b)
        tied = in_memory.head.weight.data_ptr() == in_memory.embedding.table.data_ptr()
        assert tied == bool(config["tie_word_embeddings"])
    # the stream has one generator: tensors out of the order of declaration are refused, not drawn from the wrong state
    source = RandomSource(build_model(load_config(folder), torch.float32, "cpu"), 3)
    with pytest.raises(RuntimeError, match="order of declaration"):
        source.tensor("model.norm.weight")


def test_unexpected_tensors_are_an_error_unless_told_to_ignore_them(tmp_path, capsys):
    folder = make_folder(tmp_path, "A")
    path = os.path.join(folder, "model.safetensors")
    raw = load_file(path)
    raw["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(raw, path)
    with pytest.raises(WeightsError) as err:
        _load(folder)
    assert err.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"] and "ignore_unexpected_weights=True" in str(err.value)
    model = build_model(load_config(folder), torch.float32, "cpu")
    bind_from_checkpoint(model, folder, torch.float32, "cpu", ignore_unexpected=True)
    assert "ignoring 1 tensors" in capsys.readouterr().out
    assert torch.equal(model.final_norm.weight, raw["model.norm.weight"])
    # a missing tensor is an error whatever is ignored
    del raw["model.norm.weight"]
    save_file(raw, path)
    with pytest.raises(WeightsError) as err:
        bind_from_checkpoint(model, folder, torch.float32, "cpu", ignore_unexpected=True)
    assert err.value.missing == ["model.norm.weight"] and err.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
