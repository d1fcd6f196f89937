"""What fixes the plain implementation beside the reference's text: special cases that reduce to a
library routine, and invariants, each chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from helpers import CONFIGS, make_folder, random_tokens
from plain_qwen2 import apply_rope, causal_attention, gated_mlp, qwen2_logits, read_model_folder, rms_norm, rope_tables


def test_rms_norm_is_the_library_routine_and_eps_sits_inside_the_root():
    x = torch.randn(5, 96, dtype=torch.float64)
    w = 1 + 0.1 * torch.randn(96, dtype=torch.float64)
    torch.testing.assert_close(rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5))
    tiny = torch.full((1, 8), 1e-4, dtype=torch.float64)
    got = rms_norm(tiny, torch.ones(8, dtype=torch.float64), 1e-6)
    torch.testing.assert_close(got, torch.full_like(got, 1e-4 / math.sqrt(1e-8 + 1e-6)))
    assert abs(float(got[0, 0]) - 1e-4 / (1e-4 + 1e-6)) > 0.5  # 1 / (sqrt(ms) + eps) would give ~0.99
    # the weight multiplies, with no offset: w = 0 gives 0 (a "1 + w" norm would not)
    assert float(rms_norm(x, torch.zeros(96, dtype=torch.float64), 1e-5).abs().max()) == 0.0


def test_rope_tables_and_pairing():
    d, theta = 16, 10000.0
    cos, sin = rope_tables(d, theta, 64, dtype=torch.float64)
    assert cos.shape == (64, 8)
    torch.testing.assert_close(cos[0], torch.ones(8, dtype=torch.float64))  # position 0 does not rotate
    # frequency 0 is 1 radian per position, the last one theta^-(d-2)/d
    assert abs(float(sin[1, 0]) - math.sin(1.0)) < 1e-6 and abs(float(sin[1, 7]) - math.sin(theta ** (-14 / 16))) < 1e-6
    x = torch.randn(3, 2, d, dtype=torch.float64)
    pos = torch.tensor([0, 5, 9])
    y = apply_rope(x, cos, sin, pos)
    torch.testing.assert_close(y[0], x[0])
    # the pair is (i, i + d/2), as a complex rotation: (lo + i hi) * exp(i * angle)
    z = torch.complex(x[..., :8], x[..., 8:]) * torch.polar(torch.ones(3, 1, 8, dtype=torch.float64), torch.outer(pos.double(), 1.0 / theta ** (torch.arange(0, d, 2).double() / d)).unsqueeze(1))
    torch.testing.assert_close(y, torch.cat([z.real, z.imag], -1), rtol=1e-6, atol=1e-6)
    # an interleaved pairing (2i, 2i + 1) would not keep the norm of the halves pair by pair
    torch.testing.assert_close((y[..., :8] ** 2 + y[..., 8:] ** 2), (x[..., :8] ** 2 + x[..., 8:] ** 2))
    # linear scaling divides the positions
    cos2, _ = rope_tables(d, theta, 64, factor=2.0, dtype=torch.float64)
    torch.testing.assert_close(cos2[10], cos[5], rtol=1e-6, atol=1e-6)


def test_rotated_scores_depend_on_distance_only():
    d = 32
    cos, sin = rope_tables(d, 1e6, 300, dtype=torch.float64)
    q, k = torch.randn(1, 1, d, dtype=torch.float64), torch.randn(1, 1, d, dtype=torch.float64)
    def score(m, n):
        return float((apply_rope(q, cos, sin, torch.tensor([m])) * apply_rope(k, cos, sin, torch.tensor([n]))).sum())
    # the angles are float32 products, as in the reference (src/rope.py:48-55): equal up to their rounding
    assert abs(score(17, 5) - score(117, 105)) < 1e-4 and abs(score(17, 5) - score(212, 200)) < 1e-4
    assert abs(score(17, 5) - score(5, 17)) > 1e-3  # a wrong sign of the sine would swap these


@pytest.mark.parametrize("nh,nkv", [(4, 4), (4, 2), (3, 1)])
def test_attention_is_the_library_routine(nh, nkv):
    t, d = 11, 16
    q, k, v = torch.randn(t, nh, d, dtype=torch.float64), torch.randn(t, nkv, d, dtype=torch.float64), torch.randn(t, nkv, d, dtype=torch.float64)
    got = causal_attention(q, k, v, 1 / math.sqrt(d))
    g = nh // nkv
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1).unsqueeze(0), k.repeat_interleave(g, 1).transpose(0, 1).unsqueeze(0),
        v.repeat_interleave(g, 1).transpose(0, 1).unsqueeze(0), is_causal=True).squeeze(0).transpose(0, 1)
    torch.testing.assert_close(got, want)
    torch.testing.assert_close(got[0], v[0].repeat_interleave(g, 0))  # the first token sees itself only
    # a window of 1 is "itself only" everywhere; a window wider than the sequence changes nothing
    torch.testing.assert_close(causal_attention(q, k, v, 0.25, window=1), v.repeat_interleave(g, 1))
    torch.testing.assert_close(causal_attention(q, k, v, 0.25, window=t), causal_attention(q, k, v, 0.25))


def test_mlp_is_the_library_routines():
    x = torch.randn(4, 24, dtype=torch.float64)
    wg, wu, wd = torch.randn(40, 24, dtype=torch.float64), torch.randn(40, 24, dtype=torch.float64), torch.randn(24, 40, dtype=torch.float64)
    torch.testing.assert_close(gated_mlp(x, wg, wu, wd), F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd))
    assert not torch.allclose(gated_mlp(x, wg, wu, wd), gated_mlp(x, wu, wg, wd))  # gate and up are not interchangeable


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_model_invariants(tmp_path, name):
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder, torch.float64)
    tokens = random_tokens(config["vocab_size"], 20, seed=3)
    base = qwen2_logits(config, weights, tokens, torch.float64)
    assert base.shape == (20, config["vocab_size"])
    # only distances between positions count: shifting every position changes nothing
    torch.testing.assert_close(qwen2_logits(config, weights, tokens, torch.float64, first_position=100), base, rtol=1e-3, atol=1e-4)
    # causal: a prefix gives the same logits
    torch.testing.assert_close(qwen2_logits(config, weights, tokens[:9], torch.float64), base[:9], rtol=1e-9, atol=1e-11)
    # the norms matter: with random norm weights around one, dropping the final norm's weight changes the logits
    changed = dict(weights)
    changed["model.norm.weight"] = torch.ones_like(weights["model.norm.weight"])
    assert not torch.allclose(qwen2_logits(config, changed, tokens, torch.float64), base, rtol=1e-3, atol=1e-5)
    # a bias matters too
    changed = dict(weights)
    changed["model.layers.0.self_attn.k_proj.bias"] = torch.zeros_like(weights["model.layers.0.self_attn.k_proj.bias"])
    assert not torch.allclose(qwen2_logits(config, changed, tokens, torch.float64), base, rtol=1e-4, atol=1e-7)
    # float32 agrees with float64 to rounding
    config32, weights32 = read_model_folder(folder, torch.float32)
    torch.testing.assert_close(qwen2_logits(config32, weights32, tokens).double(), base, rtol=2e-4, atol=2e-6)


def test_tied_head_uses_the_embedding_table(tmp_path):
    folder = make_folder(tmp_path, "A")
    config, weights = read_model_folder(folder, torch.float64)
    assert "lm_head.weight" not in weights and config["tie_word_embeddings"]
    tokens = random_tokens(256, 6, 1)
    untied = dict(config, tie_word_embeddings=False)
    weights2 = dict(weights)
    weights2["lm_head.weight"] = weights["model.embed_tokens.weight"]
    torch.testing.assert_close(qwen2_logits(untied, weights2, tokens, torch.float64), qwen2_logits(config, weights, tokens, torch.float64))


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_without_the_sub_layers_outputs_the_model_is_norm_of_the_embedding_times_head(tmp_path, name):
    """With every o_proj and down_proj zero the sub-layers add nothing, and what is left fixes the residual's frame:
    logits = final_norm(E[ids]) @ head^T.  A post-norm block (the residual itself normed), a residual that carries the
    normed input on, or a scale on the embeddings would each leave something behind."""
    folder = make_folder(tmp_path, name)
    config, weights = read_model_folder(folder, torch.float64)
    for key in weights:
        if key.endswith("o_proj.weight") or key.endswith("down_proj.weight"):
            weights[key] = torch.zeros_like(weights[key])
    tokens = random_tokens(config["vocab_size"], 12, seed=8)
    table = weights["model.embed_tokens.weight"]
    head = table if config["tie_word_embeddings"] else weights["lm_head.weight"]
    want = F.rms_norm(table[torch.tensor(tokens)], (config["hidden_size"],), weights["model.norm.weight"], config["rms_norm_eps"]) @ head.T
    torch.testing.assert_close(qwen2_logits(config, weights, tokens, torch.float64), want, rtol=1e-10, atol=1e-12)
    # and the feed-forward reads the NORMED residual: with the norm before it weighted zero it sees zeros and gives
    # down(silu(0) * 0) = 0, as if its down_proj were zero
    _, full = read_model_folder(folder, torch.float64)
    silenced = dict(full)
    for key in full:
        if key.endswith("post_attention_layernorm.weight"):
            silenced[key] = torch.zeros_like(full[key])
    no_mlp = dict(full)
    for key in full:
        if key.endswith("down_proj.weight"):
            no_mlp[key] = torch.zeros_like(full[key])
    torch.testing.assert_close(qwen2_logits(config, silenced, tokens, torch.float64), qwen2_logits(config, no_mlp, tokens, torch.float64), rtol=1e-10, atol=1e-12)


def test_one_layer_put_together_from_library_routines_only():
    """One layer of the third tiny configuration (6 heads of 48 channels on a width of 80: head_dim is not width / heads)
    assembled from ``F.rms_norm``, ``F.linear``, ``F.silu``, ``F.scaled_dot_product_attention`` with its DEFAULT scale
    (1 / sqrt of the last dimension = 48) and the rotation pinned above.  It fixes what the reading alone fixed: the order
    norm -> sub-layer -> add (twice), and the scale head_dim^-0.5 (width / heads = 13.3 would differ)."""
    config = dict(CONFIGS["C"], num_hidden_layers=1)
    hidden, nh, nkv, d, inner, vocab = 80, 6, 2, 48, 150, 263
    generator = torch.Generator().manual_seed(5)

    def draw(*shape, around=0.0):
        return around + 0.02 * torch.randn(*shape, generator=generator, dtype=torch.float64)

    p = "model.layers.0."
    w = {"model.embed_tokens.weight": draw(vocab, hidden), "lm_head.weight": draw(vocab, hidden), "model.norm.weight": draw(hidden, around=1.0),
         p + "input_layernorm.weight": draw(hidden, around=1.0), p + "post_attention_layernorm.weight": draw(hidden, around=1.0),
         p + "self_attn.q_proj.weight": 8 * draw(nh * d, hidden), p + "self_attn.q_proj.bias": 8 * draw(nh * d),
         p + "self_attn.k_proj.weight": 8 * draw(nkv * d, hidden), p + "self_attn.k_proj.bias": 8 * draw(nkv * d),
         p + "self_attn.v_proj.weight": draw(nkv * d, hidden), p + "self_attn.v_proj.bias": draw(nkv * d),
         p + "self_attn.o_proj.weight": draw(hidden, nh * d), p + "mlp.gate_proj.weight": draw(inner, hidden),
         p + "mlp.up_proj.weight": draw(inner, hidden), p + "mlp.down_proj.weight": draw(hidden, inner)}
    tokens = random_tokens(vocab, 17, seed=4)
    t = len(tokens)
    eps = config["rms_norm_eps"]
    cos, sin = rope_tables(d, config["rope_theta"], t, factor=2.0, dtype=torch.float64)
    positions = torch.arange(t)

    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    a = F.rms_norm(h, (hidden,), w[p + "input_layernorm.weight"], eps)
    q = apply_rope(F.linear(a, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]).view(t, nh, d), cos, sin, positions)
    k = apply_rope(F.linear(a, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]).view(t, nkv, d), cos, sin, positions)
    v = F.linear(a, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).view(t, nkv, d)
    heads = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(nh // nkv, 1).transpose(0, 1)[None],
                                           v.repeat_interleave(nh // nkv, 1).transpose(0, 1)[None], is_causal=True)[0].transpose(0, 1)
    h = h + F.linear(heads.reshape(t, nh * d), w[p + "self_attn.o_proj.weight"])
    m = F.rms_norm(h, (hidden,), w[p + "post_attention_layernorm.weight"], eps)
    h = h + F.linear(F.silu(F.linear(m, w[p + "mlp.gate_proj.weight"])) * F.linear(m, w[p + "mlp.up_proj.weight"]), w[p + "mlp.down_proj.weight"])
    want = F.linear(F.rms_norm(h, (hidden,), w["model.norm.weight"], eps), w["lm_head.weight"])

    got = qwen2_logits(config, w, tokens, torch.float64)
    torch.testing.assert_close(got, want, rtol=1e-9, atol=1e-11)
    # the scores are large enough (q and k scaled up) for another scale to show: width / heads in place of head_dim
    other = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.repeat_interleave(nh // nkv, 1).transpose(0, 1)[None],
                                           v.repeat_interleave(nh // nkv, 1).transpose(0, 1)[None], is_causal=True, scale=(hidden / nh) ** -0.5)[0].transpose(0, 1)
    assert float((other - heads).abs().max()) > 1e-4


def test_what_the_filters_keep_when_logits_are_equal_at_the_cut():
    """The plain sampler the kernels are compared with, on cases small enough to state by hand.  Tokens of equal value
    share rank and mass, so a cut inside a run of equal logits keeps the whole run: top_k = 2 over [3, 2, 2, 2, 1] keeps four
    tokens.  The reference keeps exactly k, whichever of the equal ones its sort puts first (engine/sampler.py:218-221)."""
    import numpy as np
    from torch_ops import TorchOps

    def kept(row, temperature, top_p, top_k):
        option = np.zeros(6, dtype=np.int32)
        option.view(np.float32)[0:2] = (temperature, top_p)
        option[2:] = (top_k, 11, 22, 0)
        return sorted(np.flatnonzero(np.isfinite(TorchOps.sample_row(np.asarray(row, dtype=np.float32), option)[1])))

    assert kept([3, 2, 2, 2, 1], 1.0, 1.0, 2) == [0, 1, 2, 3]
    assert kept([3, 2, 2, 2, 1], 1.0, 1.0, 1) == [0]
    assert kept([1, 2, 5, 2, 4], 1.0, 1.0, 2) == [2, 4]
    # top-p: a token is kept while the mass of the strictly larger ones is below p; the best one always is
    p = np.exp([3.0, 2, 2, 2, 1]) / np.exp([3.0, 2, 2, 2, 1]).sum()
    assert kept([3, 2, 2, 2, 1], 1.0, float(p[0]) * 0.99, 0) == [0]
    assert kept([3, 2, 2, 2, 1], 1.0, float(p[0]) * 1.01, 0) == [0, 1, 2, 3]
    assert kept([3, 2, 2, 2, 1], 1.0, 1e-20, 0) == [0]
    assert kept([3, 2, 2, 2, 1], 1.0, 1.0, 0) == [0, 1, 2, 3, 4]
