"""Each part of a layer alone against the plain functions, and parts the framework does not have: a toy mixer
with state of its own, registered, built and stepped from here without touching the framework's files; a
layer that runs twice; a layer that reads another layer's cache; a windowed layer whose pages go back."""
import math
from typing import Dict

import pytest
import torch

from plain_qwen2 import apply_rope, causal_attention, gated_mlp, rms_norm, rope_tables
from velox_amd.cache import CacheManager
from velox_amd.config.model_config import ModelConfig
from velox_amd.config.registry import architecture_name, config_from_dict, get_architecture, register_architecture
from velox_amd.engine.batch import StepEntry
from velox_amd.engine.engine import build_model
from velox_amd.engine.runner import ModelRunner
from velox_amd.parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, StateNeed, make_part, register_part, single
from velox_amd.parts.base import FeedForward, Mixer, PositionEncoding, fused_rows
from velox_amd.weights import bind_random
from velox_amd.weights.random_init import random_tensors

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from velox_amd.kernels import load_ops

    return load_ops("cuda")


class Ctx:
    """The few fields a part reads, for calling one part alone."""

    def __init__(self, ops, dtype, **fields):
        self.ops, self.dtype = ops, dtype
        self.__dict__.update(fields)


def fill(part, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    values = {}
    for attr, param in part.params().items():
        t = torch.randn(param.shape, generator=g) * (0.3 if param.role == "matrix" else 0.1)
        if param.init == "one_plus_normal":
            t = t + 1
        held = torch.float32 if param.role == "vector" else dtype
        setattr(part, attr, t.to(held).cuda())
        values[attr] = t
    return values


def test_rmsnorm_part_owns_the_residual(ops):
    norm = make_part("norm", "rmsnorm", prefix="n.", hidden_size=96, eps=1e-5)
    w = fill(norm, 0)["weight"]
    ctx = Ctx(ops, torch.float32)
    residual = torch.randn(7, 96).cuda()
    delta = torch.randn(7, 96).cuda()
    before = residual.clone()
    out = norm.forward(residual, delta, ctx)
    torch.testing.assert_close(residual, before + delta)
    torch.testing.assert_close(out.cpu(), rms_norm((before + delta).cpu(), w, 1e-5), rtol=1e-5, atol=1e-6)
    rows = torch.tensor([6, 2], dtype=torch.int32).cuda()
    kept = residual.clone()
    out = norm.forward(residual, delta, ctx, rows=rows)
    torch.testing.assert_close(residual, kept)
    torch.testing.assert_close(out.cpu(), rms_norm((kept + delta).cpu()[[6, 2]], w, 1e-5), rtol=1e-5, atol=1e-6)


def test_rotary_part_builds_the_reference_tables():
    rope = make_part("position", "rotary", rotary_dim=32, theta=1e6, max_position=300, scaling_factor=2.0)
    rope.finalize(torch.device("cuda"), torch.bfloat16)
    cos, sin = rope.rotary_tables()
    want_cos, want_sin = rope_tables(32, 1e6, 300, factor=2.0)
    assert cos.dtype == torch.float32 and cos.shape == (300, 16)
    torch.testing.assert_close(cos.cpu(), want_cos, rtol=0, atol=0)
    torch.testing.assert_close(sin.cpu(), want_sin, rtol=0, atol=0)
    assert make_part("position", "none").rotary_tables() is None


def test_gated_mlp_part(ops):
    ff = make_part("feed_forward", "gated_mlp", prefix="m.", hidden_size=80, intermediate_size=150)
    w = fill(ff, 1)
    x = torch.randn(9, 80)
    got = ff.forward(x.cuda(), Ctx(ops, torch.float32)).cpu()
    want = gated_mlp(x, w["gate_up_weight"][:150], w["gate_up_weight"][150:], w["down_weight"])
    # (as close to the float64 result as the plain float32 one is, within a factor of two: float32 sums of these sizes
    # differ by more than a fixed small tolerance from one order of adding to another)
    exact = gated_mlp(x.double(), w["gate_up_weight"][:150].double(), w["gate_up_weight"][150:].double(), w["down_weight"].double())
    assert float((got.double() - exact).abs().max()) <= 2 * float((want.double() - exact).abs().max()) + 1e-7
    torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-4 * float(want.abs().max()))  # and no gross difference


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_and_head_parts(ops, dtype):
    """The parts at the two ends alone: the looked-up rows come out as the float32 residual stream, exactly; the head is a
    product without bias on the rows it is given, in float32; tied, it declares the table's name as its source."""
    vocab, hidden = 263, 80
    embedding = make_part("embedding", "table", name="emb.weight", vocab_size=vocab, hidden_size=hidden)
    table = fill(embedding, 3, dtype)["table"]
    ids = torch.tensor([5, 262, 0, 5, 77], dtype=torch.int32).cuda()
    out = embedding.forward(ids, Ctx(ops, dtype))
    assert out.dtype == torch.float32 and torch.equal(out.cpu(), table.to(dtype).float()[ids.long().cpu()])
    assert embedding.params()["table"].product is False
    head = make_part("head", "linear", name="out.weight", vocab_size=vocab, hidden_size=hidden, tied_to=None)
    w = fill(head, 4, dtype)["weight"]
    rows = (torch.randn(6, hidden) * 0.5).to(dtype)
    logits = head.forward(rows.cuda(), Ctx(ops, dtype))
    assert logits.dtype == torch.float32 and logits.shape == (6, vocab)
    want = rows.float() @ w.to(dtype).float().T
    torch.testing.assert_close(logits.cpu(), want, rtol=2e-4, atol=2e-4)
    tied = make_part("head", "linear", name="out.weight", vocab_size=vocab, hidden_size=hidden, tied_to="emb.weight")
    assert tied.params()["weight"].alias_of == "emb.weight" and head.params()["weight"].alias_of is None


def test_pre_norm_block_alone(ops):
    """h + mixer(norm1(h)), then + ff(norm2(.)): the block's last output is handed on, not added; with the norm that reads
    it next the caller gets the same sum.  The mixer here is a stand-in without a cache."""
    from velox_amd.parts.base import Mixer

    class Twice(Mixer):
        def forward(self, x, ctx, cache, owns_cache=True):
            return 2 * x

    hidden, inter = 96, 160
    norm1 = make_part("norm", "rmsnorm", prefix="n1.", hidden_size=hidden, eps=1e-5)
    norm2 = make_part("norm", "rmsnorm", prefix="n2.", hidden_size=hidden, eps=1e-5)
    ff = make_part("feed_forward", "gated_mlp", prefix="m.", hidden_size=hidden, intermediate_size=inter)
    block = make_part("arrangement", "pre_norm", prefix="b.", mixer=Twice("x."), feed_forward=ff, mixer_norm=norm1, ff_norm=norm2)
    assert block.input_norm() is norm1 and block.cache_need() is None and block.children() == (norm1, block.mixer, norm2, ff)
    w1, w2, wf = fill(norm1, 5)["weight"], fill(norm2, 6)["weight"], fill(ff, 7)
    g = torch.Generator().manual_seed(8)
    h = torch.randn(7, hidden, generator=g)
    carried = torch.randn(7, hidden, generator=g) * 0.1  # what the block before handed on
    residual = h.clone().cuda()
    pending = block.forward(residual, carried.cuda(), Ctx(ops, torch.float32), None, True)
    start = h + carried
    after_mixer = start + 2 * rms_norm(start, w1, 1e-5)
    torch.testing.assert_close(residual.cpu(), after_mixer, rtol=1e-5, atol=1e-5)  # the mixer's output is in, the feed-forward's is pending
    want = gated_mlp(rms_norm(after_mixer, w2, 1e-5), wf["gate_up_weight"][:inter], wf["gate_up_weight"][inter:], wf["down_weight"])
    # Outputs of size 30 that are sums of terms of both signs: float32 sums of them differ by some 1e-5 from one order of
    # adding to another (over 400 draws of h the plain float32 result misses rtol 1e-4, atol 1e-5 against the kernels'
    # in 26).  The yardstick is the same formula in float64: the kernels are as close to it as the plain float32 result is
    # (measured: 0.45 of its error in the median, 1.02 at most), within a factor of two.
    exact = gated_mlp(rms_norm(after_mixer.double(), w2.double(), 1e-5), wf["gate_up_weight"][:inter].double(), wf["gate_up_weight"][inter:].double(),
                      wf["down_weight"].double())
    assert float((pending.double().cpu() - exact).abs().max()) <= 2 * float((want.double() - exact).abs().max()) + 1e-7


@pytest.mark.parametrize("nh,nkv,d,hidden,bias,window", [(4, 2, 16, 64, True, None), (6, 2, 48, 80, False, None), (3, 1, 32, 96, True, 5)])
def test_attention_part_alone(ops, nh, nkv, d, hidden, bias, window):
    """One attention layer over two sequences cut in two steps each, against plain whole-sequence attention."""
    rope = make_part("position", "rotary", rotary_dim=d, theta=10000.0, max_position=128)
    rope.finalize(torch.device("cuda"), torch.float32)
    mixer = make_part("mixer", "attention", prefix="a.", hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, head_dim=d, position=rope, qkv_bias=bias, window=window)
    w = fill(mixer, 2)
    ops.attention_library(d)
    page = 4
    cache = CacheManager([mixer.cache_need()], page, 40, 4, torch.float32, "cuda")
    from velox_amd.engine.batch import BatchBuilder, Workspace

    builder = BatchBuilder(cache, "cuda", 256, 4)
    workspace = Workspace(torch.device("cuda"))
    lengths = {"x": 23, "y": 10}
    xs = {k: torch.randn(n, hidden) for k, n in lengths.items()}
    seqs = {k: cache.new_sequence() for k in lengths}
    got: Dict[str, list] = {k: [] for k in lengths}
    done = {k: 0 for k in lengths}
    for cuts in ({"x": 9, "y": 10}, {"x": 14}):
        entries, rows = [], []
        for k, n in cuts.items():
            assert cache.append(seqs[k], done[k], n)
            entries.append(StepEntry(seqs[k], [0] * n, done[k]))
            rows.append(xs[k][done[k]:done[k] + n])
        ctx = builder.build(entries, ops, torch.float32, workspace)
        out = mixer.forward(torch.cat(rows).cuda(), ctx, ctx.cache_view(0), True).cpu()
        at = 0
        for k, n in cuts.items():
            got[k].append(out[at:at + n])
            at += n
            done[k] += n
            cache.release_behind_window(seqs[k], done[k])
    cos, sin = rope_tables(d, 10000.0, 128)
    for k, n in lengths.items():
        qkv = xs[k] @ w["qkv_weight"].T + (w["qkv_bias_vec"] if bias else 0)
        q = apply_rope(qkv[:, : nh * d].reshape(n, nh, d), cos, sin, torch.arange(n))
        kk = apply_rope(qkv[:, nh * d:(nh + nkv) * d].reshape(n, nkv, d), cos, sin, torch.arange(n))
        v = qkv[:, (nh + nkv) * d:].reshape(n, nkv, d)
        want = causal_attention(q, kk, v, 1 / math.sqrt(d), window).reshape(n, nh * d) @ w["o_weight"].T
        torch.testing.assert_close(torch.cat(got[k]), want, rtol=2e-4, atol=2e-5)
    if window is not None:
        assert seqs["x"].tables[0][0] == 0  # pages behind the window went back while the request was running


# ----------------------------------------------------------------------------------------------------
# a toy architecture defined here: a mixer with per-request state, then an attention layer that runs twice,
# the second time beside an entry that reads the first run's cache
# ----------------------------------------------------------------------------------------------------
# where the toy architectures keep their tensors in a checkpoint (an architecture chooses its own names)
HF_NAMES = dict(mixer_prefix="self_attn.", feed_forward_prefix="mlp.", mixer_norm_prefix="input_layernorm.", ff_norm_prefix="post_attention_layernorm.")
HF_ENDS = dict(embed_name="model.embed_tokens.weight", head_name="lm_head.weight", final_norm_prefix="model.norm.")


class DecayingSumMixer(Mixer):
    """y_t = W s_t,  s_t = decay * s_{t-1} + x_t, with s kept per request in the cache manager's state slots."""

    graph_safe = False  # forward reads the step's slots and lengths on the host

    def __init__(self, prefix: str, hidden_size: int, decay: float) -> None:
        super().__init__(prefix)
        self.hidden_size, self.decay = hidden_size, decay
        self.weight = None

    def params(self):
        return {"weight": single("mix.weight", (self.hidden_size, self.hidden_size))}

    def cache_need(self):
        return StateNeed((("sum", (self.hidden_size,), torch.float32),))

    def forward(self, x, ctx, cache, owns_cache=True):
        state = cache.tensors["sum"]
        out = torch.empty_like(x)
        at = 0
        for slot, n in zip(ctx.slots.tolist(), ctx.q_lens):
            s = state[slot]
            for t in range(at, at + n):
                s = self.decay * s + x[t].float()
                out[t] = (self.weight.float() @ s).to(x.dtype)
            state[slot] = s
            at += n
        return out


def toy_spec(config, max_position=None) -> ModelSpec:
    raw = config.raw
    h = raw["hidden_size"]
    norm = PartSpec.of("rmsnorm", hidden_size=h, eps=raw["eps"])
    ff = PartSpec.of("gated_mlp", hidden_size=h, intermediate_size=raw["inter"])
    attention = PartSpec.of("attention", hidden_size=h, num_heads=4, num_kv_heads=2, head_dim=16, qkv_bias=False)
    layers = [
        LayerSpec("layers.0.", PartSpec.of("toy_decaying_sum", hidden_size=h, decay=raw["decay"]), ff, norm, norm, **dict(HF_NAMES, mixer_prefix="mixer.")),
        LayerSpec("layers.1.", attention, ff, norm, norm, position="rope", **HF_NAMES),
    ]
    schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1, cache_from=1)]
    return ModelSpec(vocab_size=raw["vocab_size"], hidden_size=h, max_position=256, layers=layers, schedule=schedule, final_norm=norm,
                     positions={"rope": PartSpec.of("rotary", rotary_dim=16, theta=10000.0, max_position=256)}, tie_head=True, **HF_ENDS)


def plain_toy(tensors: Dict[str, torch.Tensor], raw, tokens):
    h, eps, decay = raw["hidden_size"], raw["eps"], raw["decay"]
    n = len(tokens)
    cos, sin = rope_tables(16, 10000.0, n)
    x = tensors["model.embed_tokens.weight"][torch.tensor(tokens)]
    kept_kv = {}

    def ff(p, m):
        return gated_mlp(m, tensors[p + "mlp.gate_proj.weight"], tensors[p + "mlp.up_proj.weight"], tensors[p + "mlp.down_proj.weight"])

    for index, (layer, cache_from) in enumerate([(0, None), (1, None), (0, None), (1, None), (1, 1)]):
        p = f"layers.{layer}."
        a = rms_norm(x, tensors[p + "input_layernorm.weight"], eps)
        if layer == 0:
            s = torch.zeros(h)
            rows = []
            for t in range(n):
                s = decay * s + a[t]
                rows.append(tensors[p + "mixer.mix.weight"] @ s)
            mixed = torch.stack(rows)
        else:
            q = apply_rope((a @ tensors[p + "self_attn.q_proj.weight"].T).reshape(n, 4, 16), cos, sin, torch.arange(n))
            if cache_from is None:
                k = apply_rope((a @ tensors[p + "self_attn.k_proj.weight"].T).reshape(n, 2, 16), cos, sin, torch.arange(n))
                v = (a @ tensors[p + "self_attn.v_proj.weight"].T).reshape(n, 2, 16)
                kept_kv[index] = (k, v)
            else:
                k, v = kept_kv[cache_from]
            mixed = causal_attention(q, k, v, 0.25).reshape(n, 64) @ tensors[p + "self_attn.o_proj.weight"].T
        x = x + mixed
        x = x + ff(p, rms_norm(x, tensors[p + "post_attention_layernorm.weight"], eps))
    return rms_norm(x, tensors["model.norm.weight"], eps) @ tensors["model.embed_tokens.weight"].T


def test_toy_architecture_with_state_repeated_layer_and_shared_cache(ops):
    register_part("mixer", "toy_decaying_sum", DecayingSumMixer)
    register_architecture("ToyForCausalLM", lambda raw: ModelConfig(architecture_name(raw), dict(raw)), toy_spec)
    raw = {"architectures": ["ToyForCausalLM"], "hidden_size": 64, "inter": 96, "vocab_size": 101, "eps": 1e-5, "decay": 0.8}
    config = config_from_dict(raw)
    model = build_model(config, torch.float32, "cuda")
    needs = model.cache_needs()
    assert [type(n).__name__ for n in needs] == ["StateNeed", "PagedNeed", "StateNeed", "PagedNeed", "NoneType"]
    bind_random(model, 4, torch.float32, "cuda", storage_dtype=torch.float32)
    tensors = dict(random_tensors(model, 4))
    ops.prepare(model, torch.float32)
    cache = CacheManager(needs, 4, 40, 3, torch.float32, "cuda")
    assert len(cache.groups) == 1 and cache.groups[0].entries == [1, 3]  # both runs of the attention layer own a cache
    runner = ModelRunner(model, cache, ops, torch.float32, "cuda", 128, 3)
    g = torch.Generator().manual_seed(0)
    prompts = {k: torch.randint(0, 101, (n,), generator=g).tolist() for k, n in (("p", 29), ("q", 12), ("r", 40))}
    seqs = {k: cache.new_sequence() for k in prompts}
    done = {k: 0 for k in prompts}
    got = {k: [] for k in prompts}
    plan = [{"p": 5, "q": 12}, {"p": 1, "r": 17}, {"p": 23, "r": 2}, {"r": 21}]
    for cuts in plan:
        entries = []
        for k, n in cuts.items():
            assert cache.append(seqs[k], done[k], n)
            entries.append(StepEntry(seqs[k], prompts[k][done[k]:done[k] + n], done[k], list(range(n))))
        logits = runner.step(entries).cpu()
        at = 0
        for k, n in cuts.items():
            got[k].append(logits[at:at + n])
            at += n
            done[k] += n
    for k, tokens in prompts.items():
        torch.testing.assert_close(torch.cat(got[k]), plain_toy(tensors, raw, tokens), rtol=2e-4, atol=2e-5)
    # a slot that is taken again starts from zero state
    cache.free_sequence(seqs["q"])
    again = cache.new_sequence()
    assert cache.append(again, 0, 12)
    logits = runner.step([StepEntry(again, prompts["q"], 0, list(range(12)))]).cpu()
    torch.testing.assert_close(logits, torch.cat(got["q"]), rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------------------------------------------
# a second toy architecture: a feed-forward with routing (every token goes to one of three small experts) and a
# position encoding that is added to the embeddings instead of rotating queries and keys.  Both are defined here.
# ----------------------------------------------------------------------------------------------------
class RoutedFeedForward(FeedForward):
    """y_t = p_t * expert_{e_t}(x_t) with e_t = argmax of the router's logits and p_t its softmax probability."""

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, num_experts: int) -> None:
        super().__init__(prefix)
        self.hidden_size, self.intermediate_size, self.num_experts = hidden_size, intermediate_size, num_experts

    def params(self):
        h, i = self.hidden_size, self.intermediate_size
        out = {"router": single("router.weight", (self.num_experts, h))}
        for e in range(self.num_experts):
            out[f"gate_up_{e}"] = fused_rows((f"experts.{e}.gate.weight", f"experts.{e}.up.weight"), ((i, h), (i, h)))
            out[f"down_{e}"] = single(f"experts.{e}.down.weight", (h, i))
        return out

    def prepare_kernels(self, ops) -> None:
        for e in range(self.num_experts):
            self.prepare_weight(ops, f"gate_up_{e}", stacked=2)
            self.prepare_weight(ops, f"down_{e}")

    def forward(self, x, ctx):
        ops = ctx.ops
        logits = ops.linear(x, self.router, None, torch.float32)  # router logits in float32
        probs = torch.softmax(logits, dim=-1)
        choice = probs.argmax(dim=-1)
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for e in range(self.num_experts):
            rows = torch.nonzero(choice == e).flatten()
            if rows.numel() == 0:
                continue
            act = ops.linear_silu_mul(x[rows].contiguous(), self.operand(f"gate_up_{e}"), ctx.dtype)
            y = ops.linear(act, self.operand(f"down_{e}"), None, torch.float32)
            out[rows] = y * probs[rows, e].unsqueeze(1)
        return out.to(ctx.dtype)


class LearnedPositions(PositionEncoding):
    def __init__(self, max_position: int, hidden_size: int, prefix: str = "model.") -> None:
        super().__init__(prefix)
        self.max_position, self.hidden_size = max_position, hidden_size
        self.table = None

    def params(self):
        return {"table": single("wpe.weight", (self.max_position, self.hidden_size))}

    def on_embeddings(self, hidden, ctx):
        hidden += self.table[ctx.positions.long()].float()
        return hidden


def routed_spec(config, max_position=None) -> ModelSpec:
    raw = config.raw
    h = raw["hidden_size"]
    norm = PartSpec.of("rmsnorm", hidden_size=h, eps=raw["eps"])
    attention = PartSpec.of("attention", hidden_size=h, num_heads=2, num_kv_heads=1, head_dim=32, qkv_bias=True)
    layers = [
        LayerSpec("layers.0.", attention, PartSpec.of("toy_routed", hidden_size=h, intermediate_size=raw["inter"], num_experts=3), norm, norm, **HF_NAMES),
        LayerSpec("layers.1.", attention, PartSpec.of("gated_mlp", hidden_size=h, intermediate_size=raw["inter"]), norm, norm, **HF_NAMES),
        LayerSpec("layers.2.", attention, PartSpec.of("toy_routed", hidden_size=h, intermediate_size=raw["inter"], num_experts=3), norm, norm, **HF_NAMES),
    ]
    return ModelSpec(vocab_size=raw["vocab_size"], hidden_size=h, max_position=128, layers=layers, schedule=[ScheduleEntry(i) for i in range(3)],
                     final_norm=norm, positions={"learned": PartSpec.of("toy_learned", max_position=128, hidden_size=h)},
                     embedding_position="learned", tie_head=False, **HF_ENDS)


def plain_routed(tensors: Dict[str, torch.Tensor], raw, tokens):
    eps, n = raw["eps"], len(tokens)
    x = tensors["model.embed_tokens.weight"][torch.tensor(tokens)] + tensors["model.wpe.weight"][:n]
    for layer in range(3):
        p = f"layers.{layer}."
        a = rms_norm(x, tensors[p + "input_layernorm.weight"], eps)
        q = (a @ tensors[p + "self_attn.q_proj.weight"].T + tensors[p + "self_attn.q_proj.bias"]).reshape(n, 2, 32)
        k = (a @ tensors[p + "self_attn.k_proj.weight"].T + tensors[p + "self_attn.k_proj.bias"]).reshape(n, 1, 32)
        v = (a @ tensors[p + "self_attn.v_proj.weight"].T + tensors[p + "self_attn.v_proj.bias"]).reshape(n, 1, 32)
        x = x + causal_attention(q, k, v, 1.0 / math.sqrt(32)).reshape(n, 64) @ tensors[p + "self_attn.o_proj.weight"].T
        m = rms_norm(x, tensors[p + "post_attention_layernorm.weight"], eps)
        if layer == 1:
            x = x + gated_mlp(m, tensors[p + "mlp.gate_proj.weight"], tensors[p + "mlp.up_proj.weight"], tensors[p + "mlp.down_proj.weight"])
            continue
        probs = torch.softmax(m @ tensors[p + "mlp.router.weight"].T, dim=-1)
        choice = probs.argmax(dim=-1)
        rows = []
        for t in range(n):
            e = int(choice[t])
            y = gated_mlp(m[t:t + 1], tensors[p + f"mlp.experts.{e}.gate.weight"], tensors[p + f"mlp.experts.{e}.up.weight"], tensors[p + f"mlp.experts.{e}.down.weight"])
            rows.append(y[0] * probs[t, e])
        x = x + torch.stack(rows)
    return rms_norm(x, tensors["model.norm.weight"], eps) @ tensors["lm_head.weight"].T


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_architecture_with_routed_experts_and_learned_positions(ops, dtype):
    """Registered, built and stepped from here; in bfloat16 the steps are decode-sized, so the attention layers hand
    deferred norms to feed-forwards that do not know them (they get plain tensors) and take sinks the toy parts ignore."""
    register_part("feed_forward", "toy_routed", RoutedFeedForward)
    register_part("position", "toy_learned", LearnedPositions)
    register_architecture("RoutedToyForCausalLM", lambda raw: ModelConfig(architecture_name(raw), dict(raw)), routed_spec)
    raw = {"architectures": ["RoutedToyForCausalLM"], "hidden_size": 64, "inter": 128, "vocab_size": 90, "eps": 1e-6}
    model = build_model(config_from_dict(raw), dtype, "cuda")
    bind_random(model, 9, dtype, "cuda", storage_dtype=dtype)
    tensors = {name: value.to(dtype).float() for name, value in random_tensors(model, 9)}
    # the router's margins are small with weights of 0.02: widen them so that rounding does not flip a choice
    for layer in (0, 2):
        model.blocks[layer].feed_forward.router.mul_(40.0)
        tensors[f"layers.{layer}.mlp.router.weight"] = model.blocks[layer].feed_forward.router.float().cpu()
    needs = model.cache_needs()
    ops.prepare(model, dtype)
    cache = CacheManager(needs, 8, 30, 3, dtype, "cuda")
    runner = ModelRunner(model, cache, ops, dtype, "cuda", 128, 3)
    g = torch.Generator().manual_seed(1)
    prompts = {k: torch.randint(0, 90, (n,), generator=g).tolist() for k, n in (("p", 21), ("q", 9), ("r", 30))}
    seqs = {k: cache.new_sequence() for k in prompts}
    done = {k: 0 for k in prompts}
    got = {k: [] for k in prompts}
    plan = [{"p": 5, "q": 9}, {"p": 1, "r": 11}, {"p": 15, "r": 1}, {"r": 16}, {"r": 2}]
    for cuts in plan:
        entries = []
        for k, n in cuts.items():
            assert cache.append(seqs[k], done[k], n)
            entries.append(StepEntry(seqs[k], prompts[k][done[k]:done[k] + n], done[k], list(range(n))))
        logits = runner.step(entries).cpu()
        at = 0
        for k, n in cuts.items():
            got[k].append(logits[at:at + n])
            at += n
            done[k] += n
    bound = dict(rtol=2e-4, atol=2e-5) if dtype == torch.float32 else dict(rtol=5e-2, atol=5e-2)
    for k, tokens in prompts.items():
        want = plain_routed(tensors, raw, tokens)
        have = torch.cat(got[k])
        if dtype == torch.bfloat16:
            # a token whose two best experts are nearly tied may go either way in bfloat16: such rows are left out
            agree = (have.argmax(-1) == want.argmax(-1)).float().mean()
            assert agree > 0.8
            close = ((have - want).abs().amax(-1) < 0.1)
            assert close.float().mean() > 0.9, f"{k}: only {int(close.sum())} of {len(close)} rows match"
        else:
            torch.testing.assert_close(have, want, **bound)


# ----------------------------------------------------------------------------------------------------
# a third toy architecture: what stands at the two ends and how a layer is arranged are parts like the others.
# An embedding with a scale, a head with a bias and a soft cap on its logits, and a block whose mixer and feed-forward
# read the same normalised input side by side; all defined and registered here.
# ----------------------------------------------------------------------------------------------------
from velox_amd.parts import Block, Embedding, OutputHead, register_arrangement  # noqa: E402
from velox_amd.parts.base import Norm, Param  # noqa: E402


class ScaledEmbedding(Embedding):
    def __init__(self, name, vocab_size, hidden_size, scale):
        super().__init__("")
        self.name, self.vocab_size, self.hidden_size, self.scale = name, vocab_size, hidden_size, scale
        self.table = None

    def params(self):
        return {"table": single(self.name, (self.vocab_size, self.hidden_size), product=False)}

    def forward(self, token_ids, ctx):
        return ctx.ops.embed(token_ids, self.table).mul_(self.scale)


class SoftcapHead(OutputHead):
    def __init__(self, name, vocab_size, hidden_size, tied_to, cap):
        super().__init__("")
        self.name, self.vocab_size, self.hidden_size, self.tied_to, self.cap = name, vocab_size, hidden_size, tied_to, cap
        self.weight = self.bias = None

    def params(self):
        weight = single(self.name, (self.vocab_size, self.hidden_size))
        if self.tied_to is not None:
            weight = Param(weight.shape, weight.sources, weight.source_shapes, weight.role, weight.init, alias_of=self.tied_to)
        return {"weight": weight, "bias": single("head.bias", (self.vocab_size,), role="vector")}

    def prepare_kernels(self, ops):
        self.prepare_weight(ops, "weight")

    def forward(self, hidden_rows, ctx):
        logits = ctx.ops.linear(hidden_rows, self.operand("weight"), self.bias, torch.float32)
        return self.cap * torch.tanh(logits / self.cap)


class CenteredNorm(Norm):
    """y = (x - mean) / sqrt(var + eps) * weight + bias: no form that a product's epilogue could take over
    (``deferred_form`` stays None), so the products before it hand back tensors and this part adds them itself."""

    def __init__(self, prefix, hidden_size, eps):
        super().__init__(prefix)
        self.hidden_size, self.eps = hidden_size, eps
        self.weight = self.bias = None

    def params(self):
        return {"weight": single("weight", (self.hidden_size,), role="vector", init="one_plus_normal"), "bias": single("bias", (self.hidden_size,), role="vector")}

    def forward(self, residual, delta, ctx, rows=None):
        if delta is not None:
            delta = ctx.ops.materialize(delta)
            delta = (delta.sum(0) if delta.dim() == 3 else delta).float()
        if rows is None:
            if delta is not None:
                residual.add_(delta)
            x = residual
        else:
            x = residual[rows.long()] + (delta[rows.long()] if delta is not None else 0.0)
        return torch.nn.functional.layer_norm(x, (self.hidden_size,), self.weight, self.bias, self.eps).to(ctx.dtype)


class ParallelBlock(Block):
    """h = h + mixer(norm(h)) + ff(norm(h)): one norm, both sub-layers read it."""

    def __init__(self, prefix, mixer, feed_forward, mixer_norm, ff_norm):
        super().__init__(prefix)
        self.mixer, self.feed_forward, self.norm = mixer, feed_forward, mixer_norm  # (ff_norm is not used and owns no tensors here)

    def children(self):
        return (self.norm, self.mixer, self.feed_forward)

    def input_norm(self):
        return self.norm

    def forward(self, residual, pending, ctx, cache, owns_cache, next_norm=None):
        normed = ctx.ops.materialize(self.norm.forward(residual, pending, ctx))
        mixed = self.mixer.forward(normed, ctx, cache, owns_cache)
        residual.add_((mixed.sum(0) if mixed.dim() == 3 else mixed).float())  # (a product may hand back partial sums)
        return self.feed_forward.forward(normed, ctx)  # added by whoever normalises next


def ends_spec(config, max_position=None) -> ModelSpec:
    raw = config.raw
    h = raw["hidden_size"]
    norm = PartSpec.of("rmsnorm", hidden_size=h, eps=raw["eps"])
    attention = PartSpec.of("attention", hidden_size=h, num_heads=3, num_kv_heads=3, head_dim=32, qkv_bias=False)
    ff = PartSpec.of("gated_mlp", hidden_size=h, intermediate_size=raw["inter"])
    centered = PartSpec.of("toy_centered", hidden_size=h, eps=raw["eps"])
    layers = [LayerSpec("blocks.0.", attention, ff, norm, norm, position="rope", arrangement="toy_parallel"),
              LayerSpec("blocks.1.", attention, ff, centered, norm, position="rope")]  # (the framework's own names for the tensors)
    return ModelSpec(vocab_size=raw["vocab_size"], hidden_size=h, max_position=128, layers=layers, schedule=[ScheduleEntry(0), ScheduleEntry(1)],
                     final_norm=centered, positions={"rope": PartSpec.of("rotary", rotary_dim=32, theta=10000.0, max_position=128)},
                     tie_head=raw["tied"], embedding=PartSpec.of("toy_scaled", scale=raw["embedding_scale"]), head=PartSpec.of("toy_softcap", cap=raw["cap"]))


def plain_ends(tensors, raw, tokens):
    eps, n = raw["eps"], len(tokens)
    cos, sin = rope_tables(32, 10000.0, n)
    table = tensors["embedding.weight"]
    x = table[torch.tensor(tokens)] * raw["embedding_scale"]

    def attend(p, a):
        q = apply_rope((a @ tensors[p + "mixer.q_proj.weight"].T).reshape(n, 3, 32), cos, sin, torch.arange(n))
        k = apply_rope((a @ tensors[p + "mixer.k_proj.weight"].T).reshape(n, 3, 32), cos, sin, torch.arange(n))
        v = (a @ tensors[p + "mixer.v_proj.weight"].T).reshape(n, 3, 32)
        return causal_attention(q, k, v, 1.0 / math.sqrt(32)).reshape(n, 96) @ tensors[p + "mixer.o_proj.weight"].T

    def ff(p, m):
        return gated_mlp(m, tensors[p + "feed_forward.gate_proj.weight"], tensors[p + "feed_forward.up_proj.weight"], tensors[p + "feed_forward.down_proj.weight"])

    a = rms_norm(x, tensors["blocks.0.mixer_norm.weight"], eps)
    x = x + attend("blocks.0.", a) + ff("blocks.0.", a)
    def centered(x, p):
        return torch.nn.functional.layer_norm(x, (x.shape[-1],), tensors[p + "weight"], tensors[p + "bias"], eps)

    x = x + attend("blocks.1.", centered(x, "blocks.1.mixer_norm."))
    x = x + ff("blocks.1.", rms_norm(x, tensors["blocks.1.feed_forward_norm.weight"], eps))
    head = table if raw["tied"] else tensors["head.weight"]
    logits = centered(x, "final_norm.") @ head.T + tensors["head.bias"]
    return raw["cap"] * torch.tanh(logits / raw["cap"])


def _step_through(runner, cache, prompts, plan):
    seqs = {k: cache.new_sequence() for k in prompts}
    done = {k: 0 for k in prompts}
    got = {k: [] for k in prompts}
    for cuts in plan:
        entries = []
        for k, n in cuts.items():
            assert cache.append(seqs[k], done[k], n)
            entries.append(StepEntry(seqs[k], prompts[k][done[k]:done[k] + n], done[k], list(range(n))))
        logits = runner.step(entries).cpu()
        at = 0
        for k, n in cuts.items():
            got[k].append(logits[at:at + n])
            at += n
            done[k] += n
    return {k: torch.cat(v) for k, v in got.items()}


@pytest.mark.parametrize("tied", [True, False])
def test_toy_architecture_with_its_own_embedding_head_and_arrangement(ops, tied):
    register_part("embedding", "toy_scaled", ScaledEmbedding)
    register_part("head", "toy_softcap", SoftcapHead)
    register_arrangement("toy_parallel", ParallelBlock)
    register_part("norm", "toy_centered", CenteredNorm)
    register_architecture("EndsToyForCausalLM", lambda raw: ModelConfig(architecture_name(raw), dict(raw)), ends_spec)
    raw = {"architectures": ["EndsToyForCausalLM"], "hidden_size": 96, "inter": 160, "vocab_size": 77, "eps": 1e-5, "embedding_scale": 9.5, "cap": 0.3, "tied": tied}
    model = build_model(config_from_dict(raw), torch.float32, "cuda")
    assert type(model.embedding) is ScaledEmbedding and type(model.head) is SoftcapHead and type(model.blocks[0]) is ParallelBlock
    assert type(model.final_norm) is CenteredNorm and type(model.blocks[1].mixer_norm) is CenteredNorm and "final_norm.bias" in dict(random_tensors(model, 11))
    bind_random(model, 11, torch.float32, "cuda", storage_dtype=torch.float32)
    tensors = dict(random_tensors(model, 11))
    assert ("head.weight" in tensors) == (not tied) and "blocks.0.feed_forward_norm.weight" not in tensors
    ops.prepare(model, torch.float32)
    cache = CacheManager(model.cache_needs(), 8, 30, 3, torch.float32, "cuda")
    runner = ModelRunner(model, cache, ops, torch.float32, "cuda", 128, 3)
    g = torch.Generator().manual_seed(2)
    prompts = {k: torch.randint(0, 77, (n,), generator=g).tolist() for k, n in (("p", 19), ("q", 8), ("r", 33))}
    got = _step_through(runner, cache, prompts, [{"p": 4, "q": 8}, {"p": 1, "r": 20}, {"p": 14, "r": 1}, {"r": 12}])
    for k, tokens in prompts.items():
        want = plain_ends(tensors, raw, tokens)
        assert float(want.abs().max()) > 0.2  # the cap bites: a head without it would fail
        torch.testing.assert_close(got[k], want, rtol=2e-4, atol=2e-5)


def test_stateful_toy_architecture_through_the_engine_with_preemption(tmp_path, ops):
    """The mixer with state of its own meets the scheduler: admission takes a zeroed slot, preemption gives slot and pages
    back and recomputes from a zeroed slot, decoding goes through the engine's loop with graphs asked for (and not
    captured, because the mixer says it reads the host).  Greedy tokens against the plain implementation."""
    from velox_amd import Engine, EngineConfig, Request, SamplingParams
    from velox_amd.weights import write_random_model

    register_part("mixer", "toy_decaying_sum", DecayingSumMixer)
    register_architecture("ToyForCausalLM", lambda raw: ModelConfig(architecture_name(raw), dict(raw)), toy_spec)
    raw = {"architectures": ["ToyForCausalLM"], "hidden_size": 64, "inter": 96, "vocab_size": 101, "eps": 1e-5, "decay": 0.8}
    folder = write_random_model(raw, str(tmp_path / "toy"), seed=4, dtype="float32")
    from safetensors.torch import load_file

    tensors = load_file(f"{folder}/model.safetensors")
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, 101, (n,), generator=g).tolist() for n in (18, 7, 25, 11)]
    steps = 14

    def plain_greedy(prompt):
        tokens = list(prompt)
        for _ in range(steps):
            tokens.append(int(plain_toy(tensors, raw, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    want = [plain_greedy(p) for p in prompts]
    for pages, expect_preemption in ((64, False), (16, True)):
        engine = Engine.from_pretrained(EngineConfig(model=folder, dtype="float32", device="cuda", max_model_len=64, max_num_seqs=4, max_num_batched_tokens=24,
                                                     max_prefill_chunk_size=6, block_size=4, num_gpu_blocks=pages, enable_cuda_graphs=True, seed=0), ops=ops)
        assert not engine.runner.uses_graphs and engine.cache.prefix is None  # (a state stands for tokens a sharer would skip)
        requests = [Request(f"r{i}", p, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True)) for i, p in enumerate(prompts)]
        engine.generate(requests)
        assert (engine.scheduler.num_preemptions > 0) == expect_preemption
        assert [r.output_token_ids for r in requests] == want
        assert engine.cache.num_used_pages() == 0 and engine.cache.state.num_free == 4


# ----------------------------------------------------------------------------------------------------
# a fourth toy architecture: a mixer that keeps ONE latent vector per token in pages (no keys and values, no heads) and
# attends over the latents themselves, beside an ordinary attention layer.  Its need names its own page tensor; the
# cache manager, the step function and replay learn of it from that need alone.
# ----------------------------------------------------------------------------------------------------
class LatentMixer(Mixer):
    """c_t = W_c x_t is written to the request's pages; y_t = W_o sum_j softmax_j(q_t . c_j / sqrt(r)) c_j over j <= t,
    with q_t = W_q x_t: keys and values are one and the same cached vector of ``rank`` numbers."""

    graph_safe = False  # forward reads the step's lengths on the host

    def __init__(self, prefix: str, hidden_size: int, rank: int) -> None:
        super().__init__(prefix)
        self.hidden_size, self.rank = hidden_size, rank
        self.w_c = self.w_q = self.w_o = None

    def params(self):
        h, r = self.hidden_size, self.rank
        return {"w_c": single("compress.weight", (r, h)), "w_q": single("query.weight", (r, h)), "w_o": single("expand.weight", (h, r))}

    def cache_need(self):
        from velox_amd.parts import PAGE, PagedNeed

        return PagedNeed((("latent", (PAGE, self.rank), torch.float32),))

    def forward(self, x, ctx, cache, owns_cache=True):
        latents = cache.tensors["latent"]  # [pages, page size, rank]
        meta = cache.batch
        c = x.float() @ self.w_c.float().T
        q = x.float() @ self.w_q.float().T
        if owns_cache:
            latents.view(-1, self.rank)[meta.slot_mapping.long()] = c
        out = torch.empty((x.shape[0], self.hidden_size), dtype=torch.float32, device=x.device)
        at = 0
        for b, n in enumerate(ctx.q_lens):
            held = int(meta.kv_lens[b])
            pages = meta.block_tables[b, : (held + cache.block_size - 1) // cache.block_size].long()
            past = latents[pages].reshape(-1, self.rank)[:held]
            scores = q[at:at + n] @ past.T / math.sqrt(self.rank)
            seen = torch.arange(held, device=x.device)[None, :] <= ctx.positions[at:at + n, None]
            weights = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)
            out[at:at + n] = (weights @ past) @ self.w_o.float().T
            at += n
        return out.to(x.dtype)


def latent_spec(config, max_position=None) -> ModelSpec:
    raw = config.raw
    h = raw["hidden_size"]
    norm = PartSpec.of("rmsnorm", hidden_size=h, eps=raw["eps"])
    ff = PartSpec.of("gated_mlp", hidden_size=h, intermediate_size=raw["inter"])
    layers = [
        LayerSpec("layers.0.", PartSpec.of("toy_latent", hidden_size=h, rank=raw["rank"]), ff, norm, norm, **dict(HF_NAMES, mixer_prefix="mixer.")),
        LayerSpec("layers.1.", PartSpec.of("attention", hidden_size=h, num_heads=4, num_kv_heads=2, head_dim=16, qkv_bias=True), ff, norm, norm, position="rope", **HF_NAMES),
        LayerSpec("layers.2.", PartSpec.of("toy_latent", hidden_size=h, rank=raw["rank"]), ff, norm, norm, **dict(HF_NAMES, mixer_prefix="mixer.")),
    ]
    return ModelSpec(vocab_size=raw["vocab_size"], hidden_size=h, max_position=max_position or 256, layers=layers, schedule=[ScheduleEntry(i) for i in range(3)],
                     final_norm=norm, positions={"rope": PartSpec.of("rotary", rotary_dim=16, theta=10000.0, max_position=max_position or 256)}, tie_head=True, **HF_ENDS)


def plain_latent(tensors, raw, tokens):
    eps, n, r = raw["eps"], len(tokens), raw["rank"]
    cos, sin = rope_tables(16, 10000.0, n)
    x = tensors["model.embed_tokens.weight"][torch.tensor(tokens)]
    causal = torch.arange(n)[None, :] <= torch.arange(n)[:, None]
    for layer in range(3):
        p = f"layers.{layer}."
        a = rms_norm(x, tensors[p + "input_layernorm.weight"], eps)
        if layer == 1:
            q = apply_rope((a @ tensors[p + "self_attn.q_proj.weight"].T + tensors[p + "self_attn.q_proj.bias"]).reshape(n, 4, 16), cos, sin, torch.arange(n))
            k = apply_rope((a @ tensors[p + "self_attn.k_proj.weight"].T + tensors[p + "self_attn.k_proj.bias"]).reshape(n, 2, 16), cos, sin, torch.arange(n))
            v = (a @ tensors[p + "self_attn.v_proj.weight"].T + tensors[p + "self_attn.v_proj.bias"]).reshape(n, 2, 16)
            mixed = causal_attention(q, k, v, 0.25).reshape(n, 64) @ tensors[p + "self_attn.o_proj.weight"].T
        else:
            c = a @ tensors[p + "mixer.compress.weight"].T
            scores = (a @ tensors[p + "mixer.query.weight"].T) @ c.T / math.sqrt(r)
            mixed = (torch.softmax(scores.masked_fill(~causal, float("-inf")), dim=-1) @ c) @ tensors[p + "mixer.expand.weight"].T
        x = x + mixed
        x = x + gated_mlp(rms_norm(x, tensors[p + "post_attention_layernorm.weight"], eps), tensors[p + "mlp.gate_proj.weight"],
                          tensors[p + "mlp.up_proj.weight"], tensors[p + "mlp.down_proj.weight"])
    return rms_norm(x, tensors["model.norm.weight"], eps) @ tensors["model.embed_tokens.weight"].T


def test_toy_architecture_with_one_latent_tensor_per_page_stepped_and_replayed(tmp_path, ops):
    """A paged mixer that is no attention: its need names one float32 tensor ``(PAGE, rank)``.  The cache manager gives it
    a pool of its own beside the attention layer's (two groups, two block tables per request), the step function runs
    it in portions and single tokens with pages used again, and the replay program drives the same model from a folder."""
    import numpy as np

    from velox_amd.engine.replay import Replayer
    from velox_amd.weights import write_random_model

    register_part("mixer", "toy_latent", LatentMixer)
    register_architecture("LatentToyForCausalLM", lambda raw: ModelConfig(architecture_name(raw), dict(raw)), latent_spec)
    raw = {"architectures": ["LatentToyForCausalLM"], "hidden_size": 64, "inter": 96, "vocab_size": 83, "eps": 1e-5, "rank": 12}
    model = build_model(config_from_dict(raw), torch.float32, "cuda")
    needs = model.cache_needs()
    assert [n.tensors[0][0] for n in needs] == ["latent", "k", "latent"]
    bind_random(model, 6, torch.float32, "cuda", storage_dtype=torch.float32)
    tensors = dict(random_tensors(model, 6))
    for name in tensors:  # sharper scores, so that a latent read from a wrong page shows
        if name.endswith("query.weight") or name.endswith("compress.weight"):
            tensors[name] = tensors[name] * 12
    for block in (model.blocks[0], model.blocks[2]):
        block.mixer.w_c.mul_(12)
        block.mixer.w_q.mul_(12)
    ops.prepare(model, torch.float32)
    cache = CacheManager(needs, 4, 20, 3, torch.float32, "cuda")
    assert len(cache.groups) == 2 and [g.entries for g in cache.groups] == [[0, 2], [1]]
    assert cache.groups[0].tensors["latent"].shape == (2, 20, 4, 12) and set(cache.groups[1].tensors) == {"k", "v"}
    assert cache.bytes_per_page() == 2 * 4 * 12 * 4 + 2 * 4 * 2 * 16 * 4
    runner = ModelRunner(model, cache, ops, torch.float32, "cuda", 128, 3)
    g = torch.Generator().manual_seed(3)
    prompts = {k: torch.randint(0, 83, (n,), generator=g).tolist() for k, n in (("p", 29), ("q", 12), ("r", 40))}
    # 19 usable pages of 4 tokens for 81 tokens in all: q ends and r takes its pages
    seqs, done, got = {}, {k: 0 for k in prompts}, {k: [] for k in prompts}
    plan = [({"p": 5, "q": 12}, ["q"]), ({"p": 2, "r": 17}, []), ({"p": 22, "r": 1}, ["p"]), ({"r": 2}, []), ({"r": 20}, ["r"])]
    for cuts, ended in plan:
        entries = []
        for k, n in cuts.items():
            if k not in seqs:
                seqs[k] = cache.new_sequence()
            assert cache.append(seqs[k], done[k], n)
            entries.append(StepEntry(seqs[k], prompts[k][done[k]:done[k] + n], done[k], list(range(n))))
        logits = runner.step(entries).cpu()
        at = 0
        for k, n in cuts.items():
            got[k].append(logits[at:at + n])
            at += n
            done[k] += n
        for k in ended:
            cache.free_sequence(seqs.pop(k))
        cache.assert_consistent(list(seqs.values()))
    for k, tokens in prompts.items():
        torch.testing.assert_close(torch.cat(got[k]), plain_latent(tensors, raw, tokens), rtol=2e-4, atol=2e-5)
    assert cache.num_used_pages() == 0

    # the same architecture from a folder through the replay program's class
    folder = write_random_model(raw, str(tmp_path / "latent"), seed=6, dtype="float32")
    from safetensors.torch import load_file

    stored = load_file(f"{folder}/model.safetensors")
    replayer = Replayer(folder, "float32", max_tokens=64, block_size=4, ops=ops)
    tokens = prompts["r"]
    first = replayer.step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:23], "want": [22]}, {"id": "b", "tokens": prompts["q"], "want": [11]}], "end": ["b"]})
    rest = [replayer.step({"step": 1 + i, "entries": [{"id": "a", "tokens": [tokens[23 + i]], "want": [0]}], "end": []}) for i in range(17)]
    want = plain_latent(stored, raw, tokens)
    torch.testing.assert_close(torch.from_numpy(np.concatenate([first[:1]] + rest)), want[22:], rtol=2e-4, atol=2e-5)
    torch.testing.assert_close(torch.from_numpy(first[1:2].copy()), plain_latent(stored, raw, prompts["q"])[-1:], rtol=2e-4, atol=2e-5)
