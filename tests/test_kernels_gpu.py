"""Each HIP kernel alone against its plain PyTorch reference (tests/torch_ops.py), in float32 and
bfloat16, at sizes other than the engine's tiny models: widths and vocabularies that are no power
of two, head sizes 16 .. 256, groups of 1, 3, 7, page sizes 4 .. 64."""
import math

import numpy as np
import pytest
import torch

from torch_ops import TorchOps, exponential_noise

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from velox_amd.kernels import load_ops

    return load_ops("cuda")


@pytest.fixture(scope="module")
def ref():
    return TorchOps()


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-3)


def rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,vocab", [(96, 320), (3584, 1000), (50, 77)])
def test_embed(ops, ref, dtype, hidden, vocab):
    table = rand((vocab, hidden), dtype, 0)
    ids = torch.randint(0, vocab, (37,), generator=torch.Generator().manual_seed(1)).to(torch.int32).cuda()
    torch.testing.assert_close(ops.embed(ids, table), ref.embed(ids, table), rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [64, 96, 3584, 1000])
def test_add_rmsnorm(ops, ref, dtype, hidden):
    tokens = 19
    residual = rand((tokens, hidden), torch.float32, 2)
    delta = rand((tokens, hidden), dtype, 3)
    weight = 1 + rand((hidden,), torch.float32, 4, 0.02)
    r_hip, r_ref = residual.clone(), residual.clone()
    got = ops.add_rmsnorm(r_hip, delta, weight, 1e-5, dtype)
    want = ref.add_rmsnorm(r_ref, delta, weight, 1e-5, dtype)
    torch.testing.assert_close(r_hip, r_ref, rtol=0, atol=0)
    torch.testing.assert_close(got.float(), want.float(), **tol(dtype))
    # no delta: the residual is untouched
    before = r_hip.clone()
    got = ops.add_rmsnorm(r_hip, None, weight, 1e-6, dtype)
    torch.testing.assert_close(r_hip, before, rtol=0, atol=0)
    torch.testing.assert_close(got.float(), ref.add_rmsnorm(r_ref, None, weight, 1e-6, dtype).float(), **tol(dtype))
    # chosen rows: nothing is written
    rows = torch.tensor([18, 0, 7, 7], dtype=torch.int32).cuda()
    got = ops.add_rmsnorm_rows(r_hip, delta, rows, weight, 1e-6, dtype)
    torch.testing.assert_close(r_hip, before, rtol=0, atol=0)
    torch.testing.assert_close(got.float(), ref.add_rmsnorm_rows(r_ref, delta, rows, weight, 1e-6, dtype).float(), **tol(dtype))


def test_rmsnorm_eps_is_inside_the_root(ops):
    # tiny inputs: rsqrt(ms + eps) and 1 / (sqrt(ms) + eps) differ by orders of magnitude
    hidden = 128
    x = torch.full((1, hidden), 1e-4, device="cuda")
    w = torch.ones(hidden, device="cuda")
    got = ops.add_rmsnorm(x.clone(), None, w, 1e-6, torch.float32)
    want = 1e-4 / math.sqrt(1e-8 + 1e-6)
    torch.testing.assert_close(got, torch.full_like(got, want), rtol=1e-5, atol=0)


@pytest.mark.parametrize("a_dtype,w_dtype,out_dtype", [
    (torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16, torch.bfloat16),
    (torch.bfloat16, torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16, torch.float32),
])
@pytest.mark.parametrize("m,n,k", [(1, 320, 96), (7, 263, 80), (65, 130, 150), (130, 64, 224), (3, 70, 37), (16, 1001, 3584), (9, 3584, 18944), (2, 13, 260)])
def test_gemm_fma(ops, ref, a_dtype, w_dtype, out_dtype, m, n, k):
    x = rand((m, k), a_dtype, 5)
    w = rand((n, k), w_dtype, 6, 0.05)
    bias = rand((n,), torch.float32, 7)
    for b in (None, bias):
        got = ops.gemm_fma(x, w, b, out_dtype)
        want = ref.linear(x, w, b, out_dtype)
        if k >= 1024 and out_dtype == torch.float32:
            # sums of thousands of terms round differently in every order of adding: the yardstick is the exact product
            # (float64), and the kernel has to be as close to it as the library's float32 product is, within a factor of two
            exact = x.double() @ w.double().T + (b.double() if b is not None else 0)
            library = (x.float() @ w.float().T + (b if b is not None else 0)).double()
            assert float((got.double() - exact).abs().max()) <= 2 * float((library - exact).abs().max()) + 1e-7
            continue
        torch.testing.assert_close(got.float(), want.float(), **tol(out_dtype))
    if m <= 16 and m > 1:
        # few rows take a kernel of their own: a row's sum depends on that row alone, to the bit, whatever else is in the batch
        alone = ops.gemm_fma(x[m - 1:].contiguous(), w, None, out_dtype)
        assert torch.equal(alone[0], ops.gemm_fma(x, w, None, out_dtype)[m - 1])


@pytest.mark.parametrize("m,n,k", [(1, 320, 96), (8, 152064 // 8, 512), (64, 1000, 3584), (300, 4608, 3584)])
def test_linear_bf16_library_path(ops, ref, m, n, k):
    x = rand((m, k), torch.bfloat16, 8)
    w = rand((n, k), torch.bfloat16, 9, 0.02)
    got = ops.linear(x, w, None, torch.bfloat16)
    want = ref.linear(x, w, None, torch.bfloat16)
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=2e-2)
    got32 = ops.linear(x, w, None, torch.float32)
    torch.testing.assert_close(got32, ref.linear(x, w, None, torch.float32), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [128, 224, 150, 18944])
def test_silu_mul(ops, ref, dtype, inter):
    gate_up = rand((11, 2 * inter), dtype, 10, 2.0)
    torch.testing.assert_close(ops.silu_mul(gate_up).float(), ref.silu_mul(gate_up).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,half,page", [(4, 2, 16, 8, 4), (3, 1, 32, 16, 8), (6, 2, 48, 24, 16), (28, 4, 128, 64, 16), (2, 2, 64, 16, 32), (5, 5, 16, 0, 4)])
def test_rope_kv_write(ops, ref, dtype, nh, nkv, d, half, page):
    tokens, pages = 23, 12
    width = (nh + 2 * nkv) * d
    qkv = rand((tokens, width), dtype, 11)
    bias = rand((width,), torch.float32, 12, 0.1)
    positions = torch.randint(0, 500, (tokens,), generator=torch.Generator().manual_seed(13)).to(torch.int32).cuda()
    slots = (torch.randperm((pages - 1) * page, generator=torch.Generator().manual_seed(14))[:tokens] + page).to(torch.int32).cuda()
    if half:
        angles = torch.outer(torch.arange(512, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float32) / half)))
        cos, sin = angles.cos().cuda(), angles.sin().cuda()
    else:
        cos = sin = None
    for use_bias in (bias, None):
        caches = []
        for impl in (ops, ref):
            k_cache = torch.zeros((pages, nkv, page, d), dtype=dtype, device="cuda")
            v_cache = torch.zeros((pages, nkv, d, page), dtype=dtype, device="cuda")
            buf = qkv.clone()
            impl.rope_kv_write(buf, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, write_kv=True, bias=use_bias)
            caches.append((buf[:, : nh * d].float(), k_cache.float(), v_cache.float()))
        for got, want in zip(*caches):
            torch.testing.assert_close(got, want, **tol(dtype))
    # write_kv=False leaves the cache alone
    k_cache = torch.zeros((pages, nkv, page, d), dtype=dtype, device="cuda")
    v_cache = torch.zeros((pages, nkv, d, page), dtype=dtype, device="cuda")
    ops.rope_kv_write(qkv.clone(), nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, write_kv=False, bias=bias)
    assert not k_cache.any() and not v_cache.any()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(28, 4, 128, 16), (4, 2, 16, 8), (3, 1, 32, 32), (6, 2, 48, 4)])
def test_rope_kv_write_for_consecutive_tokens_of_prompts(ops, ref, dtype, nh, nkv, d, page):
    """Prompt portions: consecutive tokens in consecutive slots (runs of eight are written as whole vectors), starting
    anywhere in a page, pages in any order, a single decoded token between two portions."""
    half = d // 2
    width = (nh + 2 * nkv) * d
    pages = 40
    order = (torch.randperm(pages - 1, generator=torch.Generator().manual_seed(15)) + 1).tolist()
    slots, positions = [], []
    for start, count in ((5, 37), (0, 1), (16, 70), (3, 9)):  # (first position, tokens) of each sequence's portion
        table = [order.pop() for _ in range((start + count + page - 1) // page)]
        for p in range(start, start + count):
            slots.append(table[p // page] * page + p % page)
            positions.append(p)
    tokens = len(slots)
    qkv = rand((tokens, width), dtype, 16)
    bias = rand((width,), torch.float32, 17, 0.1)
    slots = torch.tensor(slots, dtype=torch.int32).cuda()
    positions = torch.tensor(positions, dtype=torch.int32).cuda()
    angles = torch.outer(torch.arange(512, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float32) / half)))
    cos, sin = angles.cos().cuda(), angles.sin().cuda()
    results = []
    for impl in (ops, ref):
        k_cache = torch.full((pages, nkv, page, d), 3.0, dtype=dtype, device="cuda")
        v_cache = torch.full((pages, nkv, d, page), 3.0, dtype=dtype, device="cuda")
        buf = qkv.clone()
        impl.rope_kv_write(buf, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, write_kv=True, bias=bias)
        results.append((buf[:, : nh * d].float(), k_cache.float(), v_cache.float()))
    for got, want in zip(*results):
        torch.testing.assert_close(got, want, **tol(dtype))


@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("nh,nkv,d,k,page", [(4, 2, 64, 128, 4), (28, 4, 128, 3584, 16), (3, 1, 32, 192, 1), (2, 2, 96, 64, 8), (5, 5, 160, 320, 32)])
def test_qkv_projection_with_rotation_and_cache_write_in_one_kernel(ops, ref, m, nh, nkv, d, k, page):
    """The fused decode kernel against product -> bias -> rotation -> cache write done one after the other in float32,
    and against the unfused kernels; untouched cache entries stay untouched."""
    pages = 24
    width = (nh + 2 * nkv) * d
    half = d // 2
    x = rand((m, k), torch.bfloat16, 70)
    w = rand((width, k), torch.bfloat16, 71, 0.05)
    bias = rand((width,), torch.float32, 72, 0.3)
    positions = torch.randint(0, 500, (m,), generator=torch.Generator().manual_seed(73)).to(torch.int32).cuda()
    slots = (torch.randperm((pages - 1) * page, generator=torch.Generator().manual_seed(74))[:m] + page).to(torch.int32).cuda()
    angles = torch.outer(torch.arange(512, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float32) / half)))
    cos, sin = angles.cos().cuda(), angles.sin().cuda()
    pw = ops.prepare_weight(w, rotary_heads=(nh, nkv, d))
    assert pw.copy("rotary") is not None
    for use_bias in (bias, None):
        # float32 reference: exact product of the bfloat16 operands, then everything in float32
        k32 = torch.full((pages, nkv, page, d), 7.0, dtype=torch.float32, device="cuda")
        v32 = torch.full((pages, nkv, d, page), 7.0, dtype=torch.float32, device="cuda")
        wide = ref.linear(x, w, None, torch.float32)
        ref.rope_kv_write(wide, nh, nkv, d, positions, cos, sin, slots, k32, v32, page, write_kv=True, bias=use_bias)
        results = {}
        for fused in (True, False):
            k_cache = torch.full((pages, nkv, page, d), 7.0, dtype=torch.bfloat16, device="cuda")
            v_cache = torch.full((pages, nkv, d, page), 7.0, dtype=torch.bfloat16, device="cuda")
            for waves in ((8, 16) if fused else (None,)):
                q = ops.qkv_rope_write(x, pw, use_bias, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, waves=waves, fused=fused)
                results[(fused, waves)] = (q[:, : nh * d].float(), k_cache.float(), v_cache.float())
        scale = float(wide.abs().max())
        for key, (q, kc, vc) in results.items():
            fused = key[0]
            # the unfused route rounds the product to bfloat16 before the rotation: one more rounding
            bound = dict(rtol=1e-2, atol=(1e-2 if fused else 2e-2) * scale)
            torch.testing.assert_close(q, wide[:, : nh * d], msg=lambda t: f"{key} q: {t}", **bound)
            torch.testing.assert_close(kc, k32, msg=lambda t: f"{key} k: {t}", **bound)
            torch.testing.assert_close(vc, v32, msg=lambda t: f"{key} v: {t}", **bound)
        torch.testing.assert_close(results[(True, 8)][0], results[(False, None)][0], rtol=2e-2, atol=2e-2 * scale)
    # a layer that reads another layer's cache writes nothing: not a case for the fused kernel
    with pytest.raises(Exception):
        ops.qkv_rope_write(x, pw, bias, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, write_kv=False, fused=True)
    before = k_cache.clone()
    ops.qkv_rope_write(x, pw, bias, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, write_kv=False)
    assert torch.equal(before, k_cache)


@pytest.mark.parametrize("m", [17, 40, 64])
@pytest.mark.parametrize("nh,nkv,d,k,page,rotate", [(4, 2, 64, 128, 4, True), (28, 4, 128, 3584, 16, True), (3, 1, 32, 192, 1, True), (2, 2, 96, 1024, 8, False),
                                                    (5, 5, 48, 320, 32, True)])
def test_qkv_projection_at_17_to_64_rows_with_partial_sums_added_by_the_rotation(ops, ref, m, nh, nkv, d, k, page, rotate):
    """Split-K partial sums -> (sum, bias, rotation, cache write) in one kernel, against the same steps in float32; slots
    in runs of consecutive tokens (a prompt's portion) and scattered (decoding requests)."""
    pages = 80
    width = (nh + 2 * nkv) * d
    half = d // 2
    x = rand((m, k), torch.bfloat16, 90)
    w = rand((width, k), torch.bfloat16, 91, 0.05)
    bias = rand((width,), torch.float32, 92, 0.3)
    positions = torch.randint(0, 500, (m,), generator=torch.Generator().manual_seed(93)).to(torch.int32).cuda()
    scattered = torch.randperm((pages - 1) * page, generator=torch.Generator().manual_seed(94))[:m] + page
    consecutive = torch.arange(m) + page + 3
    angles = torch.outer(torch.arange(512, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float32) / half)))
    cos, sin = (angles.cos().cuda(), angles.sin().cuda()) if rotate else (None, None)
    pw = ops.prepare_weight(w, rotary_heads=(nh, nkv, d))
    scale = float(ref.linear(x, w, None, torch.float32).abs().max())
    for slots in (scattered, consecutive):
        slots = slots.to(torch.int32).cuda()
        for use_bias in (bias, None):
            k32 = torch.full((pages, nkv, page, d), 7.0, dtype=torch.float32, device="cuda")
            v32 = torch.full((pages, nkv, d, page), 7.0, dtype=torch.float32, device="cuda")
            wide = ref.linear(x, w, None, torch.float32)
            ref.rope_kv_write(wide, nh, nkv, d, positions, cos, sin, slots, k32, v32, page, write_kv=True, bias=use_bias)
            k_cache = torch.full((pages, nkv, page, d), 7.0, dtype=torch.bfloat16, device="cuda")
            v_cache = torch.full((pages, nkv, d, page), 7.0, dtype=torch.bfloat16, device="cuda")
            for splits in (None, 1, 3):
                partial = ops.skinny_gemm_splitk(x, w, splits=splits, packed=pw.copy(1))
                q = ops.rope_kv_write_partial(partial, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, bias=use_bias)
                bound = dict(rtol=1e-2, atol=1e-2 * scale)
                torch.testing.assert_close(q[:, : nh * d].float(), wide[:, : nh * d], **bound)
                torch.testing.assert_close(k_cache.float(), k32, **bound)
                torch.testing.assert_close(v_cache.float(), v32, **bound)
            # the route the engine takes for this many rows is this one
            k2, v2 = torch.full_like(k_cache, 7.0), torch.full_like(v_cache, 7.0)
            q2 = ops.qkv_rope_write(x, pw, use_bias, nh, nkv, d, positions, cos, sin, slots, k2, v2, page)
            torch.testing.assert_close(q2[:, : nh * d].float(), wide[:, : nh * d], rtol=1e-2, atol=1e-2 * scale)
            torch.testing.assert_close(k2.float(), k32, rtol=1e-2, atol=1e-2 * scale)
    # a layer that reads another layer's cache writes nothing
    before = k_cache.clone()
    ops.qkv_rope_write(x, pw, bias, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, write_kv=False)
    assert torch.equal(before, k_cache)


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("hidden,inner", [(64, 128), (3584, 3584), (200, 320), (96, 18944), (5120, 192), (8192, 64)])
def test_residual_add_and_norm_split_between_two_products(ops, ref, m, hidden, inner):
    """The decode fusion: a product adds itself to the residual and applies the norm weight (DeferredNorm); the next
    product (plain, gate/up + SiLU, or q/k/v with rotation) scales its rows.  Against residual add -> RMSNorm -> product
    done one after the other."""
    from velox_amd.parts.base import DeferredNorm, ResidualSink
    from velox_amd.parts.norms import RMSNorm

    x = rand((m, inner), torch.bfloat16, 80)
    w_out = rand((hidden, inner), torch.bfloat16, 81, 0.05)
    residual0 = rand((m, hidden), torch.float32, 82, 2.0)
    norm = RMSNorm("", hidden, 1e-5)
    norm.weight = (1.0 + rand((hidden,), torch.float32, 83, 0.1))
    p_out = ops.prepare_weight(w_out)
    if hidden % 64 != 0:
        # the next product cannot stream this width: it gets the materialised rows
        pass
    # reference: product in float32 from the bfloat16 operands, add, norm
    delta = ref.linear(x, w_out, None, torch.float32)
    want_residual = residual0 + delta
    want_normed = ref.add_rmsnorm(residual0.clone(), delta, norm.weight, norm.eps, torch.float32)
    residual = residual0.clone()
    deferred = ops.linear(x, p_out, None, torch.bfloat16, partials_ok=True, residual_norm=ResidualSink(residual, norm))
    assert isinstance(deferred, DeferredNorm) and deferred.norm is norm
    torch.testing.assert_close(residual, want_residual, rtol=1e-5, atol=1e-4 * float(want_residual.abs().max()))
    torch.testing.assert_close(ops.materialize(deferred).float(), want_normed, rtol=2e-2, atol=2e-2)
    assert norm.forward(residual, deferred, None) is deferred
    for row_tiles in (1, 2, 0):  # tiles of the weight per workgroup (0: half a tile): the same sums in the same order
        again = residual0.clone()
        other = ops._linear_into_residual(x, p_out, ResidualSink(again, norm), row_tiles=row_tiles)
        assert torch.equal(again, residual) and torch.equal(other.x, deferred.x)
        blocks = (hidden + 15) // 16
        assert other.sums.shape[1] == (2 * blocks if row_tiles == 0 else blocks)
        torch.testing.assert_close(other.sums[:m].sum(1), deferred.sums[:m].sum(1), rtol=1e-5, atol=0)
        torch.testing.assert_close(ops.materialize(other).float(), ops.materialize(deferred).float(), rtol=1e-2, atol=1e-2)
    with pytest.raises(ValueError):
        RMSNorm("", hidden, 1e-5).forward(residual, deferred, None)
    if hidden % 64 != 0:
        return
    # consumers
    normed_bf16 = want_normed.to(torch.bfloat16)
    w_next = rand((320, hidden), torch.bfloat16, 84, 0.05)
    bias = rand((320,), torch.float32, 85)
    scale = float(ref.linear(normed_bf16, w_next, None, torch.float32).abs().max())
    tol = dict(rtol=2e-2, atol=2e-2 * scale)
    torch.testing.assert_close(ops.linear(deferred, w_next, bias, torch.float32), ref.linear(normed_bf16, w_next, bias, torch.float32), **tol)  # unregistered: materialised
    p_next = ops.prepare_weight(w_next)
    torch.testing.assert_close(ops.linear(deferred, p_next, bias, torch.float32), ref.linear(normed_bf16, w_next, bias, torch.float32), **tol)
    # 64 rows of the weight per wave (the variant for very tall weights), four and eight waves
    for waves in (4, 8):
        if hidden // 16 <= 64 * waves:
            got = ops.skinny_gemm(deferred.x, w_next, bias, torch.float32, waves=waves, row_tiles=4, packed=p_next.copy(1), row_scale=deferred)
            torch.testing.assert_close(got, ref.linear(normed_bf16, w_next, bias, torch.float32), **tol)
    p_next = ops.prepare_weight(w_next, stacked=2, handle=p_next)
    want_glu = ref.linear_silu_mul(normed_bf16, w_next, torch.bfloat16).float()
    torch.testing.assert_close(ops.linear_silu_mul(deferred, p_next, torch.bfloat16).float(), want_glu, rtol=3e-2, atol=3e-2 * float(want_glu.abs().max()))
    # q/k/v with rotation: 2 heads, 1 kv head, head size 80 -> 320 rows
    nh, nkv, d, page, pages = 2, 1, 80, 8, 12
    p_next = ops.prepare_weight(w_next, rotary_heads=(nh, nkv, d), handle=p_next)
    positions = torch.randint(0, 300, (m,), generator=torch.Generator().manual_seed(86)).to(torch.int32).cuda()
    slots = (torch.randperm((pages - 1) * page, generator=torch.Generator().manual_seed(87))[:m] + page).to(torch.int32).cuda()
    angles = torch.outer(torch.arange(512, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(d // 2, dtype=torch.float32) / (d // 2))))
    cos, sin = angles.cos().cuda(), angles.sin().cuda()
    outs = []
    for source in (deferred, normed_bf16):
        k_cache = torch.zeros((pages, nkv, page, d), dtype=torch.bfloat16, device="cuda")
        v_cache = torch.zeros((pages, nkv, d, page), dtype=torch.bfloat16, device="cuda")
        q = ops.qkv_rope_write(source, p_next, bias, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page)
        outs.append((q[:, : nh * d].float(), k_cache.float(), v_cache.float()))
    for got, want in zip(*outs):
        torch.testing.assert_close(got, want, rtol=3e-2, atol=3e-2 * max(1.0, float(want.abs().max())))


def _rows_from_lanes_order(twin, k):
    """[k / 64 * 1024] in the order the skinny kernels' lanes read activations -> [16, k]."""
    return twin.view(k // 64, 2, 4, 16, 8).permute(3, 0, 2, 1, 4).reshape(16, k)


@pytest.mark.parametrize("m", [1, 5, 13, 16])
def test_decode_activations_handed_on_in_the_lanes_order(ops, ref, m, monkeypatch):
    """The gate/up kernel and the residual-add kernel leave their result a second time in the order the next product's
    lanes read it; a product gives the same bits whether it reads that copy or the row-major one."""
    from velox_amd.parts.base import DeferredNorm, ResidualSink
    from velox_amd.parts.norms import RMSNorm

    # (the engine asks for the copy from 13 rows on, where it pays; the kernels take any number up to 16)
    monkeypatch.setattr(ops, "_room_for_packed_rows", lambda rows, n: torch.empty(n // 64 * 1024, dtype=torch.bfloat16, device="cuda") if rows <= 16 and n % 64 == 0 else None)
    hidden, inner = 256, 448
    x = rand((m, hidden), torch.bfloat16, 90)
    w_gu = rand((2 * inner, hidden), torch.bfloat16, 91, 0.05)
    w_down = rand((hidden, inner), torch.bfloat16, 92, 0.05)
    p_gu = ops.prepare_weight(w_gu, stacked=2)
    p_down = ops.prepare_weight(w_down)
    act = ops.linear_silu_mul(x, p_gu, torch.bfloat16)
    twin, version = act._velox_packed_rows
    assert version == act._version and torch.equal(_rows_from_lanes_order(twin, inner)[:m], act)
    norm = RMSNorm("", hidden, 1e-6)
    norm.weight = 1.0 + rand((hidden,), torch.float32, 93, 0.1)
    results = []
    for use_twin in (True, False):
        source = act if use_twin else act.clone()  # (a clone is another tensor object: no copy hangs on it)
        assert (ops._packed_rows_of(source, inner) is not None) == use_twin
        residual = rand((m, hidden), torch.float32, 94)
        deferred = ops.linear(source, p_down, None, torch.bfloat16, partials_ok=True, residual_norm=ResidualSink(residual, norm))
        assert isinstance(deferred, DeferredNorm)
        next_twin = ops._packed_rows_of(deferred.x, hidden)
        assert torch.equal(_rows_from_lanes_order(next_twin, hidden)[:m], deferred.x)
        results.append((residual, deferred.x.clone(), deferred.sums[:m].clone(), deferred))
    for a, b in zip(results[0][:3], results[1][:3]):
        assert torch.equal(a, b)
    # the consumers of a DeferredNorm, with and without its copy
    deferred = results[0][3]
    plain = DeferredNorm(deferred.x.clone(), deferred.sums, deferred.width, deferred.eps, deferred.norm)
    bias = rand((2 * inner,), torch.float32, 95)
    assert torch.equal(ops.linear(deferred, p_gu, bias, torch.float32), ops.linear(plain, p_gu, bias, torch.float32))
    assert torch.equal(ops.linear_silu_mul(deferred, p_gu, torch.bfloat16), ops.linear_silu_mul(plain, p_gu, torch.bfloat16))
    nh, nkv, d, page, pages = 3, 2, 128, 16, 6  # (3 + 2 * 2) * 128 = 896 = 2 * inner rows
    p_gu = ops.prepare_weight(w_gu, rotary_heads=(nh, nkv, d), handle=p_gu)
    positions = torch.arange(m, dtype=torch.int32, device="cuda") * 7
    slots = (torch.randperm((pages - 1) * page, generator=torch.Generator().manual_seed(96))[:m] + page).to(torch.int32).cuda()
    angles = torch.outer(torch.arange(128, dtype=torch.float32), 1.0 / (10000.0 ** (torch.arange(d // 2, dtype=torch.float32) / (d // 2))))
    cos, sin = angles.cos().cuda(), angles.sin().cuda()
    outs = []
    for source in (deferred, plain):
        k_cache = torch.zeros((pages, nkv, page, d), dtype=torch.bfloat16, device="cuda")
        v_cache = torch.zeros((pages, nkv, d, page), dtype=torch.bfloat16, device="cuda")
        q = ops.qkv_rope_write(source, p_gu, bias, nh, nkv, d, positions, cos, sin, slots, k_cache, v_cache, page, fused=True)
        outs.append((q, k_cache, v_cache))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # a copy goes stale with its tensor
    act.add_(1)
    assert ops._packed_rows_of(act, inner) is None


def _attention_case(dtype, nh, nkv, d, page, seqs, seed, garbage=False):
    """seqs: list of (q_len, kv_len).  Builds a paged cache with shuffled pages and a flat qkv."""
    g = torch.Generator().manual_seed(seed)
    total_pages = sum((kv + page - 1) // page for _, kv in seqs) + 3
    perm = (torch.randperm(total_pages - 1, generator=g) + 1).tolist()
    k_cache = torch.zeros((total_pages, nkv, page, d), dtype=dtype)
    v_cache = torch.zeros((total_pages, nkv, d, page), dtype=dtype)
    if garbage:
        k_cache.normal_(0, 50.0, generator=g)
        v_cache.normal_(0, 50.0, generator=g)
    width = max((kv + page - 1) // page for _, kv in seqs)
    tables = torch.zeros((len(seqs), width), dtype=torch.int32)
    tokens = sum(q for q, _ in seqs)
    qkv = (torch.randn((tokens, (nh + 2 * nkv) * d), generator=g)).to(dtype)
    cu = [0]
    for b, (q_len, kv_len) in enumerate(seqs):
        n_pages = (kv_len + page - 1) // page
        mine = [perm.pop() for _ in range(n_pages)]
        tables[b, :n_pages] = torch.tensor(mine, dtype=torch.int32)
        keys = torch.randn((kv_len, nkv, d), generator=g).to(dtype)
        values = torch.randn((kv_len, nkv, d), generator=g).to(dtype)
        for n in range(kv_len):
            k_cache[mine[n // page], :, n % page, :] = keys[n]
            v_cache[mine[n // page], :, :, n % page] = values[n]
        cu.append(cu[-1] + q_len)
    return dict(
        qkv=qkv.cuda(), k_cache=k_cache.cuda(), v_cache=v_cache.cuda(), tables=tables.cuda(),
        cu=torch.tensor(cu, dtype=torch.int32).cuda(), kv=torch.tensor([kv for _, kv in seqs], dtype=torch.int32).cuda(),
        max_q=max(q for q, _ in seqs), max_kv=max(kv for _, kv in seqs),
    )


def _run_attention(impl, case, nh, nkv, d, page, window=None, splits=None, all_decode=False, workspace=None):
    return impl.paged_attention(
        case["qkv"], nh, nkv, d, case["k_cache"], case["v_cache"], page, case["tables"], case["cu"], case["kv"],
        case["max_q"], case["max_kv"], 1.0 / math.sqrt(d), window, all_decode, workspace, splits=splits,
    ).float()


ATTN_SHAPES = [(4, 2, 16, 4), (3, 1, 32, 8), (6, 2, 48, 16), (28, 4, 128, 16), (8, 8, 64, 64), (7, 1, 96, 32), (2, 1, 256, 16), (40, 8, 128, 2), (5, 1, 80, 8),
               (6, 2, 192, 16)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", ATTN_SHAPES)
def test_paged_attention_mixed_batch(ops, ref, dtype, nh, nkv, d, page):
    # whole prompts, a portion with earlier context, single decoded tokens, a two-token portion
    seqs = [(70, 70), (33, 141), (1, 97), (2, 66), (1, 1), (130, 130)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=d + nh)
    got = _run_attention(ops, case, nh, nkv, d, page)
    want = _run_attention(ref, case, nh, nkv, d, page)
    torch.testing.assert_close(got, want, **(dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", ATTN_SHAPES)
@pytest.mark.parametrize("window", [None, 200])
def test_paged_attention_decoded_tokens_before_portions(ops, ref, dtype, nh, nkv, d, page, window):
    """A mixed step as the engine lays it out: single decoded tokens first (one of them behind a long context), then
    portions of prompts.  Told how many sequences lead with one token, the wrapper sends those through the streaming
    kernel with split keys and the rest through the general kernel; every row agrees with the plain reference, and
    the decoded rows with the same rows in a step of their own, to the bit."""
    from velox_amd.engine.batch import Workspace

    seqs = [(1, 2300), (1, 97), (1, 1), (1, 640), (33, 141), (2, 66), (70, 70), (1, 30)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=d + nh + 2)
    workspace = Workspace(torch.device("cuda"))
    tolerance = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    want = _run_attention(ref, case, nh, nkv, d, page, window=window)
    one_launch = _run_attention(ops, case, nh, nkv, d, page, window=window, workspace=workspace)
    got = ops.paged_attention(case["qkv"], nh, nkv, d, case["k_cache"], case["v_cache"], page, case["tables"], case["cu"], case["kv"],
                              case["max_q"], case["max_kv"], 1.0 / math.sqrt(d), window, False, workspace, decode_prefix=4).float()
    torch.testing.assert_close(got, want, **tolerance)
    torch.testing.assert_close(one_launch, want, **tolerance)
    assert torch.equal(got[4:], one_launch[4:])  # the general kernel's rows do not depend on who else is in the launch
    alone = dict(case)
    alone["qkv"], alone["tables"], alone["kv"] = case["qkv"][:4].contiguous(), case["tables"][:4].contiguous(), case["kv"][:4].contiguous()
    alone["cu"] = torch.arange(5, dtype=torch.int32, device="cuda")
    alone["max_q"] = 1
    decoded = _run_attention(ops, alone, nh, nkv, d, page, window=window, all_decode=True, workspace=workspace)
    assert torch.equal(got[:4], decoded)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(28, 4, 128, 16), (4, 2, 16, 4), (2, 1, 256, 16), (12, 2, 128, 32)])
def test_paged_attention_portions_behind_many_keys_split_them(ops, ref, dtype, nh, nkv, d, page):
    """Few prompt tokens behind thousands of keys: the wrapper splits the keys over workgroups (and merges), alone and
    behind decoded tokens that lead the step (whose rows the second launch's merge must leave alone)."""
    from velox_amd.engine.batch import Workspace

    seqs = [(1, 4500), (1, 10), (150, 4400), (40, 40), (2, 4200)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=d + nh + 3)
    workspace = Workspace(torch.device("cuda"))
    tolerance = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    assert ops.choose_portion_splits(192, nh // nkv, nkv, 4500) > 1
    want = _run_attention(ref, case, nh, nkv, d, page)
    for prefix in (0, 2):
        got = ops.paged_attention(case["qkv"], nh, nkv, d, case["k_cache"], case["v_cache"], page, case["tables"], case["cu"], case["kv"],
                                  case["max_q"], case["max_kv"], 1.0 / math.sqrt(d), None, False, workspace, decode_prefix=prefix).float()
        torch.testing.assert_close(got, want, **tolerance)
    one_pass = _run_attention(ops, case, nh, nkv, d, page, splits=1, workspace=workspace)
    torch.testing.assert_close(one_pass, want, **tolerance)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(28, 4, 128, 16), (32, 16, 64, 64), (16, 8, 32, 8), (24, 12, 48, 4)])
@pytest.mark.parametrize("window", [None, 300])
def test_paged_attention_long_portions(ops, ref, dtype, nh, nkv, d, page, window):
    """Steps with thousands of rows take the 128-row workgroups in bfloat16: long whole prompts, a long portion behind
    a longer context, and short entries beside them.  A row's result is the same as in a small step, to rounding (the
    large workgroups add a row's keys in another order) and to the bit in float32, which has one kind of workgroup."""
    seqs = [(1100, 1100), (700, 1300), (1, 97), (300, 300), (2, 40)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=d + nh + 1)
    got = _run_attention(ops, case, nh, nkv, d, page, window=window)
    want = _run_attention(ref, case, nh, nkv, d, page, window=window)
    torch.testing.assert_close(got, want, **(dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))
    # the 300-token prompt again, in a step of its own (64-row workgroups): its rows must not have changed
    first = sum(q for q, _ in seqs[:3])
    alone = dict(case)
    alone["qkv"] = case["qkv"][first:first + 300].contiguous()
    alone["tables"] = case["tables"][3:4].contiguous()
    alone["cu"] = torch.tensor([0, 300], dtype=torch.int32, device="cuda")
    alone["kv"] = case["kv"][3:4].contiguous()
    alone["max_q"], alone["max_kv"] = 300, 300
    same = dict(rtol=0, atol=0) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(_run_attention(ops, alone, nh, nkv, d, page, window=window), got[first:first + 300], **same)


@pytest.mark.parametrize("dtype,nh,nkv,d,page,long_context,choices", [
    (torch.bfloat16, 14, 2, 128, 8, 17000, (1, 2, 3)), (torch.bfloat16, 6, 3, 64, 8, 16500, (2, 3)), (torch.float32, 4, 2, 32, 4, 9000, (0,))])
@pytest.mark.parametrize("window", [None, 5000])
def test_paged_attention_behind_more_pages_than_the_kernels_keep_ids_of(ops, ref, dtype, nh, nkv, d, page, long_context, choices, window):
    """A workgroup keeps the page ids of the keys it visits in LDS, 2,048 at a time, and fetches the next lot when its
    tiles leave the window: portions behind contexts of more than 2,048 pages in one pass over the keys (no split), in
    every kernel for portions, with a short sequence and a single token behind the long context beside them."""
    from velox_amd.engine.batch import Workspace

    assert long_context // page > 2048
    seqs = [(200, long_context), (64, 64), (1, long_context - 300)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=d + nh + 5)
    want = _run_attention(ref, case, nh, nkv, d, page, window=window)
    tolerance = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    lib = ops.attention_library(d)
    workspace = Workspace(torch.device("cuda"))
    try:
        for choice in choices:
            lib.velox_attention_portion_kernel(choice)
            got = _run_attention(ops, case, nh, nkv, d, page, window=window, splits=1, workspace=workspace)
            torch.testing.assert_close(got, want, **tolerance)
    finally:
        lib.velox_attention_portion_kernel(0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(28, 4, 128, 16), (4, 2, 16, 4), (6, 2, 96, 8), (8, 8, 64, 1)])
@pytest.mark.parametrize("window", [None, 200])
def test_paged_attention_few_rows_many_keys(ops, ref, dtype, nh, nkv, d, page, window):
    """Short portions behind long contexts: few workgroups, each with many key tiles (in bfloat16 two sets of waves
    then share a workgroup's tiles, an odd number of tiles included)."""
    seqs = [(40, 900), (3, 705), (1, 520), (17, 64 * 9 + 17)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=d + nh + 2)
    got = _run_attention(ops, case, nh, nkv, d, page, window=window)
    want = _run_attention(ref, case, nh, nkv, d, page, window=window)
    torch.testing.assert_close(got, want, **(dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 4), (28, 4, 128, 16), (3, 1, 32, 8)])
def test_paged_attention_garbage_in_unused_slots_and_null_page(ops, ref, dtype, nh, nkv, d, page):
    seqs = [(5, 37), (1, 64), (9, 9)]
    clean = _attention_case(dtype, nh, nkv, d, page, seqs, seed=3)
    dirty = _attention_case(dtype, nh, nkv, d, page, seqs, seed=3, garbage=True)
    # same seed: same real keys, values and queries? the garbage draw shifts the stream, so copy them over
    dirty["qkv"] = clean["qkv"]
    tables = clean["tables"].cpu()
    for b, (_, kv_len) in enumerate(seqs):
        for n in range(kv_len):
            p, o = int(tables[b, n // page]), n % page
            dirty["k_cache"][p, :, o, :] = clean["k_cache"][p, :, o, :]
            dirty["v_cache"][p, :, :, o] = clean["v_cache"][p, :, :, o]
    dirty["tables"] = clean["tables"]
    got_clean = _run_attention(ops, clean, nh, nkv, d, page)
    got_dirty = _run_attention(ops, dirty, nh, nkv, d, page)
    torch.testing.assert_close(got_dirty, got_clean, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 4), (28, 4, 128, 16), (7, 1, 96, 32)])
@pytest.mark.parametrize("window", [1, 5, 64, 100])
def test_paged_attention_window(ops, ref, dtype, nh, nkv, d, page, window):
    seqs = [(70, 70), (33, 141), (1, 197), (2, 66)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=11)
    got = _run_attention(ops, case, nh, nkv, d, page, window=window)
    want = _run_attention(ref, case, nh, nkv, d, page, window=window)
    torch.testing.assert_close(got, want, **(dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))


@pytest.mark.parametrize("nh,nkv,d,page", [(28, 4, 128, 16), (12, 2, 128, 8), (8, 8, 64, 64), (6, 3, 64, 16), (5, 1, 128, 32)])
@pytest.mark.parametrize("window", [None, 300])
def test_paged_attention_with_tiles_loaded_straight_into_lds(ops, ref, nh, nkv, d, page, window):
    """The kernel for portions of prompts whose tiles of keys and values reach LDS by direct loads (bfloat16, head sizes 64
    and 128, pages of 8 tokens and more), made to run wherever it can, beside the kernel it stands in for: whole prompts
    whose lengths are no multiple of a tile or of a piece of eight keys, portions behind longer contexts, short
    entries beside them, pages in no order, and loud garbage in every slot beyond the sequences' ends (values there must
    not reach the output, not even multiplied with a probability of zero) and on the null page."""
    from velox_amd.engine.batch import Workspace

    lib = ops.attention_library(d)
    seqs = [(1100, 1100), (700, 1301), (1, 97), (300, 300), (2, 40), (67, 67), (130, 1003)]
    case = _attention_case(torch.bfloat16, nh, nkv, d, page, seqs, seed=d + nh + 7)
    dirty = _attention_case(torch.bfloat16, nh, nkv, d, page, seqs, seed=d + nh + 7, garbage=True)
    dirty["qkv"], dirty["tables"] = case["qkv"], case["tables"]
    tables = case["tables"].cpu()
    used = torch.zeros(dirty["k_cache"].shape[0], page, dtype=torch.bool)
    for b, (_, kv_len) in enumerate(seqs):
        for n in range(kv_len):
            used[int(tables[b, n // page]), n % page] = True
    keep = used.cuda()
    dirty["k_cache"] = torch.where(keep[:, None, :, None], case["k_cache"], dirty["k_cache"] * float("inf"))  # +-inf where no key lives
    dirty["v_cache"] = torch.where(keep[:, None, None, :], case["v_cache"], dirty["v_cache"] * float("inf"))
    tolerance = dict(rtol=2e-2, atol=2e-2)
    want = _run_attention(ref, case, nh, nkv, d, page, window=window)
    try:
        results = {}
        for choice in (1, 2, 3):  # (the kernels it stands in for; direct loads; direct loads with two sets of waves)
            lib.velox_attention_portion_kernel(choice)
            results[choice] = _run_attention(ops, case, nh, nkv, d, page, window=window)
            torch.testing.assert_close(results[choice], want, **tolerance)
            assert torch.equal(_run_attention(ops, dirty, nh, nkv, d, page, window=window), results[choice])
        # three kernels did run (they add a row's keys in different orders)
        assert not torch.equal(results[1], results[2]) and not torch.equal(results[2], results[3])
        # split keys (few tokens behind many keys) through the same kernels, and the partial results merged
        far = _attention_case(torch.bfloat16, nh, nkv, d, page, [(150, 4400), (90, 90), (2, 4200)], seed=d + nh + 8)
        workspace = Workspace(torch.device("cuda"))
        for choice in (2, 3):
            lib.velox_attention_portion_kernel(choice)
            for splits in (1, 3, 4):
                got = _run_attention(ops, far, nh, nkv, d, page, window=window, splits=splits, workspace=workspace)
                torch.testing.assert_close(got, _run_attention(ref, far, nh, nkv, d, page, window=window), **tolerance)
        # Scores that climb along the sequence, slowly (a row's best score moves up a little with every tile, so the
        # reference of its exponents lags behind and catches up every few tiles) and in jumps (far above everything seen):
        # the kernels with direct loads keep a reference that need not be the maximum
        climbing = _attention_case(torch.bfloat16, nh, nkv, d, page, [(900, 900), (400, 1100)], seed=d + nh + 9)
        direction = torch.randn(d, generator=torch.Generator().manual_seed(3))
        direction = direction / direction.norm()
        tables = climbing["tables"].cpu()
        for b, kv_len in enumerate((900, 1100)):
            for n in range(kv_len):
                height = 0.07 * n + (40.0 if n in (300, 301, 777) else 0.0)
                climbing["k_cache"][int(tables[b, n // page]), :, n % page, :] += (height * direction).to(torch.bfloat16).cuda()
        climbing["qkv"][:, : nh * d] = (climbing["qkv"][:, : nh * d].float() * 0.3 + (direction * math.sqrt(d)).repeat(nh).cuda()).to(torch.bfloat16)
        want = _run_attention(ref, climbing, nh, nkv, d, page, window=window)
        for choice in (1, 2, 3):
            lib.velox_attention_portion_kernel(choice)
            torch.testing.assert_close(_run_attention(ops, climbing, nh, nkv, d, page, window=window), want, **tolerance)
    finally:
        lib.velox_attention_portion_kernel(0)


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_paged_attention_random_steps_agree_with_the_reference(ops, ref, seed):
    """Steps drawn at random: head size, heads and groups, page size, data type, window, splits of the keys, which kernel
    takes the portions, and one to six sequences that are single tokens, short portions or long ones, from an empty
    cache or behind up to 5,000 keys."""
    import random

    from velox_amd.engine.batch import Workspace

    rng = random.Random(seed)
    workspace = Workspace(torch.device("cuda"))
    for case_no in range(12):
        d = rng.choice([16, 48, 64, 80, 96, 128, 192, 256])
        page = rng.choice([1, 2, 4, 8, 16, 32, 64, 128])
        dtype = rng.choice(DTYPES)
        nkv = rng.choice([1, 2, 4, 8])
        nh = nkv * rng.choice([1, 2, 3, 5, 7])
        seqs = []
        for _ in range(rng.randint(1, 6)):
            kind = rng.random()
            q = 1 if kind < 0.25 else rng.randint(2, 70) if kind < 0.5 else rng.randint(71, 900)
            seqs.append((q, q + rng.choice([0, 0, rng.randint(1, 300), rng.randint(300, 5000)])))
        window = rng.choice([None, None, rng.randint(1, 3000)])
        choice = rng.choice([0, 0, 1, 2, 3])
        splits = rng.choice([None, None, 1, 2, 3])
        case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=100 * seed + case_no)
        lib = ops.attention_library(d)
        lib.velox_attention_portion_kernel(choice)
        try:
            got = _run_attention(ops, case, nh, nkv, d, page, window=window, splits=splits, workspace=workspace)
        finally:
            lib.velox_attention_portion_kernel(0)
        want = _run_attention(ref, case, nh, nkv, d, page, window=window)
        said = f"seed {seed} case {case_no}: {dtype} d={d} page={page} heads {nh}/{nkv} {seqs} window={window} kernel {choice} splits={splits}"
        torch.testing.assert_close(got, want, msg=lambda m: f"{said}: {m}", **(dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=2e-5)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 4), (28, 4, 128, 16), (3, 1, 32, 8), (2, 1, 256, 16)])
def test_decode_split_keys_equals_one_pass(ops, ref, dtype, nh, nkv, d, page):
    from velox_amd.engine.batch import Workspace

    seqs = [(1, 700), (1, 3), (1, 129), (1, 64), (1, 1)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=21)
    workspace = Workspace(torch.device("cuda"))
    one = _run_attention(ops, case, nh, nkv, d, page, splits=1, all_decode=True, workspace=workspace)
    want = _run_attention(ref, case, nh, nkv, d, page)
    t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(one, want, **t)
    for splits in (2, 3, 8, 32):  # 32 splits leave most of them empty for the short sequences
        got = _run_attention(ops, case, nh, nkv, d, page, splits=splits, all_decode=True, workspace=workspace)
        torch.testing.assert_close(got, want, **t)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_behind_more_pages_than_the_streaming_kernel_keeps_ids_of(ops, ref, dtype):
    """The streaming kernel keeps the page ids of a split's keys in LDS; a split of more pages than it has room for
    (2,048) goes through the kernel for portions instead, with the same result; with more splits the streaming kernel
    takes it again."""
    from velox_amd.engine.batch import Workspace

    nh, nkv, d, page = 6, 2, 64, 4
    seqs = [(1, 9000), (1, 77), (1, 8300)]
    case = _attention_case(dtype, nh, nkv, d, page, seqs, seed=31)
    workspace = Workspace(torch.device("cuda"))
    want = _run_attention(ref, case, nh, nkv, d, page)
    t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for splits in (1, 2, 8):  # 1 and 2: 2,250 and 1,125 + 2 pages per split, beyond and within the room for ids
        got = _run_attention(ops, case, nh, nkv, d, page, splits=splits, all_decode=True, workspace=workspace)
        torch.testing.assert_close(got, want, **t)


def test_far_key_among_hundreds_is_found(ops):
    # one key far back matches the query strongly: the output must be (nearly) that key's value
    nh, nkv, d, page = 4, 2, 64, 16
    seqs = [(1, 900)]
    case = _attention_case(torch.float32, nh, nkv, d, page, seqs, seed=5)
    target = 37
    tables = case["tables"].cpu()
    q = case["qkv"][0, : nh * d].view(nh, d)
    p, o = int(tables[0, target // page]), target % page
    for h in range(nh):
        case["k_cache"][p, h // 2, o, :] = 0
    case["k_cache"][p, 0, o, :] = 4.0 * (q[0] + q[1]) / 2
    case["k_cache"][p, 1, o, :] = 4.0 * (q[2] + q[3]) / 2
    out = _run_attention(ops, case, nh, nkv, d, page).view(nh, d)
    want = _run_attention(TorchOps(), case, nh, nkv, d, page).view(nh, d)
    torch.testing.assert_close(out, want, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("rows,vocab", [(1, 152064), (8, 151936), (64, 32003), (3, 5000), (300, 4099), (2, 2047)])
def test_argmax_over_chunks_of_the_vocabulary(ops, ref, rows, vocab):
    logits = rand((rows, vocab), torch.float32, 31, 3.0)
    torch.testing.assert_close(ops.argmax(logits), ref.argmax(logits))
    # ties across chunks: the first index wins; a maximum in the last, shorter chunk is found
    logits[0, vocab // 3] = logits[0, vocab - 5] = 60.0
    logits[rows - 1, vocab - 1] = 70.0
    got = ops.argmax(logits)
    assert int(got[rows - 1]) == vocab - 1 and (rows == 1 or int(got[0]) == vocab // 3)
    # an unaligned row start (a slice of a wider tensor)
    wide = rand((rows, vocab + 3), torch.float32, 32, 3.0)
    if (vocab + 3) % 4 == 0:
        torch.testing.assert_close(ops.argmax(wide[:, :vocab].contiguous()), ref.argmax(wide[:, :vocab]))


def test_argmax_and_sampling(ops, ref):
    vocab = 1003
    logits = rand((6, vocab), torch.float32, 30, 3.0)
    logits[2, 77] = logits[2, 900] = 50.0  # a tie: the first index wins
    torch.testing.assert_close(ops.argmax(logits), ref.argmax(logits))
    assert int(ops.argmax(logits)[2]) == 77

    options = np.zeros((6, 6), dtype=np.int32)
    f = options.view(np.float32)
    rows = [(0.0, 1.0, 0), (0.8, 1.0, 0), (1.0, 0.9, 0), (1.3, 1.0, 5), (0.7, 0.5, 50), (1.0, 1.0, 1)]
    for r, (temp, top_p, top_k) in enumerate(rows):
        f[r, 0], f[r, 1] = temp, top_p
        options[r, 2:] = (top_k, 1234 + r, 99, r)
    got = ops.sample(logits, torch.from_numpy(options).cuda()).cpu().numpy()
    for r in range(6):
        token, scores = TorchOps.sample_row(logits[r].cpu().numpy(), options[r])
        assert np.isfinite(scores[got[r]]), f"row {r}: token {got[r]} was filtered out"
        assert scores[got[r]] >= scores.max() - 1e-3, f"row {r}: token {got[r]} score {scores[got[r]]} vs best {scores.max()} ({token})"
    assert got[0] == int(logits[0].argmax())
    assert got[5] == int(logits[5].argmax())  # top_k = 1 is greedy


@pytest.mark.parametrize("vocab,spread", [(152064, 1.2), (151936 + 3, 4.0), (320, 2.0), (4099, 0.3)])
def test_sampling_keeps_exactly_the_tokens_the_filters_allow(ops, vocab, spread):
    """The threshold of top-k / top-p at the real vocabulary size, flat and peaked rows, ties across the threshold: over many
    draws per row, every drawn token is one the plain filter keeps, and the tokens at the filter's edge (the last kept ones)
    are drawn as well, so the kept set is neither too small nor too large.  A row's draw does not depend on its place."""
    settings = [(0.8, 0.9, 0), (1.0, 1.0, 7), (0.7, 0.5, 50), (1.3, 0.95, 1000), (1.0, 0.999, 0), (0.5, 0.3, 3), (1.0, 1.0, 0), (2.0, 0.6, 20000),
                (1.0, 1e-20, 0), (1.0, 1.0, 2)]  # a share of the mass so small that it rounds to nothing: the best token is still kept
    base = rand((len(settings), vocab), torch.float32, 77, spread)
    base[2, 5] = base[2, 11] = base[2, vocab - 1] = float(base[2].max()) + 0.5  # three equal tokens at the top
    base[5, :40] = float(base[5].max())  # forty equal tokens: rank 0 for all of them, so top_k = 3 keeps all forty
    base[9, 3], base[9, 8], base[9, 100], base[9, vocab - 2] = (float(base[9].max()) + x for x in (1.0, 0.5, 0.5, 0.5))  # top_k = 2 with three tokens tied at the cut
    draws = 300
    logits = base.repeat_interleave(draws, 0).contiguous()
    options = np.zeros((len(settings) * draws, 6), dtype=np.int32)
    f = options.view(np.float32)
    for r, (temp, top_p, top_k) in enumerate(settings):
        rows = slice(r * draws, (r + 1) * draws)
        f[rows, 0], f[rows, 1] = temp, top_p
        options[rows, 2] = top_k if 0 < top_k < vocab else 0
        options[rows, 3], options[rows, 4] = 4242 + r, 17
        options[rows, 5] = np.arange(draws)
    got = ops.sample(logits, torch.from_numpy(options).cuda()).cpu().numpy()
    for r, (temp, top_p, top_k) in enumerate(settings):
        _, scores = TorchOps.sample_row(base[r].cpu().numpy(), options[r * draws])
        kept = np.isfinite(scores)
        drawn = got[r * draws:(r + 1) * draws]
        assert kept[drawn].all(), f"row {r}: tokens {sorted(set(drawn[~kept[drawn]]))} were drawn but are filtered out"
        if kept.sum() <= 50:
            # few tokens are kept: 300 draws at these temperatures reach every one of them, the edge of the filter included
            x = base[r].cpu().numpy().astype(np.float64)
            share = np.where(kept, np.exp((x - x.max()) / temp), 0.0)
            probable = share / share.sum() > 0.04  # (missed by 300 draws with probability below 1e-5)
            assert set(np.flatnonzero(probable)) <= set(drawn), f"row {r}: kept tokens {sorted(set(np.flatnonzero(probable)) - set(drawn))} never drawn"
        # each draw is the best score among the kept tokens, with the generator's noise for its own counter
        for j in (0, 1, draws - 1):
            token, scores = TorchOps.sample_row(base[r].cpu().numpy(), options[r * draws + j])
            assert scores[drawn[j]] >= scores.max() - 1e-3, (r, j, int(drawn[j]), token)
    # stated without the plain filter: a share of the mass of nothing keeps the one best token, and a cut of top-k that falls
    # into a run of equal logits keeps the whole run (the reference keeps exactly k by sorted position, engine/sampler.py:218-221)
    assert set(got[8 * draws:9 * draws]) == {int(base[8].argmax())}
    assert set(got[9 * draws:10 * draws]) == {3, 8, 100, vocab - 2}
    # the same rows in another order and beside other rows: the same tokens
    order = torch.randperm(len(settings) * draws, generator=torch.Generator().manual_seed(5))[:97]
    again = ops.sample(logits[order.cuda()].contiguous(), torch.from_numpy(options[order.numpy()]).cuda()).cpu().numpy()
    assert (again == got[order.numpy()]).all()


@pytest.mark.parametrize("vocab,spread", [(152064, 1.2), (151936 + 3, 4.0), (321, 2.0), (4099, 0.3)])
def test_sampling_with_rows_cut_into_chunks_gives_the_same_tokens(ops, vocab, spread):
    """Few rows are sampled with several workgroups per row, one kernel per pass, the tables of the threshold's digits
    added up in global memory: the tokens are those of the one-workgroup kernel, bit for bit, for every number of chunks
    (chunks that end inside the last quad, chunks beyond the row's end, rows that start off a 16-byte boundary), for
    greedy rows, rows without a filter and rows with one, side by side."""
    settings = [(0.8, 0.9, 0), (1.0, 1.0, 7), (0.0, 1.0, 0), (0.7, 0.5, 50), (1.3, 0.95, 1000), (1.0, 0.999, 0), (0.5, 0.3, 3), (1.0, 1.0, 0), (2.0, 0.6, 20000),
                (1.0, 1e-20, 0)]
    base = rand((len(settings), vocab), torch.float32, 78, spread)
    base[3, 5] = base[3, 11] = base[3, vocab - 1] = float(base[3].max()) + 0.5
    base[6, :40] = float(base[6].max())
    base[2, 17] = base[2, vocab - 2] = float(base[2].max()) + 1.0  # a tie in the greedy row, in different chunks: the first wins
    draws = 5
    logits = base.repeat_interleave(draws, 0).contiguous()
    options = np.zeros((len(settings) * draws, 6), dtype=np.int32)
    f = options.view(np.float32)
    for r, (temp, top_p, top_k) in enumerate(settings):
        rows = slice(r * draws, (r + 1) * draws)
        f[rows, 0], f[rows, 1] = temp, top_p
        options[rows, 2] = top_k if 0 < top_k < vocab else 0
        options[rows, 3], options[rows, 4] = 999 + r, 3
        options[rows, 5] = np.arange(draws)
    device_options = torch.from_numpy(options).cuda()
    whole = ops.sample(logits, device_options, chunks=1).cpu().numpy()
    assert whole[2 * draws] == 17
    assert set(whole[9 * draws:10 * draws]) == {int(base[9].argmax())}  # top_p of nothing: the best token, not an id outside the vocabulary
    for chunks in (None, 2, 3, 7, 16, 64):
        got = ops.sample(logits, device_options, chunks=chunks).cpu().numpy()
        assert (got == whole).all(), (chunks, np.flatnonzero(got != whole)[:10], got[got != whole][:10], whole[got != whole][:10])
    # no row with a filter: the kernels of the digits are left out
    plain = [r for r, (temp, top_p, top_k) in enumerate(settings) if temp == 0.0 or (top_p >= 1.0 and top_k == 0)]
    pick = torch.tensor([r * draws + j for r in plain for j in range(draws)])
    got = ops.sample(logits[pick.cuda()].contiguous(), device_options[pick.cuda()].contiguous(), with_filter=False, chunks=5).cpu().numpy()
    assert (got == whole[pick.numpy()]).all()
    # a broken promise gives no token rather than one from the wrong set
    broken = ops.sample(logits, device_options, with_filter=False, chunks=5).cpu().numpy()
    has_filter = np.array([temp != 0.0 and (top_p < 1.0 or 0 < top_k < vocab) for temp, top_p, top_k in settings]).repeat(draws)
    assert (broken[has_filter] == -1).all() and (broken[~has_filter] == whole[~has_filter]).all()


def test_penalties_over_long_histories_and_a_large_vocabulary(ops, ref):
    vocab, rows, width = 152064, 4, 6000
    logits = rand((rows, vocab), torch.float32, 34, 2.0)
    g = torch.Generator().manual_seed(35)
    tokens = torch.randint(0, vocab, (rows, width), generator=g).to(torch.int32)
    tokens[1, :3000] = torch.randint(8000, 8200, (3000,), generator=g).to(torch.int32)  # many repeats inside one range of the table
    tokens[2, :] = 151000  # one token, 6000 times
    tokens = tokens.cuda()
    lengths = torch.tensor([6000, 3500, 6000, 1], dtype=torch.int32).cuda()
    coeffs = torch.tensor([[1.3, 0.5, 0.2], [2.0, 1.0, 0.01], [0.8, 0.0, 0.001], [1.1, 0.2, 0.3]], dtype=torch.float32).cuda()
    got, want = logits.clone(), logits.clone()
    ops.apply_penalties(got, tokens, lengths, coeffs)
    ref.apply_penalties(want, tokens, lengths, coeffs)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    assert int((got != logits).sum()) > 5000
    again = logits.clone()
    ops.apply_penalties(again, tokens, lengths, coeffs)
    assert torch.equal(again, got)


def test_penalties_from_a_table_of_counts_kept_on_the_device(ops, ref):
    """The table of counts is built from a request's tokens, grows by the sampler's tokens, and penalises the rows that
    point into it exactly as the history-walking kernel does with the same tokens; rows that point nowhere keep their logits."""
    vocab, rows = 152064, 5
    logits = rand((rows, vocab), torch.float32, 36, 2.0)
    g = torch.Generator().manual_seed(37)
    histories = [torch.randint(0, vocab, (n,), generator=g).to(torch.int32) for n in (6000, 1, 3500, 0, 777)]
    histories[2][:3000] = torch.randint(8000, 8200, (3000,), generator=g).to(torch.int32)
    histories[0][:500] = 151000
    counts = torch.zeros((8, vocab), dtype=torch.int32, device="cuda")
    place = [6, 0, 3, -1, 2]  # row 3 has no penalties; the table's rows are in no particular order
    for h, at in zip(histories, place):
        if at >= 0 and h.numel():
            ops.count_tokens(counts[at], h.cuda())
    new_tokens = torch.tensor([151000, 17, 8100, 5, vocab - 1], dtype=torch.int32)
    row_of = torch.tensor(place, dtype=torch.int32).cuda()
    ops.count_sampled(counts, row_of, new_tokens.cuda())
    coeffs = torch.tensor([[1.3, 0.5, 0.2], [2.0, 1.0, 0.01], [0.8, 0.0, 0.001], [1.7, 0.3, 0.3], [1.1, 0.2, 0.3]], dtype=torch.float32).cuda()
    got = logits.clone()
    ops.apply_penalties_from_counts(got, counts, row_of, coeffs)
    # the same through the history-walking kernel and through the plain formula
    width = 6001
    tokens = torch.zeros((rows, width), dtype=torch.int32)
    lengths = torch.zeros(rows, dtype=torch.int32)
    for r, (h, at) in enumerate(zip(histories, place)):
        if at < 0:
            continue
        whole = torch.cat([h, new_tokens[r:r + 1]])
        tokens[r, : whole.numel()] = whole
        lengths[r] = whole.numel()
    walked, want = logits.clone(), logits.clone()
    ops.apply_penalties(walked, tokens.cuda(), lengths.cuda(), coeffs)
    ref.apply_penalties(want, tokens.cuda(), lengths.cuda(), coeffs)
    assert torch.equal(got, walked)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
    assert torch.equal(got[3], logits[3]) and int((got != logits).sum()) > 6000
    assert int(counts[6, 151000]) == 501 + int((histories[0][500:] == 151000).sum()) and int(counts.sum()) == sum(h.numel() for h, at in zip(histories, place) if at >= 0) + 4


def test_sampling_follows_the_distribution(ops):
    vocab = 50
    logits = rand((1, vocab), torch.float32, 31, 1.5).repeat(4000, 1).contiguous()
    options = np.zeros((4000, 6), dtype=np.int32)
    options.view(np.float32)[:, 0] = 0.9
    options.view(np.float32)[:, 1] = 1.0
    options[:, 3] = 7
    options[:, 5] = np.arange(4000)
    got = ops.sample(logits, torch.from_numpy(options).cuda()).cpu().numpy()
    probs = torch.softmax(logits[0].cpu() / 0.9, -1).numpy()
    counts = np.bincount(got, minlength=vocab)
    expected = probs * 4000
    keep = expected > 5
    chi2 = (((counts - expected) ** 2) / expected)[keep].sum()
    assert chi2 < 2.0 * keep.sum() + 30, f"chi-square {chi2} over {keep.sum()} bins"


def test_penalties(ops, ref):
    vocab, rows, width = 333, 3, 40
    logits = rand((rows, vocab), torch.float32, 32, 2.0)
    tokens = torch.randint(0, 60, (rows, width), generator=torch.Generator().manual_seed(33)).to(torch.int32).cuda()
    lengths = torch.tensor([40, 0, 17], dtype=torch.int32).cuda()
    coeffs = torch.tensor([[1.3, 0.5, 0.2], [2.0, 1.0, 1.0], [0.8, 0.0, 0.7]], dtype=torch.float32).cuda()
    got, want = logits.clone(), logits.clone()
    ops.apply_penalties(got, tokens, lengths, coeffs)
    ref.apply_penalties(want, tokens, lengths, coeffs)
    torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m,n,k", [(1, 320, 64), (8, 3584, 3584), (16, 263, 128), (7, 4608, 3584), (17, 100, 192), (32, 1000, 256), (33, 70, 64), (64, 3584, 18944), (50, 152064 // 16, 448)])
def test_skinny_gemm(ops, ref, out_dtype, m, n, k):
    x = rand((m, k), torch.bfloat16, 40)
    w = rand((n, k), torch.bfloat16, 41, 0.05)
    bias = rand((n,), torch.float32, 42)
    want = ref.linear(x, w, None, torch.float32)
    scale = float(want.abs().max())
    for waves, row_tiles in ((None, None), (4, 1), (8, 1), (16, 1), (4, 4), (8, 4)):
        for b in (None, bias):
            got = ops.skinny_gemm(x, w, b, out_dtype, waves=waves, row_tiles=row_tiles).float()
            expect = want + (b if b is not None else 0)
            atol = 1e-4 * scale if out_dtype == torch.float32 else 1e-2 * scale
            torch.testing.assert_close(got, expect, rtol=1e-2 if out_dtype == torch.bfloat16 else 1e-4, atol=atol)
    # the weight in the order the lanes read it gives the same bits as the row-major weight
    packed = ops.pack_rows(w)
    got = ops.skinny_gemm(x, None, bias, out_dtype, packed=packed, n=n).float()  # with its own choice of waves and tiles
    torch.testing.assert_close(got, want + bias, rtol=1e-2 if out_dtype == torch.bfloat16 else 1e-4, atol=atol)
    for waves, row_tiles in ((4, 1), (16, 1), (4, 4)):
        torch.testing.assert_close(ops.skinny_gemm(x, None, bias, out_dtype, waves=waves, row_tiles=row_tiles, packed=packed, n=n),
                                   ops.skinny_gemm(x, w, bias, out_dtype, waves=waves, row_tiles=row_tiles), rtol=0, atol=0)
    # the same rows give the same bits whatever else is in the batch, as long as the batch stays in one size class
    # (up to 16, up to 32, up to 64 rows: the classes split K differently, which changes the order of the sums)
    fewer = 1 if m <= 16 else 17 if m <= 32 else 33
    if m > fewer:
        part = ops.skinny_gemm(x[:fewer].contiguous(), w, None, out_dtype)
        torch.testing.assert_close(ops.skinny_gemm(x, w, None, out_dtype)[:fewer], part, rtol=0, atol=0)


def test_prepared_copies_belong_to_one_weight_and_one_version(ops, ref):
    """What ``prepare_weight`` returns is held by the caller and stands in the weight's place; a plain tensor is multiplied
    as it is (no copy is ever found through an address), and a weight changed in place behind its copies is an error, not a
    product with stale values."""
    from velox_amd.kernels.hip_ops import KernelError

    x = rand((4, 128), torch.bfloat16, 60)
    first = rand((96, 128), torch.bfloat16, 61, 0.05)
    prepared = ops.prepare_weight(first)
    assert prepared.weight is first and prepared.copy(1) is not None and prepared.copy(2) is None
    want = ref.linear(x, first, None, torch.float32)
    torch.testing.assert_close(ops.linear(x, prepared, None, torch.float32), want, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(ops.linear(x, first, None, torch.float32), want, rtol=1e-4, atol=1e-4)
    other = rand((96, 128), torch.bfloat16, 62, 0.05)
    assert ops.prepare_weight(other, stacked=2, handle=prepared).weight is other  # another weight: a new handle, not an extended one
    first.mul_(2.0)
    with pytest.raises(KernelError, match="changed in place"):
        ops.linear(x, prepared, None, torch.float32)
    again = ops.prepare_weight(first, handle=prepared)
    assert again is not prepared
    torch.testing.assert_close(ops.linear(x, again, None, torch.float32), 2 * want, rtol=1e-4, atol=1e-4)
    stacked = ops.prepare_weight(other, stacked=2)
    assert stacked.copy(2) is not None and stacked.copy(1) is None
    # what the kernels cannot read in their lanes' order stays as it is
    assert ops.prepare_weight(rand((96, 100), torch.bfloat16, 63)) is None
    assert ops.prepare_weight(rand((96, 128), torch.float32, 64)) is None


def test_a_part_refuses_a_weight_bound_again_behind_prepared_copies(ops):
    from velox_amd.parts import make_part

    ff = make_part("feed_forward", "gated_mlp", prefix="m.", hidden_size=128, intermediate_size=192)
    ff.gate_up_weight = rand((384, 128), torch.bfloat16, 65, 0.05)
    ff.down_weight = rand((128, 192), torch.bfloat16, 66, 0.05)
    assert ff.operand("down_weight") is ff.down_weight  # nothing prepared yet: the tensor itself
    ff.prepare_kernels(ops)
    assert ff.operand("down_weight").weight is ff.down_weight and ff.operand("gate_up_weight").copy(2) is not None
    ff.down_weight = ff.down_weight.clone()
    with pytest.raises(RuntimeError, match="bound again"):
        ff.operand("down_weight")
    ff.prepare_kernels(ops)
    assert ff.operand("down_weight").weight is ff.down_weight


@pytest.mark.parametrize("m,inter,k", [(1, 128, 64), (8, 18944, 3584), (16, 150, 128), (7, 1000, 192), (3, 16, 64)])
def test_skinny_gemm_with_silu_epilogue(ops, ref, m, inter, k):
    x = rand((m, k), torch.bfloat16, 50)
    w = rand((2 * inter, k), torch.bfloat16, 51, 0.05)
    gate_up = ref.linear(x, w, None, torch.float32)
    want = (torch.nn.functional.silu(gate_up[:, :inter]) * gate_up[:, inter:])
    scale = float(want.abs().max())
    for waves, pairs in ((None, None), (4, 1), (8, 1), (4, 2), (8, 2)):
        got = ops.linear_silu_mul(x, w, torch.bfloat16, waves=waves, pairs=pairs).float()
        torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2 * scale)
    packed = ops.pack_rows(w, matrices=2)
    for waves, pairs in ((None, None), (4, 1), (8, 2)):
        torch.testing.assert_close(ops.linear_silu_mul(x, w, torch.bfloat16, waves=waves, pairs=pairs, packed=packed),
                                   ops.linear_silu_mul(x, w, torch.bfloat16, waves=waves, pairs=pairs), rtol=0, atol=0)
    # larger batches take the unfused route and agree with it
    big = rand((40, k), torch.bfloat16, 52)
    torch.testing.assert_close(ops.linear_silu_mul(big, w, torch.bfloat16).float(), ref.linear_silu_mul(big, w, torch.bfloat16).float(), rtol=3e-2, atol=3e-2 * scale)


@pytest.mark.parametrize("m,inter,k", [(17, 18944, 3584), (64, 18944, 3584), (32, 150, 128), (33, 1000, 192), (40, 16, 64), (64, 81, 1600), (24, 400, 320)])
def test_gate_up_product_with_silu_epilogue_at_17_to_64_rows(ops, ref, m, inter, k):
    """A registered [Wgate; Wup] at 17 .. 64 rows: one kernel (ten waves per workgroup, five pairs of gate and up tiles)
    against the product in float32 followed by silu(gate) * up; widths that are no multiple of 16 or of 80, a K that
    is no multiple of a chunk of 256."""
    x = rand((m, k), torch.bfloat16, 53)
    w = rand((2 * inter, k), torch.bfloat16, 54, 0.05)
    gate_up = ref.linear(x, w, None, torch.float32)
    want = (torch.nn.functional.silu(gate_up[:, :inter]) * gate_up[:, inter:])
    scale = float(want.abs().max())
    unregistered = ops.linear_silu_mul(x, w, torch.bfloat16).float()  # (product + SiLU kernel)
    pw = ops.prepare_weight(w, stacked=2)
    got = ops.linear_silu_mul(x, pw, torch.bfloat16).float()
    torch.testing.assert_close(got, want, rtol=1e-2, atol=1e-2 * scale)
    torch.testing.assert_close(got, unregistered, rtol=2e-2, atol=2e-2 * scale)
    # rows of a batch do not depend on one another: the first rows alone give the same bits
    few = ops.linear_silu_mul(x[:17].contiguous(), pw, torch.bfloat16).float()
    assert torch.equal(few, got[:17])


@pytest.mark.parametrize("m,n,k", [(17, 3584, 18944), (64, 3584, 3584), (33, 100, 640), (64, 4608, 3584), (40, 260, 128), (64, 72, 1600)])
def test_skinny_gemm_splitk_and_norm_that_adds_the_partials(ops, ref, m, n, k):
    x = rand((m, k), torch.bfloat16, 60)
    w = rand((n, k), torch.bfloat16, 61, 0.05)
    want = ref.linear(x, w, None, torch.float32)
    scale = float(want.abs().max())
    for splits in (None, 1, 2, 5):
        part = ops.skinny_gemm_splitk(x, w, splits=splits)
        assert part.dim() == 3 and part.shape[1:] == (m, n) and part.dtype == torch.float32
        torch.testing.assert_close(part.sum(0), want, rtol=1e-4, atol=1e-4 * scale)
        # the weight in the order the lanes read it: the same products in the same order
        torch.testing.assert_close(ops.skinny_gemm_splitk(x, w, splits=splits, packed=ops.pack_rows(w)), part, rtol=0, atol=0)
    part = ops.skinny_gemm_splitk(x, w)
    if n % 4 == 0:
        residual = rand((m, n), torch.float32, 62)
        weight = 1 + rand((n,), torch.float32, 63, 0.02)
        r_hip, r_ref = residual.clone(), residual.clone()
        got = ops.add_rmsnorm(r_hip, part, weight, 1e-6, torch.bfloat16)
        ref_out = ref.add_rmsnorm(r_ref, part, weight, 1e-6, torch.bfloat16)
        torch.testing.assert_close(r_hip, r_ref, rtol=1e-5, atol=1e-5 * scale)
        torch.testing.assert_close(got.float(), ref_out.float(), rtol=2e-2, atol=2e-2)
        rows = torch.tensor([m - 1, 0, 3], dtype=torch.int32).cuda()
        torch.testing.assert_close(ops.add_rmsnorm_rows(r_hip, part, rows, weight, 1e-6, torch.float32),
                                   ref.add_rmsnorm_rows(r_ref, part, rows, weight, 1e-6, torch.float32), rtol=1e-4, atol=1e-4)


def test_probes_report_rates_in_the_band_of_this_card(ops):
    """The two probes that bench.py reports its fractions against: a read of 2 GiB (far more than the caches hold) streams
    at more than half and less than all of the published 8 TB/s; independent bfloat16 matrix instructions run at more than
    half and no more than the published 2.5 PFLOP/s.  A probe that measured nothing (a loop the compiler removed, a
    launch that failed) or counted its work wrongly would fall out of these bands."""
    read = ops.probe_read_bandwidth(num_bytes=(2 << 30) + 48, repeats=3)
    mfma = ops.probe_mfma_rate(iterations=20000, repeats=3)
    assert 4000.0 < read < 8000.0, read
    assert 1250.0 < mfma <= 2600.0, mfma


def test_grid_barrier_probe_ends_and_counts_every_round(ops):
    """The probe of a barrier across one workgroup per compute unit runs all its rounds (nobody gives up waiting: that
    would raise) in both forms, takes between 0.2 and 200 us per barrier, and the fenced form is the dearer one."""
    relaxed = ops.probe_grid_barrier(False, rounds=200, repeats=2)
    fenced = ops.probe_grid_barrier(True, rounds=200, repeats=2)
    assert 0.2 < relaxed < 200.0 and 0.2 < fenced < 200.0, (relaxed, fenced)
    assert fenced > relaxed, (relaxed, fenced)


def test_kernel_timer_times_a_launch_inside_a_graph(ops):
    """`velox_amd.kernels.measure` (the timings that the launch rules quote): a case of scattered pages has the shapes
    the attention entry point checks, and the timer replays a graph of launches and returns a plausible time per call."""
    import math

    from velox_amd.engine.batch import Workspace
    from velox_amd.kernels.measure import attention_case, time_in_graph

    qkv, k, v, tables, cu_q, kv_lens = attention_case(2, 96, 160, 4, 2, 64, 16)
    assert tables.shape == (2, 10) and int(tables.min()) >= 1 and len(set(tables.flatten().tolist())) == 20
    workspace = Workspace(torch.device("cuda"))
    each = time_in_graph(lambda: ops.paged_attention(qkv, 4, 2, 64, k, v, 16, tables, cu_q, kv_lens, 96, 160, 1 / math.sqrt(64), None, False, workspace),
                         launches=2, rounds=2)
    assert 1.0 < each < 5000.0, each


def test_place_tokens_puts_sampled_ids_into_a_steps_rows(ops, ref):
    from velox_amd.kernels.hip_ops import KernelError

    ids = torch.arange(100, 140, dtype=torch.int32).cuda()
    tokens = torch.tensor([7, 8, 9, 10, 11], dtype=torch.int32).cuda()
    dest = torch.tensor([3, 39, 0, 17, 99, 5], dtype=torch.int32).cuda()   # (the fifth pair points outside ids: skipped)
    source = torch.tensor([4, 0, 2, 2, 1, 77], dtype=torch.int32).cuda()   # (the sixth outside tokens: skipped)
    want = ids.clone()
    ref.place_tokens(want, dest, source, tokens, 4)
    got = ids.clone()
    ops.place_tokens(got, dest, source, tokens, 6)
    assert torch.equal(got, want) and got[3] == 11 and got[39] == 7 and got[0] == 9 and got[17] == 9 and got[5] == 105
    untouched = ids.clone()
    ops.place_tokens(untouched, dest, source, tokens, 0)
    assert torch.equal(untouched, ids)
    with pytest.raises(KernelError):
        ops.place_tokens(got, dest, source, tokens, 7)
