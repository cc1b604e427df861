"""Each part alone: built from its arguments, bound to random parameters, run on a
hand-made step context and compared with the plain function of the same name."""

from __future__ import annotations

import pytest
import torch

from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def bind_random(part, dtype, prefix="p", seed=0):
    """Random parameters by the part's own declaration; returns them as float64 CPU too."""
    from kvcore_amd.parts.base import Runtime

    part.setup(Runtime(dtype, DEV))
    g = torch.Generator().manual_seed(seed)
    params, plain_params = {}, {}
    for ps in part.param_specs():
        t = torch.randn(ps.shape, generator=g) * (0.1 if ps.init != "gain" else 0.1)
        if ps.init == "gain":
            t = t + 1
        kind = {"matrix": dtype, "vector": torch.float32}[ps.kind]
        params[ps.name] = t.to(kind).to(DEV)
        plain_params[ps.name] = params[ps.name].double().cpu()
    part.bind(params)
    return plain_params


def make_ctx(dtype, positions, token_req, slots, groups=(), states=()):
    from kvcore_amd.engine.context import StepBuffers, StepContext

    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)  # noqa: E731
    T = len(positions)
    R = len(slots)
    q_lens = [token_req.count(r) for r in range(R)]
    q_start = [0]
    for n in q_lens:
        q_start.append(q_start[-1] + n)
    seq = [max(p for p, r in zip(positions, token_req) if r == i) + 1 for i in range(R)]
    return StepContext(num_tokens=T, num_reqs=R, token_ids=i32([0] * T), positions=i32(positions),
                       token_req=i32(token_req), q_start=i32(q_start), seq_lens=i32(seq),
                       slots=i32(slots), groups=list(groups), states=list(states),
                       buffers=StepBuffers(DEV), dtype=dtype, device=DEV, host_query_lens=q_lens,
                       host_seq_lens=seq, max_query_len=max(q_lens), max_seq_len=max(seq))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_part(dtype):
    from kvcore_amd.parts.base import NORMS, PartSpec

    norm = NORMS.build(PartSpec("rmsnorm", {"hidden_size": 72, "eps": 2e-5}))
    p = bind_random(norm, dtype)
    residual = torch.randn(6, 72, device=DEV)
    delta = torch.randn(6, 72, device=DEV).to(dtype)
    out = torch.empty(6, 72, dtype=dtype, device=DEV)
    want_res = residual.double().cpu() + delta.double().cpu()
    norm.forward_fused(out, residual, delta)
    assert torch.allclose(residual.double().cpu(), want_res, atol=1e-6)
    assert torch.allclose(out.double().cpu(), plain.rms_norm(want_res, p["weight"], 2e-5), **tol(dtype))


def test_rotary_part_tables_and_scaling():
    from kvcore_amd.parts.base import POSITION_ENCODINGS, PartSpec, Runtime
    from kvcore_amd.parts.rotary import rotary_inv_freq

    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 64}
    inv = rotary_inv_freq(32, 500000.0, scaling)
    want = plain.llama3_scale_inv_freq(plain.rope_inv_freq(32, 500000.0), **{k: v for k, v in scaling.items()
                                                                             if k != "rope_type"})
    assert torch.allclose(inv.double(), want, rtol=1e-6)
    assert torch.allclose(rotary_inv_freq(32, 500000.0, None).double(), plain.rope_inv_freq(32, 500000.0), rtol=1e-6)
    with pytest.raises(ValueError):
        rotary_inv_freq(32, 1e4, {"rope_type": "yarn"})
    pe = POSITION_ENCODINGS.build(PartSpec("rotary", {"rot_dim": 32, "theta": 500000.0, "scaling": scaling}))
    pe.setup(Runtime(torch.float32, DEV))
    ctx = make_ctx(torch.float32, [0, 5, 200], [0, 0, 0], [0])
    pe.prepare(ctx)
    tabs = pe.rotary(ctx)
    ang = torch.tensor([0.0, 5.0, 200.0], dtype=torch.float64)[:, None] * want[None, :]
    assert torch.allclose(tabs.cos.double().cpu(), ang.cos(), atol=1e-5)
    assert torch.allclose(tabs.sin.double().cpu(), ang.sin(), atol=1e-5)
    assert tabs.rot_dim == 32 and not tabs.interleaved


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_part(dtype):
    from kvcore_amd.parts.base import FEED_FORWARDS, PartSpec

    ffn = FEED_FORWARDS.build(PartSpec("swiglu", {"hidden_size": 48, "intermediate_size": 112, "bias": True}))
    p = bind_random(ffn, dtype)
    ctx = make_ctx(dtype, [0, 1, 2, 3, 4], [0] * 5, [0])
    x = (torch.randn(5, 48) * 2).to(dtype).to(DEV)
    y = ffn.forward(x, ctx, None)
    gw, uw = p["gate_up_proj.weight"][:112], p["gate_up_proj.weight"][112:]
    gb, ub = p["gate_up_proj.bias"][:112], p["gate_up_proj.bias"][112:]
    want = plain.swiglu_mlp(x.double().cpu(), gw, uw, p["down_proj.weight"], gb, ub, p["down_proj.bias"])
    assert torch.allclose(y.double().cpu(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [0, 6])
def test_attention_part_in_two_portions(dtype, window):
    """The attention part, fed 11 tokens and then 7 more, equals the plain attention block
    over all 18; the second call reads what the first wrote to the cache."""
    from kvcore_amd.engine.context import CacheGroupView, LayerCall
    from kvcore_amd.parts.base import MIXERS, POSITION_ENCODINGS, PartSpec, Runtime

    H, nh, nkv, d, page = 40, 6, 2, 16, 4
    pe = POSITION_ENCODINGS.build(PartSpec("rotary", {"rot_dim": d, "theta": 1000.0}))
    pe.setup(Runtime(dtype, DEV))
    attn = MIXERS.build(PartSpec("paged_attention", {
        "hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d, "scale": 0.3,
        "bias": True, "window": window}), position=pe)
    p = bind_random(attn, dtype, seed=3)
    assert attn.cache_need().window == window and attn.state_need() is None
    need = attn.cache_need()
    assert need.planes == ((nkv, d), (nkv, d)) and need.token_elems() == (nkv * d, nkv * d)
    # two schedule entries, nine pages, a plane for the keys and one for the values
    storage = [torch.full((2, 9, page * n), float("nan"), dtype=dtype, device=DEV) for n in need.token_elems()]
    table = torch.zeros(3, 8, dtype=torch.int32, device=DEV)
    table[2, :5] = torch.tensor([4, 7, 1, 8, 2], dtype=torch.int32)
    group = CacheGroupView(storage, table, page, window)
    call = LayerCall(0, 0, 0, 1, True, None)  # entry 1 of the group
    x = (torch.randn(18, H)).to(dtype).to(DEV)
    outs = []
    for lo, hi in ((0, 11), (11, 18)):
        ctx = make_ctx(dtype, list(range(lo, hi)), [0] * (hi - lo), [2], groups=[group])
        pe.prepare(ctx)
        outs.append(attn.forward(x[lo:hi].contiguous(), ctx, call).clone())
    got = torch.cat(outs).double().cpu()
    w = {}
    q_rows, kv_rows = nh * d, nkv * d
    for name, lo, hi in (("q_proj", 0, q_rows), ("k_proj", q_rows, q_rows + kv_rows),
                         ("v_proj", q_rows + kv_rows, q_rows + 2 * kv_rows)):
        w[f"a.{name}.weight"] = p["qkv_proj.weight"][lo:hi]
        w[f"a.{name}.bias"] = p["qkv_proj.bias"][lo:hi]
    w["a.o_proj.weight"], w["a.o_proj.bias"] = p["o_proj.weight"], p["o_proj.bias"]
    T = 18
    xq = x.double().cpu()
    q = (xq @ w["a.q_proj.weight"].T + w["a.q_proj.bias"]).view(T, nh, d)
    k = (xq @ w["a.k_proj.weight"].T + w["a.k_proj.bias"]).view(T, nkv, d)
    v = (xq @ w["a.v_proj.weight"].T + w["a.v_proj.bias"]).view(T, nkv, d)
    inv = plain.rope_inv_freq(d, 1000.0)
    q, k = plain.apply_rope(q, torch.arange(T), inv), plain.apply_rope(k, torch.arange(T), inv)
    o = plain.causal_gqa_attention(q, k, v, 0.3, window=window or None)
    want = o.reshape(T, nh * d) @ w["a.o_proj.weight"].T + w["a.o_proj.bias"]
    assert torch.allclose(got, want, **tol(dtype))
    assert all(torch.isnan(plane[0]).all() for plane in storage)  # entry 0 was not this call's to write


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_and_head_parts(dtype):
    from kvcore_amd.parts.embedding import OutputHead, TokenEmbedding

    emb = TokenEmbedding(vocab_size=50, hidden_size=24)
    p = bind_random(emb, dtype)
    ids = torch.tensor([3, 49, 0], dtype=torch.int32, device=DEV)
    residual = torch.empty(3, 24, device=DEV)
    emb.forward(residual, ids)
    assert torch.equal(residual.double().cpu(), p["weight"][[3, 49, 0]])
    head = OutputHead(vocab_size=50, hidden_size=24, tied=True)
    assert head.param_specs() == []
    head.bind({"weight": emb.params["weight"]})
    ctx = make_ctx(dtype, [0, 1, 2], [0, 0, 0], [0])
    hidden = torch.randn(3, 24).to(dtype).to(DEV)
    logits = torch.empty(3, 50, device=DEV)
    head.forward(logits, hidden, ctx)
    assert logits.dtype == torch.float32
    assert torch.allclose(logits.double().cpu(), hidden.double().cpu() @ p["weight"].T, **tol(dtype))


def test_prenorm_block_against_the_reference_arrangement():
    """r += delta; a = mixer(norm(r)); r += a; out = ffn(norm(r)) (llama3.py:124-142)."""
    from kvcore_amd.parts.base import BLOCKS, FeedForward, Mixer, NORMS, PartSpec

    class Doubler(Mixer):
        def forward(self, x, ctx, call):
            return x * 2

    class Negate(FeedForward):
        def forward(self, x, ctx, call):
            return -x

    H = 16
    norms = {n: NORMS.build(PartSpec("rmsnorm", {"hidden_size": H, "eps": 1e-6}))
             for n in ("input_layernorm", "post_attention_layernorm")}
    gains = {n: bind_random(norm, torch.float32, seed=i)["weight"] for i, (n, norm) in enumerate(norms.items())}
    block = BLOCKS.build(PartSpec("prenorm"), mixer=Doubler(), ffn=Negate(), norms=norms)
    assert list(block.children()) == ["input_layernorm", "self_attn", "post_attention_layernorm", "mlp"]
    ctx = make_ctx(torch.float32, [0, 1], [0, 0], [0])
    residual = torch.randn(2, H, device=DEV)
    residual2 = residual.clone()
    delta = torch.randn(2, H, device=DEV)
    r = residual.double().cpu() + delta.double().cpu()
    a = 2 * plain.rms_norm(r, gains["input_layernorm"], 1e-6)
    r2 = r + a
    want = -plain.rms_norm(r2, gains["post_attention_layernorm"], 1e-6)
    out = block.forward(delta, residual, ctx, None)
    assert torch.allclose(out.double().cpu(), want, atol=1e-5)
    assert torch.allclose(residual.double().cpu(), r2, atol=1e-5)
    with pytest.raises(ValueError, match="norms"):
        BLOCKS.build(PartSpec("prenorm"), mixer=Doubler(), ffn=Negate(), norms={})
    # the norms' names (their checkpoint sub-prefixes) are the architecture's to choose
    renamed = {"ln_2": norms["post_attention_layernorm"], "ln_1": norms["input_layernorm"]}
    other = BLOCKS.build(PartSpec("prenorm", {"input_norm": "ln_1", "post_norm": "ln_2", "mixer_name": "mix",
                                              "ffn_name": "ff"}), mixer=Doubler(), ffn=Negate(), norms=renamed)
    assert list(other.children()) == ["ln_1", "mix", "ln_2", "ff"]
    out2 = other.forward(delta, residual2, ctx, None)
    assert torch.equal(out2, out)
    with pytest.raises(ValueError, match="norms"):
        BLOCKS.build(PartSpec("prenorm", {"input_norm": "ln_1", "post_norm": "ln_3"}), mixer=Doubler(),
                     ffn=Negate(), norms=renamed)


def test_head_part_scale_vector_of_the_reference():
    """tests/test_sampler.py:10-17 of the reference: weight [[1,0],[0,1],[1,1]], hidden [2,3],
    scale 0.5 give [1.0, 1.5, 2.5], through the head part itself."""
    from kvcore_amd.parts.base import HEADS, PartSpec, Runtime

    for dtype in DTYPES:
        head = HEADS.build(PartSpec("linear_head", {"vocab_size": 3, "hidden_size": 2, "logit_scale": 0.5}))
        head.setup(Runtime(dtype, DEV))
        head.bind({"weight": torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]], dtype=dtype, device=DEV)})
        logits = torch.empty(1, 3, device=DEV)
        head.forward(logits, torch.tensor([[2.0, 3.0]], dtype=dtype, device=DEV), make_ctx(dtype, [0], [0], [0]))
        assert torch.equal(logits.cpu(), torch.tensor([[1.0, 1.5, 2.5]]))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 14, 40, 70])
def test_head_part_keeps_float32_sums_whatever_the_row_count(dtype, rows):
    """A vocabulary beyond 65536 entries sends 3, 14, 40 and 70 rows down the head's four
    branches; all of them store the float32 sums unrounded (a row's logits must not change
    their rounding with the rows beside it), with bias, soft cap and scale applied after."""
    from kvcore_amd.parts.base import HEADS, PartSpec

    V, H = 70016, 512
    head = HEADS.build(PartSpec("linear_head", {"vocab_size": V, "hidden_size": H, "bias": True,
                                                 "soft_cap": 30.0, "logit_scale": 0.25}))
    p = bind_random(head, dtype, seed=rows)
    bias = (torch.randn(V, generator=torch.Generator().manual_seed(1)) * 0.3).to(dtype).to(DEV)
    head.bind({**head.params, "bias": bias})
    x = (torch.randn(rows, H, generator=torch.Generator().manual_seed(2))).to(dtype).to(DEV)
    logits = torch.empty(rows, V, device=DEV)
    head.forward(logits, x, make_ctx(dtype, [0] * rows, list(range(rows)), list(range(rows))))
    want = x.double().cpu() @ p["weight"].T + bias.double().cpu()
    want = torch.tanh(want / 30.0) * 30.0 * 0.25
    # the operands are the same bits on both sides, so only the order of the float32 sums differs
    assert torch.allclose(logits.double().cpu(), want, atol=2e-5, rtol=1e-5)
    # and the first rows alone give the bits they had in company
    alone = torch.empty(2, V, device=DEV)
    head.forward(alone, x[:2].contiguous(), make_ctx(dtype, [0, 0], [0, 1], [0, 1]))
    assert torch.allclose(alone, logits[:2], atol=2e-5, rtol=1e-5)


def test_embedding_part_scale():
    from kvcore_amd.parts.base import EMBEDDINGS, PartSpec

    for dtype in DTYPES:
        emb = EMBEDDINGS.build(PartSpec("token_embedding", {"vocab_size": 50, "hidden_size": 24, "scale": 3.0}))
        p = bind_random(emb, dtype)
        ids = torch.tensor([4, 49, 0], dtype=torch.int32, device=DEV)
        out = torch.empty(3, 24, device=DEV)
        emb.forward(out, ids)
        assert torch.allclose(out.double().cpu(), p["weight"][ids.long().cpu()] * 3.0, atol=1e-6)


def test_attention_refuses_a_block_table_wider_than_its_decode_kernel_serves():
    """At construction of a runner, not in the middle of a generation."""
    from kvcore_amd.ops import library as ops
    from kvcore_amd.parts.base import MIXERS, PartSpec, RunLimits, Runtime

    attn = MIXERS.build(PartSpec("paged_attention", {"hidden_size": 4096, "num_heads": 32, "num_kv_heads": 8,
                                                     "head_dim": 128, "scale": 128 ** -0.5}), position=None)
    attn.setup(Runtime(torch.bfloat16, DEV))
    widest = ops.decode_attention_max_table(32, 8, 128)
    assert widest >= 8192  # 131,072 tokens in pages of 16
    attn.check_limits(RunLimits(8, 512, widest * 16, 16, widest))
    with pytest.raises(ValueError, match="block_size"):
        attn.check_limits(RunLimits(8, 512, (widest + 1) * 16, 16, widest + 1))
    # float32 runs the general kernel, which has no such limit
    attn.setup(Runtime(torch.float32, DEV))
    attn.check_limits(RunLimits(8, 512, (widest + 1) * 16, 16, widest + 1))


def test_attention_refuses_a_cache_in_another_dtype_when_it_is_built():
    """``CacheNeed.dtype`` lets a mixer keep its cache in a dtype of its own; the attention
    kernels read the model's, so a subclass that only changes the need is told so when the
    runner is built, not by a kernel in its first step."""
    from kvcore_amd.parts.attention import PagedAttention
    from kvcore_amd.parts.base import CacheNeed, RunLimits, Runtime

    class FloatCache(PagedAttention):
        def cache_need(self):
            return CacheNeed.keys_and_values(self.num_kv_heads, self.head_dim, dtype=torch.float32)

    args = dict(hidden_size=64, num_heads=4, num_kv_heads=2, head_dim=16, scale=0.25)
    attn = FloatCache(**args)
    attn.setup(Runtime(torch.bfloat16, DEV))
    with pytest.raises(ValueError, match="keeps its cache in torch.float32"):
        attn.check_limits(RunLimits(8, 512, 256, 16, 16))
    attn.setup(Runtime(torch.float32, DEV))
    attn.check_limits(RunLimits(8, 512, 256, 16, 16))
    plain_attn = PagedAttention(**args)
    plain_attn.setup(Runtime(torch.bfloat16, DEV))
    plain_attn.check_limits(RunLimits(8, 512, 256, 16, 16))
