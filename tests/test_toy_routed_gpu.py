"""More toy parts, all defined here and registered without a change to the framework's
files: a learned position table added at the embedding (so attention runs without
rotation), a feed-forward that routes every token to one of several experts (router in
float32, lowest index on ties, expert weights stacked along a leading dimension), a
layer norm with mean and bias, and two attention layers with different needs (a window
of 16 keys, and all keys), which therefore get cache groups of their own."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["ToyRoutedForCausalLM"], "vocab_size": 83, "hidden_size": 48, "heads": 3,
    "kv_heads": 1, "head_dim": 16, "experts": 3, "expert_size": 40, "eps": 1e-5, "window": 16,
    "max_position_embeddings": 96,
}
PAGE = 8


def register_toy():
    from kvcore_amd.models.spec import LayerSpec, ModelSpec
    from kvcore_amd.ops import library as ops
    from kvcore_amd.parts.base import (FEED_FORWARDS, FeedForward, Norm, ParamSource, ParamSpec,
                                       PartSpec, PositionEncoding, register_feed_forward,
                                       register_norm, register_position_encoding)
    from kvcore_amd.registry import MODEL_REGISTRY, register_architecture

    class LearnedPositions(PositionEncoding):
        """``r[t] += table[position[t]]``; nothing is rotated."""

        def __init__(self, *, max_positions, hidden_size):
            self.max_positions, self.hidden_size = max_positions, hidden_size

        def param_specs(self):
            return [ParamSpec("weight", (self.max_positions, self.hidden_size))]

        def embed(self, residual, ctx):
            pos = ctx.positions[: ctx.num_tokens].long()
            residual += self.params["weight"][pos].float()

    class MeanNorm(Norm):
        """Layer norm with mean and bias, in float32."""

        def __init__(self, *, hidden_size, eps):
            self.hidden_size, self.eps = hidden_size, eps

        def param_specs(self):
            return [ParamSpec("weight", (self.hidden_size,), kind="vector", init="gain"),
                    ParamSpec("bias", (self.hidden_size,), kind="vector", init="normal")]

        def forward_fused(self, out, residual, delta):
            if delta is not None:
                residual += delta.float()
            y = torch.nn.functional.layer_norm(residual, (self.hidden_size,), self.params["weight"],
                                               self.params["bias"], self.eps)
            out.copy_(y)

    class TopOneExperts(FeedForward):
        """``y = p_e * down_e(silu(up_e(x)))`` for the one expert ``e`` with the largest router
        logit (the lowest index among equals); ``p`` is the softmax of the router logits."""

        graph_safe = False  # the host looks at the routing

        def __init__(self, *, hidden_size, experts, expert_size):
            self.H, self.E, self.I = hidden_size, experts, expert_size

        def param_specs(self):
            up = tuple(ParamSource(f"experts.{e}.up.weight", e * self.I, self.I) for e in range(self.E))
            down = tuple(ParamSource(f"experts.{e}.down.weight", e * self.H, self.H) for e in range(self.E))
            return [ParamSpec("router.weight", (self.E, self.H), kind="vector"),
                    ParamSpec("up.weight", (self.E * self.I, self.H), sources=up),
                    ParamSpec("down.weight", (self.E * self.H, self.I), sources=down)]

        def forward(self, x, ctx, call):
            p = self.params
            logits = x.float() @ p["router.weight"].T  # float32 whatever the model dtype
            best = logits.max(dim=1, keepdim=True).values
            index = torch.arange(self.E, device=x.device).expand_as(logits)
            choice = torch.where(logits == best, index, self.E).min(dim=1).values
            prob = torch.softmax(logits, dim=1).gather(1, choice[:, None])
            out = torch.zeros_like(x)
            for e in range(self.E):
                rows = torch.nonzero(choice == e).flatten()
                if rows.numel() == 0:
                    continue
                xe = x.index_select(0, rows).contiguous()
                h = torch.empty(rows.numel(), self.I, dtype=x.dtype, device=x.device)
                ops.linear(h, xe, p["up.weight"][e * self.I:(e + 1) * self.I])
                h = torch.nn.functional.silu(h.float()).to(x.dtype)
                y = torch.empty(rows.numel(), self.H, dtype=x.dtype, device=x.device)
                ops.linear(y, h, p["down.weight"][e * self.H:(e + 1) * self.H])
                out.index_copy_(0, rows, (y.float() * prob[rows]).to(x.dtype))
            return out

    if "toy_top_one" not in FEED_FORWARDS.kinds():
        register_feed_forward("toy_top_one", TopOneExperts)
        register_norm("toy_mean_norm", MeanNorm)
        register_position_encoding("toy_learned_positions", LearnedPositions)

    def build_spec(c):
        H = c["hidden_size"]
        norm = PartSpec("toy_mean_norm", {"hidden_size": H, "eps": c["eps"]})
        norms = {"input_layernorm": norm, "post_attention_layernorm": norm}
        ffn = PartSpec("toy_top_one", {"hidden_size": H, "experts": c["experts"], "expert_size": c["expert_size"]})
        dense = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["expert_size"]})

        def attn(window):
            return PartSpec("paged_attention", {"hidden_size": H, "num_heads": c["heads"],
                                                "num_kv_heads": c["kv_heads"], "head_dim": c["head_dim"],
                                                "scale": c["head_dim"] ** -0.5, "window": window})

        layers = (LayerSpec("layers.0", attn(c["window"]), ffn, norms, position=0),
                  LayerSpec("layers.1", attn(0), dense, norms, position=0))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H,
                         max_position_embeddings=c["max_position_embeddings"], layers=layers,
                         final_norm=norm, embed_prefix="embed", final_norm_prefix="norm", head_prefix="head",
                         positions=(PartSpec("toy_learned_positions",
                                             {"max_positions": c["max_position_embeddings"], "hidden_size": H}),),
                         position_prefixes=("positions",))

    if "ToyRoutedForCausalLM" not in MODEL_REGISTRY:
        register_architecture("ToyRoutedForCausalLM", dict, build_spec)


def plain_forward(c, w, tokens):
    """The toy model written out in float64: whole sequence, no cache."""
    w = {k: v.double() for k, v in w.items()}
    T, H, d, nh = len(tokens), c["hidden_size"], c["head_dim"], c["heads"]

    def norm(x, p):
        return torch.nn.functional.layer_norm(x, (H,), w[f"{p}.weight"], w[f"{p}.bias"], c["eps"])

    def attention(x, p, window):
        q = (x @ w[f"{p}.q_proj.weight"].T).view(T, nh, d)
        k = (x @ w[f"{p}.k_proj.weight"].T).view(T, c["kv_heads"], d)
        v = (x @ w[f"{p}.v_proj.weight"].T).view(T, c["kv_heads"], d)
        o = plain.causal_gqa_attention(q, k, v, d ** -0.5, window=window or None)
        return o.reshape(T, -1) @ w[f"{p}.o_proj.weight"].T

    r = w["embed.weight"][torch.tensor(tokens)] + w["positions.weight"][:T]
    r = r + attention(norm(r, "layers.0.input_layernorm"), "layers.0.self_attn", c["window"])
    x = norm(r, "layers.0.post_attention_layernorm")
    logits = x @ w["layers.0.mlp.router.weight"].T
    choice = logits.argmax(dim=1)  # random weights: no ties
    prob = torch.softmax(logits, dim=1)
    y = torch.empty_like(x)
    for t in range(T):
        e = int(choice[t])
        h = torch.nn.functional.silu(w[f"layers.0.mlp.experts.{e}.up.weight"] @ x[t])
        y[t] = prob[t, e] * (w[f"layers.0.mlp.experts.{e}.down.weight"] @ h)
    r = r + y
    r = r + attention(norm(r, "layers.1.input_layernorm"), "layers.1.self_attn", 0)
    x = norm(r, "layers.1.post_attention_layernorm")
    r = r + plain.swiglu_mlp(x, w["layers.1.mlp.gate_proj.weight"], w["layers.1.mlp.up_proj.weight"],
                             w["layers.1.mlp.down_proj.weight"])
    return norm(r, "norm") @ w["head.weight"].T, choice


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_routed_toy_with_learned_positions_and_two_cache_groups(tmp_path, dtype):
    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.weights.loader import write_random_model

    register_toy()
    folder = write_random_model(tmp_path / "toy_routed", CONFIG, seed=4)
    cfg, weights = plain.load_model_folder(folder)
    # the expert weights are separate tensors in the file and stacked in the model
    assert {f"layers.0.mlp.experts.{e}.up.weight" for e in range(3)} <= set(weights)
    assert weights["layers.0.mlp.router.weight"].dtype == torch.float32
    session = TraceSession(str(folder), dtype, max_tokens=192, block_size=PAGE, poison_cache=True)
    model = session.model
    assert [(g.need.window, g.num_planes) for g in model.cache_groups] == [(16, 1), (0, 1)]
    assert not model.graph_safe()

    seqs = {"a": random_tokens(70, 83, 1), "b": random_tokens(41, 83, 2)}
    want, routes = {}, {}
    for k, v in seqs.items():
        want[k], routes[k] = plain_forward(cfg, weights, v)
    assert len(set(routes["a"].tolist())) == 3, "the tokens should visit every expert"
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)

    pos = {}
    def check(rec):
        out = session.run_step(rec)
        rows = out.logits.double().cpu()
        i = 0
        for item in rec["entries"]:
            start = pos.get(item["id"], 0)
            for w_ in item["want"]:
                assert torch.allclose(rows[i], want[item["id"]][start + w_], **tol), (item["id"], start + w_)
                i += 1
            pos[item["id"]] = start + len(item["tokens"])
        for rid in rec["end"]:
            pos.pop(rid)
        session.manager.check()

    a, b = seqs["a"], seqs["b"]
    check({"step": 0, "entries": [{"id": "a", "tokens": a[:33], "want": list(range(33))}], "end": []})
    ia, ib, k = 33, 0, 1
    for size in (2, 9, 1, 1, 7, 1, 5, 1, 1, 9):
        entries = [{"id": "a", "tokens": a[ia:ia + size], "want": list(range(size))}]
        ia += size
        nb = min(6, len(b) - ib)
        if nb:
            entries.append({"id": "b", "tokens": b[ib:ib + nb], "want": list(range(nb))}); ib += nb
        check({"step": k, "entries": entries, "end": ["a"] if ia == len(a) else []})
        k += 1
        if ia < len(a):
            # behind the window the first group's pages are gone; the second keeps them all
            window_pages, all_pages = session.manager.page_ids("a")
            gone = max(ia - 16 + 1, 0) // PAGE
            assert window_pages[:gone] == [0] * gone and all(p > 0 for p in window_pages[gone:])
            assert all(p > 0 for p in all_pages) and len(all_pages) == -(-ia // PAGE)
    assert ia == len(a)
    assert ib == len(b)  # fed to its end beside a; it still holds its pages
    window_pages, all_pages = session.manager.page_ids("b")
    assert sum(p > 0 for p in window_pages) <= 16 // PAGE + 1 and len(all_pages) == -(-len(b) // PAGE)
    session.run_step({"step": k, "entries": [], "end": ["b"]})
    assert session.manager.num_free_pages() == [session.num_pages - 1] * 2
