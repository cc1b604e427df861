"""A toy mixer whose paged cache is not keys and values: it keeps ONE compressed vector per
token (a single plane of ``latent`` numbers, in float32 whatever the model's dtype) and, in a
second layer, two planes of different widths.  The storage, its bytes a page and the pages'
poisoning all follow from what the mixer's ``CacheNeed`` says; nothing in the framework's
files changes for it."""

from __future__ import annotations

import json

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["ToyLatentForCausalLM"], "vocab_size": 89, "hidden_size": 48, "latent": 24,
    "wide": 40, "narrow": 8, "intermediate_size": 64, "eps": 1e-5, "max_position_embeddings": 128,
}
PAGE = 8


def register_toy():
    from kvcore_amd.models.spec import LayerSpec, ModelSpec
    from kvcore_amd.parts.base import MIXERS, CacheNeed, Mixer, ParamSpec, PartSpec, register_mixer
    from kvcore_amd.registry import MODEL_REGISTRY, register_architecture

    class PlaneMixer(Mixer):
        """Attention with one head over what it caches per token.  ``widths`` of one entry: the
        token's compressed vector ``c = W_0 x`` is key and value at once.  Two entries: a key
        ``W_0 x`` and a value ``W_1 x`` of different widths.  The query is ``W_q x`` (as wide as
        the key), the output ``W_o`` times the attended value."""

        graph_safe = False  # walks the requests on the host

        def __init__(self, *, hidden_size, widths, cache_dtype=None, position=None):
            self.H, self.widths = hidden_size, tuple(widths)
            self.cache_dtype = cache_dtype

        def param_specs(self):
            specs = [ParamSpec(f"down_{i}.weight", (w, self.H)) for i, w in enumerate(self.widths)]
            return specs + [ParamSpec("q.weight", (self.widths[0], self.H)),
                            ParamSpec("o.weight", (self.H, self.widths[-1]))]

        def cache_need(self):
            return CacheNeed(tuple((w,) for w in self.widths), dtype=self.cache_dtype)

        def forward(self, x, ctx, call):
            p = self.params
            group = ctx.groups[call.group_index]
            size = group.page_size
            T, R = ctx.num_tokens, ctx.num_reqs
            rows = ctx.slots[:R].long()[ctx.token_req[:T].long()]
            pos = ctx.positions[:T].long()
            cell = group.table[rows, pos // size].long() * size + pos % size  # where each token lives
            planes = []
            for i, w in enumerate(self.widths):
                plane = group.plane(call.cache_index, i, size, w)  # [pages, tokens a page, w]
                plane.view(-1, w)[cell] = (x.float() @ p[f"down_{i}.weight"].float().T).to(plane.dtype)
                planes.append(plane.view(-1, w))
            q = x.float() @ p["q.weight"].float().T
            out = torch.empty((T, self.widths[-1]), dtype=torch.float32, device=x.device)
            t = 0
            slots = ctx.slots[:R].tolist()
            for r, n in enumerate(ctx.host_query_lens):
                length = ctx.host_seq_lens[r]
                at = torch.arange(length, device=x.device)
                cells = group.table[slots[r], at // size].long() * size + at % size
                keys, values = planes[0][cells].float(), planes[-1][cells].float()
                scores = q[t:t + n] @ keys.T * self.widths[0] ** -0.5
                seen = at[None, :] <= (length - n + torch.arange(n, device=x.device))[:, None]
                out[t:t + n] = torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1) @ values
                t += n
            return (out @ p["o.weight"].float().T).to(x.dtype)

    if "toy_planes" not in MIXERS.kinds():
        register_mixer("toy_planes", PlaneMixer)

    def build_spec(c):
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": c["eps"]})
        norms = {"ln_1": norm, "ln_2": norm}
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        block = PartSpec("prenorm", {"mixer_name": "mix", "ffn_name": "ff"})
        layers = (
            LayerSpec("h.0", PartSpec("toy_planes", {"hidden_size": H, "widths": (c["latent"],),
                                                     "cache_dtype": torch.float32}), ffn, norms, block),
            LayerSpec("h.1", PartSpec("toy_planes", {"hidden_size": H, "widths": (c["narrow"], c["wide"])}),
                      ffn, norms, block),
        )
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H,
                         max_position_embeddings=c["max_position_embeddings"], layers=layers, final_norm=norm,
                         embed_prefix="embed", final_norm_prefix="norm", head_prefix="head")

    if "ToyLatentForCausalLM" not in MODEL_REGISTRY:
        register_architecture("ToyLatentForCausalLM", dict, build_spec)


def plain_forward(c, w, tokens, cache_rounding):
    """The toy model written out plainly in float64: whole sequence, no cache.  What the
    engine keeps in a cache of the model's dtype is rounded here as there (``cache_rounding[i]``
    for layer ``i``), since the mixer reads it back from the cache."""
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    r = w["embed.weight"][torch.tensor(tokens)]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for i, widths in enumerate(((c["latent"],), (c["narrow"], c["wide"]))):
        x = plain.rms_norm(r, w[f"h.{i}.ln_1.weight"], c["eps"])
        planes = [cache_rounding[i](x @ w[f"h.{i}.mix.down_{j}.weight"].T) for j in range(len(widths))]
        scores = (x @ w[f"h.{i}.mix.q.weight"].T) @ planes[0].T * widths[0] ** -0.5
        attended = torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1) @ planes[-1]
        r = r + attended @ w[f"h.{i}.mix.o.weight"].T
        x = plain.rms_norm(r, w[f"h.{i}.ln_2.weight"], c["eps"])
        r = r + plain.swiglu_mlp(x, w[f"h.{i}.ff.gate_proj.weight"], w[f"h.{i}.ff.up_proj.weight"],
                                 w[f"h.{i}.ff.down_proj.weight"])
    return plain.rms_norm(r, w["norm.weight"], c["eps"]) @ w["head.weight"].T


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_a_mixer_that_caches_one_vector_per_token(tmp_path, dtype):
    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.weights.loader import write_random_model

    register_toy()
    folder = write_random_model(tmp_path / "toy", CONFIG, seed=4)
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["ToyLatentForCausalLM"]
    cfg, weights = plain.load_model_folder(folder)
    session = TraceSession(str(folder), dtype, max_tokens=128, block_size=PAGE, poison_cache=True)
    model, runner = session.model, session.runner
    # two needs, two groups: one plane of 24 numbers in float32; a plane of 8 and one of 40
    assert [g.need.planes for g in model.cache_groups] == [((24,),), ((8,), (40,))]
    assert [g.need.dtype for g in model.cache_groups] == [torch.float32, None]
    assert [[tuple(p.shape[1:]) for p in grp.storage] for grp in runner.groups] == [
        [(session.num_pages, PAGE * 24)], [(session.num_pages, PAGE * 8), (session.num_pages, PAGE * 40)]]
    assert runner.groups[0].storage[0].dtype == torch.float32 and runner.groups[1].storage[0].dtype == dtype
    esize = torch.empty((), dtype=dtype).element_size()
    assert runner.cache_bytes() == session.num_pages * PAGE * (24 * 4 + 48 * esize)
    # poisoned from the start: every plane of every group
    assert all(torch.isnan(p).all() for grp in runner.groups for p in grp.storage)

    def as_cached(t):
        return t if dtype == torch.float32 else t.to(dtype).double()

    seqs = {"a": random_tokens(41, 89, 1), "b": random_tokens(27, 89, 2), "c": random_tokens(35, 89, 3)}
    want = {k: plain_forward(cfg, weights, v, (lambda t: t.float().double(), as_cached)) for k, v in seqs.items()}
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)

    def check(steps):
        pos = {}
        for rec in steps:
            rows = session.run_step(rec).logits.double().cpu()
            i = 0
            for item in rec["entries"]:
                start = pos.get(item["id"], 0)
                for w_ in item["want"]:
                    assert torch.allclose(rows[i], want[item["id"]][start + w_], **tol), (item["id"], start + w_)
                    i += 1
                pos[item["id"]] = start + len(item["tokens"])
            for rid in rec["end"]:
                pos.pop(rid)

    # whole; then portions beside single tokens on a pool so small (16 pages for 103 tokens of
    # three requests) that pages come back and are handed out again, poisoned in between
    check([{"step": 0, "entries": [{"id": "a", "tokens": seqs["a"], "want": list(range(41))}], "end": ["a"]}])
    a, b, c = seqs["a"], seqs["b"], seqs["c"]
    steps = [{"step": 1, "entries": [{"id": "b", "tokens": b[:20], "want": [19]}], "end": []}]
    ia, ib, k = 0, 20, 1
    for size in (7, 2, 13, 5, 2, 9, 3):
        k += 1
        entries = [{"id": "a", "tokens": a[ia:ia + size], "want": list(range(size))}]
        ia += size
        if ib < len(b):
            entries.append({"id": "b", "tokens": b[ib:ib + 1], "want": [0]})
            ib += 1
        steps.append({"step": k, "entries": entries,
                      "end": (["a"] if ia == len(a) else []) + (["b"] if ib == len(b) else [])})
    assert ia == len(a) and ib == len(b)
    steps.append({"step": k + 1, "entries": [{"id": "c", "tokens": c, "want": list(range(35))}], "end": ["c"]})
    check(steps)
    session.manager.check()
    assert session.manager.live_requests() == []

