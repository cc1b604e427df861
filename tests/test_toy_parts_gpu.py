"""A toy mixer with state of its own, a toy architecture that uses it beside attention,
a schedule that names a layer twice and lets a layer read another's cache: all defined
here, registered, built and stepped without a change to the framework's files."""

from __future__ import annotations

import json

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

TOY_CONFIG = {
    "architectures": ["ToyStateForCausalLM"], "vocab_size": 97, "hidden_size": 32, "heads": 2,
    "head_dim": 16, "intermediate_size": 48, "eps": 1e-5, "decay": 0.75, "max_position_embeddings": 256,
}


def register_toy():
    from kvcore_amd.models.spec import LayerSpec, ModelSpec, ScheduleEntry
    from kvcore_amd.parts.base import MIXERS, Mixer, ParamSpec, PartSpec, StateNeed, register_mixer
    from kvcore_amd.registry import MODEL_REGISTRY, register_architecture

    class DecayMixer(Mixer):
        """y_t = W s_t with s_t = decay * s_{t-1} + x_t per request: the state s is the
        mixer's own, one row per request slot, carried across steps."""

        graph_safe = False  # loops over requests on the host

        def __init__(self, *, hidden_size, decay, position=None):
            self.hidden_size, self.decay = hidden_size, decay

        def param_specs(self):
            return [ParamSpec("mix.weight", (self.hidden_size, self.hidden_size))]

        def state_need(self):
            return StateNeed((self.hidden_size,), torch.float32)

        def forward(self, x, ctx, call):
            state = ctx.states[call.state_index]
            slots = ctx.slots[: ctx.num_reqs].tolist()
            out = torch.empty_like(x)
            t = 0
            for r, n in enumerate(ctx.host_query_lens):
                s = state[slots[r]]
                if ctx.host_seq_lens[r] == n:  # the request starts here: fresh state
                    s.zero_()
                for i in range(n):
                    s.mul_(self.decay).add_(x[t + i].float())
                    out[t + i] = (self.params["mix.weight"].float() @ s).to(x.dtype)
                t += n
            return out

    if "toy_decay" not in MIXERS.kinds():
        register_mixer("toy_decay", DecayMixer)

    def parse(d):
        return dict(d)

    def build_spec(c):
        norm = PartSpec("rmsnorm", {"hidden_size": c["hidden_size"], "eps": c["eps"]})
        norms = {"input_layernorm": norm, "post_attention_layernorm": norm}
        ffn = PartSpec("swiglu", {"hidden_size": c["hidden_size"], "intermediate_size": c["intermediate_size"]})
        attn = PartSpec("paged_attention", {"hidden_size": c["hidden_size"], "num_heads": c["heads"],
                                            "num_kv_heads": 1, "head_dim": c["head_dim"], "scale": 0.25})
        toy = PartSpec("toy_decay", {"hidden_size": c["hidden_size"], "decay": c["decay"]})
        layers = (
            LayerSpec("layers.0", toy, ffn, norms, PartSpec("prenorm", {"mixer_name": "mixer"})),
            LayerSpec("layers.1", attn, ffn, norms, position=0),
            LayerSpec("layers.2", attn, ffn, norms, position=0),
        )
        # layer 0 runs twice (two states); the last entry reads the cache entry 1 wrote
        schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(2, cache_from=1))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
                         max_position_embeddings=c["max_position_embeddings"], layers=layers,
                         final_norm=norm, positions=(PartSpec("rotary", {"rot_dim": c["head_dim"], "theta": 100.0}),),
                         schedule=schedule, embed_prefix="embed", final_norm_prefix="norm", head_prefix="head")

    if "ToyStateForCausalLM" not in MODEL_REGISTRY:
        register_architecture("ToyStateForCausalLM", parse, build_spec)


def plain_toy_forward(c, w, tokens):
    """The toy model written out plainly in float64 (whole sequence, no cache)."""
    w = {k: v.double() for k, v in w.items()}
    T, H, d, nh = len(tokens), c["hidden_size"], c["head_dim"], c["heads"]
    r = w["embed.weight"][torch.tensor(tokens)]
    pos = torch.arange(T)
    inv = plain.rope_inv_freq(d, 100.0)

    def ffn(x, p):
        return plain.swiglu_mlp(x, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                w[f"{p}.mlp.down_proj.weight"])

    def toy_layer(r):
        x = plain.rms_norm(r, w["layers.0.input_layernorm.weight"], c["eps"])
        s = torch.zeros(H, dtype=torch.float64)
        y = torch.empty_like(x)
        for t in range(T):
            s = c["decay"] * s + x[t]
            y[t] = w["layers.0.mixer.mix.weight"] @ s
        r = r + y
        return r + ffn(plain.rms_norm(r, w["layers.0.post_attention_layernorm.weight"], c["eps"]), "layers.0")

    def qkv(x, p):
        q = (x @ w[f"{p}.self_attn.q_proj.weight"].T).view(T, nh, d)
        k = (x @ w[f"{p}.self_attn.k_proj.weight"].T).view(T, 1, d)
        v = (x @ w[f"{p}.self_attn.v_proj.weight"].T).view(T, 1, d)
        return plain.apply_rope(q, pos, inv), plain.apply_rope(k, pos, inv), v

    r = toy_layer(r)
    x = plain.rms_norm(r, w["layers.1.input_layernorm.weight"], c["eps"])
    q1, k1, v1 = qkv(x, "layers.1")
    r = r + plain.causal_gqa_attention(q1, k1, v1, 0.25).reshape(T, -1) @ w["layers.1.self_attn.o_proj.weight"].T
    r = r + ffn(plain.rms_norm(r, w["layers.1.post_attention_layernorm.weight"], c["eps"]), "layers.1")
    r = toy_layer(r)
    x = plain.rms_norm(r, w["layers.2.input_layernorm.weight"], c["eps"])
    q2, _, _ = qkv(x, "layers.2")  # its own queries over layer 1's keys and values
    r = r + plain.causal_gqa_attention(q2, k1, v1, 0.25).reshape(T, -1) @ w["layers.2.self_attn.o_proj.weight"].T
    r = r + ffn(plain.rms_norm(r, w["layers.2.post_attention_layernorm.weight"], c["eps"]), "layers.2")
    return plain.rms_norm(r, w["norm.weight"], c["eps"]) @ w["head.weight"].T


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_toy_architecture_with_state_is_registered_built_and_stepped(tmp_path, dtype):
    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.weights.loader import write_random_model

    register_toy()
    folder = write_random_model(tmp_path / "toy", TOY_CONFIG, seed=9)
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["ToyStateForCausalLM"]
    cfg, weights = plain.load_model_folder(folder)
    session = TraceSession(str(folder), dtype, max_tokens=256, block_size=8, poison_cache=True)
    model = session.model
    assert [c.layer_index for c in model.calls] == [0, 1, 0, 2]
    assert [c.state_index for c in model.calls] == [0, None, 1, None]  # a state per execution
    assert [(c.cache_index, c.write_cache) for c in model.calls] == [(None, True), (0, True), (None, True), (0, False)]
    assert len(model.cache_groups) == 1 and model.cache_groups[0].num_planes == 1
    assert len(session.runner.states) == 2

    seqs = {"a": random_tokens(45, 97, 1), "b": random_tokens(30, 97, 2)}
    want = {k: plain_toy_forward(cfg, weights, v) for k, v in seqs.items()}
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)

    def check(steps):
        pos = {}
        for rec in steps:
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

    # whole; then portions of one beside single tokens of the other, so that state and cache
    # cross step boundaries and the slot of a finished request is taken again
    check([{"step": 0, "entries": [{"id": "a", "tokens": seqs["a"], "want": list(range(45))}], "end": ["a"]}])
    steps, ia, ib, k = [], 0, 0, 0
    a, b = seqs["a"], seqs["b"]
    steps.append({"step": k, "entries": [{"id": "b", "tokens": b[:20], "want": [19]}], "end": []}); ib = 20
    for size in (7, 2, 13, 5, 2, 9, 7):
        k += 1
        entries = [{"id": "a", "tokens": a[ia:ia + size], "want": list(range(size))}]
        ia += size
        if ib < len(b):
            entries.append({"id": "b", "tokens": b[ib:ib + 1], "want": [0]}); ib += 1
        steps.append({"step": k, "entries": entries, "end": ["a"] if ia == len(a) else []})
    assert ia == len(a)
    check(steps)
