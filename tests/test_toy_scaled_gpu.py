"""A third toy architecture, defined here alone: an embedding with a scale, a head with a
bias, a soft cap and a logit scale, a head kind of its own, and two attention layers whose
cache groups have different page sizes (32 tokens for the first, the engine's block size for
the second).  Nothing in the framework's files changes for it."""

from __future__ import annotations

import math

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["ToyScaledForCausalLM"], "vocab_size": 101, "hidden_size": 64, "heads": 4,
    "kv_heads": 2, "head_dim": 16, "intermediate_size": 96, "eps": 1e-5, "theta": 10000.0,
    "embed_scale": 8.0, "soft_cap": 0.6, "logit_scale": 0.5, "first_page_size": 32,
    "max_position_embeddings": 256,
}
PAGE = 8


def register_toy():
    from kvcore_amd.models.spec import LayerSpec, ModelSpec
    from kvcore_amd.ops import library as ops
    from kvcore_amd.parts.base import HEADS, Head, ParamSpec, PartSpec, register_head
    from kvcore_amd.registry import MODEL_REGISTRY, register_architecture

    class HalvedHead(Head):
        """A head kind of the test's own: the linear head's product, then every logit halved
        and shifted by a learned bias (float32)."""

        def __init__(self, *, vocab_size, hidden_size):
            self.V, self.H = vocab_size, hidden_size

        def param_specs(self):
            return [ParamSpec("weight", (self.V, self.H)),
                    ParamSpec("shift", (self.V,), kind="vector", init="normal")]

        def forward(self, logits, hidden_rows, ctx):
            ops.linear(logits, hidden_rows, self.params["weight"])
            ops.logits_finish(logits, self.params["shift"], 0.0, 1.0)
            logits *= 0.5

    if "toy_halved_head" not in HEADS.kinds():
        register_head("toy_halved_head", HalvedHead)

    def build_spec(c):
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": c["eps"]})
        norms = {"input_layernorm": norm, "post_attention_layernorm": norm}
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})

        def attn(page_size):
            return PartSpec("paged_attention", {"hidden_size": H, "num_heads": c["heads"],
                                                "num_kv_heads": c["kv_heads"], "head_dim": c["head_dim"],
                                                "scale": c["head_dim"] ** -0.5, "page_size": page_size})

        layers = (LayerSpec("layers.0", attn(c["first_page_size"]), ffn, norms, position=0),
                  LayerSpec("layers.1", attn(None), ffn, norms, position=0))
        if c.get("own_head"):
            head = PartSpec("toy_halved_head", {"vocab_size": c["vocab_size"], "hidden_size": H})
        else:
            head = PartSpec("linear_head", {"vocab_size": c["vocab_size"], "hidden_size": H, "bias": True,
                                            "soft_cap": c["soft_cap"], "logit_scale": c["logit_scale"]})
        return ModelSpec(
            vocab_size=c["vocab_size"], hidden_size=H, max_position_embeddings=c["max_position_embeddings"],
            layers=layers, final_norm=norm, embed_prefix="embed", final_norm_prefix="norm", head_prefix="head",
            positions=(PartSpec("rotary", {"rot_dim": c["head_dim"], "theta": c["theta"], "scaling": None}),),
            embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"], "hidden_size": H,
                                                   "scale": c["embed_scale"]}),
            head=head)

    if "ToyScaledForCausalLM" not in MODEL_REGISTRY:
        register_architecture("ToyScaledForCausalLM", dict, build_spec)


def plain_forward(c, w, tokens):
    """The toy model written out in float64 from the plain parts: whole sequence, no cache."""
    w = {k: v.double() for k, v in w.items()}
    positions = torch.arange(len(tokens))
    inv_freq = plain.rope_inv_freq(c["head_dim"], c["theta"])
    r = w["embed.weight"][torch.tensor(tokens)] * c["embed_scale"]
    for i in range(2):
        p = f"layers.{i}"
        x = plain.rms_norm(r, w[f"{p}.input_layernorm.weight"], c["eps"])
        r = r + plain.attention_block(x, positions, w, f"{p}.self_attn", num_heads=c["heads"],
                                      num_kv_heads=c["kv_heads"], head_dim=c["head_dim"], inv_freq=inv_freq)
        x = plain.rms_norm(r, w[f"{p}.post_attention_layernorm.weight"], c["eps"])
        r = r + plain.swiglu_mlp(x, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                 w[f"{p}.mlp.down_proj.weight"])
    x = plain.rms_norm(r, w["norm.weight"], c["eps"])
    logits = x @ w["head.weight"].T
    if c.get("own_head"):
        return (logits + w["head.shift"]) * 0.5
    logits = logits + w["head.bias"]
    # kvcore/sample/logits_processor.py:50-54: the soft cap first, then the scale
    logits = torch.tanh(logits / c["soft_cap"]) * c["soft_cap"]
    return logits * c["logit_scale"]


@pytest.mark.parametrize("own_head", [False, True], ids=["linear_head_options", "own_head_kind"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_scaled_embedding_head_options_and_a_second_page_size(tmp_path, dtype, own_head):
    from safetensors.torch import load_file, save_file

    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.weights.loader import write_random_model

    register_toy()
    config = dict(CONFIG, own_head=own_head)
    folder = write_random_model(tmp_path / "toy_scaled", config, seed=9)
    if not own_head:  # the random mode zeroes biases: give the head's bias values that show
        path = folder / "model.safetensors"
        tensors = load_file(str(path))
        tensors["head.bias"] = (torch.randn(config["vocab_size"], generator=torch.Generator().manual_seed(3))
                                * 0.5).to(tensors["head.bias"].dtype)
        save_file(tensors, str(path))
    cfg, weights = plain.load_model_folder(folder)
    session = TraceSession(str(folder), dtype, max_tokens=256, block_size=PAGE, poison_cache=True)
    model = session.model
    # two groups because the page sizes differ, each with its own pool, table and storage
    assert [g.need.page_size for g in model.cache_groups] == [32, None]
    assert [g.page_size for g in session.manager.groups] == [32, PAGE]
    assert [grp.page_size for grp in session.runner.groups] == [32, PAGE]
    for grp, spec, size in zip(session.runner.groups, model.cache_groups, (32, PAGE)):
        need = spec.need
        assert [p.shape[2] for p in grp.storage] == [size * n for n in need.token_elems()]
    assert session.runner.groups[0].table.shape[1] == 256 // 32
    assert session.runner.groups[1].table.shape[1] == 256 // PAGE

    seqs = {"a": random_tokens(75, cfg["vocab_size"], 1), "b": random_tokens(44, cfg["vocab_size"], 2)}
    want = {k: plain_forward(cfg, weights, v) for k, v in seqs.items()}
    if not own_head:
        assert float(want["a"].abs().max()) > 0.8 * cfg["soft_cap"] * cfg["logit_scale"], "the cap should bite"
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=4e-2, rtol=4e-2)

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
    check({"step": 0, "entries": [{"id": "a", "tokens": a[:37], "want": list(range(37))}], "end": []})
    ia, ib, k = 37, 0, 1
    for size in (2, 9, 1, 1, 7, 1, 5, 1, 1, 10):
        entries = [{"id": "a", "tokens": a[ia:ia + size], "want": list(range(size))}]
        ia += size
        nb = min(5, len(b) - ib)
        if nb:
            entries.append({"id": "b", "tokens": b[ib:ib + nb], "want": list(range(nb))}); ib += nb
        check({"step": k, "entries": entries, "end": ["a"] if ia == len(a) else []})
        k += 1
        if ia < len(a):
            big, small = session.manager.page_ids("a")
            assert len(big) == math.ceil(ia / 32) and len(small) == math.ceil(ia / PAGE)
    assert ia == len(a)
    session.run_step({"step": k, "entries": [], "end": ["b"]})
    free = session.manager.num_free_pages()
    assert free == [g.num_pages - 1 for g in session.manager.groups]
