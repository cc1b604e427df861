"""A block arrangement defined here alone: the mixer and the feed-forward of a layer both
read the one normalised input and their outputs are added into the residual stream together
(a "parallel" block).  It is registered, built, loaded from a folder that the random-weights
mode wrote, stepped in cuts and mixed batches on poisoned pages, and compared with the same
arrangement written out from the plain parts.  Nothing in the framework's files changes for it."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["ToyParallelForCausalLM"], "vocab_size": 149, "hidden_size": 96, "heads": 6,
    "kv_heads": 2, "head_dim": 16, "intermediate_size": 160, "eps": 2e-6, "theta": 50000.0,
    "num_layers": 3, "max_position_embeddings": 256,
}
PAGE = 16


def register_toy():
    from kvcore_amd.models.spec import LayerSpec, ModelSpec
    from kvcore_amd.parts.base import BLOCKS, Block, PartSpec, register_block
    from kvcore_amd.registry import MODEL_REGISTRY, register_architecture

    class ParallelBlock(Block):
        """``r += delta; x = ln(r); pending = mixer(x) + ffn(x)``: one norm a layer, and the
        sum of both branches left pending for the next block's norm."""

        def children(self):
            return {"ln": self.norms["ln"], "attn": self.mixer, "mlp": self.ffn}

        def forward(self, delta, residual, ctx, call, next_block=None):
            width = residual.shape[1]
            x = ctx.buf("parallel_x", width)
            self.norms["ln"].forward_fused(x, residual, delta)
            a = self.mixer.forward(x, ctx, call)
            f = self.ffn.forward(x, ctx, call)
            both = ctx.buf("parallel_sum", width)
            torch.add(a, f, out=both)
            return both

    if "toy_parallel" not in BLOCKS.kinds():
        register_block("toy_parallel", ParallelBlock)

    def build_spec(c):
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": c["eps"]})
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})
        attn = PartSpec("paged_attention", {"hidden_size": H, "num_heads": c["heads"], "num_kv_heads": c["kv_heads"],
                                            "head_dim": c["head_dim"], "scale": c["head_dim"] ** -0.5})
        layers = tuple(LayerSpec(f"h.{i}", attn, ffn, {"ln": norm}, block=PartSpec("toy_parallel"), position=0)
                       for i in range(c["num_layers"]))
        return ModelSpec(
            vocab_size=c["vocab_size"], hidden_size=H, max_position_embeddings=c["max_position_embeddings"],
            layers=layers, final_norm=norm, embed_prefix="wte", final_norm_prefix="ln_f", head_prefix="head",
            positions=(PartSpec("rotary", {"rot_dim": c["head_dim"], "theta": c["theta"], "scaling": None}),))

    if "ToyParallelForCausalLM" not in MODEL_REGISTRY:
        register_architecture("ToyParallelForCausalLM", dict, build_spec)


def plain_forward(c, w, tokens, dtype):
    """The arrangement from the plain parts: whole sequence, no cache.  In bfloat16 the two
    branches are rounded before they are added, and their sum once more, as the block's
    buffers do."""
    w = {k: v.double() for k, v in w.items()}
    positions = torch.arange(len(tokens))
    inv_freq = plain.rope_inv_freq(c["head_dim"], c["theta"])

    def rounded(t):
        return t.to(dtype).double() if dtype == torch.bfloat16 else t

    r = w["wte.weight"][torch.tensor(tokens)]
    for i in range(c["num_layers"]):
        p = f"h.{i}"
        x = rounded(plain.rms_norm(r, w[f"{p}.ln.weight"], c["eps"]))
        a = plain.attention_block(x, positions, w, f"{p}.attn", num_heads=c["heads"], num_kv_heads=c["kv_heads"],
                                  head_dim=c["head_dim"], inv_freq=inv_freq)
        f = plain.swiglu_mlp(x, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                             w[f"{p}.mlp.down_proj.weight"])
        r = r + rounded(rounded(a) + rounded(f))
    x = plain.rms_norm(r, w["ln_f.weight"], c["eps"])
    return x @ w["head.weight"].T


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_a_block_arrangement_of_the_tests_own(tmp_path, dtype):
    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.weights.loader import write_random_model

    register_toy()
    folder = write_random_model(tmp_path / "toy_parallel", CONFIG, seed=17)
    cfg, weights = plain.load_model_folder(folder)
    assert sorted(k for k in weights if k.startswith("h.1.")) == [
        "h.1.attn.k_proj.weight", "h.1.attn.o_proj.weight", "h.1.attn.q_proj.weight", "h.1.attn.v_proj.weight",
        "h.1.ln.weight", "h.1.mlp.down_proj.weight", "h.1.mlp.gate_proj.weight", "h.1.mlp.up_proj.weight"]
    session = TraceSession(str(folder), dtype, max_tokens=192, block_size=PAGE, poison_cache=True)
    assert [type(b).__name__ for b in session.model.blocks] == ["ParallelBlock"] * 3

    seqs = {k: random_tokens(n, cfg["vocab_size"], seed) for k, n, seed in (("a", 70, 1), ("b", 41, 2), ("c", 58, 3))}
    want = {k: plain_forward(cfg, weights, v, dtype) for k, v in seqs.items()}
    tol = dict(atol=2e-5, rtol=1e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=3e-2)
    fed = {}

    def check(step, entries, end=()):
        rec = {"step": step, "end": list(end), "entries": [
            {"id": rid, "tokens": seqs[rid][fed.get(rid, 0):fed.get(rid, 0) + n], "want": list(range(n))}
            for rid, n in entries]}
        rows = session.run_step(rec).logits.double().cpu()
        i = 0
        for rid, n in entries:
            start = fed.get(rid, 0)
            for j in range(n):
                assert torch.allclose(rows[i], want[rid][start + j], **tol), (rid, start + j)
                i += 1
            fed[rid] = start + n
        session.manager.check()

    # a whole prompt, then portions beside single tokens, then "a" ends and "c" takes its pages
    check(0, [("a", 33)])
    check(1, [("a", 1), ("b", 17)])
    check(2, [("a", 2), ("b", 1)])
    check(3, [("a", 1), ("b", 9)])
    for k in range(4, 16):
        check(k, [("a", 1), ("b", 1)])
    check(16, [("a", 70 - fed["a"]), ("b", 1)], end=["a"])
    held = set(session.manager.page_ids("b")[0])
    check(17, [("c", 40), ("b", 1)])
    assert set(session.manager.page_ids("c")[0]).isdisjoint(held)
    for k in range(18, 18 + 41 - fed["b"]):
        check(k, [("c", 1), ("b", 1)])
    assert fed["b"] == 41
    check(99, [("c", 58 - fed["c"])], end=["b", "c"])
    assert session.manager.num_free_pages() == [g.num_pages - 1 for g in session.manager.groups]
