"""A toy architecture of standard parts whose first layer attends through a window and whose
second sees everything: two cache groups, one of which gives pages back while requests run.
Generation through the engine, with decode steps captured as graphs and launched one ahead of
the host (the pages that the window passes are then given back before the step that passed
them has finished on the device), against the plain implementation and against the same
engine taking its steps one by one."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["ToyWindowForCausalLM"], "vocab_size": 200, "hidden_size": 128, "heads": 4,
    "kv_heads": 2, "head_dim": 64, "intermediate_size": 192, "eps": 1e-5, "theta": 10000.0,
    "window": 24, "max_position_embeddings": 256,
}
PAGE = 16


def register_toy():
    from kvcore_amd.models.spec import LayerSpec, ModelSpec
    from kvcore_amd.parts.base import PartSpec
    from kvcore_amd.registry import MODEL_REGISTRY, register_architecture

    def build_spec(c):
        H = c["hidden_size"]
        norm = PartSpec("rmsnorm", {"hidden_size": H, "eps": c["eps"]})
        norms = {"input_layernorm": norm, "post_attention_layernorm": norm}
        ffn = PartSpec("swiglu", {"hidden_size": H, "intermediate_size": c["intermediate_size"]})

        def attn(window):
            return PartSpec("paged_attention", {"hidden_size": H, "num_heads": c["heads"],
                                                "num_kv_heads": c["kv_heads"], "head_dim": c["head_dim"],
                                                "scale": c["head_dim"] ** -0.5, "window": window})

        layers = (LayerSpec("layers.0", attn(c["window"]), ffn, norms, position=0),
                  LayerSpec("layers.1", attn(0), ffn, norms, position=0))
        return ModelSpec(vocab_size=c["vocab_size"], hidden_size=H,
                         max_position_embeddings=c["max_position_embeddings"], layers=layers, final_norm=norm,
                         positions=(PartSpec("rotary", {"rot_dim": c["head_dim"], "theta": c["theta"]}),),
                         embed_prefix="embed", final_norm_prefix="norm", head_prefix="head")

    if "ToyWindowForCausalLM" not in MODEL_REGISTRY:
        register_architecture("ToyWindowForCausalLM", dict, build_spec)


def plain_forward(c, w, tokens):
    w = {k: v.double() for k, v in w.items()}
    T = len(tokens)
    r = w["embed.weight"][torch.tensor(tokens)]
    inv = plain.rope_inv_freq(c["head_dim"], c["theta"])
    for i, window in enumerate((c["window"], None)):
        p = f"layers.{i}"
        x = plain.rms_norm(r, w[f"{p}.input_layernorm.weight"], c["eps"])
        r = r + plain.attention_block(x, torch.arange(T), w, f"{p}.self_attn", num_heads=c["heads"],
                                      num_kv_heads=c["kv_heads"], head_dim=c["head_dim"], inv_freq=inv,
                                      window=window)
        x = plain.rms_norm(r, w[f"{p}.post_attention_layernorm.weight"], c["eps"])
        r = r + plain.swiglu_mlp(x, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                                 w[f"{p}.mlp.down_proj.weight"])
    return plain.rms_norm(r, w["norm.weight"], c["eps"]) @ w["head.weight"].T


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 5e-2)])
def test_generation_through_a_window_with_steps_launched_ahead(tmp_path, dtype, tol):
    from kvcore_amd import CacheConfig, KVCoreConfig, ModelConfig, SamplingParams, SchedulerConfig
    from kvcore_amd.engine.llm_engine import LLMEngine
    from kvcore_amd.weights.loader import write_random_model

    register_toy()
    folder = write_random_model(tmp_path / "toy_window", CONFIG, seed=12)
    cfg, weights = plain.load_model_folder(folder)
    prompts = {f"w{i}": random_tokens(n, 200, seed=900 + i) for i, n in enumerate((5, 30, 17))}
    new_tokens = 60
    outs, engines = {}, {}
    for run_ahead in (True, False):
        engine = LLMEngine(KVCoreConfig(
            model_config=ModelConfig(model=str(folder), dtype=dtype),
            # the window group needs three pages a request, the other up to six: 3 x 6 + 1
            cache_config=CacheConfig(block_size=PAGE, num_gpu_blocks=19, poison_pages=True),
            scheduler_config=SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=32,
                                             decode_run_ahead=run_ahead)))
        core = engine.engine_core
        assert [g.window for g in core.kv_manager.groups] == [CONFIG["window"], 0]
        assert core.model.graph_safe()
        reqs = [dict(request_id=rid, prompt_token_ids=p,
                     sampling_params=SamplingParams(max_tokens=new_tokens, temperature=0.0, ignore_eos=True))
                for rid, p in prompts.items()]
        for req in reqs:
            engine.add_request(req["request_id"], req["sampling_params"], prompt_token_ids=req["prompt_token_ids"])
        results, seen_released = {}, []
        while core.has_unfinished_requests():
            for o in engine.step().request_outputs:
                if o.finished:
                    results[o.request_id] = core.take_finished_output(o.request_id).output_token_ids
            for rid in core.kv_manager.live_requests():
                seen_released.append(core.kv_manager.released_counts(rid)[0])
        outs[run_ahead] = results
        engines[run_ahead] = core
        assert max(seen_released) >= 2, "the window never passed a page"
        assert core.kv_manager.num_free_pages() == [18, 18]
        core.kv_manager.check()
    assert engines[True].runner.graph_replays > 0
    assert engines[True].scheduler.num_preemptions == 0
    if dtype == "float32":
        assert outs[True] == outs[False]
    for rid, prompt in prompts.items():
        for toks in (outs[True][rid], outs[False][rid]):
            assert len(toks) == new_tokens
            ids = list(prompt)
            for index, tok in enumerate(toks):
                logits = plain_forward(cfg, weights, ids)[-1]
                gap = float(logits.max() - logits[tok])
                assert gap <= tol, f"{rid} token {index}: plain prefers {int(logits.argmax())} by {gap:.2e}"
                ids.append(tok)
