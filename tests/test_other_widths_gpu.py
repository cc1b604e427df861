"""One layer at the layer sizes of the two other Llama 3 shapes that the engine is measured
on, against the plain implementation in float64, in float32 and in bfloat16:

* Llama-3.2-1B: hidden 2,048, 32 heads over 8 kv heads of 64, feed-forward 8,192, rope factor
  32, and the head TIED to an embedding of the whole vocabulary of 128,256 (the only real
  tied case);
* Llama-3.1-70B: hidden 8,192, 64 heads over 8 kv heads of 128 (eight query heads a kv
  head), feed-forward 28,672 (the longest sum of any product here), vocabulary 384.

Whole prompts of 70 to 300 tokens with every position compared, decode steps of 70, 40, 12
and 3 requests (each family of kernels for few rows, a few dozen rows and many), and a step
that mixes a portion of a prompt with single tokens.

Reference formulas: kvcore/model/attn_backend/torch_paged.py:90-117,
kvcore/model/models/llama3.py:189-200 and :224-225 (the tied head).
"""

from __future__ import annotations

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain
from tests.test_cuts_gpu import collect, compare, session_for
from tests.test_real_sizes_gpu import CONFIG as LAYERS_OF_8B, compare_rounding_noise, logit_rms

pytestmark = pytest.mark.gpu

PAGE = 16
SHAPES = {
    "1b": dict(LAYERS_OF_8B, num_hidden_layers=1, hidden_size=2048, num_attention_heads=32,
               num_key_value_heads=8, head_dim=64, intermediate_size=8192, vocab_size=128256,
               rope_scaling=dict(LAYERS_OF_8B["rope_scaling"], factor=32.0), tie_word_embeddings=True),
    "70b": dict(LAYERS_OF_8B, num_hidden_layers=1, hidden_size=8192, num_attention_heads=64,
                num_key_value_heads=8, head_dim=128, intermediate_size=28672, vocab_size=384),
}
LIVE_AFTER = [70, 40, 12, 3]  # requests in each decode step


def trace(cfg):
    """Token lists and step records: two whole prompts, prompts of 70 short requests ten a
    step, decode steps of 70, 40, 12 and 3 of them, and a last step in which the second half
    of a prompt runs beside the last single tokens."""
    vocab = cfg["vocab_size"]
    seqs = {"w0": random_tokens(70, vocab, seed=300), "w1": random_tokens(300, vocab, seed=301),
            "h": random_tokens(90, vocab, seed=302)}
    n_req = LIVE_AFTER[0]
    for i in range(n_req):
        alive = sum(1 for n in LIVE_AFTER if i < n) + (1 if i < 3 else 0)  # the first three go one step on
        seqs[f"r{i}"] = random_tokens(3 + i % 4 + alive, vocab, seed=310 + i)
    steps, k = [], 0
    for rid in ("w0", "w1"):
        steps.append({"step": k, "entries": [{"id": rid, "tokens": seqs[rid], "want": list(range(len(seqs[rid])))}],
                      "end": [rid]})
        k += 1
    ids = [f"r{i}" for i in range(n_req)]
    fed = {r: 3 + int(r[1:]) % 4 for r in ids}
    for lo in range(0, n_req, 10):
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": seqs[r][:fed[r]], "want": list(range(fed[r]))} for r in ids[lo:lo + 10]]})
        k += 1
    steps.append({"step": k, "end": [], "entries": [{"id": "h", "tokens": seqs["h"][:41], "want": [40]}]})
    k += 1
    for j, n in enumerate(LIVE_AFTER):
        live = ids[:n]
        nxt = LIVE_AFTER[j + 1] if j + 1 < len(LIVE_AFTER) else 3
        steps.append({"step": k, "end": live[nxt:], "entries": [
            {"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]} for r in live]})
        k += 1
        for r in live:
            fed[r] += 1
    # mixed: the rest of "h" (49 tokens, from the middle of a page) beside three single tokens
    entries = [{"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]} for r in ids[:3]]
    entries.insert(1, {"id": "h", "tokens": seqs["h"][41:], "want": list(range(49))})
    steps.append({"step": k, "end": ids[:3] + ["h"], "entries": entries})
    for r in ids[:3]:
        fed[r] += 1
    assert all(fed[r] == len(seqs[r]) for r in ids)
    return seqs, steps


@pytest.fixture(scope="module", params=sorted(SHAPES))
def shape(request, tmp_path_factory):
    from kvcore_amd.weights.loader import write_random_model

    name = request.param
    folder = write_random_model(tmp_path_factory.mktemp(f"widths_{name}"), SHAPES[name], seed=31, device="cuda:0")
    cfg, weights = plain.load_model_folder(folder)
    assert ("lm_head.weight" in weights) == (name != "1b")  # the 1B shape's head is the embedding
    weights = {n: t.double() for n, t in weights.items()}
    seqs, steps = trace(cfg)
    expect = {rid: plain.llama_forward(cfg, weights, toks, dtype=torch.float64) for rid, toks in seqs.items()}
    return name, folder, cfg, seqs, steps, expect


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_one_layer_of_the_other_shapes(shape, dtype, monkeypatch):
    from kvcore_amd.engine.runner import build_model
    from kvcore_amd.ops import library as ops

    name, folder, cfg, seqs, steps, expect = shape
    model = build_model(folder, dtype, "cuda:0")
    if name == "1b":
        assert model.head.tied and model.head.params["weight"] is model.embed.params["weight"]
    ran = set()
    for fn in ("gemm_skinny_bf16", "gemm_mid", "_fused_skinny", "decode_attention", "prefill_attention",
               "paged_attention", "gemm_f32"):
        real = getattr(ops, fn)

        def spy(*a, _real=real, _fn=fn, **kw):
            ran.add(_fn)
            return _real(*a, **kw)

        monkeypatch.setattr(ops, fn, spy)
    total = sum(-(-len(t) // 64) * 64 for t in seqs.values())
    session = session_for(folder, dtype, PAGE, max_tokens=total, max_num_seqs=72, model=model)
    got = collect(session, steps)
    assert len(got) == sum(len(t) for rid, t in seqs.items() if rid != "h") + 50
    if dtype == torch.float32:
        compare(got, expect, dtype, logit_rms=logit_rms(expect), sum_length=cfg["intermediate_size"])
        assert {"gemm_f32", "paged_attention"} <= ran and not ran & {"gemm_skinny_bf16", "gemm_mid", "_fused_skinny"}
    else:
        compare_rounding_noise(got, expect, what=f"rows at {name} widths")
        # every family of bfloat16 kernels ran: few rows with the norms folded in, a few dozen
        # rows shared through LDS, single tokens and portions on the matrix cores
        assert {"gemm_skinny_bf16", "gemm_mid", "_fused_skinny", "decode_attention", "prefill_attention"} <= ran, ran
    assert session.manager.live_requests() == []


def test_partial_packing_takes_the_matrices_whose_rows_collide_and_changes_no_bit(tmp_path):
    """A model that has no room for packed copies of all its matrices (the 70B shape on one
    device) packs those whose rows lie a multiple of 16 KB apart, whole shapes at a time, the
    small shapes first, within a budget.  One layer at the 70B widths with room for 320 MB: the
    head (384 x 8192), o_proj (8192 x 8192) and qkv_proj (10240 x 8192) are packed, gate_up
    (57344 x 8192) does not fit, down_proj (8192 x 28672, rows 56 KB apart) does not qualify.
    The logits are the bits of the model without any packed copy, and of the one with all:
    a prompt of 40 rows and single tokens, which take the same kernels with and without a packed
    copy (at 17 to 32 rows and beyond 64 a matrix without one goes to the vendor's product,
    whose sums round differently)."""
    from kvcore_amd.engine.runner import build_model
    from kvcore_amd.weights.loader import write_random_model

    cfg = SHAPES["70b"]
    folder = write_random_model(tmp_path / "w70", cfg, seed=5, device="cuda:0")
    tokens = random_tokens(50, cfg["vocab_size"], seed=9)
    steps = [{"step": 0, "entries": [{"id": "r", "tokens": tokens[:40], "want": [39]}], "end": []}]
    steps += [{"step": i + 1, "entries": [{"id": "r", "tokens": [tokens[40 + i]], "want": [0]}], "end": []}
              for i in range(10)]
    rows = {}
    for mode in ("none", "partial", "all"):
        model = build_model(folder, torch.bfloat16, "cuda:0", pack_weights={"none": False, "all": True}.get(mode))
        if mode == "partial":
            taken = model.pack_product_weights(None, budget=320 << 20)
            packed = sorted(tuple(w.shape) for w in model.product_weights() if getattr(w, "kvc_packed", None) is not None)
            assert packed == [(384, 8192), (8192, 8192), (10240, 8192)], packed
            assert taken == 2 * (384 + 8192 + 10240) * 8192
        else:
            count = sum(getattr(w, "kvc_packed", None) is not None for w in model.product_weights())
            assert count == (5 if mode == "all" else 0)
        session = session_for(folder, torch.bfloat16, PAGE, max_tokens=64, model=model)
        rows[mode] = collect(session, steps)
    assert len(rows["none"]) == 11
    for key, row in rows["none"].items():
        assert torch.equal(row, rows["partial"][key]) and torch.equal(row, rows["all"][key]), key
