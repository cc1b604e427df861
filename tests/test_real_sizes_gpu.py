"""Two layers with the layer sizes of Llama-3-8B and its whole vocabulary of 128,256 entries,
against the plain implementation in float64: the sizes that decide which kernel runs, and
the lengths of the sums (K = 4096 and 14336, a head of 128,256 rows), are the real ones.

float32: every way of cutting the work.  bfloat16: decode steps of 70, 40, 14, 12 and 3
requests, so that each branch of the head's product (few rows, rows shared through LDS, the
vendor product below and above them) and each family of layer kernels runs, beside prompts
whose every position is compared.
"""

from __future__ import annotations

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain
from tests.test_cuts_gpu import collect, compare, mixed_trace, session_for

pytestmark = pytest.mark.gpu

CONFIG = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 2,
    "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "intermediate_size": 14336, "vocab_size": 128256, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "tie_word_embeddings": False, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192,
    "hidden_act": "silu",
}
PAGE = 16


@pytest.fixture(scope="module")
def real(tmp_path_factory):
    """The model folder (drawn on the GPU, which gives the host's bits much sooner) and the
    plain implementation's weights in float64."""
    from kvcore_amd.weights.loader import write_random_model

    folder = write_random_model(tmp_path_factory.mktemp("real_sizes"), CONFIG, seed=8, device="cuda:0")
    cfg, weights = plain.load_model_folder(folder)
    weights = {name: t.double() for name, t in weights.items()}
    return folder, cfg, weights


def oracle(cfg, weights, tokens):
    return plain.llama_forward(cfg, weights, tokens, dtype=torch.float64)


def logit_rms(expect):
    return float(torch.cat([e.flatten() for e in expect.values()]).pow(2).mean().sqrt())


def compare_rounding_noise(got, expect, row_bound=0.015, peak=6.5, what="rows of 128256"):
    """The bfloat16 bound for rows of 128,256 logits.  The engine rounds activations to
    bfloat16 (2^-9 relative, 0.11% in the root mean square) at a dozen places per layer and
    once before the head, so a row of logits carries noise of about 1% of the logits' root
    mean square (measured on this model: 0.6% at a request's first position, 0.9% on average,
    1.2% at most), normally distributed (the largest of a row's 128,256 errors is 4.6 of the
    row's deviations on average, 5.5 at most: what the normal distribution gives for so many
    samples).  The tiny models' bound of 4% per logit was made for rows of a few hundred
    logits, whose largest error is 3 deviations; here it is stated as what it means: a row's
    error is at most ``row_bound`` = 1.5% of the logits' root mean square in the root mean
    square (a slice of K left out of one product, 32 of 4,096 terms, gives 9%), and no single
    logit errs by more than ``peak`` = 6.5 times that bound (a wrong weight row gives 140%).

    Rows of a few hundred logits (the two-layer models with a small vocabulary): a row's
    error and the logits' root mean square are then each estimated from V samples and scatter
    by 1/sqrt(2V) of themselves, so their ratio scatters by 1/sqrt(V) (5% at V = 384), and it
    varies from row to row besides.  Measured over all 2,048 rows of a 2,048-token prompt at
    these widths with V = 384: mean 1.28%, standard deviation 0.11%, largest 1.71%, the same
    at every depth of context (the float32 engine agrees with the plain implementation to
    1e-6 there, so this is rounding alone).  For rows of fewer than 10,000 logits a single
    row may therefore exceed ``row_bound`` by 4/sqrt(V) of it (1.81% at V = 384; a slice of K
    left out still misses it five times over), and the mean over all compared rows must keep
    ``row_bound`` itself."""
    from tests import helpers

    assert got, "nothing was compared"
    ratios = []
    for (rid, pos), row in sorted(got.items()):
        ref = expect[rid][pos]
        assert torch.isfinite(row).all(), f"non-finite logits at {rid}:{pos}"
        scale = float(ref.pow(2).mean().sqrt())
        err = row - ref
        row_err = float(err.pow(2).mean().sqrt())
        worst = float(err.abs().max())
        allowed = row_bound * (1.0 + 4.0 / ref.numel() ** 0.5) if ref.numel() < 10000 else row_bound
        ratios.append(row_err / scale)
        helpers.note_error(f"torch.bfloat16 {what} (root mean square)", row_err / (allowed * scale), row_err)
        helpers.note_error(f"torch.bfloat16 {what} (largest)", worst / (peak * row_bound * scale), worst)
        assert row_err <= allowed * scale, (
            f"request {rid} position {pos}: the row's error is {row_err / scale:.2%} of the logits' "
            f"root mean square")
        assert worst <= peak * row_bound * scale, (
            f"request {rid} position {pos}: logit {int(err.abs().argmax())} differs by {worst:.3e} "
            f"({worst / scale:.1%} of the logits' root mean square)")
    mean = sum(ratios) / len(ratios)
    assert mean <= row_bound, f"the rows' errors are {mean:.2%} of the logits' root mean square on average"


def test_float32_engine_under_every_cut(real):
    from kvcore_amd.engine.runner import build_model

    folder, cfg, weights = real
    model = build_model(folder, torch.float32, "cuda:0")
    lens = [70, 45, 38, 52, 41, 66, 33, 60]
    seqs = {f"q{i}": random_tokens(n, cfg["vocab_size"], seed=40 + i) for i, n in enumerate(lens)}
    expect = {rid: oracle(cfg, weights, t) for rid, t in seqs.items()}
    rms = logit_rms(expect)
    dtype = torch.float32
    whole = {}
    for rid in ("q0", "q1", "q2"):
        tokens = seqs[rid]
        # each request alone and whole
        session = session_for(folder, dtype, PAGE, max_tokens=len(tokens), model=model)
        got = collect(session, [{"step": 0, "entries": [
            {"id": rid, "tokens": tokens, "want": list(range(len(tokens)))}], "end": [rid]}])
        compare(got, expect, dtype, logit_rms=rms, sum_length=CONFIG["intermediate_size"])
        whole.update(got)
        # most of it in one step, the last 32 tokens one by one
        head = len(tokens) - 32
        session = session_for(folder, dtype, PAGE, max_tokens=len(tokens), model=model)
        steps = [{"step": 0, "entries": [{"id": rid, "tokens": tokens[:head], "want": [head - 1]}], "end": []}]
        steps += [{"step": j + 1, "entries": [{"id": rid, "tokens": [tokens[head + j]], "want": [0]}], "end": []}
                  for j in range(32)]
        got = collect(session, steps)
        assert len(got) == 33
        compare(got, expect, dtype, logit_rms=rms, sum_length=CONFIG["intermediate_size"])
        for key, row in got.items():
            assert torch.equal(row, whole[key]), f"one by one: {key} is not the whole prompt's bits"
        # portions of changing size, down to two tokens
        session = session_for(folder, dtype, PAGE, max_tokens=len(tokens), model=model)
        sizes, steps, at, k = [16, 7, 2, 5, 13, 2, 3, 9], [], 0, 0
        while at < len(tokens):
            size = min(sizes[k % len(sizes)], len(tokens) - at)
            if len(tokens) - at - size == 1:
                size += 1
            steps.append({"step": k, "entries": [{"id": rid, "tokens": tokens[at:at + size],
                                                  "want": list(range(size))}], "end": []})
            at += size
            k += 1
        got = collect(session, steps)
        compare(got, expect, dtype, logit_rms=rms, sum_length=CONFIG["intermediate_size"])
        for key, row in got.items():
            assert torch.equal(row, whole[key]), f"portions: {key} is not the whole prompt's bits"
    # mixed: four live requests, portions beside single tokens, pages used again
    rounded = sorted((-(-len(t) // 64) * 64 for t in seqs.values()), reverse=True)
    session = session_for(folder, dtype, PAGE, max_tokens=sum(rounded[:4]), model=model)
    got = collect(session, mixed_trace(seqs, seed=3))
    assert len(got) == sum(len(t) for t in seqs.values())
    compare(got, expect, dtype, logit_rms=rms, sum_length=CONFIG["intermediate_size"])
    for key, row in got.items():
        if key in whole:
            assert torch.equal(row, whole[key]), f"mixed: {key} is not the whole prompt's bits"
    assert sum(-(-len(t) // PAGE) for t in seqs.values()) > session.num_pages - 1


def test_bfloat16_engine_with_every_row_count(real, monkeypatch):
    from kvcore_amd.engine.runner import build_model
    from kvcore_amd.ops import library as ops

    folder, cfg, weights = real
    model = build_model(folder, torch.bfloat16, "cuda:0")
    assert len([w for w in model.product_weights() if getattr(w, "kvc_packed", None) is not None]) == 9
    n_req = 70
    # requests in each decode step; steps of single tokens run padded to the runner's batch
    # buckets (72, 40, 14, 12, 8, 4, 4 rows: every size from 8 to 16 has one), which is what the
    # head's product sees
    live_after = [70, 40, 14, 12, 8, 3, 3]
    seqs = {}
    for i in range(n_req):
        steps_alive = sum(1 for n in live_after if i < n)
        seqs[f"r{i}"] = random_tokens(4 + i % 5 + steps_alive, cfg["vocab_size"], seed=200 + i)
    expect = {rid: oracle(cfg, weights, t) for rid, t in seqs.items()}

    head_paths = []
    real_skinny, real_mid, real_mm = ops.gemm_skinny_bf16, ops.gemm_mid, torch.mm

    def spy_skinny(out, *a, **kw):
        if out.shape[1] == cfg["vocab_size"]:
            head_paths.append(("few rows", out.shape[0]))
        return real_skinny(out, *a, **kw)

    def spy_mid(out, *a, **kw):
        if out is not None and out.shape[1] == cfg["vocab_size"]:
            head_paths.append(("rows through LDS", out.shape[0]))
        return real_mid(out, *a, **kw)

    def spy_mm(x, w, **kw):
        if w.shape[1] == cfg["vocab_size"]:
            assert kw.get("out_dtype") == torch.float32
            head_paths.append(("vendor", x.shape[0]))
        return real_mm(x, w, **kw)

    monkeypatch.setattr(ops, "gemm_skinny_bf16", spy_skinny)
    monkeypatch.setattr(ops, "gemm_mid", spy_mid)
    monkeypatch.setattr(torch, "mm", spy_mm)

    total = sum(-(-len(t) // 64) * 64 for t in seqs.values())
    session = session_for(folder, torch.bfloat16, PAGE, max_tokens=total, max_num_seqs=72, model=model)
    ids = list(seqs)
    fed = {r: len(seqs[r]) - sum(1 for n in live_after if int(r[1:]) < n) for r in ids}
    steps, k = [], 0
    # prompts, ten requests a step (60 rows for the head), the last ten as two and eight
    # (12 and 48 rows), every position compared
    groups = [ids[i:i + 10] for i in range(0, n_req - 10, 10)] + [ids[60:62], ids[62:]]
    for group in groups:
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": seqs[r][:fed[r]], "want": list(range(fed[r]))} for r in group]})
        k += 1
    for j, n in enumerate(live_after):
        live = ids[:n]
        nxt = live_after[j + 1] if j + 1 < len(live_after) else 0
        steps.append({"step": k, "end": live[nxt:], "entries": [
            {"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]} for r in live]})
        k += 1
        for r in live:
            fed[r] += 1
    got = collect(session, steps)
    assert all(fed[r] == len(seqs[r]) for r in ids)
    assert len(got) == sum(len(t) for t in seqs.values())
    compare_rounding_noise(got, expect)
    seen = set(head_paths)
    rows_12 = sum(fed_0 for fed_0 in (4 + int(r[1:]) % 5 for r in ids[60:62]))
    assert {("vendor", 72), ("rows through LDS", 40), ("vendor", 14), ("few rows", 12), ("few rows", 8),
            ("few rows", 4), ("rows through LDS", 60), ("few rows", rows_12)} <= seen, seen
    assert session.manager.live_requests() == []
