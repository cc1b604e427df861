"""The engine against the plain implementation under every way of cutting the work."""

from __future__ import annotations

import pytest
import torch

from tests.helpers import CONFIGS, make_model_dir, random_tokens, tolerance
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (config, page) in CONFIGS.items():
        folder = make_model_dir(tmp_path_factory.mktemp(f"tiny_{name}"), config, seed=11 + len(name))
        cfg, weights = plain.load_model_folder(folder)
        out[name] = (folder, cfg, weights, page)
    return out


_oracle_cache: dict = {}


def oracle(name, cfg, weights, tokens):
    key = (name, tuple(tokens))
    if key not in _oracle_cache:
        _oracle_cache[key] = plain.llama_forward(cfg, weights, tokens, dtype=torch.float64)
    return _oracle_cache[key]


def session_for(folder, dtype, page, max_tokens, **kw):
    from kvcore_amd.engine.replay import TraceSession

    return TraceSession(str(folder), dtype, max_tokens=max_tokens, block_size=page,
                        poison_cache=True, **kw)


def collect(session, steps):
    """Run step records; return {(id, position): logits row (float64 CPU)}."""
    got = {}
    starts = {}
    for rec in steps:
        offsets = {}
        for item in rec["entries"]:
            offsets[item["id"]] = starts.get(item["id"], 0)
        out = session.run_step(rec)
        if out is not None and out.logits is not None:
            rows = out.logits.detach().cpu().double()
            i = 0
            for item in rec["entries"]:
                for w in item.get("want", []):
                    got[(item["id"], offsets[item["id"]] + w)] = rows[i]
                    i += 1
            assert i == rows.shape[0]
        for item in rec["entries"]:
            starts[item["id"]] = offsets[item["id"]] + len(item["tokens"])
        for rid in rec.get("end", []):
            starts.pop(rid, None)
        session.manager.check()
    return got


def compare(got, expect_by_id, dtype, logit_rms=None, sum_length=0):
    tol = tolerance(dtype, sum_length=sum_length) if logit_rms is None else tolerance(dtype, logit_rms, sum_length)
    assert got, "nothing was compared"
    from tests import helpers
    for (rid, pos), row in sorted(got.items()):
        ref = expect_by_id[rid][pos]
        assert torch.isfinite(row).all(), f"non-finite logits at {rid}:{pos}"
        err = (row - ref).abs()
        bound = tol["atol"] + tol["rtol"] * ref.abs()
        helpers.note_error(str(dtype), float((err / bound).max()), float(err.max()))
        if not (err <= bound).all():
            worst = int(torch.argmax(err - bound))
            raise AssertionError(
                f"request {rid} position {pos}: logit {worst} differs by {err[worst]:.3e} "
                f"(engine {row[worst]:.6f}, plain {ref[worst]:.6f})")


PROMPT_LENS = {"A": [7, 16, 33, 50], "B": [1, 9, 24, 40, 61], "C": [5, 32, 47, 90], "D": [3, 31, 64, 150]}
EXTRA = 34  # tokens after the prompt, so that 32 of them can be decoded one by one


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_requests_alone(models, name, dtype):
    folder, cfg, weights, page = models[name]
    for i, n in enumerate(PROMPT_LENS[name]):
        tokens = random_tokens(n + EXTRA, cfg["vocab_size"], seed=100 + i)
        session = session_for(folder, dtype, page, max_tokens=len(tokens))
        got = collect(session, [{"step": 0, "entries": [
            {"id": "r", "tokens": tokens, "want": list(range(len(tokens)))}], "end": ["r"]}])
        compare(got, {"r": oracle(name, cfg, weights, tokens)}, dtype)
        assert session.manager.num_free_pages()[0] == session.num_pages - 1


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_prefill_then_decode_one_by_one(models, name, dtype):
    folder, cfg, weights, page = models[name]
    for i, n in enumerate(PROMPT_LENS[name]):
        tokens = random_tokens(n + EXTRA, cfg["vocab_size"], seed=200 + i)
        head = len(tokens) - 32
        session = session_for(folder, dtype, page, max_tokens=len(tokens))
        steps = [{"step": 0, "entries": [{"id": "r", "tokens": tokens[:head], "want": [head - 1]}], "end": []}]
        for j in range(32):
            steps.append({"step": j + 1, "entries": [{"id": "r", "tokens": [tokens[head + j]], "want": [0]}],
                          "end": ["r"] if j == 31 else []})
        got = collect(session, steps)
        assert len(got) == 33
        compare(got, {"r": oracle(name, cfg, weights, tokens)}, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_portions_of_changing_size(models, name, dtype):
    folder, cfg, weights, page = models[name]
    sizes = [16, 7, 2, 5, 13, 2, 3, 9, 2, 11, 4, 2]
    for i, n in enumerate(PROMPT_LENS[name][1:]):
        tokens = random_tokens(n + EXTRA, cfg["vocab_size"], seed=300 + i)
        session = session_for(folder, dtype, page, max_tokens=len(tokens))
        steps, at, k = [], 0, 0
        while at < len(tokens):
            size = min(sizes[k % len(sizes)], len(tokens) - at)
            if len(tokens) - at - size == 1:  # never leave a single token: portions go down to two
                size += 1
            steps.append({"step": k, "entries": [{"id": "r", "tokens": tokens[at:at + size],
                                                  "want": list(range(size))}], "end": []})
            at += size
            k += 1
        got = collect(session, steps)
        assert len(got) == len(tokens)
        compare(got, {"r": oracle(name, cfg, weights, tokens)}, dtype)


def mixed_trace(token_lists, seed):
    """Up to four live requests: portions of some beside single tokens of others; a
    request may sit a step out; finished ones make room for the next."""
    import random

    rng = random.Random(seed)
    waiting = list(token_lists.items())
    live: dict[str, int] = {}
    steps = []
    k = 0
    while waiting or live:
        while waiting and len(live) < 4:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            tokens = token_lists[rid]
            at = live[rid]
            if rng.random() < 0.15 and len(live) > 1:
                continue  # sits this step out
            remaining = len(tokens) - at
            prompt_left = remaining - 32
            if prompt_left > 0:
                size = min(prompt_left, rng.choice([2, 3, 5, 8, 13, 21]))
                if prompt_left - size == 1:
                    size += 1
            else:
                size = 1
            entries.append({"id": rid, "tokens": tokens[at:at + size], "want": list(range(size))})
            live[rid] = at + size
            if live[rid] == len(tokens):
                end.append(rid)
                del live[rid]
        if entries:
            rng.shuffle(entries)
            steps.append({"step": k, "entries": entries, "end": end})
            k += 1
    return steps


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_mixed_batches_with_page_reuse(models, name, dtype):
    folder, cfg, weights, page = models[name]
    base = PROMPT_LENS[name]
    lens = base + [n + 3 for n in base] + [base[-1] + 17, base[0] + 1]
    token_lists = {f"q{i}": random_tokens(n + EXTRA, cfg["vocab_size"], seed=400 + i) for i, n in enumerate(lens)}
    rounded = sorted((-(-len(t) // 64) * 64 for t in token_lists.values()), reverse=True)
    max_tokens = sum(rounded[:4])  # the four largest live at once; the rest must reuse pages
    session = session_for(folder, dtype, page, max_tokens=max_tokens)
    steps = mixed_trace(token_lists, seed=5)
    used_pages = set()
    got = {}
    starts = {}
    for rec in steps:
        got.update(collect_one(session, rec, starts))
        for rid in session.manager.live_requests():
            used_pages.update(p for p in session.manager.page_ids(rid)[0] if p)
    total_needed = sum(-(-len(t) // page) for t in token_lists.values())
    assert total_needed > session.num_pages - 1, "the trace must not fit without reuse"
    expect = {rid: oracle(name, cfg, weights, t) for rid, t in token_lists.items()}
    assert len(got) == sum(len(t) for t in token_lists.values())
    compare(got, expect, dtype)
    assert session.manager.num_free_pages()[0] == session.num_pages - 1


def test_mixed_batches_with_the_keys_of_a_tile_dealt_to_several_blocks(models, monkeypatch):
    """Portions of prompts that meet many keys have each tile's keys dealt to several blocks,
    joined by a second kernel.  The tiny models' contexts are short, so the number of keys a
    block should at least have is lowered until the mixed trace runs that way."""
    from kvcore_amd.ops import library as ops
    from kvcore_amd.parts import attention

    monkeypatch.setattr(attention, "PREFILL_MIN_KEYS", 48)
    calls = []
    real = ops.prefill_attention

    def spy(*args, **kw):
        calls.append(kw.get("nsplit", 1))
        return real(*args, **kw)

    monkeypatch.setattr(ops, "prefill_attention", spy)
    name = "D"  # the tiny model whose head size the kernel for portions of prompts serves
    folder, cfg, weights, page = models[name]
    base = PROMPT_LENS[name]
    lens = base + [base[-1] + 17, base[0] + 1]
    token_lists = {f"q{i}": random_tokens(n + EXTRA, cfg["vocab_size"], seed=450 + i) for i, n in enumerate(lens)}
    rounded = sorted((-(-len(t) // 64) * 64 for t in token_lists.values()), reverse=True)
    session = session_for(folder, torch.bfloat16, page, max_tokens=sum(rounded[:4]))
    got, starts = {}, {}
    for rec in mixed_trace(token_lists, seed=6):
        got.update(collect_one(session, rec, starts))
    assert max(calls) > 1 and min(calls) == 1, "the trace should run with and without splits"
    compare(got, {rid: oracle(name, cfg, weights, t) for rid, t in token_lists.items()}, torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
def test_logits_do_not_depend_on_which_pages_are_used(models, dtype):
    """The mixed trace again with the free pages handed out in a shuffled order: the same
    bits at every position, since only the place in the cache changes, not the arithmetic."""
    folder, cfg, weights, page = models["D"]
    base = PROMPT_LENS["D"]
    lens = base + [n + 3 for n in base]
    token_lists = {f"q{i}": random_tokens(n + EXTRA, cfg["vocab_size"], seed=600 + i) for i, n in enumerate(lens)}
    rounded = sorted((-(-len(t) // 64) * 64 for t in token_lists.values()), reverse=True)
    steps = mixed_trace(token_lists, seed=9)
    results, orders = [], []
    for shuffle in (None, 3):
        session = session_for(folder, dtype, page, max_tokens=sum(rounded[:4]), shuffle_pages=shuffle)
        got, starts, first_pages = {}, {}, []
        for rec in steps:
            got.update(collect_one(session, rec, starts))
            if not first_pages:
                first_pages = [p for rid in session.manager.live_requests()
                               for p in session.manager.page_ids(rid)[0]]
        results.append(got)
        orders.append(first_pages)
    assert orders[0] != orders[1], "the shuffle did not change the pages"
    assert results[0].keys() == results[1].keys()
    for key, row in results[0].items():
        assert torch.equal(row, results[1][key]), key


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_float32_logits_are_the_same_bits_under_every_cut(models, name):
    """In float32 every product element is one sum in k order, a token's attention depends on
    its position alone and norms work row by row: so the logits at a (request, position) must
    not differ by a single bit between a whole prompt, tokens one by one, portions of changing
    size and mixed batches on reused pages."""
    folder, cfg, weights, page = models[name]
    base = PROMPT_LENS[name]
    lens = base + [base[-1] + 17, base[0] + 1]
    token_lists = {f"q{i}": random_tokens(n + EXTRA, cfg["vocab_size"], seed=900 + i) for i, n in enumerate(lens)}
    whole = {}
    for rid, tokens in token_lists.items():
        session = session_for(folder, torch.float32, page, max_tokens=len(tokens))
        whole.update(collect(session, [{"step": 0, "entries": [
            {"id": rid, "tokens": tokens, "want": list(range(len(tokens)))}], "end": [rid]}]))
    compared = 0

    def same(got, what):
        nonlocal compared
        for key, row in got.items():
            assert torch.equal(row, whole[key]), f"{what}: {key} differs from the whole prompt by " \
                                                 f"{float((row - whole[key]).abs().max()):.3e}"
            compared += 1

    sizes = [16, 7, 2, 5, 13, 2, 3, 9, 2, 11, 4, 2]
    for rid, tokens in token_lists.items():
        # most of it in one step, the last 32 tokens one by one
        head = len(tokens) - 32
        session = session_for(folder, torch.float32, page, max_tokens=len(tokens))
        steps = [{"step": 0, "entries": [{"id": rid, "tokens": tokens[:head], "want": [head - 1]}], "end": []}]
        steps += [{"step": j + 1, "entries": [{"id": rid, "tokens": [tokens[head + j]], "want": [0]}], "end": []}
                  for j in range(32)]
        same(collect(session, steps), "one by one")
        # portions of changing size
        session = session_for(folder, torch.float32, page, max_tokens=len(tokens))
        steps, at, k = [], 0, 0
        while at < len(tokens):
            size = min(sizes[k % len(sizes)], len(tokens) - at)
            if len(tokens) - at - size == 1:
                size += 1
            steps.append({"step": k, "entries": [{"id": rid, "tokens": tokens[at:at + size],
                                                  "want": list(range(size))}], "end": []})
            at += size
            k += 1
        same(collect(session, steps), "portions")
    # mixed, with so few pages that they are used again
    rounded = sorted((-(-len(t) // 64) * 64 for t in token_lists.values()), reverse=True)
    session = session_for(folder, torch.float32, page, max_tokens=sum(rounded[:4]))
    got = collect(session, mixed_trace(token_lists, seed=12))
    assert len(got) == sum(len(t) for t in token_lists.values())
    same(got, "mixed")
    assert compared > 3 * len(got) // 2


def collect_one(session, rec, starts):
    got = {}
    offsets = {item["id"]: starts.get(item["id"], 0) for item in rec["entries"]}
    out = session.run_step(rec)
    if out is not None and out.logits is not None:
        rows = out.logits.detach().cpu().double()
        i = 0
        for item in rec["entries"]:
            for w in item.get("want", []):
                got[(item["id"], offsets[item["id"]] + w)] = rows[i]
                i += 1
    for item in rec["entries"]:
        starts[item["id"]] = offsets[item["id"]] + len(item["tokens"])
    session.manager.check()
    return got


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
def test_decoding_across_a_length_class(models, dtype):
    """A long request decodes from 1000 to 1100 tokens beside a short one.  Steps of single
    tokens are captured as graphs per class of sequence length (up to 1024, up to 2048, ...)
    and the decode kernel cuts the key range by that class, so the step that crosses 1024
    changes both; the short request's key range is then shorter than the number of parts."""
    folder, cfg, weights, page = models["D"]
    long_tokens = random_tokens(1100, cfg["vocab_size"], seed=501)
    short_tokens = random_tokens(130, cfg["vocab_size"], seed=502)
    session = session_for(folder, dtype, page, max_tokens=1100 + 192)
    steps = [{"step": 0, "entries": [{"id": "L", "tokens": long_tokens[:1000], "want": [999]},
                                     {"id": "S", "tokens": short_tokens[:30], "want": [29]}], "end": []}]
    for j in range(100):
        steps.append({"step": j + 1, "entries": [
            {"id": "L", "tokens": [long_tokens[1000 + j]], "want": [0]},
            {"id": "S", "tokens": [short_tokens[30 + j]], "want": [0]}], "end": []})
    got = collect(session, steps)
    assert len(got) == 202
    compare(got, {"L": oracle("D", cfg, weights, long_tokens),
                  "S": oracle("D", cfg, weights, short_tokens)}, dtype)
    if session.runner.use_hip_graphs:
        assert session.runner.graph_replays >= 90  # two classes, each: one step eager, one captured
        # the longer class is there (the shorter one's graph goes when a step buffer grows)
        assert -(-(1100 + 192) // 64) * 64 in {key[1] for key in session.runner._graphs}


@pytest.mark.parametrize("dtype", DTYPES, ids=["f32", "bf16"])
def test_graphs_of_wide_decode_steps_replay_right_every_time(models, dtype):
    """Twenty requests decode together, so that the captured step holds the vendor matrix
    product (more than 16 rows) beside our kernels.  Every replay is compared with the plain
    implementation, and a step of another shape runs launch by launch between replays."""
    folder, cfg, weights, page = models["D"]
    n_req = 20
    seqs = {f"w{i}": random_tokens(9 + 3 * i + 12, cfg["vocab_size"], seed=700 + i) for i in range(n_req)}
    total = sum(-(-len(t) // 64) * 64 for t in seqs.values())
    session = session_for(folder, dtype, page, max_tokens=total, max_num_seqs=24)
    expect = {rid: oracle("D", cfg, weights, t) for rid, t in seqs.items()}
    steps, k = [], 0
    # prompts, four requests a step
    ids = list(seqs)
    for i in range(0, n_req, 4):
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": seqs[r][:len(seqs[r]) - 12], "want": [len(seqs[r]) - 13]} for r in ids[i:i + 4]]})
        k += 1
    # twelve decode steps of all twenty; after the sixth, a step of two tokens for one request
    # (run launch by launch) stands between the replays
    fed = {r: len(seqs[r]) - 12 for r in ids}
    for j in range(11):
        entries = []
        for r in ids:
            if j == 6 and r == ids[0]:
                continue
            entries.append({"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]})
            fed[r] += 1
        steps.append({"step": k, "end": [], "entries": entries}); k += 1
        if j == 6:
            r = ids[0]
            steps.append({"step": k, "end": [], "entries": [
                {"id": r, "tokens": seqs[r][fed[r]:fed[r] + 2], "want": [0, 1]}]}); k += 1
            fed[r] += 2
    got = collect(session, steps)
    compare(got, expect, dtype)
    if session.runner.use_hip_graphs:
        assert session.runner.graph_replays >= 8


def test_steps_of_a_few_dozen_rows_on_a_wide_model(tmp_path, monkeypatch):
    """Forty requests decode together on a model whose widths are multiples of 512: the
    products before the norms leave partial sums of slices along K that one kernel adds into
    the residual and normalises, and the gate-up product applies the activation itself.  A
    portion of a prompt rides along in some steps."""
    from kvcore_amd.ops import library as ops
    from tests.helpers import WIDE, WIDE_PAGE

    folder = make_model_dir(tmp_path / "wide", WIDE, seed=21)
    cfg, weights = plain.load_model_folder(folder)
    modes = []
    real = ops.gemm_mid

    def spy(*args, **kw):
        modes.append(kw.get("mode", 0))
        return real(*args, **kw)

    monkeypatch.setattr(ops, "gemm_mid", spy)
    n_req = 40
    tail = 3  # tokens that the first twenty requests decode after the others have ended
    seqs = {f"m{i}": random_tokens(5 + i % 7 + 10 + (tail if i < 20 else 0), cfg["vocab_size"], seed=800 + i)
            for i in range(n_req)}
    seqs["late"] = random_tokens(50, cfg["vocab_size"], seed=899)
    total = sum(-(-len(t) // 64) * 64 for t in seqs.values())
    session = session_for(folder, torch.bfloat16, WIDE_PAGE, max_tokens=total, max_num_seqs=48)
    expect = {rid: plain.llama_forward(cfg, weights, t, dtype=torch.float64) for rid, t in seqs.items()}
    ids = [r for r in seqs if r != "late"]
    steps, k = [], 0
    first = {r: len(seqs[r]) - 10 - (tail if i < 20 else 0) for i, r in enumerate(ids)}
    for i in range(0, n_req, 8):
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": seqs[r][:first[r]], "want": [first[r] - 1]} for r in ids[i:i + 8]]})
        k += 1
    fed = dict(first)
    late_at = 0
    for j in range(10):
        entries = [{"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]} for r in ids]
        for r in ids:
            fed[r] += 1
        if j in (3, 4, 7):  # 40 single tokens and a portion: 17 to 64 rows still
            n = (9, 2, 13)[(3, 4, 7).index(j)]
            entries.append({"id": "late", "tokens": seqs["late"][late_at:late_at + n], "want": list(range(n))})
            late_at += n
        steps.append({"step": k, "end": ids[20:] if j == 9 else [], "entries": entries}); k += 1
    for j in range(tail):  # twenty rows: the same kernels from seventeen rows on
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]} for r in ids[:20]]}); k += 1
        for r in ids[:20]:
            fed[r] += 1
    got = collect(session, steps)
    assert all(fed[r] == len(seqs[r]) for r in ids)
    assert 2 in modes and 1 in modes, "the partial-sum and the gated form should both have run"
    expect["late"] = expect["late"][:late_at]
    # this model's logits are larger than the tiny models' (0.46 against 0.2 in the root mean
    # square), and so is the rounding noise in them, on every path: with 4 and 12 rows (the
    # few-row kernels) and with 70 (the vendor product) the largest error measured was 0.91
    # and 1.23 of the tiny models' bound, with these 40 rows 1.13
    rms = float(torch.cat([e.flatten() for e in expect.values()]).pow(2).mean().sqrt())
    assert 0.4 < rms < 0.55
    compare(got, expect, torch.bfloat16, logit_rms=rms)


def test_layer_sizes_of_the_8b_model(tmp_path):
    """One layer with the widths of Llama-3-8B (4096 wide, 32 heads of 128 over 8 kv heads,
    14336 in the feed-forward) and a small vocabulary, against the plain implementation in
    float32: the shapes that decide which kernel runs are the real ones.  Prompts whole, then
    20 rows together (the kernels that share the rows through LDS), then 12 and 3 (the few-row
    kernels with the norms folded in), through graphs where the runner uses them."""
    config = {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": 1,
        "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
        "intermediate_size": 14336, "vocab_size": 384, "rope_theta": 500000.0,
        "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                         "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
        "tie_word_embeddings": False, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192,
        "hidden_act": "silu",
    }
    folder = make_model_dir(tmp_path / "wide8b", config, seed=5)
    cfg, weights = plain.load_model_folder(folder)
    n_req, tail = 20, 6
    seqs = {f"r{i}": random_tokens(20 + 3 * i + tail, cfg["vocab_size"], seed=900 + i) for i in range(n_req)}
    total = sum(-(-len(t) // 64) * 64 for t in seqs.values())
    session = session_for(folder, torch.bfloat16, 16, max_tokens=total, max_num_seqs=24)
    expect = {rid: plain.llama_forward(cfg, weights, t, dtype=torch.float32).double() for rid, t in seqs.items()}
    ids = list(seqs)
    steps, k = [], 0
    for i in range(0, n_req, 4):
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": seqs[r][:len(seqs[r]) - tail], "want": [0, len(seqs[r]) - tail - 1]}
            for r in ids[i:i + 4]]})
        k += 1
    fed = {r: len(seqs[r]) - tail for r in ids}
    for j in range(tail):
        live = ids if j < 2 else (ids[:12] if j < 4 else ids[:3])
        ended = ids[12:] if j == 1 else (ids[3:12] if j == 3 else [])
        steps.append({"step": k, "end": ended, "entries": [
            {"id": r, "tokens": [seqs[r][fed[r]]], "want": [0]} for r in live]})
        k += 1
        for r in live:
            fed[r] += 1
    got = collect(session, steps)
    rms = float(torch.cat([e.flatten() for e in expect.values()]).pow(2).mean().sqrt())
    compare(got, expect, torch.bfloat16, logit_rms=rms)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (head sizes in steps of 16, any head counts and groups,
    widths, feed-forward widths and vocabularies that are no power of two (some matrices can
    be packed for decode steps, others not), pages of 8 to 48 tokens, with and without biases,
    tied head and scaled rotation): whole requests and mixed
    batches with page reuse, in both dtypes, against the plain implementation."""
    import random

    from tests import helpers

    rng = random.Random(1000 + seed)
    d = rng.choice([16, 32, 48, 64, 80, 96, 112, 128])
    nkv = rng.choice([1, 2, 3, 4, 5])
    nh = nkv * rng.choice([1, 2, 3, 4, 7])
    vocab = rng.choice([97, 300, 515, 1000])
    page = rng.choice([8, 16, 32, 48])
    config = {
        "architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": rng.choice([1, 2, 3]),
        "hidden_size": rng.choice([40, 56, 72, 100, 128, 136, 192, 200, 264]), "num_attention_heads": nh,
        "num_key_value_heads": nkv, "head_dim": d, "intermediate_size": rng.choice([88, 120, 200, 256, 301, 512]),
        "vocab_size": vocab, "rope_theta": rng.choice([1e4, 5e5]),
        "rope_scaling": rng.choice([None, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                           "high_freq_factor": 4.0, "original_max_position_embeddings": 64}]),
        "tie_word_embeddings": rng.random() < 0.5, "rms_norm_eps": rng.choice([1e-5, 1e-6]),
        "max_position_embeddings": 512, "hidden_act": "silu", "attention_bias": rng.random() < 0.3,
        "mlp_bias": rng.random() < 0.3,
    }
    folder = make_model_dir(tmp_path, config, seed=seed)
    cfg, weights = plain.load_model_folder(folder)
    token_lists = {f"q{i}": random_tokens(rng.randint(1, 90) + EXTRA, vocab, seed=seed * 10 + i) for i in range(6)}
    expect = {rid: plain.llama_forward(cfg, weights, t, dtype=torch.float64) for rid, t in token_lists.items()}
    rms = max(float(torch.cat([e.flatten() for e in expect.values()]).pow(2).mean().sqrt()), helpers.TINY_LOGIT_RMS)
    for dtype in DTYPES:
        for rid, t in list(token_lists.items())[:2]:
            session = session_for(folder, dtype, page, max_tokens=len(t))
            got = collect(session, [{"step": 0, "entries": [{"id": rid, "tokens": t, "want": list(range(len(t)))}],
                                     "end": [rid]}])
            compare(got, expect, dtype, logit_rms=rms)
        rounded = sorted((-(-len(t) // 64) * 64 for t in token_lists.values()), reverse=True)
        session = session_for(folder, dtype, page, max_tokens=sum(rounded[:4]))
        got = collect(session, mixed_trace(token_lists, seed=seed))
        assert len(got) == sum(len(t) for t in token_lists.values())
        compare(got, expect, dtype, logit_rms=rms)
        assert session.manager.num_free_pages()[0] == session.num_pages - 1


def test_packed_weights_change_no_bit(models):
    """A model keeps a second copy of its matrices in the order decode steps stream them
    (where the device has room, so in every other test here).  The logits with it are those
    without it, bit for bit: whole prompt, then tokens one by one."""
    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.engine.runner import build_model

    folder, cfg, weights, page = models["D"]
    tokens = random_tokens(90, cfg["vocab_size"], seed=77)
    rows = {}
    for pack in (True, False):
        model = build_model(folder, torch.bfloat16, "cuda:0", pack_weights=pack)
        packed = [w for w in model.product_weights() if getattr(w, "kvc_packed", None) is not None]
        assert len(packed) == (len(model.product_weights()) if pack else 0)
        assert not pack or len(packed) >= 4 * cfg["num_hidden_layers"] + 1
        session = TraceSession(str(folder), torch.bfloat16, max_tokens=128, block_size=page, model=model)
        steps = [{"step": 0, "entries": [{"id": "r", "tokens": tokens[:60], "want": [59]}], "end": []}]
        steps += [{"step": i + 1, "entries": [{"id": "r", "tokens": [tokens[60 + i]], "want": [0]}], "end": []}
                  for i in range(30)]
        rows[pack] = collect(session, steps)
    assert len(rows[True]) == 31
    for key, row in rows[True].items():
        assert torch.equal(row, rows[False][key]), key
    compare(rows[True], {"r": oracle("D", cfg, weights, tokens)}, torch.bfloat16)


@pytest.mark.parametrize("name", ["A", "D"])
def test_a_captured_step_allocates_and_frees_nothing_of_its_own(models, name, monkeypatch):
    """While a decode step is captured into a graph, the step buffers are frozen and nothing
    under the step may make or drop a tensor of its own (a free that reaches the HIP runtime
    during a capture ends the process): torch's allocating constructors raise while the
    buffers are frozen, every step buffer asked for must already be there, and torch's
    allocator must hold after the capture what it held before it, apart from the graph's own
    pool."""
    from kvcore_amd.engine import context

    folder, cfg, weights, page = models[name]
    tokens = random_tokens(40, cfg["vocab_size"], seed=55)
    session = session_for(folder, torch.bfloat16, page, max_tokens=64)
    if not session.runner.use_hip_graphs:
        pytest.skip("this model's steps are not captured")
    frozen_gets = []
    real_get = context.StepBuffers.get

    def watched_get(self, name_, rows, cols, dtype, reserve=0):
        if self.frozen:
            buf = self._store.get(name_)
            assert buf is not None and buf.dtype == dtype and buf.shape[1] == cols and buf.shape[0] >= rows, \
                f"step buffer {name_!r} is not there at its full size during the capture"
            frozen_gets.append(name_)
        return real_get(self, name_, rows, cols, dtype, reserve)

    monkeypatch.setattr(context.StepBuffers, "get", watched_get)
    for fn in ("empty", "zeros", "ones", "full", "tensor", "empty_like", "zeros_like", "arange"):
        real = getattr(torch, fn)

        def guarded(*a, _real=real, _fn=fn, **kw):
            assert not session.runner.buffers.frozen, f"torch.{_fn} was called while a step was captured"
            return _real(*a, **kw)

        monkeypatch.setattr(torch, fn, guarded)
    steps = [{"step": 0, "entries": [{"id": "r", "tokens": tokens[:30], "want": [29]}], "end": []}]
    steps += [{"step": j + 1, "entries": [{"id": "r", "tokens": [tokens[30 + j]], "want": [0]}], "end": []}
              for j in range(6)]
    got = collect(session, steps)
    assert session.runner.graph_replays >= 4 and frozen_gets, "a step should have been captured"
    assert not session.runner.buffers.frozen
    compare(got, {"r": oracle(name, cfg, weights, tokens)}, torch.bfloat16)
