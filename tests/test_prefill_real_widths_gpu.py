"""The bfloat16 kernels that a long prompt runs through, at the layer sizes of Llama-3-8B: a
prompt of 2,048 tokens whole, in portions of some five hundred, and as 1,536 tokens followed
by portions of 7, 2 and 13 while other requests decode beside it on poisoned pages that are
used again.  Two layers and a vocabulary of 384 keep the plain implementation cheap (float32
on the CPU, some fifteen seconds for the long prompt); every width that decides which kernel
runs, and how long its sums are, is the real one.

Reference formulas: kvcore/model/attn_backend/torch_paged.py:90-117 (every query reads keys
``0..position`` from the cache), kvcore/model/models/llama3.py:189-200.
"""

from __future__ import annotations

import random

import pytest
import torch

from tests.helpers import random_tokens
from tests.plain import llama as plain
from tests.test_cuts_gpu import collect, session_for
from tests.test_real_sizes_gpu import CONFIG as LAYERS_OF_8B, compare_rounding_noise

pytestmark = pytest.mark.gpu

CONFIG = dict(LAYERS_OF_8B, vocab_size=384, num_hidden_layers=2)
PAGE = 16
LONG = 2048
WHAT = "rows at 8B widths, prompts of 2048"
# the first positions, edges of pages (16), of the attention kernel's tiles of rows and keys
# (64, 128, 256), of the portions below (505, 512, 1024, 1536 and the small ones after it),
# and the last ones
EDGES = [0, 1, 2, 15, 16, 17, 31, 32, 47, 48, 63, 64, 65, 127, 128, 129, 191, 192, 255, 256, 257,
         383, 384, 504, 505, 511, 512, 513, 767, 768, 1023, 1024, 1025, 1279, 1280, 1528, 1529,
         1535, 1536, 1537, 1542, 1543, 1544, 1545, 1557, 1558, 1559, 1791, 1792, 2031, 2032, 2046, 2047]


def wanted_positions() -> list[int]:
    rng = random.Random(77)
    extra = set()
    while len(extra) + len(EDGES) < 64:
        p = rng.randrange(LONG)
        if p not in EDGES:
            extra.add(p)
    return sorted(set(EDGES) | extra)


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    from kvcore_amd.engine.runner import build_model
    from kvcore_amd.weights.loader import write_random_model

    folder = write_random_model(tmp_path_factory.mktemp("prefill_real_widths"), CONFIG, seed=21, device="cuda:0")
    cfg, weights = plain.load_model_folder(folder)
    weights = {name: t.float() for name, t in weights.items()}
    model = build_model(folder, torch.bfloat16, "cuda:0")
    tokens = random_tokens(LONG, cfg["vocab_size"], seed=500)
    expect = plain.llama_forward(cfg, weights, tokens, dtype=torch.float32).double()
    return folder, cfg, weights, model, tokens, expect


class Spy:
    """Which kernels a step ran: the variants the library notes, and the vendor's products."""

    def __init__(self, monkeypatch):
        from kvcore_amd.ops import library as ops

        self.ops = ops
        self.vendor_rows: list[int] = []
        self.prefill: list[str] = []
        self.rope: list[str] = []
        real_mm, real_prefill, real_rope = torch.mm, ops.prefill_attention, ops.rope_kv_write

        def mm(x, w, **kw):
            self.vendor_rows.append(x.shape[0])
            return real_mm(x, w, **kw)

        def prefill(*a, **kw):
            real_prefill(*a, **kw)
            self.prefill.append(ops.last_variant("prefill_attention"))

        def rope(*a, **kw):
            real_rope(*a, **kw)
            self.rope.append(ops.last_variant("rope_kv_write"))

        monkeypatch.setattr(torch, "mm", mm)
        monkeypatch.setattr(ops, "prefill_attention", prefill)
        monkeypatch.setattr(ops, "rope_kv_write", rope)


def test_a_prompt_of_2048_tokens_whole(wide, monkeypatch):
    folder, cfg, weights, model, tokens, expect = wide
    spy = Spy(monkeypatch)
    want = wanted_positions()
    assert len(want) == 64 and want[0] == 0 and want[-1] == LONG - 1
    session = session_for(folder, torch.bfloat16, PAGE, max_tokens=LONG, model=model)
    got = collect(session, [{"step": 0, "entries": [{"id": "p", "tokens": tokens, "want": want}], "end": ["p"]}])
    assert sorted(pos for _, pos in got) == want
    compare_rounding_noise(got, {"p": expect}, what=WHAT)
    # what the benchmark's prefill runs: blocks of eight waves with tiles of 128 keys, eight
    # tokens a block in the rotation, the vendor's product for all 2,048 rows
    assert set(spy.prefill) == {"prefill_attention_kernel<128,1,8,8> x1"}, spy.prefill
    assert set(spy.rope) == {"rope_kv_write_tile_kernel"}
    assert spy.vendor_rows.count(LONG) == 4 * CONFIG["num_hidden_layers"], spy.vendor_rows


def test_the_same_prompt_in_portions_with_a_ragged_end(wide, monkeypatch):
    folder, cfg, weights, model, tokens, expect = wide
    spy = Spy(monkeypatch)
    want = set(wanted_positions())
    session = session_for(folder, torch.bfloat16, PAGE, max_tokens=LONG, model=model)
    steps, at = [], 0
    for k, size in enumerate((512, 512, 512, 505, 7)):
        here = [p - at for p in sorted(want) if at <= p < at + size]
        steps.append({"step": k, "entries": [{"id": "p", "tokens": tokens[at:at + size], "want": here}],
                      "end": ["p"] if at + size == LONG else []})
        at += size
    assert at == LONG
    got = collect(session, steps)
    assert {pos for _, pos in got} == want
    compare_rounding_noise(got, {"p": expect}, what=WHAT)
    # portions with a context behind them: the matrix-core kernel, with and without splits
    assert len(spy.prefill) == 5 * CONFIG["num_hidden_layers"]
    assert all(v.startswith("prefill_attention_kernel<128,") for v in spy.prefill)
    assert any(not v.endswith(" x1") for v in spy.prefill), spy.prefill  # few rows after many keys are split


def test_the_end_of_the_prompt_in_small_portions_beside_decoding_requests(wide, monkeypatch):
    """1,536 tokens in one step, then portions of 7, 2 and 13 (the first of them ends inside a
    page, most begin and end inside one), each beside the single tokens of up to three other
    requests, which come and go: their pages are given back, poisoned and handed out again,
    also to the long request.  Every row that is asked for is compared with the plain
    implementation: the long request's wanted positions, every decoded token of the others."""
    folder, cfg, weights, model, tokens, expect = wide
    spy = Spy(monkeypatch)
    want = set(wanted_positions())
    rng = random.Random(9)
    short = {}
    for i in range(14):
        total = rng.randrange(40, 121)
        short[f"s{i}"] = (random_tokens(total, cfg["vocab_size"], seed=600 + i), rng.randrange(10, 26))
    expects = {rid: plain.llama_forward(cfg, weights, toks, dtype=torch.float32).double()
               for rid, (toks, _) in short.items()}
    expects["p"] = expect
    session = session_for(folder, torch.bfloat16, PAGE, max_tokens=LONG + 3 * 128, model=model)

    waiting = list(short)
    live: dict[str, int] = {}  # tokens fed so far
    steps, at, k = [], 0, 0
    sizes = (7, 2, 13)
    pages_asked = 0
    while at < LONG or live or waiting:
        entries, end = [], []
        if at < LONG:
            size = 1536 if at == 0 else min(sizes[(k - 1) % 3], LONG - at)
            if LONG - at - size == 1:
                size += 1
            entries.append({"id": "p", "tokens": tokens[at:at + size],
                            "want": [p - at for p in sorted(want) if at <= p < at + size]})
            at += size
            if at == LONG:
                end.append("p")
        for rid in list(live):
            toks, _ = short[rid]
            entries.append({"id": rid, "tokens": [toks[live[rid]]], "want": [0]})
            live[rid] += 1
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        ending = sum(1 for rid in end if rid != "p")  # they are live until this step is over
        while waiting and len(live) + ending < 3 and (at < LONG or not live):
            rid = waiting.pop(0)
            toks, decoded = short[rid]
            head = len(toks) - decoded
            entries.append({"id": rid, "tokens": toks[:head], "want": [head - 1]})
            live[rid] = head
            pages_asked += -(-len(toks) // PAGE)
        rng.shuffle(entries)
        steps.append({"step": k, "entries": entries, "end": end})
        k += 1
    assert not waiting and len(steps) > 60
    assert pages_asked + LONG // PAGE > session.num_pages - 1, "the trace must not fit without reuse"
    mixed = [s for s in steps if len(s["entries"]) == 4]
    assert len(mixed) > 40  # most steps: a portion of the long request beside three single tokens

    got = collect(session, steps)
    assert {pos for rid, pos in got if rid == "p"} == want
    decoded_rows = sum(d + 1 for _, d in short.values())
    assert len(got) == len(want) + decoded_rows
    compare_rounding_noise(got, expects, what=WHAT)
    assert session.manager.live_requests() == []
    assert all(v.startswith("prefill_attention_kernel<128,") for v in spy.prefill) and spy.prefill


def test_decode_steps_of_a_hundred_and_more_requests(wide, monkeypatch):
    """Steps of single tokens for 190, 150, 120 and 90 requests at the 8B widths: the kernels
    that share their rows through LDS with twelve, eight and six tiles of rows a wave (the
    products cut along K up to 192 rows, the gated one up to 128), the vendor's product for the
    rest.  Every decoded position of every request against the plain implementation."""
    from kvcore_amd.ops import library as ops

    folder, cfg, weights, model, _, _ = wide
    live_after = [190, 150, 120, 90]
    seqs = {}
    for i in range(live_after[0]):
        alive = sum(1 for n in live_after if i < n)
        seqs[f"q{i}"] = random_tokens(2 + i % 4 + alive, cfg["vocab_size"], seed=900 + i)
    expect = {rid: plain.llama_forward(cfg, weights, toks, dtype=torch.float32).double() for rid, toks in seqs.items()}
    mid_rows, gated_rows = [], []
    real_mid = ops.gemm_mid

    def spy_mid(out, x, *a, **kw):
        (gated_rows if kw.get("mode") == 1 else mid_rows).append(x.shape[0])
        return real_mid(out, x, *a, **kw)

    monkeypatch.setattr(ops, "gemm_mid", spy_mid)
    vendor_rows = []
    real_mm = torch.mm
    monkeypatch.setattr(torch, "mm", lambda x, w, **kw: (vendor_rows.append(x.shape[0]), real_mm(x, w, **kw))[1])
    total = sum(-(-len(t) // 64) * 64 for t in seqs.values())
    session = session_for(folder, torch.bfloat16, PAGE, max_tokens=total, max_num_seqs=192, model=model)
    ids = list(seqs)
    fed = {r: len(seqs[r]) - sum(1 for n in live_after if int(r[1:]) < n) for r in ids}
    steps, k = [], 0
    for lo in range(0, len(ids), 10):  # prompts, ten requests a step
        steps.append({"step": k, "end": [], "entries": [
            {"id": r, "tokens": seqs[r][:fed[r]], "want": [fed[r] - 1]} for r in ids[lo:lo + 10]]})
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
    assert len(got) == len(ids) + sum(live_after)
    compare_rounding_noise(got, expect, what="decode steps of 90 to 190 rows at 8B widths")
    # padded to the sizes at which such steps are captured: 192, 160, 128 and 96 rows
    assert {192, 160, 128, 96} <= set(mid_rows), sorted(set(mid_rows))
    assert {128, 96} <= set(gated_rows) and not {192, 160} & set(gated_rows), sorted(set(gated_rows))
    assert {192, 160} <= set(vendor_rows), sorted(set(vendor_rows))
    assert session.manager.live_requests() == []
