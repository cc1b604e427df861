"""Generation through the Python entry point and the command line, against the plain
implementation: greedy (tiny A's workload), seeded temperature sampling (tiny B's),
chunked prefill, preemption when pages run out."""

from __future__ import annotations

import math
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from tests.helpers import CONFIGS, make_model_dir, random_tokens
from tests.plain import llama as plain
from tests.plain import sampling as plain_sampling

pytestmark = pytest.mark.gpu
REPO = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, (config, page) in CONFIGS.items():
        folder = make_model_dir(tmp_path_factory.mktemp(f"gen_{name}"), config, seed=21)
        out[name] = (folder, *plain.load_model_folder(folder), page)
    return out


def make_engine(folder, dtype, page, *, num_pages=None, max_seqs=4, budget=64, partial=4, threshold=0,
                run_ahead=True, graphs=True, poison=False):
    from kvcore_amd import (CacheConfig, DeviceConfig, KVCoreConfig, LoadConfig, ModelConfig, SchedulerConfig)
    from kvcore_amd.engine.llm_engine import LLMEngine

    return LLMEngine(KVCoreConfig(
        model_config=ModelConfig(model=str(folder), dtype=dtype),
        load_config=LoadConfig(seed=77),
        cache_config=CacheConfig(block_size=page, num_gpu_blocks=num_pages, poison_pages=poison),
        scheduler_config=SchedulerConfig(max_num_seqs=max_seqs, max_num_scheduled_tokens=budget,
                                         max_num_partial_prefills=partial, max_long_partial_prefills=partial,
                                         long_prefill_token_threshold=threshold,
                                         decode_run_ahead=run_ahead),
        device_config=DeviceConfig(use_hip_graphs=graphs),
    ))


def check_tokens(cfg, weights, prompt, tokens, *, temperature, seed, tol):
    """Every generated token must be the plain sampler's choice on the plain logits of the
    same prefix, or tie with it within rounding (``tol`` on the compared scores)."""
    ids = list(prompt)
    for index, tok in enumerate(tokens):
        logits = plain.llama_forward(cfg, weights, ids, dtype=torch.float64)[-1]
        if temperature < 1e-5:
            score = logits
        else:
            noise = plain_sampling.exponential_noise(seed, index, logits.numel())
            score = logits / temperature - torch.log(noise)
        gap = float(score.max() - score[tok])
        assert gap <= tol, (f"token {index}: engine chose {tok}, plain prefers {int(score.argmax())} "
                            f"by {gap:.2e}")
        ids.append(tok)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 4e-2)])
def test_greedy_generation_through_the_entry_point(folders, dtype, tol):
    from kvcore_amd import SamplingParams
    from kvcore_amd.engine.llm_engine import GenerationRequest

    folder, cfg, weights, page = folders["A"]
    prompts = {f"r{n}": random_tokens(n, 256, seed=n) for n in (7, 16, 33, 50)}
    engine = make_engine(folder, dtype, page)
    outs = engine.generate([
        GenerationRequest(rid, SamplingParams(max_tokens=16, temperature=0.0, ignore_eos=True),
                          prompt_token_ids=tuple(p)) for rid, p in prompts.items()])
    assert [o.request_id for o in outs] == list(prompts)
    for o in outs:
        assert len(o.output_token_ids) == 16 and o.finish_reason == "length"
        check_tokens(cfg, weights, prompts[o.request_id], o.output_token_ids, temperature=0.0, seed=0, tol=tol)
        if dtype == "float32":
            assert list(o.output_token_ids) == plain.greedy_generate(cfg, weights, prompts[o.request_id], 16)
    core = engine.engine_core
    assert core.kv_manager.num_free_pages() == [core.num_pages - 1]  # idle: every page is back
    assert core.kv_manager.slots.num_free == 4


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-5), ("bfloat16", 6e-2)])
def test_seeded_temperature_sampling_with_chunked_prefill(folders, dtype, tol):
    """Tiny B's workload: prompts 1/9/24/40/61, temperature 0.8 with a fixed seed, 32 new
    tokens, prompts cut into portions of 16."""
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["B"]
    prompts = {f"r{n}": random_tokens(n, 384, seed=100 + n) for n in (1, 9, 24, 40, 61)}
    engine = make_engine(folder, dtype, page, budget=40, threshold=16)
    reqs = [dict(request_id=rid, prompt_token_ids=p,
                 sampling_params=SamplingParams(max_tokens=32, temperature=0.8, seed=1234 + i, ignore_eos=True))
            for i, (rid, p) in enumerate(prompts.items())]
    outs = {o.request_id: o for o in engine.generate(reqs)}
    for i, (rid, p) in enumerate(prompts.items()):
        toks = outs[rid].output_token_ids
        assert len(toks) == 32
        check_tokens(cfg, weights, p, toks, temperature=0.8, seed=1234 + i, tol=tol)
        assert len(set(toks)) > 8  # fresh noise at every token
    # the same seeds give the same tokens, whatever the batching
    again = make_engine(folder, dtype, page, budget=64, max_seqs=2)
    outs2 = {o.request_id: o for o in again.generate(reqs)}
    if dtype == "float32":
        assert all(outs2[r].output_token_ids == outs[r].output_token_ids for r in prompts)


def test_generation_survives_running_out_of_pages(folders):
    """So few pages that running requests must be preempted and recomputed; the outputs are
    those of an engine with plenty of pages."""
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["A"]
    prompts = {f"r{i}": random_tokens(n, 256, seed=300 + i) for i, n in enumerate((20, 30, 25, 18))}
    reqs = [dict(request_id=rid, prompt_token_ids=p,
                 sampling_params=SamplingParams(max_tokens=30, temperature=0.0, ignore_eos=True))
            for rid, p in prompts.items()]
    roomy = make_engine(folder, "float32", page)
    want = {o.request_id: o.output_token_ids for o in roomy.generate(reqs)}
    tight = make_engine(folder, "float32", page, num_pages=9)  # 8 usable pages of 16 tokens
    got = {o.request_id: o.output_token_ids for o in tight.generate(reqs)}
    assert tight.engine_core.scheduler.num_preemptions > 0
    assert got == want
    assert tight.engine_core.kv_manager.num_free_pages() == [8]
    # a request that can never fit is refused at once
    tiny = make_engine(folder, "float32", page, num_pages=4)  # 3 usable pages hold 48 tokens
    with pytest.raises(ValueError, match="cache pages"):
        tiny.add_request("big", SamplingParams(max_tokens=10), prompt_token_ids=list(range(50)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("temperature", [0.0, 0.9])
def test_steps_launched_ahead_give_the_tokens_of_steps_taken_one_by_one(folders, dtype, temperature):
    """While requests only decode, the engine launches the next step before it has seen the
    tokens of the step in flight.  Requests that stop on a token (and so have run one step
    too far), that reach their length cap and that arrive later must come out as they do
    from an engine that takes every step by itself."""
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["A"]
    prompts = {f"r{i}": random_tokens(n, 256, seed=500 + i) for i, n in enumerate((9, 17, 30, 5, 12))}
    caps = {"r0": 40, "r1": 23, "r2": 40, "r3": 31, "r4": 12}

    def run(run_ahead, stop, graphs=True):
        engine = make_engine(folder, dtype, page, run_ahead=run_ahead, max_seqs=4, graphs=graphs)
        engine.engine_core.stop_token_ids = set(stop)
        launched = 0
        core = engine.engine_core
        for i, (rid, p) in enumerate(prompts.items()):
            if i == 4:
                continue
            core.add_request(rid, SamplingParams(max_tokens=caps[rid], temperature=temperature, seed=40 + i),
                             prompt_token_ids=p)
        steps = 0
        while core.has_unfinished_requests():
            core.step()
            steps += 1
            launched += core._in_flight is not None
            if steps == 6:  # a late arrival, while the others decode
                core.add_request("r4", SamplingParams(max_tokens=caps["r4"], temperature=temperature, seed=44),
                                 prompt_token_ids=prompts["r4"])
        outs = {rid: core.take_finished_output(rid) for rid in prompts}
        assert core.kv_manager.num_free_pages() == [core.num_pages - 1]
        assert core.kv_manager.slots.num_free == 4
        return {rid: (o.output_token_ids, o.finish_reason) for rid, o in outs.items()}, launched

    free, _ = run(False, ())
    # stop on tokens that r0 and r2 say in mid-course
    stop = {free["r0"][0][14], free["r2"][0][20]}
    want, none_ahead = run(False, stop)
    got, ahead = run(True, stop)
    assert none_ahead == 0 and ahead > 10
    assert any(reason.value == "stop" for _, reason in want.values())
    assert got == want
    if dtype == "float32":  # and launch by launch, without captured graphs
        plain_launches, ahead = run(True, stop, graphs=False)
        assert ahead > 10 and plain_launches == want


def test_abort_while_a_step_is_in_flight(folders):
    """A request aborted while the step launched ahead still holds it: the step's row for it
    is dropped, the others go on as if nothing had happened."""
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["A"]
    prompts = {f"r{i}": random_tokens(n, 256, seed=700 + i) for i, n in enumerate((11, 6, 21))}

    def run(abort_at):
        core = make_engine(folder, "float32", page).engine_core
        for rid, p in prompts.items():
            core.add_request(rid, SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True),
                             prompt_token_ids=p)
        steps = 0
        while core.has_unfinished_requests():
            core.step()
            steps += 1
            if steps == abort_at:
                assert core._in_flight is not None
                core.abort_requests(["r1"])
                assert all(s.request_id != "r1" for s in core._in_flight.output.scheduled)
        assert core.kv_manager.num_free_pages() == [core.num_pages - 1]
        return {rid: core.take_finished_output(rid) for rid in prompts}

    whole = run(None)
    cut = run(5)
    assert cut["r1"].finish_reason.value == "abort"
    assert cut["r1"].output_token_ids == whole["r1"].output_token_ids[:len(cut["r1"].output_token_ids)]
    assert 0 < len(cut["r1"].output_token_ids) < 20
    for rid in ("r0", "r2"):
        assert cut[rid].output_token_ids == whole[rid].output_token_ids and len(cut[rid].output_token_ids) == 20


def test_stop_token_ends_a_request(folders):
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["A"]
    prompt = random_tokens(12, 256, seed=9)
    tokens = plain.greedy_generate(cfg, weights, prompt, 8)
    engine = make_engine(folder, "float32", page)
    engine.engine_core.stop_token_ids = {tokens[3]}
    out = engine.generate([dict(request_id="s", prompt_token_ids=prompt,
                                sampling_params=SamplingParams(max_tokens=8, temperature=0.0))])[0]
    first = tokens.index(tokens[3])
    assert list(out.output_token_ids) == tokens[: first + 1] and out.finish_reason == "stop"


def test_command_line(folders, tmp_path):
    folder, cfg, weights, page = folders["A"]
    cmd = [sys.executable, str(REPO / "bin" / "kvcore_offline_batch"), "--model", str(folder),
           "--dtype", "float32", "--prompt-lens", "7,16", "--max-tokens", "5", "--seed", "3",
           "--max-num-seqs", "4", "--max-num-scheduled-tokens", "32", "--num-gpu-blocks", "32",
           "--ignore-eos", "--log-level", "WARNING", "--log-file", str(tmp_path / "run.log")]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
    assert proc.returncode == 0, proc.stderr[-2000:]
    text = proc.stdout
    for section in ("=== Run Metadata ===", "=== Requests ===", "=== Detokenized Outputs ===",
                    "=== Timing Summary ===", "engine_init_sec=", "generate_sec=", "total_elapsed_sec="):
        assert section in text
    assert text.count("finish_reason=length") == 2
    assert (tmp_path / "run.log").read_text().count("finish_reason=length") == 2
    import random

    rng = random.Random(3)
    first_prompt = [rng.randrange(256) for _ in range(7)]
    line = next(l for l in text.splitlines() if l.startswith("token_ids="))
    got = [int(x) for x in line.split("=", 1)[1].strip("()").split(",") if x.strip()]
    assert got == plain.greedy_generate(cfg, weights, first_prompt, 5)


def test_chat_messages_in_and_text_out(folders, tmp_path):
    """With a tokenizer in the model folder a request may carry chat messages: the chat
    template makes the prompt, the tokenizer's end-of-sequence id stops generation, and the
    output comes back as text (reference: kvcore/entry/llm_engine.py:38-48, 97-107)."""
    import shutil

    from kvcore_amd import SamplingParams
    from kvcore_amd.engine.llm_engine import GenerationRequest
    from tests.test_tokenizer import make_tokenizer_folder

    src, cfg, weights, page = folders["A"]
    folder = tmp_path / "with_tokenizer"
    shutil.copytree(src, folder)
    words = make_tokenizer_folder(folder)
    engine = make_engine(folder, "float32", page)
    assert words.index("<eos>") in engine.engine_core.stop_token_ids
    messages = ({"role": "user", "content": "hello world how are you"},)
    out = engine.generate([GenerationRequest("chat", SamplingParams(max_tokens=12, temperature=0.0),
                                             messages=messages)])[0]
    prompt = [words.index(w) for w in ["<|user|>", "hello", "world", "how", "are", "you", "<|assistant|>"]]
    check_tokens(cfg, weights, prompt, list(out.output_token_ids), temperature=0.0, seed=0, tol=1e-4)
    assert isinstance(out.output_text, str)
    if out.finish_reason == "stop":
        assert out.output_token_ids[-1] == words.index("<eos>")
    else:
        assert out.finish_reason == "length" and len(out.output_token_ids) == 12
    # a request without a tokenizer-made prompt needs token ids
    with pytest.raises(ValueError):
        engine.generate([GenerationRequest("bad", SamplingParams(max_tokens=2))])


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-5), ("bfloat16", 6e-2)])
def test_preemption_with_seeded_sampling_and_steps_launched_ahead(folders, dtype, tol):
    """So few pages that running requests are preempted and recomputed, with seeded
    temperature sampling, in both dtypes, with and without steps launched ahead: a preempted
    request's noise stream goes on where it was (nothing is drawn twice), every token is the
    plain sampler's choice on the plain logits, and launching ahead changes no token."""
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["A"]
    prompts = {f"r{i}": random_tokens(n, 256, seed=320 + i) for i, n in enumerate((20, 30, 25, 18))}
    reqs = [dict(request_id=rid, prompt_token_ids=p,
                 sampling_params=SamplingParams(max_tokens=30, temperature=0.8, seed=900 + i, ignore_eos=True))
            for i, (rid, p) in enumerate(prompts.items())]
    results = {}
    for run_ahead in (False, True):
        # 8 usable pages, each filled with NaN when it is taken and when it is given back
        tight = make_engine(folder, dtype, page, num_pages=9, run_ahead=run_ahead, poison=True)
        results[run_ahead] = {o.request_id: o.output_token_ids for o in tight.generate(reqs)}
        assert tight.engine_core.scheduler.num_preemptions > 0
        assert tight.engine_core.kv_manager.num_free_pages() == [8]
    assert results[True] == results[False]
    for i, (rid, p) in enumerate(prompts.items()):
        toks = results[True][rid]
        assert len(toks) == 30
        check_tokens(cfg, weights, p, toks, temperature=0.8, seed=900 + i, tol=tol)
    if dtype == "float32":  # and they are the tokens of an engine that never ran out of pages
        roomy = make_engine(folder, dtype, page)
        assert {o.request_id: o.output_token_ids for o in roomy.generate(reqs)} == results[True]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_engine_equals_a_replay_of_the_trace_its_scheduler_produced(folders, dtype):
    """Every step the engine runs is recorded as a trace step (request, tokens, wanted places,
    requests that ended) and fed again through the replay session, which has neither
    scheduler nor sampler: the logits of every step must be the engine's (in float32 bit for
    bit, wherever the replay's pages lie)."""
    from kvcore_amd import SamplingParams
    from kvcore_amd.engine.replay import TraceSession

    folder, cfg, weights, page = folders["B"]
    prompts = {f"r{n}": random_tokens(n, 384, seed=600 + n) for n in (1, 9, 24, 40, 61)}
    core = make_engine(folder, dtype, page, budget=24, threshold=16, max_seqs=3, run_ahead=False).engine_core
    steps: list[tuple[list, torch.Tensor | None]] = []
    real_step = core.runner.step

    def recording_step(entries, device_tokens=None):
        out = real_step(entries, device_tokens)
        steps.append(([(e.request_id, list(e.tokens), list(e.want)) for e in entries],
                      None if out.logits is None else out.logits.clone()))
        return out

    core.runner.step = recording_step
    for i, (rid, p) in enumerate(prompts.items()):
        if i < 4:
            core.add_request(rid, SamplingParams(max_tokens=12 + i, temperature=0.7, seed=50 + i, ignore_eos=True),
                             prompt_token_ids=p)
    ends: list[list[str]] = []
    while core.has_unfinished_requests():
        before = len(steps)
        outs = core.step()
        assert len(steps) == before + 1
        ends.append([o.request_id for o in outs.request_outputs if o.finished])
        if len(steps) == 5:  # a late arrival
            core.add_request("r61", SamplingParams(max_tokens=9, temperature=0.0, ignore_eos=True),
                             prompt_token_ids=prompts["r61"])
    assert any(len(entries) > 1 and any(len(t) > 1 for _, t, _ in entries) and any(len(t) == 1 for _, t, _ in entries)
               for entries, _ in steps), "some step should mix a portion of a prompt with decoded tokens"
    session = TraceSession(str(folder), getattr(torch, dtype), max_tokens=3 * 128, block_size=page,
                           poison_cache=True, shuffle_pages=5)
    compared = 0
    for k, ((entries, logits), end) in enumerate(zip(steps, ends)):
        out = session.run_step({"step": k, "end": end, "entries": [
            {"id": rid, "tokens": tokens, "want": want} for rid, tokens, want in entries]})
        if logits is None:
            assert out.logits is None
            continue
        assert out.logits.shape == logits.shape
        if dtype == "float32":
            assert torch.equal(out.logits, logits), f"step {k}"
        else:  # the replay plans its launches for another length limit: rounding may differ
            assert torch.allclose(out.logits, logits, atol=2e-2, rtol=2e-2), f"step {k}"
        compared += logits.shape[0]
    assert compared >= sum(12 + i for i in range(4)) + 9
    assert session.manager.live_requests() == []


def check_sampled(cfg, weights, prompt, tokens, params, *, tol, exact_filters):
    """Every token must be what ``tests/plain/sampling.sample`` draws from the plain logits
    of the same prefix with the request's options and its noise of (seed, index).  Where it is
    another token, the two must tie within rounding: the engine's token survives the filters
    (``exact_filters``: the plain filters as they are; otherwise a logit may miss the top-k
    threshold or the top-p boundary by ``tol``) and its score is within ``tol`` of the best."""
    ids = list(prompt)
    T = params.temperature
    for index, tok in enumerate(tokens):
        logits = plain.llama_forward(cfg, weights, ids, dtype=torch.float64)[-1]
        want = plain_sampling.sample(logits, temperature=T, top_k=params.top_k, top_p=params.top_p,
                                     seed=params.seed, index=index)
        if tok != want:
            assert T >= 1e-5 or float(logits.max() - logits[tok]) <= tol, f"token {index}: not the largest logit"
            if T >= 1e-5:
                scaled = logits / T
                top_p = None if params.top_p >= 1.0 else params.top_p
                kept = plain_sampling.apply_top_k_top_p(scaled, params.top_k, top_p)
                if not exact_filters and kept[tok] == -math.inf:
                    # the weakest survivor's logit, and the engine's token no further below it than rounding
                    weakest = kept[kept > -math.inf].min()
                    assert float(weakest - scaled[tok]) <= tol / T, (
                        f"token {index}: {tok} is filtered out by top_k={params.top_k} top_p={params.top_p}")
                    kept = kept.clone()
                    kept[tok] = scaled[tok]
                assert kept[tok] > -math.inf, (
                    f"token {index}: {tok} is filtered out by top_k={params.top_k} top_p={params.top_p}")
                score = kept - torch.log(plain_sampling.exponential_noise(params.seed, index, logits.numel()))
                gap = float(score.max() - score[tok])
                assert gap <= tol / T, f"token {index}: engine chose {tok}, plain draws {want} (ahead by {gap:.2e})"
        ids.append(tok)


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-5), ("bfloat16", 6e-2)])
def test_every_sampling_option_in_one_batch(folders, dtype, tol):
    """Five requests side by side, each with other options: greedy, temperature alone, top-k,
    top-p, and both; seeded, prompts cut into portions, decode steps launched ahead.  The rows
    of one sampling call carry different options, so an option packed into another's column,
    or a row given its neighbour's options, draws other tokens than the plain sampler."""
    from kvcore_amd import SamplingParams

    folder, cfg, weights, page = folders["B"]
    options = [
        SamplingParams(max_tokens=24, temperature=0.0, seed=11, ignore_eos=True),
        SamplingParams(max_tokens=24, temperature=0.8, seed=12, ignore_eos=True),
        SamplingParams(max_tokens=24, temperature=1.0, top_k=5, seed=13, ignore_eos=True),
        SamplingParams(max_tokens=24, temperature=1.3, top_p=0.5, seed=14, ignore_eos=True),
        SamplingParams(max_tokens=24, temperature=0.7, top_k=40, top_p=0.9, seed=15, ignore_eos=True),
    ]
    prompts = [random_tokens(n, 384, seed=700 + n) for n in (5, 33, 18, 47, 26)]
    engine = make_engine(folder, dtype, page, max_seqs=8, budget=40, partial=8, threshold=16, run_ahead=True)
    reqs = [dict(request_id=f"o{i}", prompt_token_ids=p, sampling_params=sp)
            for i, (p, sp) in enumerate(zip(prompts, options))]
    outs = {o.request_id: o.output_token_ids for o in engine.generate(reqs)}
    assert engine.engine_core.runner.graph_replays > 0
    for i, (p, sp) in enumerate(zip(prompts, options)):
        toks = outs[f"o{i}"]
        assert len(toks) == 24
        check_sampled(cfg, weights, p, toks, sp, tol=tol, exact_filters=dtype == "float32")
    # the filters did filter: with top_k = 5 every token is among the five largest logits of
    # its row, which unfiltered noise over 384 flat logits would almost never give
    ids = list(prompts[2])
    for tok in outs["o2"]:
        logits = plain.llama_forward(cfg, weights, ids, dtype=torch.float64)[-1]
        assert float(logits[tok]) >= float(logits.topk(5).values[-1]) - tol
        ids.append(tok)
    # the same requests one at a time draw the same tokens: a row's draw does not depend on
    # the rows beside it
    if dtype == "float32":
        alone = make_engine(folder, dtype, page, max_seqs=1, budget=64, partial=1)
        for i, req in enumerate(reqs):
            assert alone.generate([req])[0].output_token_ids == outs[f"o{i}"]


def test_command_line_top_k_and_top_p(folders, tmp_path):
    folder, cfg, weights, page = folders["B"]
    cmd = [sys.executable, str(REPO / "bin" / "kvcore_offline_batch"), "--model", str(folder),
           "--dtype", "float32", "--block-size", str(page), "--prompt-lens", "9,21", "--max-tokens", "12",
           "--seed", "6", "--temperature", "1.1", "--top-k", "7", "--top-p", "0.8",
           "--max-num-seqs", "4", "--max-num-scheduled-tokens", "32", "--num-gpu-blocks", "64",
           "--ignore-eos", "--log-level", "WARNING", "--no-log-file"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=240)
    assert proc.returncode == 0, proc.stderr[-2000:]
    import random

    from kvcore_amd import SamplingParams

    rng = random.Random(6)
    prompts = [[rng.randrange(384) for _ in range(n)] for n in (9, 21)]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("token_ids=")]
    assert len(lines) == 2
    params = SamplingParams(max_tokens=12, temperature=1.1, top_k=7, top_p=0.8, seed=6, ignore_eos=True)
    for prompt, line in zip(prompts, lines):
        got = [int(x) for x in line.split("=", 1)[1].strip("()").split(",") if x.strip()]
        assert len(got) == 12
        check_sampled(cfg, weights, prompt, got, params, tol=5e-5, exact_filters=True)
