"""Decode and prefill throughput of the Llama-3-8B shape with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the whole engine (scheduler, step function, sampler) at
batch 8 from 512-token prompts, context limit 8192.  One JSON line is printed:
``value`` is decoded tokens a second; ``prefill`` is a 2,048-token prompt in one step;
``roofline`` prices the decode step's mandatory reads (every weight once, the live
requests' cache) against 8 TB/s; ``points`` holds decode at batch 1 and 64.

Before anything is timed, the tokens are checked (``check`` in the line): one request runs
a short prompt and eight greedy decode steps through the step function; its logits must be
finite, its tokens inside the vocabulary, and every token must be the plain implementation's
choice (``tests/plain``, float32 on the CPU, the same weights) or tie with it within the
rounding noise of bfloat16.  The 2,048-token prompt that ``prefill`` times is checked on two
layers of the same sizes (``check_prefill``).  ``--check basic`` leaves the plain implementation out,
``--check none`` all of it; the 70b shape only runs the basic check.

Other workloads print a line of their own: ``--only-prefill``, ``--mixed`` (64 requests
with prompts of 16 to 2,048 tokens in portions of 512), ``--long-prompt N`` (time to the
first token of one N-token prompt in portions of 2,048), ``--sweep`` (decode at further
batch sizes and context lengths, a line each with its share of the memory bandwidth);
``--model 1b|70b`` and ``--batch`` change the shape.
"""

from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

LLAMA3_8B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32,
    "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336, "vocab_size": 128256,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "tie_word_embeddings": False, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192,
    "hidden_act": "silu",
}
LLAMA32_1B = dict(LLAMA3_8B, num_hidden_layers=16, hidden_size=2048, num_attention_heads=32,
                  num_key_value_heads=8, head_dim=64, intermediate_size=8192,
                  rope_scaling=dict(LLAMA3_8B["rope_scaling"], factor=32.0), tie_word_embeddings=True)
LLAMA31_70B = dict(LLAMA3_8B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                   num_key_value_heads=8, head_dim=128, intermediate_size=28672)
MODELS = {"8b": ("llama-3-8b-shape-random", LLAMA3_8B), "1b": ("llama-3.2-1b-shape-random", LLAMA32_1B),
          "70b": ("llama-3.1-70b-shape-random", LLAMA31_70B)}
CONTEXT_LEN = 8192
PROMPT_LEN = 512
NEW_TOKENS = 256
PREFILL_TOKENS = 2048
PAGE_SIZE = 16
HBM_PEAK = 8.0e12          # bytes/s, MI355X
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=128)
    p.add_argument("--warmup", type=int, default=16)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the model has")
    p.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    p.add_argument("--model", default="8b", choices=sorted(MODELS),
                   help="layer sizes: 8b is the headline configuration; 1b and 70b are the other "
                        "shapes of the baseline")
    p.add_argument("--prompt-len", type=int, default=None,
                   help="prompt length of the decode runs (default 512; 1,024 for the 70b shape)")
    p.add_argument("--mixed", action="store_true",
                   help="instead of the decode runs: 64 requests with prompts of 16..2048 tokens, "
                        "portions of 512, 128 new tokens each, timed as a whole")
    p.add_argument("--long-prompt", type=int, default=0, metavar="N",
                   help="time to the first token of one N-token prompt, in portions of 2,048 "
                        "tokens; prints its own line")
    p.add_argument("--page-size", type=int, default=PAGE_SIZE, help="tokens a cache page")
    p.add_argument("--pack-weights", action=argparse.BooleanOptionalAction, default=None,
                   help="second copy of the weights in the order decode steps stream them "
                        "(default: where the device has room, as the engine decides)")
    p.add_argument("--sampling", default=None, metavar="T[,K[,P]]",
                   help="sample with this temperature, top-k and top-p (seeded) instead of greedily; "
                        "not the contract's line: say so with --no-points")
    p.add_argument("--no-points", action="store_true", help="skip batch 1 and 64 and the prefill")
    p.add_argument("--only-prefill", action="store_true",
                   help="run only the 2,048-token prefill (for profiling); prints its own line")
    p.add_argument("--check", default=None, choices=["plain", "basic", "none"],
                   help="check the tokens before timing: against the plain implementation on the CPU "
                        "(default for the 8b and 1b shapes), finite logits and tokens in range only, "
                        "or not at all")
    p.add_argument("--sweep", action="store_true",
                   help="instead of the default run: decode at batch 1..64 and at contexts of 8k, 32k "
                        "and 128k tokens, a line each")
    return p.parse_args()


def check_tokens(engine, cfg, mode, dtype_name):
    """A short prompt and eight greedy decode steps through the engine's own step function and
    cache; returns the record for the result line, raises if the tokens are not right."""
    import torch

    from kvcore_amd.engine.runner import StepEntry

    rng = random.Random(7)
    vocab = cfg["vocab_size"]
    prompt = [rng.randrange(vocab) for _ in range(40)]
    manager, runner = engine.kv_manager, engine.runner
    rid = "bench-check"
    manager.admit(rid)
    slot = manager.slot_of(rid)
    runner.forget(slot)
    tokens, rows = [], []
    ids, start = list(prompt), 0
    for step in range(9):  # the prompt, then eight single tokens (the second is captured as a graph)
        assert manager.allocate(rid, start, len(ids)) is not None
        out = runner.step([StepEntry(rid, slot, start, ids, manager.page_ids(rid), (len(ids) - 1,),
                                     manager.released_counts(rid))])
        row = out.logits[0].float().cpu()
        if not bool(torch.isfinite(row).all()):
            raise RuntimeError(f"bench check: step {step} gave logits that are not finite")
        tok = int(row.argmax())
        if not 0 <= tok < vocab:
            raise RuntimeError(f"bench check: token {tok} outside the vocabulary")
        rows.append(row)
        tokens.append(tok)
        start += len(ids)
        ids = [tok]
    runner.forget(slot)
    manager.free(rid)
    record = {"tokens": len(tokens), "finite": True, "in_range": True}
    if mode != "plain":
        return record
    from tests.plain import llama as plain

    t0 = time.perf_counter()
    weights = {}
    for name, (bp, row, nrows) in engine.model.checkpoint_map().items():
        weights[name] = bp.tensor.narrow(0, row, nrows).float().cpu()
    sequence = prompt + tokens[:-1]
    logits = plain.llama_forward(cfg, weights, sequence, dtype=torch.float32)
    del weights
    agree, worst, worst_noise = 0, 0.0, 0.0
    for i, tok in enumerate(tokens):
        ref = logits[len(prompt) - 1 + i]
        rms = float(ref.pow(2).mean().sqrt())
        gap = float(ref.max() - ref[tok]) / rms           # how much the plain logits prefer another token
        noise = float((rows[i] - ref).pow(2).mean().sqrt()) / rms
        agree += int(ref.argmax()) == tok
        worst, worst_noise = max(worst, gap), max(worst_noise, noise)
    # bfloat16 rounds activations at a dozen places a layer, so a row of logits carries noise
    # that grows like the square root of the depth: 0.9 to 1.2% of the row's root mean square
    # at two layers of these sizes, 5.2% at 32.  The bound is 1.7% at two layers times
    # sqrt(layers / 2), 1.3 times what is measured at 32 layers; a wrong kernel, page or
    # position gives 100% and more.  A token may lose to another by no more than a few times
    # that noise.
    layers = cfg["num_hidden_layers"]
    noise_bound = round(0.017 * (layers / 2) ** 0.5, 4) if dtype_name == "bf16" else 2e-4
    record.update({"plain_agree": agree, "worst_gap_rms": round(worst, 5), "row_error_rms": round(worst_noise, 5),
                   "bound_rms": noise_bound, "plain_seconds": round(time.perf_counter() - t0, 1)})
    if worst_noise > noise_bound or worst > 5 * noise_bound:
        raise RuntimeError(f"bench check: the engine's tokens are not the plain implementation's: {record}")
    return record


def check_prefill(cfg, dtype, dtype_name, page_size):
    """The logits of the prompt that ``prefill`` times.  The plain implementation cannot follow
    2,048 tokens through all the layers in reasonable time, so the prompt runs through a model
    of two layers with the same layer sizes and a vocabulary of 384 (every kernel of a layer
    is launched as in the timed step: same rows, same widths, same variants), in one step,
    and twelve of its positions are compared with the plain implementation in float32 on the
    CPU.  The bound is that of the test suite for rows of so few logits: 1.5% of the logits'
    root mean square, plus 4/sqrt(384) of that for the scatter of a row (1.28% measured on
    average, 1.71% at most over all 2,048 rows)."""
    import torch

    from kvcore_amd.cache.kv_manager import KVManager, plan_groups
    from kvcore_amd.engine.runner import ModelRunner, StepEntry, build_model
    from tests.plain import llama as plain

    small = dict(cfg, num_hidden_layers=2, vocab_size=384, tie_word_embeddings=False)
    t0 = time.perf_counter()
    model = build_model(".", dtype, "cuda:0", load_format="random", seed=3, config_override=small,
                        pack_weights=False)
    pages = PREFILL_TOKENS // page_size + 2
    groups = plan_groups([g.need for g in model.cache_groups], page_size, pages)
    manager = KVManager(groups, max_num_seqs=1, max_model_len=PREFILL_TOKENS)
    runner = ModelRunner(model, page_size=[g.page_size for g in groups], num_pages=[g.num_pages for g in groups],
                         max_num_seqs=1, max_num_tokens=PREFILL_TOKENS, max_model_len=PREFILL_TOKENS)
    rng = random.Random(11)
    prompt = [rng.randrange(small["vocab_size"]) for _ in range(PREFILL_TOKENS)]
    want = (0, 15, 16, 63, 64, 127, 128, 1023, 1024, 1535, 2046, 2047)
    manager.admit("p")
    assert manager.allocate("p", 0, PREFILL_TOKENS) is not None
    out = runner.step([StepEntry("p", manager.slot_of("p"), 0, prompt, manager.page_ids("p"), want)])
    rows = out.logits.float().cpu()
    weights = {}
    for name, (bp, row, nrows) in model.checkpoint_map().items():
        weights[name] = bp.tensor.narrow(0, row, nrows).float().cpu()
    del runner, model
    logits = plain.llama_forward(small, weights, prompt, dtype=torch.float32)
    worst = 0.0
    for i, pos in enumerate(want):
        ref = logits[pos]
        if not bool(torch.isfinite(rows[i]).all()):
            raise RuntimeError(f"bench check: the prefill's logits at position {pos} are not finite")
        worst = max(worst, float((rows[i] - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt()))
    bound = round(0.015 * (1 + 4 / small["vocab_size"] ** 0.5), 4) if dtype_name == "bf16" else 2e-4
    record = {"prefill_rows": len(want), "prefill_row_error_rms": round(worst, 5), "prefill_bound_rms": bound,
              "prefill_plain_seconds": round(time.perf_counter() - t0, 1)}
    if worst > bound:
        raise RuntimeError(f"bench check: the 2,048-token prefill's logits are not the plain "
                           f"implementation's: {record}")
    return record


def weight_bytes_per_step(cfg, esize):
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, d, L = (cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                     cfg["num_hidden_layers"])
    per_layer = (nh + 2 * nkv) * d * H + nh * d * H + 3 * I * H
    return (L * per_layer + V * H) * esize


def kv_bytes(cfg, batch, ctx, esize):
    return batch * ctx * 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * esize


def prefill_flops(cfg, T, S=1):
    H, I, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, d, L = (cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                     cfg["num_hidden_layers"])
    per_layer = (nh + 2 * nkv) * d * H + nh * d * H + 3 * I * H
    return 2 * T * L * per_layer + 4 * d * nh * L * T * (T + 1) // 2 + 2 * S * V * H


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    import torch

    from kvcore_amd import (CacheConfig, DeviceConfig, KVCoreConfig, LoadConfig, ModelConfig,
                            SamplingParams, SchedulerConfig)
    from kvcore_amd.engine.engine_core import EngineCore
    from kvcore_amd.engine.runner import build_model
    from kvcore_amd.ops import library as ops_library

    model_name, base_cfg = MODELS[args.model]
    cfg = dict(base_cfg)
    prompt_len = args.prompt_len or (1024 if args.model == "70b" else PROMPT_LEN)
    full_layers = cfg["num_hidden_layers"]
    if args.layers is not None:
        cfg["num_hidden_layers"] = args.layers
    dtype = {"bf16": torch.bfloat16, "fp32": torch.float32}[args.dtype]
    esize = 2 if args.dtype == "bf16" else 4
    device = "cuda:0"
    torch.cuda.set_device(0)

    t0 = time.perf_counter()
    model = build_model(".", dtype, device, load_format="random", seed=0, config_override=cfg,
                        pack_weights=args.pack_weights)
    print(f"[bench] model built in {time.perf_counter() - t0:.1f} s, "
          f"{model.num_param_bytes() / 2**30:.2f} GiB", file=sys.stderr, flush=True)

    max_seqs = max(64, args.batch)  # request slots of the engine: every request of the batch decodes in every step
    pages_per_seq = -(-(PREFILL_TOKENS + NEW_TOKENS + prompt_len) // args.page_size)
    if args.long_prompt:
        max_seqs, pages_per_seq = 2, -(-(args.long_prompt + 16) // args.page_size)

    def make_engine(max_model_len, seqs, pages):
        return EngineCore(KVCoreConfig(
            model_config=ModelConfig(model=".", dtype=args.dtype, max_model_len=max_model_len),
            load_config=LoadConfig(load_format="random", seed=0),
            cache_config=CacheConfig(block_size=args.page_size, num_gpu_blocks=pages),
            scheduler_config=SchedulerConfig(max_num_seqs=seqs, max_num_scheduled_tokens=PREFILL_TOKENS,
                                             max_num_partial_prefills=seqs, max_long_partial_prefills=seqs),
            device_config=DeviceConfig(device=device),
        ), model=model)

    # the 70b shape fills most of the device: its cache is what the engine's own profile steps
    # find room for; the other shapes get what the runs below can use
    context_len = 4096 if args.model == "70b" else CONTEXT_LEN  # what the baseline names for each shape
    engine = make_engine(max(context_len, args.long_prompt + 16), max_seqs,
                         None if args.model == "70b" else max_seqs * pages_per_seq + 1)
    if engine.memory_profile is not None:
        print(f"[bench] cache sized by the engine: {engine.num_pages} pages of {args.page_size} tokens "
              f"({engine.runner.cache_bytes() / 2**30:.1f} GiB)", file=sys.stderr, flush=True)
    rng = random.Random(0)
    vocab = cfg["vocab_size"]
    counter = [0]
    check_mode = args.check or ("basic" if args.model == "70b" or args.only_prefill or args.mixed
                                or args.long_prompt or args.sweep else "plain")
    check = None
    if check_mode != "none":
        check = check_tokens(engine, cfg, check_mode, args.dtype)
        if check_mode == "plain" and not args.no_points:
            check.update(check_prefill(cfg, dtype, args.dtype, args.page_size))
        print(f"[bench] check: {check}", file=sys.stderr, flush=True)

    sampling = {"temperature": 0.0}
    if args.sampling:
        if not args.no_points:
            print("bench.py: --sampling is not the contract's greedy line; pass --no-points with it", file=sys.stderr)
            return 2
        parts = [float(v) for v in args.sampling.split(",")]
        sampling = {"temperature": parts[0], "seed": 1}
        if len(parts) > 1:
            sampling["top_k"] = int(parts[1])
        if len(parts) > 2:
            sampling["top_p"] = parts[2]

    def new_request(n_prompt, n_new, eng=None):
        counter[0] += 1
        rid = f"bench-{counter[0]}"
        ids = [rng.randrange(vocab) for _ in range(n_prompt)]
        (eng or engine).add_request(rid, SamplingParams(max_tokens=n_new, ignore_eos=True, **sampling),
                                    prompt_token_ids=ids)
        return rid

    def drain():
        while engine.has_unfinished_requests():
            engine.step()

    def decode_run(batch, steps, warmup, eng=None, p_len=None):
        """tokens/s over exactly `steps` decode steps at `batch`, after `warmup` of them."""
        eng = eng or engine
        p_len = p_len or prompt_len
        slack = -(-batch * p_len // PREFILL_TOKENS) + 2  # steps others decode while prompts run
        for _ in range(batch):
            new_request(p_len, warmup + steps + 1 + slack, eng)
        # prompts first; a request samples its first token when its prompt ends
        while any(r.num_computed_tokens < r.num_prompt_tokens
                  for r in eng.scheduler.requests.values()):
            eng.step()
        for _ in range(warmup):
            eng.step()
        ctx_start = p_len + 1 + warmup
        torch.cuda.synchronize()
        t_start = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t_start
        eng.abort_requests(None)
        mean_ctx = ctx_start + steps / 2
        return batch * steps / elapsed, elapsed / steps, mean_ctx

    def decode_line(batch, steps, warmup, eng=None, p_len=None):
        v, sec, ctx = decode_run(batch, steps, warmup, eng, p_len)
        need = weight_bytes_per_step(cfg, esize) + kv_bytes(cfg, batch, ctx, esize)
        return {"workload": "decode", "model": model_name, "dtype": args.dtype, "batch": batch,
                "context": int(ctx), "tokens_per_s": round(v, 1), "ms_per_step": round(sec * 1e3, 4),
                "gb_per_step": round(need / 1e9, 3), "hbm_gb_per_s": round(need / sec / 1e9, 1),
                "hbm_frac": round(need / sec / HBM_PEAK, 4)}

    def prefill_run():
        times = []
        for i in range(4):
            new_request(PREFILL_TOKENS, 1)
            torch.cuda.synchronize()
            t_start = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t_start)
            drain()
        return sorted(times[1:])[1]  # median of the three after the warm-up run

    def context_engine(ctx_len, b):
        """An engine whose requests may reach ``ctx_len`` tokens of context."""
        room = ctx_len + 128
        return make_engine(room, b, b * -(-room // args.page_size) + 1)

    def context_line(ctx_len, b, eng, steps=32, warmup=4):
        # every request stays below ctx_len for the whole run (requests whose prompts end
        # first decode while the others' prompts run), so that no step of the timed
        # region is the first of a longer length class and captures its graph there
        ahead = -(-b * ctx_len // PREFILL_TOKENS) + 2 + warmup + steps + 8
        return decode_line(b, steps, warmup, eng, ctx_len - ahead)

    def first_token_run(n, eng, runs=3):
        """Seconds to the first token of one ``n``-token prompt in portions of 2,048."""
        times = []
        for i in range(runs):
            new_request(n, 1, eng)
            torch.cuda.synchronize()
            t_start = time.perf_counter()
            while eng.has_unfinished_requests():
                eng.step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t_start)
        return min(times[1:])

    if args.sweep:
        for b in (1, 2, 4, 8, 9, 12, 16, 24, 32, 48, 64):
            print(json.dumps(decode_line(b, 48, 8)), flush=True)
        del engine
        for ctx_len, batches in ((8192, (1, 8)), (32768, (1, 8)), (131072, (1,))):
            for b in batches:
                eng = context_engine(ctx_len, b)
                print(json.dumps(context_line(ctx_len, b, eng)), flush=True)
                del eng
                torch.cuda.empty_cache()
        eng = make_engine(context_len, 256, 256 * pages_per_seq + 1)
        for b in (96, 128, 192, 256):
            print(json.dumps(decode_line(b, 32, 4, eng)), flush=True)
        return 0
    if args.long_prompt:
        sec = first_token_run(args.long_prompt, engine)
        print(json.dumps({"workload": f"first token of a {args.long_prompt}-token prompt in portions of "
                                      f"{PREFILL_TOKENS}", "model": model_name, "dtype": args.dtype,
                          "ms": round(sec * 1e3, 2), "tokens_per_s": round(args.long_prompt / sec, 1),
                          "frac": round(prefill_flops(cfg, args.long_prompt) / sec / PEAK_FLOPS[args.dtype], 4)}))
        return 0
    if args.mixed:
        engine.scheduler.config = SchedulerConfig(
            max_num_seqs=max_seqs, max_num_scheduled_tokens=PREFILL_TOKENS, max_num_partial_prefills=max_seqs,
            max_long_partial_prefills=max_seqs, long_prefill_token_threshold=512)
        lens = [rng.randrange(16, 2049) for _ in range(64)]
        runs = []
        for _ in range(2):  # the first pass also captures the graphs of the decode steps it meets
            for n in lens:
                new_request(n, 128)
            torch.cuda.synchronize()
            t_start = time.perf_counter()
            steps = 0
            while engine.has_unfinished_requests():
                engine.step()
                steps += 1
            torch.cuda.synchronize()
            runs.append(time.perf_counter() - t_start)
        sec = runs[1]
        print(json.dumps({"workload": "mixed: 64 requests, prompts U[16,2048], portions of 512, 128 new tokens",
                          "model": model_name, "dtype": args.dtype, "seconds": round(sec, 4),
                          "first_pass_seconds": round(runs[0], 4), "steps": steps,
                          "prompt_tokens": sum(lens), "generated_tokens": 64 * 128,
                          "generated_tokens_per_s": round(64 * 128 / sec, 1),
                          "total_tokens_per_s": round((sum(lens) + 64 * 128) / sec, 1)}))
        return 0
    if args.only_prefill:
        sec = prefill_run()
        print(json.dumps({"prefill_tokens": PREFILL_TOKENS, "ms": round(sec * 1e3, 3),
                          "tokens_per_s": round(PREFILL_TOKENS / sec, 1),
                          "frac": round(prefill_flops(cfg, PREFILL_TOKENS) / sec / PEAK_FLOPS[args.dtype], 4)}))
        return 0
    # what a kernel that only reads, and one that only multiplies, reach on this chip: the
    # second yardstick beside the data sheet's
    peaks = ops_library.measure_peaks(device)
    measured_hbm, measured_mfma = peaks["read_bytes_per_s"], peaks["mfma_bf16_flops_per_s"]
    value, sec_per_step, mean_ctx = decode_run(args.batch, args.steps, args.warmup)
    bytes_step = weight_bytes_per_step(cfg, esize) + kv_bytes(cfg, args.batch, mean_ctx, esize)
    achieved = bytes_step / sec_per_step
    result = {
        "metric": f"decode tok/s ({model_name}, batch {args.batch}, {prompt_len}-token prompts)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(sec_per_step * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {
            "model": model_name, "layers": cfg["num_hidden_layers"],
            "layers_full": full_layers, "hidden": cfg["hidden_size"],
            "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"],
            "vocab": cfg["vocab_size"], "global_batch": args.batch, "seq_len": context_len,
            "prompt_len": prompt_len, "new_tokens": NEW_TOKENS, "page_size": args.page_size,
            "prefill_tokens": PREFILL_TOKENS, "parallelism": "single-gpu",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK, 4),
                     "measured_read_peak": round(measured_hbm / 1e9, 1),
                     "frac_of_measured": round(achieved / measured_hbm, 4)},
    }
    if check is not None:
        result["check"] = check
    if not args.no_points:
        sec = prefill_run()
        flops = prefill_flops(cfg, PREFILL_TOKENS)
        result["prefill"] = {"value": round(PREFILL_TOKENS / sec, 1), "tokens": PREFILL_TOKENS,
                             "ms": round(sec * 1e3, 3),
                             "frac": round(flops / sec / PEAK_FLOPS[args.dtype], 4)}
        if args.dtype == "bf16":
            result["prefill"]["measured_mfma_peak_tflops"] = round(measured_mfma / 1e12, 1)
            result["prefill"]["frac_of_measured"] = round(flops / sec / measured_mfma, 4)
        points = {}
        for b in (1, 16, 32, 64):
            steps = max(16, min(args.steps, 64))
            v, sec_b, ctx_b = decode_run(b, steps, min(args.warmup, 8))
            points[f"decode_b{b}"] = round(v, 2)
            need = weight_bytes_per_step(cfg, esize) + kv_bytes(cfg, b, ctx_b, esize)
            points[f"decode_b{b}_hbm_frac"] = round(need / sec_b / HBM_PEAK, 4)
        if args.model != "70b":
            # further sizes: decode with 8k and 32k tokens of context a request (a length class
            # each), and the time to the first token of an 8,192-token prompt in portions of 2,048
            del engine
            torch.cuda.empty_cache()
            for ctx_len, key in ((8192, "8k"), (32768, "32k")):
                eng = context_engine(ctx_len, 8)
                line = context_line(ctx_len, 8, eng, steps=24, warmup=4)
                points[f"decode_b8_ctx{key}"] = line["tokens_per_s"]
                points[f"decode_b8_ctx{key}_ms"] = line["ms_per_step"]
                points[f"decode_b8_ctx{key}_hbm_frac"] = line["hbm_frac"]
                if ctx_len == 8192:
                    sec_first = first_token_run(8192, eng)
                    points["first_token_8192_ms"] = round(sec_first * 1e3, 2)
                    points["first_token_8192_frac"] = round(
                        prefill_flops(cfg, 8192) / sec_first / PEAK_FLOPS[args.dtype], 4)
                del eng
                torch.cuda.empty_cache()
        result["points"] = points
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
