"""Offline batch generation from the command line.

Reference: scripts/run_llm_engine_offline_batch.py:127-271: the option names and
meanings it has are kept (``--model --device --block-size --max-model-len
--max-num-seqs --max-num-scheduled-tokens --max-num-partial-prefills
--max-long-partial-prefills --long-prefill-token-threshold --attn-backend
--local-files-only --log-level --log-file``; ``--revision`` and ``--trust-remote-code``
are recognised and refused or ignored, since models are local folders and no code of
theirs is ever run),
as are its output sections (run metadata, request summary, outputs, timing summary).
Its hard-coded chat requests are not: requests come from ``--requests FILE`` (a JSON
list of ``{"request_id", "messages" | "prompt_token_ids", "max_tokens", "temperature",
...}``) or are synthetic token prompts of ``--prompt-lens``.
"""

from __future__ import annotations

import argparse
import contextlib
import json
import random
import sys
import time
from datetime import datetime
from pathlib import Path


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(description="Run offline batch generation through LLMEngine.")
    p.add_argument("--model", required=True, help="model folder (config.json, *.safetensors)")
    p.add_argument("--device", default="cuda:0")
    p.add_argument("--attn-backend", default=None, choices=["hip"],
                   help="Attention backend override. Defaults to KVCoreConfig auto selection.")
    p.add_argument("--revision", default=None, help="not supported: models are local folders")
    p.add_argument("--trust-remote-code", action="store_true",
                   help="accepted and ignored: no code from a model folder is ever run")
    p.add_argument("--local-files-only", action=argparse.BooleanOptionalAction, default=True,
                   help="models are always read from local folders; --no-local-files-only is refused")
    p.add_argument("--dtype", default=None, choices=[None, "bfloat16", "bf16", "float32", "fp32"])
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--max-model-len", type=int, default=None)
    p.add_argument("--max-num-seqs", type=int, default=1024)
    p.add_argument("--max-num-scheduled-tokens", type=int, default=1024)
    p.add_argument("--max-num-partial-prefills", type=int, default=128)
    p.add_argument("--max-long-partial-prefills", type=int, default=128)
    p.add_argument("--long-prefill-token-threshold", type=int, default=0)
    p.add_argument("--decode-run-ahead", action=argparse.BooleanOptionalAction, default=True,
                   help="while requests only decode, launch the next step before the tokens of the "
                        "step in flight have reached the host")
    p.add_argument("--pack-decode-weights", action=argparse.BooleanOptionalAction, default=None,
                   help="keep a second copy of the weight matrices in the order decode steps stream "
                        "them (default: where the device has room)")
    p.add_argument("--num-gpu-blocks", type=int, default=None)
    p.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    p.add_argument("--poison-pages", action="store_true",
                   help="debugging aid: fill every cache page with NaN when a request gets it and "
                        "when it is given back")
    p.add_argument("--random-weights", action="store_true",
                   help="fill the parameters from --seed; the folder needs only config.json")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--requests", default=None, help="JSON file with a list of requests")
    p.add_argument("--prompt-lens", default="7,16,33,50",
                   help="synthetic prompts of these lengths when --requests is not given")
    p.add_argument("--max-tokens", type=int, default=16)
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--log-level", default="INFO")
    p.add_argument("--log-file", default=None,
                   help="Path for teeing terminal output. Defaults to logs/<script>_<timestamp>.log.")
    p.add_argument("--no-log-file", action="store_true", help="do not tee to a file")
    args = p.parse_args(argv)
    if args.revision is not None or not args.local_files_only:
        p.error("models are read from local folders only: --revision and --no-local-files-only "
                "have no meaning here")
    return args


class _Tee:
    def __init__(self, *streams):
        self.streams = streams

    def write(self, data):
        for s in self.streams:
            s.write(data)
        return len(data)

    def flush(self):
        for s in self.streams:
            s.flush()


@contextlib.contextmanager
def tee_terminal_output(path: Path | None):
    if path is None:
        yield
        return
    path.parent.mkdir(parents=True, exist_ok=True)
    with open(path, "w", encoding="utf-8") as f:
        out, err = sys.stdout, sys.stderr
        sys.stdout, sys.stderr = _Tee(out, f), _Tee(err, f)
        try:
            yield
        finally:
            sys.stdout, sys.stderr = out, err


def build_config(args: argparse.Namespace):
    from kvcore_amd import (CacheConfig, DeviceConfig, KVCoreConfig, LoadConfig, ModelConfig,
                            SchedulerConfig)

    return KVCoreConfig(
        model_config=ModelConfig(model=str(Path(args.model).expanduser()), dtype=args.dtype,
                                 max_model_len=args.max_model_len, attn_backend=args.attn_backend),
        load_config=LoadConfig(load_format="random" if args.random_weights else "safetensors",
                               seed=args.seed, pack_decode_weights=args.pack_decode_weights),
        cache_config=CacheConfig(block_size=args.block_size, num_gpu_blocks=args.num_gpu_blocks,
                                 gpu_memory_utilization=args.gpu_memory_utilization,
                                 poison_pages=args.poison_pages),
        scheduler_config=SchedulerConfig(
            max_num_seqs=args.max_num_seqs,
            max_num_scheduled_tokens=args.max_num_scheduled_tokens,
            max_num_partial_prefills=args.max_num_partial_prefills,
            max_long_partial_prefills=args.max_long_partial_prefills,
            long_prefill_token_threshold=args.long_prefill_token_threshold,
            decode_run_ahead=args.decode_run_ahead,
        ),
        device_config=DeviceConfig(device=args.device),
    )


def build_generation_requests(args: argparse.Namespace, vocab_size: int):
    from kvcore_amd import SamplingParams
    from kvcore_amd.engine.llm_engine import GenerationRequest

    def params(spec: dict) -> SamplingParams:
        return SamplingParams(
            max_tokens=int(spec.get("max_tokens", args.max_tokens)),
            temperature=float(spec.get("temperature", args.temperature)),
            top_p=float(spec.get("top_p", args.top_p)),
            top_k=spec.get("top_k", args.top_k),
            seed=spec.get("seed", args.seed),
            ignore_eos=bool(spec.get("ignore_eos", args.ignore_eos)),
        )

    requests = []
    if args.requests:
        specs = json.loads(Path(args.requests).read_text())
        for i, spec in enumerate(specs):
            requests.append(GenerationRequest(
                request_id=str(spec.get("request_id", f"req-{i}")),
                sampling_params=params(spec),
                messages=None if spec.get("messages") is None else tuple(spec["messages"]),
                prompt_token_ids=None if spec.get("prompt_token_ids") is None
                else tuple(int(t) for t in spec["prompt_token_ids"]),
            ))
    else:
        rng = random.Random(args.seed)
        for i, n in enumerate(int(x) for x in args.prompt_lens.split(",") if x):
            ids = tuple(rng.randrange(vocab_size) for _ in range(n))
            requests.append(GenerationRequest(f"req-{i}", params({}), prompt_token_ids=ids))
    if not requests:
        raise ValueError("no requests: give --requests or --prompt-lens")
    return requests


def main(argv=None) -> int:
    program_start = time.perf_counter()
    args = parse_args(argv)
    log_path = None
    if not args.no_log_file:
        stamp = datetime.now().strftime("%Y%m%d_%H%M%S")
        log_path = Path(args.log_file) if args.log_file else Path("logs") / f"offline_batch_{stamp}.log"
    with tee_terminal_output(log_path):
        from kvcore_amd.engine.llm_engine import LLMEngine
        from kvcore_amd.engine.log import configure_logging

        configure_logging(args.log_level, force=True)
        print("=== Run Metadata ===")
        print(f"start_time={datetime.now().astimezone().isoformat(timespec='seconds')}")
        print(f"log_file={log_path}")
        print(f"model={Path(args.model).expanduser()}")
        print(f"device={args.device}")
        print(f"dtype={args.dtype}")
        print(f"random_weights={args.random_weights}")
        print(f"block_size={args.block_size}")
        print(f"max_num_seqs={args.max_num_seqs}")
        print(f"max_num_scheduled_tokens={args.max_num_scheduled_tokens}")

        engine_start = time.perf_counter()
        config = build_config(args)
        print(f"attn_backend={config.model_config.attn_backend}")
        if args.trust_remote_code:
            print("trust_remote_code is ignored: no code from a model folder is ever run")
        engine = LLMEngine(config)
        engine_elapsed = time.perf_counter() - engine_start
        print(f"engine_init_sec={engine_elapsed:.3f}")
        core = engine.engine_core
        print(f"num_gpu_blocks={core.num_pages}")
        print(f"kv_bytes_per_block={core.bytes_per_page()}")
        print(f"kv_cache_bytes={core.runner.cache_bytes()}")
        if core.memory_profile is not None:  # the cache was sized by the profile steps
            for name, value in vars(core.memory_profile).items():
                print(f"memory_profile.{name}={value}")

        requests = build_generation_requests(args, engine.engine_core.model.spec.vocab_size)
        print("\n=== Requests ===")
        for r in requests:
            size = len(r.prompt_token_ids) if r.prompt_token_ids is not None else len(r.messages or ())
            kind = "tokens" if r.prompt_token_ids is not None else "messages"
            print(f"[{r.request_id}] {kind}={size} max_tokens={r.sampling_params.max_tokens} "
                  f"temperature={r.sampling_params.temperature}")

        generate_start = time.perf_counter()
        outputs = engine.generate(requests)
        generate_elapsed = time.perf_counter() - generate_start

        print("\n=== Detokenized Outputs ===")
        for output in outputs:
            print(f"\n[{output.request_id}] finish_reason={output.finish_reason}")
            print(f"token_ids={output.output_token_ids}")
            print(output.output_text)

        generated = sum(len(o.output_token_ids) for o in outputs)
        print("\n=== Timing Summary ===")
        print(f"end_time={datetime.now().astimezone().isoformat(timespec='seconds')}")
        print(f"num_requests={len(requests)}")
        print(f"generated_tokens={generated}")
        print(f"engine_init_sec={engine_elapsed:.3f}")
        print(f"generate_sec={generate_elapsed:.3f}")
        print(f"total_elapsed_sec={time.perf_counter() - program_start:.3f}")
        if args.device.startswith("cuda"):
            import torch

            free, total = torch.cuda.mem_get_info(torch.device(args.device))
            print("\n=== Device Memory ===")
            print(f"device_total_bytes={total}")
            print(f"device_used_bytes={total - free}")
            print(f"torch_reserved_bytes={torch.cuda.memory_reserved(torch.device(args.device))}")
            print(f"torch_peak_allocated_bytes={torch.cuda.max_memory_allocated(torch.device(args.device))}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
