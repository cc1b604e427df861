"""Trace replay: feeds given token ids through a model step by step and writes logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step run as one batch through the engine's own model, step function,
cache manager and kernels.  For a step in which logits are wanted, ``<out>/<step>.f32``
holds them as little-endian float32 ``[wanted, vocab]`` in the order of the entries and
of ``want``.  After every step a line ``done <step>`` is printed.  Nothing is sampled.

The reference has no such program; its tests drive ``execute_model`` with hand-built
scheduler outputs instead (tests/test_model_runner_kv_boundary.py:119-134).
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens live requests hold at any time (each rounded up to 64)")
    p.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    p.add_argument("--max-num-seqs", type=int, default=8, help="request slots")
    p.add_argument("--device", default="cuda:0")
    p.add_argument("--poison-cache", action="store_true",
                   help="fill the cache with NaN first, so a read of a slot nobody wrote shows")
    p.add_argument("--shuffle-pages", type=int, default=None, metavar="SEED",
                   help="hand pages out in a seeded random order (the logits must not change)")
    p.add_argument("--show-pages", action="store_true",
                   help="print each step's page ids per request on standard error")
    return p.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.max_tokens <= 0:
        print("trace_run: --max-tokens must be positive", file=sys.stderr)
        return 2
    print("trace_run: loading (kernels are compiled at the first call)", file=sys.stderr, flush=True)
    import numpy as np
    import torch

    from kvcore_amd.engine.replay import TraceSession
    from kvcore_amd.ops import library as ops

    ops.load()
    if not torch.cuda.is_available():
        print("trace_run: no GPU is visible; this engine has no CPU path", file=sys.stderr)
        return 3
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    session = TraceSession(args.model, dtype, max_tokens=args.max_tokens, block_size=args.block_size,
                           max_num_seqs=args.max_num_seqs, device=args.device,
                           poison_cache=args.poison_cache, shuffle_pages=args.shuffle_pages)
    print("trace_run: ready", file=sys.stderr, flush=True)

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        if args.show_pages:
            live_before = {str(item["id"]) for item in record.get("entries", [])}
        out = session.run_step(record)
        if args.show_pages:
            pages = {rid: session.manager.page_ids(rid) for rid in sorted(live_before)
                     if session.manager.is_admitted(rid)}
            print(f"pages {record['step']} {json.dumps(pages)}", file=sys.stderr, flush=True)
        if out is not None and out.logits is not None:
            host = out.logits.detach().to("cpu", torch.float32).numpy()
            np.ascontiguousarray(host, dtype="<f4").tofile(out_dir / f"{record['step']}.f32")
        else:
            torch.cuda.synchronize()
        print(f"done {record['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
