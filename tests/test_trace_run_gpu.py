"""bin/trace_run as a user runs it: a child process, steps on its standard input, one
``done`` line per step, logits in files; and long decoding through the same session."""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from tests.helpers import CONFIGS, make_model_dir, random_tokens, tolerance
from tests.plain import llama as plain

pytestmark = pytest.mark.gpu
REPO = Path(__file__).resolve().parent.parent


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    config, page = CONFIGS["A"]
    folder = make_model_dir(tmp_path / "model", config, seed=5)
    cfg, weights = plain.load_model_folder(folder)
    V = cfg["vocab_size"]
    a, b, c = random_tokens(50, V, 1), random_tokens(40, V, 2), random_tokens(70, V, 3)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:18], "want": [0, 17]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:39], "want": []},
                                {"id": "a", "tokens": a[18:20], "want": [0, 1]}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[20:50], "want": [29]},
                                {"id": "b", "tokens": b[39:40], "want": [0]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [0, 33, 69]}], "end": ["c"]},
        {"step": 4, "entries": [], "end": []},
    ]
    expect = {0: [("a", 0), ("a", 17)], 1: [("a", 18), ("a", 19)], 2: [("a", 49), ("b", 39)],
              3: [("c", 0), ("c", 33), ("c", 69)]}
    out_dir = tmp_path / "out"
    # 128 tokens: a and b live together (64 + 64); c (70 -> 128) must reuse their pages
    proc = subprocess.Popen([sys.executable, str(REPO / "bin" / "trace_run"), "--model", str(folder),
                             "--dtype", dtype, "--out", str(out_dir), "--max-tokens", "128"],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for rec in steps:
            proc.stdin.write(json.dumps(rec) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {rec['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    oracle = {"a": plain.llama_forward(cfg, weights, a), "b": plain.llama_forward(cfg, weights, b),
              "c": plain.llama_forward(cfg, weights, c)}
    tol = tolerance(torch.float32 if dtype == "float32" else torch.bfloat16)
    assert sorted(p.name for p in out_dir.iterdir()) == ["0.f32", "1.f32", "2.f32", "3.f32"]
    for step, owners in expect.items():
        data = np.fromfile(out_dir / f"{step}.f32", dtype="<f4").reshape(len(owners), V)
        for row, (rid, pos) in zip(data, owners):
            assert torch.allclose(torch.from_numpy(row).double(), oracle[rid][pos], **tol), (step, rid, pos)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_long_decoding_and_first_tokens(tmp_path, dtype):
    """A sequence decoded one token at a time from its very first token, far past several
    pages and 64-key tiles: 400 steps of one token."""
    from kvcore_amd.engine.replay import TraceSession

    config, page = CONFIGS["C"]
    folder = make_model_dir(tmp_path / "model", config, seed=6)
    cfg, weights = plain.load_model_folder(folder)
    tokens = random_tokens(400, cfg["vocab_size"], 8)
    want = plain.llama_forward(cfg, weights, tokens)
    session = TraceSession(str(folder), dtype, max_tokens=448, block_size=page, poison_cache=True)
    tol = tolerance(dtype)
    for i, tok in enumerate(tokens):
        out = session.run_step({"step": i, "entries": [{"id": "r", "tokens": [tok], "want": [0]}], "end": []})
        row = out.logits[0].double().cpu()
        assert torch.allclose(row, want[i], **tol), f"position {i}"
