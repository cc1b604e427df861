"""How many cache pages the engine gives itself when nobody says: the branch in which the
device's memory, not the traffic, sets the number.

Reference: kvcore/model/model_runner.py:696-768 (a dummy forward at the step's token budget,
torch's peak, ``gpu_memory_utilization`` of the device minus that peak over the bytes of a
block).  The command line's own defaults (1,024 slots, 1,024 tokens a step) on the 8B shape
take that branch: every slot at full length would want a terabyte of pages.
"""

from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from tests.test_real_sizes_gpu import CONFIG as LAYERS_OF_8B

pytestmark = pytest.mark.gpu

REPO = Path(__file__).resolve().parent.parent


def fields(text: str) -> dict[str, str]:
    out = {}
    for line in text.splitlines():
        if "=" in line and not line.startswith("["):
            key, _, value = line.partition("=")
            out[key.strip()] = value.strip()
    return out


def test_command_line_defaults_size_the_cache_by_measurement(tmp_path):
    """``bin/kvcore_offline_batch --random-weights`` on the 8B shape with the default
    ``--max-num-seqs 1024 --max-num-scheduled-tokens 1024``: it must not run out of memory,
    must stay within ``gpu_memory_utilization`` of the device while it generates for eight
    prompts of 1,000 tokens, and must have given the cache what the device had left: within 3%
    of (0.9 x total - everything else the process and its neighbours hold at the end of the
    run) / bytes a page, "everything else" being read from the device after the generation,
    not from the engine's own profile."""
    config = dict(LAYERS_OF_8B, num_hidden_layers=32)
    (tmp_path / "config.json").write_text(json.dumps(config))
    torch.cuda.empty_cache()  # what this process has cached counts as a neighbour's
    cmd = [sys.executable, str(REPO / "bin" / "kvcore_offline_batch"), "--model", str(tmp_path),
           "--random-weights", "--dtype", "bf16", "--prompt-lens", ",".join(["1000"] * 8),
           "--max-tokens", "12", "--ignore-eos", "--seed", "5", "--log-level", "INFO", "--no-log-file"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-3000:] + proc.stderr[-3000:]
    got = fields(proc.stdout)
    assert (got["max_num_seqs"], got["max_num_scheduled_tokens"]) == ("1024", "1024")
    assert proc.stdout.count("finish_reason=length") == 8
    total = int(got["device_total_bytes"])
    used = int(got["device_used_bytes"])
    pages = int(got["num_gpu_blocks"])
    per_page = int(got["kv_bytes_per_block"])
    cache_bytes = int(got["kv_cache_bytes"])
    # 32 layers x keys and values x 8 heads x 16 tokens x 128 x 2 bytes
    assert per_page == 32 * 2 * 8 * 16 * 128 * 2
    assert cache_bytes == pages * per_page
    # the memory set the number: far fewer pages than every slot at full length would take
    assert pages == int(got["memory_profile.pages"]) < int(got["memory_profile.useful_pages"])
    assert used <= 0.9 * total, f"{used / 2**30:.1f} GiB in use of {total / 2**30:.1f}"
    assert int(got["torch_reserved_bytes"]) <= 0.9 * total
    room = 0.9 * total - (used - cache_bytes)
    assert abs(pages * per_page - room) <= 0.03 * room, (
        f"{pages} pages take {pages * per_page / 2**30:.1f} GiB; the device had {room / 2**30:.1f} GiB "
        f"for them")
    # more than a million tokens of cache on this device
    assert pages * 16 > 1_000_000


def test_a_tiny_model_gets_what_its_slots_can_use(tmp_path):
    """Where every slot at full length needs less than the device has, that is the number,
    profile or not, and the engine generates as with a given count."""
    from kvcore_amd import CacheConfig, KVCoreConfig, LoadConfig, ModelConfig, SamplingParams, SchedulerConfig
    from kvcore_amd.engine.llm_engine import LLMEngine
    from tests.helpers import TINY_D, random_tokens

    (tmp_path / "config.json").write_text(json.dumps(TINY_D))
    outs = {}
    for pages in (None, 300):
        engine = LLMEngine(KVCoreConfig(
            model_config=ModelConfig(model=str(tmp_path), dtype="bfloat16", max_model_len=512),
            load_config=LoadConfig(load_format="random", seed=3),
            cache_config=CacheConfig(block_size=16, num_gpu_blocks=pages),
            scheduler_config=SchedulerConfig(max_num_seqs=6, max_num_scheduled_tokens=40)))
        core = engine.engine_core
        if pages is None:
            assert core.num_pages == 6 * 32 + 1 == core.memory_profile.useful_pages
            assert core.memory_profile.pages == core.num_pages
            assert core.memory_profile.live > 0 and core.memory_profile.budget > core.memory_profile.live
        else:
            assert core.num_pages == 300 and core.memory_profile is None
        reqs = [dict(request_id=f"r{i}", prompt_token_ids=random_tokens(n, 512, seed=70 + i),
                     sampling_params=SamplingParams(max_tokens=9, temperature=0.0, ignore_eos=True))
                for i, n in enumerate((3, 50, 17, 90))]
        outs[pages] = {o.request_id: o.output_token_ids for o in engine.generate(reqs)}
        core.kv_manager.check()
    assert outs[None] == outs[300]


def test_profile_steps_run_on_a_model_with_state_and_parts_that_are_not_graph_safe(tmp_path):
    """The profile steps drive whatever the registry built: here the toy architecture with a
    mixer that keeps state of its own and walks the requests on the host (no graphs), a layer
    that runs twice and one that reads another's cache.  The engine sizes itself and then
    generates what an engine with a given page count generates."""
    from kvcore_amd import CacheConfig, KVCoreConfig, ModelConfig, SamplingParams, SchedulerConfig
    from kvcore_amd.engine.llm_engine import LLMEngine
    from kvcore_amd.weights.loader import write_random_model
    from tests.helpers import random_tokens
    from tests.test_toy_parts_gpu import TOY_CONFIG, register_toy

    register_toy()
    folder = write_random_model(tmp_path / "toy", TOY_CONFIG, seed=9)
    outs = {}
    for pages in (None, 64):
        engine = LLMEngine(KVCoreConfig(
            model_config=ModelConfig(model=str(folder), dtype="float32", max_model_len=96),
            cache_config=CacheConfig(block_size=8, num_gpu_blocks=pages),
            scheduler_config=SchedulerConfig(max_num_seqs=3, max_num_scheduled_tokens=24)))
        core = engine.engine_core
        assert not core.model.graph_safe()
        if pages is None:
            assert core.memory_profile is not None and core.num_pages == 3 * 12 + 1
        reqs = [dict(request_id=f"t{i}", prompt_token_ids=random_tokens(n, 97, seed=40 + i),
                     sampling_params=SamplingParams(max_tokens=7, temperature=0.0, ignore_eos=True))
                for i, n in enumerate((30, 4, 19, 11))]
        outs[pages] = {o.request_id: o.output_token_ids for o in engine.generate(reqs)}
        core.kv_manager.check()
    assert outs[None] == outs[64] and all(len(t) == 7 for t in outs[None].values())
