from __future__ import annotations

import json

import pytest

from kvcore_amd.config.engine_config import (CacheConfig, KVCoreConfig, ModelConfig, SchedulerConfig,
                                             canonical_dtype)
from kvcore_amd.config.model_config import ConfigError, LlamaConfig, RopeScaling, read_config_json
from kvcore_amd.models.llama import llama_spec
from kvcore_amd.registry import (MODEL_REGISTRY, register_architecture, resolve_architecture,
                                 unregister_architecture)
from tests.helpers import TINY_A, TINY_B, TINY_C


def test_every_size_comes_from_the_file():
    for raw in (TINY_A, TINY_B, TINY_C):
        c = LlamaConfig.from_dict(raw)
        assert c.vocab_size == raw["vocab_size"] and c.hidden_size == raw["hidden_size"]
        assert c.num_hidden_layers == raw["num_hidden_layers"]
        assert c.num_key_value_heads == raw["num_key_value_heads"] and c.head_dim == raw["head_dim"]
        assert c.rms_norm_eps == raw["rms_norm_eps"] and c.rope_theta == raw["rope_theta"]
        spec = llama_spec(c)
        attn = spec.layers[0].mixer.args
        assert attn["scale"] == raw["head_dim"] ** -0.5  # llama3.py:60
        assert spec.layers[0].norms["input_layernorm"].args["eps"] == raw["rms_norm_eps"]
        assert spec.layers[0].ffn.args["intermediate_size"] == raw["intermediate_size"]
        assert spec.tie_word_embeddings == raw["tie_word_embeddings"]
        assert len(spec.layers) == raw["num_hidden_layers"]
        assert LlamaConfig.from_dict(c.to_dict()) == c


def test_defaults_follow_the_reference():
    raw = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "head_dim", "rope_theta")}
    c = LlamaConfig.from_dict(raw)
    assert c.num_key_value_heads == c.num_attention_heads  # engine_core.py:164
    assert c.head_dim == c.hidden_size // c.num_attention_heads  # llama3.py:59
    assert c.rope_theta == 10000.0  # rotary_embedding.py:49
    raw["rope_parameters"] = {"rope_theta": 123.0}
    assert LlamaConfig.from_dict(raw).rope_theta == 123.0  # rotary_embedding.py:40-43


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "rms_norm_eps", "max_position_embeddings"])
def test_a_missing_required_key_is_named(key):
    raw = {k: v for k, v in TINY_A.items() if k != key}
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(raw)


def test_refused_values():
    with pytest.raises(ConfigError, match="activation"):
        LlamaConfig.from_dict({**TINY_A, "hidden_act": "gelu"})  # llama3.py:28-31
    with pytest.raises(ConfigError, match="rope_type"):
        LlamaConfig.from_dict({**TINY_A, "rope_scaling": {"rope_type": "yarn", "factor": 2.0}})
    with pytest.raises(ConfigError, match="multiple"):
        LlamaConfig.from_dict({**TINY_A, "num_key_value_heads": 3})
    with pytest.raises(ConfigError, match="low_freq_factor"):
        LlamaConfig.from_dict({**TINY_A, "rope_scaling": {"rope_type": "llama3", "factor": 2.0}})
    assert RopeScaling.from_dict({"rope_type": "default"}) == RopeScaling()


def test_eos_may_be_an_int_or_a_list():
    assert LlamaConfig.from_dict({**TINY_A, "eos_token_id": 7}).eos_token_ids == (7,)
    assert LlamaConfig.from_dict({**TINY_A, "eos_token_id": [7, 9]}).eos_token_ids == (7, 9)


def test_generation_config_adds_stop_ids(tmp_path):
    """An instruct checkpoint lists its end-of-turn id in generation_config.json only."""
    import json

    from kvcore_amd.config.model_config import ConfigError, read_generation_eos

    assert read_generation_eos(tmp_path) == ()
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [128001, 128009]}))
    assert read_generation_eos(tmp_path) == (128001, 128009)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": 5, "temperature": 0.6}))
    assert read_generation_eos(tmp_path) == (5,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"temperature": 0.6}))
    assert read_generation_eos(tmp_path) == ()
    (tmp_path / "generation_config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        read_generation_eos(tmp_path)
    # the engine joins them with config.json's and the tokenizer's: a deliberate addition to the
    # reference's join (engine_core.py:209-217), which knows only those two
    from kvcore_amd.engine.engine_core import join_stop_token_ids

    class Tokenizer:
        def get_stop_token_ids(self):
            return {7, 128001}

    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [128001, 128009]}))
    assert join_stop_token_ids((128001,), tmp_path, None) == {128001, 128009}
    assert join_stop_token_ids((128001,), tmp_path, Tokenizer()) == {7, 128001, 128009}
    assert join_stop_token_ids((128001,), None, Tokenizer()) == {7, 128001}  # a model given, no folder read
    assert join_stop_token_ids((), None, None) == set()


def test_registry_key_is_the_architecture_name_with_model_type_as_fallback():
    assert resolve_architecture(TINY_A).name == "LlamaForCausalLM"
    assert resolve_architecture({"model_type": "llama"}).name == "LlamaForCausalLM"
    with pytest.raises(ValueError, match="Supported"):
        resolve_architecture({"architectures": ["NoSuchModel"], "model_type": "none"})
    with pytest.raises(ValueError, match="already registered"):
        register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec)
    register_architecture("ToyForTest", LlamaConfig.from_dict, llama_spec)
    try:
        assert resolve_architecture({"architectures": ["ToyForTest"]}).name == "ToyForTest"
    finally:
        unregister_architecture("ToyForTest")
    assert "ToyForTest" not in MODEL_REGISTRY


def test_read_config_json(tmp_path):
    with pytest.raises(FileNotFoundError):
        read_config_json(tmp_path / "missing")
    with pytest.raises(FileNotFoundError):
        read_config_json(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert read_config_json(tmp_path)["vocab_size"] == 256


def test_engine_config_validation():
    """kvcore/config.py:15-93."""
    assert canonical_dtype("torch.bfloat16") == "bfloat16" and canonical_dtype("fp32") == "float32"
    with pytest.raises(ValueError):
        canonical_dtype("float16")
    with pytest.raises(ValueError):
        ModelConfig(model="x", max_model_len=0)
    with pytest.raises(ValueError):
        CacheConfig(block_size=0)
    with pytest.raises(ValueError):
        CacheConfig(gpu_memory_utilization=0.0)
    with pytest.raises(ValueError):
        SchedulerConfig(max_num_seqs=0)
    with pytest.raises(ValueError):
        SchedulerConfig(long_prefill_token_threshold=-1)
    with pytest.raises(ValueError):
        SchedulerConfig(max_num_partial_prefills=0)
    # unset, every request that has a slot may be in its prompt; set, the number stands
    assert SchedulerConfig().max_num_partial_prefills == 8
    assert SchedulerConfig(max_num_seqs=32).max_num_partial_prefills == 32
    assert SchedulerConfig(max_num_seqs=32, max_num_partial_prefills=1).max_num_partial_prefills == 1
    cfg = KVCoreConfig(ModelConfig(model="x", dtype="bf16"))
    assert cfg.model_config.dtype == "bfloat16"
    # the attention backend is filled in when unset (config.py:170-192); the reference's own
    # backends are refused by name
    assert ModelConfig(model="x").attn_backend is None and cfg.model_config.attn_backend == "hip"
    with pytest.raises(ValueError, match="hip"):
        ModelConfig(model="x", attn_backend="triton_paged")
    assert (cfg.cache_config.block_size, cfg.scheduler_config.max_num_seqs,
            cfg.scheduler_config.max_num_scheduled_tokens) == (16, 8, 512)


def test_a_cache_need_describes_its_planes():
    from kvcore_amd.parts.base import CacheNeed

    kv = CacheNeed.keys_and_values(8, 128, window=0, page_size=None)
    assert kv.planes == ((8, 128), (8, 128)) and kv.token_elems() == (1024, 1024)
    assert CacheNeed(((512,),)).token_elems() == (512,)
    assert CacheNeed([[2, 3], [5]]) == CacheNeed(((2, 3), (5,)))  # lists become tuples: needs are keys
    assert len({CacheNeed(((4, 16), (4, 16))), CacheNeed.keys_and_values(4, 16)}) == 1
    for bad in ((), ((),), ((4, 0),)):
        with pytest.raises(ValueError):
            CacheNeed(bad)
