"""The Llama 3 dense decoder as a ``ModelSpec``.

Reference: kvcore/model/models/llama3.py: every layer is RMSNorm, grouped-query
attention with rotated q/k (scale ``head_dim ** -0.5``, :60), RMSNorm, SwiGLU (:107-142);
tensor names are the checkpoint's (``model.layers.{i}.self_attn.q_proj.weight`` and so
on, stacked by :249-262).
"""

from __future__ import annotations

from kvcore_amd.config.model_config import LlamaConfig
from kvcore_amd.parts.base import PartSpec

from .spec import LayerSpec, ModelSpec


def llama_spec(config: LlamaConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"hidden_size": config.hidden_size, "eps": config.rms_norm_eps})
    attention = PartSpec("paged_attention", {
        "hidden_size": config.hidden_size,
        "num_heads": config.num_attention_heads,
        "num_kv_heads": config.num_key_value_heads,
        "head_dim": config.head_dim,
        "scale": config.head_dim ** -0.5,
        "bias": config.attention_bias,
    })
    ffn = PartSpec("swiglu", {
        "hidden_size": config.hidden_size,
        "intermediate_size": config.intermediate_size,
        "bias": config.mlp_bias,
    })
    rotary = PartSpec("rotary", {
        "rot_dim": config.head_dim,
        "theta": config.rope_theta,
        "scaling": config.rope_scaling.to_dict(),
    })
    layers = tuple(
        LayerSpec(
            prefix=f"model.layers.{i}",
            mixer=attention,
            ffn=ffn,
            norms={"input_layernorm": norm, "post_attention_layernorm": norm},
            block=PartSpec("prenorm", {"mixer_name": "self_attn", "ffn_name": "mlp",
                                       "input_norm": "input_layernorm",
                                       "post_norm": "post_attention_layernorm"}),
            position=0,
        )
        for i in range(config.num_hidden_layers)
    )
    return ModelSpec(
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        max_position_embeddings=config.max_position_embeddings,
        layers=layers,
        final_norm=norm,
        positions=(rotary,),
        tie_word_embeddings=config.tie_word_embeddings,
        eos_token_ids=config.eos_token_ids,
    )
